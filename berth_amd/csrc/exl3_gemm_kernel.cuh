// EXL3 linear for many rows: trellis decode fused into an fp16 MFMA GEMM
// (v_mfma_f32_32x32x16_f16, fp32 accumulate).  Covers the row counts the
// reference spreads over a cooperative GEMM (<= 144 rows) and reconstruct +
// dense GEMM (> 144 rows), crates/berth-kernels/csrc/prefill_lin/linear.cu:184-344;
// the weight is never written back to memory.
//
//   launch 1: a_had = Hh(a * suh)                        (had_r_128, pre-scale)
//   launch 2: c = Hh(a_had @ W) * svh                    (this file)
//
// Work split: a workgroup of 4 waves owns BM = 32*MB rows x 256 columns; each
// wave owns 64 of the columns for all BM rows, so decoded weights stay in the
// registers of the wave that decoded them.  Per 32 rows of K a wave decodes 2
// tile rows x 4 tile columns: lanes 0..31 take tile row kt, lanes 32..63 tile row
// kt+1, eight lanes per tile (octet layout).  The four register quads a lane ends
// up with ((column u or u+8) x (k 0..7 or 8..15 of its tile row)) are exactly four
// MFMA B operands: B[k-slot][col-slot] with col-slot = lane % 32 and k-slot =
// 8*(lane/32) + i.  The A operand for the same slots is a_had[row][16*(kt +
// lane/32) + 8h + i], one 16-byte LDS read.  Column slots map to columns
// 16*(slot/8) + slot%8 + 8f; the epilogue undoes that when it stages the fp32
// tile in LDS for the output Hadamard.
//
// K can be split over S workgroups (few rows, or few columns: not enough tiles to
// fill the chip).  The last workgroup to arrive at a tile (self-resetting counters)
// finishes it: the others leave their partial accumulators in the library workspace
// in register layout, and the finisher adds all parts in k order, so the result does
// not depend on timing.
#pragma once

#include "exl3_gemv_kernel.cuh"

namespace berth {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// one linear of a bundle whose lists the host knows
struct GemmSlice {
    const uint32_t* trellis;
    const _Float16* svh;
    void* c;
    int width;                  // columns of this linear (a multiple of 128, at most N)
    int n_stride;               // columns of the whole weight the slice is cut from: elements between
                                // output rows and, in tiles of 16, between the tile rows of its trellis
    const _Float16* a_had;      // the rotated copy of the input it multiplies, [M][K]
};
constexpr int kGemmMaxSlices = 16;

struct GemmParams {
    const _Float16* a_had[2];   // [rows][K], already rotated (one per linear of the launch)
    ExpertLin lin;              // dense mode
    void* c[2];
    int M, K, N, out_fp32;
    // grouped mode (problems != nullptr): blockIdx.z = problem (<= BM rows),
    // blockIdx.y = which of the launch's linears
    const ExpertLin* experts;
    const GroupProblem* problems;
    const int* num_problems;
    int lins_per_expert, lin_base;
    ExpertLin shared[3];        // an always-on expert passed by value (problem.expert == shared_expert)
    int shared_expert;
    // mixed grouped launches (exl3_gemm_mixed_kernel): problems of up to 128 rows, whose units
    // of work come first; those of `problems` follow
    const GroupProblem* big_problems;
    const int* num_big;
    int max_big;
    int tiles_y;                // dense: row blocks; grouped: capacity of the problem list
    int tile0;                  // dense: first (row block, column block) tile of this launch, row-major
    // split-K
    int S;
    float* partials;            // [unit][S][4 waves][MB][2][16][64]
    unsigned* counters;         // [unit], cstride words apart ("arrived"; "written" kGemmWrittenBase further on)
    int cstride;
    // balanced dense launches (exl3_gemm_balanced_kernel): the launch's (tile, k-block) units,
    // tile-major, are dealt out evenly to gridDim.x workgroups
    int units;                  // tiles * K/128; 0: not a balanced launch
    int unit_q, unit_r;         // units = unit_q * gridDim.x + unit_r
    int max_parts;              // upper bound of workgroups that share one tile
    // A tile's finisher waits for the other sharers' partial sums with a bound: after
    // spin_limit polls it gives up, zeroes the tile's counters, stores 1 + the tile's counter
    // index to *fault (host-visible memory; may be null) and leaves the tile unwritten.
    unsigned* fault;
    unsigned spin_limit;
    // Bundles (crates/berth-kernels/src/ops.rs:264-293 with more than 8 rows): num_slices
    // linears that share K and the row count run as one dense launch.  Every slice owns
    // ceil(N / 256) column blocks of the launch (N = the widest slice); a block past the end of
    // a narrower slice is empty.  The slice's tensors come from the device lists when b_list is
    // set (uniform mode: c_ptrs null, outputs [slice][M][N] behind c[0], rotated input = slab
    // `slice`; sliced mode: all seven lists; a_had[0] holds the rotated inputs, slab_stride
    // elements apart), else from `slice` by value.
    int num_slices;             // 0: one linear (lin, c[0], a_had[0])
    size_t slab_stride;
    const uint64_t* b_list;
    const uint64_t* svh_list;
    const uint64_t* c_ptrs;
    const int* size_n_list;
    const int* n_stride_list;
    const int* had_src_list;
    GemmSlice slice[kGemmMaxSlices];
};

// the tensors of the column block `nblk` of a dense launch
struct TileView {
    ExpertLin lin;
    const _Float16* a_had;
    void* cout;
    int N;                      // columns of the linear
    int ldc;                    // elements between output rows
    int nblk;                   // column block inside the linear
    bool empty;                 // the block lies past the end of its (narrower) slice
};
__device__ __forceinline__ TileView dense_tile_view(const GemmParams& p, const int nblk)
{
    TileView v;
    v.lin = p.lin;
    v.a_had = p.a_had[0];
    v.cout = p.c[0];
    v.N = p.N;
    v.ldc = p.N;
    v.nblk = nblk;
    v.empty = false;
    if (p.num_slices > 0) {
        const int per = (p.N + 255) >> 8;
        const int sl = nblk / per;
        v.nblk = nblk - sl * per;
        if (p.b_list) {
            int slab = sl;
            v.lin.trellis = (const uint32_t*)p.b_list[sl];
            v.lin.svh = (const _Float16*)p.svh_list[sl];
            if (p.c_ptrs) {
                v.N = p.size_n_list[sl];
                v.ldc = p.n_stride_list[sl];
                slab = p.had_src_list[sl];
                v.cout = (void*)p.c_ptrs[sl];
            } else {
                v.cout = (char*)p.c[0] + (size_t)sl * p.M * p.N * (p.out_fp32 ? 4 : 2);
            }
            v.a_had = p.a_had[0] + (size_t)slab * p.slab_stride;
        } else {
            const GemmSlice& g = p.slice[sl];
            v.lin.trellis = g.trellis;
            v.lin.svh = g.svh;
            v.cout = g.c;
            v.N = g.width;
            v.ldc = g.n_stride;
            v.a_had = g.a_had;
        }
        v.empty = v.nblk * 256 >= v.N;
    }
    return v;
}

// The finisher's wait for `counter` to reach `want`, bounded.  Called by one thread.  A
// workgroup that has arrived is running and depends on nothing, so the counter gets there
// within microseconds unless the counters were left inconsistent (two launches sharing the
// workspace at once, a launch that was aborted); then this ends the wait instead of hanging.
__device__ __forceinline__ bool wait_counter_bounded(unsigned* counter, unsigned want, unsigned limit)
{
    for (unsigned polls = 0; __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != want; ++polls) {
        if (polls >= limit) return false;
        __builtin_amdgcn_s_sleep(2);
    }
    return true;
}

// the k-blocks of one tile that a workgroup accumulates, and its place among the
// workgroups that share the tile
struct KRange {
    int kb0, kb1, step;         // k-blocks kb0, kb0 + step, ... < kb1
    int part, parts;            // this workgroup's position (k order) and the number of sharers
    size_t slot0;               // first partial-sum slot of the tile
    size_t counter;             // arrival counter of the tile
};

constexpr int kGemmWrittenBase = 32768;   // second half of the counter table: "partial sums written" per tile

constexpr int kAStride = 128 + 8;   // halves per LDS row of the A tile (272 B: conflict-free b128 reads)

// one output tile: rows of problem / row block `tile_y`, 256 columns
template <int BITS, int CB, int MB, bool DENSE>  // MB = 32-row blocks per workgroup; DENSE: never a problem list
__device__ __forceinline__ void gemm_tile(const GemmParams& p, const int tile_y, const int nblk, const KRange kr,
                                          const int which, unsigned char* smem, const GroupProblem* problems = nullptr)
{
    constexpr int BM = MB * 32;
    _Float16* a_tile = (_Float16*)smem;                 // [2][BM][kAStride]
    float* z_tile = (float*)smem;                       // epilogue: [32][256 + 4]
    constexpr int kZStride = 256 + 4;
    __shared__ unsigned s_last;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int half_id = lane >> 5;                      // which of the two tile rows
    const int slot = lane & 31;                         // MFMA row / column slot
    int m0 = tile_y * BM;
    int m_end = p.M;
    ExpertLin lin = p.lin;
    const _Float16* a_had = p.a_had[0];
    void* cout = p.c[0];
    int N = p.N, ldc = p.N, nblk_lin = nblk;
    if constexpr (DENSE) {
        const TileView v = dense_tile_view(p, nblk);
        if (v.empty) return;                            // the same for every workgroup that shares the tile
        lin = v.lin;
        a_had = v.a_had;
        cout = v.cout;
        N = v.N;
        ldc = v.ldc;
        nblk_lin = v.nblk;
    }
    const int n0 = nblk_lin * 256;
    if constexpr (!DENSE) {
        // (dynamic indexing of the parameter block: kept out of the dense instantiations, where
        // it would force the whole block into private memory)
        const GroupProblem gp = problems[tile_y];
        lin = gp.expert == p.shared_expert ? p.shared[p.lin_base + which]
                                           : p.experts[gp.expert * p.lins_per_expert + p.lin_base + which];
        m0 = gp.row0;
        m_end = gp.row0 + gp.nrows;
        a_had = p.a_had[which];
        cout = p.c[which];
    }
    const int rows_here = min(BM, m_end - m0);          // >= 1
    const int nw = n0 + wave * 64;                      // first column of this wave
    const bool active = nw < N;
    const int tn = ldc >> 4;                            // tiles per tile row of the weight (of the whole weight, for a slice)
    constexpr int tile_dw = 8 * BITS;
    const size_t row_dw = (size_t)tn * tile_dw;
    const int KB = p.K >> 7;

    float16_t acc[MB][2];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int f = 0; f < 2; ++f)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][f][r] = 0.0f;

    if constexpr (MB == 1) {
        // ---- 32-row tile: every wave is on its own.  The A operand of a lane (row
        // `slot`, 8 k values) is one 16-byte load straight from the rotated rows, so
        // there is no LDS tile and no barrier in the loop.  Trellis and A registers are
        // reloaded for the wave's next k-block as soon as a step has consumed them
        // (rolling prefetch, one k-block ahead); on the last k-block the reload reads
        // the same addresses again and is ignored, which keeps the loop free of branches.
        if (active && kr.kb0 < kr.kb1) {
            const global_ptr<const uint32_t> tb = as_global(lin.trellis) + (size_t)half_id * row_dw +
                                                 (size_t)((nw >> 4) + (slot >> 3)) * tile_dw + (slot & 7) * BITS;
            const int arow = m0 + min(slot, rows_here - 1);         // rows past the problem repeat its last row
            const global_ptr<const half8_t> ab =
                (global_ptr<const half8_t>)(as_global(a_had) + (size_t)arow * p.K + 16 * half_id);
            uint32_t cur[4][BITS];
            half8_t av[4][2];
            {
                const global_ptr<const uint32_t> t0 = tb + (size_t)(kr.kb0 * 8) * row_dw;
                const global_ptr<const half8_t> a0 = ab + kr.kb0 * 16;
#pragma unroll
                for (int st = 0; st < 4; ++st) {
                    load_tile_dwords<BITS>(t0 + (size_t)(2 * st) * row_dw, cur[st]);
                    av[st][0] = a0[4 * st];
                    av[st][1] = a0[4 * st + 1];
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            for (int kb = kr.kb0; kb < kr.kb1; kb += kr.step) {
                const int nkb = kb + kr.step < kr.kb1 ? kb + kr.step : kb;
                const global_ptr<const uint32_t> tnx = tb + (size_t)(nkb * 8) * row_dw;
                const global_ptr<const half8_t> anx = ab + nkb * 16;
#pragma unroll
                for (int st = 0; st < 4; ++st) {
                    uint32_t prev = fetch_prev(lane, cur[st][BITS - 1]);
                    uint32_t w2[16];
                    decode_lane<BITS, CB>(cur[st], prev, w2);
                    load_tile_dwords<BITS>(tnx + (size_t)(2 * st) * row_dw, cur[st]);
                    half8_t b[2][2];
#pragma unroll
                    for (int f = 0; f < 2; ++f)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const uint4 q = {w2[2 * f + h], w2[4 + 2 * f + h], w2[8 + 2 * f + h], w2[12 + 2 * f + h]};
                            b[f][h] = __builtin_bit_cast(half8_t, q);
                        }
                    const half8_t a0 = av[st][0], a1 = av[st][1];
                    av[st][0] = anx[4 * st];
                    av[st][1] = anx[4 * st + 1];
                    __builtin_amdgcn_sched_barrier(0);
                    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b[0][0], acc[0][0], 0, 0, 0);
                    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b[1][0], acc[0][1], 0, 0, 0);
                    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b[0][1], acc[0][0], 0, 0, 0);
                    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b[1][1], acc[0][1], 0, 0, 0);
                }
            }
        }
    } else {
        // lane's trellis position inside a k-block: tile row 2*step + half_id, tile (nw/16 + slot/8)
        const uint32_t* tbase = lin.trellis + (size_t)half_id * row_dw +
                                (size_t)((nw >> 4) + (slot >> 3)) * tile_dw + (slot & 7) * BITS;

        // Operands run ahead in registers: this thread's share of the next k-block's A tile
        // (a_nxt, 32 bytes per 256-thread pass; the tile is double-buffered in LDS, so a
        // k-block costs one barrier) and the trellis dwords of the wave's four steps (ring),
        // each reloaded for the next k-block as soon as its step is decoded.
        //
        // A step's 32 weights per lane are 16 pairs; the even pairs are the B operands for
        // k 0..7 of each lane's 16 (A operand a0), the odd pairs those for k 8..15 (a1).  The
        // loop runs in half-steps: the eight MFMAs of one half are issued two at a time, and
        // behind every two a quarter of the decode of the NEXT half (the odd pairs of the same
        // step, or the even pairs of the next step, which across the barrier is step 0 of the
        // next k-block), so the vector pipe decodes while the matrix pipe multiplies.  Row
        // blocks past the end of the rows are multiplied too (their A rows are zero): the loop
        // has no branch.  The order is given to the scheduler as groups after each half-step.
        constexpr int kAPasses = BM * 8 / 256;
        uint32_t ring[4][BITS];
        u32x4_t a_nxt[kAPasses][2];
        const int a_row = threadIdx.x >> 3, a_ch = threadIdx.x & 7;       // + 32 rows per pass
        auto load_a = [&](int kb) {
    #pragma unroll
            for (int ps = 0; ps < kAPasses; ++ps) {
                const int r = a_row + 32 * ps;
                u32x4_t v0 = {0, 0, 0, 0}, v1 = {0, 0, 0, 0};
                if (m0 + r < m_end) {
                    const global_ptr<const u32x4_t> src =
                        (global_ptr<const u32x4_t>)(as_global(a_had) + (size_t)(m0 + r) * p.K + kb * 128 + a_ch * 16);
                    v0 = src[0];
                    v1 = src[1];
                }
                a_nxt[ps][0] = v0;
                a_nxt[ps][1] = v1;
            }
        };
        auto load_b_step = [&](int kb, int st) {
            const global_ptr<const uint32_t> nb = as_global(tbase) + (size_t)(kb * 8 + 2 * st) * row_dw;
    #pragma unroll
            for (int j = 0; j < BITS; ++j) ring[st][j] = nb[j];
        };
        // the eight pairs of one half, numbered j = 4f + q: out[f][q] = pair 4q + 2f + h
        auto decode_pairs = [&](const LaneWindows<BITS>& w, int h, int j0, int n, uint32_t (&out)[2][4]) {
    #pragma unroll
            for (int j = j0; j < j0 + n; ++j) {
                const int f = j >> 2, q = j & 3;
                const int pr = 4 * q + 2 * f + h;
                out[f][q] = decode_pair<CB>(w.state(2 * pr), w.state(2 * pr + 1));
            }
        };
        uint32_t b_half[2][2][4];                       // [which half-step buffer][f][q]
        LaneWindows<BITS> win;
        if (kr.kb0 < kr.kb1) {
            load_a(kr.kb0);
            if (active) {
    #pragma unroll
                for (int st = 0; st < 4; ++st) load_b_step(kr.kb0, st);
                win = LaneWindows<BITS>(ring[0], fetch_prev(lane, ring[0][BITS - 1]));
                decode_pairs(win, 0, 0, 8, b_half[0]);
            }
        }

        int buf = 0;
        for (int kb = kr.kb0; kb < kr.kb1; kb += kr.step, buf ^= 1) {
            // publish this k-block's A tile; the other buffer may still be read by slower waves
            _Float16* a_buf = a_tile + (size_t)buf * BM * kAStride;
    #pragma unroll
            for (int ps = 0; ps < kAPasses; ++ps) {
                u32x4_t* dst = (u32x4_t*)(a_buf + (a_row + 32 * ps) * kAStride + a_ch * 16);
                dst[0] = a_nxt[ps][0];
                dst[1] = a_nxt[ps][1];
            }
            // the next k-block (on the last one the same again: read and ignored, no branch)
            const int nkb = kb + kr.step < kr.kb1 ? kb + kr.step : kb;
            load_a(nkb);
            __syncthreads();

            if (active) {
                const _Float16* a_lane = a_buf + slot * kAStride + 16 * half_id;
                // A operand of half-step hs = 2 * st + h, row block mb: k = 32 * st + 16 * half_id + 8 * h .. + 7 of the k-block
                auto a_operand = [&](int hs, int mb) {
                    return *(const half8_t*)(a_lane + mb * 32 * kAStride + 32 * (hs >> 1) + 8 * (hs & 1));
                };
                half8_t a_op = a_operand(0, 0);
    #pragma unroll
                for (int hs = 0; hs < 8; ++hs) {
                    const int st = hs >> 1, h = hs & 1;
                    __builtin_amdgcn_sched_barrier(0);
                    uint32_t (&b_cur)[2][4] = b_half[h];
                    uint32_t (&b_nx)[2][4] = b_half[h ^ 1];
                    const half8_t b0 = __builtin_bit_cast(half8_t, uint4{b_cur[0][0], b_cur[0][1], b_cur[0][2], b_cur[0][3]});
                    const half8_t b1 = __builtin_bit_cast(half8_t, uint4{b_cur[1][0], b_cur[1][1], b_cur[1][2], b_cur[1][3]});
                    if (h == 1) {
                        // the step after this one: its windows, then (below) its even pairs
                        const int ns = (st + 1) & 3;
                        win = LaneWindows<BITS>(ring[ns], fetch_prev(lane, ring[ns][BITS - 1]));
                    }
    #pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        const half8_t a_now = a_op;
                        if (mb + 1 < MB) a_op = a_operand(hs, mb + 1);
                        else if (hs < 7) a_op = a_operand(hs + 1, 0);
                        acc[mb][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_now, b0, acc[mb][0], 0, 0, 0);
                        acc[mb][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_now, b1, acc[mb][1], 0, 0, 0);
                        decode_pairs(win, h ^ 1, mb * (8 / MB), 8 / MB, b_nx);
                    }
                    // the step's dwords are decoded once its odd pairs exist: request the next k-block's
                    if (h == 0) load_b_step(nkb, st);
    #define BERTH_GEMM_CHUNK(valu0, valu1)                                              \
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                              \
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                              \
        __builtin_amdgcn_sched_group_barrier(0x002, valu0, 0);                          \
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                              \
        __builtin_amdgcn_sched_group_barrier(0x002, valu1, 0);
                    static_assert(MB == 4, "the groups below describe eight MFMAs per half-step");
                    BERTH_GEMM_CHUNK(9, 9) BERTH_GEMM_CHUNK(9, 9) BERTH_GEMM_CHUNK(9, 9) BERTH_GEMM_CHUNK(9, 9)
    #undef BERTH_GEMM_CHUNK
                }
            }
        }

    }

    // ---- split-K handoff.  Register r of a lane holds tile row 8*(r/4) + 4*half_id + r%4,
    // so only registers with 8*(r/4) < rows matter.
    if (kr.parts > 1) {
        // Arrive first.  The last workgroup to arrive finishes the tile: it waits until the
        // others have written their partial sums (they bump the tile's second counter after
        // their stores; a workgroup that has arrived is running and depends on nothing, so
        // the wait is short and cannot block) and adds the parts in k order.  If it holds
        // part 0 itself it starts from its registers and never writes them out.
        constexpr size_t kPerWg = (size_t)4 * MB * 2 * 16 * 64;
        unsigned* arrived = p.counters + kr.counter * p.cstride;
        unsigned* written = arrived + kGemmWrittenBase;
        if (threadIdx.x == 0) {
            unsigned old = __hip_atomic_fetch_add(arrived, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = (old == (unsigned)(kr.parts - 1)) ? 1u : 0u;
        }
        __syncthreads();
        const bool finisher = s_last != 0;
        const float* all = p.partials + kr.slot0 * kPerWg + (size_t)wave * MB * 2 * 16 * 64;
        if (!(finisher && kr.part == 0)) {
            float* mine = p.partials + (kr.slot0 + kr.part) * kPerWg + (size_t)wave * MB * 2 * 16 * 64;
            if (active) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int f = 0; f < 2; ++f)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            if (mb * 32 + 8 * (r >> 2) < rows_here)
                                __hip_atomic_store(mine + ((mb * 2 + f) * 16 + r) * 64 + lane, acc[mb][f][r],
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (!finisher) {
            wait_own_stores();
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __syncthreads();
            if (threadIdx.x == 0) __hip_atomic_fetch_add(written, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
        if (threadIdx.x == 0) {
            const bool complete = wait_counter_bounded(written, (unsigned)(kr.parts - 1), p.spin_limit);
            __hip_atomic_store(written, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(arrived, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (!complete && p.fault)
                __hip_atomic_store(p.fault, 1u + (unsigned)kr.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            s_last = complete ? 1u : 2u;
        }
        __syncthreads();
        if (s_last == 2u) return;       // gave up: the tile stays unwritten, the host is told
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (active) {
            // part 0 first (from memory unless it is this workgroup's own), then parts 1, 2, ...
            // added in order.  64 (128-row tiles) or 128 (32-row tiles) loads a lane are in
            // flight at a time: half of a part's register blocks, or four whole parts.
            constexpr int kGroup = MB == 1 ? 2 : 4;             // (mb, f) register blocks per batch
            constexpr int kParts = MB == 1 ? 4 : 1;             // parts per batch
            const int first = kr.part == 0 ? 1 : 0;
            for (int j0 = first; j0 < kr.parts; j0 += kParts) {
#pragma unroll
                for (int g0 = 0; g0 < MB * 2; g0 += kGroup) {
                    float tmp[kParts][kGroup][16];
#pragma unroll
                    for (int jj = 0; jj < kParts; ++jj) {
                        const int j = j0 + jj < kr.parts ? j0 + jj : kr.parts - 1;      // past the end: ignored
                        const float* src = all + (size_t)j * kPerWg;
#pragma unroll
                        for (int b = 0; b < kGroup; ++b) {
                            const int blk = g0 + b;             // = mb * 2 + f
                            if ((blk >> 1) * 32 >= rows_here) continue;                 // workgroup-uniform
#pragma unroll
                            for (int r = 0; r < 16; ++r)
                                tmp[jj][b][r] = __hip_atomic_load(src + (blk * 16 + r) * 64 + lane, __ATOMIC_RELAXED,
                                                                  __HIP_MEMORY_SCOPE_AGENT);
                        }
                    }
#pragma unroll
                    for (int jj = 0; jj < kParts; ++jj) {
                        if (j0 + jj >= kr.parts) break;
#pragma unroll
                        for (int b = 0; b < kGroup; ++b) {
                            const int blk = g0 + b;
                            if ((blk >> 1) * 32 >= rows_here) continue;
#pragma unroll
                            for (int r = 0; r < 16; ++r)
                                acc[blk >> 1][blk & 1][r] =
                                    j0 + jj == 0 ? tmp[jj][b][r] : acc[blk >> 1][blk & 1][r] + tmp[jj][b][r];
                        }
                    }
                }
            }
        }
    }

    // ---- epilogue, 32 rows at a time: stage fp32 tile, output Hadamard, svh, store
    const int col_in_wave = (slot >> 3) * 16 + (slot & 7);     // + 8f
    // output scales: a lane of the epilogue owns columns 8 * (lane % 16) .. + 7 of a block
    const int l16 = lane & 15;
    half8_t sv_blk[2];
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
        const int gn = n0 + blk * 128;
        sv_blk[blk] = gn < N ? ((global_ptr<const half8_t>)as_global(lin.svh + gn))[l16] : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        if (mb * 32 >= rows_here) break;                        // workgroup-uniform
        __syncthreads();
        if (active) {
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = 8 * (r >> 2) + 4 * half_id + (r & 3);
                    z_tile[row * kZStride + wave * 64 + col_in_wave + 8 * f] = acc[mb][f][r];
                }
        }
        __syncthreads();
        const int rows_blk = min(32, rows_here - mb * 32);
        // 64 vectors (32 rows x 2 column blocks); a wave rotates four per pass, sixteen lanes each
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int vec = pass * 16 + wave * 4 + (lane >> 4);
            const int row = vec >> 1, blk = vec & 1;
            const int gn = n0 + blk * 128;
            if (row < rows_blk && gn < N) {
                float v[8];
                const float4_t* zp = (const float4_t*)&z_tile[row * kZStride + blk * 128 + 8 * l16];
                const float4_t z0 = zp[0], z1 = zp[1];
#pragma unroll
                for (int i = 0; i < 4; ++i) { v[i] = z0[i]; v[4 + i] = z1[i]; }
                had128_row16(v, lane);
                const half8_t sv = blk ? sv_blk[1] : sv_blk[0];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = (v[i] * kRsqrt128) * (float)sv[i];
                const size_t at = (size_t)(m0 + mb * 32 + row) * ldc + gn + 8 * l16;
                if (p.out_fp32) {
                    global_ptr<float4_t> dst = (global_ptr<float4_t>)(as_global((float*)cout) + at);
                    dst[0] = float4_t{v[0], v[1], v[2], v[3]};
                    dst[1] = float4_t{v[4], v[5], v[6], v[7]};
                } else {
                    half8_t o;
#pragma unroll
                    for (int i = 0; i < 8; ++i) o[i] = (_Float16)v[i];
                    *(global_ptr<half8_t>)(as_global((_Float16*)cout) + at) = o;
                }
            }
        }
    }
}

// Dense launches: blockIdx.x = (tile - tile0) * S + split with tiles numbered row
// block by row block, so that one linear can be issued as several launches with
// different split factors.  Grouped launches: blockIdx.x = column block * S + split,
// blockIdx.y the linear, blockIdx.z the problem, so that the workgroups of the (few)
// real problems of every linear are dispatched before the empty tail of the list.
template <int BITS, int CB, int MB>
__global__ __launch_bounds__(256, 2) void exl3_gemm_kernel(GemmParams p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int unit = blockIdx.x / p.S;
    const int split = blockIdx.x - unit * p.S;
    const int nblocks = ((p.N + 255) >> 8) * (p.num_slices > 0 ? p.num_slices : 1);
    KRange kr;
    kr.kb0 = split;
    kr.kb1 = p.K >> 7;
    kr.step = p.S;
    kr.part = split;
    kr.parts = p.S;
    if (!p.problems) {
        const int tile = p.tile0 + unit;
        kr.counter = (size_t)unit;
        kr.slot0 = kr.counter * p.S;
        gemm_tile<BITS, CB, MB, true>(p, tile / nblocks, tile % nblocks, kr, 0, smem);
        return;
    }
    if ((int)blockIdx.z >= *p.num_problems) return;
    // grouped: (linear, problem, column block)
    kr.counter = ((size_t)blockIdx.y * p.tiles_y + blockIdx.z) * nblocks + unit;
    kr.slot0 = kr.counter * p.S;
    gemm_tile<BITS, CB, MB, false>(p, blockIdx.z, unit, kr, blockIdx.y, smem, p.problems);
}

// Grouped launch over two problem lists at once: blockIdx.z < max_big takes a problem of up
// to 128 rows (weights decoded once for all of them, so an expert with many rows costs one
// decode per 128 rows instead of one per 32), the values after that the problems of up to 32
// rows.  Both kinds sit in one launch, the long tiles first, so the short ones fill in around
// them (as two launches the 128-row tiles would run alone on a fraction of the compute units).
// blockIdx.x = column block (whole K per workgroup: no hand-over), blockIdx.y the linear.
// Measured and dropped: cutting K in two with the split-K hand-over, for every tile or for the
// 128-row tiles only (the shorter units pack better, the hand-over of 128 KB of partial sums per
// tile costs far more than that gains: 150 -> 183 us per layer), 128-column units whose four waves
// cut K in two and add through LDS (gate + up of 256 tokens x 512 experts 61.3 -> 54.9 us, but its
// down projection 32.0 -> 39.6 and both launches of 64 tokens x 128 experts 5 - 6 us slower: twice
// the units pay twice the problem -> expert -> pointer chain), and resident workgroups that take units
// from a counter (the same schedule as the hardware's, with slower code).
template <int BITS, int CB>
__global__ __launch_bounds__(256, 2) void exl3_gemm_mixed_kernel(GemmParams p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    KRange kr;
    kr.kb0 = 0;
    kr.kb1 = p.K >> 7;
    kr.step = 1;
    kr.part = 0;
    kr.parts = 1;
    kr.counter = 0;
    kr.slot0 = 0;
    const int z = blockIdx.z;
    if (z < p.max_big) {
        if (z >= *p.num_big) return;
        gemm_tile<BITS, CB, 4, false>(p, z, blockIdx.x, kr, blockIdx.y, smem, p.big_problems);
        return;
    }
    if (z - p.max_big >= *p.num_problems) return;
    gemm_tile<BITS, CB, 1, false>(p, z - p.max_big, blockIdx.x, kr, blockIdx.y, smem, p.problems);
}

// Dense launches whose tile count does not divide over the compute units: the
// (tile, k-block) units of the launch, tile-major, are cut into gridDim.x equal
// contiguous ranges, one per workgroup (two workgroups per compute unit), so every
// workgroup does the same amount of decode and MFMA work.  A range covers the end
// of one tile, possibly whole tiles, and the start of another; a tile shared by
// several workgroups is finished by the last of them to arrive, which adds the
// partial sums in k order, so the result does not depend on timing.
// Workgroup w owns unit_q + 1 units if w < unit_r, else unit_q (units = unit_q * G + unit_r),
// starting at w * unit_q + min(w, unit_r).  32-bit arithmetic on workgroup-uniform values
// only, so the k loop and its addresses stay in scalar registers as in the plain kernel.
__device__ __forceinline__ int range_start(const GemmParams& p, int w) { return w * p.unit_q + min(w, p.unit_r); }
__device__ __forceinline__ int range_owner(const GemmParams& p, int x)
{
    const int big = p.unit_r * (p.unit_q + 1);      // units held by the workgroups with one extra
    return x < big ? x / (p.unit_q + 1) : p.unit_r + (x - big) / p.unit_q;
}

// Workgroups are handed to the eight compute dies round-robin (workgroup i runs on die
// i % 8), and every die has its own L2.  Renumbering them so that a die gets a contiguous
// eighth of the ranges makes the tiles of one die share their rows of the activation
// (one 128-row block, 1.3 MB at K = 5120, instead of all of them): a quarter less traffic
// behind the L2 on the 27B gate projection at 512 rows.
__device__ __forceinline__ int die_major_index(int i, int n)
{
    return (n & 7) == 0 ? (i & 7) * (n >> 3) + (i >> 3) : i;
}

template <int BITS, int CB, int MB>
__device__ __forceinline__ void gemm_segment(const GemmParams& p, const int w, const int u, const int stop,
                                             unsigned char* smem)
{
    const int nblocks = ((p.N + 255) >> 8) * (p.num_slices > 0 ? p.num_slices : 1);
    const int KB = p.K >> 7;
    const int tile = u / KB;
    const int t0 = tile * KB;                                   // the tile's first unit
    const int w_first = range_owner(p, t0);
    const int w_last = range_owner(p, t0 + KB - 1);
    KRange kr;
    kr.kb0 = u - t0;
    kr.kb1 = stop - t0;
    kr.step = 1;
    kr.part = w - w_first;
    kr.parts = w_last - w_first + 1;
    kr.counter = (size_t)tile;
    kr.slot0 = (size_t)tile * p.max_parts;
    const int t = p.tile0 + tile;
    gemm_tile<BITS, CB, MB, true>(p, t / nblocks, t % nblocks, kr, 0, smem);
}

// A range runs through the end of one tile, any whole tiles after it and the start of another.
template <int BITS, int CB, int MB>
__global__ __launch_bounds__(256, 2) void exl3_gemm_balanced_kernel(GemmParams p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int KB = p.K >> 7;
    const int w = die_major_index((int)blockIdx.x, (int)gridDim.x);
    const int u_end = range_start(p, w + 1);
    int u = range_start(p, w);
    // the first two segments are written out (as the body of a loop the compiler's scheduler does
    // not reliably keep the interleaved order of the main loop); the loop takes the rest
    {
        const int stop = min(u_end, (u / KB + 1) * KB);
        gemm_segment<BITS, CB, MB>(p, w, u, stop, smem);
        u = stop;
    }
    if (u < u_end) {
        __syncthreads();                                        // the epilogue's LDS tile is the next A tile
        const int stop = min(u_end, (u / KB + 1) * KB);
        gemm_segment<BITS, CB, MB>(p, w, u, stop, smem);
        u = stop;
    }
    while (u < u_end) {
        __syncthreads();
        const int stop = min(u_end, (u / KB + 1) * KB);
        gemm_segment<BITS, CB, MB>(p, w, u, stop, smem);
        u = stop;
    }
}

}  // namespace berth

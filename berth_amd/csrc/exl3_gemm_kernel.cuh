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
// fill the chip).  Partial accumulators go to the library workspace in register
// layout; the last workgroup to arrive (self-resetting counter) adds them in split
// order and runs the epilogue, so the result does not depend on timing.
#pragma once

#include "exl3_gemv_kernel.cuh"

namespace berth {

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
    int tiles_y;                // dense: row blocks; grouped: capacity of the problem list
    int tile0;                  // dense: first (row block, column block) tile of this launch, row-major
    // split-K
    int S;
    float* partials;            // [unit][S][4 waves][MB][2][16][64]
    unsigned* counters;         // [unit]
};

constexpr int kAStride = 128 + 8;   // halves per LDS row of the A tile (272 B: conflict-free b128 reads)

// one output tile: rows of problem / row block `tile_y`, 256 columns
template <int BITS, int CB, int MB>  // MB = 32-row blocks per workgroup
__device__ __forceinline__ void gemm_tile(const GemmParams& p, const int tile_y, const int nblk, const int split,
                                          const int which, unsigned char* smem)
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
    const int n0 = nblk * 256;
    int m0 = tile_y * BM;
    int m_end = p.M;
    ExpertLin lin = p.lin;
    if (p.problems) {
        const GroupProblem gp = p.problems[tile_y];
        lin = gp.expert == p.shared_expert ? p.shared[p.lin_base + which]
                                           : p.experts[gp.expert * p.lins_per_expert + p.lin_base + which];
        m0 = gp.row0;
        m_end = gp.row0 + gp.nrows;
    }
    const int rows_here = min(BM, m_end - m0);          // >= 1
    const _Float16* a_had = p.a_had[which];
    void* cout = p.c[which];
    const int nw = n0 + wave * 64;                      // first column of this wave
    const bool active = nw < p.N;
    const int tn = p.N >> 4;
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
        if (active && split < KB) {
            const global_ptr<const uint32_t> tb = as_global(lin.trellis) + (size_t)half_id * row_dw +
                                                 (size_t)((nw >> 4) + (slot >> 3)) * tile_dw + (slot & 7) * BITS;
            const int arow = m0 + min(slot, rows_here - 1);         // rows past the problem repeat its last row
            const global_ptr<const half8_t> ab =
                (global_ptr<const half8_t>)(as_global(a_had) + (size_t)arow * p.K + 16 * half_id);
            uint32_t cur[4][BITS];
            half8_t av[4][2];
            {
                const global_ptr<const uint32_t> t0 = tb + (size_t)(split * 8) * row_dw;
                const global_ptr<const half8_t> a0 = ab + split * 16;
#pragma unroll
                for (int st = 0; st < 4; ++st) {
                    load_tile_dwords<BITS>(t0 + (size_t)(2 * st) * row_dw, cur[st]);
                    av[st][0] = a0[4 * st];
                    av[st][1] = a0[4 * st + 1];
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            for (int kb = split; kb < KB; kb += p.S) {
                const int nkb = kb + p.S < KB ? kb + p.S : kb;
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

        // Both operands run one k-block ahead in registers: the trellis dwords of the
        // wave's four steps (nxt) and this thread's share of the A tile (a_nxt, 32 bytes
        // per 256-thread pass).  The A tile is double-buffered in LDS, so a k-block costs
        // one barrier.
        constexpr int kAPasses = BM * 8 / 256;
        uint32_t nxt[4][BITS];
        uint4 a_nxt[kAPasses][2];
        const int a_row = threadIdx.x >> 3, a_ch = threadIdx.x & 7;       // + 32 rows per pass
        auto load_a = [&](int kb) {
    #pragma unroll
            for (int ps = 0; ps < kAPasses; ++ps) {
                const int r = a_row + 32 * ps;
                uint4 v0 = {0, 0, 0, 0}, v1 = {0, 0, 0, 0};
                if (m0 + r < m_end) {
                    const uint4* src = (const uint4*)(a_had + (size_t)(m0 + r) * p.K + kb * 128 + a_ch * 16);
                    v0 = src[0];
                    v1 = src[1];
                }
                a_nxt[ps][0] = v0;
                a_nxt[ps][1] = v1;
            }
        };
        auto load_b = [&](int kb) {
            const uint32_t* nb = tbase + (size_t)(kb * 8) * row_dw;
    #pragma unroll
            for (int st = 0; st < 4; ++st)
    #pragma unroll
                for (int j = 0; j < BITS; ++j) nxt[st][j] = nb[(size_t)(2 * st) * row_dw + j];
        };
        if (split < KB) {
            load_a(split);
            if (active) load_b(split);
        }

        int buf = 0;
        for (int kb = split; kb < KB; kb += p.S, buf ^= 1) {
            uint32_t cur[4][BITS];
    #pragma unroll
            for (int st = 0; st < 4; ++st)
    #pragma unroll
                for (int j = 0; j < BITS; ++j) cur[st][j] = nxt[st][j];

            // publish this k-block's A tile; the other buffer may still be read by slower waves
            _Float16* a_buf = a_tile + (size_t)buf * BM * kAStride;
    #pragma unroll
            for (int ps = 0; ps < kAPasses; ++ps) {
                uint4* dst = (uint4*)(a_buf + (a_row + 32 * ps) * kAStride + a_ch * 16);
                dst[0] = a_nxt[ps][0];
                dst[1] = a_nxt[ps][1];
            }
            if (kb + p.S < KB) {
                load_a(kb + p.S);
                if (active) load_b(kb + p.S);
            }
            __syncthreads();

            if (active) {
    #pragma unroll
                for (int st = 0; st < 4; ++st) {
                    uint32_t prev = fetch_prev(lane, cur[st][BITS - 1]);
                    uint32_t w2[16];
                    decode_lane<BITS, CB>(cur[st], prev, w2);
                    half8_t b[2][2];
    #pragma unroll
                    for (int f = 0; f < 2; ++f)
    #pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const uint4 q = {w2[2 * f + h], w2[4 + 2 * f + h], w2[8 + 2 * f + h], w2[12 + 2 * f + h]};
                            b[f][h] = __builtin_bit_cast(half8_t, q);
                        }
                    // A operand: row = mb*32 + slot, k = 32*st + 16*half_id + 8h .. +7 inside the k-block
    #pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        if (MB > 1 && mb * 32 >= rows_here) break;          // workgroup-uniform
                        const _Float16* arow = a_buf + (mb * 32 + slot) * kAStride + 32 * st + 16 * half_id;
                        const half8_t a0 = *(const half8_t*)(arow);
                        const half8_t a1 = *(const half8_t*)(arow + 8);
                        acc[mb][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b[0][0], acc[mb][0], 0, 0, 0);
                        acc[mb][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b[1][0], acc[mb][1], 0, 0, 0);
                        acc[mb][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b[0][1], acc[mb][0], 0, 0, 0);
                        acc[mb][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b[1][1], acc[mb][1], 0, 0, 0);
                    }
                }
            }
        }

    }

    // ---- split-K handoff.  Register r of a lane holds tile row 8*(r/4) + 4*half_id + r%4,
    // so only registers with 8*(r/4) < rows matter.
    if (p.S > 1) {
        const int nblocks = (p.N + 255) >> 8;
        // dense: tiles of this launch count from 0; grouped: (linear, problem, column block)
        const size_t unit = p.problems ? ((size_t)which * p.tiles_y + tile_y) * nblocks + nblk
                                       : (size_t)tile_y * nblocks + nblk - p.tile0;
        constexpr size_t kPerWg = (size_t)4 * MB * 2 * 16 * 64;
        float* mine = p.partials + (unit * p.S + split) * kPerWg + (size_t)wave * MB * 2 * 16 * 64;
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
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned old = __hip_atomic_fetch_add(p.counters + unit, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = (old == (unsigned)(p.S - 1)) ? 1u : 0u;
        }
        __syncthreads();
        if (!s_last) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (threadIdx.x == 0) __hip_atomic_store(p.counters + unit, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (active) {
            const float* all = p.partials + unit * p.S * kPerWg + (size_t)wave * MB * 2 * 16 * 64;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int f = 0; f < 2; ++f) {
                    if (mb * 32 >= rows_here) continue;
                    // sixteen registers x four splits in flight together; adds in split order
                    float sum[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) sum[r] = 0.0f;
                    for (int ss = 0; ss < p.S; ss += 4) {
                        float part[4][16];
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const int sj = ss + j < p.S ? ss + j : p.S - 1;      // past the end: re-read, ignored
#pragma unroll
                            for (int r = 0; r < 16; ++r)
                                part[j][r] = __hip_atomic_load(all + (size_t)sj * kPerWg + ((mb * 2 + f) * 16 + r) * 64 + lane,
                                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
#pragma unroll
                        for (int j = 0; j < 4; ++j)
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                const float nv = sum[r] + part[j][r];
                                sum[r] = ss + j < p.S ? nv : sum[r];
                            }
                    }
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[mb][f][r] = sum[r];
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
        sv_blk[blk] = gn < p.N ? ((global_ptr<const half8_t>)as_global(lin.svh + gn))[l16] : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
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
            if (row < rows_blk && gn < p.N) {
                float v[8];
                const float4_t* zp = (const float4_t*)&z_tile[row * kZStride + blk * 128 + 8 * l16];
                const float4_t z0 = zp[0], z1 = zp[1];
#pragma unroll
                for (int i = 0; i < 4; ++i) { v[i] = z0[i]; v[4 + i] = z1[i]; }
                had128_row16(v, lane);
                const half8_t sv = blk ? sv_blk[1] : sv_blk[0];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = (v[i] * kRsqrt128) * (float)sv[i];
                const size_t at = (size_t)(m0 + mb * 32 + row) * p.N + gn + 8 * l16;
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
    if (!p.problems) {
        const int nblocks = (p.N + 255) >> 8;
        const int tile = p.tile0 + unit;
        gemm_tile<BITS, CB, MB>(p, tile / nblocks, tile % nblocks, split, 0, smem);
        return;
    }
    if ((int)blockIdx.z >= *p.num_problems) return;
    gemm_tile<BITS, CB, MB>(p, blockIdx.z, unit, split, blockIdx.y, smem);
}

}  // namespace berth

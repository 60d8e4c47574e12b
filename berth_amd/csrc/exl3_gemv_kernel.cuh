// EXL3 linear for 1..8 rows per problem: trellis decode fused into a VALU dot
// product.  One kernel body serves the dense entry points (one problem, the
// whole grid) and the grouped MoE launches (one problem per routed expert chunk,
// several linears per launch).
//
//   c = ( Hh(x * suh) @ W ) -> Hh(.) * svh          (Hh = 128-block Hadamard / sqrt(128))
//
//   * a wave owns (128 output columns) x (128-row k-blocks); per k-block it
//     rotates the activation itself (fp32 butterflies, rounded to fp16, written
//     to a_had by the column-block-0 workgroups when a_had is given), streams 8
//     tile rows with one `bits`-dword load per lane, decodes 32 weights per lane
//     and accumulates fp32 dot products against the rotated activation in LDS;
//   * the 4 waves of a workgroup split K and reduce in LDS in wave order;
//   * if K is split over S workgroups the partial sums go to the library's
//     workspace and the last workgroup to arrive adds them in split order,
//     applies the output Hadamard and svh and stores c.  The arrival counter
//     resets itself.  Summation order never depends on timing.
//   * the input row of a problem can be gathered (routed tokens) and can be the
//     SiLU gate silu(g) * u of two fp16 rows, evaluated with the same stepwise
//     fp16 arithmetic as the stand-alone SiLU kernel.
#pragma once

#include <stddef.h>

#include "exl3_decode.cuh"
#include "hadamard.cuh"
#include "moe_route.cuh"

namespace berth {

// device-resident description of one EXL3 linear (matches berth_exl3_lin)
struct ExpertLin {
    const uint32_t* trellis;
    const _Float16* suh;
    const _Float16* svh;
};

struct GemvParams {
    // input rows: x[r] = a + src(r) * K, src(r) = gather ? gather[r] / gather_div : r.
    // With a_up the input is silu(a[r]) * a_up[r] (both in row order r).
    const _Float16* a;
    const _Float16* a_up;
    const int32_t* gather;
    int gather_div;
    // dense mode (problems == nullptr): one linear, rows 0..rows-1
    ExpertLin lin;
    int rows;
    // grouped mode: problem list built on the device; blockIdx.y selects which of
    // the `lin_base + blockIdx.y`-th linear of each expert and the output buffer
    const ExpertLin* experts;
    const GroupProblem* problems;
    const int* num_problems;
    int lins_per_expert;
    int lin_base;
    ExpertLin shared[3];        // an always-on expert passed by value (problem.expert == shared_expert)
    int shared_expert;
    int pair;                   // dense mode with gridDim.y == 2: linear shared[blockIdx.y] on the same rows
    // multi-linear mode (multi != 0), the argument lists of
    // crates/berth-kernels/src/ops.rs:264-293, all device arrays: one problem per
    // entry of b_list; multi == 2 is the sliced form (per-slice width, row stride
    // and source index; outputs through c_ptrs), multi == 1 the uniform form
    const uint64_t* b_list;
    const uint64_t* suh_list;
    const uint64_t* svh_list;
    const uint64_t* c_ptrs;
    const int* size_n_list;
    const int* n_stride_list;
    const int* had_src_list;
    int multi;
    int multi_in_rows;          // rows between the inputs of consecutive problems (0: shared input)
    void* c[2];                 // output per blockIdx.y, rows in problem order
    _Float16* a_had;            // optional (dense mode only)
    float* partials;            // [problem][lin][NB][S][MMAX][128]
    unsigned* counters;         // [problem][lin][NB], cstride words apart
    int cstride;
    int K, N, NB, KB, S, out_fp32;
    int half_units;             // 1: a unit of the K walk is half a k-block (one row only)
    // one-token expert combine folded into the down projection (grouped mode, one
    // row per problem, fp32 rows in c[0]): the last problem to finish a column
    // block writes comb_out[h] = fma chain over j of comb_w[j] * c[0][comb_inv[j]][h]
    // starting from comb_shared[h] (or 0), the arithmetic of the separate combine
    // kernel.  comb_out == nullptr: off.
    const float* comb_w;
    const int32_t* comb_inv;
    const float* comb_shared;
    float* comb_out;
    unsigned* comb_counters;    // [NB], cstride words apart, zero between launches
    int comb_k;
    // Single hand-over form of the folded combine (comb_sv != nullptr; at most kCombMaxProblems
    // problems, problem i's row is row i): the split-K parts of *all* problems of a column
    // block are counted on one counter, and the last workgroup to arrive finishes every
    // problem of the block (parts in split order, output rotation, output scale) and then
    // runs the chain, so the rows never wait for a second counter.  comb_sv takes a copy of
    // each problem's output scale [unit][64 half2] so that the finisher needs no expert
    // record; comb_shared_prob is the problem whose row starts the chain (-1: comb_shared or 0).
    uint32_t* comb_sv;
    int comb_shared_prob;
    // Grouped one-row launches.  ROUTE instantiation: where the wave that stores the routing
    // results also leaves the records of linear `resolved_lin` of the experts in sorted order,
    // then of the always-on expert (null: nowhere).  Other instantiations: `resolved` non-null
    // replaces the problem list and the expert table (problem i is row i, linear resolved[i];
    // the grid holds exactly the problems there are).
    const ExpertLin* resolved;
    int resolved_lin;
    ExpertLin* resolved_out;
    // grouped mode, one token, ROUTE instantiation: there is no problem list yet; problem i is
    // the selected expert with sorted position i, which every wave works out itself from the
    // router's segment sums (route.parts); the first workgroup's first wave stores the routing
    // results for the launches that follow.  route.k (+ 1 with an always-on expert) problems.
    RouteParams route;
};

constexpr int kCombMaxProblems = 16;

// silu(g) * u with every step rounded to fp16: e = exp(-g); s = 1 + e; r = 1 / s;
// t = g * r; out = t * u (crates/berth-kernels/csrc/ops/act.cu:35-69 and its fixture)
__device__ __forceinline__ _Float16 silu_mul_h(_Float16 g, _Float16 u)
{
    _Float16 e = (_Float16)expf(-(float)g);
    _Float16 s = (_Float16)1.0f + e;
    _Float16 r = (_Float16)(1.0f / (float)s);
    _Float16 t = g * r;
    return t * u;
}

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

template <int BITS>
__device__ __forceinline__ void load_tile_dwords(global_ptr<const uint32_t> p, uint32_t (&out)[BITS])
{
    if constexpr (BITS % 4 == 0) {
#pragma unroll
        for (int j = 0; j < BITS / 4; ++j) {
            const u32x4_t v = *((global_ptr<const u32x4_t>)p + j);
            out[4 * j] = v.x; out[4 * j + 1] = v.y; out[4 * j + 2] = v.z; out[4 * j + 3] = v.w;
        }
    } else if constexpr (BITS % 2 == 0) {
#pragma unroll
        for (int j = 0; j < BITS / 2; ++j) {
            const u32x2_t v = *((global_ptr<const u32x2_t>)p + j);
            out[2 * j] = v.x; out[2 * j + 1] = v.y;
        }
    } else {
#pragma unroll
        for (int j = 0; j < BITS; ++j) out[j] = *((global_ptr<const uint32_t>)p + j);
    }
}

// what one wave needs to walk its k-blocks
struct GemvWalk {
    global_ptr<const uint32_t> tbase;   // tile row 0 of the wave's column block
    global_ptr<const half2_t> suh;
    global_ptr<const _Float16> a;
    global_ptr<const _Float16> a_up;
    global_ptr<_Float16> a_had;         // row 0 of this problem's slab
    size_t row_dw;                      // dwords per tile row
    int K, KB, kb0, step, rows;
};

// The K loop of one wave.  Rolling prefetch: the 8 tile rows of a k-block live in
// registers; as soon as a tile row has been decoded its registers are reloaded
// with the same tile row of the wave's next k-block, so loads stay one k-block
// ahead of the decode.  The loop body is straight-line code with loads only (the
// a_had store lives in its own instantiation, used by the column-block-0
// workgroups): with a store or a branch in the body the compiler's wait counts
// degrade to "wait for everything", which serialises the pipeline.
//
// TRS is the number of tile rows of a k-block one unit of the walk covers: 8 (a whole
// k-block per unit) or 4 (half a k-block: both halves rotate the whole 128-element block
// of the activation, each decodes only its 4 tile rows).  Half units double the number of
// waves a narrow, shallow weight can spread over.  The walk's step is a multiple of 4, so
// which half a wave owns never changes along its walk.
template <int BITS, int CB, int MMAX, bool SILU, bool WRITE_HAD, int TRS>
__device__ __forceinline__ void gemv_accumulate(const GemvWalk& w, const int (&src)[MMAX],
                                                uint32_t (&xs)[MMAX][64], float (&acc)[MMAX][2])
{
    const int lane = threadIdx.x & 63;
    const int lane_dw = lane * BITS;
    const int rows = w.rows;
#pragma unroll
    for (int m = 0; m < MMAX; ++m) acc[m][0] = acc[m][1] = 0.0f;

    constexpr int UPK = 8 / TRS;                        // units per k-block
    uint32_t own[TRS][BITS];
    half2_t xr[MMAX], ur[MMAX], sc;
    int unit = w.kb0;                                   // w.kb0, w.step and w.KB count units
    if (unit >= w.KB) return;
    const int sub = unit % UPK;                         // constant along the walk
    int kb = unit / UPK;
    {
        // same issue order as inside the loop (activation first, then the tile rows),
        // so that the wait counts the compiler derives at the loop head stay exact
        sc = w.suh[kb * 64 + lane];
#pragma unroll
        for (int m = 0; m < MMAX; ++m) {
            if (MMAX > 1 && m >= rows) break;
            xr[m] = ((global_ptr<const half2_t>)(w.a + (size_t)src[m] * w.K + kb * 128))[lane];
            if (SILU) ur[m] = ((global_ptr<const half2_t>)(w.a_up + (size_t)src[m] * w.K + kb * 128))[lane];
        }
        __builtin_amdgcn_sched_barrier(0);
        const global_ptr<const uint32_t> base = w.tbase + (size_t)(kb * 8 + sub * TRS) * w.row_dw;
#pragma unroll
        for (int tr = 0; tr < TRS; ++tr) {
            load_tile_dwords<BITS>(base + tr * w.row_dw + lane_dw, own[tr]);
            __builtin_amdgcn_sched_barrier(0);          // tile row 0 must be the oldest load in flight
        }
    }

    for (; unit < w.KB; unit += w.step) {
        kb = unit / UPK;
        const int nunit = unit + w.step;
        const int nkb = nunit / UPK;
        const bool has_next = nunit < w.KB;
        const int pkb = has_next ? nkb : kb;            // k-block whose activation is prefetched
        // rotate this k-block of the activation: Hh(x * suh), rounded to fp16
#pragma unroll
        for (int m = 0; m < MMAX; ++m) {
            if (MMAX > 1 && m >= rows) break;           // wave-uniform; rows past `rows` are never read
            half2_t x = xr[m];
            if (SILU) {
                x.x = silu_mul_h(x.x, ur[m].x);
                x.y = silu_mul_h(x.y, ur[m].y);
            }
            float v0 = (float)x.x * (float)sc.x;
            float v1 = (float)x.y * (float)sc.y;
            had128_wave(v0, v1, lane);
            half2_t r;
            r.x = (_Float16)(v0 * kRsqrt128);
            r.y = (_Float16)(v1 * kRsqrt128);
            xs[m][lane] = as_u32(r);
            if (WRITE_HAD && (UPK == 1 || sub == 0))
                ((global_ptr<half2_t>)(w.a_had + (size_t)m * w.K + kb * 128))[lane] = r;
        }
        sc = w.suh[pkb * 64 + lane];
#pragma unroll
        for (int m = 0; m < MMAX; ++m) {
            if (MMAX > 1 && m >= rows) break;
            xr[m] = ((global_ptr<const half2_t>)(w.a + (size_t)src[m] * w.K + pkb * 128))[lane];
            if (SILU) ur[m] = ((global_ptr<const half2_t>)(w.a_up + (size_t)src[m] * w.K + pkb * 128))[lane];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        __builtin_amdgcn_sched_barrier(0);

        // No branch inside the tile-row loop (the compiler would sink the decode below
        // it): a wave on its last k-block re-reads tile row 0 of its column block,
        // always the same cached KiB, and ignores the result.
        const global_ptr<const uint32_t> nbase =
            w.tbase + (has_next ? (size_t)(nkb * 8 + sub * TRS) * w.row_dw : (size_t)0);
        const size_t nrow_dw = has_next ? w.row_dw : 0;
        const uint32_t* xsub = &xs[0][sub * TRS * 8];
#pragma unroll
        for (int tr = 0; tr < TRS; ++tr) {
            uint32_t prev = fetch_prev(lane, own[tr][BITS - 1]);
            uint32_t w2[16];
            decode_lane<BITS, CB>(own[tr], prev, w2);
            load_tile_dwords<BITS>(nbase + tr * nrow_dw + lane_dw, own[tr]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int m = 0; m < MMAX; ++m) {
                if (MMAX > 1 && m >= rows) break;       // wave-uniform
                const uint4* xp = (const uint4*)(xsub + m * 64 + tr * 8);
                uint4 xa = xp[0], xb = xp[1];
                const uint32_t xk[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
                for (int q = 0; q < 16; ++q)
                    acc[m][pair_col_half(q)] = __builtin_amdgcn_fdot2(
                        as_half2(w2[q]), as_half2(xk[pair_kk(q)]), acc[m][pair_col_half(q)], false);
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

template <int BITS, int CB, int MMAX, bool SILU, int TRS = 8, bool ROUTE = false>
__global__ __launch_bounds__(256, 4) void exl3_gemv_kernel(GemvParams p)
{
    __shared__ uint32_t xs[4][MMAX][64];    // wave-private: rotated k-block, one half2 per entry
    __shared__ float red[4][MMAX][128];
    __shared__ unsigned s_last;

    // every field the other instantiations read sits in the first six lines of the argument block
    static_assert(offsetof(GemvParams, resolved) + 8 <= 6 * 64 && sizeof(GemvParams) > 9 * 64 &&
                  sizeof(GemvParams) <= 10 * 64, "the argument block's lines as they are touched here");
    touch_kernel_arguments<ROUTE ? 10 : 6>();
    const int lane = threadIdx.x & 63;
    // wave-uniform on purpose: everything derived from it (k-block, addresses) stays in SGPRs
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int per_problem = p.NB * p.S;
    const int prob = blockIdx.x / per_problem;
    const int local = blockIdx.x - prob * per_problem;
    const int nb = local % p.NB;
    const int s = local / p.NB;
    const int which = blockIdx.y;

    ExpertLin lin = p.pair ? p.shared[which] : p.lin;
    int row0 = 0, rows = p.rows;
    auto expert_lin = [&](int expert) -> ExpertLin {
        return expert == p.shared_expert ? p.shared[p.lin_base + which]
                                         : p.experts[expert * p.lins_per_expert + p.lin_base + which];
    };
    if constexpr (ROUTE) {
        static_assert(MMAX == 1 && !SILU, "the inline routing serves the one-token gate / up launch");
        // One wave works the routing out and the others take its answer: a quarter of the reads
        // of the segment sums, which every workgroup of the launch wants at the same moment
        // (measured: 1.2 us off the layer against all four waves doing it side by side).
        __shared__ int s_expert;
        if (wave == 0) {
            // The first workgroup's first wave stores the routing results.  It also leaves, for
            // the launch that follows, the record of linear `resolved_lin` of the expert at
            // each sorted position (then of the always-on expert), so that that launch reaches
            // its weights with one dependent read instead of two.  It asks for the records of
            // all experts (at most 128: lane l holds experts l and l + 64) ahead of the
            // routing, so that its stores do not wait for a read that depends on the routing.
            const bool writer = blockIdx.x == 0 && blockIdx.y == 0;
            const bool resolve = writer && p.resolved_out;
            unsigned rec[2][6];
            if (resolve) {
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int e2 = min(lane + 64 * i, p.route.E - 1);
                    const unsigned* src = (const unsigned*)(p.experts + e2 * p.lins_per_expert + p.resolved_lin);
#pragma unroll
                    for (int q = 0; q < 6; ++q) rec[i][q] = src[q];
                }
            }
            const RouteOneToken r = route_one_token(p.route, lane, writer);
            const int e = route_expert_at(p.route, r, lane, prob);
            if (lane == 0) s_expert = e;
            if (resolve) {
                unsigned got[6];
#pragma unroll
                for (int q = 0; q < 6; ++q) {
                    const unsigned lo = (unsigned)__shfl((int)rec[0][q], r.sel & 63, 64);
                    const unsigned hi = (unsigned)__shfl((int)rec[1][q], r.sel & 63, 64);
                    got[q] = r.sel >= 64 ? hi : lo;
                }
                if (lane < p.route.k) {
                    unsigned* dst = (unsigned*)(p.resolved_out + r.rank);
#pragma unroll
                    for (int q = 0; q < 6; ++q) dst[q] = got[q];
                }
                if (lane == 0 && p.shared_expert >= 0) p.resolved_out[p.route.k] = p.shared[p.resolved_lin];
            }
        }
        __syncthreads();
        const int expert = __builtin_amdgcn_readfirstlane(s_expert);
        lin = expert_lin(expert);
        row0 = prob;
        rows = 1;
    } else if (p.resolved) {
        // one-row problems whose linears an earlier launch resolved: problem i is row i
        lin = p.resolved[prob];
        row0 = prob;
        rows = 1;
    } else if (p.problems) {
        // the list holds an entry for every problem index of the grid: this one is read
        // together with the count, not after it (one dependent read less ahead of the
        // first weight load); the empty asm keeps the compiler from sinking the read
        // below the branch again
        const GroupProblem gp = p.problems[prob];
        const int count = *p.num_problems;
        asm volatile("" ::"s"(gp.expert), "s"(count));
        if (prob >= count) return;
        lin = expert_lin(gp.expert);
        row0 = gp.row0;
        rows = gp.nrows;
    }
    int n_stride = p.N;             // columns of the full weight: tile-row stride and output row stride
    int in_row0 = 0;                // first input row of this problem
    int had_slab = 0;               // a_had slab of this problem
    void* cout = p.c[which];
    if (p.multi) {
        lin.trellis = (const uint32_t*)p.b_list[prob];
        lin.svh = (const _Float16*)p.svh_list[prob];
        if (p.multi == 2) {
            if (nb * 128 >= p.size_n_list[prob]) return;
            n_stride = p.n_stride_list[prob];
            had_slab = p.had_src_list[prob];
            lin.suh = (const _Float16*)p.suh_list[had_slab];
            cout = (void*)p.c_ptrs[prob];
        } else {
            lin.suh = (const _Float16*)p.suh_list[prob];
            had_slab = prob;
            in_row0 = prob * p.multi_in_rows;
            cout = (char*)p.c[0] + (size_t)prob * p.rows * p.N * (p.out_fp32 ? 4 : 2);
        }
    }
    const int unit = (prob * (int)gridDim.y + which) * p.NB + nb;   // counter / partial slot

    const int wc = p.S * 4;
    const int tn = n_stride >> 4;
    constexpr int tile_dw = 8 * BITS;
    const size_t row_dw = (size_t)tn * tile_dw;   // dwords per tile row

    // source row of each of this problem's rows
    int src[MMAX];
#pragma unroll
    for (int m = 0; m < MMAX; ++m) {
        int r = row0 + in_row0 + (m < rows ? m : 0);
        src[m] = ROUTE ? 0 : (p.gather ? p.gather[r] / p.gather_div : r);
    }

    float acc[MMAX][2];
    {
        GemvWalk w;
        w.tbase = as_global(lin.trellis) + (size_t)(nb * 8) * tile_dw;
        w.suh = (global_ptr<const half2_t>)as_global(lin.suh);
        w.a = as_global(p.a);
        w.a_up = as_global(p.a_up);
        w.a_had = as_global(p.a_had) + ((size_t)had_slab * rows + row0) * p.K;
        w.row_dw = row_dw;
        w.K = p.K;
        w.KB = p.KB * (8 / TRS);
        w.kb0 = s * 4 + wave;
        w.step = wc;
        w.rows = rows;
        if (p.a_had && nb == 0 && which == 0) gemv_accumulate<BITS, CB, MMAX, SILU, true, TRS>(w, src, xs[wave], acc);
        else gemv_accumulate<BITS, CB, MMAX, SILU, false, TRS>(w, src, xs[wave], acc);
    }

    // ---- reduce the 4 waves (k split inside the workgroup), wave order
    const int col = (lane >> 3) * 16 + (lane & 7);
#pragma unroll
    for (int m = 0; m < MMAX; ++m) {
        red[wave][m][col] = acc[m][0];
        red[wave][m][col + 8] = acc[m][1];
    }
    __syncthreads();

    const int t = threadIdx.x;
    float z[MMAX];
    if (t < 128) {
#pragma unroll
        for (int m = 0; m < MMAX; ++m)
            z[m] = ((red[0][m][t] + red[1][m][t]) + red[2][m][t]) + red[3][m][t];
    }

    // the output scale is requested before the hand-over, whose waits it would otherwise queue behind
    const half2_t sv = ((global_ptr<const half2_t>)as_global(lin.svh + nb * 128))[lane];

    if constexpr (SILU && MMAX == 1) {
        if (p.comb_sv) {
            // ---- one hand-over for split-K and combine (see GemvParams::comb_sv).  Every value
            // below is formed by the operations, in the order, of the two-stage path further
            // down (parts added in split order from 0.0f when S > 1, rotation, 1/sqrt(128), output
            // scale, fma chain in slot order), so the two paths give the same bits.
            __shared__ float crow[kCombMaxProblems][128];
            const int count = min(*p.num_problems, kCombMaxProblems);
            float* mine = p.partials + ((size_t)unit * p.S + s) * 128;
            if (t < 128) __hip_atomic_store(mine + t, z[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (s == 0 && wave == 0)
                __hip_atomic_store(p.comb_sv + (size_t)unit * 64 + lane, as_u32(sv), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            wait_own_stores();
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __syncthreads();
            if (t == 0) {
                unsigned old = __hip_atomic_fetch_add(p.comb_counters + (size_t)nb * p.cstride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                s_last = (old + 1 == (unsigned)(count * p.S)) ? 1u : 0u;
            }
            __syncthreads();
            if (!s_last) return;
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            if (t == 0) __hip_atomic_store(p.comb_counters + (size_t)nb * p.cstride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

            union Pair { unsigned long long u; float f[2]; };
            const int col0 = nb * 128;
            // operands of the chain, written by an earlier launch: lane j holds slot j's
            float wj = 0.0f;
            int rj = 0;
            if (lane < p.comb_k) {
                wj = p.comb_w[lane];
                rj = p.comb_inv[lane];
            }
            float start = 0.0f;
            if (t < 128 && p.comb_shared_prob < 0 && p.comb_shared) start = p.comb_shared[col0 + t];

            // wave w finishes problems w, w + 4, w + 8, w + 12; all their parts are requested
            // in batches of sixteen rows, then added in split order
            const int mine_n = count > wave ? (count - wave + 3) >> 2 : 0;
            const int total = mine_n * p.S;
            uint32_t svj[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int j = wave + 4 * q;
                svj[q] = j < count ? __hip_atomic_load(p.comb_sv + ((size_t)j * p.NB + nb) * 64 + lane, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT)
                                   : 0u;
            }
            float zz[4][2] = {};
            int jl = 0, sp = 0;
            for (int r0 = 0; r0 < total; r0 += 16) {
                Pair part[16];
                const int jl0 = jl, sp0 = sp;
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    part[u].u = 0ull;
                    if (r0 + u < total) {
                        const float* row = p.partials + ((size_t)((size_t)(wave + 4 * jl) * p.NB + nb) * p.S + sp) * 128;
                        part[u].u = __hip_atomic_load((const unsigned long long*)(row + 2 * lane), __ATOMIC_RELAXED,
                                                      __HIP_MEMORY_SCOPE_AGENT);
                    }
                    if (++sp == p.S) { sp = 0; ++jl; }
                }
                jl = jl0;
                sp = sp0;
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    if (r0 + u < total) {
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            if (jl == q) {
                                zz[q][0] = p.S == 1 ? part[u].f[0] : zz[q][0] + part[u].f[0];
                                zz[q][1] = p.S == 1 ? part[u].f[1] : zz[q][1] + part[u].f[1];
                            }
                    }
                    if (++sp == p.S) { sp = 0; ++jl; }
                }
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int j = wave + 4 * q;
                if (j < count) {
                    float v0 = zz[q][0], v1 = zz[q][1];
                    had128_wave(v0, v1, lane);
                    const half2_t sj = as_half2(svj[q]);
                    v0 = (v0 * kRsqrt128) * (float)sj.x;
                    v1 = (v1 * kRsqrt128) * (float)sj.y;
                    crow[j][2 * lane] = v0;
                    crow[j][2 * lane + 1] = v1;
                    // the row itself, for callers that read the rows of the projection
                    float2_t o = {v0, v1};
                    *(float2_t*)((float*)cout + (size_t)j * n_stride + col0 + 2 * lane) = o;
                }
            }
            __syncthreads();
            if (t < 128) {
                float a = p.comb_shared_prob >= 0 && p.comb_shared_prob < count ? crow[p.comb_shared_prob][t] : start;
                for (int j = 0; j < p.comb_k; ++j) {
                    const float wv = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), j));
                    const int r = __builtin_amdgcn_readlane(rj, j);
                    const float row = (unsigned)r < (unsigned)count ? crow[r][t] : 0.0f;
                    a = __builtin_fmaf(wv, row, a);
                }
                p.comb_out[col0 + t] = a;
            }
            return;
        }
    }

    if (p.S > 1) {
        // ---- cross-workgroup split-K: last arrival reduces in split order.
        // The partial sums travel as agent-scope atomic stores and loads, which go
        // straight to the level of the memory hierarchy all compute dies share, so
        // no cache-wide write-back or invalidate is needed: it is enough that this
        // workgroup's stores have completed (every wave waits for its own) before the
        // arrival counter is bumped.
        float* mine = p.partials + ((size_t)((size_t)unit * p.S + s) * MMAX) * 128;
        if (t < 128) {
#pragma unroll
            for (int m = 0; m < MMAX; ++m)
                if (MMAX == 1 || m < rows)
                    __hip_atomic_store(mine + m * 128 + t, z[m], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        wait_own_stores();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (t == 0) {
            unsigned old = __hip_atomic_fetch_add(p.counters + (size_t)unit * p.cstride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = (old == (unsigned)(p.S - 1)) ? 1u : 0u;
        }
        __syncthreads();
        if (!s_last) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (t < 128) {
            const float* all = p.partials + ((size_t)((size_t)unit * p.S) * MMAX) * 128;
#pragma unroll
            for (int m = 0; m < MMAX; ++m) z[m] = 0.0f;
            // all loads of a batch in flight together; the adds stay in split order
            constexpr int PB = MMAX == 1 ? 16 : 4;
            for (int s0 = 0; s0 < p.S; s0 += PB) {
                float part[PB][MMAX];
#pragma unroll
                for (int j = 0; j < PB; ++j)
#pragma unroll
                    for (int m = 0; m < MMAX; ++m)
                        part[j][m] = (s0 + j < p.S && (MMAX == 1 || m < rows))
                            ? __hip_atomic_load(all + ((size_t)(s0 + j) * MMAX + m) * 128 + t, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT)
                            : 0.0f;
#pragma unroll
                for (int j = 0; j < PB; ++j)
#pragma unroll
                    for (int m = 0; m < MMAX; ++m)
                        if (s0 + j < p.S) z[m] += part[j][m];
            }
        }
        if (t == 0) __hip_atomic_store(p.counters + (size_t)unit * p.cstride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- output Hadamard, svh, store
    __syncthreads();            // everyone is done reading red[]
    if (t < 128) {
#pragma unroll
        for (int m = 0; m < MMAX; ++m) red[0][m][t] = z[m];
    }
    __syncthreads();
    for (int m = wave; m < rows; m += 4) {
        float v0 = red[0][m][2 * lane];
        float v1 = red[0][m][2 * lane + 1];
        had128_wave(v0, v1, lane);
        v0 = (v0 * kRsqrt128) * (float)sv.x;
        v1 = (v1 * kRsqrt128) * (float)sv.y;
        size_t at = (size_t)(row0 + m) * n_stride + nb * 128 + 2 * lane;
        if constexpr (SILU && MMAX == 1) {
            if (p.comb_out) {
                // m == 0, wave 0.  The row goes out as agent-scope atomic stores so
                // that whichever workgroup arrives last can read every row of this
                // column block without a cache write-back; the stores have to be
                // complete before the arrival is counted.
                union Pair { unsigned long long u; float f[2]; };
                Pair mine;
                mine.f[0] = v0;
                mine.f[1] = v1;
                __hip_atomic_store((unsigned long long*)((float*)cout + at), mine.u, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                unsigned old = 0;
                if (lane == 0)
                    old = __hip_atomic_fetch_add(p.comb_counters + (size_t)nb * p.cstride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                old = (unsigned)__builtin_amdgcn_readfirstlane((int)old);
                if (old + 1 != (unsigned)*p.num_problems) return;
                if (lane == 0) __hip_atomic_store(p.comb_counters + (size_t)nb * p.cstride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                const int h = nb * 128 + 2 * lane;
                Pair acc2;
                acc2.u = 0ull;
                if (p.comb_shared)
                    acc2.u = __hip_atomic_load((const unsigned long long*)(p.comb_shared + h), __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
                float a0 = acc2.f[0], a1 = acc2.f[1];
                // eight rows in flight at a time; the fma chain stays in slot order
                for (int j0 = 0; j0 < p.comb_k; j0 += 8) {
                    Pair part[8];
                    float wj[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int j = j0 + u < p.comb_k ? j0 + u : p.comb_k - 1;
                        wj[u] = p.comb_w[j];
                        const float* row = (const float*)cout + (size_t)p.comb_inv[j] * n_stride + h;
                        part[u].u = __hip_atomic_load((const unsigned long long*)row, __ATOMIC_RELAXED,
                                                      __HIP_MEMORY_SCOPE_AGENT);
                    }
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        if (j0 + u < p.comb_k) {
                            a0 = __builtin_fmaf(wj[u], part[u].f[0], a0);
                            a1 = __builtin_fmaf(wj[u], part[u].f[1], a1);
                        }
                }
                float2_t o2 = {a0, a1};
                *(float2_t*)(p.comb_out + h) = o2;
                return;
            }
        }
        if (p.out_fp32) {
            float2_t o = {v0, v1};
            *(float2_t*)((float*)cout + at) = o;
        } else {
            half2_t o = {(_Float16)v0, (_Float16)v1};
            *(half2_t*)((_Float16*)cout + at) = o;
        }
    }
}

}  // namespace berth

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

#include "exl3_decode.cuh"
#include "hadamard.cuh"

namespace berth {

// device-resident description of one EXL3 linear (matches berth_exl3_lin)
struct ExpertLin {
    const uint32_t* trellis;
    const _Float16* suh;
    const _Float16* svh;
};

// one unit of grouped work: rows [row0, row0 + nrows) of the expert-sorted order
struct GroupProblem {
    int expert;
    int row0;
    int nrows;
    int pad;
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
    void* c[2];                 // output per blockIdx.y, rows in problem order
    _Float16* a_had;            // optional (dense mode only)
    float* partials;            // [problem][lin][NB][S][MMAX][128]
    unsigned* counters;         // [problem][lin][NB]
    int K, N, NB, KB, S, out_fp32;
};

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

template <int BITS>
__device__ __forceinline__ void load_tile_dwords(const uint32_t* __restrict__ p, uint32_t (&out)[BITS])
{
    if constexpr (BITS % 4 == 0) {
        const uint4* q = (const uint4*)p;
#pragma unroll
        for (int j = 0; j < BITS / 4; ++j) {
            uint4 v = q[j];
            out[4 * j] = v.x; out[4 * j + 1] = v.y; out[4 * j + 2] = v.z; out[4 * j + 3] = v.w;
        }
    } else if constexpr (BITS % 2 == 0) {
        const uint2* q = (const uint2*)p;
#pragma unroll
        for (int j = 0; j < BITS / 2; ++j) {
            uint2 v = q[j];
            out[2 * j] = v.x; out[2 * j + 1] = v.y;
        }
    } else {
#pragma unroll
        for (int j = 0; j < BITS; ++j) out[j] = p[j];
    }
}

template <int BITS, int CB, int MMAX>
__global__ __launch_bounds__(256) void exl3_gemv_kernel(GemvParams p)
{
    __shared__ uint32_t xs[4][MMAX][64];    // wave-private: rotated k-block, one half2 per entry
    __shared__ float red[4][MMAX][128];
    __shared__ unsigned s_last;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int per_problem = p.NB * p.S;
    const int prob = blockIdx.x / per_problem;
    const int local = blockIdx.x - prob * per_problem;
    const int nb = local % p.NB;
    const int s = local / p.NB;
    const int which = blockIdx.y;

    ExpertLin lin = p.lin;
    int row0 = 0, rows = p.rows;
    if (p.problems) {
        if (prob >= *p.num_problems) return;
        const GroupProblem gp = p.problems[prob];
        lin = p.experts[gp.expert * p.lins_per_expert + p.lin_base + which];
        row0 = gp.row0;
        rows = gp.nrows;
    }
    const int unit = (prob * (int)gridDim.y + which) * p.NB + nb;   // counter / partial slot

    const int wc = p.S * 4;
    const int tn = p.N >> 4;
    constexpr int tile_dw = 8 * BITS;
    const int paddr = prev_lane_addr(lane);
    const size_t row_dw = (size_t)tn * tile_dw;   // dwords per tile row

    // source row of each of this problem's rows
    int src[MMAX];
#pragma unroll
    for (int m = 0; m < MMAX; ++m) {
        int r = row0 + (m < rows ? m : 0);
        src[m] = p.gather ? p.gather[r] / p.gather_div : r;
    }

    float acc[MMAX][2];
#pragma unroll
    for (int m = 0; m < MMAX; ++m) acc[m][0] = acc[m][1] = 0.0f;

    for (int kb = s * 4 + wave; kb < p.KB; kb += wc) {
        uint32_t own[8][BITS];
        const uint32_t* base = lin.trellis + (size_t)(kb * 8) * row_dw + (size_t)(nb * 8) * tile_dw + lane * BITS;
#pragma unroll
        for (int tr = 0; tr < 8; ++tr) load_tile_dwords<BITS>(base + tr * row_dw, own[tr]);

        // rotate this k-block of the activation: Hh(x * suh), rounded to fp16
        const half2_t sc = ((const half2_t*)(lin.suh + kb * 128))[lane];
#pragma unroll
        for (int m = 0; m < MMAX; ++m) {
            if (MMAX > 1 && m >= rows) break;               // wave-uniform; rows past `rows` are never read
            half2_t x = ((const half2_t*)(p.a + (size_t)src[m] * p.K + kb * 128))[lane];
            if (p.a_up) {
                const half2_t u = ((const half2_t*)(p.a_up + (size_t)src[m] * p.K + kb * 128))[lane];
                x.x = silu_mul_h(x.x, u.x);
                x.y = silu_mul_h(x.y, u.y);
            }
            float v0 = (float)x.x * (float)sc.x;
            float v1 = (float)x.y * (float)sc.y;
            had128_wave(v0, v1, lane);
            half2_t r;
            r.x = (_Float16)(v0 * kRsqrt128);
            r.y = (_Float16)(v1 * kRsqrt128);
            xs[wave][m][lane] = as_u32(r);
            if (p.a_had && nb == 0)
                ((half2_t*)(p.a_had + (size_t)(row0 + m) * p.K + kb * 128))[lane] = r;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

#pragma unroll
        for (int tr = 0; tr < 8; ++tr) {
            uint32_t prev = fetch_prev(paddr, own[tr][BITS - 1]);
            uint32_t w2[16];
            decode_lane<BITS, CB>(own[tr], prev, w2);
#pragma unroll
            for (int m = 0; m < MMAX; ++m) {
                if (MMAX > 1 && m >= rows) break;           // wave-uniform
                const uint4* xp = (const uint4*)&xs[wave][m][tr * 8];
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

    if (p.S > 1) {
        // ---- cross-workgroup split-K: last arrival reduces in split order.
        // The partial sums travel as agent-scope atomic stores and loads, which go
        // straight to the level of the memory hierarchy all compute dies share, so
        // no cache-wide write-back or invalidate is needed: it is enough that this
        // workgroup's stores have completed (the workgroup-scope release waits for
        // them) before the arrival counter is bumped.
        float* mine = p.partials + ((size_t)((size_t)unit * p.S + s) * MMAX) * 128;
        if (t < 128) {
#pragma unroll
            for (int m = 0; m < MMAX; ++m)
                __hip_atomic_store(mine + m * 128 + t, z[m], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (t == 0) {
            unsigned old = __hip_atomic_fetch_add(p.counters + unit, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = (old == (unsigned)(p.S - 1)) ? 1u : 0u;
        }
        __syncthreads();
        if (!s_last) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (t < 128) {
            const float* all = p.partials + ((size_t)((size_t)unit * p.S) * MMAX) * 128;
#pragma unroll
            for (int m = 0; m < MMAX; ++m) z[m] = 0.0f;
            // loads in flight eight splits at a time; the adds stay in split order
            for (int s0 = 0; s0 < p.S; s0 += 8) {
                float part[8][MMAX];
#pragma unroll
                for (int j = 0; j < 8; ++j)
#pragma unroll
                    for (int m = 0; m < MMAX; ++m)
                        part[j][m] = (s0 + j < p.S)
                            ? __hip_atomic_load(all + ((size_t)(s0 + j) * MMAX + m) * 128 + t, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT)
                            : 0.0f;
#pragma unroll
                for (int j = 0; j < 8; ++j)
#pragma unroll
                    for (int m = 0; m < MMAX; ++m)
                        if (s0 + j < p.S) z[m] += part[j][m];
            }
        }
        if (t == 0) __hip_atomic_store(p.counters + unit, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- output Hadamard, svh, store
    __syncthreads();            // everyone is done reading red[]
    if (t < 128) {
#pragma unroll
        for (int m = 0; m < MMAX; ++m) red[0][m][t] = z[m];
    }
    __syncthreads();
    const half2_t sv = ((const half2_t*)(lin.svh + nb * 128))[lane];
    void* cout = p.c[which];
    for (int m = wave; m < rows; m += 4) {
        float v0 = red[0][m][2 * lane];
        float v1 = red[0][m][2 * lane + 1];
        had128_wave(v0, v1, lane);
        v0 = (v0 * kRsqrt128) * (float)sv.x;
        v1 = (v1 * kRsqrt128) * (float)sv.y;
        size_t at = (size_t)(row0 + m) * p.N + nb * 128 + 2 * lane;
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

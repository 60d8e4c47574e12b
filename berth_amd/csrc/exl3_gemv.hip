// EXL3 linear for 1..8 rows: trellis decode fused into a VALU dot product.
//
//   c = ( Hh(a * suh) @ W ) -> Hh(.) * svh          (Hh = 128-block Hadamard / sqrt(128))
//
// One launch does the whole operator of crates/berth-kernels/csrc/linear.cu:209-286
// (the m = 1 path the reference routes to its int8 GEMV) and of the small-row
// cases of crates/berth-kernels/csrc/prefill_lin/linear.cu:277-343:
//   * a wave owns (128 output columns) x (128-row k-blocks); per k-block it
//     rotates the activation itself (fp32 butterflies, rounded to fp16, written
//     to a_had by the column-block-0 workgroups), streams 8 tile rows of 1 KiB
//     (at 4 bpw) with one `bits`-dword load per lane, decodes 32 weights per lane
//     and accumulates fp32 dot products against the rotated activation in LDS;
//   * the 4 waves of a workgroup split K and reduce in LDS in wave order;
//   * if K is split over S workgroups the partial sums go to the library's
//     workspace and the last workgroup to arrive adds them in split order,
//     applies the output Hadamard and svh and stores c.  The arrival counter
//     resets itself.  Summation order never depends on timing.
#include "exl3_decode.cuh"
#include "hadamard.cuh"
#include "launch.h"

#include <cstdlib>

namespace berth {

struct GemvParams {
    const _Float16* a;
    const uint32_t* trellis;
    void* c;
    const _Float16* suh;
    _Float16* a_had;
    const _Float16* svh;
    float* partials;        // [NB][S][MMAX][128]
    unsigned* counters;     // [NB]
    int rows, K, N, NB, KB, S, out_fp32;
};

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
    const int nb = blockIdx.x % p.NB;
    const int s = blockIdx.x / p.NB;
    const int wc = p.S * 4;
    const int tn = p.N >> 4;
    constexpr int tile_dw = 8 * BITS;
    const int paddr = prev_lane_addr(lane);
    const size_t row_dw = (size_t)tn * tile_dw;   // dwords per tile row

    float acc[MMAX][2];
#pragma unroll
    for (int m = 0; m < MMAX; ++m) acc[m][0] = acc[m][1] = 0.0f;

    for (int kb = s * 4 + wave; kb < p.KB; kb += wc) {
        uint32_t own[8][BITS];
        const uint32_t* base = p.trellis + (size_t)(kb * 8) * row_dw + (size_t)(nb * 8) * tile_dw + lane * BITS;
#pragma unroll
        for (int tr = 0; tr < 8; ++tr) load_tile_dwords<BITS>(base + tr * row_dw, own[tr]);

        // rotate this k-block of the activation: Hh(a * suh), rounded to fp16
        const half2_t sc = ((const half2_t*)(p.suh + kb * 128))[lane];
#pragma unroll
        for (int m = 0; m < MMAX; ++m) {
            half2_t x = {(_Float16)0, (_Float16)0};
            if (m < p.rows) x = ((const half2_t*)(p.a + (size_t)m * p.K + kb * 128))[lane];
            float v0 = (float)x.x * (float)sc.x;
            float v1 = (float)x.y * (float)sc.y;
            had128_wave(v0, v1, lane);
            half2_t r;
            r.x = (_Float16)(v0 * kRsqrt128);
            r.y = (_Float16)(v1 * kRsqrt128);
            xs[wave][m][lane] = as_u32(r);
            if (nb == 0 && m < p.rows)
                ((half2_t*)(p.a_had + (size_t)m * p.K + kb * 128))[lane] = r;
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
        // ---- cross-workgroup split-K: last arrival reduces in split order
        float* mine = p.partials + ((size_t)(nb * p.S + s) * MMAX) * 128;
        if (t < 128) {
#pragma unroll
            for (int m = 0; m < MMAX; ++m)
                __hip_atomic_store(mine + m * 128 + t, z[m], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // The partial sums travel as agent-scope atomic stores and loads, which go
        // straight to the level of the memory hierarchy all compute dies share, so
        // no cache-wide write-back or invalidate is needed: it is enough that this
        // wave's stores have completed (the workgroup-scope release waits for them)
        // before the arrival counter is bumped.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (t == 0) {
            unsigned old = __hip_atomic_fetch_add(p.counters + nb, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = (old == (unsigned)(p.S - 1)) ? 1u : 0u;
        }
        __syncthreads();
        if (!s_last) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (t < 128) {
            const float* all = p.partials + ((size_t)(nb * p.S) * MMAX) * 128;
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
        if (t == 0) __hip_atomic_store(p.counters + nb, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- output Hadamard, svh, store
    __syncthreads();            // everyone is done reading red[]
    if (t < 128) {
#pragma unroll
        for (int m = 0; m < MMAX; ++m) red[0][m][t] = z[m];
    }
    __syncthreads();
    const half2_t sv = ((const half2_t*)(p.svh + nb * 128))[lane];
    for (int m = wave; m < p.rows; m += 4) {
        float v0 = red[0][m][2 * lane];
        float v1 = red[0][m][2 * lane + 1];
        had128_wave(v0, v1, lane);
        v0 = (v0 * kRsqrt128) * (float)sv.x;
        v1 = (v1 * kRsqrt128) * (float)sv.y;
        size_t at = (size_t)m * p.N + nb * 128 + 2 * lane;
        if (p.out_fp32) {
            float2_t o = {v0, v1};
            *(float2_t*)((float*)p.c + at) = o;
        } else {
            half2_t o = {(_Float16)v0, (_Float16)v1};
            *(half2_t*)((_Float16*)p.c + at) = o;
        }
    }
}

template <int BITS, int CB>
static void launch_rows(const GemvParams& p, int mmax, int grid, hipStream_t stream)
{
    switch (mmax) {
    case 1: hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 1>), dim3(grid), dim3(256), 0, stream, p); break;
    case 2: hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 2>), dim3(grid), dim3(256), 0, stream, p); break;
    case 4: hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 4>), dim3(grid), dim3(256), 0, stream, p); break;
    default: hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 8>), dim3(grid), dim3(256), 0, stream, p); break;
    }
}

template <int BITS>
static void launch_cb(const GemvParams& p, int cb, int mmax, int grid, hipStream_t stream)
{
    switch (cb) {
    case 0: launch_rows<BITS, 0>(p, mmax, grid, stream); break;
    case 1: launch_rows<BITS, 1>(p, mmax, grid, stream); break;
    default: launch_rows<BITS, 2>(p, mmax, grid, stream); break;
    }
}

std::string launch_gemv(const LinearArgs& a)
{
    if (a.size_m < 1 || a.size_m > 8) throw std::runtime_error("exl3 gemv: rows must be in 1..=8");
    if (a.size_k % 128 != 0) throw std::runtime_error("exl3 linear: size_k must be a multiple of 128");
    Workspace& ws = workspace_for_current_device();
    const int mmax = a.size_m == 1 ? 1 : a.size_m == 2 ? 2 : a.size_m <= 4 ? 4 : 8;

    GemvParams p;
    p.a = (const _Float16*)a.a;
    p.trellis = (const uint32_t*)a.trellis;
    p.c = a.c;
    p.suh = (const _Float16*)a.suh;
    p.a_had = (_Float16*)a.a_had;
    p.svh = (const _Float16*)a.svh;
    p.partials = ws.partials;
    p.counters = ws.counters;
    p.rows = a.size_m;
    p.K = a.size_k;
    p.N = a.size_n;
    p.NB = a.size_n / 128;
    p.KB = a.size_k / 128;
    p.out_fp32 = a.out_fp32;

    // waves per column block: enough workgroups to cover the chip several times,
    // at most one k-block per wave
    static const int wg_per_cu = [] {
        const char* e = std::getenv("BERTH_GEMV_WG_PER_CU");
        int v = e ? std::atoi(e) : 0;
        return v > 0 ? v : 6;
    }();
    const long target_wg = (long)ws.cu_count * wg_per_cu;
    int S = (int)((target_wg + p.NB - 1) / p.NB);
    const int s_max = (p.KB + 3) / 4;
    if (S > s_max) S = s_max;
    if (S < 1) S = 1;
    while (S > 1 && (size_t)p.NB * S * mmax * 128 * sizeof(float) > kPartialBytes) --S;
    if (p.NB > kCounters) throw std::runtime_error("exl3 gemv: size_n exceeds the split-K counter table");
    p.S = S;
    const int grid = p.NB * S;

    switch (a.k_bits) {
    case 1: launch_cb<1>(p, a.codebook, mmax, grid, a.stream); break;
    case 2: launch_cb<2>(p, a.codebook, mmax, grid, a.stream); break;
    case 3: launch_cb<3>(p, a.codebook, mmax, grid, a.stream); break;
    case 4: launch_cb<4>(p, a.codebook, mmax, grid, a.stream); break;
    case 5: launch_cb<5>(p, a.codebook, mmax, grid, a.stream); break;
    case 6: launch_cb<6>(p, a.codebook, mmax, grid, a.stream); break;
    case 7: launch_cb<7>(p, a.codebook, mmax, grid, a.stream); break;
    default: launch_cb<8>(p, a.codebook, mmax, grid, a.stream); break;
    }
    hip_ok(hipGetLastError(), "exl3_gemv_kernel launch");
    return "exl3_gemv_kernel<" + std::to_string(a.k_bits) + "," + std::to_string(a.codebook) + "," +
           std::to_string(mmax) + "> grid=" + std::to_string(grid) + " block=256 split_k=" +
           std::to_string(S) + (a.out_fp32 ? " out=f32" : " out=f16");
}

}  // namespace berth

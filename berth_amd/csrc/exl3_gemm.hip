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
#include "exl3_gemv_kernel.cuh"
#include "launch.h"

#include <cstdlib>

namespace berth {

struct GemmParams {
    const _Float16* a_had[2];   // [rows][K], already rotated (one per linear of the launch)
    ExpertLin lin;              // dense mode
    void* c[2];
    int M, K, N, out_fp32;
    // grouped mode (problems != nullptr): blockIdx.y = problem (<= BM rows),
    // blockIdx.z = which of the launch's linears
    const ExpertLin* experts;
    const GroupProblem* problems;
    const int* num_problems;
    int lins_per_expert, lin_base;
    // split-K
    int S;
    float* partials;            // [unit][S][4 waves][MB][2][16][64]
    unsigned* counters;         // [unit]
};

constexpr int kAStride = 128 + 8;   // halves per LDS row of the A tile (272 B: conflict-free b128 reads)

template <int BITS, int CB, int MB>  // MB = 32-row blocks per workgroup
__global__ __launch_bounds__(256, 2) void exl3_gemm_kernel(GemmParams p)
{
    constexpr int BM = MB * 32;
    extern __shared__ __align__(16) unsigned char smem[];
    _Float16* a_tile = (_Float16*)smem;                 // [2][BM][kAStride]
    float* z_tile = (float*)smem;                       // epilogue: [32][256 + 4]
    constexpr int kZStride = 256 + 4;
    __shared__ unsigned s_last;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int half_id = lane >> 5;                      // which of the two tile rows
    const int slot = lane & 31;                         // MFMA row / column slot
    const int nblk = blockIdx.x / p.S;
    const int split = blockIdx.x - nblk * p.S;
    const int n0 = nblk * 256;
    const int which = blockIdx.z;
    int m0 = blockIdx.y * BM;
    int m_end = p.M;
    ExpertLin lin = p.lin;
    if (p.problems) {
        if ((int)blockIdx.y >= *p.num_problems) return;
        const GroupProblem gp = p.problems[blockIdx.y];
        lin = p.experts[gp.expert * p.lins_per_expert + p.lin_base + which];
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

    // ---- split-K handoff.  Register r of a lane holds tile row 8*(r/4) + 4*half_id + r%4,
    // so only registers with 8*(r/4) < rows matter.
    if (p.S > 1) {
        const int nblocks = (p.N + 255) >> 8;
        const size_t unit = ((size_t)blockIdx.z * gridDim.y + blockIdx.y) * nblocks + nblk;
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
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        if (mb * 32 + 8 * r4 >= rows_here) continue;
                        float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                        for (int ss = 0; ss < p.S; ss += 4) {
                            float part[4][4];
#pragma unroll
                            for (int j = 0; j < 4; ++j)
#pragma unroll
                                for (int q = 0; q < 4; ++q)
                                    part[j][q] = (ss + j < p.S)
                                        ? __hip_atomic_load(all + (size_t)(ss + j) * kPerWg +
                                                                ((mb * 2 + f) * 16 + 4 * r4 + q) * 64 + lane,
                                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                        : 0.0f;
#pragma unroll
                            for (int j = 0; j < 4; ++j)
#pragma unroll
                                for (int q = 0; q < 4; ++q)
                                    if (ss + j < p.S) sum[q] += part[j][q];
                        }
#pragma unroll
                        for (int q = 0; q < 4; ++q) acc[mb][f][4 * r4 + q] = sum[q];
                    }
                }
        }
    }

    // ---- epilogue, 32 rows at a time: stage fp32 tile, output Hadamard, svh, store
    const int col_in_wave = (slot >> 3) * 16 + (slot & 7);     // + 8f
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
        for (int task = wave; task < rows_blk * 2; task += 4) {
            const int row = task >> 1, blk = task & 1;
            const int gm = m0 + mb * 32 + row;
            const int gn = n0 + blk * 128;
            if (gn >= p.N) continue;
            float v0 = z_tile[row * kZStride + blk * 128 + 2 * lane];
            float v1 = z_tile[row * kZStride + blk * 128 + 2 * lane + 1];
            had128_wave(v0, v1, lane);
            const half2_t sv = ((const half2_t*)(lin.svh + gn))[lane];
            v0 = (v0 * kRsqrt128) * (float)sv.x;
            v1 = (v1 * kRsqrt128) * (float)sv.y;
            const size_t at = (size_t)gm * p.N + gn + 2 * lane;
            if (p.out_fp32) {
                float2_t o = {v0, v1};
                *(float2_t*)((float*)cout + at) = o;
            } else {
                half2_t o = {(_Float16)v0, (_Float16)v1};
                *(half2_t*)((_Float16*)cout + at) = o;
            }
        }
    }
}

template <int BITS, int CB, int MB>
static void gemm_launch_mb(const GemmParams& p, hipStream_t stream, std::string& desc, dim3 grid)
{
    constexpr int BM = MB * 32;
    const size_t smem_a = (size_t)2 * BM * kAStride * sizeof(_Float16);     // double-buffered A tile
    const size_t smem_z = (size_t)32 * (256 + 4) * sizeof(float);
    const size_t smem = smem_a > smem_z ? smem_a : smem_z;
    if (smem > 64 * 1024) {
        static const hipError_t attr = hipFuncSetAttribute((const void*)exl3_gemm_kernel<BITS, CB, MB>,
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        hip_ok(attr, "exl3_gemm_kernel shared-memory attribute");
    }
    hipLaunchKernelGGL((exl3_gemm_kernel<BITS, CB, MB>), grid, dim3(256), smem, stream, p);
    desc = "exl3_gemm_kernel<" + std::to_string(BITS) + "," + std::to_string(CB) + "," + std::to_string(BM) +
           "x256> grid=" + std::to_string(grid.x) + "x" + std::to_string(grid.y) + "x" + std::to_string(grid.z) +
           " split_k=" + std::to_string(p.S) + " smem=" + std::to_string(smem);
}

template <int BITS, int CB>
static void gemm_launch(const GemmParams& p, int mb, hipStream_t stream, std::string& desc, dim3 grid)
{
    if (mb == 1) gemm_launch_mb<BITS, CB, 1>(p, stream, desc, grid);
    else gemm_launch_mb<BITS, CB, 4>(p, stream, desc, grid);
}

template <int BITS>
static void gemm_cb(const GemmParams& p, int cb, int mb, hipStream_t stream, std::string& desc, dim3 grid)
{
    switch (cb) {
    case 0: gemm_launch<BITS, 0>(p, mb, stream, desc, grid); break;
    case 1: gemm_launch<BITS, 1>(p, mb, stream, desc, grid); break;
    default: gemm_launch<BITS, 2>(p, mb, stream, desc, grid); break;
    }
}

static void gemm_bits(const GemmParams& p, int bits, int cb, int mb, hipStream_t stream, std::string& desc, dim3 grid)
{
    switch (bits) {
    case 1: gemm_cb<1>(p, cb, mb, stream, desc, grid); break;
    case 2: gemm_cb<2>(p, cb, mb, stream, desc, grid); break;
    case 3: gemm_cb<3>(p, cb, mb, stream, desc, grid); break;
    case 4: gemm_cb<4>(p, cb, mb, stream, desc, grid); break;
    case 5: gemm_cb<5>(p, cb, mb, stream, desc, grid); break;
    case 6: gemm_cb<6>(p, cb, mb, stream, desc, grid); break;
    case 7: gemm_cb<7>(p, cb, mb, stream, desc, grid); break;
    default: gemm_cb<8>(p, cb, mb, stream, desc, grid); break;
    }
}

// split-K factor for `tiles` output tiles of MB*32 x 256: fill the chip about twice,
// keep at least two k-blocks per workgroup, stay inside the workspace
static int gemm_split(const Workspace& ws, long tiles, int KB, int mb)
{
    static const int per_cu = [] {
        const char* e = std::getenv("BERTH_GEMM_WG_PER_CU");
        int v = e ? std::atoi(e) : 0;
        return v > 0 ? v : 2;
    }();
    long S = ((long)ws.cu_count * per_cu + tiles - 1) / tiles;
    if (S > KB / 2) S = KB / 2;
    if (S < 1) S = 1;
    const size_t per_wg = (size_t)4 * mb * 2 * 16 * 64 * sizeof(float);
    while (S > 1 && (size_t)tiles * S * per_wg > kPartialBytes) --S;
    if (tiles > kCounters) S = 1;
    return (int)S;
}

std::string launch_gemm(const LinearArgs& a)
{
    if (a.size_k % 128 != 0) throw std::runtime_error("exl3 linear: size_k must be a multiple of 128");
    Workspace& ws = workspace_for_current_device();
    std::string d0 = launch_had_r_128(a.a, a.a_had, a.suh, 1, a.size_m, a.size_k, 0, a.stream);
    GemmParams p{};
    p.a_had[0] = (const _Float16*)a.a_had;
    p.lin.trellis = (const uint32_t*)a.trellis;
    p.lin.svh = (const _Float16*)a.svh;
    p.c[0] = a.c;
    p.M = a.size_m;
    p.K = a.size_k;
    p.N = a.size_n;
    p.out_fp32 = a.out_fp32;
    p.partials = ws.partials;
    p.counters = ws.counters;
    const int mb = a.size_m <= 32 ? 1 : 4;
    const int nblocks = (a.size_n + 255) / 256;
    const int mtiles = (a.size_m + mb * 32 - 1) / (mb * 32);
    p.S = gemm_split(ws, (long)nblocks * mtiles, a.size_k / 128, mb);
    std::string desc;
    gemm_bits(p, a.k_bits, a.codebook, mb, a.stream, desc, dim3(nblocks * p.S, mtiles, 1));
    hip_ok(hipGetLastError(), "exl3_gemm_kernel launch");
    return d0 + " + " + desc + (a.out_fp32 ? " out=f32" : " out=f16");
}

// grouped: problems of at most 32 rows each; a_had rows are in problem order
std::string launch_gemm_grouped(const GroupedArgs& g)
{
    if (g.size_k % 128 != 0 || g.size_n % 128 != 0)
        throw std::runtime_error("moe grouped linear: sizes must be multiples of 128");
    Workspace& ws = workspace_for_current_device();
    GemmParams p{};
    p.a_had[0] = (const _Float16*)g.a_had;
    p.a_had[1] = (const _Float16*)g.a_had2;
    p.c[0] = g.c0;
    p.c[1] = g.c1;
    p.M = 0;
    p.K = g.size_k;
    p.N = g.size_n;
    p.out_fp32 = g.out_fp32;
    p.experts = (const ExpertLin*)g.experts;
    p.problems = (const GroupProblem*)g.problems;
    p.num_problems = g.num_problems;
    p.lins_per_expert = g.lins_per_expert;
    p.lin_base = g.lin_base;
    p.partials = ws.partials;
    p.counters = ws.counters;
    const int nblocks = (g.size_n + 255) / 256;
    const long tiles = (long)g.max_problems * g.num_lins * nblocks;
    p.S = gemm_split(ws, tiles, g.size_k / 128, 1);
    if (g.max_problems > 65535) throw std::runtime_error("moe grouped linear: too many problems");
    std::string desc;
    gemm_bits(p, g.k_bits, g.codebook, 1, g.stream, desc, dim3(nblocks * p.S, g.max_problems, g.num_lins));
    hip_ok(hipGetLastError(), "exl3_gemm_kernel grouped launch");
    return desc + " grouped";
}

// ---- plain fp16 GEMM (crates/berth-kernels/csrc/prefill_lin/linear.cu:387-418):
// C[m][ldc] = A[m][k] @ B[k][n], fp32 accumulate.  One wave per 32x32 output
// tile, operands read straight from global memory.
__global__ __launch_bounds__(256) void hgemm_kernel(const _Float16* __restrict__ a,
                                                    const _Float16* __restrict__ b, void* c, int M,
                                                    int K, int N, int ldc, int c_fp32)
{
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int slot = lane & 31, kh = lane >> 5;
    const int m0 = blockIdx.y * 32;
    const int n0 = (blockIdx.x * 4 + wave) * 32;
    if (n0 >= N) return;
    float16_t acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    const int row = m0 + slot, col = n0 + slot;
    for (int k0 = 0; k0 < K; k0 += 16) {
        half8_t av, bv;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int k = k0 + 8 * kh + i;
            av[i] = (row < M && k < K) ? a[(size_t)row * K + k] : (_Float16)0;
            bv[i] = (col < N && k < K) ? b[(size_t)k * N + col] : (_Float16)0;
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, acc, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int gm = m0 + 8 * (r >> 2) + 4 * kh + (r & 3);
        if (gm < M && col < N) {
            if (c_fp32) ((float*)c)[(size_t)gm * ldc + col] = acc[r];
            else ((_Float16*)c)[(size_t)gm * ldc + col] = (_Float16)acc[r];
        }
    }
}

std::string launch_hgemm(const void* a, const void* b, void* c, int m, int k, int n, int ldc,
                         int c_fp32, hipStream_t stream)
{
    dim3 grid((n + 127) / 128, (m + 31) / 32);
    hipLaunchKernelGGL(hgemm_kernel, grid, dim3(256), 0, stream, (const _Float16*)a, (const _Float16*)b, c,
                       m, k, n, ldc, c_fp32);
    hip_ok(hipGetLastError(), "hgemm_kernel launch");
    return "hgemm_kernel grid=" + std::to_string(grid.x) + "x" + std::to_string(grid.y) + " block=256" +
           (c_fp32 ? " out=f32" : " out=f16");
}

}  // namespace berth

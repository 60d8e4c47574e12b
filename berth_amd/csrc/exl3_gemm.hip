// EXL3 linear for many rows: trellis decode fused into an fp16 MFMA GEMM
// (v_mfma_f32_32x32x16_f16, fp32 accumulate).  Covers the row counts the
// reference spreads over a cooperative GEMM (<= 144 rows) and reconstruct +
// dense GEMM (> 144 rows), crates/berth-kernels/csrc/prefill_lin/linear.cu:184-344;
// the weight is never written back to memory.
//
//   launch 1: a_had = Hh(a * suh)                        (had_r_128, pre-scale)
//   launch 2: c = Hh(a_had @ W) * svh                    (this file)
//
// Work split: a workgroup of 4 waves owns BM rows x 256 columns; each wave owns
// 64 of the columns for all BM rows, so decoded weights stay in the registers of
// the wave that decoded them.  Per 32 rows of K a wave decodes 2 tile rows x 4
// tile columns: lanes 0..31 take tile row kt, lanes 32..63 tile row kt+1, eight
// lanes per tile (octet layout).  The four register quads a lane ends up with
// ((column u or u+8) x (k 0..7 or 8..15 of its tile row)) are exactly four MFMA
// B operands: B[k-slot][col-slot] with col-slot = lane % 32 and k-slot =
// 8*(lane/32) + i.  The A operand for the same slots is a_had[row][16*(kt +
// lane/32) + 8h + i], one 16-byte LDS read.  Column slots map to columns
// 16*(slot/8) + slot%8 + 8f; the epilogue undoes that when it stages the fp32
// tile in LDS for the output Hadamard.
#include "exl3_gemv_kernel.cuh"
#include "launch.h"

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
};

constexpr int kAStride = 128 + 8;   // halves per LDS row of the A tile (272 B: conflict-free b128 reads)

template <int BITS, int CB, int MB>  // MB = 32-row blocks per workgroup
__global__ __launch_bounds__(256) void exl3_gemm_kernel(GemmParams p)
{
    constexpr int BM = MB * 32;
    extern __shared__ __align__(16) unsigned char smem[];
    _Float16* a_tile = (_Float16*)smem;                 // [BM][kAStride]
    float* z_tile = (float*)smem;                       // epilogue: [32][256 + 4]
    constexpr int kZStride = 256 + 4;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int half_id = lane >> 5;                      // which of the two tile rows
    const int slot = lane & 31;                         // MFMA row / column slot
    const int n0 = blockIdx.x * 256;
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
    const _Float16* a_had = p.a_had[which];
    void* cout = p.c[which];
    const int nw = n0 + wave * 64;                      // first column of this wave
    const bool active = nw < p.N;
    const int tn = p.N >> 4;
    constexpr int tile_dw = 8 * BITS;
    const size_t row_dw = (size_t)tn * tile_dw;
    const int paddr = prev_lane_addr(lane);
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

    uint32_t nxt[4][BITS];
    if (active) {
#pragma unroll
        for (int st = 0; st < 4; ++st)
#pragma unroll
            for (int j = 0; j < BITS; ++j) nxt[st][j] = tbase[(size_t)(2 * st) * row_dw + j];
    }

    for (int kb = 0; kb < KB; ++kb) {
        uint32_t cur[4][BITS];
#pragma unroll
        for (int st = 0; st < 4; ++st)
#pragma unroll
            for (int j = 0; j < BITS; ++j) cur[st][j] = nxt[st][j];

        __syncthreads();        // previous k-block's readers are done with a_tile
        // stage a_had[m0 .. m0+BM)[kb*128 .. +128) : 16 halves (32 B) per thread per pass
        for (int idx = threadIdx.x; idx < BM * 8; idx += 256) {
            const int r = idx >> 3, ch = idx & 7;
            uint4 v0 = {0, 0, 0, 0}, v1 = {0, 0, 0, 0};
            if (m0 + r < m_end) {
                const uint4* src = (const uint4*)(a_had + (size_t)(m0 + r) * p.K + kb * 128 + ch * 16);
                v0 = src[0];
                v1 = src[1];
            }
            uint4* dst = (uint4*)(a_tile + r * kAStride + ch * 16);
            dst[0] = v0;
            dst[1] = v1;
        }
        if (active && kb + 1 < KB) {
            const uint32_t* nb = tbase + (size_t)((kb + 1) * 8) * row_dw;
#pragma unroll
            for (int st = 0; st < 4; ++st)
#pragma unroll
                for (int j = 0; j < BITS; ++j) nxt[st][j] = nb[(size_t)(2 * st) * row_dw + j];
        }
        __syncthreads();

        if (active) {
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                uint32_t prev = fetch_prev(paddr, cur[st][BITS - 1]);
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
                    const _Float16* arow = a_tile + (mb * 32 + slot) * kAStride + 32 * st + 16 * half_id;
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

    // ---- epilogue, 32 rows at a time: stage fp32 tile, output Hadamard, svh, store
    const int col_in_wave = (slot >> 3) * 16 + (slot & 7);     // + 8f
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
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
        // 32 rows x 2 column blocks = 64 Hadamards, 16 per wave
        for (int task = wave; task < 64; task += 4) {
            const int row = task >> 1, blk = task & 1;
            const int gm = m0 + mb * 32 + row;
            const int gn = n0 + blk * 128;
            if (gm >= m_end || gn >= p.N) continue;
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

template <int BITS, int CB>
static void gemm_launch(const GemmParams& p, hipStream_t stream, std::string& desc, int grid_y = 0, int grid_z = 1)
{
    constexpr int MB = 4;
    constexpr int BM = MB * 32;
    const size_t smem_a = (size_t)BM * kAStride * sizeof(_Float16);
    const size_t smem_z = (size_t)32 * (256 + 4) * sizeof(float);
    const size_t smem = smem_a > smem_z ? smem_a : smem_z;
    dim3 grid((p.N + 255) / 256, grid_y ? grid_y : (p.M + BM - 1) / BM, grid_z);
    hipLaunchKernelGGL((exl3_gemm_kernel<BITS, CB, MB>), grid, dim3(256), smem, stream, p);
    desc = "exl3_gemm_kernel<" + std::to_string(BITS) + "," + std::to_string(CB) + "," + std::to_string(BM) +
           "x256> grid=" + std::to_string(grid.x) + "x" + std::to_string(grid.y) + " block=256 smem=" +
           std::to_string(smem);
}

template <int BITS>
static void gemm_cb(const GemmParams& p, int cb, hipStream_t stream, std::string& desc, int gy = 0, int gz = 1)
{
    switch (cb) {
    case 0: gemm_launch<BITS, 0>(p, stream, desc, gy, gz); break;
    case 1: gemm_launch<BITS, 1>(p, stream, desc, gy, gz); break;
    default: gemm_launch<BITS, 2>(p, stream, desc, gy, gz); break;
    }
}

static void gemm_bits(const GemmParams& p, int bits, int cb, hipStream_t stream, std::string& desc, int gy = 0, int gz = 1)
{
    switch (bits) {
    case 1: gemm_cb<1>(p, cb, stream, desc, gy, gz); break;
    case 2: gemm_cb<2>(p, cb, stream, desc, gy, gz); break;
    case 3: gemm_cb<3>(p, cb, stream, desc, gy, gz); break;
    case 4: gemm_cb<4>(p, cb, stream, desc, gy, gz); break;
    case 5: gemm_cb<5>(p, cb, stream, desc, gy, gz); break;
    case 6: gemm_cb<6>(p, cb, stream, desc, gy, gz); break;
    case 7: gemm_cb<7>(p, cb, stream, desc, gy, gz); break;
    default: gemm_cb<8>(p, cb, stream, desc, gy, gz); break;
    }
}

std::string launch_gemm(const LinearArgs& a)
{
    if (a.size_k % 128 != 0) throw std::runtime_error("exl3 linear: size_k must be a multiple of 128");
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
    std::string desc;
    gemm_bits(p, a.k_bits, a.codebook, a.stream, desc);
    hip_ok(hipGetLastError(), "exl3_gemm_kernel launch");
    return d0 + " + " + desc + (a.out_fp32 ? " out=f32" : " out=f16");
}

// grouped: problems of at most 128 rows each; a_had rows are in problem order
std::string launch_gemm_grouped(const GroupedArgs& g)
{
    if (g.size_k % 128 != 0 || g.size_n % 128 != 0)
        throw std::runtime_error("moe grouped linear: sizes must be multiples of 128");
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
    std::string desc;
    gemm_bits(p, g.k_bits, g.codebook, g.stream, desc, g.max_problems, g.num_lins);
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

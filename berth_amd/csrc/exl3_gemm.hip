// Launchers of the EXL3 MFMA GEMM (exl3_gemm_kernel.cuh): dense rows through
// berth_prefill_exl3_linear / berth_exl3_linear, grouped MoE problems, and the
// plain fp16 GEMM of crates/berth-kernels/csrc/prefill_lin/linear.cu:387-418.
#include "exl3_gemm_kernel.cuh"
#include "launch.h"

#include <cstdlib>
#include <cstring>

namespace berth {

static_assert(kGemmWrittenBase * 2 == kCounters, "the GEMM keeps two counters per tile");
static_assert(kGemmMaxSlices == kBundleMaxSlices, "one limit for the by-value slices of a bundle");

// one translation unit per codebook (exl3_gemm_cb{0,1,2}.hip) keeps the build parallel
void launch_gemm_cb0(const GemmParams& p, int bits, int mb, hipStream_t stream, std::string& desc, dim3 grid);
void launch_gemm_cb1(const GemmParams& p, int bits, int mb, hipStream_t stream, std::string& desc, dim3 grid);
void launch_gemm_cb2(const GemmParams& p, int bits, int mb, hipStream_t stream, std::string& desc, dim3 grid);

static void gemm_bits(const GemmParams& p, int bits, int cb, int mb, hipStream_t stream, std::string& desc, dim3 grid)
{
    switch (cb) {
    case 0: launch_gemm_cb0(p, bits, mb, stream, desc, grid); break;
    case 1: launch_gemm_cb1(p, bits, mb, stream, desc, grid); break;
    default: launch_gemm_cb2(p, bits, mb, stream, desc, grid); break;
    }
}

// split-K factor for `tiles` output tiles of MB*32 x 256: one workgroup per compute unit
// (fewer workgroups share a tile); two for a dense launch of at most 32 rows with at least a
// quarter as many tiles as compute units (a workgroup of four waves leaves a compute unit's
// vector pipes half idle, and each workgroup still keeps several k-blocks: the 27B gate + up
// bundle at 16 rows 63 -> 54 us; with few tiles the extra hand-overs cost more than that, q/k/v
// 24 -> 30 us, and with several row tiles nothing is gained: k at 512 rows 34.9 -> 36.0 us),
// at least two k-blocks per workgroup, inside the workspace
static int gemm_split(const Workspace& ws, long tiles, int KB, int mb, bool one_row_tile = false)
{
    const int per_cu = knobs().gemm_wg_per_cu > 0 ? knobs().gemm_wg_per_cu
                                                  : (mb == 1 && one_row_tile && tiles * 4 >= ws.cu_count ? 2 : 1);
    long S = ((long)ws.cu_count * per_cu + tiles - 1) / tiles;
    if (S > KB / 2) S = KB / 2;
    if (S < 1) S = 1;
    const size_t per_wg = (size_t)4 * mb * 2 * 16 * 64 * sizeof(float);
    while (S > 1 && (size_t)tiles * S * per_wg > kPartialBytes) --S;
    if (tiles > kCounters / 2) S = 1;          // two counters per tile
    return (int)S;
}

// words between the counters of neighbouring tiles (see counter_stride); `tiles` bounds the
// tile count of every launch the call makes
static int gemm_counter_stride(long tiles)
{
    const int cap = knobs().counter_stride;
    int stride = 1;
    while (stride * 2 <= cap && tiles * stride * 2 <= kCounters / 2) stride *= 2;
    return stride;
}

// Tile shape and work split of a dense launch: `nblocks` column blocks of 256 (all slices of
// a bundle together), size_m rows.  Fills the split fields of p and launches.
static void dispatch_dense(const Workspace& ws, GemmParams& p, int k_bits, int codebook, int size_m, int size_k,
                           int nblocks, hipStream_t stream, std::string& desc)
{
    // 128-row tiles decode a weight once per 128 rows, but need enough tiles to spread
    // over the chip; narrow outputs (few column tiles) run as 32-row tiles instead
    p.cstride = gemm_counter_stride((long)nblocks * ((size_m + 31) / 32));
    const long tiles128 = (long)nblocks * ((size_m + 127) / 128);
    const int mb_plain = (size_m <= 32 || tiles128 * 4 < ws.cu_count) ? 1 : 4;
    const int KB = size_k / 128;
    p.tile0 = 0;
    const int balance = knobs().gemm_balanced;
    // 0: never 256-row tiles; 1 (default): where they are faster; 2: wherever they are possible
    const int rows256 = knobs().gemm_rows256;
    // 128-row tiles rarely divide over the compute units (272 tiles on 256 units leave most of
    // the chip idle for the second half of the launch): deal the (tile, k-block) units out evenly.
    // 128-row tiles: one workgroup per compute unit (a wave interleaves its own decode with its
    // MFMAs, so a second workgroup per unit adds nothing and more workgroups share a tile: the 27B
    // down projection at 512 rows takes 147 us with 256 workgroups, 160 with 512).  256-row tiles
    // (more than 128 rows, wide outputs): a weight is decoded once per 256 rows; one workgroup of
    // eight waves fills a compute unit.
    auto balanced = [&](int mb) {
        const int mtiles = (size_m + mb * 32 - 1) / (mb * 32);
        const long tiles = (long)nblocks * mtiles;
        const long units = tiles * KB;
        long slots = ws.cu_count;
        if (balance > 1) slots = balance;
        const long G = units < slots ? units : slots;
        const long per_wg = units / G;                                   // >= 1
        const long parts = (KB + per_wg - 1) / per_wg + 1;               // workgroups that can share a tile
        const size_t part_bytes = (size_t)4 * mb * 2 * 16 * 64 * sizeof(float);
        if (!(tiles <= kCounters / 2 && units < (1L << 30) &&
              (size_t)tiles * parts * part_bytes <= kPartialBytes))
            return false;
        p.tiles_y = mtiles;
        p.S = 1;
        p.units = (int)units;
        p.unit_q = (int)(units / G);
        p.unit_r = (int)(units % G);
        p.max_parts = (int)parts;
        gemm_bits(p, k_bits, codebook, mb, stream, desc, dim3((unsigned)G, 1, 1));
        return true;
    };
    bool done = false;
    if (balance && mb_plain == 4) {
        // 256-row tiles pay when there are enough of them that few workgroups share a tile
        // (measured at 512 rows: gate/up 5120x17408, 136 tiles, 148 -> 139 us; q, o and down
        // with 40..48 tiles are 5 % slower than with 128-row tiles)
        const long tiles256 = (long)nblocks * ((size_m + 255) / 256);
        if (size_m > 128 && (rows256 >= 2 || (rows256 == 1 && tiles256 * 2 >= ws.cu_count))) done = balanced(8);
        if (!done) done = balanced(4);
    }
    if (!done) {
        const int mtiles = (size_m + mb_plain * 32 - 1) / (mb_plain * 32);
        const long tiles = (long)nblocks * mtiles;
        p.tiles_y = mtiles;
        p.units = 0;
        p.S = gemm_split(ws, tiles, KB, mb_plain, size_m <= 32);
        gemm_bits(p, k_bits, codebook, mb_plain, stream, desc, dim3((unsigned)(tiles * p.S), 1, 1));
    }
    hip_ok(hipGetLastError(), "exl3_gemm_kernel launch");
}

std::string launch_gemm(const LinearArgs& a)
{
    if (a.size_k % 128 != 0) throw std::runtime_error("exl3 linear: size_k must be a multiple of 128");
    LaunchScope scope(a.stream);
    Workspace& ws = scope.ws;
    throw_pending_device_fault(ws);
    std::string d0 = launch_had_r_128(a.a, a.a_had, a.suh, 1, a.size_m, a.size_k, 0, a.stream);
    GemmParams p{};
    p.fault = ws.fault_dev;
    p.spin_limit = spin_limit();
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
    std::string desc;
    dispatch_dense(ws, p, a.k_bits, a.codebook, a.size_m, a.size_k, (a.size_n + 255) / 256, a.stream, desc);
    return d0 + " + " + desc + (a.out_fp32 ? " out=f32" : " out=f16");
}

// berth_ops_mgemm with more than 8 rows: the bundle's linears as one dense MFMA launch behind
// one launch that rotates every distinct input (slab s of a_had = Hh(input(s) * suh[s])).
std::string launch_gemm_bundle(const MgemmArgs& m)
{
    if (m.size_k % 128 != 0) throw std::runtime_error("exl3_mgemm: size_k must be a multiple of 128");
    const bool sliced = m.had_src_list != nullptr;
    if (m.host_lists && m.bszm_out > kGemmMaxSlices)
        throw std::runtime_error("exl3_mgemm (host lists): at most " + std::to_string(kGemmMaxSlices) + " slices");
    LaunchScope scope(m.stream);
    Workspace& ws = scope.ws;
    throw_pending_device_fault(ws);
    const int slabs = sliced ? m.num_had_src : m.bszm_out;
    const size_t slab_stride = (size_t)m.size_m * m.size_k;
    GemmParams p{};
    p.fault = ws.fault_dev;
    p.spin_limit = spin_limit();
    p.a_had[0] = (const _Float16*)m.a_had;
    p.c[0] = m.c;
    p.M = m.size_m;
    p.K = m.size_k;
    p.N = m.size_n;
    p.out_fp32 = m.c_fp32;
    p.partials = ws.partials;
    p.counters = ws.counters;
    p.num_slices = m.bszm_out;
    p.slab_stride = slab_stride;
    const void* suh_host[kGemmMaxSlices] = {};
    if (m.host_lists) {
        const uint64_t* b = (const uint64_t*)m.b_list;
        const uint64_t* su = (const uint64_t*)m.suh_list;
        const uint64_t* sv = (const uint64_t*)m.svh_list;
        if (slabs > kGemmMaxSlices) throw std::runtime_error("exl3_mgemm (host lists): too many input rotations");
        for (int i = 0; i < slabs; ++i) suh_host[i] = (const void*)su[i];
        for (int i = 0; i < m.bszm_out; ++i) {
            GemmSlice& g = p.slice[i];
            g.trellis = (const uint32_t*)b[i];
            g.svh = (const _Float16*)sv[i];
            if (sliced) {
                const int src = m.had_src_list[i];
                if (src < 0 || src >= m.num_had_src) throw std::runtime_error("exl3_mgemm (host lists): had_src_list entry out of range");
                if (m.size_n_list[i] < 0 || m.size_n_list[i] > m.size_n || m.size_n_list[i] % 128 != 0)
                    throw std::runtime_error("exl3_mgemm (host lists): size_n_list entry must be a multiple of 128 within size_n");
                g.c = (void*)((const uint64_t*)m.c_ptrs)[i];
                g.width = m.size_n_list[i];
                g.n_stride = m.n_stride_list[i];
                g.a_had = (const _Float16*)m.a_had + (size_t)src * slab_stride;
            } else {
                g.c = (char*)m.c + (size_t)i * m.size_m * m.size_n * (m.c_fp32 ? 4 : 2);
                g.width = m.size_n;
                g.n_stride = m.size_n;
                g.a_had = (const _Float16*)m.a_had + (size_t)i * slab_stride;
            }
        }
    } else {
        p.b_list = (const uint64_t*)m.b_list;
        p.svh_list = (const uint64_t*)m.svh_list;
        if (sliced) {
            p.c_ptrs = (const uint64_t*)m.c_ptrs;
            p.size_n_list = m.size_n_list;
            p.n_stride_list = m.n_stride_list;
            p.had_src_list = m.had_src_list;
        }
    }
    const size_t in_stride = (!sliced && m.bszm_in > 1) ? slab_stride : 0;
    std::string d0 = launch_had_r_128_slabs(m.a, in_stride, m.a_had, slab_stride, m.host_lists ? nullptr : m.suh_list,
                                            suh_host, slabs, m.size_m, m.size_k, m.stream);
    const long nblocks = (long)m.bszm_out * ((m.size_n + 255) / 256);
    if (nblocks * ((m.size_m + 31) / 32) > kCounters / 2) throw std::runtime_error("exl3_mgemm: too many output tiles");
    std::string desc;
    dispatch_dense(ws, p, m.k_bits, m.codebook, m.size_m, m.size_k, (int)nblocks, m.stream, desc);
    return std::string(sliced ? "sliced x" : "uniform x") + std::to_string(m.bszm_out) + (m.host_lists ? " by value " : " ") + d0 +
           " + " + desc + (m.c_fp32 ? " out=f32" : " out=f16");
}

std::string launch_gemm_pair(const PairArgs& a, void* a_had_second)
{
    if (a.size_k % 128 != 0) throw std::runtime_error("exl3 linear: size_k must be a multiple of 128");
    LaunchScope scope(a.stream);
    Workspace& ws = scope.ws;
    throw_pending_device_fault(ws);
    GemmParams p{};
    p.fault = ws.fault_dev;
    p.spin_limit = spin_limit();
    p.a_had[0] = (const _Float16*)a.a_had;
    p.c[0] = a.c[0];
    p.M = a.size_m;
    p.K = a.size_k;
    p.N = a.size_n;
    p.out_fp32 = 0;
    p.partials = ws.partials;
    p.counters = ws.counters;
    p.num_slices = 2;
    void* const slabs[2] = {a.a_had, a_had_second};
    for (int i = 0; i < 2; ++i) {
        GemmSlice& g = p.slice[i];
        g.trellis = (const uint32_t*)a.trellis[i];
        g.svh = (const _Float16*)a.svh[i];
        g.c = a.c[i];
        g.width = a.size_n;
        g.n_stride = a.size_n;
        g.a_had = (const _Float16*)slabs[i];
    }
    std::string d0 = launch_had_r_128_slabs(a.a, 0, a.a_had, 0, nullptr, a.suh, 2, a.size_m, a.size_k, a.stream, slabs);
    const long nblocks = 2L * ((a.size_n + 255) / 256);
    if (nblocks * ((a.size_m + 31) / 32) > kCounters / 2) throw std::runtime_error("exl3 linear pair: too many output tiles");
    std::string desc;
    dispatch_dense(ws, p, a.k_bits, a.codebook, a.size_m, a.size_k, (int)nblocks, a.stream, desc);
    return "pair " + d0 + " + " + desc + " out=f16";
}

// grouped: problems of at most 32 * g.mb rows each; a_had rows are in problem order
std::string launch_gemm_grouped(const GroupedArgs& g)
{
    const int mb = g.mb == 4 ? 4 : 1;
    if (g.size_k % 128 != 0 || g.size_n % 128 != 0)
        throw std::runtime_error("moe grouped linear: sizes must be multiples of 128");
    LaunchScope scope(g.stream);
    Workspace& ws = scope.ws;
    throw_pending_device_fault(ws);
    GemmParams p{};
    p.fault = ws.fault_dev;
    p.spin_limit = spin_limit();
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
    p.shared_expert = g.shared ? g.shared_expert : -1;
    if (g.shared) std::memcpy(p.shared, g.shared, sizeof(p.shared));
    p.partials = ws.partials;
    p.counters = ws.counters;
    const int nblocks = (g.size_n + 255) / 256;
    const long tiles = (long)g.max_problems * g.num_lins * nblocks;
    p.cstride = gemm_counter_stride(tiles);
    p.S = gemm_split(ws, tiles, g.size_k / 128, mb);
    if (g.max_problems + g.max_big > 65535) throw std::runtime_error("moe grouped linear: too many problems");
    std::string desc;
    p.tiles_y = g.max_problems;
    if (g.max_big > 0) {
        // both lists in one launch, whole K per workgroup
        p.big_problems = (const GroupProblem*)g.big_problems;
        p.num_big = g.num_big;
        p.max_big = g.max_big;
        p.S = 1;
        gemm_bits(p, g.k_bits, g.codebook, mb, g.stream, desc, dim3(nblocks, g.num_lins, g.max_problems + g.max_big));
        hip_ok(hipGetLastError(), "exl3_gemm_mixed_kernel launch");
        return desc + " grouped";
    }
    gemm_bits(p, g.k_bits, g.codebook, mb, g.stream, desc, dim3(nblocks * p.S, g.num_lins, g.max_problems));
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

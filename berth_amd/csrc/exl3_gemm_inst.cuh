// Per-codebook instantiations of the MFMA GEMM kernel (included by
// exl3_gemm_cb{0,1,2}.hip with BERTH_GEMM_CB defined): 32-row and 128-row tiles for
// every bit rate, the balanced variant of the 128-row kernel, and the 256-row kernel.
#include "exl3_gemm_kernel.cuh"
#include "exl3_gemm_wide_kernel.cuh"
#include "launch.h"

namespace berth {

template <int BITS, int CB, int MB>
static void gemm_launch_mb(const GemmParams& p, hipStream_t stream, std::string& desc, dim3 grid)
{
    constexpr int BM = MB * 32;
    const size_t smem_a = (size_t)2 * BM * kAStride * sizeof(_Float16);     // double-buffered A tile
    const size_t smem_z = (size_t)32 * (256 + 4) * sizeof(float);
    const size_t smem = smem_a > smem_z ? smem_a : smem_z;
    if (smem > 64 * 1024) {
        static bool raised[64] = {};
        raise_dynamic_lds_limit((const void*)exl3_gemm_kernel<BITS, CB, MB>, (int)smem, raised,
                                "exl3_gemm_kernel shared-memory attribute");
    }
    if (p.units > 0) {
        // balanced dense launch (128-row tiles only): two workgroups per compute unit
        if constexpr (MB == 4) {
            static bool raised2[64] = {};
            raise_dynamic_lds_limit((const void*)exl3_gemm_balanced_kernel<BITS, CB, MB>, (int)smem, raised2,
                                    "exl3_gemm_balanced_kernel shared-memory attribute");
            hipLaunchKernelGGL((exl3_gemm_balanced_kernel<BITS, CB, MB>), grid, dim3(256), smem, stream, p);
            desc = "exl3_gemm_balanced_kernel<" + std::to_string(BITS) + "," + std::to_string(CB) + "," +
                   std::to_string(BM) + "x256> grid=" + std::to_string(grid.x) + " units=" + std::to_string(p.units) +
                   " max_parts=" + std::to_string(p.max_parts) + " smem=" + std::to_string(smem);
            return;
        }
        throw std::runtime_error("exl3 gemm: balanced launches use 128-row tiles");
    }
    hipLaunchKernelGGL((exl3_gemm_kernel<BITS, CB, MB>), grid, dim3(256), smem, stream, p);
    desc = "exl3_gemm_kernel<" + std::to_string(BITS) + "," + std::to_string(CB) + "," + std::to_string(BM) +
           "x256> grid=" + std::to_string(grid.x) + "x" + std::to_string(grid.y) + "x" + std::to_string(grid.z) +
           " split_k=" + std::to_string(p.S) + " smem=" + std::to_string(smem);
}

// 256-row tiles (balanced dense launches only): eight waves, decoded weights shared through LDS
template <int BITS, int CB>
static void gemm_launch_wide(const GemmParams& p, hipStream_t stream, std::string& desc, dim3 grid)
{
    if (p.units <= 0) throw std::runtime_error("exl3 gemm: 256-row tiles exist only as balanced launches");
    static bool raised[64] = {};
    raise_dynamic_lds_limit((const void*)exl3_gemm_wide_kernel<BITS, CB>, kWideSmem, raised,
                            "exl3_gemm_wide_kernel shared-memory attribute");
    hipLaunchKernelGGL((exl3_gemm_wide_kernel<BITS, CB>), grid, dim3(512), kWideSmem, stream, p);
    desc = "exl3_gemm_wide_kernel<" + std::to_string(BITS) + "," + std::to_string(CB) + ",256x256> grid=" +
           std::to_string(grid.x) + " units=" + std::to_string(p.units) + " max_parts=" + std::to_string(p.max_parts) +
           " smem=" + std::to_string(kWideSmem);
}

// two problem lists in one grouped launch: 128-row problems first, 32-row problems behind them
template <int BITS, int CB>
static void gemm_launch_mixed(const GemmParams& p, hipStream_t stream, std::string& desc, dim3 grid)
{
    const size_t smem = (size_t)2 * 128 * kAStride * sizeof(_Float16);
    static bool raised[64] = {};
    raise_dynamic_lds_limit((const void*)exl3_gemm_mixed_kernel<BITS, CB>, (int)smem, raised,
                            "exl3_gemm_mixed_kernel shared-memory attribute");
    hipLaunchKernelGGL((exl3_gemm_mixed_kernel<BITS, CB>), grid, dim3(256), smem, stream, p);
    desc = "exl3_gemm_mixed_kernel<" + std::to_string(BITS) + "," + std::to_string(CB) + ",128x256+32x256> grid=" +
           std::to_string(grid.x) + "x" + std::to_string(grid.y) + "x(" + std::to_string(p.max_big) + "+" +
           std::to_string(grid.z - p.max_big) + ") smem=" + std::to_string(smem);
}

template <int BITS, int CB>
static void gemm_launch(const GemmParams& p, int mb, hipStream_t stream, std::string& desc, dim3 grid)
{
    if (p.max_big > 0) gemm_launch_mixed<BITS, CB>(p, stream, desc, grid);
    else if (mb == 1) gemm_launch_mb<BITS, CB, 1>(p, stream, desc, grid);
    else if (mb == 8) gemm_launch_wide<BITS, CB>(p, stream, desc, grid);
    else gemm_launch_mb<BITS, CB, 4>(p, stream, desc, grid);
}

#define BERTH_CAT2(a, b) a##b
#define BERTH_CAT(a, b) BERTH_CAT2(a, b)

void BERTH_CAT(launch_gemm_cb, BERTH_GEMM_CB)(const GemmParams& p, int bits, int mb, hipStream_t stream,
                                              std::string& desc, dim3 grid)
{
    constexpr int CB = BERTH_GEMM_CB;
    switch (bits) {
    case 1: gemm_launch<1, CB>(p, mb, stream, desc, grid); break;
    case 2: gemm_launch<2, CB>(p, mb, stream, desc, grid); break;
    case 3: gemm_launch<3, CB>(p, mb, stream, desc, grid); break;
    case 4: gemm_launch<4, CB>(p, mb, stream, desc, grid); break;
    case 5: gemm_launch<5, CB>(p, mb, stream, desc, grid); break;
    case 6: gemm_launch<6, CB>(p, mb, stream, desc, grid); break;
    case 7: gemm_launch<7, CB>(p, mb, stream, desc, grid); break;
    default: gemm_launch<8, CB>(p, mb, stream, desc, grid); break;
    }
}

}  // namespace berth

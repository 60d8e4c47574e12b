// Per-codebook instantiations of the GEMV kernel (included by exl3_gemv_cb{0,1,2}.hip
// with BERTH_GEMV_CB defined).  Instantiated row capacities: 1 (decode) and 8 (small
// batches, grouped problems); the SiLU-gated input exists for the grouped down
// projection (one row per problem, or up to 8).
#include "exl3_gemv_kernel.cuh"
#include "launch.h"

namespace berth {

template <int BITS, int CB>
static void launch_rows(const GemvParams& p, int mmax, dim3 grid, hipStream_t stream)
{
    if (p.route.parts) {
        // one-token gate / up launch of an MoE layer with the routing's last part inline
        if (p.half_units) hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 1, false, 4, true>), grid, dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 1, false, 8, true>), grid, dim3(256), 0, stream, p);
    } else if (p.half_units && mmax == 1) {
        if (p.a_up) hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 1, true, 4>), grid, dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 1, false, 4>), grid, dim3(256), 0, stream, p);
    } else if (p.a_up && mmax == 1) hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 1, true>), grid, dim3(256), 0, stream, p);
    else if (p.a_up) hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 8, true>), grid, dim3(256), 0, stream, p);
    else if (mmax == 1) hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 1, false>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((exl3_gemv_kernel<BITS, CB, 8, false>), grid, dim3(256), 0, stream, p);
}

#define BERTH_CAT2(a, b) a##b
#define BERTH_CAT(a, b) BERTH_CAT2(a, b)

void BERTH_CAT(launch_gemv_cb, BERTH_GEMV_CB)(const GemvParams& p, int bits, int mmax, dim3 grid, hipStream_t stream)
{
    constexpr int CB = BERTH_GEMV_CB;
    switch (bits) {
    case 1: launch_rows<1, CB>(p, mmax, grid, stream); break;
    case 2: launch_rows<2, CB>(p, mmax, grid, stream); break;
    case 3: launch_rows<3, CB>(p, mmax, grid, stream); break;
    case 4: launch_rows<4, CB>(p, mmax, grid, stream); break;
    case 5: launch_rows<5, CB>(p, mmax, grid, stream); break;
    case 6: launch_rows<6, CB>(p, mmax, grid, stream); break;
    case 7: launch_rows<7, CB>(p, mmax, grid, stream); break;
    default: launch_rows<8, CB>(p, mmax, grid, stream); break;
    }
}

}  // namespace berth

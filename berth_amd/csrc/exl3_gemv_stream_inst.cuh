// Per-codebook instantiations of the one-row streaming GEMV kernel (included by
// exl3_gemv_stream_cb{0,1,2}.hip with BERTH_GEMV_CB defined): every bit rate, plain and
// SiLU-gated input, all-arithmetic decode (table mask 0) and the hybrid decode masks.
#include "exl3_gemv_stream_kernel.cuh"
#include "launch.h"

namespace berth {

template <int BITS, int CB, int IN, int LUTMASK>
static void launch_stream_one(const StreamParams& p, dim3 grid, hipStream_t stream)
{
    constexpr int lds_bytes = stream_lds_bytes(LUTMASK);
    static bool raised[64] = {};
    raise_dynamic_lds_limit((const void*)exl3_gemv_stream_kernel<BITS, CB, IN, LUTMASK>, lds_bytes, raised,
                            "exl3_gemv_stream_kernel: dynamic LDS limit");
    hipLaunchKernelGGL((exl3_gemv_stream_kernel<BITS, CB, IN, LUTMASK>), grid, dim3(1024), lds_bytes, stream, p);
}

template <int BITS, int CB>
static void launch_stream_bits(const StreamParams& p, int lutmask, dim3 grid, hipStream_t stream)
{
    const int in = p.norm_x ? kInNorm : (p.a_up ? kInSilu : kInPlain);
    auto by_input = [&](auto mask) {
        constexpr int M = decltype(mask)::value;
        if (in == kInNorm) launch_stream_one<BITS, CB, kInNorm, M>(p, grid, stream);
        else if (in == kInSilu) launch_stream_one<BITS, CB, kInSilu, M>(p, grid, stream);
        else launch_stream_one<BITS, CB, kInPlain, M>(p, grid, stream);
    };
    switch (lutmask) {
    case 0x0: by_input(std::integral_constant<int, 0x0>{}); break;
    default: by_input(std::integral_constant<int, 0xA>{}); break;
    }
}

#define BERTH_CAT2(a, b) a##b
#define BERTH_CAT(a, b) BERTH_CAT2(a, b)

void BERTH_CAT(launch_gemv_stream_cb, BERTH_GEMV_CB)(const StreamParams& p, int bits, int lutmask, dim3 grid,
                                                    hipStream_t stream)
{
    constexpr int CB = BERTH_GEMV_CB;
    switch (bits) {
    case 1: launch_stream_bits<1, CB>(p, lutmask, grid, stream); break;
    case 2: launch_stream_bits<2, CB>(p, lutmask, grid, stream); break;
    case 3: launch_stream_bits<3, CB>(p, lutmask, grid, stream); break;
    case 4: launch_stream_bits<4, CB>(p, lutmask, grid, stream); break;
    case 5: launch_stream_bits<5, CB>(p, lutmask, grid, stream); break;
    case 6: launch_stream_bits<6, CB>(p, lutmask, grid, stream); break;
    case 7: launch_stream_bits<7, CB>(p, lutmask, grid, stream); break;
    default: launch_stream_bits<8, CB>(p, lutmask, grid, stream); break;
    }
}

}  // namespace berth

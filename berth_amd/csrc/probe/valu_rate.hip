// Measurement probe for the benchmark (not on the product path): the rate at which the
// vector ALU of this device issues the instruction mix of the mul1 trellis decode.
//
// The decode of one weight costs a fixed number of vector instructions (window extraction,
// 32-bit hash multiply, byte sum, half of a packed fp16 fma, half of a dot product), so
// "lane-instructions per second / instructions per weight" is the weight rate the decode
// cannot exceed whatever the memory system delivers.  This probe issues exactly that mix
// (per pair of weights: 2 v_bfe_u32, 2 v_mul_lo_u32, v_sad_u8, v_sad_hi_u8, v_pk_fma_f16,
// v_dot2c_f32_f16) from sixteen waves per compute unit with no memory traffic and reports
// lane-instructions per second, measured with HIP events.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

constexpr int kPairsPerIter = 16;           // 16 pairs x 8 instructions = 128 vector instructions per iteration

__global__ __launch_bounds__(256, 4) void valu_mix_kernel(float* out, int iters, uint32_t seed)
{
    uint32_t w = (threadIdx.x + blockIdx.x * 256u) * 2654435761u + seed;
    float acc = 0.0f;
    const uint32_t k = 0x83DCD12Du, bias = 0x64006400u, mul = 0x1EEE1EEEu, add = 0xC931C931u, x = 0x3C003800u;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int p = 0; p < kPairsPerIter; ++p) {
            uint32_t s0, s1;
            asm volatile("v_bfe_u32 %0, %3, 4, 16\n\t"
                         "v_bfe_u32 %1, %3, 8, 16\n\t"
                         "v_mul_lo_u32 %0, %0, %4\n\t"
                         "v_mul_lo_u32 %1, %1, %4\n\t"
                         "v_sad_u8 %0, %0, 0, %5\n\t"
                         "v_sad_hi_u8 %0, %1, 0, %0\n\t"
                         "v_pk_fma_f16 %0, %0, %6, %7\n\t"
                         "v_dot2c_f32_f16 %2, %0, %8"
                         : "=&v"(s0), "=&v"(s1), "+v"(acc)
                         : "v"(w), "s"(k), "v"(bias), "v"(mul), "v"(add), "v"(x));
        }
    }
    if (acc == 12345.678f) out[0] = acc;    // keeps the work; never true for these inputs in practice
}

}  // namespace

// lane-instructions per second of the decode mix on the current device; < 0 on error
extern "C" double berth_probe_valu_lane_instr_per_s(void)
{
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess) return -1.0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return -1.0;
    float* out = nullptr;
    if (hipMalloc(&out, 256) != hipSuccess) return -1.0;
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    const int iters = 4000;
    const dim3 grid(cus * 4), block(256);
    hipLaunchKernelGGL(valu_mix_kernel, grid, block, 0, 0, out, iters, 1u);
    double best = -1.0;
    for (int rep = 0; rep < 3; ++rep) {
        hipEventRecord(e0, 0);
        hipLaunchKernelGGL(valu_mix_kernel, grid, block, 0, 0, out, iters, 2u + rep);
        hipEventRecord(e1, 0);
        if (hipEventSynchronize(e1) != hipSuccess) break;
        float ms = 0.0f;
        hipEventElapsedTime(&ms, e0, e1);
        const double lane_instr = (double)grid.x * 256.0 * iters * kPairsPerIter * 8.0;
        const double rate = lane_instr / (ms * 1e-3);
        if (rate > best) best = rate;
    }
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    hipFree(out);
    return best;
}

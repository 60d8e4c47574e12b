// Native helpers of bench.py (measurement only, not on the product path; built into
// libberth_bench.so beside bench.py):
//
//   * berth_probe_valu: the rate at which the vector ALU of this device issues the
//     instruction mix of the mul1 trellis decode, right after idle (boost clock) and after
//     the device has been kept busy for a given time (sustained clock).
//   * berth_bench_run: a host loop that issues prepared calls of the C ABI one by one, the
//     way the reference's engine does (eager launches from compiled code), so that the
//     benchmark's eager figure measures the library and the device rather than the
//     interpreter that drives the benchmark.
//
// The decode of one weight costs a fixed number of vector instructions (window extraction,
// 32-bit hash multiply, byte sum, half of a packed fp16 fma, half of a dot product), so
// "lane-instructions per second / instructions per weight" is the weight rate the decode
// cannot exceed whatever the memory system delivers.  The probe issues exactly that mix
// (per pair of weights: 2 v_bfe_u32, 2 v_mul_lo_u32, v_sad_u8, v_sad_hi_u8, v_pk_fma_f16,
// v_dot2c_f32_f16) from sixteen waves per compute unit with no memory traffic.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "include/berth_kernels_hip.h"

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

// Lane-instructions per second of the decode mix on the current device.  out[0]: the best of
// three 3 ms launches issued from an idle device (the clock a 10 - 30 us launch sees);
// out[1]: one such launch timed after the device has run the same kernel back to back for
// `sustain_ms` milliseconds (the clock a long launch settles at).  Returns 0, or -1 on error.
extern "C" int berth_probe_valu(double sustain_ms, double* out)
{
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess) return -1;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return -1;
    float* buf = nullptr;
    if (hipMalloc(&buf, 256) != hipSuccess) return -1;
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    const int iters = 4000;
    const dim3 grid(cus * 4), block(256);
    const double lane_instr = (double)grid.x * 256.0 * iters * kPairsPerIter * 8.0;
    auto timed = [&](uint32_t seed) -> double {
        hipEventRecord(e0, 0);
        hipLaunchKernelGGL(valu_mix_kernel, grid, block, 0, 0, buf, iters, seed);
        hipEventRecord(e1, 0);
        if (hipEventSynchronize(e1) != hipSuccess) return -1.0;
        float ms = 0.0f;
        hipEventElapsedTime(&ms, e0, e1);
        return lane_instr / (ms * 1e-3);
    };
    hipLaunchKernelGGL(valu_mix_kernel, grid, block, 0, 0, buf, 16, 1u);      // loads the code object
    hipDeviceSynchronize();
    double best = -1.0;
    for (int rep = 0; rep < 3; ++rep) {
        const double r = timed(2u + rep);
        if (r > best) best = r;
        hipDeviceSynchronize();
    }
    out[0] = best;
    // keep the device busy, then time one more launch in the same queue
    const double one_ms = lane_instr / best * 1e3;
    const int fill = (int)(sustain_ms / one_ms) + 1;
    for (int i = 0; i < fill; ++i) hipLaunchKernelGGL(valu_mix_kernel, grid, block, 0, 0, buf, iters, 100u + i);
    out[1] = timed(7u);
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    hipFree(buf);
    return out[0] > 0 && out[1] > 0 ? 0 : -1;
}

// One prepared call of the C ABI.  kind 0: berth_exl3_linear(p[0..5], i[0..5], stream);
// kind 1: berth_ops_mgemm_hostlists, kind 2: berth_ops_mgemm (p[0..5], i[0..7], p[6..9], i[8], stream);
// kind 3: berth_exl3_mlp(p[0], lins = p[1] (host), p[2..6], i[0..4], stream);
// kind 4: berth_ops_silu_mul(p[0..2], numel = i[0], act_limit 0, stream);
// kind 5: berth_exl3_mlp_block(p[0..2], norm = p[3] (host), lins = p[4] (host), p[5..10], i[0..4], stream);
// kind 6: berth_ops_rms_norm_res_in(p[0..3], rows = i[0], dim = i[1], epsilon 1e-6, bias 1, scale 1, bf16 weight, stream);
// kind 7: berth_ops_add_f32(p[0..2], n = i[0], stream).
struct BenchCall {
    int kind;
    int i[12];
    const void* p[12];
};

// Issues calls[(s % distinct) * per_step + j] for s = 0 .. steps - 1, j = 0 .. per_step - 1 on
// `stream`, without synchronising.  Returns 0, or 1 + the index of the first call that failed.
extern "C" int berth_bench_run(const BenchCall* calls, int per_step, int distinct, int steps, void* stream)
{
    for (int s = 0; s < steps; ++s) {
        const BenchCall* step = calls + (size_t)(s % distinct) * per_step;
        for (int j = 0; j < per_step; ++j) {
            const BenchCall& c = step[j];
            int rc = -1;
            switch (c.kind) {
            case 0:
                rc = berth_exl3_linear(c.p[0], c.p[1], (void*)c.p[2], c.p[3], (void*)c.p[4], c.p[5], c.i[0], c.i[1], c.i[2],
                                       c.i[3], c.i[4], c.i[5], stream);
                break;
            case 1:
                rc = berth_ops_mgemm_hostlists(c.p[0], c.p[1], (void*)c.p[2], c.p[3], (void*)c.p[4], c.p[5], c.i[0], c.i[1],
                                               c.i[2], c.i[3], c.i[4], c.i[5], c.i[6], c.i[7], (const int*)c.p[6], c.p[7],
                                               (const int*)c.p[8], (const int*)c.p[9], c.i[8], stream) > 0 ? 0 : -1;
                break;
            case 2:
                rc = berth_ops_mgemm(c.p[0], c.p[1], (void*)c.p[2], c.p[3], (void*)c.p[4], c.p[5], c.i[0], c.i[1], c.i[2],
                                     c.i[3], c.i[4], c.i[5], c.i[6], c.i[7], (const int*)c.p[6], c.p[7], (const int*)c.p[8],
                                     (const int*)c.p[9], c.i[8], stream) > 0 ? 0 : -1;
                break;
            case 3:
                rc = berth_exl3_mlp(c.p[0], (const berth_exl3_lin*)c.p[1], (void*)c.p[2], (void*)c.p[3], (void*)c.p[4],
                                    (void*)c.p[5], (void*)c.p[6], c.i[0], c.i[1], c.i[2], c.i[3], c.i[4], stream);
                break;
            case 4: rc = berth_ops_silu_mul(c.p[0], c.p[1], (void*)c.p[2], (int64_t)c.i[0], 0.0f, stream); break;
            case 5:
                rc = berth_exl3_mlp_block(c.p[0], c.p[1], (void*)c.p[2], (const berth_rms_norm*)c.p[3],
                                          (const berth_exl3_lin*)c.p[4], (void*)c.p[5], (void*)c.p[6], (void*)c.p[7],
                                          (void*)c.p[8], (void*)c.p[9], (void*)c.p[10], c.i[0], c.i[1], c.i[2], c.i[3],
                                          c.i[4], stream);
                break;
            case 6:
                rc = berth_ops_rms_norm_res_in(c.p[0], c.p[1], (void*)c.p[2], (void*)c.p[3], c.i[0], c.i[1], 1e-6f, 1.0f, 1.0f,
                                               1, stream);
                break;
            case 7: rc = berth_ops_add_f32(c.p[0], c.p[1], (void*)c.p[2], c.i[0], stream); break;
            default: break;
            }
            if (rc != 0) return 1 + s * per_step + j;
        }
    }
    return 0;
}

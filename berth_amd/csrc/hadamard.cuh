// 128-point Sylvester Hadamard on one wavefront, two elements per lane.
//
// Butterfly order is fixed (stage h = 1, 2, 4 .. 64; element i with i & h == 0 gets
// a + b, element i + h gets a - b, a the lower element), in fp32, so that the
// rotated activation rounds to the same fp16 bits on every implementation that
// follows the same order.  Scale 1/sqrt(128) as in
// crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:44-46.
#pragma once

#include <hip/hip_runtime.h>

namespace berth {

// lane l holds elements 2l (v0) and 2l+1 (v1) of a 128 vector
__device__ __forceinline__ void had128_wave(float& v0, float& v1, int lane)
{
    float a = v0, b = v1;
    v0 = a + b;
    v1 = a - b;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        float p0 = __shfl_xor(v0, d, 64);
        float p1 = __shfl_xor(v1, d, 64);
        bool upper = (lane & d) != 0;
        v0 = upper ? (p0 - v0) : (v0 + p0);
        v1 = upper ? (p1 - v1) : (v1 + p1);
    }
}

}  // namespace berth

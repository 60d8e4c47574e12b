// Test kernels for the device-runtime library's code-object path (libberth_hip.so:
// berth_hip_module_load_*, berth_hip_function_launch), compiled to a stand-alone gfx950 code
// object.  They play the role of the reference runtime's own test kernels
// (crates/berth-cuda/tests/fill_i32.cu, touch_dyn_smem.cu).
#include <hip/hip_runtime.h>

// one thread writes the scalar argument
extern "C" __global__ void fill_i32(int* out, int value) { *out = value; }

// y[i] = a * x[reversed position inside the workgroup] + y[i], the reversal through
// dynamic LDS (blockDim.x floats)
extern "C" __global__ void axpy_reversed_lds(const float* x, float* y, float a, int n)
{
    extern __shared__ float stage[];
    const int base = blockIdx.x * blockDim.x, i = base + threadIdx.x;
    stage[threadIdx.x] = i < n ? x[i] : 0.0f;
    __syncthreads();
    const int j = blockDim.x - 1 - threadIdx.x;
    if (i < n) y[i] = a * stage[j] + y[i];
}

// touches the first and the last byte of a dynamic LDS allocation of `bytes` bytes; a launch
// with more than the default limit (64 KiB) is refused until the limit has been raised
extern "C" __global__ void touch_dyn_lds(int* out, int bytes)
{
    extern __shared__ unsigned char lds[];
    if (threadIdx.x == 0) {
        lds[0] = 1;
        lds[bytes - 1] = 2;
        *out = (int)lds[0] + (int)lds[bytes - 1];
    }
}

// Hadamard rows, SiLU gate.
#include "exl3_decode.cuh"
#include "hadamard.cuh"
#include "launch.h"

namespace berth {

// crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:31-67: per row and per
// 128 columns, out = Hh(in * scale) (pre) or Hh(in) * scale (post).  One wave per
// 128 block, four blocks per workgroup.
template <typename T, bool PRE>
__global__ __launch_bounds__(256) void had_r_128_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                        const _Float16* __restrict__ scale,
                                                        long blocks, int col_blocks)
{
    const int lane = threadIdx.x & 63;
    const long blk = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blk >= blocks) return;
    const int cb = (int)(blk % col_blocks);
    const size_t at = (size_t)blk * 128 + 2 * lane;
    float v0 = (float)in[at], v1 = (float)in[at + 1];
    float s0 = 1.0f, s1 = 1.0f;
    if (scale) {
        s0 = (float)scale[cb * 128 + 2 * lane];
        s1 = (float)scale[cb * 128 + 2 * lane + 1];
    }
    if (PRE) { v0 *= s0; v1 *= s1; }
    had128_wave(v0, v1, lane);
    v0 *= kRsqrt128;
    v1 *= kRsqrt128;
    if (!PRE) { v0 *= s0; v1 *= s1; }
    out[at] = (T)v0;
    out[at + 1] = (T)v1;
}

std::string launch_had_r_128(const void* in, void* out, const void* scale, int pre_scale,
                             int rows, int cols, int fp32, hipStream_t stream)
{
    const int col_blocks = cols / 128;
    const long blocks = (long)rows * col_blocks;
    const dim3 grid((unsigned)((blocks + 3) / 4));
    const _Float16* sc = (const _Float16*)scale;
    if (fp32) {
        if (pre_scale) hipLaunchKernelGGL((had_r_128_kernel<float, true>), grid, dim3(256), 0, stream, (const float*)in, (float*)out, sc, blocks, col_blocks);
        else hipLaunchKernelGGL((had_r_128_kernel<float, false>), grid, dim3(256), 0, stream, (const float*)in, (float*)out, sc, blocks, col_blocks);
    } else {
        if (pre_scale) hipLaunchKernelGGL((had_r_128_kernel<_Float16, true>), grid, dim3(256), 0, stream, (const _Float16*)in, (_Float16*)out, sc, blocks, col_blocks);
        else hipLaunchKernelGGL((had_r_128_kernel<_Float16, false>), grid, dim3(256), 0, stream, (const _Float16*)in, (_Float16*)out, sc, blocks, col_blocks);
    }
    hip_ok(hipGetLastError(), "had_r_128 launch");
    return std::string(fp32 ? "had_ff_r_128_kernel<" : "had_hf_r_128_kernel<") + (pre_scale ? "1,0>" : "0,1>") +
           " grid=" + std::to_string(grid.x) + " block=256";
}

// crates/berth-kernels/csrc/ops/act.cu:35-69.  The reference's fixture is
// reproduced bit for bit by half arithmetic with every step rounded to fp16:
// e = exp(-g); s = 1 + e; r = 1 / s; t = g * r; out = t * u.  exp and the
// reciprocal are evaluated in fp32 and rounded once to fp16.
__global__ __launch_bounds__(256) void silu_mul_kernel(const half2_t* __restrict__ gate,
                                                       const half2_t* __restrict__ up,
                                                       half2_t* __restrict__ out, int64_t pairs,
                                                       float act_limit)
{
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= pairs) return;
    half2_t g = gate[i], u = up[i], o;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        _Float16 gj = g[j], uj = u[j];
        if (act_limit != 0.0f) {
            float gl = fminf((float)gj, act_limit);
            float ul = fmaxf(fminf((float)uj, act_limit), -act_limit);
            gj = (_Float16)gl;
            uj = (_Float16)ul;
        }
        _Float16 e = (_Float16)expf(-(float)gj);
        _Float16 s = (_Float16)1.0f + e;
        _Float16 r = (_Float16)(1.0f / (float)s);
        _Float16 t = gj * r;
        o[j] = t * uj;
    }
    out[i] = o;
}

std::string launch_silu_mul(const void* gate, const void* up, void* out, int64_t numel,
                            float act_limit, hipStream_t stream)
{
    const int64_t pairs = numel / 2;
    const unsigned blocks = (unsigned)((pairs + 255) / 256);
    hipLaunchKernelGGL(silu_mul_kernel, dim3(blocks), dim3(256), 0, stream, (const half2_t*)gate,
                       (const half2_t*)up, (half2_t*)out, pairs, act_limit);
    hip_ok(hipGetLastError(), "silu_mul launch");
    return "silu_mul_kernel block=256 grid=" + std::to_string(blocks);
}

// crates/berth-exl3/src/signs.rs:25-46: packed su / sv -> fp16 signs.  Little-endian
// u16 words, bit i of a word is element i of its 16; a set bit is -1.0 (0xBC00),
// a clear bit +1.0 (0x3C00).  One thread per output pair.
__global__ __launch_bounds__(256) void unpack_signs_kernel(const uint16_t* __restrict__ packed,
                                                           uint32_t* __restrict__ out, int64_t pairs)
{
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= pairs) return;
    const uint32_t word = packed[i >> 3];
    const uint32_t two = (word >> (2 * (i & 7))) & 3u;
    out[i] = 0x3C003C00u | ((two & 1u) << 15) | ((two & 2u) << 30);
}

std::string launch_unpack_signs(const void* packed, void* out, int64_t words, hipStream_t stream)
{
    const int64_t pairs = words * 8;
    const unsigned blocks = (unsigned)((pairs + 255) / 256);
    hipLaunchKernelGGL(unpack_signs_kernel, dim3(blocks), dim3(256), 0, stream, (const uint16_t*)packed,
                       (uint32_t*)out, pairs);
    hip_ok(hipGetLastError(), "unpack_signs launch");
    return "unpack_signs_kernel block=256 grid=" + std::to_string(blocks);
}

}  // namespace berth

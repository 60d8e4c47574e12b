// Hadamard rows, SiLU gate.
#include "exl3_decode.cuh"
#include "hadamard.cuh"
#include "launch.h"

namespace berth {

// crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:31-67: per row and per
// 128 columns, out = Hh(in * scale) (pre) or Hh(in) * scale (post).
template <typename T, bool PRE>
__global__ __launch_bounds__(256) void had_r_128_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                        const _Float16* __restrict__ scale,
                                                        long blocks, int col_blocks)
{
    // sixteen lanes per 128 block, eight consecutive elements per lane (one or two 16-byte
    // accesses): a wave takes four neighbouring blocks at a time and strides over the tensor
    typedef T vec8_t __attribute__((ext_vector_type(8)));
    const int lane = threadIdx.x & 63;
    const int l16 = lane & 15;
    const long waves = (long)gridDim.x * 4;
    const long groups = (blocks + 3) / 4;
    for (long g = (long)blockIdx.x * 4 + (threadIdx.x >> 6); g < groups; g += waves) {
        const long blk = g * 4 + (lane >> 4);
        const bool live = blk < blocks;
        const long b = live ? blk : blocks - 1;             // lanes past the end redo the last block and store nothing
        const int cb = (int)(b % col_blocks);
        const size_t at = (size_t)b * 128 + 8 * l16;
        const vec8_t x = *(const vec8_t*)(in + at);
        float v[8], sc[8];
        if (scale) {
            const half8_t s8 = *(const half8_t*)(scale + cb * 128 + 8 * l16);
#pragma unroll
            for (int i = 0; i < 8; ++i) sc[i] = (float)s8[i];
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) sc[i] = 1.0f;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            v[i] = (float)x[i];
            if (PRE) v[i] *= sc[i];
        }
        had128_row16(v, lane);
        vec8_t o;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float r = v[i] * kRsqrt128;
            if (!PRE) r *= sc[i];
            o[i] = (T)r;
        }
        if (live) *(vec8_t*)(out + at) = o;
    }
}

// The rotated inputs of a bundle in one launch: blockIdx.y is the slab, whose sign scales come
// from a device list of pointers or from the pointers passed by value.
struct SuhTable {
    const _Float16* suh[kBundleMaxSlices];
    _Float16* out[kBundleMaxSlices];        // null: slab s goes to out + s * out_stride
};
__global__ __launch_bounds__(256) void had_r_128_slabs_kernel(const _Float16* __restrict__ in, size_t in_stride,
                                                              _Float16* __restrict__ out, size_t out_stride,
                                                              const uint64_t* __restrict__ suh_list, SuhTable tab,
                                                              long blocks, int col_blocks)
{
    const int slab = blockIdx.y;
    const _Float16* scale = suh_list ? (const _Float16*)suh_list[slab] : tab.suh[slab];
    in += (size_t)slab * in_stride;
    out = (!suh_list && tab.out[slab]) ? tab.out[slab] : out + (size_t)slab * out_stride;
    const int lane = threadIdx.x & 63;
    const int l16 = lane & 15;
    const long waves = (long)gridDim.x * 4;
    const long groups = (blocks + 3) / 4;
    for (long g = (long)blockIdx.x * 4 + (threadIdx.x >> 6); g < groups; g += waves) {
        const long blk = g * 4 + (lane >> 4);
        const bool live = blk < blocks;
        const long b = live ? blk : blocks - 1;             // lanes past the end redo the last block and store nothing
        const int cb = (int)(b % col_blocks);
        const size_t at = (size_t)b * 128 + 8 * l16;
        const half8_t x = *(const half8_t*)(in + at);
        const half8_t s8 = *(const half8_t*)(scale + cb * 128 + 8 * l16);
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (float)x[i] * (float)s8[i];
        had128_row16(v, lane);
        half8_t o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (_Float16)(v[i] * kRsqrt128);
        if (live) *(half8_t*)(out + at) = o;
    }
}

std::string launch_had_r_128_slabs(const void* in, size_t in_stride, void* out, size_t out_stride, const void* suh_list,
                                   const void* const* suh_host, int slabs, int rows, int cols, hipStream_t stream,
                                   void* const* out_host)
{
    if (slabs < 1 || slabs > 65535) throw std::runtime_error("had_r_128 slabs: between 1 and 65535 slabs");
    SuhTable tab{};
    if (!suh_list) {
        if (slabs > kBundleMaxSlices) throw std::runtime_error("had_r_128 slabs: too many slabs for the by-value table");
        for (int i = 0; i < slabs; ++i) {
            tab.suh[i] = (const _Float16*)suh_host[i];
            tab.out[i] = out_host ? (_Float16*)out_host[i] : nullptr;
        }
    }
    const int col_blocks = cols / 128;
    const long blocks = (long)rows * col_blocks;
    const long wgs = (blocks + 15) / 16;
    const dim3 grid((unsigned)(wgs < 4096 ? wgs : 4096), (unsigned)slabs);
    hipLaunchKernelGGL(had_r_128_slabs_kernel, grid, dim3(256), 0, stream, (const _Float16*)in, in_stride, (_Float16*)out,
                       out_stride, (const uint64_t*)suh_list, tab, blocks, col_blocks);
    hip_ok(hipGetLastError(), "had_r_128 slabs launch");
    return "had_r_128_slabs_kernel grid=" + std::to_string(grid.x) + "x" + std::to_string(grid.y) + " block=256";
}

std::string launch_had_r_128(const void* in, void* out, const void* scale, int pre_scale,
                             int rows, int cols, int fp32, hipStream_t stream)
{
    const int col_blocks = cols / 128;
    const long blocks = (long)rows * col_blocks;
    const long wgs = (blocks + 15) / 16;                    // four blocks per wave, four waves per workgroup
    const dim3 grid((unsigned)(wgs < 4096 ? wgs : 4096));
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

// crates/berth-kernels/csrc/ops/add.cu: c = a + b in fp32 (the residual add after the MLP).
__global__ __launch_bounds__(256) void add_f32_kernel(const float* a, const float* b, float* c, int n)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) c[i] = a[i] + b[i];
}

std::string launch_add_f32(const void* a, const void* b, void* c, int n, hipStream_t stream)
{
    const unsigned blocks = (unsigned)((n + 255) / 256);
    hipLaunchKernelGGL(add_f32_kernel, dim3(blocks), dim3(256), 0, stream, (const float*)a, (const float*)b, (float*)c, n);
    hip_ok(hipGetLastError(), "add_f32 launch");
    return "add_f32 block=256 grid=" + std::to_string(blocks);
}

// c[r][j] += bias[j] for a linear that carries a bias (crates/berth-exl3/src/linear.rs:131-133; the
// reference's engine refuses such a linear, crates/berth-engine/src/mlp.rs:67-75).  c is the linear's
// output as written, fp16 or fp32; the sum is formed in fp32 and rounded once to c's type.
template <bool F32>
__global__ __launch_bounds__(256) void add_bias_kernel(void* c, const float* __restrict__ bias, int n, long long total)
{
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const float b = bias[(int)(i % n)];
    if (F32) {
        ((float*)c)[i] += b;
    } else {
        _Float16* h = (_Float16*)c;
        h[i] = (_Float16)((float)h[i] + b);
    }
}

std::string launch_add_bias(void* c, const void* bias, int rows, int n, int c_fp32, hipStream_t stream)
{
    const long long total = (long long)rows * n;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (c_fp32)
        hipLaunchKernelGGL(add_bias_kernel<true>, dim3(blocks), dim3(256), 0, stream, c, (const float*)bias, n, total);
    else
        hipLaunchKernelGGL(add_bias_kernel<false>, dim3(blocks), dim3(256), 0, stream, c, (const float*)bias, n, total);
    hip_ok(hipGetLastError(), "add_bias launch");
    return std::string("add_bias ") + (c_fp32 ? "f32" : "f16") + " block=256 grid=" + std::to_string(blocks);
}

// RMS norm of fp32 rows to fp16, optionally with the fused residual
// (crates/berth-kernels/src/ops.rs:398-500, csrc/ops/norm.cu): residual += x in
// place (fp32), then y = fp16((v * rmf) * (w + constant_bias) * constant_scale),
// rmf = fp32(1 / sqrt(mean(v^2) + epsilon)).  The mean is accumulated in double so
// that it does not depend on the order of the reduction.  One workgroup per row.
template <bool RES, bool WBF16>
__global__ __launch_bounds__(256) void rms_norm_kernel(const float* __restrict__ x, const uint16_t* __restrict__ weight,
                                                       _Float16* __restrict__ y, float* residual, int dim,
                                                       float epsilon, float constant_bias, float constant_scale)
{
    __shared__ double s_part[4];
    __shared__ float s_rmf;
    const int row = blockIdx.x, tid = threadIdx.x;
    const float4_t* xr = (const float4_t*)(x + (size_t)row * dim);
    float4_t* rr = RES ? (float4_t*)(residual + (size_t)row * dim) : nullptr;
    double ss = 0.0;
    for (int i = tid; i < dim / 4; i += 256) {
        float4_t v = xr[i];
        if (RES) {
            const float4_t r = rr[i];
            v = float4_t{r.x + v.x, r.y + v.y, r.z + v.z, r.w + v.w};
            rr[i] = v;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) ss += (double)v[j] * (double)v[j];
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) ss += __shfl_xor(ss, d, 64);
    if ((tid & 63) == 0) s_part[tid >> 6] = ss;
    __syncthreads();
    if (tid == 0) {
        const double total = ((s_part[0] + s_part[1]) + s_part[2]) + s_part[3];
        s_rmf = (float)(1.0 / sqrt(total / dim + (double)epsilon));
    }
    __syncthreads();
    const float rmf = s_rmf;
    for (int i = tid; i < dim / 4; i += 256) {
        const float4_t v = RES ? rr[i] : xr[i];     // RES: this thread wrote these four itself
        half4_t o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint16_t wb = weight[4 * i + j];
            const float w = WBF16 ? __builtin_bit_cast(float, (uint32_t)wb << 16)
                                  : (float)__builtin_bit_cast(_Float16, wb);
            float t = v[j] * rmf;
            t = t * (w + constant_bias);
            t = t * constant_scale;
            o[j] = (_Float16)t;
        }
        *(half4_t*)(y + (size_t)row * dim + 4 * i) = o;
    }
}

std::string launch_rms_norm(const void* x, const void* weight, void* y, void* residual, int rows, int dim,
                            float epsilon, float constant_bias, float constant_scale, int weight_bf16,
                            hipStream_t stream)
{
    const dim3 grid((unsigned)rows), block(256);
    const float* xf = (const float*)x;
    const uint16_t* w = (const uint16_t*)weight;
    _Float16* yh = (_Float16*)y;
    float* r = (float*)residual;
    if (residual) {
        if (weight_bf16) hipLaunchKernelGGL((rms_norm_kernel<true, true>), grid, block, 0, stream, xf, w, yh, r, dim, epsilon, constant_bias, constant_scale);
        else hipLaunchKernelGGL((rms_norm_kernel<true, false>), grid, block, 0, stream, xf, w, yh, r, dim, epsilon, constant_bias, constant_scale);
    } else {
        if (weight_bf16) hipLaunchKernelGGL((rms_norm_kernel<false, true>), grid, block, 0, stream, xf, w, yh, r, dim, epsilon, constant_bias, constant_scale);
        else hipLaunchKernelGGL((rms_norm_kernel<false, false>), grid, block, 0, stream, xf, w, yh, r, dim, epsilon, constant_bias, constant_scale);
    }
    hip_ok(hipGetLastError(), "rms_norm launch");
    return std::string("rms_norm_kernel<") + (residual ? "2" : "0") + ",float,half," + (weight_bf16 ? "bfloat16" : "half") +
           ",float> block=256 grid=" + std::to_string(rows);
}

// RMS norm of fp16 rows to fp16 with a bf16 weight and no residual
// (crates/berth-kernels/src/ops.rs:108-118,600-640, csrc/ops/norm.cu:80-112: the
// normalisation ahead of the MTP input projection).  The fp16 input widens exactly to
// fp32; from there the arithmetic is that of rms_norm_kernel.
__global__ __launch_bounds__(256) void rms_norm_f16_kernel(const _Float16* __restrict__ x, const uint16_t* __restrict__ weight,
                                                           _Float16* __restrict__ y, int dim, float epsilon,
                                                           float constant_bias, float constant_scale)
{
    __shared__ double s_part[4];
    __shared__ float s_rmf;
    const int row = blockIdx.x, tid = threadIdx.x;
    const half4_t* xr = (const half4_t*)(x + (size_t)row * dim);
    double ss = 0.0;
    for (int i = tid; i < dim / 4; i += 256) {
        const half4_t v = xr[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) ss += (double)(float)v[j] * (double)(float)v[j];
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) ss += __shfl_xor(ss, d, 64);
    if ((tid & 63) == 0) s_part[tid >> 6] = ss;
    __syncthreads();
    if (tid == 0) {
        const double total = ((s_part[0] + s_part[1]) + s_part[2]) + s_part[3];
        s_rmf = (float)(1.0 / sqrt(total / dim + (double)epsilon));
    }
    __syncthreads();
    const float rmf = s_rmf;
    for (int i = tid; i < dim / 4; i += 256) {
        const half4_t v = xr[i];
        half4_t o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float w = __builtin_bit_cast(float, (uint32_t)weight[4 * i + j] << 16);
            float t = (float)v[j] * rmf;
            t = t * (w + constant_bias);
            t = t * constant_scale;
            o[j] = (_Float16)t;
        }
        *(half4_t*)(y + (size_t)row * dim + 4 * i) = o;
    }
}

std::string launch_rms_norm_f16(const void* x, const void* weight, void* y, int rows, int dim, float epsilon,
                                float constant_bias, float constant_scale, hipStream_t stream)
{
    hipLaunchKernelGGL(rms_norm_f16_kernel, dim3((unsigned)rows), dim3(256), 0, stream, (const _Float16*)x,
                       (const uint16_t*)weight, (_Float16*)y, dim, epsilon, constant_bias, constant_scale);
    hip_ok(hipGetLastError(), "rms_norm_f16 launch");
    return "rms_norm_kernel<0,half,half,bfloat16,half> block=256 grid=" + std::to_string(rows);
}

// Embedding rows (crates/berth-kernels/src/ops.rs:99-127, csrc/ops/embed.cu): out[t] =
// weight[ids[t]], bf16 -> fp32 (an exact widen) or bf16 -> fp16 (the widen, then one
// round-to-nearest-even).  ids are not range-checked, as in the reference.
template <bool F16>
__global__ __launch_bounds__(256) void embed_bf16_kernel(const uint16_t* __restrict__ weight, const int* __restrict__ ids,
                                                         void* __restrict__ out, int hidden)
{
    const int token = blockIdx.x;
    const uint16_t* row = weight + (size_t)ids[token] * hidden;
    for (int i = threadIdx.x; i < hidden; i += 256) {
        const float v = __builtin_bit_cast(float, (uint32_t)row[i] << 16);
        if (F16) ((_Float16*)out)[(size_t)token * hidden + i] = (_Float16)v;
        else ((float*)out)[(size_t)token * hidden + i] = v;
    }
}

std::string launch_embed_tokens(const void* weight, const int* ids, void* out, int hidden, int n, int f16,
                                hipStream_t stream)
{
    if (f16) hipLaunchKernelGGL(embed_bf16_kernel<true>, dim3((unsigned)n), dim3(256), 0, stream, (const uint16_t*)weight, ids, out, hidden);
    else hipLaunchKernelGGL(embed_bf16_kernel<false>, dim3((unsigned)n), dim3(256), 0, stream, (const uint16_t*)weight, ids, out, hidden);
    hip_ok(hipGetLastError(), f16 ? "embed_tokens_f16 launch" : "embed_tokens launch");
    return std::string(f16 ? "embed_bf16_f16" : "embed_bf16_f32") + " block=256 grid=" + std::to_string(n);
}

// out[row] = embedding[row] followed by hidden[row], fp16 (crates/berth-kernels/src/ops.rs:136-143,
// csrc/ops/copy.cu: the concatenation ahead of the MTP input projection)
__global__ __launch_bounds__(256) void cat_f16_last_kernel(const uint16_t* __restrict__ embedding,
                                                           const uint16_t* __restrict__ hidden,
                                                           uint16_t* __restrict__ out, int width)
{
    const size_t row = blockIdx.x;
    for (int i = threadIdx.x; i < width; i += 256) {
        out[row * 2 * width + i] = embedding[row * width + i];
        out[row * 2 * width + width + i] = hidden[row * width + i];
    }
}

std::string launch_cat_f16_last(const void* embedding, const void* hidden, void* out, int rows, int width,
                                hipStream_t stream)
{
    hipLaunchKernelGGL(cat_f16_last_kernel, dim3((unsigned)rows), dim3(256), 0, stream, (const uint16_t*)embedding,
                       (const uint16_t*)hidden, (uint16_t*)out, width);
    hip_ok(hipGetLastError(), "cat_f16_last launch");
    return "cat_f16_last block=256 grid=" + std::to_string(rows);
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

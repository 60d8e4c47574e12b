// Trellis -> fp16 weight matrix (the inner weight W, before any Hadamard).
// Counterpart of the reconstruct launch in
// crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:69-93: grid over
// (128-column blocks, tile rows), output row-major [K][slice_n].
// A wave decodes one tile row x 128 columns (8 tiles), transposes it through LDS
// and stores 16 rows of 256 contiguous bytes.
#include "exl3_decode.cuh"
#include "hadamard.cuh"
#include "launch.h"

namespace berth {

template <int BITS, int CB>
__global__ __launch_bounds__(256) void exl3_reconstruct_kernel(
    _Float16* __restrict__ out, const uint32_t* __restrict__ trellis, int tiles_n_full,
    int tile_n_offset, int slice_n, int tile_rows)
{
    __shared__ _Float16 tile[4][16][128 + 8];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nb = blockIdx.x;                       // 128-column block inside the slice
    const int kt = blockIdx.y * 4 + wave;            // tile row
    if (kt >= tile_rows) return;
    constexpr int tile_dw = 8 * BITS;

    uint32_t own[BITS];
    const uint32_t* src = trellis + ((size_t)kt * tiles_n_full + tile_n_offset + nb * 8) * tile_dw + lane * BITS;
#pragma unroll
    for (int j = 0; j < BITS; ++j) own[j] = src[j];
    uint32_t prev = fetch_prev(lane, own[BITS - 1]);
    uint32_t w2[16];
    decode_lane<BITS, CB>(own, prev, w2);

    const int col = (lane >> 3) * 16 + (lane & 7);
#pragma unroll
    for (int p = 0; p < 16; ++p) {
        half2_t v = as_half2(w2[p]);
        const int k = 2 * pair_kk(p);
        const int c = col + 8 * pair_col_half(p);
        tile[wave][k][c] = v.x;
        tile[wave][k + 1][c] = v.y;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // 16 rows x 128 halves = 16 rows x 64 half2: lane writes one half2 per row
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        half2_t v = *(const half2_t*)&tile[wave][r][2 * lane];
        *(half2_t*)(out + (size_t)(kt * 16 + r) * slice_n + nb * 128 + 2 * lane) = v;
    }
}

// Trellis -> fp16 EFFECTIVE weight: both 128-block Hadamards and both sign scales folded
// into the weight, so that a plain GEMM x @ W_eff gives the operator's output
// (crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:96-123, the reference's route for
// 1024 rows and more).  Per 128 x 128 block (kb, nb):
//     W_eff = diag(suh_kb) * Hh * W * Hh * diag(svh_nb),      Hh = H_128 / sqrt(128).
// One workgroup per block: decode into LDS as fp32, butterflies down the columns (over k),
// then along the rows (over n), both in the fixed order of had128; the element is then
// ((v / sqrt(128)) / sqrt(128)) * suh[k] * svh[n], rounded to fp16 once.
template <int BITS, int CB>
__global__ __launch_bounds__(256) void exl3_reconstruct_had_kernel(
    _Float16* __restrict__ out, const uint32_t* __restrict__ trellis, const _Float16* __restrict__ suh,
    const _Float16* __restrict__ svh, int tiles_n_full, int tile_n_offset, int slice_n)
{
    constexpr int kPitch = 128 + 4;                  // floats per LDS row: 16-byte aligned rows, columns spread over banks
    __shared__ __attribute__((aligned(16))) float blk[128][kPitch];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nb = blockIdx.x;                       // 128-column block inside the slice
    const int kb = blockIdx.y;                       // 128-row block
    constexpr int tile_dw = 8 * BITS;

    // decode: wave w takes tile rows 2w and 2w + 1 of the block
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int tr = 2 * wave + h;
        uint32_t own[BITS];
        const uint32_t* src = trellis + ((size_t)(kb * 8 + tr) * tiles_n_full + tile_n_offset + nb * 8) * tile_dw + lane * BITS;
#pragma unroll
        for (int j = 0; j < BITS; ++j) own[j] = src[j];
        uint32_t prev = fetch_prev(lane, own[BITS - 1]);
        uint32_t w2[16];
        decode_lane<BITS, CB>(own, prev, w2);
        const int col = (lane >> 3) * 16 + (lane & 7);
#pragma unroll
        for (int p = 0; p < 16; ++p) {
            half2_t v = as_half2(w2[p]);
            const int k = tr * 16 + 2 * pair_kk(p);
            const int c = col + 8 * pair_col_half(p);
            blk[k][c] = (float)v.x;
            blk[k + 1][c] = (float)v.y;
        }
    }
    __syncthreads();

    // down the columns: wave w takes columns 32w .. 32w + 31, four at a time (one per
    // 16-lane row of the wave), a lane holds eight consecutive k of its column
    const int sub = lane >> 4, l16 = lane & 15;
#pragma unroll 1
    for (int pass = 0; pass < 8; ++pass) {
        const int n = wave * 32 + pass * 4 + sub;
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = blk[8 * l16 + i][n];
        had128_row16(v, lane);
#pragma unroll
        for (int i = 0; i < 8; ++i) blk[8 * l16 + i][n] = v[i];
    }
    __syncthreads();

    // along the rows, scales, one rounding, 16-byte stores
    const global_ptr<const _Float16> g_suh = as_global(suh), g_svh = as_global(svh);
    float sv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) sv[i] = (float)g_svh[nb * 128 + 8 * l16 + i];
#pragma unroll 1
    for (int pass = 0; pass < 8; ++pass) {
        const int r = wave * 32 + pass * 4 + sub;
        float v[8];
        const float4_t lo = *(const float4_t*)&blk[r][8 * l16], hi = *(const float4_t*)&blk[r][8 * l16 + 4];
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
        v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
        had128_row16(v, lane);
        const float su = (float)g_suh[kb * 128 + r];
        half8_t o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (_Float16)((((v[i] * kRsqrt128) * kRsqrt128) * su) * sv[i]);
        *(half8_t*)(out + (size_t)(kb * 128 + r) * slice_n + nb * 128 + 8 * l16) = o;
    }
}

template <int BITS>
static void reconstruct_cb(int cb, dim3 grid, hipStream_t stream, _Float16* out, const uint32_t* tr,
                           int tiles_n_full, int tile_n_offset, int slice_n, int tile_rows)
{
    switch (cb) {
    case 0: hipLaunchKernelGGL((exl3_reconstruct_kernel<BITS, 0>), grid, dim3(256), 0, stream, out, tr, tiles_n_full, tile_n_offset, slice_n, tile_rows); break;
    case 1: hipLaunchKernelGGL((exl3_reconstruct_kernel<BITS, 1>), grid, dim3(256), 0, stream, out, tr, tiles_n_full, tile_n_offset, slice_n, tile_rows); break;
    default: hipLaunchKernelGGL((exl3_reconstruct_kernel<BITS, 2>), grid, dim3(256), 0, stream, out, tr, tiles_n_full, tile_n_offset, slice_n, tile_rows); break;
    }
}

std::string launch_reconstruct(void* unpacked, const void* packed, int size_k, int slice_n,
                               int full_n, int n_offset, int k_bits, int codebook,
                               hipStream_t stream)
{
    const int tile_rows = size_k / 16;
    dim3 grid(slice_n / 128, (tile_rows + 3) / 4);
    _Float16* out = (_Float16*)unpacked;
    const uint32_t* tr = (const uint32_t*)packed;
    const int tnf = full_n / 16, tno = n_offset / 16;
    switch (k_bits) {
    case 1: reconstruct_cb<1>(codebook, grid, stream, out, tr, tnf, tno, slice_n, tile_rows); break;
    case 2: reconstruct_cb<2>(codebook, grid, stream, out, tr, tnf, tno, slice_n, tile_rows); break;
    case 3: reconstruct_cb<3>(codebook, grid, stream, out, tr, tnf, tno, slice_n, tile_rows); break;
    case 4: reconstruct_cb<4>(codebook, grid, stream, out, tr, tnf, tno, slice_n, tile_rows); break;
    case 5: reconstruct_cb<5>(codebook, grid, stream, out, tr, tnf, tno, slice_n, tile_rows); break;
    case 6: reconstruct_cb<6>(codebook, grid, stream, out, tr, tnf, tno, slice_n, tile_rows); break;
    case 7: reconstruct_cb<7>(codebook, grid, stream, out, tr, tnf, tno, slice_n, tile_rows); break;
    default: reconstruct_cb<8>(codebook, grid, stream, out, tr, tnf, tno, slice_n, tile_rows); break;
    }
    hip_ok(hipGetLastError(), "exl3_reconstruct_kernel launch");
    return "exl3_reconstruct_kernel<" + std::to_string(k_bits) + "," + std::to_string(codebook) +
           "> grid=" + std::to_string(grid.x) + "x" + std::to_string(grid.y) + " block=256";
}

template <int BITS>
static void reconstruct_had_cb(int cb, dim3 grid, hipStream_t stream, _Float16* out, const uint32_t* tr,
                               const _Float16* suh, const _Float16* svh, int tiles_n_full, int tile_n_offset, int slice_n)
{
    switch (cb) {
    case 0: hipLaunchKernelGGL((exl3_reconstruct_had_kernel<BITS, 0>), grid, dim3(256), 0, stream, out, tr, suh, svh, tiles_n_full, tile_n_offset, slice_n); break;
    case 1: hipLaunchKernelGGL((exl3_reconstruct_had_kernel<BITS, 1>), grid, dim3(256), 0, stream, out, tr, suh, svh, tiles_n_full, tile_n_offset, slice_n); break;
    default: hipLaunchKernelGGL((exl3_reconstruct_had_kernel<BITS, 2>), grid, dim3(256), 0, stream, out, tr, suh, svh, tiles_n_full, tile_n_offset, slice_n); break;
    }
}

std::string launch_reconstruct_had(void* unpacked, const void* packed, const void* suh, const void* svh,
                                   int size_k, int slice_n, int full_n, int n_offset, int k_bits, int codebook,
                                   hipStream_t stream)
{
    dim3 grid(slice_n / 128, size_k / 128);
    _Float16* out = (_Float16*)unpacked;
    const uint32_t* tr = (const uint32_t*)packed;
    const _Float16* su = (const _Float16*)suh;
    const _Float16* sv = (const _Float16*)svh + n_offset;       // as reconstruct.cu:114
    const int tnf = full_n / 16, tno = n_offset / 16;
    switch (k_bits) {
    case 1: reconstruct_had_cb<1>(codebook, grid, stream, out, tr, su, sv, tnf, tno, slice_n); break;
    case 2: reconstruct_had_cb<2>(codebook, grid, stream, out, tr, su, sv, tnf, tno, slice_n); break;
    case 3: reconstruct_had_cb<3>(codebook, grid, stream, out, tr, su, sv, tnf, tno, slice_n); break;
    case 4: reconstruct_had_cb<4>(codebook, grid, stream, out, tr, su, sv, tnf, tno, slice_n); break;
    case 5: reconstruct_had_cb<5>(codebook, grid, stream, out, tr, su, sv, tnf, tno, slice_n); break;
    case 6: reconstruct_had_cb<6>(codebook, grid, stream, out, tr, su, sv, tnf, tno, slice_n); break;
    case 7: reconstruct_had_cb<7>(codebook, grid, stream, out, tr, su, sv, tnf, tno, slice_n); break;
    default: reconstruct_had_cb<8>(codebook, grid, stream, out, tr, su, sv, tnf, tno, slice_n); break;
    }
    hip_ok(hipGetLastError(), "exl3_reconstruct_had_kernel launch");
    return "exl3_reconstruct_had_kernel<" + std::to_string(k_bits) + "," + std::to_string(codebook) +
           "> grid=" + std::to_string(grid.x) + "x" + std::to_string(grid.y) + " block=256";
}

}  // namespace berth

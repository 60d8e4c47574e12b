// Trellis -> fp16 weight matrix (the inner weight W, before any Hadamard).
// Counterpart of the reconstruct launch in
// crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:69-93: grid over
// (128-column blocks, tile rows), output row-major [K][slice_n].
// A wave decodes one tile row x 128 columns (8 tiles), transposes it through LDS
// and stores 16 rows of 256 contiguous bytes.
#include "exl3_decode.cuh"
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

}  // namespace berth

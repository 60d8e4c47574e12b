// EXL3 linear for more than 128 rows: 256-row x 256-column tiles, every weight decoded
// once per tile and shared through LDS.
//
// The 128-row kernel keeps decoded weights in the registers of the wave that decoded
// them, so a weight is decoded once per 128 rows.  Here a weight is decoded once per 256
// rows, by one of the eight waves of a workgroup, and the other waves take it from LDS:
//
//   decode   wave w, lane l decodes, per 64 rows of K ("macro-step"), the 32 weights of
//            one octet lane: tile row w/2 of the four, tile column 8*(w%2) + l/8; its four
//            16-byte results (8 consecutive k of one column each) go to the B tile in LDS,
//            laid out [k octet][column], so an MFMA B operand is one 16-byte read and 32
//            lanes read 512 contiguous bytes.
//   MFMA     wave w owns rows 128*(w/4) .. +127 and columns 64*(w%4) .. +63 of the tile:
//            32 MFMAs per macro-step, A and B operands from LDS.
//
// A and B tiles are double-buffered; per macro-step one barrier.  Inside a macro-step a wave
// issues its 32 MFMAs on the current buffers, every operand read one pair of MFMAs ahead, and
// decodes its share of the next macro-step; the loop has no branch (row blocks past the end of
// the rows are multiplied too and never stored).  Whether the decode is issued in sixteenths
// between the MFMAs or as one block behind them makes no difference here (the other wave of
// the SIMD fills either gap): the 27B gate projection at 512 rows takes 124-130 us both ways,
// 141 with a branch around every row block's MFMAs and the decode ahead of them.  Trellis
// registers run four macro-steps ahead of the decode, A registers two.
//
// Handoff between workgroups that share a tile and the epilogue are those of the
// 128-row kernel (partial sums in register layout, summed in k order by the last
// workgroup to arrive; fp32 tile staged in LDS, output Hadamard, svh).
#pragma once

#include "exl3_gemm_kernel.cuh"

namespace berth {

constexpr int kWideAStride = 64 + 8;                    // halves per LDS row of the A tile (144 B)
constexpr int kWideABytes = 256 * kWideAStride * 2;     // one A buffer: 36864
constexpr int kWideBBytes = 8 * 256 * 16;               // one B buffer: [8 k octets][256 columns] x 16 B
constexpr int kWideSmem = 2 * kWideABytes + 2 * kWideBBytes;    // 139264

template <int BITS, int CB>
__device__ __forceinline__ void gemm_tile_wide(const GemmParams& p, const int tile_y, const int nblk, const KRange kr,
                                               unsigned char* smem)
{
    constexpr int MB = 4;
    constexpr int kZStride = 256 + 4;
    __shared__ unsigned s_last;

    const int lane = threadIdx.x & 63;
    const int wave8 = threadIdx.x >> 6;
    const int rh = wave8 >> 2;                          // row half of the MFMA tile; also the phase order
    const int cq = wave8 & 3;                           // column quarter of the MFMA tile
    const int slot = lane & 31;
    const int kh = lane >> 5;
    const TileView view = dense_tile_view(p, nblk);
    if (view.empty) return;                             // the same for every workgroup that shares the tile
    const int n0 = view.nblk * 256;
    const int m_end = p.M;
    const int m_tile = tile_y * 256;
    const int m0 = m_tile + rh * 128;
    const int rows_here = min(128, m_end - m0);         // <= 0: this row half is empty
    const int rows_first = min(128, m_end - m_tile);    // rows of the first half, >= 1
    const ExpertLin lin = view.lin;
    const _Float16* a_had = view.a_had;
    void* cout = view.cout;
    const int N = view.N, ldc = view.ldc;
    const bool active = n0 + cq * 64 < N;               // this wave's 64 output columns exist
    const int tn = ldc >> 4;                            // tiles per tile row of the weight (of the whole weight, for a slice)
    constexpr int tile_dw = 8 * BITS;
    const size_t row_dw = (size_t)tn * tile_dw;

    unsigned char* a_lds = smem;                        // [2][256][kWideAStride] halves
    unsigned char* b_lds = smem + 2 * kWideABytes;      // [2][8][256] x 16 B

    float16_t acc[MB][2];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int f = 0; f < 2; ++f)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][f][r] = 0.0f;

    {
        // ---- decode role: tile row dtr of the macro-step, tile column dtc of the 16
        const int dtr = wave8 >> 1;
        int dtc = (wave8 & 1) * 8 + (lane >> 3);
        const int du = lane & 7;
        // tile columns past the end of the weight are decoded from the first half of the
        // block instead (never used): no branch around loads
        const int dtc_ld = (n0 >> 4) + dtc < (N >> 4) ? dtc : dtc - 8;
        const global_ptr<const uint32_t> tbase = as_global(lin.trellis) + (size_t)dtr * row_dw +
                                                 (size_t)((n0 >> 4) + dtc_ld) * tile_dw + du * BITS;
        // B tile destinations of this lane: column dtc*16 + du + 8f, k octet 2*dtr + h
        unsigned char* b_dst = b_lds + ((size_t)(2 * dtr) * 256 + dtc * 16 + du) * 16;
        // ---- A fill role: thread t loads 64 bytes: row t/2, k 32*(t%2) .. +31 of the macro-step
        const int fr = threadIdx.x >> 1, fh = threadIdx.x & 1;
        const int fr_ld = min(m_tile + fr, m_end - 1);  // rows past the end repeat the last row
        const global_ptr<const u32x4_t> a_src =
            (global_ptr<const u32x4_t>)(as_global(a_had) + (size_t)fr_ld * p.K + fh * 32);
        unsigned char* a_dst = a_lds + (size_t)fr * (kWideAStride * 2) + fh * 64;
        // ---- MFMA role: operand addresses inside a buffer
        const unsigned char* a_op = a_lds + (size_t)(rh * 128 + slot) * (kWideAStride * 2) + kh * 16;
        const unsigned char* b_op = b_lds + ((size_t)kh * 256 + cq * 64 + slot) * 16;

        // Operand registers run ahead of the decode: trellis dwords four macro-steps (they come
        // from HBM and are read once), A rows two (they mostly come from the L2).
        uint32_t tr_ring[4][BITS];
        u32x4_t a_ring[2][4];
        // macro-step index s counts from the start of the range: k-block kb0 + s/2, half s%2
        const int nsteps = 2 * (kr.kb1 - kr.kb0);
        auto issue_tr = [&](int s, uint32_t (&dst)[BITS]) {
            const int sc = s < nsteps ? s : nsteps - 1;             // past the end: reread, ignored
            const global_ptr<const uint32_t> t = tbase + (size_t)(kr.kb0 * 8 + sc * 4) * row_dw;
#pragma unroll
            for (int j = 0; j < BITS; ++j) dst[j] = t[j];
        };
        auto issue_a = [&](int s, u32x4_t (&dst)[4]) {
            const int sc = s < nsteps ? s : nsteps - 1;
            const global_ptr<const u32x4_t> a = a_src + ((size_t)kr.kb0 * 128 + (size_t)sc * 64) / 8;
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[i] = a[i];
        };
        auto decode_and_fill = [&](int buf, const uint32_t (&tr)[BITS], const u32x4_t (&ar)[4]) {
            uint32_t prev = fetch_prev(lane, tr[BITS - 1]);
            uint32_t w2[16];
            decode_lane<BITS, CB>(tr, prev, w2);
            unsigned char* bd = b_dst + (size_t)buf * kWideBBytes;
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const u32x4_t q = {w2[2 * f + h], w2[4 + 2 * f + h], w2[8 + 2 * f + h], w2[12 + 2 * f + h]};
                    *(u32x4_t*)(bd + ((size_t)h * 256 + 8 * f) * 16) = q;
                }
            unsigned char* ad = a_dst + (size_t)buf * kWideABytes;
#pragma unroll
            for (int i = 0; i < 4; ++i) *(u32x4_t*)(ad + i * 16) = ar[i];
        };
        // One macro-step: the 32 MFMAs on buffer `buf` (operands of the next two MFMAs read one
        // pair ahead) and the decode of the next macro-step into the other buffers; the A rows of
        // the next macro-step go to LDS with the first four pairs, the decoded weights at the end.
        // Row blocks past the end of the rows are multiplied too (their A rows repeat the last
        // row) and never stored: the loop has no branch.
        auto fused_step = [&](int buf, const uint32_t (&tr)[BITS], const u32x4_t (&ar)[4]) {
            const unsigned char* ao = a_op + (size_t)buf * kWideABytes;
            const unsigned char* bo = b_op + (size_t)buf * kWideBBytes;
            unsigned char* ad = a_dst + (size_t)(buf ^ 1) * kWideABytes;
            unsigned char* bd = b_dst + (size_t)(buf ^ 1) * kWideBBytes;
            const uint32_t prev = fetch_prev(lane, tr[BITS - 1]);
            const LaneWindows<BITS> win(tr, prev);
            uint32_t w2[16];
            half8_t b0 = *(const half8_t*)(bo);
            half8_t b1 = *(const half8_t*)(bo + 32 * 16);
            half8_t an = *(const half8_t*)(ao);
#pragma unroll
            for (int g = 0; g < 16; ++g) {
                const int kk = g >> 2, mb = g & 3;
                const half8_t a_now = an, b0_now = b0, b1_now = b1;
                if (g < 15) {
                    const int kn = (g + 1) >> 2, mn = (g + 1) & 3;
                    an = *(const half8_t*)(ao + (size_t)mn * 32 * (kWideAStride * 2) + kn * 32);
                    if (mn == 0) {
                        b0 = *(const half8_t*)(bo + (size_t)(2 * kn) * 256 * 16);
                        b1 = *(const half8_t*)(bo + (size_t)(2 * kn) * 256 * 16 + 32 * 16);
                    }
                }
                acc[mb][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_now, b0_now, acc[mb][0], 0, 0, 0);
                acc[mb][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_now, b1_now, acc[mb][1], 0, 0, 0);
                w2[g] = decode_pair<CB>(win.state(2 * g), win.state(2 * g + 1));
                if (g < 4) *(u32x4_t*)(ad + g * 16) = ar[g];
            }
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const u32x4_t q = {w2[2 * f + h], w2[4 + 2 * f + h], w2[8 + 2 * f + h], w2[12 + 2 * f + h]};
                    *(u32x4_t*)(bd + ((size_t)h * 256 + 8 * f) * 16) = q;
                }
        };

        // prologue: macro-step 0 decoded into buffer 0; the rings hold trellis 1..4 and A 1..2
        issue_tr(0, tr_ring[0]);
        issue_a(0, a_ring[0]);
        issue_tr(1, tr_ring[1]);
        issue_a(1, a_ring[1]);
        issue_tr(2, tr_ring[2]);
        issue_tr(3, tr_ring[3]);
        decode_and_fill(0, tr_ring[0], a_ring[0]);
        issue_tr(4, tr_ring[0]);
        issue_a(2, a_ring[0]);
        __syncthreads();
        // sub-step u of a round works on macro-step s + u: MFMAs on buffer u % 2, and macro-step
        // s + u + 1 (ring slots (u + 1) % 4 and (u + 1) % 2) is decoded into the other buffer
        for (int s = 0; s < nsteps; s += 4) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (s + u >= nsteps) break;                         // workgroup-uniform
                const int buf = u & 1;
                fused_step(buf, tr_ring[(u + 1) & 3], a_ring[(u + 1) & 1]);
                issue_tr(s + u + 5, tr_ring[(u + 1) & 3]);
                issue_a(s + u + 3, a_ring[(u + 1) & 1]);
                __syncthreads();
            }
        }
    }

    // ---- handoff between the workgroups that share the tile (as in exl3_gemm_kernel.cuh)
    if (kr.parts > 1) {
        constexpr size_t kPerWave = (size_t)MB * 2 * 16 * 64;
        constexpr size_t kPerWg = 8 * kPerWave;
        unsigned* arrived = p.counters + kr.counter * p.cstride;
        unsigned* written = arrived + kGemmWrittenBase;
        if (threadIdx.x == 0) {
            unsigned old = __hip_atomic_fetch_add(arrived, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = (old == (unsigned)(kr.parts - 1)) ? 1u : 0u;
        }
        __syncthreads();
        const bool finisher = s_last != 0;
        const size_t wave_off = (size_t)wave8 * kPerWave;
        const float* all = p.partials + kr.slot0 * kPerWg + wave_off;
        if (!(finisher && kr.part == 0)) {
            float* mine = p.partials + (kr.slot0 + kr.part) * kPerWg + wave_off;
            if (active) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int f = 0; f < 2; ++f)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            if (mb * 32 + 8 * (r >> 2) < rows_here)
                                __hip_atomic_store(mine + ((mb * 2 + f) * 16 + r) * 64 + lane, acc[mb][f][r],
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (!finisher) {
            wait_own_stores();
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __syncthreads();
            if (threadIdx.x == 0) __hip_atomic_fetch_add(written, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
        if (threadIdx.x == 0) {
            const bool complete = wait_counter_bounded(written, (unsigned)(kr.parts - 1), p.spin_limit);
            __hip_atomic_store(written, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(arrived, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (!complete && p.fault)
                __hip_atomic_store(p.fault, 1u + (unsigned)kr.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            s_last = complete ? 1u : 2u;
        }
        __syncthreads();
        if (s_last == 2u) return;       // gave up: the tile stays unwritten, the host is told
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (active) {
            constexpr int kGroup = 4;                           // (mb, f) register blocks per batch
            const int first = kr.part == 0 ? 1 : 0;
            for (int j = first; j < kr.parts; ++j) {
                const float* src = all + (size_t)j * kPerWg;
#pragma unroll
                for (int g0 = 0; g0 < MB * 2; g0 += kGroup) {
                    float tmp[kGroup][16];
#pragma unroll
                    for (int bq = 0; bq < kGroup; ++bq) {
                        const int blk = g0 + bq;                // = mb * 2 + f
                        if ((blk >> 1) * 32 >= rows_here) continue;
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            tmp[bq][r] = __hip_atomic_load(src + (blk * 16 + r) * 64 + lane, __ATOMIC_RELAXED,
                                                           __HIP_MEMORY_SCOPE_AGENT);
                    }
#pragma unroll
                    for (int bq = 0; bq < kGroup; ++bq) {
                        const int blk = g0 + bq;
                        if ((blk >> 1) * 32 >= rows_here) continue;
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            acc[blk >> 1][blk & 1][r] = j == 0 ? tmp[bq][r] : acc[blk >> 1][blk & 1][r] + tmp[bq][r];
                    }
                }
            }
        }
    }

    // ---- epilogue, 32 rows at a time per row half: stage the fp32 tile, output Hadamard, svh,
    // store.  Both halves take the barriers as often as the first half needs them.
    float* z_tile = (float*)(smem + (size_t)rh * 32 * kZStride * sizeof(float));
    const int l16 = lane & 15;
    half8_t sv_blk[2];
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
        const int gn = n0 + blk * 128;
        sv_blk[blk] = gn < N ? ((global_ptr<const half8_t>)as_global(lin.svh + gn))[l16] : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        if (mb * 32 >= rows_first) break;                       // workgroup-uniform
        __syncthreads();
        if (active && mb * 32 < rows_here) {
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = 8 * (r >> 2) + 4 * kh + (r & 3);
                    z_tile[row * kZStride + cq * 64 + f * 32 + slot] = acc[mb][f][r];
                }
        }
        __syncthreads();
        const int rows_blk = min(32, rows_here - mb * 32);      // <= 0: nothing to store
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int vec = pass * 16 + cq * 4 + (lane >> 4);
            const int row = vec >> 1, blk = vec & 1;
            const int gn = n0 + blk * 128;
            if (row < rows_blk && gn < N) {
                float v[8];
                const float4_t* zp = (const float4_t*)&z_tile[row * kZStride + blk * 128 + 8 * l16];
                const float4_t z0 = zp[0], z1 = zp[1];
#pragma unroll
                for (int i = 0; i < 4; ++i) { v[i] = z0[i]; v[4 + i] = z1[i]; }
                had128_row16(v, lane);
                const half8_t sv = blk ? sv_blk[1] : sv_blk[0];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = (v[i] * kRsqrt128) * (float)sv[i];
                const size_t at = (size_t)(m0 + mb * 32 + row) * ldc + gn + 8 * l16;
                if (p.out_fp32) {
                    global_ptr<float4_t> dst = (global_ptr<float4_t>)(as_global((float*)cout) + at);
                    dst[0] = float4_t{v[0], v[1], v[2], v[3]};
                    dst[1] = float4_t{v[4], v[5], v[6], v[7]};
                } else {
                    half8_t o;
#pragma unroll
                    for (int i = 0; i < 8; ++i) o[i] = (_Float16)v[i];
                    *(global_ptr<half8_t>)(as_global((_Float16*)cout) + at) = o;
                }
            }
        }
    }
}

template <int BITS, int CB>
__device__ __forceinline__ void gemm_segment_wide(const GemmParams& p, const int w, const int u, const int stop,
                                                  unsigned char* smem)
{
    const int nblocks = ((p.N + 255) >> 8) * (p.num_slices > 0 ? p.num_slices : 1);
    const int KB = p.K >> 7;
    const int tile = u / KB;
    const int t0 = tile * KB;
    const int w_first = range_owner(p, t0);
    const int w_last = range_owner(p, t0 + KB - 1);
    KRange kr;
    kr.kb0 = u - t0;
    kr.kb1 = stop - t0;
    kr.step = 1;
    kr.part = w - w_first;
    kr.parts = w_last - w_first + 1;
    kr.counter = (size_t)tile;
    kr.slot0 = (size_t)tile * p.max_parts;
    const int t = p.tile0 + tile;
    gemm_tile_wide<BITS, CB>(p, t / nblocks, t % nblocks, kr, smem);
}

// Balanced dense launch over 256-row tiles: the (tile, k-block) units are dealt out as in
// exl3_gemm_balanced_kernel, one workgroup of eight waves per compute unit.
template <int BITS, int CB>
__global__ __launch_bounds__(512, 1) void exl3_gemm_wide_kernel(GemmParams p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int KB = p.K >> 7;
    const int w = die_major_index((int)blockIdx.x, (int)gridDim.x);
    const int u_end = range_start(p, w + 1);
    // a range is the end of one tile, any whole tiles and the start of another
    for (int u = range_start(p, w); u < u_end;) {
        const int stop = min(u_end, (u / KB + 1) * KB);
        gemm_segment_wide<BITS, CB>(p, w, u, stop, smem);
        u = stop;
        if (u < u_end) __syncthreads();                         // the epilogue's LDS tile is the next A tile
    }
}

}  // namespace berth

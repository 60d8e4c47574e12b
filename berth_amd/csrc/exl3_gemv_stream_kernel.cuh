// EXL3 linear for ONE row, as a single resident round of workgroups: one workgroup of
// sixteen waves per compute unit, every wave a contiguous run of tile rows.
//
//   c = ( Hh(x * suh) @ W ) -> Hh(.) * svh          (Hh = 128-block Hadamard / sqrt(128))
//
// The operator of crates/berth-kernels/csrc/linear.cu:209-286 at m = 1 (and of the m = 1
// bundles of crates/berth-kernels/csrc/ops/mgemm.cu:125-272), for weights large enough
// that every wave gets several tile rows.
//
//   * Work of a problem (one linear, or one slice of a bundle) = its (column block, tile
//     row) units, column block major: U = (N/128) * (K/16) units of `32*bits` bytes per
//     lane-octet, 8 octets (128 columns) per wave.  The problem's waves split the units
//     evenly: wave W takes q units, the first `rem` waves one more.  No second round, no
//     tail of half-empty compute units: the grid is at most the number of compute units
//     and every wave does the same amount of decode.
//   * A wave keeps a ring of two tile rows in registers; a tile row is reloaded with the
//     tile row two units ahead as soon as it has been decoded.  The walk crosses column
//     block boundaries without draining the ring.
//   * The workgroup rotates the activation of the k-blocks its units touch once, into
//     LDS (every wave takes some k-blocks), and writes a_had for the k-blocks whose
//     column-block-0 units it owns.  Those loads go out first of all, ahead of the split
//     arithmetic of the wave and of its first tile row: the barrier behind the rotation
//     is what the whole workgroup waits for.
//   * Decode is optionally a hybrid: of the four weight pairs of a dword, those selected
//     by LUTMASK come from a 128 KiB state -> fp16 table in LDS, which the workgroup builds
//     in place while its first loads are in flight, the others from the codebook
//     arithmetic.  The table read costs address + read + pack (2.5 vector instructions
//     per weight with the dot product) against 4.4 for the arithmetic; the LDS read rate
//     bounds how many can go that way.
//   * Partial sums: a wave writes one 128-column partial per column block it touched
//     into LDS, and the pieces of a column block are added in wave order.  A column block
//     that lies entirely inside the workgroup's units is finished there.  Otherwise every
//     workgroup that shares it adds its part, converted to 64-bit fixed point, onto the
//     block's accumulator words with one atomic add that returns the old value: integer
//     sums do not depend on the order of the adds, and the add that completes the count
//     has learnt the total in that same round trip and finishes the block.  So results
//     repeat bit for bit, and the hand-over is one memory round trip.
#pragma once

#include "exl3_gemv_kernel.cuh"


#include <utility>

namespace berth {

constexpr int kStreamWaves = 16;
constexpr int kStreamXsBlocks = 64;        // k-blocks of rotated activation a workgroup can hold
constexpr int kStreamMaxCb = 15;           // column blocks one workgroup's units can touch
constexpr int kStreamPieces = kStreamWaves + kStreamMaxCb - 1;
// dynamic LDS of a launch: [table 128 KiB, if any][rotated activation][partial pieces][piece bounds]
__host__ __device__ constexpr int stream_lds_bytes(int lutmask)
{
    return (lutmask ? 131072 : 0) + kStreamXsBlocks * 256 + kStreamPieces * 512 + 128 + 128;
}

// one problem of a bundle whose lists the host knows (mode 3)
struct StreamSlice {
    const uint32_t* trellis;
    const _Float16* suh;
    const _Float16* svh;
    void* c;
    int n_stride;
    uint16_t width128;          // columns / 128
    uint16_t had_slab;
};
constexpr int kStreamMaxSlices = 16;

struct StreamParams {
    const _Float16* a;          // input row(s): fp16 [K] (per problem when in_stride != 0)
    const _Float16* a_up;       // optional: the input is silu(a) * a_up
    ExpertLin lin[2];           // mode 0: the problems by value (one linear, or a pair)
    void* c[2];                 // mode 0 outputs; modes 1, 2: c[0] is the uniform-mode output base
    // modes 1 (uniform) and 2 (sliced): the device lists of crates/berth-kernels/src/ops.rs:264-293
    const uint64_t* b_list;
    const uint64_t* suh_list;
    const uint64_t* svh_list;
    const uint64_t* c_ptrs;
    const int* size_n_list;
    const int* n_stride_list;
    const int* had_src_list;
    _Float16* a_had;            // optional; slab per rotation source
    int mode;                   // 0 by value, 1 uniform lists, 2 sliced lists, 3 slices by value
    int in_stride;              // elements between the inputs of consecutive problems (0: shared)
    int K, N, NB, TR;           // N: row stride of trellis and output in mode 0 / 1; TR = K / 16
    int out_fp32;
    int Gp;                     // workgroups per problem (gridDim.x = problems * Gp)
    unsigned mgp;               // floor(2^32 / Gp) + 1
    unsigned q, rem;            // units per wave; the first `rem` waves of a problem take q + 1
    unsigned mq, mq1, mtr;      // floor(2^32 / d) + 1 for d = q, q + 1, TR (exact for the operands used)
    unsigned long long* accum;  // [problem][column block][128] fixed-point sums, zero between launches
    unsigned* fault;            // host-visible word for a finisher that gives up its bounded wait
    unsigned spin_limit;
    // IN == kInNorm: the input row is rms(norm_res + norm_x) * (weight + bias) * scale, rounded to
    // fp16, with norm_x and norm_res fp32 [K]; their sum also goes to norm_res_out (not an alias)
    const float* norm_x;
    const float* norm_res;
    float* norm_res_out;
    const uint16_t* norm_weight;
    float norm_eps, norm_bias, norm_scale;
    int norm_weight_bf16;
    const float* out_add;       // optional fp32 [N] (one problem, fp32 output): added to the output row
    StreamSlice slice[kStreamMaxSlices];    // mode 3: the problems, by value
};

__device__ __forceinline__ unsigned div_magic(unsigned n, unsigned m) { return __umulhi(n, m); }

typedef __attribute__((address_space(3))) const uint16_t* lds_u16_ptr;

// LDS byte address 2 * s of the table entry of the 16-bit state in the low / high half of r
__device__ __forceinline__ uint32_t lut_addr_lo(uint32_t r)
{
    uint32_t a;
    asm("v_add_u32_sdwa %0, %1, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_0" : "=v"(a) : "v"(r));
    return a;
}
__device__ __forceinline__ uint32_t lut_addr_hi(uint32_t r)
{
    uint32_t a;
    asm("v_add_u32_sdwa %0, %1, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_1 src1_sel:WORD_1" : "=v"(a) : "v"(r));
    return a;
}
__device__ __forceinline__ uint32_t lut_read(uint32_t addr) { return *(lds_u16_ptr)(uintptr_t)addr; }

__host__ __device__ constexpr int popcount4(int m) { return (m & 1) + ((m >> 1) & 1) + ((m >> 2) & 1) + ((m >> 3) & 1); }

// Decode of a lane's 32 weights of one tile row, some pairs through the table, in three
// steps so that the table reads are in flight while the other pairs are computed:
// addresses() fills the table addresses, the caller issues the reads, finish() decodes
// the arithmetic pairs and packs the table values.
//
// 4 bits per weight: pair pp of dword j (w2[4j + pp]) holds the windows that end q bits
// into the dword's big-endian chunk, pp 0: q = 4, 8; 1: q = 12, 16; 2: q = 20, 24; 3: q =
// 28, 32.  A funnel shift of (previous chunk : chunk) by 16 - ph leaves the windows ending
// at q = ph and q = 16 + ph in the two halves of one register, and q = 16 and 32 are the
// halves of the dword as loaded; a half becomes a table address with one SDWA add.
// Other bit rates: windows from the shared extraction, address = state << 1; pair p goes
// through the table when bit (p & 3) of LUTMASK is set.
template <int BITS, int CB, int LUTMASK>
struct HybridDecode {
    static constexpr int kTablePairs = 4 * popcount4(LUTMASK);
    uint32_t X[BITS == 4 ? 5 : 1];
    uint32_t m[BITS == 4 ? 4 : 1];

    __device__ __forceinline__ void addresses(const uint32_t (&own)[BITS], uint32_t prev,
                                              uint32_t (&addr)[kTablePairs ? 2 * kTablePairs : 1])
    {
        if constexpr (BITS == 4) {
            X[0] = __builtin_amdgcn_alignbit(prev, prev, 16);
#pragma unroll
            for (int j = 0; j < 4; ++j) X[j + 1] = __builtin_amdgcn_alignbit(own[j], own[j], 16);
            int n = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t X0 = X[j], X1 = X[j + 1], raw = own[j], rawprev = j == 0 ? prev : own[j - 1];
                uint32_t r4 = 0, r8 = 0, r12 = 0;
                if constexpr ((LUTMASK & 1) || (LUTMASK & 4)) {
                    r4 = __builtin_amdgcn_alignbit(X0, X1, 12);
                    r8 = __builtin_amdgcn_alignbit(X0, X1, 8);
                }
                if constexpr ((LUTMASK & 2) || (LUTMASK & 8)) r12 = __builtin_amdgcn_alignbit(X0, X1, 4);
                if constexpr (!(LUTMASK & 1) || !(LUTMASK & 2)) m[j] = (rawprev & 0xffff0000u) | (raw & 0x0000ffffu);
                if constexpr (LUTMASK & 1) { addr[n++] = lut_addr_hi(r4); addr[n++] = lut_addr_hi(r8); }
                if constexpr (LUTMASK & 2) { addr[n++] = lut_addr_hi(r12); addr[n++] = lut_addr_lo(raw); }
                if constexpr (LUTMASK & 4) { addr[n++] = lut_addr_lo(r4); addr[n++] = lut_addr_lo(r8); }
                if constexpr (LUTMASK & 8) { addr[n++] = lut_addr_lo(r12); addr[n++] = lut_addr_hi(raw); }
            }
        } else if constexpr (LUTMASK != 0) {
            LaneWindows<BITS> win(own, prev);
            int n = 0;
#pragma unroll
            for (int p = 0; p < 16; ++p)
                if ((LUTMASK >> (p & 3)) & 1) {
                    addr[n++] = win.state(2 * p) << 1;
                    addr[n++] = win.state(2 * p + 1) << 1;
                }
        }
    }

    __device__ __forceinline__ void finish(const uint32_t (&own)[BITS], uint32_t prev,
                                           const uint32_t (&t)[kTablePairs ? 2 * kTablePairs : 1], uint32_t (&w2)[16])
    {
        if constexpr (LUTMASK == 0) {
            decode_lane<BITS, CB>(own, prev, w2);
        } else if constexpr (BITS == 4) {
            int n = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t X1 = X[j + 1];
                if constexpr (LUTMASK & 1) { w2[4 * j] = t[n] | (t[n + 1] << 16); n += 2; }
                else w2[4 * j] = decode_pair<CB>(__builtin_amdgcn_ubfe(m[j], 12, 16), __builtin_amdgcn_ubfe(m[j], 8, 16));
                if constexpr (LUTMASK & 2) { w2[4 * j + 1] = t[n] | (t[n + 1] << 16); n += 2; }
                else w2[4 * j + 1] = decode_pair<CB>(__builtin_amdgcn_ubfe(m[j], 4, 16), __builtin_amdgcn_ubfe(X1, 16, 16));
                if constexpr (LUTMASK & 4) { w2[4 * j + 2] = t[n] | (t[n + 1] << 16); n += 2; }
                else w2[4 * j + 2] = decode_pair<CB>(__builtin_amdgcn_ubfe(X1, 12, 16), __builtin_amdgcn_ubfe(X1, 8, 16));
                if constexpr (LUTMASK & 8) { w2[4 * j + 3] = t[n] | (t[n + 1] << 16); n += 2; }
                else w2[4 * j + 3] = decode_pair<CB>(__builtin_amdgcn_ubfe(X1, 4, 16), __builtin_amdgcn_ubfe(X1, 0, 16));
            }
        } else {
            LaneWindows<BITS> win(own, prev);
            int n = 0;
#pragma unroll
            for (int p = 0; p < 16; ++p) {
                if ((LUTMASK >> (p & 3)) & 1) { w2[p] = t[n] | (t[n + 1] << 16); n += 2; }
                else w2[p] = decode_pair<CB>(win.state(2 * p), win.state(2 * p + 1));
            }
        }
    }
};


// Cross-workgroup sums of a column block travel as 64-bit words of three fields: bits 16..63
// the value as a signed integer in units of 2^-18, bits 8..15 the number of contributions that
// did not fit (magnitude 2^23 or more, or not a number), bits 0..7 the number of contributions.
// Integer addition is associative, so the sharers' atomic adds give the same bits in whatever
// order they land, and the add that returns the full count has learnt the total in the same
// round trip.  At most 64 sharers add to a word, so neither the counts nor the value wrap; a
// word with a contribution that did not fit yields a NaN.
constexpr int kFixedBits = 18;
constexpr int kFixedMaxSharers = 64;
__device__ __forceinline__ unsigned long long to_fixed_tagged(float z)
{
    const double d = (double)z * (double)(1 << kFixedBits);
    if (!(__builtin_fabs(d) < 2199023255552.0)) return 0x101ull;          // 2^41
    return ((unsigned long long)(long long)__builtin_rint(d) << 16) | 1ull;
}
__device__ __forceinline__ float from_fixed_tagged(unsigned long long t)
{
    if ((t >> 8) & 0xffull) return __builtin_nanf("");
    return (float)((double)((long long)t >> 16) * (1.0 / (double)(1 << kFixedBits)));
}

// f(0); if more: f(1); ... each call nested inside the previous one's branch
template <int J, int N, class F>
__device__ __forceinline__ void nested_tail(unsigned count, F&& f)
{
    if constexpr (J < N) {
        if ((unsigned)J < count) {
            f(std::integral_constant<int, J>{});
            nested_tail<J + 1, N>(count, f);
        }
    }
}

// Tile rows a wave keeps in flight.  Two: with sixteen waves per compute unit that is what the
// memory's latency takes at the rate the decode consumes them; deeper rings only lengthen the
// queues that everything else (the first loads of the launch, the hand-over at its end) waits in
// (27B layer set at 4 bits per weight, four launches: 67.1 us with four, 65.3 with two).
template <int BITS> struct StreamRing {
    static constexpr int depth = 2;
};

// a pointer every lane of the wave agrees on, moved to scalar registers
template <typename T>
__device__ __forceinline__ global_ptr<T> uniform_ptr(global_ptr<T> q)
{
    const uint64_t v = (uint64_t)q;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return (global_ptr<T>)(((uint64_t)hi << 32) | lo);
}

// What the input row is: the fp16 row as given; silu(a) * a_up (the gated activation of an MLP's
// down projection, formed with the fp16 steps of berth_ops_silu_mul); or the RMS norm of a
// fp32 row with the residual added first (the steps of berth_ops_rms_norm_res_in).
constexpr int kInPlain = 0, kInSilu = 1, kInNorm = 2;

template <int BITS, int CB, int IN, int LUTMASK>
__global__ __launch_bounds__(1024, 1) void exl3_gemv_stream_kernel(StreamParams p)
{
    constexpr bool SILU = IN == kInSilu, NORM = IN == kInNorm;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    constexpr int kLutBytes = LUTMASK ? 131072 : 0;       // the table sits at LDS offset 0
    constexpr int kXsOff = kLutBytes;
    constexpr int kRedOff = kXsOff + kStreamXsBlocks * 256;
    constexpr int kMetaOff = kRedOff + kStreamPieces * 512;
    constexpr int RING = StreamRing<BITS>::depth;
    uint32_t* const xs = (uint32_t*)(lds + kXsOff);
    float* const red = (float*)(lds + kRedOff);
    unsigned* const piece_first = (unsigned*)(lds + kMetaOff);
    unsigned* const piece_last = piece_first + 16;
    double* const norm_part = (double*)(lds + kMetaOff + 128);         // NORM: one sum of squares per wave

    // The scalar fields sit in the first six lines of the argument block; the by-value problems
    // behind them are read by the launches that use them (touching all sixteen lines at the
    // head cost every launch: 1.4 us per four-launch layer set, measured).
    static_assert(offsetof(StreamParams, slice) <= 6 * 64 && sizeof(StreamParams) <= 16 * 64, "argument lines touched below");
    touch_kernel_arguments<6>();
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned prob = div_magic(blockIdx.x, p.mgp);
    const unsigned gl = blockIdx.x - prob * (unsigned)p.Gp;

    // ---- this problem's tensors
    ExpertLin lin = p.lin[p.mode == 0 ? prob : 0];
    int n_stride = p.N, had_slab = 0, width = p.N;
    void* cout = p.c[p.mode == 0 ? prob : 0];
    if (p.mode == 3) {
        const StreamSlice& sl = p.slice[prob];
        lin.trellis = sl.trellis;
        lin.suh = sl.suh;
        lin.svh = sl.svh;
        cout = sl.c;
        width = (int)sl.width128 * 128;
        n_stride = sl.n_stride;
        had_slab = (int)sl.had_slab;
    } else if (p.mode) {
        lin.trellis = (const uint32_t*)p.b_list[prob];
        lin.svh = (const _Float16*)p.svh_list[prob];
        if (p.mode == 2) {
            width = p.size_n_list[prob];
            n_stride = p.n_stride_list[prob];
            had_slab = p.had_src_list[prob];
            lin.suh = (const _Float16*)p.suh_list[had_slab];
            cout = (void*)p.c_ptrs[prob];
        } else {
            lin.suh = (const _Float16*)p.suh_list[prob];
            had_slab = (int)prob;
            cout = (char*)p.c[0] + (size_t)prob * p.N * (p.out_fp32 ? 4 : 2);
        }
    }
    const bool write_had = p.a_had && (p.mode != 0 || prob == 0);

    // ---- the static split, workgroup level: units [u0, u1)
    // (a slice narrower than the bundle's width ends early: its units stop at its last column block)
    const unsigned TR = (unsigned)p.TR;
    const unsigned u_end = (unsigned)(width >> 7) * TR;
    const unsigned W0 = gl * kStreamWaves;
    const unsigned u0 = min(W0 * p.q + min(W0, p.rem), u_end);
    const unsigned u1 = min((W0 + kStreamWaves) * p.q + min(W0 + kStreamWaves, p.rem), u_end);
    if (u0 >= u1) return;
    const unsigned cb_first = div_magic(u0, p.mtr);
    // The k-blocks these units touch are a cyclic run of nk k-blocks from that of the first
    // unit (the walk wraps from the last tile row of a column block to tile row 0 of the
    // next); k-block a_lo + i, taken modulo K / 128, is held in slot i of the LDS region.
    const unsigned KB = TR >> 3;
    const unsigned r_lo = u0 - cb_first * TR;
    unsigned a_lo = r_lo >> 3;
    unsigned nk = ((r_lo & 7u) + (u1 - u0) + 7u) >> 3;
    if (nk >= KB) {
        nk = KB;
        a_lo = 0;
    }
    // ---- first of all the activation and the scales of this wave's share of those k-blocks
    // (slots wave, wave + 16, ...): the rotation is what the whole workgroup waits for
    constexpr int kRot = kStreamXsBlocks / kStreamWaves;
    const global_ptr<const half2_t> xin = (global_ptr<const half2_t>)as_global(p.a + (size_t)prob * p.in_stride);
    const global_ptr<const half2_t> uin = (global_ptr<const half2_t>)as_global(p.a_up + (size_t)prob * p.in_stride);
    const global_ptr<const half2_t> sin = (global_ptr<const half2_t>)as_global(lin.suh);
    half2_t rot_x[kRot], rot_s[kRot], rot_u[kRot];
    float2_t nrm_v[NORM ? kRot : 1];
    uint32_t nrm_w[NORM ? kRot : 1];
    unsigned rot_kb[kRot];
#pragma unroll
    for (int t = 0; t < kRot; ++t) {
        const unsigned i = (unsigned)wave + t * kStreamWaves;
        unsigned kb = a_lo + (i < nk ? i : 0u);                         // past the end: any valid k-block, unused
        kb = kb >= KB ? kb - KB : kb;
        rot_kb[t] = kb;
        if constexpr (NORM) {
            const float2_t xv = ((global_ptr<const float2_t>)as_global(p.norm_x))[kb * 64 + lane];
            const float2_t rv = ((global_ptr<const float2_t>)as_global(p.norm_res))[kb * 64 + lane];
            nrm_w[t] = ((global_ptr<const uint32_t>)as_global((const uint32_t*)p.norm_weight))[kb * 64 + lane];
            nrm_v[t] = float2_t{rv.x + xv.x, rv.y + xv.y};
        } else {
            rot_x[t] = xin[kb * 64 + lane];
        }
        rot_s[t] = sin[kb * 64 + lane];
        if (SILU) rot_u[t] = uin[kb * 64 + lane];
    }
    // NORM: this thread's strided share of the whole row, for the sum of squares, asked for now
    // so that it arrives behind the split arithmetic instead of being waited for later
    constexpr int kNormAhead = 4;                           // covers K <= 8192; a longer row is read in the loop below
    float2_t row_x[NORM ? kNormAhead : 1], row_r[NORM ? kNormAhead : 1];
    if constexpr (NORM) {
#pragma unroll
        for (int j = 0; j < kNormAhead; ++j) {
            const unsigned e = threadIdx.x + (unsigned)j * (kStreamWaves * 64);
            const unsigned ec = e < (unsigned)p.K / 2 ? e : 0u;         // past the end: any valid element, unused
            row_x[j] = ((global_ptr<const float2_t>)as_global(p.norm_x))[ec];
            row_r[j] = ((global_ptr<const float2_t>)as_global(p.norm_res))[ec];
        }
    }

    // ---- this wave's units [uw0, uw1) and its first tile row
    const unsigned Ww = W0 + (unsigned)wave;
    const unsigned uw0 = min(Ww * p.q + min(Ww, p.rem), u_end);
    const unsigned uw1 = min((Ww + 1) * p.q + min(Ww + 1, p.rem), u_end);
    constexpr int tile_dw = 8 * BITS;
    const long row_dw = (long)(n_stride >> 4) * tile_dw;
    const long wrap_dw = (long)(8 * tile_dw) - (long)(TR - 1) * row_dw;
    // (a wave without units, possible only behind the end of a narrow slice, reads the
    // workgroup's first unit and never uses it)
    const unsigned ufirst = uw0 < uw1 ? uw0 : u0;
    unsigned cb = div_magic(ufirst, p.mtr);
    unsigned r = ufirst - cb * TR;
    const int lane_dw = lane * BITS;
    // the walk's pointer is the same in every lane: held in scalar registers, so that stepping it
    // costs no vector instruction and the loads take it as their scalar base
    global_ptr<const uint32_t> pbase =
        uniform_ptr(as_global(lin.trellis) + (long)cb * (8 * tile_dw) + (long)r * row_dw);
    unsigned p_r = r;                                       // tile row of the unit pbase points at
    unsigned p_left = uw0 < uw1 ? uw1 - uw0 - 1 : 0u;       // units after it that are still this wave's
    uint32_t own[RING][BITS];
    auto prologue_row = [&](int j) {
        load_tile_dwords<BITS>(pbase + lane_dw, own[j]);
        const long step = p_left == 0 ? 0 : (p_r == TR - 1 ? wrap_dw : row_dw);
        pbase += step;
        p_r = p_left == 0 ? p_r : (p_r == TR - 1 ? 0u : p_r + 1);
        p_left = p_left == 0 ? 0u : p_left - 1;
        __builtin_amdgcn_sched_barrier(0);
    };
    // Only the first tile row goes out ahead of the rotation: whole rings of sixteen waves are
    // more than the compute unit's request queue holds, the later waves would sit in the
    // issue of their loads until the burst has drained at the memory's rate, and the barrier
    // below waits for the slowest wave.
    prologue_row(0);
    // the output scale of the column block this wave finishes at the end: asked for now, so
    // that the hand-over does not wait for it
    const unsigned cb_last = div_magic(u1 - 1, p.mtr);
    const unsigned ncb = cb_last - cb_first + 1;
    half2_t sv_mine = {};
    float2_t add_mine = {0.0f, 0.0f};
    if ((unsigned)wave < ncb && (cb_first + (unsigned)wave) * 128u < (unsigned)width) {
        sv_mine = ((global_ptr<const half2_t>)as_global(lin.svh + (cb_first + (unsigned)wave) * 128))[lane];
        if (p.out_add) add_mine = ((global_ptr<const float2_t>)as_global(p.out_add + (cb_first + (unsigned)wave) * 128))[lane];
    }
    if (threadIdx.x < 16) {
        piece_first[threadIdx.x] = 0xffffffffu;
        piece_last[threadIdx.x] = 0u;
    }

    // ---- the table: built in place while the first tile rows and the activation are on
    // their way (the vector ALU has nothing else to do until they arrive).  Thread t writes
    // the entries of states 2 (t + 1024 j), + 1 as one dword: consecutive lanes, consecutive
    // dwords.
    if constexpr (LUTMASK != 0) {
        uint32_t* const tab = (uint32_t*)lds;
#pragma unroll 8
        for (int j = 0; j < 32; ++j) {
            const uint32_t s2 = 2u * (threadIdx.x + 1024u * (unsigned)j);
            tab[threadIdx.x + 1024u * (unsigned)j] = decode_pair<CB>(s2, s2 + 1u);
        }
    }
    // ---- NORM: every workgroup sums the squares of the whole row (its k-blocks may be only a
    // part of it), in double: per thread over a strided share, per wave by butterflies, the
    // sixteen waves' sums added in order; then y = ((v * rmf) * (w + bias)) * scale rounded to
    // fp16, as rms_norm_kernel forms it
    if constexpr (NORM) {
        double ss = 0.0;
#pragma unroll
        for (int j = 0; j < kNormAhead; ++j) {
            const unsigned e = threadIdx.x + (unsigned)j * (kStreamWaves * 64);
            if (e < (unsigned)p.K / 2) {
                const float2_t v = {row_r[j].x + row_x[j].x, row_r[j].y + row_x[j].y};
                ss += (double)v.x * (double)v.x;
                ss += (double)v.y * (double)v.y;
                // the first workgroup of the first problem writes the updated residual stream
                if (prob == 0 && gl == 0) ((global_ptr<float2_t>)as_global(p.norm_res_out))[e] = v;
            }
        }
        for (unsigned e = threadIdx.x + kNormAhead * kStreamWaves * 64; e < (unsigned)p.K / 2; e += kStreamWaves * 64) {
            const float2_t xv = ((global_ptr<const float2_t>)as_global(p.norm_x))[e];
            const float2_t rv = ((global_ptr<const float2_t>)as_global(p.norm_res))[e];
            const float2_t v = {rv.x + xv.x, rv.y + xv.y};
            ss += (double)v.x * (double)v.x;
            ss += (double)v.y * (double)v.y;
            // the first workgroup of the first problem writes the updated residual stream
            if (prob == 0 && gl == 0) ((global_ptr<float2_t>)as_global(p.norm_res_out))[e] = v;
        }
        // butterflies over lane distances 32 .. 1 (the order of the separate norm kernel's wave sum),
        // the partner's two dwords fetched with DPP moves and the row swaps instead of LDS permutes
        auto partner = [](double v, auto move) {
            const uint64_t b = __builtin_bit_cast(uint64_t, v);
            const float lo = move(__builtin_bit_cast(float, (uint32_t)b));
            const float hi = move(__builtin_bit_cast(float, (uint32_t)(b >> 32)));
            return __builtin_bit_cast(double, (uint64_t)__builtin_bit_cast(uint32_t, lo) |
                                                  ((uint64_t)__builtin_bit_cast(uint32_t, hi) << 32));
        };
        ss += partner(ss, [](float f) { return lane_xor_swap32(f); });
        ss += partner(ss, [](float f) { return lane_xor_swap16(f); });
        ss += partner(ss, [](float f) { return lane_xor_dpp<8>(f); });
        ss += partner(ss, [](float f) { return lane_xor_dpp<4>(f); });
        ss += partner(ss, [](float f) { return lane_xor_dpp<2>(f); });
        ss += partner(ss, [](float f) { return lane_xor_dpp<1>(f); });
        if (lane == 0) norm_part[wave] = ss;
        __syncthreads();
        double total = 0.0;
#pragma unroll
        for (int w = 0; w < kStreamWaves; ++w) total += norm_part[w];
        const float rmf = (float)(1.0 / sqrt(total / (double)p.K + (double)p.norm_eps));
#pragma unroll
        for (int t = 0; t < kRot; ++t) {
            const float w0 = p.norm_weight_bf16 ? __builtin_bit_cast(float, nrm_w[t] << 16)
                                                : (float)__builtin_bit_cast(_Float16, (uint16_t)(nrm_w[t] & 0xffffu));
            const float w1 = p.norm_weight_bf16 ? __builtin_bit_cast(float, nrm_w[t] & 0xffff0000u)
                                                : (float)__builtin_bit_cast(_Float16, (uint16_t)(nrm_w[t] >> 16));
            float t0 = nrm_v[t].x * rmf, t1 = nrm_v[t].y * rmf;
            t0 = t0 * (w0 + p.norm_bias);
            t1 = t1 * (w1 + p.norm_bias);
            t0 = t0 * p.norm_scale;
            t1 = t1 * p.norm_scale;
            rot_x[t].x = (_Float16)t0;
            rot_x[t].y = (_Float16)t1;
        }
    }
    // ---- rotate; a_had: the workgroup that owns tile row 8 * kb of column block 0 writes k-block kb
    const global_ptr<half2_t> hout = (global_ptr<half2_t>)as_global(p.a_had + (size_t)had_slab * p.K);
#pragma unroll
    for (int t = 0; t < kRot; ++t) {
        const unsigned i = (unsigned)wave + t * kStreamWaves;
        if (i >= nk) break;
        half2_t x = rot_x[t];
        if (SILU) {
            x.x = silu_mul_h(x.x, rot_u[t].x);
            x.y = silu_mul_h(x.y, rot_u[t].y);
        }
        float v0 = (float)x.x * (float)rot_s[t].x;
        float v1 = (float)x.y * (float)rot_s[t].y;
        had128_wave(v0, v1, lane);
        half2_t rotated;
        rotated.x = (_Float16)(v0 * kRsqrt128);
        rotated.y = (_Float16)(v1 * kRsqrt128);
        xs[i * 64 + lane] = as_u32(rotated);
        if (write_had && u0 <= 8 * rot_kb[t] && 8 * rot_kb[t] < u1) hout[rot_kb[t] * 64 + lane] = rotated;
    }
    __syncthreads();
    // the rest of the ring goes out behind the barrier: a wave whose loads wait for room in
    // the compute unit's request queue then holds up nobody but itself
#pragma unroll
    for (int j = 1; j < RING; ++j) prologue_row(j);

    // ---- the walk
    // LDS byte offset of the rotated activation of tile row r of the current column block
    const unsigned xoff_wrap = kXsOff + (a_lo ? (KB - a_lo) * 256u : 0u);     // tile row 0 of a later column block
    unsigned xoff = kXsOff + (r << 5) - a_lo * 256u;
    if (cb != cb_first) xoff = xoff_wrap + (r << 5);
    unsigned piece = (unsigned)wave + (cb - cb_first);
    unsigned left = uw0 < uw1 ? uw1 - uw0 : 0u;
    float acc0 = 0.0f, acc1 = 0.0f;
    const int col = (lane >> 3) * 16 + (lane & 7);

    auto flush = [&](unsigned pc) {
        red[pc * 128 + col] = acc0;
        red[pc * 128 + col + 8] = acc1;
        if (lane == 0) {
            atomicMin(&piece_first[pc - (unsigned)wave], (unsigned)wave);
            atomicMax(&piece_last[pc - (unsigned)wave], (unsigned)wave);
        }
    };

    // One tile row: table addresses and reads first, the next tile row's load, the
    // arithmetic pairs while the table reads are in flight, then the dot products.
    auto stage = [&](uint32_t (&mine)[BITS], bool prefetch) {
        using Dec = HybridDecode<BITS, CB, LUTMASK>;
        constexpr int NT = Dec::kTablePairs ? 2 * Dec::kTablePairs : 1;
        Dec dec;
        const uint32_t prev = fetch_prev(lane, mine[BITS - 1]);
        uint32_t addr[NT], t[NT], w2[16];
        dec.addresses(mine, prev, addr);
        const uint4* xp = (const uint4*)(lds + xoff);
        const uint4 xa = xp[0], xb = xp[1];
        if constexpr (Dec::kTablePairs != 0) {
#pragma unroll
            for (int i = 0; i < NT; ++i) t[i] = lut_read(addr[i]);
        }
        __builtin_amdgcn_sched_barrier(0);
        auto reload = [&]() {
            if (prefetch) {
                load_tile_dwords<BITS>(pbase + lane_dw, mine);
                const long step = p_left == 0 ? 0 : (p_r == TR - 1 ? wrap_dw : row_dw);
                pbase += step;
                p_r = p_left == 0 ? p_r : (p_r == TR - 1 ? 0u : p_r + 1);
                p_left = p_left == 0 ? 0u : p_left - 1;
            }
        };
        // the 4-bit hybrid keeps what it still needs of the tile row in its own registers,
        // so the reload can go out before the arithmetic pairs
        if constexpr (BITS == 4 && LUTMASK != 0) {
            reload();
            dec.finish(mine, prev, t, w2);
        } else {
            dec.finish(mine, prev, t, w2);
            reload();
        }
        __builtin_amdgcn_sched_barrier(0);
        const uint32_t xk[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
        for (int qq = 0; qq < 16; ++qq) {
            if (pair_col_half(qq)) acc1 = __builtin_amdgcn_fdot2(as_half2(w2[qq]), as_half2(xk[pair_kk(qq)]), acc1, false);
            else acc0 = __builtin_amdgcn_fdot2(as_half2(w2[qq]), as_half2(xk[pair_kk(qq)]), acc0, false);
        }
        ++r;
        xoff += 32;
        if (r == TR) {
            flush(piece);
            acc0 = acc1 = 0.0f;
            ++piece;
            ++cb;
            r = 0;
            xoff = xoff_wrap;
        }
    };

    // whole rings: straight-line, one exit, so that the wait before each tile row's use
    // is exactly "all but the RING - 1 loads issued after it"
    const unsigned groups = left / RING;
    // A wave runs its tile rows at the highest user priority and steps it down over the
    // second half of its run (to 2 at a half, 1 at three quarters, 0 for the last eighth).
    // Measured on the four launches of a 27B layer set, interleaved runs on one machine:
    // 66.4 us without, 64.9 with a constant 3, 63.3 with quarter steps, 62.9 with these;
    // the opposite ramp and two ramps per run are no better than none.
    const unsigned g1 = groups >> 1, g2 = groups - (groups >> 2), g3 = groups - (groups >> 3);
    __builtin_amdgcn_s_setprio(3);
    for (unsigned g = 0; g < groups; ++g) {
        if (g == g1) __builtin_amdgcn_s_setprio(2);
        if (g == g2) __builtin_amdgcn_s_setprio(1);
        if (g == g3) __builtin_amdgcn_s_setprio(0);
#pragma unroll
        for (int j = 0; j < RING; ++j) stage(own[j], true);
    }
    __builtin_amdgcn_s_setprio(0);
    // the remaining tile rows (fewer than RING), nested so that each is reached one way only
    const unsigned tail = left - groups * RING;
    nested_tail<0, RING - 1>(tail, [&](auto J) { stage(own[decltype(J)::value], false); });
    if (r != 0 && uw0 < uw1) flush(piece);
    __syncthreads();

    // ---- finish the column blocks: wave w takes column blocks cb_first + w, + 16, ...
    const long pslot = (long)prob * p.NB;
    static_assert(kStreamMaxCb <= kStreamWaves, "one pass: wave w finishes column block cb_first + w");
    for (unsigned cbi = (unsigned)wave; cbi < ncb; cbi += kStreamWaves) {
        const unsigned cbx = cb_first + cbi;
        if (cbx * 128u >= (unsigned)width) continue;             // a narrower slice of a bundle: nothing there
        const half2_t sv = sv_mine;
        const unsigned wf = piece_first[cbi], wl = piece_last[cbi];
        float z0 = 0.0f, z1 = 0.0f;
        for (unsigned wv = wf; wv <= wl; ++wv) {
            const float2_t part = *(const float2_t*)&red[(wv + cbi) * 128 + 2 * lane];
            z0 += part.x;
            z1 += part.y;
        }
        const bool whole = u0 <= cbx * TR && (cbx + 1) * TR <= u1;
        if (!whole) {
            // contributors: the workgroups from the owner of the column block's first unit
            // to the owner of its last unit
            const unsigned ua = cbx * TR, ub = (cbx + 1) * TR - 1;
            const unsigned big = p.rem * (p.q + 1);
            const unsigned wa = ua < big ? div_magic(ua, p.mq1) : p.rem + div_magic(ua - big, p.mq);
            const unsigned wb = ub < big ? div_magic(ub, p.mq1) : p.rem + div_magic(ub - big, p.mq);
            const unsigned count = (wb >> 4) - (wa >> 4) + 1;
            unsigned long long* const word = p.accum + ((size_t)(pslot + cbx) * 128 + 2 * lane);
            const unsigned long long f0 = to_fixed_tagged(z0), f1 = to_fixed_tagged(z1);
            unsigned long long t0 = __hip_atomic_fetch_add(word, f0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + f0;
            unsigned long long t1 = __hip_atomic_fetch_add(word + 1, f1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + f1;
            // the sharer whose add completed column 0 finishes the column block
            const unsigned arrived = (unsigned)__builtin_amdgcn_readfirstlane((int)((unsigned)t0 & 0xffu));
            if (arrived != count) {
                // more contributions than sharers: the accumulator was not zero when the launch
                // began (an earlier launch died, or two launches overlapped on this device).
                // Nobody can finish the block then: it stays unwritten, and the host is told.
                if (arrived > count && p.fault && lane == 0)
                    __hip_atomic_store(p.fault, 0x40000001u + (unsigned)cbx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                continue;
            }
            // usually every column is complete by then; one that another sharer's add had not
            // reached yet is read again (that sharer's add is in flight: the wait is short)
            unsigned spins = 0;
            while (true) {
                const bool done = ((unsigned)t0 & 0xffu) == count && ((unsigned)t1 & 0xffu) == count;
                if (__builtin_amdgcn_ballot_w64(!done) == 0ull) break;
                if (++spins > p.spin_limit) {
                    // a contributor is missing: say so, and leave no plausible numbers behind
                    if (p.fault && lane == 0)
                        __hip_atomic_store(p.fault, 0x40000001u + (unsigned)cbx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    t0 = t1 = 0x100ull;
                    break;
                }
                if (!done) {
                    t0 = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    t1 = __hip_atomic_load(word + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(word + 1, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            z0 = from_fixed_tagged(t0);
            z1 = from_fixed_tagged(t1);
        }
        // output Hadamard, svh, store
        had128_wave(z0, z1, lane);
        z0 = (z0 * kRsqrt128) * (float)sv.x;
        z1 = (z1 * kRsqrt128) * (float)sv.y;
        const size_t at = (size_t)cbx * 128 + 2 * lane;
        if (p.out_fp32) {
            float2_t o = {z0 + add_mine.x, z1 + add_mine.y};
            *(float2_t*)((float*)cout + at) = o;
        } else {
            half2_t o = {(_Float16)z0, (_Float16)z1};
            *(half2_t*)((_Float16*)cout + at) = o;
        }
    }
}

}  // namespace berth

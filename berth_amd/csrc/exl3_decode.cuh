// EXL3 trellis decode for one lane: 32 consecutive stream positions of a 16x16
// tile -> 16 packed fp16 pairs.  Shared by the reconstruct, GEMV and GEMM kernels.
//
// Tensor contract (crates/berth-exl3/src/linear.rs:285-324,
// crates/berth-kernels/src/lib.rs:88-107): trellis is u16 [K/16][N/16][16*bits];
// one [kt][nt] entry is one tile of 256 weights, `bits` new bits per weight, and
// the weight's 16-bit state is the window of the tile's bit stream (u16 words in
// order, most significant bit first, wrapping) that ends with those bits.
//
// Lane layout used everywhere in this library ("octet layout"): 8 lanes share a
// tile; lane u of the octet owns stream positions 32u .. 32u+31, i.e. `bits`
// consecutive dwords of the tile.  With the upstream tile order (stream position
// 8L+e of MMA lane L is k = 2(L%4) + {0,1,8,9}[e%4], n = L/4 + 8(e/4)) those 32
// positions are exactly the 16 k values of tile columns u and u+8, and stream
// positions 2p, 2p+1 are a (k, k+1) pair.  Pair p = 4q + 2f + h holds
// k = 2q + 8h + {0,1} of column u + 8f.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace berth {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr float kRsqrt128 = 0.088388347648f;  // crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:44

// pair index p (stream positions 2p, 2p+1) -> which column half and k pair
__host__ __device__ constexpr int pair_col_half(int p) { return (p >> 1) & 1; }          // f
__host__ __device__ constexpr int pair_kk(int p) { return (p >> 2) + 4 * (p & 1); }      // k/2 in the tile

// Pointers that reach a kernel through memory (device tables of pointers) lose
// their address space; these casts restore "global" so that loads and stores are
// global_* instructions rather than flat_* ones.
template <typename T>
using global_ptr = __attribute__((address_space(1))) T*;
template <typename T>
__device__ __forceinline__ global_ptr<const T> as_global(const T* p) { return (global_ptr<const T>)p; }
template <typename T>
__device__ __forceinline__ global_ptr<T> as_global(T* p) { return (global_ptr<T>)p; }

// A workgroup that is about to tell another workgroup, through an agent-scope counter, that
// its stores are there: every wave first waits until its own stores have completed.  The
// workgroup-scope release fence does not do that (the waves of a workgroup share their
// caches, so the compiler emits no wait on vector memory for it), and neither does a barrier.
//
// The cross-workgroup handoffs of this library (split-K partial sums, the folded MoE combine,
// the small-batch router) rest on three properties of gfx950 rather than on agent-scope
// fences, whose whole-L2 write-back and invalidate cost more than the kernels they would
// guard: relaxed agent-scope atomic stores and loads bypass the per-die L2 (they are served
// by the memory side, which all dies share), s_waitcnt vmcnt(0) returns only when a wave's
// stores have been acknowledged there, and an agent-scope atomic read-modify-write is ordered
// after it in program order.  The guard below keeps the code from being built for a target
// where that has not been established.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "the split-K handoffs of this library are written for gfx950"
#endif
__device__ __forceinline__ void wait_own_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Touches the first LINES 64-byte lines of the kernel-argument block with one scalar read
// each, all in flight together, so that the argument fields the compiler reads one by one
// further down (behind branches, each with a wait of its own) find their line in the scalar
// cache instead of paying a miss per line in sequence.  The caller's argument block must
// span LINES * 64 bytes (the hidden arguments that follow the explicit ones count).
// Measured on one machine, library against library: the one-row GEMV launches gain 2.5 us
// per 27B linear set (81.9 -> 79.4) and the one-token MoE layer 1.1 us; the MFMA kernels and
// the many-token MoE kernels lost 1-2 % with it (one more wait at the head of workgroups
// that are not latency-bound), so only the VALU GEMV kernel and the one-token router call it.
template <int LINES>
__device__ __forceinline__ void touch_kernel_arguments()
{
    static_assert(LINES == 3 || LINES == 6 || LINES == 10 || LINES == 16, "instantiated line counts");
    const auto ka = __builtin_amdgcn_kernarg_segment_ptr();
    int t0, t1, t2, t3, t4, t5;
    if constexpr (LINES == 16) {
        int t6, t7, t8, t9, t10, t11, t12, t13, t14, t15;
        asm volatile("s_load_dword %0, %16, 0x0\n\ts_load_dword %1, %16, 0x40\n\ts_load_dword %2, %16, 0x80\n\t"
                     "s_load_dword %3, %16, 0xc0\n\ts_load_dword %4, %16, 0x100\n\ts_load_dword %5, %16, 0x140\n\t"
                     "s_load_dword %6, %16, 0x180\n\ts_load_dword %7, %16, 0x1c0\n\ts_load_dword %8, %16, 0x200\n\t"
                     "s_load_dword %9, %16, 0x240\n\ts_load_dword %10, %16, 0x280\n\ts_load_dword %11, %16, 0x2c0\n\t"
                     "s_load_dword %12, %16, 0x300\n\ts_load_dword %13, %16, 0x340\n\ts_load_dword %14, %16, 0x380\n\t"
                     "s_load_dword %15, %16, 0x3c0\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5), "=&s"(t6), "=&s"(t7),
                       "=&s"(t8), "=&s"(t9), "=&s"(t10), "=&s"(t11), "=&s"(t12), "=&s"(t13), "=&s"(t14), "=&s"(t15)
                     : "s"(ka));
    } else
    if constexpr (LINES == 10) {
        int t6, t7, t8, t9;
        asm volatile("s_load_dword %0, %10, 0x0\n\ts_load_dword %1, %10, 0x40\n\ts_load_dword %2, %10, 0x80\n\t"
                     "s_load_dword %3, %10, 0xc0\n\ts_load_dword %4, %10, 0x100\n\ts_load_dword %5, %10, 0x140\n\t"
                     "s_load_dword %6, %10, 0x180\n\ts_load_dword %7, %10, 0x1c0\n\ts_load_dword %8, %10, 0x200\n\t"
                     "s_load_dword %9, %10, 0x240\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5), "=&s"(t6), "=&s"(t7),
                       "=&s"(t8), "=&s"(t9)
                     : "s"(ka));
    } else if constexpr (LINES == 6)
        asm volatile("s_load_dword %0, %6, 0x0\n\ts_load_dword %1, %6, 0x40\n\ts_load_dword %2, %6, 0x80\n\t"
                     "s_load_dword %3, %6, 0xc0\n\ts_load_dword %4, %6, 0x100\n\ts_load_dword %5, %6, 0x140\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5) : "s"(ka));
    else
        asm volatile("s_load_dword %0, %3, 0x0\n\ts_load_dword %1, %3, 0x40\n\ts_load_dword %2, %3, 0x80\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&s"(t0), "=&s"(t1), "=&s"(t2) : "s"(ka));
}

__device__ __forceinline__ half2_t as_half2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }
__device__ __forceinline__ uint32_t as_u32(half2_t v) { return __builtin_bit_cast(uint32_t, v); }

// ---- codebooks (crates/berth-kernels/src/lib.rs:54-63: 0 default/3INST, 1 MCG, 2 MUL1)

// MUL1: x = state * 0x83DCD12D (ptx/sm86_probes.cu:248); t = sum of the four bytes
// of x (:143); weight = fma_f16(1024 + t, 0x1EEE, 0xC931).  v_sad_u8 adds the byte
// sum onto 0x6400 (fp16 1024.0) in the low half, v_sad_hi_u8 does the same for the
// second state in the high half, and one packed fp16 FMA finishes both weights.
__device__ __forceinline__ uint32_t mul1_pair(uint32_t s0, uint32_t s1)
{
    uint32_t x0 = s0 * 0x83DCD12Du;
    uint32_t x1 = s1 * 0x83DCD12Du;
    uint32_t lo = __builtin_amdgcn_sad_u8(x0, 0u, 0x64006400u);
    uint32_t pk = __builtin_amdgcn_sad_hi_u8(x1, 0u, lo);
    const half2_t kinv = as_half2(0x1EEE1EEEu);
    const half2_t kbias = as_half2(0xC931C931u);
    return as_u32(__builtin_elementwise_fma(as_half2(pk), kinv, kbias));
}

// 3INST / MCG: x = state * a (+ c); x = (x & 0x8FFF8FFF) ^ 0x3B603B60
// (ptx/sm86_probes.cu:157); weight = half(lo16) + half(hi16), one fp16 add.
template <int CB>
__device__ __forceinline__ _Float16 inst3_one(uint32_t s)
{
    uint32_t x = (CB == 0) ? s * 89226354u + 64248484u : s * 0xCBAC1FEDu;
    x = (x & 0x8FFF8FFFu) ^ 0x3B603B60u;
    half2_t v = as_half2(x);
    return v.x + v.y;
}

template <int CB>
__device__ __forceinline__ uint32_t decode_pair(uint32_t s0, uint32_t s1)
{
    if constexpr (CB == 2) {
        return mul1_pair(s0, s1);
    } else {
        half2_t r;
        r.x = inst3_one<CB>(s0);
        r.y = inst3_one<CB>(s1);
        return as_u32(r);
    }
}

// ---- window extraction
// `own` are the lane's BITS dwords as loaded (little-endian pairs of u16 words),
// `prev` is the dword just before them in the tile (the last dword of the previous
// lane of the octet, wrapping inside the tile).  Stream order inside a dword is
// low u16 word first, so chunk c in stream order is rot16(dword).
template <int BITS>
struct LaneWindows {
    uint32_t c[BITS + 1];   // big-endian 32-bit chunks: c[0] = prev, c[1..] = own
    uint32_t m[BITS + 1];   // m[j] = low 16 of c[j-1] : high 16 of c[j]  (j >= 1)

    LaneWindows() = default;
    __device__ __forceinline__ LaneWindows(const uint32_t (&own)[BITS], uint32_t prev)
    {
        c[0] = __builtin_amdgcn_alignbit(prev, prev, 16);
        m[0] = 0;
#pragma unroll
        for (int j = 0; j < BITS; ++j) {
            c[j + 1] = __builtin_amdgcn_alignbit(own[j], own[j], 16);
            // low word of the previous dword's stream-last u16, then this dword's first u16
            uint32_t before = (j == 0) ? prev : own[j - 1];
            m[j + 1] = (before & 0xffff0000u) | (own[j] & 0x0000ffffu);
        }
    }

    // state of local stream position i (0..31)
    __device__ __forceinline__ uint32_t state(int i) const
    {
        const int end = 32 + BITS * (i + 1);        // one past the window, local bit index
        const int ce = (end - 1) >> 5;              // chunk holding the window's last bit
        const int sh = 32 * (ce + 1) - end;         // distance of the window from that chunk's lsb
        if (sh <= 16) return __builtin_amdgcn_ubfe(c[ce], sh, 16);
        return __builtin_amdgcn_ubfe(m[ce], sh - 16, 16);
    }
};

// Decode the lane's 32 weights into 16 packed pairs (pair p = positions 2p, 2p+1).
template <int BITS, int CB>
__device__ __forceinline__ void decode_lane(const uint32_t (&own)[BITS], uint32_t prev,
                                            uint32_t (&w2)[16])
{
    LaneWindows<BITS> win(own, prev);
#pragma unroll
    for (int p = 0; p < 16; ++p)
        w2[p] = decode_pair<CB>(win.state(2 * p), win.state(2 * p + 1));
}

// The dword just before a lane's own dwords belongs to the previous lane of its
// octet (octet-local rotate by one: lane u = 0 takes it from lane u = 7).  Two DPP
// moves inside the 16-lane row and a select; no LDS traffic.
__device__ __forceinline__ uint32_t fetch_prev(int lane, uint32_t last_own)
{
    // lanes whose source falls outside the row read 0 (bound_ctrl): those are exactly the lanes
    // that take the other move's result, so neither move needs its destination set up first
    const int v = (int)last_own;
    const int from_below = __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, true);    // row_shr:1, lane i <- i-1
    const int from_above = __builtin_amdgcn_update_dpp(0, v, 0x107, 0xF, 0xF, true);    // row_shl:7, lane i <- i+7
    return (uint32_t)((lane & 7) ? from_below : from_above);
}

}  // namespace berth

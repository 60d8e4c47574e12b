// MoE layer on top of the EXL3 linears: route -> permute -> grouped expert FFNs
// -> weighted combine.  The reference has no MoE implementation (its engine
// rejects such layers, crates/berth-engine/src/model.rs:404-409); what it fixes is
// the shape of the problem — MoeDims / Ffn::Moe{router, shared, experts}
// (crates/berth-plan/src/shape.rs:64-69, plan.rs:24-59), "an expert is three EXL3
// linears" (docs/exl3.md:39) and the expert-selection arguments of its multi-
// linear kernel (crates/berth-kernels/csrc/ops/mgemm.cu:194-228).  The arithmetic
// contract implemented here:
//   logits[t][e] = sum over 64-row segments of (sum_h x[t][h] * wr[h][e], fp32 fma in
//                  row order), segments added in order, then + bias[e];
//   top-k on the logits, largest first, ties to the lowest expert index;
//   weights = exp(logit - max) normalised over the selected k (renorm) or over
//   all experts; pairs (token, slot) stable-sorted by expert;
//   out[t] = shared(x[t]) + sum_j w[t][j] * FFN_{idx[t][j]}(x[t]) in slot order (fp32 fma).
#include "exl3_gemv_kernel.cuh"
#include "launch.h"

#include "../../include/berth_kernels_hip.h"

#include <cstdlib>

namespace berth {

constexpr int kValuPairs = 8;       // calls with one token or at most this many rows use the VALU kernel only
constexpr int kGemmRows = 32;       // rows per small MFMA problem
constexpr int kGemmBigRows = 128;   // rows per big MFMA problem

// ------------------------------------------------------------------ route

__global__ __launch_bounds__(256) void moe_route_kernel(RouteParams p)
{
    __shared__ float xs[kRouteTT][kRouteSeg];
    __shared__ unsigned s_last;
    const int seg = blockIdx.x, grp = blockIdx.y;
    const int t0 = grp * kRouteTT;
    const int h0 = seg * kRouteSeg;
    const int hn = min(kRouteSeg, p.H - h0);
    const int tid = threadIdx.x;

    for (int i = tid; i < kRouteTT * kRouteSeg; i += 256) {
        const int tt = i / kRouteSeg, h = i % kRouteSeg;
        float v = 0.0f;
        if (t0 + tt < p.T && h < hn) v = (float)p.x[(size_t)(t0 + tt) * p.H + h0 + h];
        xs[tt][h] = v;
    }
    __syncthreads();

    for (int e = tid; e < p.E; e += 256) {
        float part[kRouteTT];
#pragma unroll
        for (int tt = 0; tt < kRouteTT; ++tt) part[tt] = 0.0f;
        // the whole segment of router rows in flight at once (rows past the segment
        // re-read its last row and meet the zeros that pad xs); fma chains in row order
        _Float16 wv[kRouteSeg];
#pragma unroll
        for (int i = 0; i < kRouteSeg; ++i) wv[i] = p.wr[(size_t)(h0 + min(i, hn - 1)) * p.E + e];
#pragma unroll
        for (int i = 0; i < kRouteSeg; ++i) {
#pragma unroll
            for (int tt = 0; tt < kRouteTT; ++tt) part[tt] = __builtin_fmaf(xs[tt][i], (float)wv[i], part[tt]);
        }
#pragma unroll
        for (int tt = 0; tt < kRouteTT; ++tt)
            if (t0 + tt < p.T)
                __hip_atomic_store(p.parts + ((size_t)(t0 + tt) * p.nseg + seg) * p.E + e, part[tt],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    wait_own_stores();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (tid == 0) {
        unsigned old = __hip_atomic_fetch_add(p.counters + grp * kRouteCounterStride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (old == (unsigned)(p.nseg - 1)) ? 1u : 0u;
    }
    __syncthreads();
    if (!s_last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (tid == 0) __hip_atomic_store(p.counters + grp * kRouteCounterStride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // ---- last workgroup of the token group: wave tt finishes token t0 + tt
    const int lane = tid & 63, tt = tid >> 6;
    const int t = t0 + tt;
    if (t >= p.T) return;
    constexpr int PER = kRoutePer;
    float lg[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = lane + 64 * i;
        float v = -INFINITY;
        if (e < p.E) {
            v = 0.0f;
            const float* src = p.parts + (size_t)t * p.nseg * p.E + e;
            // 32 loads in flight at a time (indices past the end re-read the last segment
            // and are ignored); the adds stay in segment order
            for (int s0 = 0; s0 < p.nseg; s0 += 32) {
                float part[32];
#pragma unroll
                for (int j = 0; j < 32; ++j)
                    part[j] = __hip_atomic_load(src + (size_t)min(s0 + j, p.nseg - 1) * p.E, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int j = 0; j < 32; ++j) {
                    const float nv = v + part[j];
                    v = s0 + j < p.nseg ? nv : v;
                }
            }
            if (p.bias) v += p.bias[e];
            if (p.logits) p.logits[(size_t)t * p.E + e] = v;
        }
        lg[i] = v;
    }
    const int sel = route_topk(lg, lane, p, t);
    if (p.sort.perm) route_sort_one_token(p.sort, lane, sel);
}

// One token and a small router (at most 128 experts, an even number; at most 4096 rows):
// a single workgroup of sixteen waves streams the whole router weight, so the segment sums
// meet in LDS instead of travelling through memory and a counter.  Wave w takes segments w,
// w + 16, ...; a lane holds two neighbouring experts (one 4-byte load per row) and the
// segment's activations come from the lanes of one coalesced load (v_readlane: the row index
// is the same for the whole wave).  Same arithmetic as moe_route_kernel: fma chains in row
// order per 64-row segment, segments added in order, bias, top-k, sort.
constexpr int kRouteOneMaxSeg = 64;
constexpr int kRouteOneMaxE = 128;

__global__ __launch_bounds__(1024) void moe_route_one_token_kernel(RouteParams p)
{
    static_assert(sizeof(RouteParams) > 2 * 64, "argument lines");
    touch_kernel_arguments<3>();
    __shared__ float part_s[kRouteOneMaxSeg][kRouteOneMaxE];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int pairs = p.E >> 1;                         // lanes with work
    const int col = min(lane, pairs - 1);               // idle lanes repeat the last pair and store nothing
    const global_ptr<const uint32_t> wr = (global_ptr<const uint32_t>)as_global((const uint32_t*)p.wr);

    for (int seg = wave; seg < p.nseg; seg += 16) {
        const int h0 = seg * kRouteSeg;
        const int hn = min(kRouteSeg, p.H - h0);
        // one activation per lane (zero past the end of the input), broadcast row by row with
        // v_readlane; rows past the end of a partial segment re-read its last row and meet zeros
        const float xv = lane < hn ? (float)p.x[h0 + lane] : 0.0f;
        uint32_t wv[kRouteSeg];
#pragma unroll
        for (int i = 0; i < kRouteSeg; ++i) wv[i] = wr[(size_t)(h0 + min(i, hn - 1)) * pairs + col];
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int i = 0; i < kRouteSeg; ++i) {
            const float xi = lane_value(xv, i);
            const half2_t w2 = as_half2(wv[i]);
            a0 = __builtin_fmaf(xi, (float)w2.x, a0);
            a1 = __builtin_fmaf(xi, (float)w2.y, a1);
        }
        if (lane < pairs) {
            part_s[seg][2 * lane] = a0;
            part_s[seg][2 * lane + 1] = a1;
        }
    }
    __syncthreads();
    if (wave != 0) return;

    constexpr int PER = kRoutePer;
    float lg[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = lane + 64 * i;
        float v = -INFINITY;
        if (i < kRouteOneMaxE / 64 && e < p.E) {
            v = 0.0f;
            for (int sg = 0; sg < p.nseg; ++sg) v += part_s[sg][e];
            if (p.bias) v += p.bias[e];
            if (p.logits) p.logits[e] = v;
        }
        lg[i] = v;
    }
    const int sel = route_topk(lg, lane, p, 0);
    if (p.sort.perm) route_sort_one_token(p.sort, lane, sel);
}

// One token and a small router, first part only: workgroup `seg` (one wave) leaves the sums
// of its 64 rows in parts[seg][e].  The routing's last part (ordered sum of the segments,
// top-k, sort) is then redone by every workgroup of the gate / up launch for itself
// (route_finish_one_token), which costs less than one workgroup doing it once and all the
// others waiting for its launch to end.  Same fma chains as moe_route_one_token_kernel.
__global__ __launch_bounds__(64) void moe_route_segments_kernel(RouteParams p)
{
    const int lane = threadIdx.x;
    const int seg = blockIdx.x;
    const int pairs = p.E >> 1;
    const int col = min(lane, pairs - 1);
    const global_ptr<const uint32_t> wr = (global_ptr<const uint32_t>)as_global((const uint32_t*)p.wr);
    const int h0 = seg * kRouteSeg;
    const int hn = min(kRouteSeg, p.H - h0);
    const float xv = lane < hn ? (float)p.x[h0 + lane] : 0.0f;
    uint32_t wv[kRouteSeg];
#pragma unroll
    for (int i = 0; i < kRouteSeg; ++i) wv[i] = wr[(size_t)(h0 + min(i, hn - 1)) * pairs + col];
    float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
    for (int i = 0; i < kRouteSeg; ++i) {
        const float xi = lane_value(xv, i);
        const half2_t w2 = as_half2(wv[i]);
        a0 = __builtin_fmaf(xi, (float)w2.x, a0);
        a1 = __builtin_fmaf(xi, (float)w2.y, a1);
    }
    if (lane < pairs) {
        float2_t o = {a0, a1};
        *(float2_t*)(p.parts + (size_t)seg * p.E + 2 * lane) = o;
    }
}

// Many tokens: the same arithmetic in two launches, so that the segment sums of a
// token are added by a workgroup of its own instead of the last workgroup of a
// token group.  First launch: partial sums of a few tokens x one 64-row
// segment; second launch: one workgroup per token adds the segments in order,
// adds the bias and selects.
constexpr int kRouteBigGroup = 16;  // most tokens a first-launch workgroup takes
constexpr int kRouteBigT = 32;      // calls with at least this many tokens take the two-launch path

// How the 256 threads of a first-launch workgroup are used: `lanes` threads cover the expert
// pairs (64, 128 or 256: a router of up to 128 experts needs one wave), and 256 / lanes token
// subgroups sit side by side, so a small router does not leave three waves of four idle.  A
// thread takes four tokens, or eight when all 256 threads are on expert pairs (a wide router:
// fewer workgroups re-read its rows).  More than 512 experts: a thread walks pairs tid,
// tid + 256, ...
inline __host__ __device__ int route_big_lanes(int E)
{
    const int pairs = (E + 1) >> 1;
    return pairs <= 64 ? 64 : (pairs <= 128 ? 128 : 256);
}
inline __host__ __device__ int route_big_tokens(int E) { return route_big_lanes(E) == 256 ? 8 : 4; }
inline __host__ __device__ int route_big_group(int E) { return route_big_tokens(E) * (256 / route_big_lanes(E)); }

// partial sums of TT tokens x two neighbouring experts over one segment.
// EVEN: the expert count is even, so the pair is one aligned 4-byte load per row.
// Eight rows of the router weight are loaded back to back (no branch in between:
// the loads are what the loop waits for); the fma chains stay in row order.
// xs: this thread's tokens, [row][TT] with row stride `xs_stride` floats.
template <bool EVEN, int TT>
__device__ __forceinline__ void route_pair_segment(const RouteParams& p, const float* xs, int xs_stride, int e0,
                                                   int h0, int hn, float (&part)[2][TT])
{
    const bool two = e0 + 1 < p.E;
    const _Float16* wcol = p.wr + (size_t)h0 * p.E + e0;
    const int second = two ? 1 : 0;                     // odd counts: the last expert has no neighbour
    // the weights of the next eight rows are loaded before the fma chains of the
    // current eight start (rows past the segment re-read its last row)
    auto load8 = [&](int hb, half2_t (&wv)[8], float (&s0)[8], float (&s1)[8]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int h = hb + i < hn ? hb + i : hn - 1;
            if (EVEN) {
                wv[i] = *(const half2_t*)(wcol + (size_t)h * p.E);
            } else {
                s0[i] = (float)wcol[(size_t)h * p.E];
                s1[i] = (float)wcol[(size_t)h * p.E + second];
            }
        }
    };
    half2_t wn[8];
    float sn0[8], sn1[8];
    load8(0, wn, sn0, sn1);
    for (int hb = 0; hb < hn; hb += 8) {
        float w0[8], w1[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            w0[i] = EVEN ? (float)wn[i].x : sn0[i];
            w1[i] = EVEN ? (float)wn[i].y : sn1[i];
        }
        load8(hb + 8 < hn ? hb + 8 : hb, wn, sn0, sn1);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            // rows past the segment hold zeros in xs: they add +-0 to the partial sum, and
            // the sign of a zero partial sum never reaches a logit (0 + partial comes first)
            const float4_t* xrow = (const float4_t*)(xs + (size_t)(hb + i) * xs_stride);
#pragma unroll
            for (int q = 0; q < TT / 4; ++q) {
                const float4_t xv = xrow[q];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    part[0][4 * q + j] = __builtin_fmaf(xv[j], w0[i], part[0][4 * q + j]);
                    part[1][4 * q + j] = __builtin_fmaf(xv[j], w1[i], part[1][4 * q + j]);
                }
            }
        }
    }
}

template <int TT>
__global__ __launch_bounds__(256) void moe_route_partial_kernel(RouteParams p)
{
    __shared__ __align__(16) float xs[kRouteSeg][kRouteBigGroup];   // [row][token]: one b128 read per 4 tokens
    const int lanes = route_big_lanes(p.E);
    const int group = TT * (256 / lanes);                           // tokens of this workgroup
    const int seg = blockIdx.x, grp = blockIdx.y;
    const int t0 = grp * group;
    const int h0 = seg * kRouteSeg;
    const int hn = min(kRouteSeg, p.H - h0);
    const int tid = threadIdx.x;
    for (int i = tid; i < group * kRouteSeg; i += 256) {
        const int tt = i / kRouteSeg, h = i % kRouteSeg;
        float v = 0.0f;
        if (t0 + tt < p.T && h < hn) v = (float)p.x[(size_t)(t0 + tt) * p.H + h0 + h];
        xs[h][tt] = v;
    }
    __syncthreads();
    const bool even = (p.E & 1) == 0;
    const int sub = tid / lanes;                                    // token subgroup of this thread
    const int ts = t0 + sub * TT;
    for (int e0 = 2 * (tid % lanes); e0 < p.E; e0 += 2 * lanes) {
        float part[2][TT];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) part[0][tt] = part[1][tt] = 0.0f;
        if (even) route_pair_segment<true, TT>(p, &xs[0][sub * TT], kRouteBigGroup, e0, h0, hn, part);
        else route_pair_segment<false, TT>(p, &xs[0][sub * TT], kRouteBigGroup, e0, h0, hn, part);
        const bool two = e0 + 1 < p.E;
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            if (ts + tt < p.T) {
                float* dst = p.parts + ((size_t)(ts + tt) * p.nseg + seg) * p.E + e0;
                dst[0] = part[0][tt];
                if (two) dst[1] = part[1][tt];
            }
        }
    }
}

__global__ __launch_bounds__(256) void moe_route_finish_kernel(RouteParams p)
{
    __shared__ float s_logit[kMaxExperts];
    const int t = blockIdx.x, tid = threadIdx.x;
    // two experts per pass, 32 segment loads of each in flight together (indices past
    // the end re-read the last segment / the last expert and are ignored)
    for (int e = tid; e < p.E; e += 512) {
        const int e2 = e + 256 < p.E ? e + 256 : e;
        const float* src0 = p.parts + (size_t)t * p.nseg * p.E + e;
        const float* src1 = p.parts + (size_t)t * p.nseg * p.E + e2;
        float v0 = 0.0f, v1 = 0.0f;
        for (int s0 = 0; s0 < p.nseg; s0 += 32) {
            float part0[32], part1[32];
#pragma unroll
            for (int j = 0; j < 32; ++j) {
                const size_t at = (size_t)min(s0 + j, p.nseg - 1) * p.E;
                part0[j] = src0[at];
                part1[j] = src1[at];
            }
#pragma unroll
            for (int j = 0; j < 32; ++j) {
                const float n0 = v0 + part0[j], n1 = v1 + part1[j];
                v0 = s0 + j < p.nseg ? n0 : v0;
                v1 = s0 + j < p.nseg ? n1 : v1;
            }
        }
        if (p.bias) { v0 += p.bias[e]; v1 += p.bias[e2]; }
        if (p.logits) {
            p.logits[(size_t)t * p.E + e] = v0;
            if (e2 != e) p.logits[(size_t)t * p.E + e2] = v1;
        }
        s_logit[e] = v0;
        if (e2 != e) s_logit[e2] = v1;
    }
    __syncthreads();
    if (tid >= 64) return;
    float lg[kRoutePer];
#pragma unroll
    for (int i = 0; i < kRoutePer; ++i) {
        const int e = tid + 64 * i;
        lg[i] = e < p.E ? s_logit[e] : -INFINITY;
    }
    route_topk(lg, tid, p, t);
}

// Many tokens, an even number of experts: the whole routing of TT tokens x a slab of 128 experts
// in one workgroup of sixteen waves, so that the segment sums never travel through memory (two
// launches of the form above write and read 4 * nseg bytes per (token, expert): 16.8 MB each way
// for 256 tokens x 512 experts).  Wave w takes segments w, w + 16, ...; a lane holds two
// neighbouring experts (one 4-byte load per router row) and TT tokens, whose activations are
// wave-uniform and come through the scalar cache.  The segment sums meet in LDS
// ([segment][token][expert]); after the barrier thread (token, expert) adds them in segment order
// and adds the bias.  With one slab the workgroup selects right away (wave tt: token tt); with
// several the logits go to memory and the last slab of a token group to arrive selects.  Same
// arithmetic as every other routing kernel here: fma chains in row order per 64-row segment,
// segments added in order.
constexpr int kSlabExperts = 128;
// LDS of a workgroup: segment sums [nseg][tt][128] fp32, then the tokens' rows [tt][H] as fp32 (H = 64 nseg)
inline __host__ __device__ int route_slab_lds_bytes(int nseg, int tt) { return nseg * tt * kSlabExperts * 4 + tt * nseg * kRouteSeg * 4; }

template <int TT>
__global__ __launch_bounds__(1024) void moe_route_slab_kernel(RouteParams p)
{
    extern __shared__ __align__(16) float s_parts[];               // [nseg][TT][128]
    __shared__ unsigned s_last;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);     // uniform: the token loads stay scalar
    // token group fastest: consecutive workgroups go to different dies, so every die works on all
    // slabs (one slab's rows alone fall on a quarter of an L2's channels)
    const int grp = blockIdx.x, slab = blockIdx.y, nslab = gridDim.y;
    const int t0 = grp * TT;
    const int e0 = slab * kSlabExperts + 2 * lane;
    const int e_ld = e0 < p.E ? e0 : p.E - 2;                       // lanes past the end redo the last pair, unused
    const global_ptr<const half2_t> wcol = (global_ptr<const half2_t>)as_global(p.wr + e_ld);
    const size_t wstride = (size_t)p.E / 2;                         // half2 elements per router row
    // thread (token, expert of the slab) of the ordered sum further down; its bias is asked for now
    const int tt_mine = threadIdx.x >> 7, c = threadIdx.x & 127;
    const int e_mine = slab * kSlabExperts + c, t_mine = t0 + tt_mine;
    const bool mine = tt_mine < TT && e_mine < p.E;
    const float bias_mine = mine && p.bias ? p.bias[e_mine] : 0.0f;
    // the tokens' rows go to LDS once, widened to fp32 (tokens past the end: the last token,
    // unused); a step then reads its sixteen rows of every token with wave-uniform addresses
    // (broadcast reads).
    float* const s_x = s_parts + (size_t)p.nseg * TT * kSlabExperts;
    {
        const int per_row = p.H / 2;                                        // dwords
        for (int i = threadIdx.x; i < TT * per_row; i += 1024) {
            const int tt = i / per_row, d = i - tt * per_row;
            const uint32_t v = ((global_ptr<const uint32_t>)as_global((const uint32_t*)(p.x + (size_t)min(t0 + tt, p.T - 1) * p.H)))[d];
            const half2_t h = __builtin_bit_cast(half2_t, v);
            *(float2_t*)&s_x[2 * i] = float2_t{(float)h.x, (float)h.y};
        }
    }
    __syncthreads();

    // The wave's segments as one run of steps of kStep rows (H is a multiple of 64 here),
    // software-pipelined: the router rows of the next step are requested before the fma chains
    // of the current one start, across segment boundaries.  With few tokens a step holds few
    // fmas, so it takes more rows: the loop is then paced by the loads in flight.
    constexpr int kStep = TT >= 4 ? 16 : 32;
    constexpr int kPerSeg = kRouteSeg / kStep;
    const int nsteps = wave < p.nseg ? kPerSeg * ((p.nseg - wave + 15) / 16) : 0;
    auto load_rows = [&](int step, half2_t (&dst)[kStep]) {
        const int sc = step < nsteps ? step : nsteps - 1;                  // past the end: reread, unused
        const int row0 = (wave + 16 * (sc / kPerSeg)) * kRouteSeg + (sc % kPerSeg) * kStep;
        const global_ptr<const half2_t> src = wcol + (size_t)row0 * wstride;
#pragma unroll
        for (int i = 0; i < kStep; ++i) dst[i] = src[(size_t)i * wstride];
    };
    float part[TT][2];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) part[tt][0] = part[tt][1] = 0.0f;
    auto run_step = [&](int step, const half2_t (&wv)[kStep]) {
        const int seg = wave + 16 * (step / kPerSeg);
        const int row0 = seg * kRouteSeg + (step % kPerSeg) * kStep;
#pragma unroll
        for (int q = 0; q < kStep / 4; ++q) {                               // four rows at a time
            float4_t xd[TT];
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) xd[tt] = *(const float4_t*)(s_x + (size_t)tt * p.H + row0 + 4 * q);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float w0 = (float)wv[4 * q + r].x, w1 = (float)wv[4 * q + r].y;
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) {
                    part[tt][0] = __builtin_fmaf(xd[tt][r], w0, part[tt][0]);
                    part[tt][1] = __builtin_fmaf(xd[tt][r], w1, part[tt][1]);
                }
            }
        }
        if (step % kPerSeg == kPerSeg - 1) {                                // the segment is complete
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
                *(float2_t*)&s_parts[((size_t)seg * TT + tt) * kSlabExperts + 2 * lane] = float2_t{part[tt][0], part[tt][1]};
                part[tt][0] = part[tt][1] = 0.0f;
            }
        }
    };
    if (nsteps > 0) {
        half2_t wa[kStep], wb[kStep];
        load_rows(0, wa);
#pragma unroll 1
        for (int step = 0; step < nsteps; step += 2) {
            load_rows(step + 1, wb);
            run_step(step, wa);
            load_rows(step + 2, wa);
            run_step(step + 1, wb);
        }
    }
    __syncthreads();

    // ---- thread (token, expert of the slab): segments added in order, bias
    float v = 0.0f;
    if (mine) {
        for (int seg = 0; seg < p.nseg; ++seg) v += s_parts[((size_t)seg * TT + tt_mine) * kSlabExperts + c];
        if (p.bias) v += bias_mine;
        if (p.logits && t_mine < p.T) p.logits[(size_t)t_mine * p.E + e_mine] = v;
    }
    float lg[kRoutePer];
#pragma unroll
    for (int i = 0; i < kRoutePer; ++i) lg[i] = -INFINITY;
    if (nslab == 1) {
        __syncthreads();                                            // every sum is formed: the segment sums can go
        if (mine) s_parts[tt_mine * kSlabExperts + c] = v;
        __syncthreads();
        if (wave >= TT || t0 + wave >= p.T) return;
#pragma unroll
        for (int i = 0; i < 2; ++i)
            if (lane + 64 * i < p.E) lg[i] = s_parts[wave * kSlabExperts + lane + 64 * i];
        route_topk_n<2>(lg, lane, p, t0 + wave);
        return;
    }
    // ---- several slabs: logits to memory ([T][E], the head of the segment-sum scratch), the last
    // slab of the token group to arrive selects
    float* const all = p.parts;
    if (mine && t_mine < p.T)
        __hip_atomic_store(all + (size_t)t_mine * p.E + e_mine, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    wait_own_stores();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned* counter = p.counters + (size_t)grp * kRouteCounterStride;
        const unsigned old = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (old == (unsigned)(nslab - 1)) ? 1u : 0u;
        if (s_last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (wave >= TT || t0 + wave >= p.T) return;
    const int t = t0 + wave;
#pragma unroll
    for (int i = 0; i < kRoutePer; ++i) {
        const int e = lane + 64 * i;
        if (e < p.E) lg[i] = __hip_atomic_load(all + (size_t)t * p.E + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    route_topk(lg, lane, p, t);
}

// ---------------------------------------------------------------- permute


// One workgroup.  Counting sort by expert, stable in pair order: the pairs of one
// expert come from distinct tokens, so the rank of pair (t, slot) inside its expert
// is the number of earlier tokens that chose the expert.  Tokens are taken 64 at a
// time: a 64-bit mask per expert records which of them chose it, and the rank is a
// population count below the token's bit.  Nothing depends on scheduling.
__global__ __launch_bounds__(1024) void moe_permute_kernel(PermuteParams p)
{
    __shared__ int tot[kMaxExperts + 1];                    // rows per expert
    __shared__ int off[kMaxExperts + 2];                    // first sorted row of each expert
    __shared__ int pfirst[kMaxExperts + 2];                 // first (small or VALU) problem of each expert
    __shared__ int bfirst[kMaxExperts + 2];                 // first big problem of each expert
    __shared__ int done[kMaxExperts + 1];                   // rows of the expert placed so far
    __shared__ unsigned long long mask[kMaxExperts + 1];
    __shared__ unsigned long long wave_sum[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int P = p.T * p.k;
    const int E1 = p.E + (p.shared_rows ? 1 : 0);           // experts including the always-on one

    for (int e = tid; e <= p.E; e += 1024) { tot[e] = 0; done[e] = 0; mask[e] = 0; }
    __syncthreads();
    for (int q = tid; q < P; q += 1024) atomicAdd(&tot[p.idx[q]], 1);
    if (p.shared_rows && tid == 0) tot[p.E] = p.T;
    __syncthreads();

    // exclusive scan over the experts of (rows, small problems, big problems), packed
    // in one 64-bit add: 22 + 21 + 21 bits
    {
        const int c = tid < E1 ? tot[tid] : 0;
        int nbig = 0, nsmall = 0;
        if (c > 0) {
            if (p.use_valu) nsmall = 1;
            else {
                nbig = p.big_min <= kGemmBigRows ? c / kGemmBigRows : 0;
                int rem = c - nbig * kGemmBigRows;
                if (rem >= p.big_min) { ++nbig; rem = 0; }
                nsmall = (rem + kGemmRows - 1) / kGemmRows;
            }
        }
        const unsigned long long mine = ((unsigned long long)nbig << 43) | ((unsigned long long)nsmall << 22) | (unsigned)c;
        unsigned long long v = mine;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const unsigned long long o = __shfl_up(v, d, 64);
            if (lane >= d) v += o;
        }
        if (lane == 63) wave_sum[wave] = v;
        __syncthreads();
        unsigned long long before = 0;
        for (int w = 0; w < wave; ++w) before += wave_sum[w];
        const unsigned long long excl = before + v - mine;
        if (tid < E1) {
            off[tid] = (int)(excl & 0x3fffffu);
            pfirst[tid] = (int)((excl >> 22) & 0x1fffffu);
            bfirst[tid] = (int)(excl >> 43);
        }
        if (tid == E1 - 1) {
            const unsigned long long all = excl + mine;
            off[E1] = (int)(all & 0x3fffffu);
            const int total_small = (int)((all >> 22) & 0x1fffffu);
            p.counts[0] = p.use_valu ? total_small : 0;
            p.counts[1] = p.use_valu ? 0 : total_small;
            p.counts[2] = (int)(all >> 43);
        }
    }
    __syncthreads();
    for (int x = tid; x <= p.E; x += 1024) p.offsets[x] = off[x];
    if (tid < E1) {
        const int m = tot[tid];
        if (m > 0) {
            if (p.use_valu) {
                p.vprob[pfirst[tid]] = GroupProblem{tid, off[tid], m, 0};
            } else {
                int r = 0;
                for (int j = bfirst[tid]; m - r >= p.big_min; r += kGemmBigRows, ++j)
                    p.bprob[j] = GroupProblem{tid, off[tid] + r, min(kGemmBigRows, m - r), 0};
                for (int j = pfirst[tid]; r < m; r += kGemmRows, ++j)
                    p.mprob[j] = GroupProblem{tid, off[tid] + r, min(kGemmRows, m - r), 0};
            }
        }
    }

    for (int t0 = 0; t0 < p.T; t0 += 64) {
        const int nq = min(64, p.T - t0) * p.k;
        const int q0 = t0 * p.k;
        for (int i = tid; i < nq; i += 1024) atomicOr(&mask[p.idx[q0 + i]], 1ull << (i / p.k));
        __syncthreads();
        for (int i = tid; i < nq; i += 1024) {
            const int q = q0 + i, e = p.idx[q];
            const int at = off[e] + done[e] + __popcll(mask[e] & ((1ull << (i / p.k)) - 1ull));
            p.perm[at] = q;
            p.inv[q] = at;
            p.row_expert[at] = e;
        }
        __syncthreads();
        for (int e = tid; e < p.E; e += 1024) {
            done[e] += __popcll(mask[e]);
            mask[e] = 0;
        }
        __syncthreads();
    }
    if (p.shared_rows) {
        for (int t = tid; t < p.T; t += 1024) {
            p.perm[P + t] = t * p.k;
            p.row_expert[P + t] = p.E;
        }
    }
}

// ------------------------------------- rotated inputs for the MFMA problems

struct HadRowsParams {
    const _Float16* a;          // input rows
    const _Float16* a_up;       // with a_up: input = silu(a[r]) * a_up[r]
    const int32_t* gather;      // source row = gather[r] / gather_div, or r
    int gather_div;
    const int32_t* row_expert;
    const ExpertLin* experts;
    ExpertLin shared[3];        // the always-on expert (row_expert == shared_expert)
    int shared_expert;
    int lins_per_expert, lin_base;
    int num_lins;               // 1 or 2: the same input rotated under the scales of linear lin_base (+ 1)
    _Float16* out[2];           // per linear
    int P, K;
};

// An item is one 128 block of one row under one linear's scales; sixteen lanes (one DPP row)
// rotate it, eight consecutive elements per lane (16-byte accesses).  blockIdx.x walks the
// (row, block) items, sixteen per workgroup, so that a narrow K does not leave waves idle;
// blockIdx.y is the linear.  Measured on 2816 rows (K 2048 under two linears / K 512 under one):
// 14.4 / 5.0 us; with both linears in one thread 14.4 / 5.9 us, with two or four items per lane
// group on top of that 13.7 / 6.4 and 15.9 / 7.9 us.  The K 2048 pair writes 23 MB.
__global__ __launch_bounds__(256) void moe_had_rows_kernel(HadRowsParams p)
{
    const int lane = threadIdx.x & 63;
    const int l16 = lane & 15;
    const int which = blockIdx.y;
    const int nkb = p.K >> 7;
    const int total = p.P * nkb;
    const int first = blockIdx.x * 16 + (threadIdx.x >> 4);
    const bool live = first < total;
    const int item = live ? first : total - 1;              // groups past the end redo the last item, store nothing
    const int row = item / nkb;
    const int at = (item - row * nkb) * 128 + 8 * l16;
    const int ex = p.row_expert[row];
    const int src = p.gather ? p.gather[row] / p.gather_div : row;
    const _Float16* scale = ex == p.shared_expert ? p.shared[p.lin_base + which].suh
                                                  : p.experts[(size_t)ex * p.lins_per_expert + p.lin_base + which].suh;
    half8_t x = *(const half8_t*)(p.a + (size_t)src * p.K + at);
    const half8_t sc = *(const half8_t*)(scale + at);
    if (p.a_up) {
        const half8_t u = *(const half8_t*)(p.a_up + (size_t)src * p.K + at);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = silu_mul_h(x[i], u[i]);
    }
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)x[i] * (float)sc[i];
    had128_row16(v, lane);
    half8_t o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (_Float16)(v[i] * kRsqrt128);
    if (live) *(half8_t*)(p.out[which] + (size_t)row * p.K + at) = o;
}

inline void launch_had_rows(const HadRowsParams& h, hipStream_t stream)
{
    const long items = (long)h.P * (h.K >> 7);
    hipLaunchKernelGGL(moe_had_rows_kernel, dim3((unsigned)((items + 15) / 16), h.num_lins), dim3(256), 0, stream, h);
    hip_ok(hipGetLastError(), "moe_had_rows_kernel launch");
}

// ------------------------------------------------- shared expert's gate

// scale[t] = sigmoid(z), z = x[t] . wg with the routing's arithmetic: an fp32 fma chain in row
// order over every 64-row segment, the segment sums added in segment order (the per-token scale
// on the always-on expert's row that Qwen-MoE checkpoints carry as shared_expert_gate.weight;
// the reference has no MoE arithmetic).  One wave per token, lane l takes segments l, l + 64, ...
__global__ __launch_bounds__(64) void moe_shared_gate_kernel(const _Float16* __restrict__ x, const float* __restrict__ wg,
                                                             float* __restrict__ scale, int H)
{
    const int t = blockIdx.x, lane = threadIdx.x;
    const int nseg = (H + kRouteSeg - 1) / kRouteSeg;
    float z = 0.0f;
    for (int s0 = 0; s0 < nseg; s0 += 64) {
        const int seg = s0 + lane;
        float part = 0.0f;
        if (seg < nseg) {
            const int h0 = seg * kRouteSeg, hn = min(kRouteSeg, H - h0);
            for (int i = 0; i < hn; ++i) part = __builtin_fmaf((float)x[(size_t)t * H + h0 + i], wg[h0 + i], part);
        }
        const int n = min(64, nseg - s0);
        for (int j = 0; j < n; ++j) z += lane_value(part, j);       // segment order; the same sum in every lane
    }
    if (lane == 0) scale[t] = 1.0f / (1.0f + expf(-z));
}

// ---------------------------------------------------------------- combine

// out[t][h] = shared_out[t][h] (times shared_scale[t] when given) + sum_j w[t][j] *
// slot_out[inv[t * k + j]][h], fma in slot order.  VEC consecutive columns per thread; the positions, weights and rows of eight slots are
// requested together, the chain of fmas stays in slot order.
template <int VEC>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ slot_out,
                                                          const float* __restrict__ shared_out,
                                                          const float* __restrict__ shared_scale,
                                                          const float* __restrict__ w,
                                                          const int32_t* __restrict__ inv,
                                                          float* __restrict__ out, int T, int H, int k)
{
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    const int per_row = H / VEC;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)T * per_row) return;
    const int t = (int)(i / per_row), h = (int)(i % per_row) * VEC;
    vec_t acc;
    if (shared_out) {
        acc = *(const vec_t*)(shared_out + (size_t)t * H + h);
        if (shared_scale) {
            const float sc = shared_scale[t];
#pragma unroll
            for (int c = 0; c < VEC; ++c) acc[c] *= sc;
        }
    } else {
        acc = vec_t(0.0f);
    }
    for (int j0 = 0; j0 < k; j0 += 8) {
        int pos[8];
        float wj[8];
        vec_t v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int jj = j0 + j < k ? j0 + j : k - 1;
            pos[j] = inv[t * k + jj];
            wj[j] = w[t * k + jj];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = *(const vec_t*)(slot_out + (size_t)pos[j] * H + h);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (j0 + j < k) {
#pragma unroll
                for (int c = 0; c < VEC; ++c) acc[c] = __builtin_fmaf(wj[j], v[j][c], acc[c]);
            }
        }
    }
    *(vec_t*)(out + (size_t)t * H + h) = acc;
}

inline void launch_combine(const float* slot_out, const float* shared_out, const float* shared_scale, const float* w,
                           const int32_t* inv, float* out, int T, int H, int k, hipStream_t stream)
{
    const bool vec4 = H % 4 == 0 && ((uintptr_t)slot_out | (uintptr_t)shared_out | (uintptr_t)out) % 16 == 0;
    const size_t threads = (size_t)T * (vec4 ? H / 4 : H);
    const dim3 grid((unsigned)((threads + 255) / 256));
    if (vec4)
        hipLaunchKernelGGL(moe_combine_kernel<4>, grid, dim3(256), 0, stream, slot_out, shared_out, shared_scale, w, inv, out,
                           T, H, k);
    else
        hipLaunchKernelGGL(moe_combine_kernel<1>, grid, dim3(256), 0, stream, slot_out, shared_out, shared_scale, w, inv, out,
                           T, H, k);
    hip_ok(hipGetLastError(), "moe_combine_kernel launch");
}

// ------------------------------------------------------------ host side

namespace {

thread_local std::string g_moe_err, g_moe_launch;

size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

// byte offsets inside the scratch of berth_moe_permute: the sorted rows' experts, the three
// problem counts, one-row (VALU) problems and 32-row (MFMA) problems
struct PermuteScratch {
    size_t row_expert, counts, vprob, mprob, bprob, total;
    int max_m, max_b, big_min;
};

// An expert's rows beyond 32 go to MFMA problems of up to 128 rows (the weights are decoded
// once per problem, so once per 128 rows instead of once per 32); a remainder of fewer than
// `big_min` rows stays a 32-row problem.  BERTH_MOE_BIG_MIN: 0 keeps 32-row problems only.
// Calls with few rows keep them too: there the launch splits K over several workgroups,
// which the mixed launch does not.
constexpr int kBigMinRows = 256;
int moe_big_min(size_t rows)
{
    const int v = knobs().moe_big_min;
    return v > 0 && v <= kGemmBigRows && rows >= (size_t)kBigMinRows ? v : 0;
}
// capacities of the two problem lists of `rows` rows over `experts` experts
void problem_capacity(size_t rows, size_t experts, int big_min, int& max_m, int& max_b)
{
    if (big_min > 0) {
        max_m = (int)std::min<size_t>(((size_t)(big_min + kGemmRows - 2) / kGemmRows) * experts, rows);
        max_b = (int)(rows / big_min);
    } else {
        max_m = (int)(std::min<size_t>(experts, rows) + rows / kGemmRows + 1);
        max_b = 0;
    }
}

PermuteScratch permute_scratch_layout(int T, int k, int E)
{
    const size_t P = (size_t)T * k, small = std::min<size_t>((size_t)E, P);
    PermuteScratch s{};
    size_t at = 0;
    s.row_expert = at; at = align_up(at + P * 4);
    s.counts = at; at = align_up(at + 16);
    s.vprob = at; at = align_up(at + small * sizeof(GroupProblem));
    s.mprob = at;
    s.big_min = moe_big_min(P);
    problem_capacity(P, (size_t)E, s.big_min, s.max_m, s.max_b);
    at = align_up(at + (size_t)std::max(s.max_m, 1) * sizeof(GroupProblem));
    s.bprob = at;
    s.total = align_up(at + (size_t)std::max(s.max_b, 1) * sizeof(GroupProblem));
    return s;
}

struct MoeLayout {
    size_t idx, w, parts, offsets, perm, inv, row_expert, counts, vprob, mprob, bprob;
    size_t ah0, ah1, g, u, ahd, slot_out, sg, su, s_ahad, shared_out, vlin, gate_scale, total;
    int max_v, max_m, max_b, big_min, nseg;
};

// One token: the down projection's last arrival per column block also combines the block.
// BERTH_MOE_FOLD_COMBINE: 0 keeps the separate combine launch, 1 the two-stage form (split-K
// hand-over per expert, then a second counter per column block); otherwise, with at most
// sixteen problems, the single hand-over (one counter per column block for both).
int fold_combine_mode() { return knobs().moe_fold_combine; }

// One token with a small router: the routing's last part runs inside the gate / up launch
// (BERTH_MOE_INLINE_ROUTE=0 keeps the single-workgroup routing kernel).
bool inline_route_enabled() { return knobs().moe_inline_route != 0; }

// The always-on expert runs as one more expert of the grouped launches (rows P ..
// P + T - 1, token order) when it has the routed experts' intermediate size.
// One token with the inline routing: the gate / up launch leaves the down projection's
// {trellis, suh, svh} records in sorted order, and the down launch reads those instead of the
// problem list and the expert table (BERTH_MOE_RESOLVED=0: off).
bool resolved_records_enabled() { return knobs().moe_resolved != 0; }

bool shared_is_folded(int I, int shared_I) { return shared_I > 0 && shared_I == I; }

MoeLayout moe_layout(int T, int H, int E, int k, int I, int shared_I)
{
    MoeLayout L{};
    const size_t P = (size_t)T * k;
    const bool fold = shared_is_folded(I, shared_I);
    const size_t R = P + (fold ? (size_t)T : 0);        // rows of the grouped launches
    L.nseg = (H + kRouteSeg - 1) / kRouteSeg;
    const bool use_valu = T == 1 || R <= (size_t)kValuPairs;      // one row per problem, or very few rows
    L.max_v = use_valu ? (int)(std::min<size_t>((size_t)E, P) + (fold ? 1 : 0)) : 0;
    const size_t E1 = (size_t)E + (fold ? 1 : 0);
    L.big_min = use_valu ? 0 : moe_big_min(R);
    if (!use_valu) problem_capacity(R, E1, L.big_min, L.max_m, L.max_b);
    size_t at = 0;
    auto take = [&](size_t bytes) { size_t r = at; at = align_up(at + bytes); return r; };
    L.idx = take(P * 4);
    L.w = take(P * 4);
    L.parts = take((size_t)T * L.nseg * E * 4);
    L.offsets = take((size_t)(E + 1) * 4);
    L.perm = take(R * 4);
    L.inv = take(P * 4);
    L.row_expert = take(R * 4);
    L.counts = take(16);
    L.vprob = take((size_t)std::max(L.max_v, 1) * sizeof(GroupProblem));
    L.mprob = take((size_t)std::max(L.max_m, 1) * sizeof(GroupProblem));
    L.bprob = take((size_t)std::max(L.max_b, 1) * sizeof(GroupProblem));
    L.ah0 = take(L.max_m ? R * H * 2 : 0);
    L.ah1 = take(L.max_m ? R * H * 2 : 0);
    L.g = take(R * I * 2);
    L.u = take(R * I * 2);
    L.ahd = take(L.max_m ? R * I * 2 : 0);
    L.slot_out = take(R * H * 4);
    if (fold) {
        L.sg = L.su = L.s_ahad = at;
        L.shared_out = L.slot_out + P * H * 4;
    } else {
        L.sg = take((size_t)T * shared_I * 2);
        L.su = take((size_t)T * shared_I * 2);
        L.s_ahad = take((size_t)T * std::max(H, shared_I) * 2);
        L.shared_out = take(shared_I ? (size_t)T * H * 4 : 0);
    }
    L.vlin = take((size_t)std::max(L.max_v, 1) * sizeof(ExpertLin));
    L.gate_scale = take((size_t)T * 4);
    L.total = at;
    return L;
}

void check_route_shape(int T, int H, int E, int k)
{
    if (T < 1 || H < 1 || E < 1 || k < 1) throw std::runtime_error("moe: sizes must be positive");
    if (k > E) throw std::runtime_error("moe: top-k exceeds the number of experts");
    if (E > kMaxExperts) throw std::runtime_error("moe: at most 1024 experts");
    if (k > kMaxTopK) throw std::runtime_error("moe: top-k must be at most 32");
}

std::string run_route(const void* x, const void* wr, const float* bias, int32_t* idx, float* w,
                      float* logits, float* parts, int T, int H, int E, int k, int renorm,
                      hipStream_t stream, const PermuteParams* sort = nullptr)
{
    LaunchScope scope(stream);
    Workspace& ws = scope.ws;
    RouteParams p{};
    p.x = (const _Float16*)x;
    p.wr = (const _Float16*)wr;
    p.bias = bias;
    p.parts = parts;
    p.counters = ws.counters;
    p.idx = idx;
    p.w = w;
    p.logits = logits;
    p.T = T; p.H = H; p.E = E; p.k = k; p.renorm = renorm;
    p.nseg = (H + kRouteSeg - 1) / kRouteSeg;
    if (sort && T == 1) p.sort = *sort;
    const int groups = (T + kRouteTT - 1) / kRouteTT;
    if (T >= kRouteBigT && E % 2 == 0 && H % kRouteSeg == 0 && p.nseg <= 128 && knobs().moe_route_slab) {
        // one launch: tokens per workgroup as many as the segment sums leave room for in 64 KiB
        // of LDS, fewer while that leaves compute units without a workgroup
        const int nslab = (E + kSlabExperts - 1) / kSlabExperts;
        int tt = 4;
        constexpr int kSlabLdsMax = 144 * 1024;
        while (tt > 1 && (route_slab_lds_bytes(p.nseg, tt) > kSlabLdsMax || (long)nslab * ((T + tt - 1) / tt) < ws.cu_count / 2)) tt /= 2;
        const int tgroups = (T + tt - 1) / tt;
        if (route_slab_lds_bytes(p.nseg, tt) <= kSlabLdsMax && (long)tgroups * kRouteCounterStride <= kCounters) {
            dim3 grid(tgroups, nslab);
            const size_t lds = (size_t)route_slab_lds_bytes(p.nseg, tt);
            static bool raised[3][64] = {};
            if (tt == 4) {
                raise_dynamic_lds_limit((const void*)moe_route_slab_kernel<4>, kSlabLdsMax, raised[0], "moe_route_slab_kernel shared-memory attribute");
                hipLaunchKernelGGL(moe_route_slab_kernel<4>, grid, dim3(1024), lds, stream, p);
            } else if (tt == 2) {
                raise_dynamic_lds_limit((const void*)moe_route_slab_kernel<2>, kSlabLdsMax, raised[1], "moe_route_slab_kernel shared-memory attribute");
                hipLaunchKernelGGL(moe_route_slab_kernel<2>, grid, dim3(1024), lds, stream, p);
            } else {
                raise_dynamic_lds_limit((const void*)moe_route_slab_kernel<1>, kSlabLdsMax, raised[2], "moe_route_slab_kernel shared-memory attribute");
                hipLaunchKernelGGL(moe_route_slab_kernel<1>, grid, dim3(1024), lds, stream, p);
            }
            hip_ok(hipGetLastError(), "moe_route_slab_kernel launch");
            return "moe_route_slab_kernel<" + std::to_string(tt) + "> grid=" + std::to_string(nslab) + "x" +
                   std::to_string(tgroups);
        }
    }
    if (T >= kRouteBigT) {
        const int group = route_big_group(E);
        dim3 grid(p.nseg, (T + group - 1) / group);
        if (route_big_tokens(E) == 8) hipLaunchKernelGGL(moe_route_partial_kernel<8>, grid, dim3(256), 0, stream, p);
        else hipLaunchKernelGGL(moe_route_partial_kernel<4>, grid, dim3(256), 0, stream, p);
        hip_ok(hipGetLastError(), "moe_route_partial_kernel launch");
        hipLaunchKernelGGL(moe_route_finish_kernel, dim3(T), dim3(256), 0, stream, p);
        hip_ok(hipGetLastError(), "moe_route_finish_kernel launch");
        return "moe_route_partial_kernel grid=" + std::to_string(grid.x) + "x" + std::to_string(grid.y) +
               " + moe_route_finish_kernel grid=" + std::to_string(T);
    }
    if (T == 1 && E % 2 == 0 && E <= kRouteOneMaxE && p.nseg <= kRouteOneMaxSeg) {
        hipLaunchKernelGGL(moe_route_one_token_kernel, dim3(1), dim3(1024), 0, stream, p);
        hip_ok(hipGetLastError(), "moe_route_one_token_kernel launch");
        return std::string("moe_route_one_token_kernel grid=1") + (p.sort.perm ? " (with the sort of the one token)" : "");
    }
    if ((long)groups * kRouteCounterStride > kCounters) throw std::runtime_error("moe route: too many tokens for the counter table");
    dim3 grid(p.nseg, groups);
    hipLaunchKernelGGL(moe_route_kernel, grid, dim3(256), 0, stream, p);
    hip_ok(hipGetLastError(), "moe_route_kernel launch");
    return "moe_route_kernel grid=" + std::to_string(grid.x) + "x" + std::to_string(grid.y) +
           (p.sort.perm ? " (with the sort of the one token)" : "");
}

PermuteParams permute_params(const int32_t* idx, unsigned char* wsb, const MoeLayout& L, int T, int k, int E, bool fold)
{
    PermuteParams p{};
    p.idx = idx;
    p.offsets = (int32_t*)(wsb + L.offsets);
    p.perm = (int32_t*)(wsb + L.perm);
    p.inv = (int32_t*)(wsb + L.inv);
    p.row_expert = (int32_t*)(wsb + L.row_expert);
    p.counts = (int32_t*)(wsb + L.counts);
    p.vprob = (GroupProblem*)(wsb + L.vprob);
    p.mprob = (GroupProblem*)(wsb + L.mprob);
    p.bprob = (GroupProblem*)(wsb + L.bprob);
    p.T = T;
    p.k = k;
    p.E = E;
    p.use_valu = L.max_v > 0 ? 1 : 0;
    p.shared_rows = fold ? 1 : 0;
    p.big_min = L.big_min > 0 ? L.big_min : (1 << 30);
    return p;
}

std::string run_permute(const PermuteParams& p, hipStream_t stream)
{
    hipLaunchKernelGGL(moe_permute_kernel, dim3(1), dim3(1024), 0, stream, p);
    hip_ok(hipGetLastError(), "moe_permute_kernel launch");
    return "moe_permute_kernel";
}

}  // namespace
}  // namespace berth

using namespace berth;

extern "C" const char* berth_moe_last_error(void) { return g_moe_err.c_str(); }
extern "C" const char* berth_moe_last_launch(void) { return g_moe_launch.c_str(); }

#define MOE_TRY_BEGIN try { g_moe_err.clear(); g_moe_launch.clear();
#define MOE_TRY_END return 0; } catch (const std::exception& err) { g_moe_err = err.what(); g_moe_launch.clear(); (void)hipGetLastError(); return -1; }

extern "C" size_t berth_moe_workspace_bytes(int T, int H, int E, int k, int I, int shared_I)
{
    if (T < 1 || H < 1 || E < 1 || k < 1 || I < 1 || shared_I < 0) return 0;
    return moe_layout(T, H, E, k, I, shared_I).total;
}

// byte offsets, inside a workspace of berth_moe_workspace_bytes, of the buffers a
// caller may want to inspect after berth_moe_layer: {idx, w, offsets, perm, inv,
// gate_out, up_out, slot_out, shared_out}
extern "C" int berth_moe_workspace_offsets(int T, int H, int E, int k, int I, int shared_I, size_t out[9])
{
    if (T < 1 || H < 1 || E < 1 || k < 1 || I < 1 || shared_I < 0 || !out) return -1;
    const MoeLayout L = moe_layout(T, H, E, k, I, shared_I);
    const size_t v[9] = {L.idx, L.w, L.offsets, L.perm, L.inv, L.g, L.u, L.slot_out, L.shared_out};
    for (int i = 0; i < 9; ++i) out[i] = v[i];
    return 0;
}

// the always-on expert's own intermediates when its width differs from the routed experts'
// (it is then no row of the grouped launches): {gate fp16 [T][shared_I], up fp16 [T][shared_I]};
// above 8 rows the second one ends up holding silu(gate) * up
extern "C" int berth_moe_workspace_shared_offsets(int T, int H, int E, int k, int I, int shared_I, size_t out[2])
{
    if (T < 1 || H < 1 || E < 1 || k < 1 || I < 1 || shared_I < 1 || shared_I == I || !out) return -1;
    const MoeLayout L = moe_layout(T, H, E, k, I, shared_I);
    out[0] = L.sg;
    out[1] = L.su;
    return 0;
}

extern "C" int berth_moe_route(const void* x, const void* wr, const float* bias, int32_t* idx, float* w,
                               float* logits, void* parts_scratch, int T, int H, int E, int k,
                               int renorm, void* stream)
{
    MOE_TRY_BEGIN
    if (!x || !wr || !idx || !w || !parts_scratch) throw std::runtime_error("moe route: null device pointer");
    check_route_shape(T, H, E, k);
    g_moe_launch = run_route(x, wr, bias, idx, w, logits, (float*)parts_scratch, T, H, E, k, renorm,
                             (hipStream_t)stream);
    MOE_TRY_END
}

extern "C" int berth_moe_permute(const int32_t* idx, int32_t* offsets, int32_t* perm, int32_t* inv,
                                 void* scratch, int T, int k, int E, void* stream)
{
    MOE_TRY_BEGIN
    if (!idx || !offsets || !perm || !inv || !scratch) throw std::runtime_error("moe permute: null device pointer");
    if (T < 1 || k < 1 || E < 1) throw std::runtime_error("moe: sizes must be positive");
    if (E > kMaxExperts) throw std::runtime_error("moe: at most 1024 experts");
    // scratch holds the row maps, the counts and the problem lists
    const size_t P = (size_t)T * k;
    unsigned char* sb = (unsigned char*)scratch;
    const PermuteScratch at = permute_scratch_layout(T, k, E);
    PermuteParams p{};
    p.idx = idx;
    p.offsets = offsets;
    p.perm = perm;
    p.inv = inv;
    p.row_expert = (int32_t*)(sb + at.row_expert);
    p.counts = (int32_t*)(sb + at.counts);
    p.vprob = (GroupProblem*)(sb + at.vprob);
    p.mprob = (GroupProblem*)(sb + at.mprob);
    p.bprob = (GroupProblem*)(sb + at.bprob);
    p.T = T;
    p.k = k;
    p.E = E;
    p.use_valu = (T == 1 || P <= (size_t)kValuPairs) ? 1 : 0;
    p.shared_rows = 0;
    p.big_min = !p.use_valu && at.big_min > 0 ? at.big_min : (1 << 30);
    hipLaunchKernelGGL(moe_permute_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, p);
    hip_ok(hipGetLastError(), "moe_permute_kernel launch");
    g_moe_launch = "moe_permute_kernel";
    MOE_TRY_END
}

extern "C" size_t berth_moe_permute_scratch_bytes(int T, int k, int E)
{
    if (T < 1 || k < 1 || E < 1) return 0;
    return permute_scratch_layout(T, k, E).total;
}

// One stage of the layer on its own: a grouped EXL3 linear (or the gate / up pair) over the
// expert-sorted rows, driven by the problem lists berth_moe_permute left in its scratch.
extern "C" int berth_moe_grouped_exl3(const void* a, const void* a_up, const int32_t* gather, int gather_div,
                                      const void* experts, int lins_per_expert, int lin_base, int num_lins,
                                      void* c0, void* c1, const void* permute_scratch, void* a_had, int T, int k,
                                      int E, int size_k, int size_n, int k_bits, int codebook, int c_fp32,
                                      void* stream_)
{
    MOE_TRY_BEGIN
    hipStream_t stream = (hipStream_t)stream_;
    if (!a || !experts || !c0 || !permute_scratch) throw std::runtime_error("moe grouped linear: null device pointer");
    if (T < 1 || k < 1 || E < 1 || size_k < 1 || size_n < 1) throw std::runtime_error("moe: sizes must be positive");
    if (k > E) throw std::runtime_error("moe: top-k exceeds the number of experts");
    if (E > kMaxExperts) throw std::runtime_error("moe: at most 1024 experts");
    if ((long)T * k > 65535) throw std::runtime_error("moe grouped linear: at most 65535 (token, slot) pairs per call");
    if (num_lins != 1 && num_lins != 2) throw std::runtime_error("moe grouped linear: num_lins must be 1 or 2");
    if ((num_lins == 2) != (c1 != nullptr)) throw std::runtime_error("moe grouped linear: c1 goes with the second linear");
    if (num_lins == 2 && a_up) throw std::runtime_error("moe grouped linear: the silu input serves one linear");
    if (lins_per_expert < 1 || lin_base < 0 || lin_base + num_lins > lins_per_expert)
        throw std::runtime_error("moe grouped linear: lin_base + num_lins exceeds lins_per_expert");
    if (gather && gather_div < 1) throw std::runtime_error("moe grouped linear: gather_div must be positive");
    if (k_bits < 1 || k_bits > 8) throw std::runtime_error("moe grouped linear: K must be in 1..=8");
    if (codebook < 0 || codebook > 2) throw std::runtime_error("moe grouped linear: codebook must be 0, 1, or 2");
    if (c_fp32 != 0 && c_fp32 != 1) throw std::runtime_error("moe grouped linear: c_fp32 must be 0 or 1");
    if (size_k % 128 || size_n % 128) throw std::runtime_error("moe grouped linear: sizes must be multiples of 128");
    const int P = T * k;
    const bool use_valu = T == 1 || P <= kValuPairs;        // what berth_moe_permute chose for these sizes
    if (!use_valu && !a_had) throw std::runtime_error("moe grouped linear: a_had is required above 8 rows");
    const unsigned char* sb = (const unsigned char*)permute_scratch;
    const PermuteScratch at = permute_scratch_layout(T, k, E);

    GroupedArgs g{};
    g.a = a;
    g.a_up = a_up;
    g.gather = gather;
    g.gather_div = gather ? gather_div : 1;
    g.experts = experts;
    g.shared = nullptr;
    g.shared_expert = -1;
    g.single_row = T == 1 ? 1 : 0;
    g.lins_per_expert = lins_per_expert;
    g.lin_base = lin_base;
    g.num_lins = num_lins;
    g.c0 = c0;
    g.c1 = c1;
    g.size_k = size_k;
    g.size_n = size_n;
    g.k_bits = k_bits;
    g.codebook = codebook;
    g.out_fp32 = c_fp32;
    g.stream = stream;
    if (use_valu) {
        g.problems = sb + at.vprob;
        g.num_problems = (const int*)(sb + at.counts);
        g.max_problems = (int)std::min<size_t>((size_t)E, (size_t)P);
        g_moe_launch = launch_gemv_grouped(g);
    } else {
        HadRowsParams h{};
        h.a = (const _Float16*)a;
        h.a_up = (const _Float16*)a_up;
        h.gather = gather;
        h.gather_div = g.gather_div;
        h.row_expert = (const int32_t*)(sb + at.row_expert);
        h.experts = (const ExpertLin*)experts;
        h.shared_expert = -1;
        h.lins_per_expert = lins_per_expert;
        h.lin_base = lin_base;
        h.out[0] = (_Float16*)a_had;
        h.out[1] = (_Float16*)a_had + (size_t)P * size_k;
        h.P = P;
        h.K = size_k;
        h.num_lins = num_lins;
        launch_had_rows(h, stream);
        g.a_had = h.out[0];
        g.a_had2 = num_lins == 2 ? h.out[1] : nullptr;
        g.problems = sb + at.mprob;
        g.num_problems = (const int*)(sb + at.counts) + 1;
        g.max_problems = at.max_m;
        g.mb = 1;
        if (at.max_b > 0) {
            g.big_problems = sb + at.bprob;
            g.num_big = (const int*)(sb + at.counts) + 2;
            g.max_big = at.max_b;
        }
        g_moe_launch = "moe_had_rows_kernel + " + launch_gemm_grouped(g);
    }
    MOE_TRY_END
}

// out[t] = shared_out[t] + sum_j w[t][j] * slot_out[inv[t * k + j]] in slot order
extern "C" int berth_moe_combine(const void* slot_out, const void* shared_out, const float* w, const int32_t* inv,
                                 void* out, int T, int H, int k, void* stream)
{
    MOE_TRY_BEGIN
    if (!slot_out || !w || !inv || !out) throw std::runtime_error("moe combine: null device pointer");
    if (T < 1 || H < 1 || k < 1) throw std::runtime_error("moe: sizes must be positive");
    launch_combine((const float*)slot_out, (const float*)shared_out, nullptr, w, inv, (float*)out, T, H, k,
                   (hipStream_t)stream);
    g_moe_launch = "moe_combine_kernel";
    MOE_TRY_END
}

extern "C" int berth_moe_layer(const void* x, const void* wr, const float* bias, const void* experts,
                               const berth_exl3_lin* shared, void* out, int32_t* idx_out, float* w_out,
                               void* workspace, size_t workspace_bytes, int T, int H, int E, int k,
                               int I, int shared_I, int k_bits, int codebook, int renorm, void* stream_)
{
    return berth_moe_layer_gated(x, wr, bias, experts, shared, nullptr, out, idx_out, w_out, workspace, workspace_bytes, T,
                                 H, E, k, I, shared_I, k_bits, codebook, renorm, stream_);
}

extern "C" int berth_moe_layer_gated(const void* x, const void* wr, const float* bias, const void* experts,
                                     const berth_exl3_lin* shared, const float* shared_gate, void* out,
                                     int32_t* idx_out, float* w_out, void* workspace, size_t workspace_bytes, int T,
                                     int H, int E, int k, int I, int shared_I, int k_bits, int codebook, int renorm,
                                     void* stream_)
{
    MOE_TRY_BEGIN
    hipStream_t stream = (hipStream_t)stream_;
    if (!x || !wr || !experts || !out || !workspace) throw std::runtime_error("moe layer: null device pointer");
    check_route_shape(T, H, E, k);
    if (I < 1) throw std::runtime_error("moe: sizes must be positive");
    if ((long)T * k > 65535) throw std::runtime_error("moe layer: at most 65535 (token, slot) pairs per call");
    if (k_bits < 1 || k_bits > 8) throw std::runtime_error("moe layer: K must be in 1..=8");
    if (codebook < 0 || codebook > 2) throw std::runtime_error("moe layer: codebook must be 0, 1, or 2");
    if (H % 128 || I % 128) throw std::runtime_error("moe layer: hidden and intermediate sizes must be multiples of 128");
    if (shared && (shared_I < 128 || shared_I % 128))
        throw std::runtime_error("moe layer: shared intermediate size must be a multiple of 128");
    if (shared_gate && !shared) throw std::runtime_error("moe layer: a shared-expert gate without a shared expert");
    if (!shared) shared_I = 0;
    const bool fold = shared_is_folded(I, shared_I);
    if (fold && E + 1 > kMaxExperts) throw std::runtime_error("moe: at most 1023 routed experts next to a shared expert");
    const MoeLayout L = moe_layout(T, H, E, k, I, shared_I);
    if (workspace_bytes < L.total)
        throw std::runtime_error("moe layer: workspace too small (" + std::to_string(workspace_bytes) + " < " +
                                 std::to_string(L.total) + ")");
    unsigned char* wsb = (unsigned char*)workspace;
    const int P = T * k;
    const int R = P + (fold ? T : 0);
    int32_t* idx = (int32_t*)(wsb + L.idx);
    float* w = (float*)(wsb + L.w);
    std::string desc;
    if (shared)
        for (int i = 0; i < 3; ++i)
            if (!shared[i].trellis || !shared[i].suh || !shared[i].svh)
                throw std::runtime_error("moe layer: null shared-expert pointer");

    const PermuteParams pp = permute_params(idx, wsb, L, T, k, E, fold);
    RouteParams inline_route{};
    const bool route_inline = T == 1 && E % 2 == 0 && E <= kRouteOneMaxE && L.nseg <= kRouteOneMaxSeg && L.max_v > 0 &&
                              inline_route_enabled();
    const bool use_resolved = route_inline && resolved_records_enabled();
    if (route_inline) {
        RouteParams& r = inline_route;
        r.x = (const _Float16*)x;
        r.wr = (const _Float16*)wr;
        r.bias = bias;
        r.parts = (float*)(wsb + L.parts);
        r.idx = idx;
        r.w = w;
        r.T = 1; r.H = H; r.E = E; r.k = k; r.renorm = renorm;
        r.nseg = L.nseg;
        r.sort = pp;
        hipLaunchKernelGGL(moe_route_segments_kernel, dim3(L.nseg), dim3(64), 0, stream, r);
        hip_ok(hipGetLastError(), "moe_route_segments_kernel launch");
        desc += "moe_route_segments_kernel grid=" + std::to_string(L.nseg) + " (top-k and sort inside the next launch)";
    } else {
        desc += run_route(x, wr, bias, idx, w, nullptr, (float*)(wsb + L.parts), T, H, E, k, renorm, stream, &pp);
        if (T > 1) desc += " + " + run_permute(pp, stream);
    }

    GroupedArgs g{};
    g.experts = experts;
    g.shared = fold ? shared : nullptr;
    g.shared_expert = fold ? E : -1;
    g.single_row = T == 1 ? 1 : 0;
    g.lins_per_expert = 3;
    g.k_bits = k_bits;
    g.codebook = codebook;
    g.stream = stream;

    // gate and up: input rows gathered from x, fp16 out in sorted order
    g.a = x;
    g.a_up = nullptr;
    g.gather = (const int32_t*)(wsb + L.perm);
    g.gather_div = k;
    g.lin_base = 0;
    g.num_lins = 2;
    g.c0 = wsb + L.g;
    g.c1 = wsb + L.u;
    g.size_k = H;
    g.size_n = I;
    g.out_fp32 = 0;
    if (L.max_v > 0) {
        g.problems = wsb + L.vprob;
        g.num_problems = (const int*)(wsb + L.counts);
        g.max_problems = L.max_v;
        g.route_params = route_inline ? &inline_route : nullptr;
        if (use_resolved) {
            g.resolved_out = wsb + L.vlin;
            g.resolved_lin = 2;
        }
        desc += " + " + launch_gemv_grouped(g);
        g.route_params = nullptr;
        g.resolved_out = nullptr;
    }
    if (L.max_m > 0) {
        HadRowsParams h{};
        h.a = (const _Float16*)x;
        h.gather = (const int32_t*)(wsb + L.perm);
        h.gather_div = k;
        h.row_expert = (const int32_t*)(wsb + L.row_expert);
        h.experts = (const ExpertLin*)experts;
        h.shared_expert = g.shared_expert;
        if (fold) for (int i = 0; i < 3; ++i) h.shared[i] = ExpertLin{(const uint32_t*)shared[i].trellis, (const _Float16*)shared[i].suh, (const _Float16*)shared[i].svh};
        h.lins_per_expert = 3;
        h.lin_base = 0;
        h.out[0] = (_Float16*)(wsb + L.ah0);
        h.out[1] = (_Float16*)(wsb + L.ah1);
        h.P = R;
        h.K = H;
        h.num_lins = 2;
        launch_had_rows(h, stream);
        g.a_had = wsb + L.ah0;
        g.a_had2 = wsb + L.ah1;
        desc += " + moe_had_rows_kernel";
        if (L.max_b > 0) {
            g.big_problems = wsb + L.bprob;
            g.num_big = (const int*)(wsb + L.counts) + 2;
            g.max_big = L.max_b;
        }
        g.problems = wsb + L.mprob;
        g.num_problems = (const int*)(wsb + L.counts) + 1;
        g.max_problems = L.max_m;
        g.mb = 1;
        desc += " + " + launch_gemm_grouped(g);
    }

    // shared expert: three dense linears on every token (ahead of the routed down
    // projection, which may finish the layer)
    const float* shared_out = nullptr;
    if (fold) {
        shared_out = (const float*)(wsb + L.shared_out);
        desc += " (shared expert in the grouped launches)";
    } else if (shared) {
        auto dense = [&](const void* a, const berth_exl3_lin& lin, void* c, int kk, int nn, int fp32) {
            LinearArgs la{a, lin.trellis, c, lin.suh, wsb + L.s_ahad, lin.svh, T, kk, nn, k_bits, codebook, fp32, stream};
            return T <= 8 ? launch_gemv(la) : launch_gemm(la);
        };
        if (T <= 8) {
            // gate and up in one launch, silu(g) * u formed inside the down projection
            PairArgs pa{x, {shared[0].trellis, shared[1].trellis}, {shared[0].suh, shared[1].suh},
                        {shared[0].svh, shared[1].svh}, {wsb + L.sg, wsb + L.su}, wsb + L.s_ahad, T, H, shared_I,
                        k_bits, codebook, stream};
            launch_gemv_pair(pa);
            LinearArgs down{wsb + L.sg, shared[2].trellis, wsb + L.shared_out, shared[2].suh, wsb + L.s_ahad,
                            shared[2].svh, T, shared_I, H, k_bits, codebook, 1, stream};
            down.a_up = wsb + L.su;
            launch_gemv(down);
        } else {
            dense(x, shared[0], wsb + L.sg, H, shared_I, 0);
            dense(x, shared[1], wsb + L.su, H, shared_I, 0);
            launch_silu_mul(wsb + L.sg, wsb + L.su, wsb + L.su, (int64_t)T * shared_I, 0.0f, stream);
            dense(wsb + L.su, shared[2], wsb + L.shared_out, shared_I, H, 1);
        }
        shared_out = (const float*)(wsb + L.shared_out);
        desc += " + shared expert";
    }

    // down: input silu(g) * u evaluated while the activation is rotated, fp32 out
    g.a = wsb + L.g;
    g.a_up = wsb + L.u;
    g.gather = nullptr;
    g.gather_div = 1;
    g.lin_base = 2;
    g.num_lins = 1;
    g.c0 = wsb + L.slot_out;
    g.c1 = nullptr;
    g.size_k = I;
    g.size_n = H;
    g.out_fp32 = 1;
    // one token: the last expert to finish a column block of the down projection
    // also combines that block, so no combine launch follows
    // (not with a gate on the always-on expert's row: the combine launch applies it)
    const bool fold_combine = T == 1 && L.max_v > 0 && L.max_m == 0 && fold_combine_mode() != 0 && !shared_gate;
    if (fold_combine) {
        g.comb_w = (const float*)w;
        g.comb_inv = (const int32_t*)(wsb + L.inv);
        g.comb_shared = shared_out;
        g.comb_out = (float*)out;
        g.comb_k = k;
        // with the always-on expert among the problems its row (row k) starts the chain
        g.comb_single = fold_combine_mode() != 1 && L.max_v <= kCombMaxProblems ? 1 : 0;
        g.comb_shared_prob = fold ? k : -1;
    }
    if (L.max_v > 0) {
        g.problems = wsb + L.vprob;
        g.num_problems = (const int*)(wsb + L.counts);
        g.max_problems = L.max_v;
        g.resolved = use_resolved ? wsb + L.vlin : nullptr;
        desc += " + " + launch_gemv_grouped(g);
        g.resolved = nullptr;
    }
    if (L.max_m > 0) {
        HadRowsParams h{};
        h.a = (const _Float16*)(wsb + L.g);
        h.a_up = (const _Float16*)(wsb + L.u);
        h.gather_div = 1;
        h.row_expert = (const int32_t*)(wsb + L.row_expert);
        h.experts = (const ExpertLin*)experts;
        h.shared_expert = g.shared_expert;
        if (fold) for (int i = 0; i < 3; ++i) h.shared[i] = ExpertLin{(const uint32_t*)shared[i].trellis, (const _Float16*)shared[i].suh, (const _Float16*)shared[i].svh};
        h.lins_per_expert = 3;
        h.lin_base = 2;
        h.out[0] = (_Float16*)(wsb + L.ahd);
        h.P = R;
        h.K = I;
        h.num_lins = 1;
        launch_had_rows(h, stream);
        g.a_had = wsb + L.ahd;
        g.a_had2 = nullptr;
        desc += " + moe_had_rows_kernel";
        if (L.max_b > 0) {
            g.big_problems = wsb + L.bprob;
            g.num_big = (const int*)(wsb + L.counts) + 2;
            g.max_big = L.max_b;
        }
        g.problems = wsb + L.mprob;
        g.num_problems = (const int*)(wsb + L.counts) + 1;
        g.max_problems = L.max_m;
        g.mb = 1;
        desc += " + " + launch_gemm_grouped(g);
    }

    if (!fold_combine) {
        const float* scale = nullptr;
        if (shared_gate) {
            hipLaunchKernelGGL(moe_shared_gate_kernel, dim3(T), dim3(64), 0, stream, (const _Float16*)x, shared_gate,
                               (float*)(wsb + L.gate_scale), H);
            hip_ok(hipGetLastError(), "moe_shared_gate_kernel launch");
            scale = (const float*)(wsb + L.gate_scale);
            desc += " + moe_shared_gate_kernel";
        }
        launch_combine((const float*)(wsb + L.slot_out), shared_out, scale, (const float*)w,
                       (const int32_t*)(wsb + L.inv), (float*)out, T, H, k, stream);
        desc += " + moe_combine_kernel";
    }
    if (idx_out) hip_ok(hipMemcpyAsync(idx_out, idx, (size_t)P * 4, hipMemcpyDeviceToDevice, stream), "idx copy");
    if (w_out) hip_ok(hipMemcpyAsync(w_out, w, (size_t)P * 4, hipMemcpyDeviceToDevice, stream), "w copy");
    g_moe_launch = desc;
    MOE_TRY_END
}

// Routing pieces shared by the MoE kernels and by the one-row grouped GEMV, whose workgroups
// redo the last, cheap part of the one-token routing themselves (ordered sum of the segment
// sums, top-k, sorted positions) instead of waiting for a launch that does it once.
//
// Arithmetic contract of the routing (the reference has no MoE arithmetic; the shapes follow
// crates/berth-plan/src/shape.rs:64-69 and plan.rs:24-59):
//   logits[e] = sum over 64-row segments of (sum_h x[h] * wr[h][e], fp32 fma in row order),
//               segments added in order, then + bias[e];
//   top-k on the logits, largest first, ties to the lowest expert index;
//   weights = exp(logit - max) normalised over the selected k (renorm) or over all experts.
#pragma once

#include "exl3_decode.cuh"
#include "hadamard.cuh"

namespace berth {

// one unit of grouped work: rows [row0, row0 + nrows) of the expert-sorted order
struct GroupProblem {
    int expert;
    int row0;
    int nrows;
    int pad;
};

constexpr int kRouteSeg = 64;       // rows of the router weight per partial sum
constexpr int kRouteTT = 4;         // tokens per route workgroup
constexpr int kRouteCounterStride = 32;   // words between the arrival counters of neighbouring token groups
constexpr int kMaxExperts = 1024;
constexpr int kMaxTopK = 32;

struct PermuteParams {
    const int32_t* idx;     // [P] expert of each (token, slot) pair, P = T * k; distinct within a token
    int32_t* offsets;       // [E + 1]
    int32_t* perm;          // [R] sorted position -> pair (pair / k = token)
    int32_t* inv;           // [P] pair -> sorted position
    int32_t* row_expert;    // [R] sorted position -> expert
    int32_t* counts;        // [3] number of VALU problems, small MFMA problems, big MFMA problems
    GroupProblem* vprob;
    GroupProblem* mprob;    // <= 32 rows each
    GroupProblem* bprob;    // <= 128 rows each
    int T, k, E;
    int use_valu;           // 1: every expert is one VALU problem (<= 8 rows each); 0: MFMA problems: an
                            // expert's rows go to big problems of 128 and the rest to small ones of <= 32
    int shared_rows;        // 1: rows P .. P + T - 1 belong to an always-on expert with index E (token order)
    int big_min;            // a remainder of at least this many rows becomes a (partial) big problem
};

struct RouteParams {
    const _Float16* x;      // [T][H]
    const _Float16* wr;     // [H][E]
    const float* bias;      // [E] or null
    float* parts;           // [T][nseg][E]
    unsigned* counters;     // [ceil(T / kRouteTT)]
    int32_t* idx;           // [T][k]
    float* w;               // [T][k]
    float* logits;          // [T][E] or null
    int T, H, E, k, nseg, renorm;
    // one token only: the wave that selected the experts also sorts them and writes
    // what the permute kernel would (sort.perm != nullptr), saving its launch
    PermuteParams sort;
};

// Top-k of one token by one wave: lane holds the logits of experts lane + 64 i.
// Largest first, ties to the lowest expert index; weights exp(l - max) normalised
// over the selected k (renorm) or over all experts.
constexpr int kRoutePer = kMaxExperts / 64;

__device__ __forceinline__ float lane_value(float v, int lane_index)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane_index));
}

// the same value in every lane: butterflies over lane distances 1 .. 32
__device__ __forceinline__ float wave_max(float v)
{
    v = fmaxf(v, lane_xor_dpp<1>(v));
    v = fmaxf(v, lane_xor_dpp<2>(v));
    v = fmaxf(v, lane_xor_dpp<4>(v));
    v = fmaxf(v, lane_xor_dpp<8>(v));
    v = fmaxf(v, lane_xor_swap16(v));
    return fmaxf(v, lane_xor_swap32(v));
}
// PER: how many of the lane's registers can hold experts (ceil(E / 64) rounded up to 2, 8 or 16)
template <int PER>
__device__ __forceinline__ int route_topk_n(const float (&lg)[kRoutePer], int lane, const RouteParams& p, int t,
                                            bool store = true)
{
    unsigned taken = 0;
    float sel_logit = 0.0f;         // lane j keeps the logit of slot j
    int sel_idx = 0;
    // One slot per round: the largest remaining logit of the wave (max butterflies), then the
    // lowest expert index among the registers that hold it (ballots).  One short reduction of
    // one value instead of a reduction of (value, index) pairs with a tie rule.
    for (int j = 0; j < p.k; ++j) {
        float lv = -INFINITY;
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (lane + 64 * i < p.E && !((taken >> i) & 1u)) lv = fmaxf(lv, lg[i]);
        const float bv = wave_max(lv);
        // the lowest expert index that holds it: register i of lane l is expert l + 64 i, so
        // the first register with a holder wins and, inside it, the lowest lane (a ballot
        // and a find-first-set on the scalar side instead of a second butterfly chain)
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = PER - 1; i >= 0; --i) {
            const unsigned long long holders =
                __builtin_amdgcn_ballot_w64(lane + 64 * i < p.E && !((taken >> i) & 1u) && lg[i] == bv);
            if (holders) bi = 64 * i + __builtin_ctzll(holders);
        }
        if ((bi & 63) == lane) taken |= 1u << (bi >> 6);
        if (lane == j) { sel_logit = bv; sel_idx = bi; }
    }
    // lane j is wave-uniform here: v_readlane instead of a round trip through the LDS crossbar
    const float mx = lane_value(sel_logit, 0);
    float ev = (lane < p.k) ? expf(sel_logit - mx) : 0.0f;
    float denom = 0.0f;
    if (p.renorm) {
        for (int j = 0; j < p.k; ++j) denom += lane_value(ev, j);       // slot order
    } else {
        float loc = 0.0f;
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (lane + 64 * i < p.E) loc += expf(lg[i] - mx);
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) loc += __shfl_xor(loc, d, 64);
        denom = loc;
    }
    if (store && lane < p.k) {
        p.idx[(size_t)t * p.k + lane] = sel_idx;
        p.w[(size_t)t * p.k + lane] = ev / denom;
    }
    return sel_idx;     // lane j < k: expert of slot j
}

__device__ __forceinline__ int route_topk(const float (&lg)[kRoutePer], int lane, const RouteParams& p, int t)
{
    if (p.E <= 128) return route_topk_n<2>(lg, lane, p, t);         // workgroup-uniform
    if (p.E <= 512) return route_topk_n<8>(lg, lane, p, t);
    return route_topk_n<kRoutePer>(lg, lane, p, t);
}

// One token: what moe_permute_kernel writes, by the wave that holds the selection
// (lane j < k has the expert of slot j; the k experts are distinct).  Sorted position
// of slot j = number of selected experts with a smaller index; every expert is one
// single-row VALU problem; an always-on expert (shared_rows) takes row k.
__device__ __forceinline__ void route_sort_one_token(const PermuteParams& q, int lane, int sel_idx)
{
    const int k = q.k;
    int rank = 0;
    for (int j = 0; j < k; ++j) {
        const int other = __builtin_amdgcn_readlane(sel_idx, j);
        rank += (lane < k && other < sel_idx) ? 1 : 0;
    }
    if (lane < k) {
        q.perm[rank] = lane;
        q.inv[lane] = rank;
        q.row_expert[rank] = sel_idx;
        q.vprob[rank] = GroupProblem{sel_idx, rank, 1, 0};
    }
    // offsets[e] = number of selected experts below e
    for (int e0 = 0; e0 <= q.E; e0 += 64) {         // wave-uniform loop: every lane takes part in the exchanges
        const int e = e0 + lane;
        int below = 0;
        for (int j = 0; j < k; ++j) below += (__builtin_amdgcn_readlane(sel_idx, j) < e) ? 1 : 0;
        if (e <= q.E) q.offsets[e] = below;
    }
    if (lane == 0) {
        if (q.shared_rows) {
            q.perm[k] = 0;
            q.row_expert[k] = q.E;
            q.vprob[k] = GroupProblem{q.E, k, 1, 0};
        }
        q.counts[0] = k + (q.shared_rows ? 1 : 0);
        q.counts[1] = 0;
        q.counts[2] = 0;
    }
}


// One token, at most 128 experts: the routing's last part by one wave, from the segment sums
// parts[seg][e] that moe_route_segments_kernel left in memory: logits (segments added in
// order, bias), top-k, and the sorted position of every selected expert (lane j < k: expert of
// slot j and its sorted position).  Every wave that calls this gets the same bits; the wave
// with `writer` set also stores the routing results (logits, idx, w, and what the sort of the
// one token writes).
struct RouteOneToken {
    int sel;
    int rank;
};

__device__ __forceinline__ RouteOneToken route_one_token(const RouteParams& p, int lane, bool writer)
{
    float lg[kRoutePer];
#pragma unroll
    for (int i = 0; i < kRoutePer; ++i) lg[i] = -INFINITY;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int e = lane + 64 * i;
        if (e < p.E) {
            const float* src = p.parts + e;
            float v = 0.0f;
            // 32 loads in flight at a time (indices past the end re-read the last segment and
            // are ignored); the adds stay in segment order
            for (int s0 = 0; s0 < p.nseg; s0 += 32) {
                float part[32];
#pragma unroll
                for (int j = 0; j < 32; ++j) part[j] = src[(size_t)min(s0 + j, p.nseg - 1) * p.E];
#pragma unroll
                for (int j = 0; j < 32; ++j) {
                    const float nv = v + part[j];
                    v = s0 + j < p.nseg ? nv : v;
                }
            }
            if (p.bias) v += p.bias[e];
            if (writer && p.logits) p.logits[e] = v;
            lg[i] = v;
        }
    }
    RouteOneToken r;
    r.sel = route_topk_n<2>(lg, lane, p, 0, writer);
    if (writer && p.sort.perm) route_sort_one_token(p.sort, lane, r.sel);
    r.rank = 0;
    for (int j = 0; j < p.k; ++j) {
        const int other = __builtin_amdgcn_readlane(r.sel, j);
        r.rank += other < r.sel ? 1 : 0;
    }
    return r;
}

// the expert whose sorted position is `want_rank` (the always-on expert E for want_rank == k)
__device__ __forceinline__ int route_expert_at(const RouteParams& p, const RouteOneToken& r, int lane, int want_rank)
{
    if (want_rank >= p.k) return p.E;
    const unsigned long long holder = __builtin_amdgcn_ballot_w64(lane < p.k && r.rank == want_rank);
    return __builtin_amdgcn_readlane(r.sel, (int)__builtin_ctzll(holder));
}

}  // namespace berth

// EXL3 linear for 1..8 rows: trellis decode fused into a VALU dot product.
//
//   c = ( Hh(a * suh) @ W ) -> Hh(.) * svh          (Hh = 128-block Hadamard / sqrt(128))
//
// One launch does the whole operator of crates/berth-kernels/csrc/linear.cu:209-286
// (the m = 1 path the reference routes to its int8 GEMV) and of the small-row
// cases of crates/berth-kernels/csrc/prefill_lin/linear.cu:277-343:
//   * a wave owns (128 output columns) x (128-row k-blocks); per k-block it
//     rotates the activation itself (fp32 butterflies, rounded to fp16, written
//     to a_had by the column-block-0 workgroups), streams 8 tile rows of 1 KiB
//     (at 4 bpw) with one `bits`-dword load per lane, decodes 32 weights per lane
//     and accumulates fp32 dot products against the rotated activation in LDS;
//   * the 4 waves of a workgroup split K and reduce in LDS in wave order;
//   * if K is split over S workgroups the partial sums go to the library's
//     workspace and the last workgroup to arrive adds them in split order,
//     applies the output Hadamard and svh and stores c.  The arrival counter
//     resets itself.  Summation order never depends on timing.
#include "exl3_gemv_stream_kernel.cuh"
#include "launch.h"

#include <algorithm>
#include <optional>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace berth {

// one translation unit per codebook (exl3_gemv_cb{0,1,2}.hip) keeps the build parallel
void launch_gemv_cb0(const GemvParams& p, int bits, int mmax, dim3 grid, hipStream_t stream);
void launch_gemv_cb1(const GemvParams& p, int bits, int mmax, dim3 grid, hipStream_t stream);
void launch_gemv_cb2(const GemvParams& p, int bits, int mmax, dim3 grid, hipStream_t stream);

static void launch_bits(const GemvParams& p, int bits, int cb, int mmax, dim3 grid, hipStream_t stream)
{
    switch (cb) {
    case 0: launch_gemv_cb0(p, bits, mmax, grid, stream); break;
    case 1: launch_gemv_cb1(p, bits, mmax, grid, stream); break;
    default: launch_gemv_cb2(p, bits, mmax, grid, stream); break;
    }
}

void launch_gemv_stream_cb0(const StreamParams& p, int bits, int lutmask, dim3 grid, hipStream_t stream);
void launch_gemv_stream_cb1(const StreamParams& p, int bits, int lutmask, dim3 grid, hipStream_t stream);
void launch_gemv_stream_cb2(const StreamParams& p, int bits, int lutmask, dim3 grid, hipStream_t stream);

// ---- the one-row streaming kernel: the static split and when it applies
//
// Of a problem's U = (N/128) * (K/16) units every wave of its Gp workgroups takes q (the
// first `rem` waves q + 1).  The kernel applies when every wave gets at least
// `stream_min_units` tile rows (below that the fixed cost of a sixteen-wave workgroup, its
// table copy and its barriers, is not paid back), when the rotated activation of a
// workgroup's units fits its LDS region and when the exact-division multipliers are exact
// for the operands the kernel divides.
struct StreamPlan {
    bool ok = false;
    int problems = 0, Gp = 0;
    unsigned q = 0, rem = 0, mq = 0, mq1 = 0, mtr = 0;
};

// Hybrid decode (BERTH_GEMV_STREAM_LUT: bit pp set = pair pp of every dword comes from a
// 128 KiB state -> weight table in LDS that the workgroup builds at its start; 0: arithmetic
// only; unset: by size).  Building the table costs about two tile rows of decode per wave and
// a table weight still costs 2.5 vector instructions against 4.4, with the random 2-byte LDS
// reads as the next bound: it pays for long launches only (4 bpw, at least 1 MiB of weights
// per workgroup: 335 MB weight 103.6 -> 92.4 us), not for the 10-30 us launches of a layer set.
static int stream_lut_mask(int bits, unsigned long long bytes_per_workgroup)
{
    const int forced = knobs().gemv_stream_lut;
    if (forced >= 0) return forced;
    return bits == 4 && bytes_per_workgroup >= (1ull << 20) ? 0xA : 0;
}

static unsigned magic(unsigned d) { return (unsigned)((1ull << 32) / d) + 1u; }

static StreamPlan plan_stream(const Workspace& ws, int problems, int K, int N)
{
    StreamPlan pl;
    const Knobs& kn = knobs();
    if (!kn.gemv_stream || problems < 1 || problems > ws.cu_count || !ws.accum) return pl;
    const unsigned TR = (unsigned)K / 16, NB = (unsigned)N / 128, KB = (unsigned)K / 128;
    const unsigned long long U = (unsigned long long)NB * TR;
    if (U >= (1ull << 31)) return pl;
    const unsigned min_units = (unsigned)kn.gemv_stream_min_units;
    int Gp = ws.cu_count / problems;
    if (kn.gemv_stream_wgs > 0 && Gp > kn.gemv_stream_wgs) Gp = kn.gemv_stream_wgs;
    if (U / ((unsigned)Gp * kStreamWaves) < min_units) {
        if (!kn.gemv_stream_shrink) return pl;
        Gp = (int)(U / (min_units * kStreamWaves));
        if (Gp < 1) return pl;
    }
    const unsigned waves = (unsigned)Gp * kStreamWaves;
    const unsigned q = (unsigned)(U / waves), rem = (unsigned)(U % waves);
    // exact division by multiply-high needs dividend * divisor < 2^32
    if (U * (q + 2) >= (1ull << 32) || U * TR >= (1ull << 32)) return pl;
    const unsigned L = kStreamWaves * (q + 1);                 // most units of one workgroup
    if ((L + TR - 1) / TR + 1 > (unsigned)kStreamMaxCb) return pl;
    if (KB > (unsigned)kStreamXsBlocks && (L + 16 >= TR || L / 8 + 2 > (unsigned)kStreamXsBlocks)) return pl;
    // workgroups that can share a column block: bounded by the accumulator word's count field
    const unsigned sharers = (TR + kStreamWaves * q - 1) / (kStreamWaves * q) + 1;
    if (sharers > (unsigned)kFixedMaxSharers) return pl;
    if ((unsigned long long)problems * NB > (unsigned long long)ws.accum_slots) return pl;
    pl.ok = true;
    pl.problems = problems;
    pl.Gp = Gp;
    pl.q = q;
    pl.rem = rem;
    pl.mq = magic(q);
    pl.mq1 = magic(q + 1);
    pl.mtr = magic(TR);
    return pl;
}

bool gemv_stream_applies(int problems, int size_k, int size_n, bool whole_rows)
{
    if (size_k % 128 != 0 || size_n % 128 != 0) return false;
    const StreamPlan pl = plan_stream(workspace_for_current_device(), problems, size_k, size_n);
    if (!pl.ok) return false;
    return !whole_rows || (unsigned)kStreamWaves * pl.q >= (unsigned)size_k / 16;
}

static std::string run_stream(const Workspace& ws, const StreamPlan& pl, StreamParams& p, int bits, int cb,
                              hipStream_t stream)
{
    throw_pending_device_fault(ws);
    int mask = stream_lut_mask(bits, (unsigned long long)pl.q * kStreamWaves * 256 * bits);
    if (mask != 0) mask = 0xA;          // the one hybrid mask that is instantiated
    p.accum = ws.accum;
    p.fault = ws.fault_dev;
    p.spin_limit = spin_limit();
    p.TR = p.K / 16;
    p.NB = p.N / 128;
    p.Gp = pl.Gp;
    p.mgp = magic((unsigned)pl.Gp);
    p.q = pl.q;
    p.rem = pl.rem;
    p.mq = pl.mq;
    p.mq1 = pl.mq1;
    p.mtr = pl.mtr;
    const dim3 grid((unsigned)(pl.problems * pl.Gp));
    switch (cb) {
    case 0: launch_gemv_stream_cb0(p, bits, mask, grid, stream); break;
    case 1: launch_gemv_stream_cb1(p, bits, mask, grid, stream); break;
    default: launch_gemv_stream_cb2(p, bits, mask, grid, stream); break;
    }
    hip_ok(hipGetLastError(), "exl3_gemv_stream_kernel launch");
    char m[16];
    std::snprintf(m, sizeof m, "0x%x", mask);
    return "exl3_gemv_stream_kernel<" + std::to_string(bits) + "," + std::to_string(cb) + (p.a_up ? ",silu" : "") +
           ",table=" + m + "> grid=" + std::to_string(grid.x) + " block=1024 units_per_wave=" + std::to_string(pl.q) +
           (p.out_fp32 ? " out=f32" : " out=f16");
}

static int wg_per_cu()
{
    const int x = knobs().gemv_wg_per_cu;
    return x > 0 ? x : 6;
}

// split-K factor: about wg_per_cu workgroups per compute unit (2-3 waves per SIMD
// keep the vector ALU busy; each wave then walks several k-blocks with its loads
// one k-block ahead), at most one k-block per wave, within the workspace
static int pick_split(const Workspace& ws, long units, int KB, int mmax, bool trial = false)
{
    const long target_wg = (long)ws.cu_count * wg_per_cu();
    long S = (target_wg + units / 2) / units;
    const int s_max = (KB + 3) / 4;
    if (S > s_max) S = s_max;
    if (S < 1) S = 1;
    const size_t need = (size_t)units * S * mmax * 128 * sizeof(float);
    if (S > 1 && need > ws.partial_bytes && ws.strict) {
        if (trial) return 1 << 30;      // the caller drops this choice
        throw std::runtime_error("exl3 gemv: this launch needs " + std::to_string(need) +
                                 " bytes of split-K scratch; the scratch given holds " + std::to_string(ws.partial_bytes));
    }
    while (S > 1 && (size_t)units * S * mmax * 128 * sizeof(float) > ws.partial_bytes) --S;
    return (int)S;
}

// One-row launches whose whole k-blocks would leave each SIMD at most 1.5 waves (the
// grouped launches of a single token's experts) walk half k-blocks instead: twice the
// waves, each with half the decode.  Measured: the one-token MoE layer gains 1.8 us;
// the attention projections of the dense set (1.9 and 2.5 waves per SIMD, split 10 -> 20)
// lose 1.5 us each to the per-wave fixed work and the longer split-K reduction, so the
// bound sits below them, and the split stays within one batch of the finisher's loads.
static void pick_units(const Workspace& ws, GemvParams& p, long units, int mmax)
{
    const int allow = knobs().gemv_half_units;
    p.half_units = 0;
    if (allow && mmax == 1 && units * p.KB <= (long)ws.cu_count * 6) {
        const int S = pick_split(ws, units, 2 * p.KB, mmax, true);
        if (S <= 16) {
            p.half_units = 1;
            p.S = S;
            return;
        }
    }
    p.S = pick_split(ws, units, p.KB, mmax);
}

std::string launch_gemv(const LinearArgs& a, const Workspace* scratch)
{
    if (a.size_m < 1 || a.size_m > 8) throw std::runtime_error("exl3 gemv: rows must be in 1..=8");
    if (a.size_k % 128 != 0) throw std::runtime_error("exl3 linear: size_k must be a multiple of 128");
    std::optional<LaunchScope> scope;
    if (!scratch) scope.emplace(a.stream);
    const Workspace& ws = scratch ? *scratch : scope->ws;
    throw_pending_device_fault(ws);
    const int mmax = a.size_m == 1 ? 1 : 8;
    if (a.size_m == 1) {
        const StreamPlan pl = plan_stream(ws, 1, a.size_k, a.size_n);
        if (pl.ok) {
            StreamParams sp{};
            sp.a = (const _Float16*)a.a;
            sp.a_up = (const _Float16*)a.a_up;
            sp.lin[0] = {(const uint32_t*)a.trellis, (const _Float16*)a.suh, (const _Float16*)a.svh};
            sp.c[0] = a.c;
            sp.a_had = (_Float16*)a.a_had;
            sp.K = a.size_k;
            sp.N = a.size_n;
            sp.out_fp32 = a.out_fp32;
            if (a.out_add) {
                if (!a.out_fp32) throw std::runtime_error("exl3 gemv: a row is added to an fp32 output only");
                sp.out_add = a.out_add;
            }
            return run_stream(ws, pl, sp, a.k_bits, a.codebook, a.stream);
        }
    }
    if (a.out_add) throw std::runtime_error("exl3 gemv: the added output row needs the one-row streaming kernel");

    GemvParams p{};
    p.a = (const _Float16*)a.a;
    p.lin.trellis = (const uint32_t*)a.trellis;
    p.lin.suh = (const _Float16*)a.suh;
    p.lin.svh = (const _Float16*)a.svh;
    p.a_up = (const _Float16*)a.a_up;
    p.rows = a.size_m;
    p.c[0] = a.c;
    p.a_had = (_Float16*)a.a_had;
    p.partials = ws.partials;
    p.counters = ws.counters;
    p.K = a.size_k;
    p.N = a.size_n;
    p.NB = a.size_n / 128;
    p.KB = a.size_k / 128;
    p.out_fp32 = a.out_fp32;
    if (p.NB > ws.counter_slots) throw std::runtime_error("exl3 gemv: size_n exceeds the split-K counter table");
    p.cstride = counter_stride(ws, p.NB);
    pick_units(ws, p, p.NB, mmax);
    const int grid = p.NB * p.S;
    launch_bits(p, a.k_bits, a.codebook, mmax, dim3(grid), a.stream);
    hip_ok(hipGetLastError(), "exl3_gemv_kernel launch");
    return "exl3_gemv_kernel<" + std::to_string(a.k_bits) + "," + std::to_string(a.codebook) + "," +
           std::to_string(mmax) + (a.a_up ? ",silu" : "") + "> grid=" + std::to_string(grid) + " block=256 split_k=" +
           std::to_string(p.S) + (p.half_units ? "/half" : "") + (a.out_fp32 ? " out=f32" : " out=f16");
}

std::string launch_gemv_pair(const PairArgs& a)
{
    if (a.size_m < 1 || a.size_m > 8) throw std::runtime_error("exl3 gemv: rows must be in 1..=8");
    if (a.size_k % 128 != 0) throw std::runtime_error("exl3 linear: size_k must be a multiple of 128");
    LaunchScope scope(a.stream);
    Workspace& ws = scope.ws;
    throw_pending_device_fault(ws);
    const int mmax = a.size_m == 1 ? 1 : 8;
    if (a.size_m == 1) {
        const StreamPlan pl = plan_stream(ws, 2, a.size_k, a.size_n);
        if (pl.ok) {
            StreamParams sp{};
            sp.a = (const _Float16*)a.a;
            for (int i = 0; i < 2; ++i) {
                sp.lin[i] = {(const uint32_t*)a.trellis[i], (const _Float16*)a.suh[i], (const _Float16*)a.svh[i]};
                sp.c[i] = a.c[i];
            }
            sp.a_had = (_Float16*)a.a_had;
            sp.K = a.size_k;
            sp.N = a.size_n;
            sp.out_fp32 = 0;
            if (a.norm) {
                sp.norm_x = a.norm->x;
                sp.norm_res = a.norm->res;
                sp.norm_res_out = a.norm->res_out;
                sp.norm_weight = (const uint16_t*)a.norm->weight;
                sp.norm_eps = a.norm->epsilon;
                sp.norm_bias = a.norm->constant_bias;
                sp.norm_scale = a.norm->constant_scale;
                sp.norm_weight_bf16 = a.norm->weight_bf16;
            }
            return std::string(a.norm ? "pair,norm " : "pair ") + run_stream(ws, pl, sp, a.k_bits, a.codebook, a.stream);
        }
    }
    if (a.norm) throw std::runtime_error("exl3 gemv: the norm input needs the one-row streaming kernel");
    GemvParams p{};
    p.a = (const _Float16*)a.a;
    p.pair = 1;
    for (int i = 0; i < 2; ++i) {
        p.shared[i].trellis = (const uint32_t*)a.trellis[i];
        p.shared[i].suh = (const _Float16*)a.suh[i];
        p.shared[i].svh = (const _Float16*)a.svh[i];
        p.c[i] = a.c[i];
    }
    p.shared_expert = -1;
    p.rows = a.size_m;
    p.a_had = (_Float16*)a.a_had;
    p.partials = ws.partials;
    p.counters = ws.counters;
    p.K = a.size_k;
    p.N = a.size_n;
    p.NB = a.size_n / 128;
    p.KB = a.size_k / 128;
    p.out_fp32 = 0;
    const long units = 2L * p.NB;
    if (units > kCounters) throw std::runtime_error("exl3 gemv: size_n exceeds the split-K counter table");
    p.cstride = counter_stride(ws, units);
    pick_units(ws, p, units, mmax);
    dim3 grid((unsigned)(p.NB * p.S), 2);
    launch_bits(p, a.k_bits, a.codebook, mmax, grid, a.stream);
    hip_ok(hipGetLastError(), "exl3_gemv_kernel pair launch");
    return "exl3_gemv_kernel<" + std::to_string(a.k_bits) + "," + std::to_string(a.codebook) + "," +
           std::to_string(mmax) + "> pair grid=" + std::to_string(grid.x) + "x2 block=256 split_k=" +
           std::to_string(p.S) + (p.half_units ? "/half" : "") + " out=f16";
}

std::string launch_mgemm(const MgemmArgs& m)
{
    if (m.size_k % 128 != 0) throw std::runtime_error("exl3_mgemm: size_k must be a multiple of 128");
    if (m.size_m > 8) return launch_gemm_bundle(m);
    LaunchScope scope(m.stream);
    Workspace& ws = scope.ws;
    throw_pending_device_fault(ws);
    const bool sliced = m.had_src_list != nullptr;
    const int mmax = m.size_m == 1 ? 1 : 8;
    if (m.host_lists) {
        // the lists are host memory: the problems travel by value in the kernel arguments
        const StreamPlan pl = m.size_m == 1 && m.bszm_out <= kStreamMaxSlices && m.size_n / 128 <= 65535
                                  ? plan_stream(ws, m.bszm_out, m.size_k, m.size_n) : StreamPlan{};
        if (!pl.ok)
            throw std::runtime_error("exl3_mgemm (host lists): serves one row, at most " + std::to_string(kStreamMaxSlices) +
                                     " slices and weights large enough for the streaming kernel; pass device lists to "
                                     "berth_ops_mgemm otherwise");
        StreamParams sp{};
        sp.a = (const _Float16*)m.a;
        sp.a_had = (_Float16*)m.a_had;
        sp.mode = 3;
        sp.in_stride = (!sliced && m.bszm_in > 1) ? m.size_k : 0;
        sp.K = m.size_k;
        sp.N = m.size_n;
        sp.out_fp32 = m.c_fp32;
        const uint64_t* b = (const uint64_t*)m.b_list;
        const uint64_t* su = (const uint64_t*)m.suh_list;
        const uint64_t* sv = (const uint64_t*)m.svh_list;
        for (int i = 0; i < m.bszm_out; ++i) {
            StreamSlice& sl = sp.slice[i];
            sl.trellis = (const uint32_t*)b[i];
            sl.svh = (const _Float16*)sv[i];
            if (sliced) {
                const int src = m.had_src_list[i];
                if (src < 0 || src >= m.num_had_src) throw std::runtime_error("exl3_mgemm (host lists): had_src_list entry out of range");
                if (m.size_n_list[i] < 0 || m.size_n_list[i] > m.size_n || m.size_n_list[i] % 128 != 0)
                    throw std::runtime_error("exl3_mgemm (host lists): size_n_list entry must be a multiple of 128 within size_n");
                sl.suh = (const _Float16*)su[src];
                sl.c = (void*)((const uint64_t*)m.c_ptrs)[i];
                sl.width128 = (uint16_t)(m.size_n_list[i] / 128);
                sl.n_stride = m.n_stride_list[i];
                sl.had_slab = (uint16_t)src;
            } else {
                sl.suh = (const _Float16*)su[i];
                sl.c = (char*)m.c + (size_t)i * m.size_n * (m.c_fp32 ? 4 : 2);
                sl.width128 = (uint16_t)(m.size_n / 128);
                sl.n_stride = m.size_n;
                sl.had_slab = (uint16_t)i;
            }
        }
        return std::string(sliced ? "sliced x" : "uniform x") + std::to_string(m.bszm_out) + " by value " +
               run_stream(ws, pl, sp, m.k_bits, m.codebook, m.stream);
    }
    if (m.size_m == 1) {
        const StreamPlan pl = plan_stream(ws, m.bszm_out, m.size_k, m.size_n);
        if (pl.ok) {
            StreamParams sp{};
            sp.a = (const _Float16*)m.a;
            sp.c[0] = m.c;
            sp.a_had = (_Float16*)m.a_had;
            sp.b_list = (const uint64_t*)m.b_list;
            sp.suh_list = (const uint64_t*)m.suh_list;
            sp.svh_list = (const uint64_t*)m.svh_list;
            sp.c_ptrs = (const uint64_t*)m.c_ptrs;
            sp.size_n_list = m.size_n_list;
            sp.n_stride_list = m.n_stride_list;
            sp.had_src_list = m.had_src_list;
            sp.mode = sliced ? 2 : 1;
            sp.in_stride = (!sliced && m.bszm_in > 1) ? m.size_k : 0;
            sp.K = m.size_k;
            sp.N = m.size_n;
            sp.out_fp32 = m.c_fp32;
            return std::string(sliced ? "sliced x" : "uniform x") + std::to_string(m.bszm_out) + " " +
                   run_stream(ws, pl, sp, m.k_bits, m.codebook, m.stream);
        }
    }
    GemvParams p{};
    p.a = (const _Float16*)m.a;
    p.rows = m.size_m;
    p.c[0] = m.c;
    p.a_had = (_Float16*)m.a_had;
    p.b_list = (const uint64_t*)m.b_list;
    p.suh_list = (const uint64_t*)m.suh_list;
    p.svh_list = (const uint64_t*)m.svh_list;
    p.c_ptrs = (const uint64_t*)m.c_ptrs;
    p.size_n_list = m.size_n_list;
    p.n_stride_list = m.n_stride_list;
    p.had_src_list = m.had_src_list;
    p.multi = sliced ? 2 : 1;
    p.multi_in_rows = (!sliced && m.bszm_in > 1) ? m.size_m : 0;
    p.partials = ws.partials;
    p.counters = ws.counters;
    p.K = m.size_k;
    p.N = m.size_n;
    p.NB = m.size_n / 128;
    p.KB = m.size_k / 128;
    p.out_fp32 = m.c_fp32;
    const long units = (long)m.bszm_out * p.NB;
    if (units > kCounters) throw std::runtime_error("exl3_mgemm: too many (slice, column block) units");
    p.cstride = counter_stride(ws, units);
    pick_units(ws, p, units, mmax);
    dim3 grid((unsigned)(m.bszm_out * p.NB * p.S));
    launch_bits(p, m.k_bits, m.codebook, mmax, grid, m.stream);
    hip_ok(hipGetLastError(), "exl3_gemv_kernel multi launch");
    return "exl3_gemv_kernel<" + std::to_string(m.k_bits) + "," + std::to_string(m.codebook) + "," +
           std::to_string(mmax) + "> " + (sliced ? "sliced" : "uniform") + " x" + std::to_string(m.bszm_out) +
           " grid=" + std::to_string(grid.x) + " block=256 split_k=" + std::to_string(p.S) + (p.half_units ? "/half" : "") +
           (m.c_fp32 ? " out=f32" : " out=f16");
}

std::string launch_gemv_grouped(const GroupedArgs& g)
{
    if (g.size_k % 128 != 0 || g.size_n % 128 != 0)
        throw std::runtime_error("moe grouped linear: sizes must be multiples of 128");
    LaunchScope scope(g.stream);
    Workspace& ws = scope.ws;
    throw_pending_device_fault(ws);
    GemvParams p{};
    p.a = (const _Float16*)g.a;
    p.a_up = (const _Float16*)g.a_up;
    p.gather = g.gather;
    p.gather_div = g.gather_div;
    p.experts = (const ExpertLin*)g.experts;
    p.problems = (const GroupProblem*)g.problems;
    p.num_problems = g.num_problems;
    p.lins_per_expert = g.lins_per_expert;
    p.lin_base = g.lin_base;
    p.shared_expert = g.shared ? g.shared_expert : -1;
    if (g.shared) std::memcpy(p.shared, g.shared, sizeof(p.shared));
    p.c[0] = g.c0;
    p.c[1] = g.c1;
    p.partials = ws.partials;
    p.counters = ws.counters;
    p.K = g.size_k;
    p.N = g.size_n;
    p.NB = g.size_n / 128;
    p.KB = g.size_k / 128;
    p.out_fp32 = g.out_fp32;
    const long units = (long)g.max_problems * g.num_lins * p.NB;
    if (units > kCounters) throw std::runtime_error("moe grouped linear: too many (problem, column block) units");
    p.cstride = counter_stride(ws, units);
    const int mmax = g.single_row ? 1 : 8;
    if (g.route_params) {
        if (!g.single_row || g.a_up || g.gather_div < 1)
            throw std::runtime_error("moe grouped linear: the inline routing serves the one-token gate / up launch");
        p.route = *(const RouteParams*)g.route_params;
        if (g.resolved_out && (g.resolved_lin < 0 || g.resolved_lin >= g.lins_per_expert))
            throw std::runtime_error("moe grouped linear: resolved linear index out of range");
        p.resolved_out = (ExpertLin*)g.resolved_out;
        p.resolved_lin = g.resolved_lin;
    } else if (g.resolved) {
        if (!g.single_row) throw std::runtime_error("moe grouped linear: resolved records serve one-row problems");
        p.resolved = (const ExpertLin*)g.resolved;
    }
    if (g.comb_out) {
        if (!g.single_row || g.num_lins != 1 || !g.out_fp32 || !g.a_up || !g.comb_w || !g.comb_inv || g.comb_k < 1)
            throw std::runtime_error("moe grouped linear: the folded combine needs one-row problems of a silu-input fp32 linear");
        if (units + p.NB > kCounters) throw std::runtime_error("moe grouped linear: too many units for the folded combine");
        p.comb_w = g.comb_w;
        p.comb_inv = g.comb_inv;
        p.comb_shared = g.comb_shared;
        p.comb_out = g.comb_out;
        p.cstride = counter_stride(ws, units + p.NB);
        p.comb_counters = ws.counters + (size_t)units * p.cstride;
        p.comb_k = g.comb_k;
    }
    pick_units(ws, p, units, mmax);
    if (g.comb_out && g.comb_single) {
        if (g.max_problems > kCombMaxProblems || g.comb_k > kCombMaxProblems || g.comb_shared_prob >= g.max_problems)
            throw std::runtime_error("moe grouped linear: the single hand-over serves at most " +
                                     std::to_string(kCombMaxProblems) + " problems");
        const size_t part_floats = (size_t)units * p.S * 128;
        if ((part_floats + (size_t)units * 64) * 4 > ws.partial_bytes)
            throw std::runtime_error("moe grouped linear: split-K workspace too small for the single hand-over");
        p.comb_sv = (uint32_t*)(ws.partials + part_floats);
        p.comb_shared_prob = g.comb_shared_prob;
    }
    dim3 grid((unsigned)(g.max_problems * p.NB * p.S), (unsigned)g.num_lins);
    launch_bits(p, g.k_bits, g.codebook, mmax, grid, g.stream);
    hip_ok(hipGetLastError(), "exl3_gemv_kernel grouped launch");
    return "exl3_gemv_kernel<" + std::to_string(g.k_bits) + "," + std::to_string(g.codebook) + "," +
           std::to_string(mmax) + "> grouped grid=" +
           std::to_string(grid.x) + "x" + std::to_string(grid.y) + " split_k=" + std::to_string(p.S) + (p.half_units ? "/half" : "") +
           (g.comb_out ? (p.comb_sv ? " +combine(one hand-over)" : " +combine") : "") + (g.route_params ? " +route" : "") +
           (g.resolved ? " resolved" : "");
}

}  // namespace berth

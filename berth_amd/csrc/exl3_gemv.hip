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
#include "exl3_gemv_kernel.cuh"
#include "launch.h"

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

static int wg_per_cu()
{
    static const int v = [] {
        const char* e = std::getenv("BERTH_GEMV_WG_PER_CU");
        int x = e ? std::atoi(e) : 0;
        return x > 0 ? x : 6;
    }();
    return v;
}

// split-K factor: about wg_per_cu workgroups per compute unit (2-3 waves per SIMD
// keep the vector ALU busy; each wave then walks several k-blocks with its loads
// one k-block ahead), at most one k-block per wave, within the workspace
static int pick_split(const Workspace& ws, long units, int KB, int mmax)
{
    const long target_wg = (long)ws.cu_count * wg_per_cu();
    long S = (target_wg + units / 2) / units;
    const int s_max = (KB + 3) / 4;
    if (S > s_max) S = s_max;
    if (S < 1) S = 1;
    while (S > 1 && (size_t)units * S * mmax * 128 * sizeof(float) > kPartialBytes) --S;
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
    static const int allow = [] {
        const char* e = std::getenv("BERTH_GEMV_HALF_UNITS");
        return e ? std::atoi(e) : 1;
    }();
    p.half_units = 0;
    if (allow && mmax == 1 && units * p.KB <= (long)ws.cu_count * 6) {
        const int S = pick_split(ws, units, 2 * p.KB, mmax);
        if (S <= 16) {
            p.half_units = 1;
            p.S = S;
            return;
        }
    }
    p.S = pick_split(ws, units, p.KB, mmax);
}

std::string launch_gemv(const LinearArgs& a)
{
    if (a.size_m < 1 || a.size_m > 8) throw std::runtime_error("exl3 gemv: rows must be in 1..=8");
    if (a.size_k % 128 != 0) throw std::runtime_error("exl3 linear: size_k must be a multiple of 128");
    Workspace& ws = workspace_for_current_device();
    const int mmax = a.size_m == 1 ? 1 : 8;

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
    if (p.NB > kCounters) throw std::runtime_error("exl3 gemv: size_n exceeds the split-K counter table");
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
    Workspace& ws = workspace_for_current_device();
    const int mmax = a.size_m == 1 ? 1 : 8;
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
    if (m.size_m > 8) throw std::runtime_error("exl3_mgemm: more than 8 rows is not built (use one linear per call)");
    Workspace& ws = workspace_for_current_device();
    const bool sliced = m.had_src_list != nullptr;
    const int mmax = m.size_m == 1 ? 1 : 8;
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
    Workspace& ws = workspace_for_current_device();
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
    const int mmax = g.single_row ? 1 : 8;
    if (g.comb_out) {
        if (!g.single_row || g.num_lins != 1 || !g.out_fp32 || !g.a_up || !g.comb_w || !g.comb_inv || g.comb_k < 1)
            throw std::runtime_error("moe grouped linear: the folded combine needs one-row problems of a silu-input fp32 linear");
        if (units + p.NB > kCounters) throw std::runtime_error("moe grouped linear: too many units for the folded combine");
        p.comb_w = g.comb_w;
        p.comb_inv = g.comb_inv;
        p.comb_shared = g.comb_shared;
        p.comb_out = g.comb_out;
        p.comb_counters = ws.counters + units;
        p.comb_k = g.comb_k;
    }
    pick_units(ws, p, units, mmax);
    dim3 grid((unsigned)(g.max_problems * p.NB * p.S), (unsigned)g.num_lins);
    launch_bits(p, g.k_bits, g.codebook, mmax, grid, g.stream);
    hip_ok(hipGetLastError(), "exl3_gemv_kernel grouped launch");
    return "exl3_gemv_kernel<" + std::to_string(g.k_bits) + "," + std::to_string(g.codebook) + "," +
           std::to_string(mmax) + "> grouped grid=" +
           std::to_string(grid.x) + "x" + std::to_string(grid.y) + " split_k=" + std::to_string(p.S) + (p.half_units ? "/half" : "") +
           (g.comb_out ? " +combine" : "");
}

}  // namespace berth

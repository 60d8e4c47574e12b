// Internal C++ interface between the C-ABI entry points and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdlib>
#include <stdexcept>
#include <string>

namespace berth {

inline void hip_ok(hipError_t e, const char* what)
{
    if (e != hipSuccess)
        throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// Raises the dynamic-LDS limit of a kernel once per device (the attribute is kept per
// device; a function-local static would set it on the first device only).
inline void raise_dynamic_lds_limit(const void* kernel, int bytes, bool (&done)[64], const char* what)
{
    int device = 0;
    hip_ok(hipGetDevice(&device), "hipGetDevice");
    if (device < 0 || device >= 64 || done[device]) return;
    hip_ok(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes), what);
    done[device] = true;
}

// Per-device scratch owned by the library, allocated on first use and kept for
// the life of the process: split-K partial sums and their arrival counters
// (the role of the fixed workspace of
// crates/berth-kernels/csrc/int8_sq.cu:20-47).
struct Workspace {
    float* partials = nullptr;      // kPartialBytes
    unsigned* counters = nullptr;   // kCounters entries, zero between launches
    unsigned long long* accum = nullptr;   // zero between launches: fixed-point column-block sums of the streaming GEMV
    int accum_slots = 0;            // column blocks (1 KiB each) behind `accum`
    int device = -1;
    int cu_count = 0;
    // One word of host-pinned memory that kernels can write (device address fault_dev, host
    // address fault_host): a split-K finisher that gives up its bounded wait stores a code
    // there; the next launch of such a kernel on the device reports it and clears it.
    unsigned* fault_dev = nullptr;
    volatile unsigned* fault_host = nullptr;
    size_t partial_bytes = 0;       // capacity of `partials`
    int counter_slots = 0;          // most counters a launch may use
    size_t counter_words = 0;       // words behind `counters` (counters can be spread over them)
    bool strict = false;            // true: a launch that would not fit is refused instead of split less
    // the stream of the device's previous launch, and the event later launches on other streams wait for
    hipStream_t last_stream = nullptr;
    bool have_last = false;
    bool multi_stream = false;      // events are being recorded behind every launch
    bool event_recorded = false;
    int same_stream_run = 0;
    hipEvent_t order_event = nullptr;
};
constexpr size_t kPartialBytes = (size_t)256 << 20;
constexpr int kCounters = 65536;
constexpr int kAccumSlots = 16384;     // column blocks of a streaming launch (16 MiB of accumulators)
// The BERTH_* environment knobs, read once per process into one record; no launch calls
// getenv.  berth_kernels_reload_env() reads them again (tests that switch a knob inside one
// process call it after changing the environment).
struct Knobs {
    int gemv_stream;            // BERTH_GEMV_STREAM            0: never take the streaming kernel
    int gemv_stream_min_units;  // BERTH_GEMV_STREAM_MIN_UNITS  fewest tile rows per wave for which it is taken
    int gemv_stream_shrink;     // BERTH_GEMV_STREAM_SHRINK     1: fewer workgroups instead of falling back
    int gemv_stream_wgs;        // BERTH_GEMV_STREAM_WGS        cap on the workgroups per problem (0: none)
    int gemv_stream_lut;        // BERTH_GEMV_STREAM_LUT        table mask of the hybrid decode (-1: by size)
    int gemv_wg_per_cu;         // BERTH_GEMV_WG_PER_CU         workgroups per compute unit of the 1..8-row kernel
    int gemv_half_units;        // BERTH_GEMV_HALF_UNITS        0: never walk half k-blocks
    int gemv_max_rows;          // BERTH_GEMV_MAX_ROWS          rows up to this count take the VALU kernel (1..8)
    int gemm_wg_per_cu;         // BERTH_GEMM_WG_PER_CU
    int gemm_balanced;          // BERTH_GEMM_BALANCED
    int gemm_rows256;           // BERTH_GEMM_ROWS256
    int counter_stride;         // BERTH_COUNTER_STRIDE         cap on the words between arrival counters (1..32)
    int moe_big_min;            // BERTH_MOE_BIG_MIN
    int moe_route_slab;         // BERTH_MOE_ROUTE_SLAB: 0 keeps the two-launch routing of many tokens
    int moe_fold_combine;       // BERTH_MOE_FOLD_COMBINE
    int moe_inline_route;       // BERTH_MOE_INLINE_ROUTE
    int moe_resolved;           // BERTH_MOE_RESOLVED
    unsigned spin_limit;        // BERTH_SPIN_LIMIT             polls of a bounded wait before it gives up
    int stream_order;           // BERTH_STREAM_ORDER           0: launches of different streams are not ordered
};
const Knobs& knobs();
void reload_knobs();

// Words between the arrival counters of a one-row launch that needs `units` of them: as far
// apart as the table allows, up to one counter per 128 bytes.  Neighbouring words send the
// arrivals of a whole launch (hundreds within a microsecond) through one atomic unit: measured,
// counters 32 bytes or more apart take 1.8 us off the four launches of a 27B layer set and
// 2.9 us off the one-token MoE layer, and 32 bytes .. 16 KiB apart all measure the same.
// Every launch leaves the counters it used at zero, so launches with different strides can
// follow each other.  (BERTH_COUNTER_STRIDE caps the stride; 1 packs the counters.)
inline int counter_stride(const Workspace& ws, long units)
{
    const int cap = knobs().counter_stride;
    int stride = 1;
    while (stride * 2 <= cap && units * stride * 2 <= (long)ws.counter_words) stride *= 2;
    return stride;
}
Workspace& workspace_for_current_device();
// The workspace serves one launch at a time per device.  Launches of one stream are ordered
// by the stream; a launch that arrives on another stream than the device's previous one must
// not start while that one may still be running, or the two mix their partial sums and
// counters.  LaunchScope, held by a launcher around its launches, sees to that without ever
// touching the previous stream's handle (its owner may have destroyed it): the first time the
// stream changes the device is drained once; from then on every scope records an event behind
// its launches and a launch on another stream waits for that event.  After 32 launches in
// a row on one stream the events stop again (each costs the device about 2.7 us), so a
// single-stream caller pays nothing and a rare change of stream pays one drain.  Streams
// that are being captured into a graph are left alone.
struct LaunchScope {
    explicit LaunchScope(hipStream_t stream);
    ~LaunchScope();
    LaunchScope(const LaunchScope&) = delete;
    LaunchScope& operator=(const LaunchScope&) = delete;
    Workspace& ws;
    hipStream_t stream;
    bool record = false;
};
// throws if a kernel of an earlier launch on this device reported a fault (and clears the report)
void throw_pending_device_fault(const Workspace& ws);
// polls a split-K finisher spends on its wait before it gives up (BERTH_SPIN_LIMIT, default 2^20)
inline unsigned spin_limit() { return knobs().spin_limit; }

struct LinearArgs {
    const void* a;
    const void* trellis;
    void* c;
    const void* suh;
    void* a_had;
    const void* svh;
    int size_m, size_k, size_n, k_bits, codebook, out_fp32;
    hipStream_t stream;
    const void* a_up = nullptr;   // VALU kernel only: the input is silu(a) * a_up, element by element
    const float* out_add = nullptr;   // streaming kernel only (one row, fp32 output): a row added to the output
};

// RMS norm with the residual added first, as the input of a launch of the streaming kernel
// (the arithmetic of berth_ops_rms_norm_res_in; the sum goes to res_out, which aliases neither)
struct NormInput {
    const float* x;             // fp32 [K]
    const float* res;           // fp32 [K]
    float* res_out;             // fp32 [K]
    const void* weight;         // fp16 or bf16 [K]
    float epsilon, constant_bias, constant_scale;
    int weight_bf16;
};

// two linears of one shape on the same input rows in one launch (gate and up of an MLP)
struct PairArgs {
    const void* a;
    const void* trellis[2];
    const void* suh[2];
    const void* svh[2];
    void* c[2];                 // fp16 [size_m][size_n] each
    void* a_had;                // [size_m][size_k]
    int size_m, size_k, size_n, k_bits, codebook;
    hipStream_t stream;
    const NormInput* norm = nullptr;    // one row, streaming kernel only: `a` is then unused
};
std::string launch_gemv_pair(const PairArgs& args);
// whether a one-row launch of `problems` linears of this shape takes the streaming kernel (and,
// with whole_rows, whether every workgroup of it then holds the whole input row)
bool gemv_stream_applies(int problems, int size_k, int size_n, bool whole_rows);

// grouped (MoE) launches: problems, experts and num_problems are device memory
struct GroupedArgs {
    const void* a;              // input rows (fp16); with a_up the input is silu(a) * a_up
    const void* a_up;
    const int32_t* gather;      // optional: source row = gather[r] / gather_div
    int gather_div;
    const void* experts;        // ExpertLin[num_experts * lins_per_expert]
    const void* shared;         // host: three {trellis, suh, svh} of the always-on expert, or null
    int shared_expert;          // expert index the problem list uses for it (-1: none)
    int single_row;             // every problem has exactly one row
    int mb;                     // MFMA path: rows per problem / 32 (1 or 4)
    const void* problems;       // GroupProblem[max_problems]
    const int* num_problems;
    int max_problems;
    // MFMA path, optional: problems of up to 128 rows that run in the same launch, ahead of
    // `problems` (which then hold at most 32 rows each)
    const void* big_problems = nullptr;
    const int* num_big = nullptr;
    int max_big = 0;
    int lins_per_expert, lin_base, num_lins;   // num_lins 1 or 2 consecutive linears per launch
    void* c0;
    void* c1;
    const void* a_had;          // MFMA path: rotated input rows [rows][K] of the first linear
    const void* a_had2;         // ... and of the second linear of the launch
    int size_k, size_n, k_bits, codebook, out_fp32;
    hipStream_t stream;
    // VALU path, single_row, one linear, fp32 out, silu input: also combine the
    // problems' rows into comb_out[size_n] (weights comb_w[comb_k], rows
    // comb_inv[comb_k] of c0, start value comb_shared[size_n] or zero)
    // VALU path, single_row, first launch of a one-token layer: RouteParams of the routing whose
    // last part every workgroup redoes for itself (the problem list does not exist yet)
    const void* route_params = nullptr;
    const float* comb_w = nullptr;
    const int32_t* comb_inv = nullptr;
    const float* comb_shared = nullptr;
    float* comb_out = nullptr;
    int comb_k = 0;
    // comb_single: split-K and combine share one hand-over (at most sixteen problems, problem i
    // writing row i); comb_shared_prob is then the problem whose row starts the chain, or -1
    // when comb_shared (a row written by an earlier launch, or null) does
    int comb_single = 0;
    int comb_shared_prob = -1;
    // with route_params: where the launch's first workgroup leaves {trellis, suh, svh} of linear
    // `resolved_lin` of the experts in sorted order (then the always-on one), or null.
    // `resolved` (single_row, no route_params): those records, read instead of the problem
    // list and the expert table; the launch then holds exactly max_problems problems.
    void* resolved_out = nullptr;
    int resolved_lin = 0;
    const void* resolved = nullptr;
};
std::string launch_gemv_grouped(const GroupedArgs& args);
std::string launch_gemm_grouped(const GroupedArgs& args);

// multi-linear launch (crates/berth-kernels/src/ops.rs:247-367); every list is a device array
struct MgemmArgs {
    const void* a;
    const void* b_list;
    void* c;
    const void* suh_list;
    void* a_had;
    const void* svh_list;
    int size_m, size_k, size_n, k_bits, codebook, c_fp32, bszm_in, bszm_out;
    const int* size_n_list;
    const void* c_ptrs;
    const int* n_stride_list;
    const int* had_src_list;
    int num_had_src;
    hipStream_t stream;
    bool host_lists = false;    // the seven lists are host memory (one row, the streaming kernel only)
};
std::string launch_mgemm(const MgemmArgs& args);
// more than 8 rows: the bundle as one dense MFMA launch
std::string launch_gemm_bundle(const MgemmArgs& args);
// out slab s = Hh(in(s) * suh(s)) for s < slabs (fp16; in(s) = in + s * in_stride, out slabs
// out_stride elements apart, or at out_host[s] when that is given with a null list); suh(s) from
// the device list, or from the host array when the list is null
std::string launch_had_r_128_slabs(const void* in, size_t in_stride, void* out, size_t out_stride, const void* suh_list,
                                   const void* const* suh_host, int slabs, int rows, int cols, hipStream_t stream,
                                   void* const* out_host = nullptr);
// gate and up of an MLP above 8 rows as one bundle: two linears of one shape on one input, each
// with its own output and its own buffer for the rotated input
std::string launch_gemm_pair(const PairArgs& pair, void* a_had_second);
constexpr int kBundleMaxSlices = 16;    // slices of a bundle whose lists travel by value

// rows 1..8: VALU dot-product kernel.  Returns the launch description.  `scratch`: the
// split-K scratch to use instead of the device's lazily allocated workspace.
std::string launch_gemv(const LinearArgs& args, const Workspace* scratch = nullptr);
// any row count: fp16 MFMA kernel (rows padded to 32 inside the kernel).
std::string launch_gemm(const LinearArgs& args);
// trellis -> fp16 [K][slice_n] (row stride slice_n), columns n_offset.. of a
// [K][full_n] weight
std::string launch_reconstruct(void* unpacked, const void* packed, int size_k, int slice_n,
                               int full_n, int n_offset, int k_bits, int codebook,
                               hipStream_t stream);
// trellis -> fp16 effective weight (both Hadamards and sign scales folded in)
std::string launch_reconstruct_had(void* unpacked, const void* packed, const void* suh, const void* svh,
                                   int size_k, int slice_n, int full_n, int n_offset, int k_bits, int codebook,
                                   hipStream_t stream);
// per row, per 128 columns: Hadamard with pre- or post-scale
std::string launch_had_r_128(const void* in, void* out, const void* scale, int pre_scale,
                             int rows, int cols, int fp32, hipStream_t stream);
std::string launch_add_f32(const void* a, const void* b, void* c, int n, hipStream_t stream);
std::string launch_add_bias(void* c, const void* bias, int rows, int n, int c_fp32, hipStream_t stream);
std::string launch_rms_norm(const void* x, const void* weight, void* y, void* residual, int rows, int dim,
                            float epsilon, float constant_bias, float constant_scale, int weight_bf16,
                            hipStream_t stream);
std::string launch_rms_norm_f16(const void* x, const void* weight, void* y, int rows, int dim, float epsilon,
                                float constant_bias, float constant_scale, hipStream_t stream);
std::string launch_embed_tokens(const void* weight, const int* ids, void* out, int hidden, int n, int f16,
                                hipStream_t stream);
std::string launch_cat_f16_last(const void* embedding, const void* hidden, void* out, int rows, int width,
                                hipStream_t stream);
std::string launch_unpack_signs(const void* packed, void* out, int64_t words, hipStream_t stream);
std::string launch_silu_mul(const void* gate, const void* up, void* out, int64_t numel,
                            float act_limit, hipStream_t stream);
std::string launch_hgemm(const void* a, const void* b, void* c, int m, int k, int n, int ldc,
                         int c_fp32, hipStream_t stream);

}  // namespace berth

/*
 * berth_kernels_hip.h — C ABI of libberth_kernels_hip.so (MI355X / gfx950).
 *
 * Drop-in for the `extern "C"` surface the reference's berth-kernels crate binds
 * for the EXL3 linear path.  Each declaration cites the reference interface it
 * replaces.  Conventions, all taken from the reference
 * (crates/berth-kernels/src/lib.rs:88-133,179-192; csrc/linear.cu:362-404):
 *   - every pointer is a raw device address; the caller owns every buffer;
 *   - `stream` is a hipStream_t passed as void*, NULL = the default stream;
 *     launches are asynchronous on it and never synchronise;
 *   - return 0 on success, -1 on error; the message is a thread-local C string
 *     (`*_last_error`) valid until the next call of the same family on the
 *     thread and empty after a success; `*_last_launch` names the kernel that
 *     ran and is empty after a failure;
 *   - argument validation happens before any device call; C++ exceptions never
 *     cross this boundary; bias is not applied;
 *   - the library owns lazily allocated per-device internals (a 256 MiB split-K
 *     workspace and its counters) that are never freed or grown; concurrent
 *     launches on one device are not serialised and share that workspace.
 */
#ifndef BERTH_KERNELS_HIP_H
#define BERTH_KERNELS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* codebook: 0 default (3INST), 1 mcg, 2 mul1 — crates/berth-kernels/src/lib.rs:54-63 */

/* ---- single linear, the decode shim --------------------------------------
 * replaces crates/berth-kernels/src/ffi.rs:7-21 / csrc/linear.cu:362-394.
 * a fp16 [size_m][size_k]; trellis int16 [size_k/16][size_n/16][16*k_bits];
 * c fp16|fp32 [size_m][size_n]; suh fp16 [size_k]; a_had fp16 [size_m][size_k]
 * (written); svh fp16 [size_n].  size_k % 128 == 0, size_n % 128 == 0,
 * k_bits 1..8, any size_m >= 1. */
int berth_exl3_linear(const void* a, const void* trellis, void* c, const void* suh,
                      void* a_had, const void* svh, int size_m, int size_k, int size_n,
                      int k_bits, int codebook, int out_fp32, void* stream);
/* The same operator for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference (its shim allocates its workspace lazily, crates/berth-kernels/src/lib.rs:116-117).
 * Allocates nothing: the split-K partial sums and arrival counters live in a fixed array
 * inside the library (8 MiB + 256 KiB per GPU, held until the process ends).  Same arguments
 * and conventions as berth_exl3_linear, with these limits: size_m <= 8; a launch whose
 * split-K partial sums would not fit the 8 MiB is refused with an error (no weight of the
 * shapes named in this header's tests comes near it at one row); size_n / 128 <= 65536.
 * Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams)
 * race, as overlapping calls of berth_exl3_linear do on the library's workspace. */
int berth_exl3_linear_noalloc(const void* a, const void* trellis, void* c, const void* suh,
                              void* a_had, const void* svh, int size_m, int size_k, int size_n,
                              int k_bits, int codebook, int out_fp32, void* stream);
const char* berth_exl3_last_error(void);   /* ffi.rs:23, linear.cu:396 */
const char* berth_exl3_last_launch(void);  /* ffi.rs:24, linear.cu:401 */

/* Host-only symbols of the reference boundary, kept so that the unchanged crate links and
 * its known-answer tests hold; nothing on this device consumes their results.
 * tune keys (crates/berth-kernels/src/ffi.rs:33-46, src/ops.rs:40-53; csrc/linear.cu:347-360,
 * csrc/ops/mgemm.cu:276-294, csrc/autotune.cu:61-66): the reference's shape-tuner cache keys.
 * gemv_cfg (crates/berth-kernels/src/prefill_lin.rs:69-78, csrc/prefill_lin/gemv.cu:71-99):
 * which QTIP GEMV configuration the reference's rows-2..8 route would take (0, 1, or -1).
 * smoke (ffi.rs:29-30, csrc/linear.cu:404-465): one small one-row linear on buffers the
 * function allocates and frees itself (4 bpw 128x256, and 6 bpw 128x512); 0 on success. */
uint64_t berth_exl3_gemm_tune_key(int size_m, int size_k, int size_n, int k_bits, int out_fp32, int device,
                                  int cc, int sms, int codebook);
uint64_t berth_exl3_salt_hash(uint64_t hash);
uint64_t berth_ops_mgemm_tune_key(int size_m, int size_k, int size_n, int k_bits, int c_fp32, int device, int cc,
                                  int sms, int codebook, int bszm_in, int bszm_out, int sliced);
int berth_exl3_gemv_cfg(int cc, int size_m, int size_k, int size_n, int k_bits, int codebook, int mode,
                        int narrow_coresident);
int berth_exl3_smoke_int8(int out_fp32);
int berth_exl3_smoke_gemm(void);

/* No counterpart in the reference (its shim allocates lazily, crates/berth-kernels/src/lib.rs:116-117):
 * allocates the per-device internals of `device` now rather than inside the first launch,
 * which would otherwise allocate and synchronise (and fail under stream capture). */
int berth_kernels_init(int device);

/* Diagnostics, no counterpart in the reference: the per-device internals of the current
 * device (allocated by this call if no launch has done so yet): the split-K partial-sum
 * workspace and the arrival-counter table (zero between launches).  Any out pointer may be
 * NULL.  The internals serve one launch at a time per device: launches that overlap on two
 * streams mix their partial sums and counters.  A tile finisher of the MFMA kernels that
 * finds its counters inconsistent gives up after a bounded wait (BERTH_SPIN_LIMIT polls,
 * default 2^20), leaves its tile unwritten and the next call that would launch an MFMA
 * kernel on the device returns -1 with that report instead of launching. */
int berth_kernels_workspace(void** partials, size_t* partial_bytes, void** counters, int* counter_slots);

/* Diagnostics, no counterpart in the reference: the one-row streaming GEMV's column-block
 * accumulators of the current device, `slots` blocks of 128 64-bit words that every launch
 * leaves at zero (value in units of 2^-18 in bits 16..63, contributions that did not fit in
 * bits 8..15, contributions in bits 0..7). */
int berth_kernels_accumulators(void** accum, int* slots);

/* No counterpart in the reference.  Host-only query for the caller's synchronisation points:
 * 0 when no kernel on `device` has reported a fault since the last report, else the fault
 * code, and the report is cleared (-1: no such device).  A bounded wait inside a kernel that
 * gives up stores its code in a host-visible word; launches on the device check the word too
 * and fail with the report, but a caller that synchronises and launches nothing of this library
 * afterwards learns of it only here.  Codes below 0x40000000: 1 + the tile an MFMA split-K
 * finisher left unwritten; from 0x40000001: 0x40000001 + the column block a streaming GEMV
 * launch left unwritten (contributions left over in its accumulator) or filled with NaN (a
 * contribution missing). */
long long berth_kernels_pending_fault(int device);

/* No counterpart in the reference.  The BERTH_* environment knobs are read once per process;
 * this reads them again (for tests that switch a knob inside one process).  Not to be called
 * while another thread is launching. */
void berth_kernels_reload_env(void);

/* crates/berth-kernels/csrc/linear.cu:301-332.  cc is the gfx target number
 * (950 on MI355X); sms is the compute-unit count. */
int berth_device_cc(int device);
int berth_device_sms(int device);

/* ---- rows > 1, the prefill shim -------------------------------------------
 * replaces crates/berth-kernels/src/prefill_lin.rs:36-79 /
 * csrc/prefill_lin/linear.cu:348-430.  Same tensors as above; w_scratch (fp16,
 * size_k * min(size_n, 32768)) must be non-NULL when size_m > 144 as in the
 * reference contract, though this implementation decodes inside the GEMM and
 * does not write it. */
int berth_prefill_exl3_linear(const void* a, const void* trellis, void* c, const void* suh,
                              void* a_had, const void* svh, void* w_scratch, int size_m,
                              int size_k, int size_n, int k_bits, int codebook, int c_fp32,
                              void* stream);
/* C[m][ldc] (fp16|fp32) = A[m][k] @ B[k][n], fp16 operands, fp32 accumulate */
int berth_prefill_hgemm(const void* a, const void* b, void* c, int size_m, int size_k,
                        int size_n, int ldc, int c_fp32, void* stream);
const char* berth_prefill_last_error(void);
const char* berth_prefill_last_launch(void);

/* The reference keeps these three internal (C++ linkage,
 * crates/berth-kernels/csrc/prefill_lin/api.h, reconstruct.cu:31-123); they are
 * exported here because the dequantised weight is a parity target of its own.
 * reconstruct: unpacked fp16 [size_k][slice_n] = columns n_offset.. of the
 * decoded [size_k][full_n] inner weight.  reconstruct_had (reconstruct.cu:96-123,
 * the reference's weight for 1024 rows and more): the same slice of the
 * EFFECTIVE weight diag(suh) * Hh * W * Hh * diag(svh) per 128 x 128 block, so
 * that a plain GEMM a @ unpacked is the operator's output; suh fp16 [size_k],
 * svh fp16 [full_n] (the slice's part is taken at n_offset); size_k % 128 == 0.
 * had_r_128: per row and 128 columns, out = Hh(in*scale) when pre_scale, else
 * Hh(in)*scale; fp32 selects float tensors. */
int berth_prefill_reconstruct(void* unpacked, const void* packed, int size_k, int slice_n,
                              int full_n, int n_offset, int k_bits, int codebook, void* stream);
int berth_prefill_reconstruct_had(void* unpacked, const void* packed, const void* suh, const void* svh,
                                  int size_k, int slice_n, int full_n, int n_offset, int k_bits,
                                  int codebook, void* stream);
int berth_prefill_had_r_128(const void* input, void* output, const void* scale, int pre_scale,
                            int rows, int cols, int fp32, void* stream);

/* ---- packed signs --------------------------------------------------------------
 * replaces crates/berth-exl3/src/signs.rs:25-46 for tensors that are already on
 * the device: packed su / sv (little-endian u16 words, bit i of a word = element
 * i, set = -1.0) -> fp16 signs, 16 per word.  packed_bytes must be even (the
 * reference's error text otherwise); errors and launch text go to
 * berth_exl3_last_error / berth_exl3_last_launch. */
int berth_exl3_unpack_signs(const void* packed, void* out, int64_t packed_bytes, void* stream);

/* ---- ops -------------------------------------------------------------------
 * replaces crates/berth-kernels/src/ops.rs:82-90 / csrc/ops/act.cu:35-69:
 * out = silu(gate) * up, fp16, numel even, act_limit 0 = no clamp; out may
 * alias up. */
int berth_ops_silu_mul(const void* gate, const void* up, void* out, int64_t numel,
                       float act_limit, void* stream);
/* replaces crates/berth-kernels/src/ops.rs:55-80,398-500 / csrc/ops/norm.cu:128-225: RMS norm
 * of fp32 rows to fp16, y = rms(x) * (weight + constant_bias) * constant_scale with rms =
 * 1/sqrt(mean(x^2) + epsilon); weight fp16 (weight_bf16 0) or bf16 (1), dim a multiple of
 * 4.  _res_in first adds x into the fp32 residual in place and normalises the sum. */
int berth_ops_rms_norm(const void* x, const void* weight, void* y, int rows, int dim, float epsilon,
                       float constant_bias, float constant_scale, int weight_bf16, void* stream);
int berth_ops_rms_norm_res_in(const void* x, const void* weight, void* y, void* residual, int rows, int dim,
                              float epsilon, float constant_bias, float constant_scale, int weight_bf16,
                              void* stream);
/* replaces crates/berth-kernels/src/ops.rs:91-97,522-552 / csrc/ops/add.cu: c = a + b, fp32,
 * n elements; c may alias a. */
int berth_ops_add_f32(const void* a, const void* b, void* c, int n, void* stream);
/* No counterpart in the reference, whose engine refuses a linear that carries a bias
 * (crates/berth-engine/src/mlp.rs:67-75, attn.rs:867-869; the tensor itself is classified at
 * crates/berth-exl3/src/linear.rs:131-133,219-231).  c[rows][n] += bias[n]: c is a linear's output
 * as written (fp16, or fp32 when c_fp32), bias fp32; the sum is formed in fp32 and rounded once. */
int berth_ops_add_bias(void* c, const float* bias, int rows, int n, int c_fp32, void* stream);
/* replaces crates/berth-kernels/src/ops.rs:108-118,600-640 / csrc/ops/norm.cu:80-112,163-190: the
 * same norm for fp16 rows with a bf16 weight, fp16 out, no residual. */
int berth_ops_rms_norm_f16(const void* x, const void* weight, void* y, int rows, int dim, float epsilon,
                           float constant_bias, float constant_scale, void* stream);
/* The remaining device entries of the reference's ops module, glue either side of the
 * linear path, so that the unchanged Rust module links (crates/berth-kernels/src/ops.rs:99-143 /
 * csrc/ops/embed.cu, csrc/ops/copy.cu): embedding rows bf16 [vocab][hidden] -> fp32 (exact
 * widen) or fp16 (one rounding) for n token ids (not range-checked); device-to-device copy;
 * out[row] = embedding[row] ++ hidden[row] in fp16. */
int berth_ops_embed_tokens(const void* weight, const int* ids, void* out, int hidden, int n, void* stream);
int berth_ops_embed_tokens_f16(const void* weight, const int* ids, void* out, int hidden, int n, void* stream);
int berth_ops_memcpy_d2d(void* dst, const void* src, unsigned long long bytes, void* stream);
int berth_ops_cat_f16_last(const void* embedding, const void* hidden, void* out, int rows, int hidden_size,
                           void* stream);
/* replaces crates/berth-kernels/src/ops.rs:17-38,247-367 / csrc/ops/mgemm.cu:296-340:
 * several EXL3 linears in one launch.  Every list is a DEVICE array.  Sliced
 * mode (all four slice lists given, bszm_in == 1): bszm_out slices sharing the
 * input a [size_m][size_k]; b_list[s] = trellis of the source advanced to the
 * slice's first tile column; suh_list[src] per source (num_had_src of them);
 * svh_list[s] = svh + n0; c_ptrs[s] = output + n0 with row stride
 * n_stride_list[s] (the source's full N, also the trellis row stride);
 * size_n_list[s] <= size_n = slice width; had_src_list[s] = source index;
 * a_had holds num_had_src slabs of size_m*size_k.  Uniform mode (lists NULL):
 * bszm_out linears of one shape, inputs a[i] (bszm_in == bszm_out) or a[0]
 * (bszm_in == 1), outputs c[i] contiguous.  Any row count: up to 8 rows run the
 * dot-product kernels (the rotation of the input inside the launch), more rows one
 * launch that rotates the input once per source / linear and one dense MFMA launch
 * over all slices (the reference sends 9..32 rows of its fused q/k/v and gate/up
 * bundles through this call, crates/berth-engine/src/prefill.rs:81-85).  Returns 1
 * on success (the reference returns its kernel-shape tag there), -1 on error. */
int berth_ops_mgemm(const void* a, const void* b_list, void* c, const void* suh_list, void* a_had,
                    const void* svh_list, int size_m, int size_k, int size_n, int k_bits,
                    int codebook, int c_fp32, int bszm_in, int bszm_out, const int* size_n_list,
                    const void* c_ptrs, const int* n_stride_list, const int* had_src_list,
                    int num_had_src, void* stream);
/* No counterpart in the reference: berth_ops_mgemm with its lists in HOST memory (b_list,
 * suh_list, svh_list and c_ptrs arrays of device addresses as uint64, the three int lists as
 * ints; a, c and a_had stay device pointers).  For callers that built the lists themselves and
 * still hold them: the problems then travel by value in the kernel arguments, which takes the
 * two dependent device reads (list entry, then the source's scale pointer) out of the head of
 * the launch (1.5 - 2.5 us of a 12 - 30 us launch).  Serves one row (at most 16 slices and
 * weights large enough for the one-row streaming kernel) and more than 8 rows (at most 16
 * slices, the MFMA kernels); anything else returns -1 and the caller passes device lists to
 * berth_ops_mgemm.  Same return values and error slot. */
int berth_ops_mgemm_hostlists(const void* a, const void* b_list, void* c, const void* suh_list, void* a_had,
                              const void* svh_list, int size_m, int size_k, int size_n, int k_bits,
                              int codebook, int c_fp32, int bszm_in, int bszm_out, const int* size_n_list,
                              const void* c_ptrs, const int* n_stride_list, const int* had_src_list,
                              int num_had_src, void* stream);
const char* berth_ops_last_error(void);    /* ops.rs:145 */
const char* berth_ops_last_launch(void);   /* ops.rs:146 */

/* ---- MoE layer ---------------------------------------------------------------
 * No counterpart in the reference, whose engine rejects MoE layers
 * (crates/berth-engine/src/model.rs:404-409).  The shapes follow its plan schema
 * (MoeDims / Ffn::Moe, crates/berth-plan/src/shape.rs:64-69, plan.rs:24-59: router,
 * optional shared expert, E routed experts of three EXL3 linears each) and the
 * expert-selection arguments of its multi-linear kernel
 * (crates/berth-kernels/csrc/ops/mgemm.cu:194-228).  Same conventions as above;
 * the message slots are berth_moe_last_error / berth_moe_last_launch.
 *
 * Arithmetic: logits = x @ wr in fp32 (64-row partial sums in row order, added in
 * order) + bias; top-k on the logits, ties to the lowest index; weights =
 * softmax over the selected k (renorm != 0) or over all experts; (token, slot)
 * pairs stable-sorted by expert; expert FFN = down(silu(gate(x)) * up(x)) with
 * fp16 gate/up outputs and fp32 down output; out = shared(x) + sum_j w_j *
 * FFN_j(x) in slot order. */
typedef struct {
    const void* trellis;    /* int16 [K/16][N/16][16*k_bits] */
    const void* suh;        /* fp16 [K] */
    const void* svh;        /* fp16 [N] */
} berth_exl3_lin;

/* ---- one dense MLP block ----------------------------------------------------
 * y = down(silu(gate(x)) * up(x)), the four calls of MlpLayer::forward
 * (crates/berth-engine/src/mlp.rs:118-150: two berth_exl3_linear with fp16
 * output, berth_ops_silu_mul with act_limit 0, berth_exl3_linear with fp32
 * output) in one entry.  Up to 8 rows run as two launches: gate and up share one
 * launch and the rotated input, and the down projection evaluates silu(g) * u
 * while it rotates its input (same fp16 steps as berth_ops_silu_mul, so the
 * activation is bit-identical to the unfused sequence).  More rows run on the MFMA
 * kernels: gate and up as one bundle (one launch rotates the input with either
 * linear's scales, one dense launch runs both; the up projection's rotated copy
 * waits in act_had, so this form needs intermediate >= hidden, else gate and up run
 * one after the other), berth_ops_silu_mul, the down projection.
 * lins: HOST array {gate, up, down} of device pointers.  x fp16 [m][hidden];
 * gate_out, up_out fp16 [m][intermediate] (written; above 8 rows up_out ends up
 * holding the activation); a_had fp16 [m][hidden] and act_had fp16
 * [m][intermediate] (written: the rotated inputs); y fp32 [m][hidden].
 * hidden % 128 == 0, intermediate % 128 == 0.  Errors and launch text go to
 * berth_exl3_last_error / berth_exl3_last_launch. */
int berth_exl3_mlp(const void* x, const berth_exl3_lin* lins, void* gate_out, void* up_out,
                   void* a_had, void* act_had, void* y, int size_m, int hidden, int intermediate,
                   int k_bits, int codebook, void* stream);

/* No counterpart in the reference as one call: the FFN block of a decoder layer as its engine
 * issues it (crates/berth-engine/src/mlp.rs:118-150 between the two glue ops of
 * crates/berth-kernels/src/ops.rs:430-500 and :522-552):
 *     residual_out = residual + x                                  (fp32, exact)
 *     h = rms(residual_out) * (weight + constant_bias) * constant_scale   (fp16; berth_ops_rms_norm_res_in)
 *     y = berth_exl3_mlp(h) + residual_out                         (fp32; berth_ops_add_f32)
 * x, residual, residual_out, y fp32 [m][hidden]; residual_out must alias neither x nor residual
 * (the in-place update of the reference's op would race with the workgroups still reading
 * it); y may alias x.  h_norm fp16 [m][hidden] is scratch (written when the launches are not
 * fused).  The other buffers are berth_exl3_mlp's.  One row: where the gate / up pair takes the
 * one-row streaming kernel the norm is formed while that launch rotates its input (same fp32
 * steps as berth_ops_rms_norm_res_in; the sum of squares in double, whose order of summation
 * differs), and where the down projection takes it the residual is added where it writes its
 * output: two launches when both do.  Anything else runs the same arithmetic as separate
 * launches. */
typedef struct {
    const void* weight;         /* fp16 or bf16 [hidden] */
    float epsilon, constant_bias, constant_scale;
    int weight_bf16;
} berth_rms_norm;
int berth_exl3_mlp_block(const void* x, const void* residual, void* residual_out, const berth_rms_norm* norm,
                         const berth_exl3_lin* lins, void* h_norm, void* gate_out, void* up_out, void* a_had,
                         void* act_had, void* y, int size_m, int hidden, int intermediate, int k_bits,
                         int codebook, void* stream);

/* x fp16 [T][H]; wr fp16 [H][E] (the unquantised router, mlp.gate.weight laid out
 * input-major); bias fp32 [E] or NULL; idx int32 [T][k]; w fp32 [T][k]; logits fp32
 * [T][E] or NULL; parts_scratch fp32 [T][ceil(H/64)][E]. */
int berth_moe_route(const void* x, const void* wr, const float* bias, int32_t* idx, float* w,
                    float* logits, void* parts_scratch, int T, int H, int E, int k, int renorm,
                    void* stream);
/* offsets int32 [E+1]; perm int32 [T*k] (sorted position -> t*k + j); inv its
 * inverse; scratch of berth_moe_permute_scratch_bytes bytes. */
int berth_moe_permute(const int32_t* idx, int32_t* offsets, int32_t* perm, int32_t* inv,
                      void* scratch, int T, int k, int E, void* stream);
size_t berth_moe_permute_scratch_bytes(int T, int k, int E);
/* One stage on its own: a grouped EXL3 linear over the expert-sorted rows.  No counterpart in the
 * reference; the per-expert weight lists play the role of b_list / suh_list / svh_list in its
 * multi-linear launch (crates/berth-kernels/src/ops.rs:268-280, csrc/ops/mgemm.cu:194-228).
 * Sorted row r (r < T*k) belongs to the expert berth_moe_permute assigned it; its input is row
 * gather[r] / gather_div of `a` (gather NULL: row r), or silu(a[r]) * a_up[r] when a_up is given;
 * its weights are experts[e * lins_per_expert + lin_base (+1)], a DEVICE array of berth_exl3_lin.
 * num_lins 2 runs two consecutive linears on the same input (gate and up) into c0 and c1.
 * Outputs are [T*k][size_n] in sorted order, fp16 or fp32 (c_fp32).  permute_scratch: the scratch
 * berth_moe_permute filled for the same T, k, E (read only).  a_had: fp16 scratch
 * [num_lins][T*k][size_k], needed above 8 rows (the MFMA path), else may be NULL. */
int berth_moe_grouped_exl3(const void* a, const void* a_up, const int32_t* gather, int gather_div,
                           const void* experts, int lins_per_expert, int lin_base, int num_lins, void* c0,
                           void* c1, const void* permute_scratch, void* a_had, int T, int k, int E, int size_k,
                           int size_n, int k_bits, int codebook, int c_fp32, void* stream);
/* The last stage on its own: out[t] = shared_out[t] (or 0) + sum_j w[t][j] * slot_out[inv[t*k + j]],
 * fp32 fma in slot order.  slot_out fp32 [T*k][H] in sorted order, shared_out fp32 [T][H] or NULL,
 * w fp32 [T][k], inv int32 [T*k] from berth_moe_permute, out fp32 [T][H]. */
int berth_moe_combine(const void* slot_out, const void* shared_out, const float* w, const int32_t* inv,
                      void* out, int T, int H, int k, void* stream);
/* Whole layer.  experts: DEVICE array of 3*E berth_exl3_lin (gate, up, down of
 * expert 0, then expert 1, ...).  shared: HOST array of 3 berth_exl3_lin holding
 * device pointers, or NULL.  out fp32 [T][H]; idx_out / w_out optional copies of
 * the routing; workspace of berth_moe_workspace_bytes bytes, caller-owned. */
int berth_moe_layer(const void* x, const void* wr, const float* bias, const void* experts,
                    const berth_exl3_lin* shared, void* out, int32_t* idx_out, float* w_out,
                    void* workspace, size_t workspace_bytes, int T, int H, int E, int k, int I,
                    int shared_I, int k_bits, int codebook, int renorm, void* stream);
/* The same layer with a gate on the always-on expert: shared_gate fp32 [H] on the device (the
 * shared_expert_gate.weight of Qwen-MoE checkpoints) scales that expert's row of token t by
 * sigmoid(x[t] . shared_gate) before the routed experts are added; the dot product is an fp32 fma
 * chain in row order per 64-row segment, segments added in order.  NULL: berth_moe_layer.  The
 * reference has no MoE arithmetic (crates/berth-engine/src/model.rs:404-409); the shape of the
 * layer follows crates/berth-plan/src/plan.rs:24-59. */
int berth_moe_layer_gated(const void* x, const void* wr, const float* bias, const void* experts,
                          const berth_exl3_lin* shared, const float* shared_gate, void* out, int32_t* idx_out,
                          float* w_out, void* workspace, size_t workspace_bytes, int T, int H, int E, int k,
                          int I, int shared_I, int k_bits, int codebook, int renorm, void* stream);
size_t berth_moe_workspace_bytes(int T, int H, int E, int k, int I, int shared_I);
/* byte offsets inside that workspace of {idx, w, offsets, perm, inv, gate_out
 * fp16 [T*k][I], up_out fp16 [T*k][I], slot_out fp32 [T*k][H] (rows in expert-
 * sorted order), shared_out fp32 [T][H]}, valid after berth_moe_layer returns */
int berth_moe_workspace_offsets(int T, int H, int E, int k, int I, int shared_I, size_t out[9]);
/* the always-on expert's own gate and up outputs, fp16 [T][shared_I] each, when shared_I != I
 * (with shared_I == I they are rows T*k .. of gate_out / up_out); above 8 rows the second one
 * ends up holding silu(gate) * up.  -1 when there is no such buffer. */
int berth_moe_workspace_shared_offsets(int T, int H, int E, int k, int I, int shared_I, size_t out[2]);
const char* berth_moe_last_error(void);
const char* berth_moe_last_launch(void);

#ifdef __cplusplus
}
#endif
#endif

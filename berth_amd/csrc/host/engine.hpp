// Host-side owners of the EXL3 linear path in C++, above the two C ABIs
// (include/berth_hip.h for the device runtime, include/berth_kernels_hip.h for
// the kernels).  Same roles, names and checks as the reference's engine-side
// types: Gpu (crates/berth-engine/src/device.rs:14-43), Exl3Linear with
// forward / forward_rows / forward_n (device.rs:77-367), RowScratch
// (device.rs:176-212), MlpLayer (crates/berth-engine/src/mlp.rs:25-334), and a
// MoeLayer for the Ffn::Moe{router, shared, experts} of
// crates/berth-plan/src/plan.rs:24-59 with every tensor resident in HBM.
// Exl3Linear::load, MlpLayer::load and upload_tensor read an EXL3 checkpoint
// directory through exl3_checkpoint.hpp (device.rs:49-125, mlp.rs:52-112).
// Header-only; no torch, no HIP headers: everything goes through the C ABIs.
#pragma once

#include "../../../include/berth_hip.h"
#include "../../../include/berth_kernels_hip.h"
#include "exl3_checkpoint.hpp"

#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace berth::engine {

// crates/berth-engine: Error::Input (caller mistakes), Error::Kernel (launch refused), Error::Device
struct InputError : std::invalid_argument { using std::invalid_argument::invalid_argument; };
struct KernelError : std::runtime_error { using std::runtime_error::runtime_error; };
// Error::Weights: a checkpoint whose tensors do not fit what the engine handles
struct WeightsError : std::runtime_error { using std::runtime_error::runtime_error; };
struct DeviceError : std::runtime_error {
    int code;
    DeviceError(int c, const std::string& what) : std::runtime_error(what), code(c) {}
};

inline void device_ok(int rc, const char* what)
{
    if (rc != 0) throw DeviceError(rc, std::string(what) + ": " + berth_hip_last_error());
}

enum class Codebook : int { Default = 0, Mcg = 1, Mul1 = 2 };   // crates/berth-kernels/src/lib.rs:54-63
enum class OutDtype : int { F16 = 0, F32 = 1 };                  // crates/berth-kernels/src/lib.rs:69-75
inline size_t out_bytes(OutDtype o) { return o == OutDtype::F32 ? 4 : 2; }

constexpr int kMaxReconstructN = 32768;     // crates/berth-engine/src/device.rs:193
constexpr int kMaxForwardNRows = 144;       // crates/berth-engine/src/device.rs:288-300

// device 0 .. n, its context and the stream every launch goes on (device.rs:14-43)
class Gpu {
public:
    explicit Gpu(int ordinal = 0)
    {
        device_ok(berth_hip_context_new(ordinal, &ctx_), "context");
        int rc = berth_hip_stream_new(ctx_, &stream_);
        if (rc != 0) {
            berth_hip_context_free(ctx_);
            device_ok(rc, "stream");
        }
        uint32_t n = 0;
        device_ok(berth_hip_context_multiprocessor_count(ctx_, &n), "multiprocessor count");
        sm_count_ = (int)n;
    }
    ~Gpu()
    {
        if (stream_) berth_hip_stream_free(stream_);
        if (ctx_) berth_hip_context_free(ctx_);
    }
    Gpu(const Gpu&) = delete;
    Gpu& operator=(const Gpu&) = delete;

    berth_hip_context* context() const { return ctx_; }
    const berth_hip_stream* stream() const { return stream_; }
    void* raw_stream() const { return (void*)(uintptr_t)berth_hip_stream_handle(stream_); }
    int sm_count() const { return sm_count_; }
    void synchronize() const { device_ok(berth_hip_stream_synchronize(stream_), "stream synchronize"); }

private:
    berth_hip_context* ctx_ = nullptr;
    berth_hip_stream* stream_ = nullptr;
    int sm_count_ = 0;
};

// crates/berth-cuda/src/buffer.rs:36-286: owns device memory; drop = context sync, then free
template <typename T>
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    static DeviceBuffer zeroed(const Gpu& gpu, size_t len)
    {
        DeviceBuffer b;
        b.gpu_ = &gpu;
        b.len_ = len;
        device_ok(berth_hip_buffer_zeroed(gpu.context(), gpu.stream(), (len ? len : 1) * sizeof(T), &b.ptr_), "buffer zeroed");
        return b;
    }
    static DeviceBuffer from_host(const Gpu& gpu, const T* src, size_t len)
    {
        DeviceBuffer b;
        b.gpu_ = &gpu;
        b.len_ = len;
        device_ok(berth_hip_buffer_alloc(gpu.context(), (len ? len : 1) * sizeof(T), &b.ptr_), "buffer alloc");
        if (len) device_ok(berth_hip_copy_from_host(gpu.stream(), b.ptr_, src, len * sizeof(T)), "copy from host");
        return b;
    }
    static DeviceBuffer from_host(const Gpu& gpu, const std::vector<T>& v) { return from_host(gpu, v.data(), v.size()); }
    DeviceBuffer(DeviceBuffer&& o) noexcept { *this = std::move(o); }
    DeviceBuffer& operator=(DeviceBuffer&& o) noexcept
    {
        release();
        gpu_ = o.gpu_; ptr_ = o.ptr_; len_ = o.len_;
        o.ptr_ = 0; o.len_ = 0;
        return *this;
    }
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    ~DeviceBuffer() { release(); }

    size_t len() const { return len_; }
    size_t num_bytes() const { return len_ * sizeof(T); }
    uint64_t ptr() const { return ptr_; }
    void* raw() const { return (void*)(uintptr_t)ptr_; }
    std::vector<T> copy_to_host() const
    {
        std::vector<T> v(len_);
        if (len_) device_ok(berth_hip_copy_to_host(gpu_->stream(), v.data(), ptr_, num_bytes()), "copy to host");
        return v;
    }

private:
    void release()
    {
        if (ptr_) {
            (void)berth_hip_context_synchronize(gpu_->context());
            (void)berth_hip_buffer_free(gpu_->context(), ptr_);
            ptr_ = 0;
        }
    }
    const Gpu* gpu_ = nullptr;
    uint64_t ptr_ = 0;
    size_t len_ = 0;
};

using Half = uint16_t;      // fp16 bit patterns on the host

// the checkpoint's EXL3 linear with this prefix (device.rs:167-173)
inline const exl3::LinearExl3& find_linear(const exl3::Checkpoint& ckpt, const std::string& prefix)
{
    const exl3::LinearExl3* l = ckpt.find_linear(prefix);
    if (!l) throw WeightsError(prefix + " is not an EXL3 linear");
    return *l;
}

// one checkpoint tensor, as stored, copied to the device (device.rs:65-74)
inline DeviceBuffer<uint8_t> upload_tensor(const Gpu& gpu, const exl3::Checkpoint& ckpt, const std::string& name)
{
    const exl3::TensorInfo* info = ckpt.tensors.get(name);
    if (!info) throw WeightsError("tensor " + name + " is missing");
    return DeviceBuffer<uint8_t>::from_host(gpu, exl3::read_tensor(*info));
}

// scratch shared by every linear of a prefill chunk (device.rs:176-212)
struct RowScratch {
    RowScratch(const Gpu& gpu, int max_rows_, int max_k_, int max_n_)
        : a_had(DeviceBuffer<Half>::zeroed(gpu, (size_t)max_rows_ * max_k_)),
          weight(DeviceBuffer<Half>::zeroed(gpu, (size_t)max_k_ * (max_n_ < kMaxReconstructN ? max_n_ : kMaxReconstructN))),
          max_rows(max_rows_), max_k(max_k_), max_n(max_n_) {}
    DeviceBuffer<Half> a_had, weight;
    int max_rows, max_k, max_n;
};

// one EXL3 linear on the device (device.rs:77-367)
class Exl3Linear {
public:
    // trellis: u16 words [size_k/16][size_n/16][16*k_bits]; suh [size_k], svh [size_n] fp16
    Exl3Linear(const Gpu& gpu, std::string prefix, const uint16_t* trellis, size_t trellis_words,
               const Half* suh, int size_k, const Half* svh, int size_n, Codebook codebook = Codebook::Mul1)
        : prefix_(std::move(prefix)), size_k_(size_k), size_n_(size_n), codebook_(codebook)
    {
        if (size_k <= 0 || size_n <= 0 || size_k % 16 || size_n % 16)
            throw InputError(prefix_ + ": sizes must be positive multiples of 16");
        const size_t tiles = (size_t)(size_k / 16) * (size_n / 16);
        if (trellis_words == 0 || trellis_words % (tiles * 16))
            throw InputError(prefix_ + ": trellis must be (K/16, N/16, 16*bits)");
        k_bits_ = (int)(trellis_words / (tiles * 16));
        if (k_bits_ < 1 || k_bits_ > 8) throw InputError(prefix_ + ": bits per weight must be in 1..=8");
        trellis_ = DeviceBuffer<uint16_t>::from_host(gpu, trellis, trellis_words);
        suh_ = DeviceBuffer<Half>::from_host(gpu, suh, (size_t)size_k);
        svh_ = DeviceBuffer<Half>::from_host(gpu, svh, (size_t)size_n);
        a_had_ = DeviceBuffer<Half>::zeroed(gpu, (size_t)size_k);
    }

    // <prefix>.trellis, .suh / .svh (or packed .su / .sv, expanded on the device) from a
    // checkpoint (device.rs:92-125).  Half-integer rates are refused as in the reference;
    // packed signs, which the reference refuses at this point, are accepted.
    static Exl3Linear load(const Gpu& gpu, const exl3::Checkpoint& ckpt, const std::string& prefix)
    {
        const exl3::LinearExl3& linear = find_linear(ckpt, prefix);
        if (linear.k.is_half()) throw WeightsError(prefix + ": half-integer rate");
        Exl3Linear out;
        out.prefix_ = prefix;
        out.k_bits_ = linear.k.whole();
        out.codebook_ = linear.codebook == exl3::Codebook::Mul1  ? Codebook::Mul1
                        : linear.codebook == exl3::Codebook::Mcg ? Codebook::Mcg
                                                                 : Codebook::Default;
        out.suh_ = load_scale(gpu, linear.input_scale, &out.size_k_);
        out.svh_ = load_scale(gpu, linear.output_scale, &out.size_n_);
        const auto& shape = linear.trellis.shape;
        if (out.size_k_ <= 0 || out.size_n_ <= 0 || shape[0] * 16 != (uint64_t)out.size_k_ ||
            shape[1] * 16 != (uint64_t)out.size_n_)
            throw WeightsError(prefix + ": trellis " + std::to_string(shape[0]) + "x" + std::to_string(shape[1]) +
                               " tiles do not match " + std::to_string(out.size_k_) + " x " +
                               std::to_string(out.size_n_) + " scales");
        const std::vector<uint8_t> body = exl3::read_tensor(linear.trellis);
        out.trellis_ = DeviceBuffer<uint16_t>::from_host(gpu, (const uint16_t*)body.data(), body.size() / 2);
        out.a_had_ = DeviceBuffer<Half>::zeroed(gpu, (size_t)out.size_k_);
        return out;
    }

    const std::string& prefix() const { return prefix_; }
    int size_k() const { return size_k_; }
    int size_n() const { return size_n_; }
    int k_bits() const { return k_bits_; }
    Codebook codebook() const { return codebook_; }
    size_t trellis_bytes() const { return trellis_.num_bytes(); }
    berth_exl3_lin table_entry() const { return berth_exl3_lin{trellis_.raw(), suh_.raw(), svh_.raw()}; }

    // one row (device.rs:127-165)
    void forward(const Gpu& gpu, const DeviceBuffer<Half>& a, uint64_t c, size_t c_bytes, OutDtype out) const
    {
        if (a.len() < (size_t)size_k_ || c_bytes < (size_t)size_n_ * out_bytes(out))
            throw InputError(prefix_ + ": buffer too small");
        if (berth_exl3_linear(a.raw(), trellis_.raw(), (void*)(uintptr_t)c, suh_.raw(), a_had_.raw(), svh_.raw(), 1,
                              size_k_, size_n_, k_bits_, (int)codebook_, (int)out, gpu.raw_stream()) != 0)
            throw KernelError(berth_exl3_last_error());
    }

    // rows > 1 with the chunk's scratch (device.rs:210-272)
    void forward_rows(const Gpu& gpu, const RowScratch& scratch, const DeviceBuffer<Half>& a, uint64_t c,
                      size_t c_bytes, int rows, OutDtype out) const
    {
        if (rows < 2) throw InputError(prefix_ + ": forward_rows needs rows > 1");
        if (rows > scratch.max_rows || size_k_ > scratch.max_k || size_n_ > scratch.max_n)
            throw InputError(prefix_ + ": " + std::to_string(rows) + " x " + std::to_string(size_k_) + " x " +
                             std::to_string(size_n_) + " exceeds the row scratch");
        if (a.len() < (size_t)rows * size_k_ || c_bytes < (size_t)rows * size_n_ * out_bytes(out))
            throw InputError(prefix_ + ": buffer too small");
        void* weight = rows > kMaxForwardNRows ? scratch.weight.raw() : nullptr;
        if (berth_prefill_exl3_linear(a.raw(), trellis_.raw(), (void*)(uintptr_t)c, suh_.raw(), scratch.a_had.raw(),
                                      svh_.raw(), weight, rows, size_k_, size_n_, k_bits_, (int)codebook_, (int)out,
                                      gpu.raw_stream()) != 0)
            throw KernelError(berth_prefill_last_error());
    }

    // 1..144 rows with a caller-owned rotated-input buffer (device.rs:288-366)
    void forward_n(const Gpu& gpu, const DeviceBuffer<Half>& a_had, const DeviceBuffer<Half>& a, uint64_t c,
                   size_t c_bytes, int rows, OutDtype out) const
    {
        if (rows == 1) return forward(gpu, a, c, c_bytes, out);
        if (rows == 0 || rows > kMaxForwardNRows)
            throw InputError(prefix_ + ": forward_n rows " + std::to_string(rows) + " are outside 1..=144");
        const size_t need = (size_t)rows * size_k_;
        if (a_had.len() < need || a.len() < need || c_bytes < (size_t)rows * size_n_ * out_bytes(out))
            throw InputError(prefix_ + ": buffer too small");
        if (berth_prefill_exl3_linear(a.raw(), trellis_.raw(), (void*)(uintptr_t)c, suh_.raw(), a_had.raw(), svh_.raw(),
                                      nullptr, rows, size_k_, size_n_, k_bits_, (int)codebook_, (int)out,
                                      gpu.raw_stream()) != 0)
            throw KernelError(berth_prefill_last_error());
    }

private:
    Exl3Linear() = default;
    // fp16 vector as stored, or packed sign words expanded to fp16 +-1 on the device
    static DeviceBuffer<Half> load_scale(const Gpu& gpu, const exl3::HadamardScale& scale, int* channels)
    {
        const std::vector<uint8_t> body = exl3::read_tensor(scale.tensor);
        if (!scale.packed) {
            *channels = (int)(body.size() / 2);
            return DeviceBuffer<Half>::from_host(gpu, (const Half*)body.data(), body.size() / 2);
        }
        *channels = (int)(body.size() * 8);
        DeviceBuffer<uint8_t> packed = DeviceBuffer<uint8_t>::from_host(gpu, body);
        DeviceBuffer<Half> out = DeviceBuffer<Half>::zeroed(gpu, body.size() * 8);
        if (berth_exl3_unpack_signs(packed.raw(), out.raw(), (int64_t)body.size(), gpu.raw_stream()) != 0)
            throw KernelError(berth_exl3_last_error());
        gpu.synchronize();      // `packed` is released on return
        return out;
    }
    std::string prefix_;
    int size_k_ = 0, size_n_ = 0, k_bits_ = 0;
    Codebook codebook_ = Codebook::Mul1;
    DeviceBuffer<uint16_t> trellis_;
    DeviceBuffer<Half> suh_, svh_, a_had_;
};

// gate -> up -> silu_mul -> down (mlp.rs:118-150 decode, :219-303 prefill)
class MlpLayer {
public:
    MlpLayer(const Gpu& gpu, Exl3Linear gate, Exl3Linear up, Exl3Linear down, int max_rows = 1)
        : gate_(std::move(gate)), up_(std::move(up)), down_(std::move(down)), max_rows_(max_rows)
    {
        hidden_ = gate_.size_k();
        intermediate_ = gate_.size_n();
        if (up_.size_k() != hidden_ || up_.size_n() != intermediate_ || down_.size_k() != intermediate_ ||
            down_.size_n() != hidden_)
            throw InputError("mlp: projection shapes do not chain");
        g_ = DeviceBuffer<Half>::zeroed(gpu, (size_t)max_rows * intermediate_);
        u_ = DeviceBuffer<Half>::zeroed(gpu, (size_t)max_rows * intermediate_);
        x_had_ = DeviceBuffer<Half>::zeroed(gpu, (size_t)max_rows * hidden_);
        act_had_ = DeviceBuffer<Half>::zeroed(gpu, (size_t)max_rows * intermediate_);
        // the one-call path takes one bit rate and codebook for the three linears
        uniform_ = gate_.k_bits() == up_.k_bits() && gate_.k_bits() == down_.k_bits() &&
                   gate_.codebook() == up_.codebook() && gate_.codebook() == down_.codebook();
    }
    // layer `layer`'s MLP weights (mlp.rs:52-56)
    static MlpLayer load(const Gpu& gpu, const exl3::Checkpoint& ckpt, uint32_t layer, int max_rows = 1)
    {
        return load_prefixed(gpu, ckpt, "model.language_model.layers." + std::to_string(layer) + ".mlp", max_rows);
    }
    // {prefix}.gate_proj, .up_proj and .down_proj (mlp.rs:58-112); a bias is refused because
    // it would not be applied
    static MlpLayer load_prefixed(const Gpu& gpu, const exl3::Checkpoint& ckpt, const std::string& prefix,
                                  int max_rows = 1)
    {
        const std::string parts[3] = {prefix + ".gate_proj", prefix + ".up_proj", prefix + ".down_proj"};
        for (const std::string& part : parts)
            if (find_linear(ckpt, part).bias) throw WeightsError(part + ": bias is present and is not applied");
        Exl3Linear gate = Exl3Linear::load(gpu, ckpt, parts[0]);
        Exl3Linear up = Exl3Linear::load(gpu, ckpt, parts[1]);
        Exl3Linear down = Exl3Linear::load(gpu, ckpt, parts[2]);
        auto dims = [](const Exl3Linear& l) { return std::to_string(l.size_k()) + "x" + std::to_string(l.size_n()); };
        if (gate.size_k() != up.size_k() || gate.size_n() != up.size_n())
            throw WeightsError(prefix + ": gate is " + dims(gate) + ", up is " + dims(up));
        if (down.size_k() != gate.size_n() || down.size_n() != gate.size_k())
            throw WeightsError(prefix + ": down is " + dims(down) + ", gate is " + dims(gate));
        if (gate.size_n() < 2 || gate.size_n() % 2 != 0)
            throw WeightsError(prefix + ": intermediate " + std::to_string(gate.size_n()) + " must be positive and even");
        return MlpLayer(gpu, std::move(gate), std::move(up), std::move(down), max_rows);
    }

    int hidden() const { return hidden_; }
    int intermediate() const { return intermediate_; }

    // x fp16 [rows][hidden] -> y fp32 [rows][hidden] through berth_exl3_mlp: gate and up in one
    // launch, silu(g) * u evaluated inside the down projection (two launches up to 8 rows)
    void forward_fused(const Gpu& gpu, const DeviceBuffer<Half>& x, DeviceBuffer<float>& y, int rows = 1) const
    {
        if (!uniform_) throw InputError("mlp: the one-call path needs one bit rate and codebook");
        if (rows < 1 || rows > max_rows_) throw InputError("mlp: rows exceed the layer scratch");
        if (x.len() < (size_t)rows * hidden_ || y.len() < (size_t)rows * hidden_)
            throw InputError(gate_.prefix() + ": buffer too small");
        const berth_exl3_lin lins[3] = {gate_.table_entry(), up_.table_entry(), down_.table_entry()};
        if (berth_exl3_mlp(x.raw(), lins, g_.raw(), u_.raw(), x_had_.raw(), act_had_.raw(), y.raw(), rows, hidden_,
                           intermediate_, gate_.k_bits(), (int)gate_.codebook(), gpu.raw_stream()) != 0)
            throw KernelError(berth_exl3_last_error());
    }
    // x fp16 [hidden] -> y fp32 [hidden], the reference's four calls (mlp.rs:118-150)
    void forward(const Gpu& gpu, const DeviceBuffer<Half>& x, DeviceBuffer<float>& y) const
    {
        if (x.len() < (size_t)hidden_ || y.len() < (size_t)hidden_) throw InputError(gate_.prefix() + ": buffer too small");
        gate_.forward(gpu, x, g_.ptr(), g_.num_bytes(), OutDtype::F16);
        up_.forward(gpu, x, u_.ptr(), u_.num_bytes(), OutDtype::F16);
        silu(gpu, intermediate_);
        down_.forward(gpu, u_, y.ptr(), y.num_bytes(), OutDtype::F32);
    }
    // x fp16 [rows][hidden] -> y fp32 [rows][hidden]
    void prefill(const Gpu& gpu, const RowScratch& scratch, const DeviceBuffer<Half>& x, DeviceBuffer<float>& y,
                 int rows) const
    {
        if (rows > max_rows_) throw InputError("mlp: rows exceed the layer scratch");
        gate_.forward_rows(gpu, scratch, x, g_.ptr(), g_.num_bytes(), rows, OutDtype::F16);
        up_.forward_rows(gpu, scratch, x, u_.ptr(), u_.num_bytes(), rows, OutDtype::F16);
        silu(gpu, (int64_t)rows * intermediate_);
        down_.forward_rows(gpu, scratch, u_, y.ptr(), y.num_bytes(), rows, OutDtype::F32);
    }

private:
    void silu(const Gpu& gpu, int64_t numel) const
    {
        // act_limit 0: no clamp (mlp.rs:20-22); out aliases up (mlp.rs:280-299)
        if (berth_ops_silu_mul(g_.raw(), u_.raw(), u_.raw(), numel, 0.0f, gpu.raw_stream()) != 0)
            throw KernelError(berth_ops_last_error());
    }
    Exl3Linear gate_, up_, down_;
    int hidden_ = 0, intermediate_ = 0, max_rows_;
    bool uniform_ = false;
    DeviceBuffer<Half> g_, u_, x_had_, act_had_;
};

// router + E routed experts of three linears + optional always-on shared expert
class MoeLayer {
public:
    struct Expert { Exl3Linear gate, up, down; };
    // router: fp16 [hidden][experts]; bias: optional fp32 [experts]
    MoeLayer(const Gpu& gpu, const Half* router, int hidden, int num_experts, std::vector<Expert> experts, int top_k,
             const float* bias = nullptr, bool renorm = true)
        : hidden_(hidden), num_experts_(num_experts), top_k_(top_k), renorm_(renorm), experts_(std::move(experts))
    {
        if ((int)experts_.size() != num_experts) throw InputError("moe: router width and expert count differ");
        intermediate_ = experts_[0].gate.size_n();
        k_bits_ = experts_[0].gate.k_bits();
        codebook_ = experts_[0].gate.codebook();
        std::vector<berth_exl3_lin> table;
        for (const Expert& e : experts_) {
            if (e.gate.size_k() != hidden || e.gate.size_n() != intermediate_ || e.up.size_k() != hidden ||
                e.up.size_n() != intermediate_ || e.down.size_k() != intermediate_ || e.down.size_n() != hidden ||
                e.gate.k_bits() != k_bits_ || e.up.k_bits() != k_bits_ || e.down.k_bits() != k_bits_)
                throw InputError("moe: expert shapes / bit rates must be uniform");
            table.push_back(e.gate.table_entry());
            table.push_back(e.up.table_entry());
            table.push_back(e.down.table_entry());
        }
        table_ = DeviceBuffer<berth_exl3_lin>::from_host(gpu, table);
        router_ = DeviceBuffer<Half>::from_host(gpu, router, (size_t)hidden * num_experts);
        if (bias) bias_ = DeviceBuffer<float>::from_host(gpu, bias, (size_t)num_experts);
    }
    void set_shared(Expert shared)
    {
        shared_.clear();
        shared_.push_back(std::move(shared));
    }

    // x fp16 [tokens][hidden] -> out fp32 [tokens][hidden]; idx_out / w_out optional [tokens][top_k]
    void forward(const Gpu& gpu, const DeviceBuffer<Half>& x, DeviceBuffer<float>& out, int tokens,
                 DeviceBuffer<int32_t>* idx_out = nullptr, DeviceBuffer<float>* w_out = nullptr)
    {
        if (x.len() < (size_t)tokens * hidden_ || out.len() < (size_t)tokens * hidden_)
            throw InputError("moe: buffer too small");
        const int shared_i = shared_.empty() ? 0 : shared_[0].gate.size_n();
        const size_t need = berth_moe_workspace_bytes(tokens, hidden_, num_experts_, top_k_, intermediate_, shared_i);
        if (ws_.len() < need) ws_ = DeviceBuffer<uint8_t>::zeroed(gpu, need);
        berth_exl3_lin sh[3];
        if (!shared_.empty()) {
            sh[0] = shared_[0].gate.table_entry();
            sh[1] = shared_[0].up.table_entry();
            sh[2] = shared_[0].down.table_entry();
        }
        if (berth_moe_layer(x.raw(), router_.raw(), bias_.len() ? (const float*)bias_.raw() : nullptr, table_.raw(),
                            shared_.empty() ? nullptr : sh, out.raw(), idx_out ? (int32_t*)idx_out->raw() : nullptr,
                            w_out ? (float*)w_out->raw() : nullptr, ws_.raw(), ws_.len(), tokens, hidden_, num_experts_,
                            top_k_, intermediate_, shared_i, k_bits_, (int)codebook_, renorm_ ? 1 : 0,
                            gpu.raw_stream()) != 0)
            throw KernelError(berth_moe_last_error());
    }

private:
    int hidden_, num_experts_, top_k_, intermediate_ = 0, k_bits_ = 0;
    bool renorm_;
    Codebook codebook_ = Codebook::Mul1;
    std::vector<Expert> experts_;
    std::vector<Expert> shared_;
    DeviceBuffer<berth_exl3_lin> table_;
    DeviceBuffer<Half> router_;
    DeviceBuffer<float> bias_;
    DeviceBuffer<uint8_t> ws_;
};

}  // namespace berth::engine

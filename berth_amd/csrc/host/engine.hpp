// Host-side owners of the EXL3 linear path in C++, above the two C ABIs
// (include/berth_hip.h for the device runtime, include/berth_kernels_hip.h for
// the kernels).  Same roles, names and checks as the reference's engine-side
// types: Gpu (crates/berth-engine/src/device.rs:14-43), Exl3Linear with
// forward / forward_rows / forward_n (device.rs:77-367), RowScratch
// (device.rs:176-212), MlpLayer (crates/berth-engine/src/mlp.rs:25-334), and a
// MoeLayer for the Ffn::Moe{router, shared, experts} of
// crates/berth-plan/src/plan.rs:24-59 with every tensor resident in HBM.
// Exl3Linear::load, MlpLayer::load, MoeLayer::load and upload_tensor read an EXL3
// checkpoint directory through exl3_checkpoint.hpp (device.rs:49-125, mlp.rs:52-112);
// MoeLayer::load is sized by the plan's Ffn::Moe record (plan.hpp).
// Header-only; no torch, no HIP headers: everything goes through the C ABIs.
#pragma once

#include "../../../include/berth_hip.h"
#include "../../../include/berth_kernels_hip.h"
#include "exl3_checkpoint.hpp"
#include "plan.hpp"

#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
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

// Loader conventions that no file of the reference fixes (it refuses a bias and never opens a
// stacked expert tensor): each is announced once per process on stderr, with the first tensor
// that used it, so that a wrong guess shows up in a log instead of only in the outputs.
// BERTH_QUIET_UNPINNED=1 silences the notes.
enum class Unpinned { Bias = 0, StackedExperts = 1, SharedExpertGate = 2 };
inline void note_unpinned(Unpinned what, const std::string& tensor)
{
    static std::atomic<unsigned> said{0};
    const unsigned bit = 1u << (unsigned)what;
    if (said.fetch_or(bit) & bit) return;
    const char* quiet = std::getenv("BERTH_QUIET_UNPINNED");
    if (quiet && *quiet && *quiet != '0') return;
    static const char* const text[] = {
        "a linear's .bias is added in fp32 after the output scales (y = W x + b)",
        "stacked expert tensors are read K-major, expert after expert, gate columns before up columns",
        "shared_expert_gate scales the shared expert's row by sigmoid(x . w)",
    };
    std::fprintf(stderr, "berth: convention not fixed by the reference, applied as assumed: %s (first: %s)\n",
                 text[(unsigned)what], tensor.c_str());
}

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

// fp32 -> fp16 bits, round to nearest even, overflow to infinity, NaN kept quiet
inline Half f32_to_f16_bits(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7FFFFFFFu;
    if (x >= 0x7F800000u) return (Half)(sign | 0x7C00u | (x > 0x7F800000u ? 0x200u : 0));
    if (x >= 0x477FF000u) return (Half)(sign | 0x7C00u);                 // rounds to 65520 or above
    if (x < 0x33000001u) return (Half)sign;                              // at most half of the smallest subnormal
    if (x < 0x38800000u) {                                               // subnormal result
        const int shift = 126 - (int)(x >> 23);                          // 14..24
        const uint32_t man = (x & 0x7FFFFFu) | 0x800000u;
        const uint32_t q = man >> shift, rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
        return (Half)(sign | (q + (rem > half || (rem == half && (q & 1)))));
    }
    const uint32_t q = ((x - 0x38000000u) >> 13), rem = x & 0x1FFFu;
    return (Half)(sign | (q + (rem > 0x1000u || (rem == 0x1000u && (q & 1)))));
}
inline float f16_bits_to_f32(Half h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1F, man = h & 0x3FFu;
    uint32_t x;
    if (exp == 0x1F) {
        x = sign | 0x7F800000u | (man << 13);
    } else if (exp) {
        x = sign | ((exp + 112) << 23) | (man << 13);
    } else if (man) {
        int e = 113;
        uint32_t m = man;
        while (!(m & 0x400u)) { m <<= 1; --e; }
        x = sign | ((uint32_t)e << 23) | ((m & 0x3FFu) << 13);
    } else {
        x = sign;
    }
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

// an F16 / BF16 / F32 checkpoint tensor as fp32 values (the dtypes a bias may have: linear.rs:219-231)
inline std::vector<float> read_float_tensor(const exl3::TensorInfo& info)
{
    const std::vector<uint8_t> body = exl3::read_tensor(info);
    std::vector<float> out;
    if (info.dtype == exl3::DType::F32) {
        out.resize(body.size() / 4);
        std::memcpy(out.data(), body.data(), out.size() * 4);
    } else if (info.dtype == exl3::DType::F16 || info.dtype == exl3::DType::Bf16) {
        out.resize(body.size() / 2);
        for (size_t i = 0; i < out.size(); ++i) {
            uint16_t v;
            std::memcpy(&v, body.data() + 2 * i, 2);
            if (info.dtype == exl3::DType::F16) {
                out[i] = f16_bits_to_f32(v);
            } else {
                const uint32_t x = (uint32_t)v << 16;
                std::memcpy(&out[i], &x, 4);
            }
        }
    } else {
        throw WeightsError(info.name + ": expected a float tensor, got " + exl3::dtype_name(info.dtype));
    }
    return out;
}

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

    // <prefix>.trellis, .suh / .svh (or packed .su / .sv, expanded on the device) and an
    // optional .bias from a checkpoint (device.rs:92-125).  Half-integer rates are refused as
    // in the reference; packed signs, which the reference refuses at this point, are accepted;
    // a bias, which the reference's engine refuses (mlp.rs:67-75), is kept in fp32 and added
    // to every output row after the linear (y = W x + b).
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
        if (linear.bias) {
            note_unpinned(Unpinned::Bias, prefix + ".bias");
            out.set_bias(gpu, read_float_tensor(*linear.bias));
        }
        return out;
    }

    // fp32 bias of size_n values, added to every output row after the linear
    void set_bias(const Gpu& gpu, const std::vector<float>& bias)
    {
        if ((int)bias.size() != size_n_)
            throw WeightsError(prefix_ + ": bias has " + std::to_string(bias.size()) + " values for " +
                               std::to_string(size_n_) + " outputs");
        bias_ = DeviceBuffer<float>::from_host(gpu, bias);
    }
    bool has_bias() const { return bias_.len() != 0; }

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
        add_bias(gpu, c, 1, out);
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
        add_bias(gpu, c, rows, out);
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
        add_bias(gpu, c, rows, out);
    }

private:
    Exl3Linear() = default;
    void add_bias(const Gpu& gpu, uint64_t c, int rows, OutDtype out) const
    {
        if (!has_bias()) return;
        if (berth_ops_add_bias((void*)(uintptr_t)c, (const float*)bias_.raw(), rows, size_n_, out == OutDtype::F32 ? 1 : 0,
                               gpu.raw_stream()) != 0)
            throw KernelError(berth_ops_last_error());
    }
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
    DeviceBuffer<float> bias_;
};

// Several EXL3 linears that share one input, as one sliced berth_ops_mgemm (the q/k/v bundle
// of crates/berth-engine/src/attn.rs:1934-1973 and gdn.rs:1102-1130; list layout
// crates/berth-kernels/src/ops.rs:264-293): every source is cut into slices of the greatest
// common width.  Any row count: one row and more than 8 rows pass the lists by value when
// there are at most 16 slices, 2..8 rows read them from device memory.
class MultiLinear {
public:
    MultiLinear(const Gpu& gpu, std::vector<const Exl3Linear*> sources) : sources_(std::move(sources))
    {
        if (sources_.empty()) throw InputError("multi-linear: no sources");
        size_k_ = sources_[0]->size_k();
        k_bits_ = sources_[0]->k_bits();
        codebook_ = sources_[0]->codebook();
        int width = 0;
        for (const Exl3Linear* s : sources_) {
            if (s->size_k() != size_k_ || s->k_bits() != k_bits_ || s->codebook() != codebook_)
                throw InputError("multi-linear: sources must share in-features, bit rate and codebook");
            if (s->has_bias()) throw InputError("multi-linear: a source with a bias runs as its own linear");
            int a = width, b = s->size_n();
            while (b) { const int t = a % b; a = b; b = t; }
            width = a;
        }
        if (width % 128) throw InputError("multi-linear: slice width must be a multiple of 128");
        width_ = width;
        const uint64_t tile_bytes = (uint64_t)16 * k_bits_ * 2;
        for (size_t si = 0; si < sources_.size(); ++si) {
            const berth_exl3_lin e = sources_[si]->table_entry();
            suh_.push_back((uint64_t)(uintptr_t)e.suh);
            for (int n0 = 0; n0 < sources_[si]->size_n(); n0 += width) {
                b_.push_back((uint64_t)(uintptr_t)e.trellis + (uint64_t)(n0 / 16) * tile_bytes);
                svh_.push_back((uint64_t)(uintptr_t)e.svh + (uint64_t)n0 * 2);
                stride_.push_back(sources_[si]->size_n());
                src_.push_back((int)si);
                n0_.push_back(n0);
                size_n_.push_back(width);
            }
        }
        d_b_ = DeviceBuffer<uint64_t>::from_host(gpu, b_);
        d_svh_ = DeviceBuffer<uint64_t>::from_host(gpu, svh_);
        d_suh_ = DeviceBuffer<uint64_t>::from_host(gpu, suh_);
        d_stride_ = DeviceBuffer<int>::from_host(gpu, stride_);
        d_src_ = DeviceBuffer<int>::from_host(gpu, src_);
        d_size_n_ = DeviceBuffer<int>::from_host(gpu, size_n_);
        gpu.synchronize();                                      // the host vectors may move from here on
    }

    int slices() const { return (int)b_.size(); }
    int width() const { return width_; }

    // a fp16 [rows][K]; outs[i] = device address of source i's output [rows][N_i] in `out`
    void forward(const Gpu& gpu, const DeviceBuffer<Half>& a, const std::vector<uint64_t>& outs, int rows, OutDtype out)
    {
        if (rows < 1) throw InputError("multi-linear: rows must be positive");
        if (outs.size() != sources_.size()) throw InputError("multi-linear: one output per source");
        if (a.len() < (size_t)rows * size_k_) throw InputError("multi-linear: input too small");
        const size_t need = sources_.size() * (size_t)rows * size_k_;
        if (a_had_.len() < need) a_had_ = DeviceBuffer<Half>::zeroed(gpu, need);
        const size_t esz = out_bytes(out);
        std::vector<uint64_t> c(b_.size());
        for (size_t i = 0; i < c.size(); ++i) c[i] = outs[(size_t)src_[i]] + (uint64_t)n0_[i] * esz;
        const bool by_value = slices() <= 16 && ((rows == 1 && host_lists_) || rows > 8);
        if (by_value) {
            const int rc = berth_ops_mgemm_hostlists(a.raw(), b_.data(), (void*)(uintptr_t)outs[0], suh_.data(), a_had_.raw(),
                                                     svh_.data(), rows, size_k_, width_, k_bits_, (int)codebook_, (int)out, 1,
                                                     slices(), size_n_.data(), c.data(), stride_.data(), src_.data(),
                                                     (int)sources_.size(), gpu.raw_stream());
            if (rc > 0) return;
            const std::string err = berth_ops_last_error();
            if (rows > 1 || err.find("host lists") == std::string::npos) throw KernelError(err);
            host_lists_ = false;                                // too small for the streaming kernel: device lists from now on
        }
        if (c != c_host_) {
            gpu.synchronize();                                  // a launch in flight may still read the old list
            d_c_ = DeviceBuffer<uint64_t>::from_host(gpu, c);
            gpu.synchronize();
            c_host_ = c;
        }
        if (berth_ops_mgemm(a.raw(), d_b_.raw(), (void*)(uintptr_t)outs[0], d_suh_.raw(), a_had_.raw(), d_svh_.raw(), rows,
                            size_k_, width_, k_bits_, (int)codebook_, (int)out, 1, slices(), (const int*)d_size_n_.raw(),
                            d_c_.raw(), (const int*)d_stride_.raw(), (const int*)d_src_.raw(), (int)sources_.size(),
                            gpu.raw_stream()) <= 0)
            throw KernelError(berth_ops_last_error());
    }

private:
    std::vector<const Exl3Linear*> sources_;
    int size_k_ = 0, k_bits_ = 0, width_ = 0;
    Codebook codebook_ = Codebook::Mul1;
    std::vector<uint64_t> b_, svh_, suh_, c_host_;
    std::vector<int> stride_, src_, n0_, size_n_;
    DeviceBuffer<uint64_t> d_b_, d_svh_, d_suh_, d_c_;
    DeviceBuffer<int> d_stride_, d_src_, d_size_n_;
    DeviceBuffer<Half> a_had_;
    bool host_lists_ = true;
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
        has_bias_ = gate_.has_bias() || up_.has_bias() || down_.has_bias();
    }
    // layer `layer`'s MLP weights (mlp.rs:52-56)
    static MlpLayer load(const Gpu& gpu, const exl3::Checkpoint& ckpt, uint32_t layer, int max_rows = 1)
    {
        return load_prefixed(gpu, ckpt, "model.language_model.layers." + std::to_string(layer) + ".mlp", max_rows);
    }
    // {prefix}.gate_proj, .up_proj and .down_proj (mlp.rs:58-112).  The reference refuses a bias
    // here (mlp.rs:67-75); this loader keeps it, forward / prefill add it after each linear, and
    // forward_fused, which has no place for it, refuses the layer.
    static MlpLayer load_prefixed(const Gpu& gpu, const exl3::Checkpoint& ckpt, const std::string& prefix,
                                  int max_rows = 1)
    {
        const std::string parts[3] = {prefix + ".gate_proj", prefix + ".up_proj", prefix + ".down_proj"};
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
    bool has_bias() const { return has_bias_; }

    // x fp16 [rows][hidden] -> y fp32 [rows][hidden] through berth_exl3_mlp: gate and up in one
    // launch, silu(g) * u evaluated inside the down projection (two launches up to 8 rows)
    void forward_fused(const Gpu& gpu, const DeviceBuffer<Half>& x, DeviceBuffer<float>& y, int rows = 1) const
    {
        if (!uniform_) throw InputError("mlp: the one-call path needs one bit rate and codebook");
        if (has_bias_) throw InputError("mlp: the one-call path does not add a bias");
        if (rows < 1 || rows > max_rows_) throw InputError("mlp: rows exceed the layer scratch");
        if (x.len() < (size_t)rows * hidden_ || y.len() < (size_t)rows * hidden_)
            throw InputError(gate_.prefix() + ": buffer too small");
        const berth_exl3_lin lins[3] = {gate_.table_entry(), up_.table_entry(), down_.table_entry()};
        if (berth_exl3_mlp(x.raw(), lins, g_.raw(), u_.raw(), x_had_.raw(), act_had_.raw(), y.raw(), rows, hidden_,
                           intermediate_, gate_.k_bits(), (int)gate_.codebook(), gpu.raw_stream()) != 0)
            throw KernelError(berth_exl3_last_error());
    }
    // The FFN block around the MLP through berth_exl3_mlp_block: residual_out = residual + x,
    // y = mlp(rms_norm(residual_out)) + residual_out; x, residual, residual_out, y fp32
    // [rows][hidden], norm_weight bf16 (or fp16) [hidden].  One row of large linears is two
    // launches; residual_out must be a buffer of its own.
    void forward_block(const Gpu& gpu, const DeviceBuffer<float>& x, const DeviceBuffer<float>& residual,
                       DeviceBuffer<float>& residual_out, const DeviceBuffer<uint16_t>& norm_weight, DeviceBuffer<float>& y,
                       float epsilon = 1e-6f, float constant_bias = 1.0f, float constant_scale = 1.0f,
                       bool weight_bf16 = true, int rows = 1) const
    {
        if (!uniform_) throw InputError("mlp: the one-call path needs one bit rate and codebook");
        if (has_bias_) throw InputError("mlp: the one-call path does not add a bias");
        if (rows < 1 || rows > max_rows_) throw InputError("mlp: rows exceed the layer scratch");
        const size_t n = (size_t)rows * hidden_;
        if (x.len() < n || residual.len() < n || residual_out.len() < n || y.len() < n || norm_weight.len() < (size_t)hidden_)
            throw InputError(gate_.prefix() + ": buffer too small");
        if (h_norm_.len() < n) h_norm_ = DeviceBuffer<Half>::zeroed(gpu, (size_t)max_rows_ * hidden_);
        const berth_exl3_lin lins[3] = {gate_.table_entry(), up_.table_entry(), down_.table_entry()};
        const berth_rms_norm norm{norm_weight.raw(), epsilon, constant_bias, constant_scale, weight_bf16 ? 1 : 0};
        if (berth_exl3_mlp_block(x.raw(), residual.raw(), residual_out.raw(), &norm, lins, h_norm_.raw(), g_.raw(), u_.raw(),
                                 x_had_.raw(), act_had_.raw(), y.raw(), rows, hidden_, intermediate_, gate_.k_bits(),
                                 (int)gate_.codebook(), gpu.raw_stream()) != 0)
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
    bool uniform_ = false, has_bias_ = false;
    DeviceBuffer<Half> g_, u_, x_had_, act_had_;
    mutable DeviceBuffer<Half> h_norm_;     // scratch of forward_block, allocated on first use
};

// An EXL3 linear that stacks `blocks` equal linears along K: tile rows [b * K/16, (b+1) * K/16)
// and input scales [b * K, (b+1) * K) belong to block b; the output scale either spans the
// columns once or once per block.  window() copies one block's rows, restricted to a column
// range, into an ordinary linear.  This is how a checkpoint's `experts.gate_up_proj` /
// `experts.down_proj` pair (crates/berth-plan/tests/plan.rs:111-118) is read here; the reference
// names those tensors but never opens one, so the stacking order is this loader's assumption.
class StackedLinear {
public:
    StackedLinear(const exl3::Checkpoint& ckpt, const std::string& prefix, int blocks) : prefix_(prefix), blocks_(blocks)
    {
        const exl3::LinearExl3& linear = find_linear(ckpt, prefix);
        note_unpinned(Unpinned::StackedExperts, prefix);
        if (linear.k.is_half()) throw WeightsError(prefix + ": half-integer rate");
        if (linear.input_scale.packed || linear.output_scale.packed)
            throw WeightsError(prefix + ": packed signs in a stacked expert tensor");
        if (linear.bias) throw WeightsError(prefix + ": bias is present and is not applied");
        bits_ = linear.k.whole();
        tiles_k_all_ = linear.trellis.shape[0];
        tiles_n_ = linear.trellis.shape[1];
        codebook_ = linear.codebook == exl3::Codebook::Mul1  ? Codebook::Mul1
                    : linear.codebook == exl3::Codebook::Mcg ? Codebook::Mcg
                                                             : Codebook::Default;
        if (blocks < 1 || tiles_k_all_ % (uint64_t)blocks)
            throw WeightsError(prefix + ": " + std::to_string(tiles_k_all_) + " tile rows do not split into " +
                               std::to_string(blocks) + " experts");
        trellis_ = exl3::read_tensor(linear.trellis);
        suh_ = exl3::read_tensor(linear.input_scale.tensor);
        svh_ = exl3::read_tensor(linear.output_scale.tensor);
        const uint64_t n = tiles_n_ * 16;
        if (suh_.size() / 2 != tiles_k_all_ * 16 || (svh_.size() / 2 != n && svh_.size() / 2 != n * (uint64_t)blocks))
            throw WeightsError(prefix + ": scales do not match the stacked tensor");
        svh_per_block_ = blocks > 1 && svh_.size() / 2 == n * (uint64_t)blocks;
    }
    int size_k() const { return (int)(tiles_k_all_ / (uint64_t)blocks_ * 16); }
    int size_n() const { return (int)(tiles_n_ * 16); }

    Exl3Linear window(const Gpu& gpu, const std::string& name, int block, int n0, int n) const
    {
        const uint64_t tiles_k = tiles_k_all_ / (uint64_t)blocks_, words = 16ull * bits_;
        if (block < 0 || block >= blocks_ || n0 < 0 || n < 16 || n0 % 16 || n % 16 || (uint64_t)(n0 + n) > tiles_n_ * 16)
            throw WeightsError(prefix_ + ": window " + name + " lies outside the stacked tensor");
        std::vector<uint16_t> tr((size_t)(tiles_k * (n / 16) * words));
        const uint16_t* src = (const uint16_t*)trellis_.data();
        for (uint64_t r = 0; r < tiles_k; ++r)
            std::memcpy(tr.data() + r * (n / 16) * words,
                        src + (((uint64_t)block * tiles_k + r) * tiles_n_ + (uint64_t)n0 / 16) * words,
                        (size_t)(n / 16) * words * 2);
        const Half* su = (const Half*)suh_.data() + (size_t)block * tiles_k * 16;
        const Half* sv = (const Half*)svh_.data() + (svh_per_block_ ? (size_t)block * tiles_n_ * 16 : 0) + n0;
        return Exl3Linear(gpu, name, tr.data(), tr.size(), su, (int)(tiles_k * 16), sv, n, codebook_);
    }

private:
    std::string prefix_;
    int blocks_, bits_ = 0;
    uint64_t tiles_k_all_ = 0, tiles_n_ = 0;
    bool svh_per_block_ = false;
    Codebook codebook_ = Codebook::Mul1;
    std::vector<uint8_t> trellis_, suh_, svh_;
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
    // Layer `layer`'s MoE block from a checkpoint, sized by the plan's Ffn::Moe record
    // (crates/berth-plan/src/plan.rs:45-57; tensor names as in crates/berth-plan/tests/plan.rs:96-120
    // and tests/from_exl3_bytes.rs):
    //   {mlp}.gate.weight                      router, [experts][hidden] in F16 / BF16 / F32 as a linear
    //                                          layer stores it; transposed here to [hidden][experts] fp16
    //   {mlp}.experts.<e>.{gate,up,down}_proj  one EXL3 linear per routed expert and projection, or
    //   {mlp}.experts.{gate_up,down}_proj      the stacked pair (StackedLinear; gate columns, then up)
    //   {mlp}.shared_expert.{gate,up,down}_proj the always-on expert
    //   {mlp}.shared_expert_gate.weight        optional, [1][hidden] or [hidden] in F16 / BF16 / F32: the
    //                                          always-on expert's row of token t is scaled by
    //                                          sigmoid(x[t] . weight) (the reference never opens this
    //                                          tensor: the formula is this loader's assumption)
    // with {mlp} = model.language_model.layers.<layer>.mlp.  Refused: a plan layer that is not MoE,
    // sizes that differ from the plan's, a quantized router and a bias on an expert linear (the
    // grouped launches have no place for it).
    static MoeLayer load(const Gpu& gpu, const exl3::Checkpoint& ckpt, uint32_t layer, const plan::Ffn& ffn,
                         bool renorm = true)
    {
        if (!ffn.is_moe) throw InputError("moe: layer " + std::to_string(layer) + " is planned with a dense MLP");
        const std::string mlp = "model.language_model.layers." + std::to_string(layer) + ".mlp";
        const int E = (int)ffn.router.num_experts, I = (int)ffn.experts.intermediate_size;

        if (ckpt.find_linear(mlp + ".gate")) throw WeightsError(mlp + ".gate: a quantized router is not handled");
        const exl3::TensorInfo* gate = ckpt.tensors.get(mlp + ".gate.weight");
        if (!gate) throw WeightsError("tensor " + mlp + ".gate.weight is missing");
        if (gate->shape.size() != 2 || gate->shape[0] != (uint64_t)E)
            throw WeightsError(gate->name + ": expected [" + std::to_string(E) + "][hidden]");
        const int H = (int)gate->shape[1];
        const std::vector<float> w = read_float_tensor(*gate);
        std::vector<Half> router((size_t)H * E);
        for (int e = 0; e < E; ++e)
            for (int h = 0; h < H; ++h) router[(size_t)h * E + e] = f32_to_f16_bits(w[(size_t)e * H + h]);
        std::vector<float> shared_gate;
        if (const exl3::TensorInfo* sg = ckpt.tensors.get(mlp + ".shared_expert_gate.weight")) {
            uint64_t n = 1;
            for (uint64_t d : sg->shape) n *= d;
            if (n != (uint64_t)H || sg->shape.size() > 2)
                throw WeightsError(sg->name + ": expected [1][" + std::to_string(H) + "]");
            shared_gate = read_float_tensor(*sg);
            note_unpinned(Unpinned::SharedExpertGate, sg->name);
        }

        auto checked = [&](Exl3Linear lin, int k, int n) {
            if (lin.size_k() != k || lin.size_n() != n)
                throw WeightsError(lin.prefix() + ": " + std::to_string(lin.size_k()) + "x" + std::to_string(lin.size_n()) +
                                   " where the plan has " + std::to_string(k) + "x" + std::to_string(n));
            if (lin.has_bias()) throw WeightsError(lin.prefix() + ": bias is present and is not applied");
            return lin;
        };
        std::vector<Expert> experts;
        experts.reserve((size_t)E);
        const std::string pool = mlp + ".experts";
        if (ckpt.find_linear(pool + ".gate_up_proj")) {
            const StackedLinear gate_up(ckpt, pool + ".gate_up_proj", E), down(ckpt, pool + ".down_proj", E);
            if (gate_up.size_k() != H || gate_up.size_n() != 2 * I || down.size_k() != I || down.size_n() != H)
                throw WeightsError(pool + ": stacked tensors are " + std::to_string(gate_up.size_k()) + "x" +
                                   std::to_string(gate_up.size_n()) + " and " + std::to_string(down.size_k()) + "x" +
                                   std::to_string(down.size_n()) + " per expert where the plan has " + std::to_string(H) +
                                   "x" + std::to_string(2 * I) + " and " + std::to_string(I) + "x" + std::to_string(H));
            for (int e = 0; e < E; ++e) {
                const std::string p = pool + "." + std::to_string(e);
                experts.push_back(Expert{gate_up.window(gpu, p + ".gate_proj", e, 0, I),
                                         gate_up.window(gpu, p + ".up_proj", e, I, I),
                                         down.window(gpu, p + ".down_proj", e, 0, H)});
            }
        } else {
            for (int e = 0; e < E; ++e) {
                const std::string p = pool + "." + std::to_string(e);
                experts.push_back(Expert{checked(Exl3Linear::load(gpu, ckpt, p + ".gate_proj"), H, I),
                                         checked(Exl3Linear::load(gpu, ckpt, p + ".up_proj"), H, I),
                                         checked(Exl3Linear::load(gpu, ckpt, p + ".down_proj"), I, H)});
            }
        }
        MoeLayer out(gpu, router.data(), H, E, std::move(experts), (int)ffn.router.experts_per_tok, nullptr, renorm);
        const int SI = (int)ffn.shared.intermediate_size;
        const std::string sh = mlp + ".shared_expert";
        out.set_shared(Expert{checked(Exl3Linear::load(gpu, ckpt, sh + ".gate_proj"), H, SI),
                              checked(Exl3Linear::load(gpu, ckpt, sh + ".up_proj"), H, SI),
                              checked(Exl3Linear::load(gpu, ckpt, sh + ".down_proj"), SI, H)});
        if (!shared_gate.empty()) out.set_shared_gate(gpu, shared_gate);
        return out;
    }
    int hidden() const { return hidden_; }
    int num_experts() const { return num_experts_; }
    int top_k() const { return top_k_; }
    int intermediate() const { return intermediate_; }
    int shared_intermediate() const { return shared_.empty() ? 0 : shared_[0].gate.size_n(); }

    void set_shared(Expert shared)
    {
        if (shared.gate.k_bits() != k_bits_ || shared.up.k_bits() != k_bits_ || shared.down.k_bits() != k_bits_ ||
            shared.gate.codebook() != codebook_)
            throw InputError("moe: the shared expert must use the routed experts' bit rate and codebook");
        shared_.clear();
        shared_.push_back(std::move(shared));
    }

    // weights [hidden] of the per-token scale sigmoid(x . w) on the always-on expert's row
    void set_shared_gate(const Gpu& gpu, const std::vector<float>& w)
    {
        if (shared_.empty()) throw InputError("moe: a shared-expert gate without a shared expert");
        if ((int)w.size() != hidden_)
            throw InputError("moe: shared-expert gate has " + std::to_string(w.size()) + " weights for hidden size " +
                             std::to_string(hidden_));
        shared_gate_ = DeviceBuffer<float>::from_host(gpu, w);
    }
    bool has_shared_gate() const { return shared_gate_.len() != 0; }

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
        if (berth_moe_layer_gated(x.raw(), router_.raw(), bias_.len() ? (const float*)bias_.raw() : nullptr,
                                  table_.raw(), shared_.empty() ? nullptr : sh,
                                  shared_gate_.len() ? (const float*)shared_gate_.raw() : nullptr, out.raw(),
                                  idx_out ? (int32_t*)idx_out->raw() : nullptr, w_out ? (float*)w_out->raw() : nullptr,
                                  ws_.raw(), ws_.len(), tokens, hidden_, num_experts_, top_k_, intermediate_, shared_i,
                                  k_bits_, (int)codebook_, renorm_ ? 1 : 0, gpu.raw_stream()) != 0)
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
    DeviceBuffer<float> shared_gate_;
    DeviceBuffer<uint8_t> ws_;
};

}  // namespace berth::engine

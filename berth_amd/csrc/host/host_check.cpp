// Runs the C++ host layer (engine.hpp) on case files written by the test suite and
// writes the results back, so that the tests can compare them with the CPU oracle:
//   host_check linear <dir>   meta.txt: K N rows out_fp32 mode(0 forward/forward_n, 1 forward_rows)
//   host_check mlp <dir>      meta.txt: hidden intermediate rows [fused(0/1)]
//   host_check moe <dir>      meta.txt: tokens hidden experts top_k intermediate shared(0/1) has_bias(0/1)
//   host_check ckpt-info <checkpoint dir>                    (no device) lists the linears the reader found
//   host_check ckpt-linear <checkpoint dir> <prefix> <dir>   Exl3Linear::load, one row of <dir>/x.bin, fp32 out
//   host_check ckpt-mlp <checkpoint dir> <layer> <dir>       MlpLayer::load, one row of <dir>/x.bin
//   host_check ckpt-plan <checkpoint dir>                    (no device) config -> shape -> plan -> placement
//   host_check f16 <dir>                                     (no device) x.f32 -> fp16 bits y.u16 and back y.f32
//   host_check ckpt-moe <checkpoint dir> <layer> <dir>       MoeLayer::load from the plan's Ffn::Moe record,
//                                                            meta.txt: tokens; x.bin [tokens][hidden]
// Tensors are raw little-endian files in <dir>; outputs go to <dir>/y.bin (+ idx.bin).
#include "engine.hpp"

#include <cstdio>
#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>

using namespace berth::engine;

template <typename T>
static std::vector<T> read_file(const std::string& path)
{
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) throw std::runtime_error("cannot open " + path);
    const std::streamsize n = f.tellg();
    f.seekg(0);
    std::vector<T> v((size_t)n / sizeof(T));
    f.read((char*)v.data(), n);
    return v;
}

template <typename T>
static void write_file(const std::string& path, const std::vector<T>& v)
{
    std::ofstream f(path, std::ios::binary);
    f.write((const char*)v.data(), (std::streamsize)(v.size() * sizeof(T)));
}

static std::vector<long> read_meta(const std::string& dir)
{
    std::ifstream f(dir + "/meta.txt");
    if (!f) throw std::runtime_error("cannot open " + dir + "/meta.txt");
    std::vector<long> v;
    long x;
    while (f >> x) v.push_back(x);
    return v;
}

static Exl3Linear load_linear(const Gpu& gpu, const std::string& dir, const std::string& name, int K, int N)
{
    const auto tr = read_file<uint16_t>(dir + "/" + name + ".trellis.bin");
    const auto suh = read_file<Half>(dir + "/" + name + ".suh.bin");
    const auto svh = read_file<Half>(dir + "/" + name + ".svh.bin");
    if ((int)suh.size() != K || (int)svh.size() != N) throw InputError(name + ": suh / svh length");
    return Exl3Linear(gpu, name, tr.data(), tr.size(), suh.data(), K, svh.data(), N);
}

static int run_linear(const Gpu& gpu, const std::string& dir)
{
    const auto m = read_meta(dir);
    const int K = (int)m.at(0), N = (int)m.at(1), rows = (int)m.at(2);
    const OutDtype out = m.at(3) ? OutDtype::F32 : OutDtype::F16;
    const bool use_rows = m.at(4) != 0;
    Exl3Linear lin = load_linear(gpu, dir, "lin", K, N);
    const auto x = DeviceBuffer<Half>::from_host(gpu, read_file<Half>(dir + "/x.bin"));
    auto c = DeviceBuffer<uint8_t>::zeroed(gpu, (size_t)rows * N * out_bytes(out));

    // a buffer that is too small is refused before anything is launched (device.rs:132-140)
    bool refused = false;
    try {
        lin.forward(gpu, x, c.ptr(), 2, out);
    } catch (const InputError&) {
        refused = true;
    }
    if (!refused) throw std::runtime_error("short output buffer was not refused");

    berth_hip_event *e0 = nullptr, *e1 = nullptr;
    device_ok(berth_hip_event_new(gpu.context(), &e0), "event");
    device_ok(berth_hip_event_new(gpu.context(), &e1), "event");
    device_ok(berth_hip_event_record(e0, gpu.stream()), "record");
    if (use_rows) {
        RowScratch scratch(gpu, rows, K, N);
        lin.forward_rows(gpu, scratch, x, c.ptr(), c.num_bytes(), rows, out);
    } else {
        auto a_had = DeviceBuffer<Half>::zeroed(gpu, (size_t)rows * K);
        lin.forward_n(gpu, a_had, x, c.ptr(), c.num_bytes(), rows, out);
    }
    device_ok(berth_hip_event_record(e1, gpu.stream()), "record");
    device_ok(berth_hip_event_synchronize(e1), "event synchronize");
    float ms = -1.0f;
    device_ok(berth_hip_event_elapsed_ms(e0, e1, &ms), "elapsed");
    berth_hip_event_free(e0);
    berth_hip_event_free(e1);
    write_file(dir + "/y.bin", c.copy_to_host());
    std::printf("linear ok rows=%d elapsed_ms=%.3f launch=%s\n", rows, ms,
                rows == 1 ? berth_exl3_last_launch() : berth_prefill_last_launch());
    return 0;
}

// meta: K rows fp32 N_0 N_1 ...; sources src0, src1, ...; outputs y0.bin, y1.bin, ...
static int run_bundle(const Gpu& gpu, const std::string& dir)
{
    const auto m = read_meta(dir);
    const int K = (int)m.at(0), rows = (int)m.at(1);
    const OutDtype out = m.at(2) ? OutDtype::F32 : OutDtype::F16;
    std::vector<Exl3Linear> lins;
    for (size_t i = 3; i < m.size(); ++i) lins.push_back(load_linear(gpu, dir, "src" + std::to_string(i - 3), K, (int)m[i]));
    std::vector<const Exl3Linear*> sources;
    for (const Exl3Linear& l : lins) sources.push_back(&l);
    MultiLinear multi(gpu, sources);
    const auto x = DeviceBuffer<Half>::from_host(gpu, read_file<Half>(dir + "/x.bin"));
    std::vector<DeviceBuffer<uint8_t>> ys;
    std::vector<uint64_t> outs;
    for (const Exl3Linear& l : lins) {
        ys.push_back(DeviceBuffer<uint8_t>::zeroed(gpu, (size_t)rows * l.size_n() * out_bytes(out)));
        outs.push_back(ys.back().ptr());
    }
    bool refused = false;
    try {
        multi.forward(gpu, x, {outs[0]}, rows, out);            // one output for several sources
    } catch (const InputError&) {
        refused = true;
    }
    if (!refused && lins.size() > 1) throw std::runtime_error("a short output list was not refused");
    multi.forward(gpu, x, outs, rows, out);
    multi.forward(gpu, x, outs, rows, out);                     // the second call finds its lists in place
    gpu.synchronize();
    for (size_t i = 0; i < ys.size(); ++i) write_file(dir + "/y" + std::to_string(i) + ".bin", ys[i].copy_to_host());
    std::printf("bundle ok rows=%d slices=%d width=%d launch=%s\n", rows, multi.slices(), multi.width(), berth_ops_last_launch());
    return 0;
}

static int run_mlp(const Gpu& gpu, const std::string& dir)
{
    const auto m = read_meta(dir);
    const int H = (int)m.at(0), I = (int)m.at(1), rows = (int)m.at(2);
    MlpLayer mlp(gpu, load_linear(gpu, dir, "gate", H, I), load_linear(gpu, dir, "up", H, I),
                 load_linear(gpu, dir, "down", I, H), rows);
    const auto x = DeviceBuffer<Half>::from_host(gpu, read_file<Half>(dir + "/x.bin"));
    auto y = DeviceBuffer<float>::zeroed(gpu, (size_t)rows * H);
    const bool fused = m.size() > 3 && m[3] != 0;
    if (fused) {
        mlp.forward_fused(gpu, x, y, rows);
    } else if (rows == 1) {
        mlp.forward(gpu, x, y);
    } else {
        RowScratch scratch(gpu, rows, H > I ? H : I, H > I ? H : I);
        mlp.prefill(gpu, scratch, x, y, rows);
    }
    gpu.synchronize();
    write_file(dir + "/y.bin", y.copy_to_host());
    std::printf("mlp ok rows=%d fused=%d launch=%s\n", rows, fused ? 1 : 0, fused ? berth_exl3_last_launch() : "");
    return 0;
}

static int run_moe(const Gpu& gpu, const std::string& dir)
{
    const auto m = read_meta(dir);
    const int T = (int)m.at(0), H = (int)m.at(1), E = (int)m.at(2), k = (int)m.at(3), I = (int)m.at(4);
    const bool shared = m.at(5) != 0, has_bias = m.at(6) != 0;
    std::vector<MoeLayer::Expert> experts;
    for (int e = 0; e < E; ++e) {
        const std::string p = "e" + std::to_string(e);
        experts.push_back(MoeLayer::Expert{load_linear(gpu, dir, p + ".gate", H, I), load_linear(gpu, dir, p + ".up", H, I),
                                           load_linear(gpu, dir, p + ".down", I, H)});
    }
    const auto router = read_file<Half>(dir + "/router.bin");
    std::vector<float> bias;
    if (has_bias) bias = read_file<float>(dir + "/bias.bin");
    MoeLayer layer(gpu, router.data(), H, E, std::move(experts), k, has_bias ? bias.data() : nullptr);
    if (shared)
        layer.set_shared(MoeLayer::Expert{load_linear(gpu, dir, "shared.gate", H, I), load_linear(gpu, dir, "shared.up", H, I),
                                          load_linear(gpu, dir, "shared.down", I, H)});
    const auto x = DeviceBuffer<Half>::from_host(gpu, read_file<Half>(dir + "/x.bin"));
    auto y = DeviceBuffer<float>::zeroed(gpu, (size_t)T * H);
    auto idx = DeviceBuffer<int32_t>::zeroed(gpu, (size_t)T * k);
    layer.forward(gpu, x, y, T, &idx);
    gpu.synchronize();
    write_file(dir + "/y.bin", y.copy_to_host());
    write_file(dir + "/idx.bin", idx.copy_to_host());
    std::printf("moe ok tokens=%d launch=%s\n", T, berth_moe_last_launch());
    return 0;
}

static int run_ckpt_info(const std::string& dir)
{
    const berth::exl3::Checkpoint ckpt = berth::exl3::Checkpoint::open(dir);
    std::printf("arch=%s layers=%u hidden=%u tensors=%zu linears=%zu other=%zu\n", ckpt.config.arch_string.c_str(),
                ckpt.config.num_hidden_layers, ckpt.config.hidden_size, ckpt.tensors.len(), ckpt.linears().size(),
                ckpt.other_tensors().size());
    for (const auto& l : ckpt.linears())
        std::printf("linear %s k=%s codebook=%d packed=%d/%d bias=%d\n", l.prefix.c_str(), l.k.to_string().c_str(),
                    (int)l.codebook, (int)l.input_scale.packed, (int)l.output_scale.packed, l.bias ? 1 : 0);
    return 0;
}

static int run_ckpt_linear(const Gpu& gpu, const std::string& ckpt_dir, const std::string& prefix, const std::string& dir)
{
    const berth::exl3::Checkpoint ckpt = berth::exl3::Checkpoint::open(ckpt_dir);
    Exl3Linear lin = Exl3Linear::load(gpu, ckpt, prefix);
    const auto x = DeviceBuffer<Half>::from_host(gpu, read_file<Half>(dir + "/x.bin"));
    auto y = DeviceBuffer<float>::zeroed(gpu, (size_t)lin.size_n());
    lin.forward(gpu, x, y.ptr(), y.num_bytes(), OutDtype::F32);
    gpu.synchronize();
    write_file(dir + "/y.bin", y.copy_to_host());
    std::printf("ckpt-linear ok %s K=%d N=%d bits=%d codebook=%d launch=%s\n", lin.prefix().c_str(), lin.size_k(),
                lin.size_n(), lin.k_bits(), (int)lin.codebook(), berth_exl3_last_launch());
    return 0;
}

static int run_ckpt_mlp(const Gpu& gpu, const std::string& ckpt_dir, uint32_t layer, const std::string& dir)
{
    const berth::exl3::Checkpoint ckpt = berth::exl3::Checkpoint::open(ckpt_dir);
    MlpLayer mlp = MlpLayer::load(gpu, ckpt, layer);
    const auto x = DeviceBuffer<Half>::from_host(gpu, read_file<Half>(dir + "/x.bin"));
    auto y = DeviceBuffer<float>::zeroed(gpu, (size_t)mlp.hidden());
    mlp.forward(gpu, x, y);
    gpu.synchronize();
    write_file(dir + "/y.bin", y.copy_to_host());
    std::printf("ckpt-mlp ok layer=%u hidden=%d intermediate=%d\n", layer, mlp.hidden(), mlp.intermediate());
    return 0;
}

static int run_ckpt_plan(const std::string& ckpt_dir)
{
    namespace plan = berth::plan;
    const berth::exl3::Checkpoint ckpt = berth::exl3::Checkpoint::open(ckpt_dir);
    const plan::ModelPlan model = plan::build_plan(plan::model_shape(ckpt.config));
    const plan::TensorBytes bytes = plan::tensor_bytes(ckpt);
    const plan::Placement placed = plan::place(model, bytes, plan::HbmBudget{});
    size_t moe_layers = 0, expert_tensors = 0;
    for (const plan::LayerPlan& l : model.layers) moe_layers += l.ffn.is_moe ? 1 : 0;
    for (const auto& t : bytes.tensors) expert_tensors += plan::is_routed_expert(t.first) ? 1 : 0;
    std::printf("plan arch=%s layers=%zu moe_layers=%zu tensors=%zu expert_tensors=%zu resident=%llu "
                "bytes_moved=%llu\n",
                model.arch_string.c_str(), model.layers.size(), moe_layers, bytes.tensors.size(), expert_tensors,
                (unsigned long long)placed.resident, (unsigned long long)placed.bytes_moved);
    if (moe_layers) {
        const plan::Ffn& f = model.layers[0].ffn;
        std::printf("ffn router=%u/%u shared=%u experts=%u/%u/%u\n", f.router.num_experts, f.router.experts_per_tok,
                    f.shared.intermediate_size, f.experts.num_experts, f.experts.experts_per_tok,
                    f.experts.intermediate_size);
    }
    return 0;
}

static int run_ckpt_moe(const Gpu& gpu, const std::string& ckpt_dir, uint32_t layer, const std::string& dir)
{
    namespace plan = berth::plan;
    const berth::exl3::Checkpoint ckpt = berth::exl3::Checkpoint::open(ckpt_dir);
    const plan::ModelPlan model = plan::build_plan(plan::model_shape(ckpt.config));
    if (layer >= model.layers.size()) throw InputError("layer " + std::to_string(layer) + " is not in the plan");
    MoeLayer moe = MoeLayer::load(gpu, ckpt, layer, model.layers[layer].ffn);
    const int T = (int)read_meta(dir).at(0);
    const auto x = DeviceBuffer<Half>::from_host(gpu, read_file<Half>(dir + "/x.bin"));
    auto y = DeviceBuffer<float>::zeroed(gpu, (size_t)T * moe.hidden());
    auto idx = DeviceBuffer<int32_t>::zeroed(gpu, (size_t)T * moe.top_k());
    moe.forward(gpu, x, y, T, &idx);
    gpu.synchronize();
    write_file(dir + "/y.bin", y.copy_to_host());
    write_file(dir + "/idx.bin", idx.copy_to_host());
    std::printf("ckpt-moe ok layer=%u tokens=%d hidden=%d experts=%d top_k=%d intermediate=%d shared=%d launch=%s\n", layer, T,
                moe.hidden(), moe.num_experts(), moe.top_k(), moe.intermediate(), moe.shared_intermediate(),
                berth_moe_last_launch());
    return 0;
}

int main(int argc, char** argv)
{
    if (argc < 3) {
        std::fprintf(stderr, "usage: host_check linear|mlp|moe <dir> | ckpt-info <ckpt> | ckpt-plan <ckpt> | ckpt-linear <ckpt> "
                             "<prefix> <dir> | ckpt-mlp <ckpt> <layer> <dir> | ckpt-moe <ckpt> <layer> <dir>\n");
        return 2;
    }
    try {
        const std::string what = argv[1], dir = argv[2];
        if (what == "ckpt-info") return run_ckpt_info(dir);
        if (what == "ckpt-plan") return run_ckpt_plan(dir);
        if (what == "f16") {
            const auto x = read_file<float>(dir + "/x.f32");
            std::vector<Half> h(x.size());
            std::vector<float> back(x.size());
            for (size_t i = 0; i < x.size(); ++i) {
                h[i] = f32_to_f16_bits(x[i]);
                back[i] = f16_bits_to_f32(h[i]);
            }
            write_file(dir + "/y.u16", h);
            write_file(dir + "/y.f32", back);
            return 0;
        }
        Gpu gpu(0);
        if (what == "ckpt-linear" && argc >= 5) return run_ckpt_linear(gpu, dir, argv[3], argv[4]);
        if (what == "ckpt-mlp" && argc >= 5) return run_ckpt_mlp(gpu, dir, (uint32_t)std::stoul(argv[3]), argv[4]);
        if (what == "ckpt-moe" && argc >= 5) return run_ckpt_moe(gpu, dir, (uint32_t)std::stoul(argv[3]), argv[4]);
        if (what == "linear") return run_linear(gpu, dir);
        if (what == "bundle") return run_bundle(gpu, dir);
        if (what == "mlp") return run_mlp(gpu, dir);
        if (what == "moe") return run_moe(gpu, dir);
        std::fprintf(stderr, "unknown case %s\n", what.c_str());
        return 2;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "host_check failed: %s\n", e.what());
        return 1;
    }
}

// Times BASELINE's configurations through the host layer, i.e. along the whole drop-in path:
// lazy graph construction, signature, plan cache, kernel launches, with a device
// synchronisation closing every materialisation (the reference's fusion benchmark
// materialises through item(): benchmarks/core/fusion/fusion_benchmark.cpp:38-49, 62-72).
// Prints one JSON object.  Inputs are synthetic and resident on the GPU before timing.
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "axhip.h"
#include "axiom/axiom.hpp"

using namespace axiom;
using Clock = std::chrono::steady_clock;

static const char *g_only = nullptr; // argv[3]: run only the configurations whose name contains this

template <typename F> static void measure(const char *name, F f, int warmup, int iters, double work, const char *unit, bool last) {
    if (g_only && !std::strstr(name, g_only)) return;
    for (int i = 0; i < warmup; ++i) f();
    backends::hip::synchronize();
    std::vector<double> us;
    for (int i = 0; i < iters; ++i) {
        const auto t0 = Clock::now();
        f();
        backends::hip::synchronize();
        us.push_back(std::chrono::duration<double, std::micro>(Clock::now() - t0).count());
    }
    std::sort(us.begin(), us.end());
    const double med = us[us.size() / 2];
    // the same work the way a program issues it: materialisations queued back to back (they are asynchronous), one
    // wait for 16 of them
    std::vector<double> piped;
    constexpr int BURST = 16;
    for (int r = 0; r < std::max(4, iters / BURST); ++r) {
        const auto t0 = Clock::now();
        for (int i = 0; i < BURST; ++i) f();
        backends::hip::synchronize();
        piped.push_back(std::chrono::duration<double, std::micro>(Clock::now() - t0).count() / BURST);
    }
    std::sort(piped.begin(), piped.end());
    const double pmed = piped[piped.size() / 2];
    graph::record_gpu_plan_kernels(true); // one more, untimed, to learn which kernels the graph runs on
    f();
    backends::hip::synchronize();
    graph::record_gpu_plan_kernels(false);
    std::string kernels;
    for (const auto &k : graph::last_gpu_plan_kernels()) kernels += (kernels.empty() ? "" : " ") + k;
    (void)last; // every entry leads with its comma, so a filtered run still prints valid JSON
    std::printf(",\n  \"%s\": {\"median_us\": %.1f, \"min_us\": %.1f, \"%s\": %.1f, \"queued_16_per_wait_us\": %.1f, \"queued_%s\": %.1f, \"last_graph_kernels\": \"%s\"}",
                name, med, us.front(), unit, work / (med * 1e-6) / 1e9, pmed, unit, work / (pmed * 1e-6) / 1e9, kernels.c_str());
}

int main(int argc, char **argv) {
    const int iters = argc > 1 ? std::atoi(argv[1]) : 50, warmup = argc > 2 ? std::atoi(argv[2]) : 10;
    g_only = argc > 3 ? argv[3] : nullptr;
    if (!system::is_gpu_available()) {
        std::fprintf(stderr, "host_bench: no GPU visible; the gfx950 backend has no CPU fallback\n");
        return 3;
    }
    Tensor::manual_seed(42);
    std::printf("{\n");
    { // the floor under every figure below: one launch of a kernel that writes four bytes, then the wait for it
        auto one = Tensor::zeros({1}, DType::Float32).gpu();
        void *dst = one.storage()->raw();
        std::vector<double> us;
        for (int i = 0; i < warmup + iters; ++i) {
            const auto t0 = Clock::now();
            axhip_fill(dst, AXHIP_DTYPE_F32, 1.0, 1, nullptr);
            backends::hip::synchronize();
            if (i >= warmup) us.push_back(std::chrono::duration<double, std::micro>(Clock::now() - t0).count());
        }
        std::sort(us.begin(), us.end());
        std::printf("  \"launch_and_wait_floor\": {\"median_us\": %.1f, \"min_us\": %.1f}", us[us.size() / 2], us.front());
    }
    { // configs[0]: the reference's CPU-runnable case, fp32, on the fp32 matrix instruction here
        auto q = Tensor::randn({1, 8, 512, 64}, DType::Float32, Device::GPU), k = Tensor::randn({1, 8, 512, 64}, DType::Float32, Device::GPU),
             v = Tensor::randn({1, 8, 512, 64}, DType::Float32, Device::GPU);
        measure("c1_sdpa_f32_b1h8s512d64", [&] { ops::scaled_dot_product_attention(q, k, v, Tensor(), 0.125f, false).sync(); }, warmup, iters, 536870912.0,
                "GFLOP_per_s", false);
    }
    { // configs[1]
        auto a = Tensor::randn({8192, 8192}, DType::Float32, Device::GPU), b = Tensor::randn({8192, 8192}, DType::Float32, Device::GPU);
        measure("c2_chain_f32_8192x8192", [&] { ops::softmax((ops::relu(a) + 1) * b, -1).sum(1).sync(); }, warmup, iters, 536903680.0, "GB_per_s", false);
    }
    { // configs[2]
        auto x = Tensor::randn({16384, 4096}, DType::BFloat16, Device::GPU);
        auto gamma = Tensor::uniform(0.5, 1.5, {4096}, DType::BFloat16, Device::GPU), beta = Tensor::uniform(-0.1, 0.1, {4096}, DType::BFloat16, Device::GPU);
        measure("c3_gelu_layernorm_bf16_16384x4096", [&] { ops::gelu(ops::layer_norm(x, gamma, beta, -1, 1e-5f)).sync(); }, warmup, iters, 268451840.0, "GB_per_s", false);
        measure("c3_gelu_rmsnorm_bf16_16384x4096", [&] { ops::gelu(ops::rms_norm(x, gamma, -1, 1e-5f)).sync(); }, warmup, iters, 268443648.0, "GB_per_s", false);
    }
    { // configs[3]
        auto q = Tensor::randn({4, 32, 4096, 128}, DType::BFloat16, Device::GPU), k = Tensor::randn({4, 32, 4096, 128}, DType::BFloat16, Device::GPU),
             v = Tensor::randn({4, 32, 4096, 128}, DType::BFloat16, Device::GPU);
        measure("c4_sdpa_bf16_causal_b4h32s4096d128", [&] { ops::scaled_dot_product_attention(q, k, v, Tensor(), -1.0f, true).sync(); }, warmup, iters, 549755813888.0,
                "GFLOP_per_s", false);
    }
    { // configs[4]: y = LN(x + out_proj(SDPA(split(q, k, v))))
        const size_t S = 1500, Dm = 1280;
        auto x = Tensor::randn({1, S, Dm}, DType::BFloat16, Device::GPU);
        std::map<std::string, Tensor> w;
        for (const char *p : {"q_proj", "k_proj", "v_proj", "out_proj"}) {
            w[std::string(p) + ".weight"] = (Tensor::randn({Dm, Dm}, DType::Float32, Device::GPU) * 0.02f).astype(DType::BFloat16);
            w[std::string(p) + ".bias"] = Tensor::zeros({Dm}, DType::BFloat16);
        }
        nn::MultiHeadAttention mha(20);
        mha.load_state_dict(w);
        mha.to(Device::GPU);
        nn::LayerNorm ln;
        ln.load_state_dict({{"weight", Tensor::ones({Dm}, DType::BFloat16)}, {"bias", Tensor::zeros({Dm}, DType::BFloat16)}});
        ln.to(Device::GPU);
        // written as model code is, one step per statement: a Tensor temporary that is still alive when the graph
        // is materialised counts as a handle on its node (see shared_nodes() in gpu_graph.cpp) and would keep the
        // projection's own result in memory instead of letting the residual ride in the GEMM epilogue
        auto block = [&] {
            Tensor y = x + mha.forward(x, x, x);
            y = ln.forward(y);
            y.sync();
        };
        measure("c5_whisper_block_bf16_s1500_d1280_h20", block, warmup, iters, 31180800000.0, "GFLOP_per_s", false);
        // the whole pre-norm encoder layer of the reference's examples/whisper_poc.cpp:57-86:
        // LN -> MHA -> +x -> LN -> fc1 -> gelu -> fc2 -> +h   (24*S*D^2 + 4*S^2*D flop)
        nn::LayerNorm ln2;
        ln2.load_state_dict({{"weight", Tensor::ones({Dm}, DType::BFloat16)}, {"bias", Tensor::zeros({Dm}, DType::BFloat16)}});
        ln2.to(Device::GPU);
        nn::Linear fc1, fc2;
        fc1.load_state_dict({{"weight", (Tensor::randn({4 * Dm, Dm}, DType::Float32, Device::GPU) * 0.02f).astype(DType::BFloat16)}, {"bias", Tensor::zeros({4 * Dm}, DType::BFloat16, Device::GPU)}});
        fc2.load_state_dict({{"weight", (Tensor::randn({Dm, 4 * Dm}, DType::Float32, Device::GPU) * 0.02f).astype(DType::BFloat16)}, {"bias", Tensor::zeros({Dm}, DType::BFloat16, Device::GPU)}});
        auto layer = [&] {
            auto h = ln(x);
            h = x + mha.forward(h, h, h);
            auto y = h + fc2(fc1(ln2(h)).gelu());
            y.sync();
        };
        measure("whisper_encoder_layer_bf16_s1500_d1280_h20", layer, warmup, iters, 24.0 * S * Dm * Dm + 4.0 * S * S * Dm, "GFLOP_per_s", true);
    }
    std::printf("\n}\n");
    return 0;
}

// GPU cases through the host layer: device semantics, lazy fusion, attention, nn modules.
// They follow the reference's tests/test_unified_memory.cpp (device-tag / round-trip /
// auto-sync cases), test_fusion_extended.cpp:456-523, test_cpu_gpu_parity.cpp,
// test_flash_attention.cpp, test_nn_attention.cpp, test_nn_layers.cpp and
// test_tensor_normalization.cpp, with the CPU side of each comparison supplied by the oracle.
#include <map>

#include <atomic>
#include <thread>

#include "oracle_util.hpp"
#include "test_framework.hpp"

using namespace axiom;
using axtest::max_abs_diff;

static std::vector<float> host_floats(const Tensor &t) {
    Tensor c = t.cpu().astype(DType::Float32).ascontiguousarray();
    return std::vector<float>(c.typed_data<float>(), c.typed_data<float>() + c.size());
}

// ------------------------------------------------------------ device semantics
GPU_TEST(DeviceTransfer, GpuTagRoundTripAndAutoSync) { // tests/test_unified_memory.cpp:102-122, 160-191
    auto a = axtest::randn({37, 53}, 1);
    auto g = a.gpu();
    EXPECT_TRUE(g.device() == Device::GPU);
    EXPECT_TRUE(a.device() == Device::CPU);
    EXPECT_NE(g.storage().get(), a.storage().get()); // explicit copy, no shared memory
    EXPECT_TRUE(g.cpu().allclose(a, 0, 0));
    EXPECT_THROW(g.typed_data<float>(), DeviceError);
    EXPECT_THROW(g.item<float>({0, 0}), DeviceError);
    auto r = ops::add(g, g); // compute, then .cpu() waits for it
    EXPECT_TRUE(r.is_lazy());
    EXPECT_NEAR(r.cpu().item<float>({3, 4}), 2 * a.item<float>({3, 4}), 0);
    auto h = a.astype(DType::BFloat16).gpu();
    EXPECT_EQ(h.dtype(), DType::BFloat16);
    EXPECT_TRUE(h.astype(DType::Float32).cpu().allclose(a.astype(DType::BFloat16).astype(DType::Float32), 0, 0)); // GPU cast
    auto t = g.transpose({1, 0});
    EXPECT_FALSE(t.is_contiguous());
    EXPECT_TRUE(t.ascontiguousarray().cpu().allclose(a.transpose({1, 0}).ascontiguousarray(), 0, 0)); // GPU gather
    EXPECT_NEAR(Tensor::full<float>({1}, 7.0f, Device::GPU).item<float>(), 7.0f, 0);
}

// ------------------------------------------------------------------ fusion
GPU_TEST(FusionGpu, BasicAdd) {
    auto a = Tensor::full<float>({64, 64}, 2.0f, Device::GPU);
    auto b = Tensor::full<float>({64, 64}, 3.0f, Device::GPU);
    ASSERT_NEAR(ops::add(a, b).cpu().item<float>({0, 0}), 5.0f, 1e-5f);
}
GPU_TEST(FusionGpu, UnaryChain) {
    auto x = Tensor::full<float>({64, 64}, 4.0f, Device::GPU);
    ASSERT_NEAR(ops::exp(ops::sqrt(x)).cpu().item<float>({0, 0}), std::exp(2.0f), 1e-4f);
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u); // one launch
}
GPU_TEST(FusionGpu, BinaryUnaryFusion) {
    auto a = Tensor::full<float>({64, 64}, -1.0f, Device::GPU);
    auto b = Tensor::full<float>({64, 64}, 0.5f, Device::GPU);
    ASSERT_NEAR(ops::relu(ops::add(a, b)).cpu().item<float>({0, 0}), 0.0f, 1e-6f);
}
GPU_TEST(FusionGpu, LongerChain) {
    auto a = Tensor::full<float>({64, 64}, 0.5f, Device::GPU);
    auto b = Tensor::full<float>({64, 64}, 2.0f, Device::GPU);
    auto c = Tensor::full<float>({64, 64}, -0.5f, Device::GPU);
    auto result = ops::tanh(ops::sigmoid(ops::add(ops::multiply(a, b), c)));
    ASSERT_NEAR(result.cpu().item<float>({0, 0}), std::tanh(1.0f / (1.0f + std::exp(-0.5f))), 1e-4f);
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
}
GPU_TEST(FusionGpu, ReductionAndFusedReduction) {
    auto a = Tensor::full<float>({4, 4}, 2.0f, Device::GPU);
    auto b = Tensor::full<float>({4, 4}, 3.0f, Device::GPU);
    ASSERT_NEAR(ops::sum(a).cpu().item<float>(), 32.0f, 1e-4f);
    auto r = ops::sum(ops::add(a, b));
    EXPECT_EQ(r.shape(), Shape({1}));
    ASSERT_NEAR(r.cpu().item<float>(), 80.0f, 1e-4f); // tests/test_fusion_extended.cpp:346-352
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
    auto big = Tensor::full<float>({1024, 1024}, 2.0f, Device::GPU);
    ASSERT_NEAR(ops::sum(big).cpu().item<float>(), 2097152.0f, 1.0f); // :436-443
    ASSERT_NEAR(ops::mean(big).cpu().item<float>(), 2.0f, 1e-5f);
}
GPU_TEST(FusionGpu, EagerParity) {
    auto a = Tensor::full<float>({32, 32}, 1.5f, Device::GPU);
    auto b = Tensor::full<float>({32, 32}, 0.5f, Device::GPU);
    const float lazy_val = ops::sigmoid(ops::add(a, b)).cpu().item<float>({0, 0});
    {
        graph::EagerModeScope eager;
        auto s = ops::add(a, b);
        EXPECT_FALSE(s.is_lazy() && !s.lazy_node()->is_materialized_); // every op ran at once
        ASSERT_NEAR(lazy_val, ops::sigmoid(s).cpu().item<float>({0, 0}), 1e-6f);
    }
}
GPU_TEST(FusionGpu, LongChainOfScalars) { // tests/test_fusion_extended.cpp:561-572
    auto x = Tensor::ones({8}, DType::Float32, Device::GPU);
    for (int i = 0; i < 10; ++i) x = x + 1.0f;
    EXPECT_NEAR(x.cpu().item<float>({3}), 11.0f, 0);
    auto y = Tensor::ones({8}, DType::Float32, Device::GPU);
    for (int i = 0; i < 40; ++i) y = y * 1.0f + 1.0f; // longer than one kernel's chain: split, still right
    EXPECT_NEAR(y.cpu().item<float>({0}), 41.0f, 0);
}
GPU_TEST(FusionGpu, SharedNodesAndRecompute) { // tests/test_fusion_extended.cpp:252-299
    auto a = axtest::randn({16, 32}, 3).gpu();
    auto s = ops::exp(a);             // consumed twice below: materialised once
    auto y = ops::add(ops::relu(s), ops::sqrt(s));
    auto want = host_floats(a);
    auto got = host_floats(y);
    for (size_t i = 0; i < want.size(); ++i) {
        const float e = std::exp(want[i]);
        EXPECT_NEAR(got[i], std::max(e, 0.0f) + std::sqrt(e), 1e-4 * (1 + std::fabs(e)));
    }
    EXPECT_TRUE(s.lazy_node() == nullptr || s.lazy_node()->is_materialized_); // the shared node kept its result
    EXPECT_NEAR(s.cpu().item<float>({0, 0}), std::exp(want[0]), 1e-5 * std::exp(want[0]) + 1e-6);
    auto x = ops::relu(a);            // fused through by z; reading x later recomputes it
    auto z = x + 1.0f;
    EXPECT_NEAR(z.cpu().item<float>({1, 1}), std::max(want[33], 0.0f) + 1.0f, 1e-6);
    EXPECT_NEAR(x.cpu().item<float>({1, 1}), std::max(want[33], 0.0f), 0);
}
GPU_TEST(FusionGpu, PlanCacheHitsAndMisses) { // tests/test_graph_compiler.cpp:79-125
    auto &cache = graph::GraphCache::instance();
    cache.clear();
    auto run = [](size_t n, float v) {
        auto a = Tensor::full<float>({n, 8}, v, Device::GPU);
        return ops::relu(a * 2.0f).cpu().item<float>({0, 0});
    };
    EXPECT_NEAR(run(4, 1.0f), 2.0f, 0);
    EXPECT_EQ(cache.misses(), 1u);
    EXPECT_EQ(cache.hits(), 0u);
    EXPECT_NEAR(run(4, -3.0f), 0.0f, 0); // same structure, other data
    EXPECT_EQ(cache.hits(), 1u);
    EXPECT_NEAR(run(5, 1.5f), 3.0f, 0);  // other shape: new plan
    EXPECT_EQ(cache.misses(), 2u);
    EXPECT_EQ(cache.size(), 2u);
}
GPU_TEST(FusionGpu, TwoHostThreadsMaterialiseAtOnce) {
    // Two host threads build and materialise graphs at the same time: one plan that both share (the plan cache is hit
    // from both sides) and one per thread; every result is checked.  What the threads share is the plan cache, the
    // caching allocator, the device scalar cache and the library's stream.
    auto a = axtest::randn({64, 96}, 5), b = axtest::randn({64, 96}, 6);
    const Tensor ag = a.gpu(), bg = b.gpu();
    const std::vector<float> av = host_floats(a), bv = host_floats(b);
    std::atomic<int> bad{0}, done{0};
    auto worker = [&](int id) {
        try {
            for (int it = 0; it < 200; ++it) {
                Tensor shared = ops::relu(ag + bg) * 2.0f;                                   // same signature in both threads
                Tensor own = id == 0 ? ops::softmax(ag * 0.5f, -1) : ops::sum(ops::square(bg - 1.0f), {1}, false); // one per thread
                const std::vector<float> s = host_floats(shared.cpu()), o = host_floats(own.cpu());
                for (size_t i = 0; i < s.size(); i += 97)
                    if (std::fabs(s[i] - std::max(av[i] + bv[i], 0.0f) * 2.0f) > 1e-5f) ++bad;
                if (id == 0) {
                    for (size_t r = 0; r < 64; r += 9) {
                        double sum = 0;
                        for (size_t c = 0; c < 96; ++c) sum += o[r * 96 + c];
                        if (std::fabs(sum - 1.0) > 1e-4) ++bad;
                    }
                } else {
                    for (size_t r = 0; r < 64; r += 9) {
                        double want = 0;
                        for (size_t c = 0; c < 96; ++c) want += (bv[r * 96 + c] - 1.0) * (bv[r * 96 + c] - 1.0);
                        if (std::fabs(o[r] - want) > 1e-3 * (1.0 + want)) ++bad;
                    }
                }
            }
            ++done;
        } catch (const std::exception &) {
            ++bad;
        }
    };
    std::thread t0(worker, 0), t1(worker, 1);
    t0.join();
    t1.join();
    EXPECT_EQ(done.load(), 2);
    EXPECT_EQ(bad.load(), 0);
}
GPU_TEST(FusionGpu, BroadcastKinds) { // tests/test_cpu_gpu_parity.cpp broadcast cases
    auto a = axtest::randn({4, 5}, 5), row = axtest::randn({5}, 6), col = axtest::randn({4, 1}, 7);
    auto ga = a.gpu();
    auto r = host_floats(ops::multiply(ops::add(ga, row.gpu()), col.gpu()));
    auto d = host_floats(ops::subtract(col.gpu(), ga)); // chain on the right-hand side
    auto o = host_floats(ops::add(col.gpu(), row.gpu())); // both operands broadcast
    for (size_t i = 0; i < 4; ++i)
        for (size_t j = 0; j < 5; ++j) {
            const float av = a.item<float>({i, j}), rv = row.item<float>({j}), cv = col.item<float>({i, 0});
            EXPECT_NEAR(r[i * 5 + j], (av + rv) * cv, 0);
            EXPECT_NEAR(d[i * 5 + j], cv - av, 0);
            EXPECT_NEAR(o[i * 5 + j], cv + rv, 0);
        }
    EXPECT_NEAR((2.0f / Tensor::full<float>({3}, 4.0f, Device::GPU)).cpu().item<float>({1}), 0.5f, 0);
}

// ------------------------------------------------- BASELINE configs[1]: C2 chain
GPU_TEST(FusedChain, ReluAddMulSoftmaxRowSumIsOneKernel) {
    const size_t R = 256, C = 8192;
    auto a = axtest::randn({R, C}, 11), b = axtest::randn({R, C}, 12);
    auto ga = a.gpu(), gb = b.gpu();
    auto sm = ops::softmax((ops::relu(ga) + 1) * gb, -1);
    auto out = sm.sum(1);
    auto got = host_floats(out);
    ASSERT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
    EXPECT_EQ(graph::last_gpu_plan_kernels()[0], std::string("rows_static_relu_adds_mulf_softmax_sum_f32_g256_it8"));
    std::vector<float> want(R), want_sm(R * C);
    axo_chain_relu_add_mul_softmax_sum(a.typed_data<float>(), b.typed_data<float>(), want.data(), want_sm.data(), R, C);
    for (size_t i = 0; i < R; ++i) EXPECT_NEAR(got[i], want[i], 1e-4 + 1e-4 * std::fabs(want[i]));
    // the intermediate softmax, evaluated on its own
    auto got_sm = host_floats(ops::softmax((ops::relu(ga) + 1) * gb, -1));
    double worst = 0;
    for (size_t i = 0; i < R * C; ++i) worst = std::max(worst, std::fabs(double(got_sm[i]) - want_sm[i]) - 1e-4 * std::fabs(want_sm[i]));
    EXPECT_LE(worst, 1e-4);
}

// ---------------------------------------------- BASELINE configs[2]: norm chains
static void norm_chain_case(DType dt, bool rms, size_t R, size_t C) {
    auto x = axtest::randn({R, C}, 21, dt), gamma = axtest::uniform({C}, 22, 0.5f, 1.5f, dt), beta = axtest::uniform({C}, 23, -0.1f, 0.1f, dt);
    auto gx = x.gpu(), gg = gamma.gpu(), gb = beta.gpu();
    auto y = rms ? ops::gelu(ops::rms_norm(gx, gg, -1, 1e-5f)) : ops::gelu(ops::layer_norm(gx, gg, gb, -1, 1e-5f));
    EXPECT_EQ(y.dtype(), dt); // the GPU keeps the input dtype (src/graph/graph_registry.cpp:622-627)
    auto got = host_floats(y);
    ASSERT_EQ(graph::last_gpu_plan_kernels().size(), 1u); // norm + gelu in one launch
    // fp32 evaluation of the same (rounded) inputs through the oracle: norm then gelu.  This is the
    // reference's own yardstick for half types (tests/test_flash_attention.cpp:233-249).
    std::vector<float> n(R * C), want(R * C);
    auto xf = x.astype(DType::Float32), gf = gamma.astype(DType::Float32), bf = beta.astype(DType::Float32);
    if (rms) axo_rms_norm(AXO_F32, xf.data(), gf.data(), n.data(), R, C, 1e-5f);
    else axo_layer_norm(AXO_F32, xf.data(), gf.data(), bf.data(), n.data(), R, C, 1e-5f);
    axo_unary(AXO_OP_GELU, AXO_F32, n.data(), want.data(), R * C);
    const double tol = dt == DType::Float32 ? 1e-4 : 2e-2;
    double worst = 0;
    for (size_t i = 0; i < R * C; ++i) worst = std::max(worst, std::fabs(double(got[i]) - want[i]) - (dt == DType::Float32 ? 1e-4 * std::fabs(want[i]) : 0.0));
    EXPECT_LE(worst, tol);
    if (dt != DType::Float32) {
        // distance to the literal CPU path, which rounds the row mean (and for RMS every x*x) to the
        // half type before continuing in fp32 and returns float32: one half-precision ulp of the
        // statistic on top of the output rounding
        const int odt = axtest::oracle_dtype(dt);
        if (rms) axo_rms_norm(odt, x.data(), gamma.data(), n.data(), R, C, 1e-5f);
        else axo_layer_norm(odt, x.data(), gamma.data(), beta.data(), n.data(), R, C, 1e-5f);
        axo_unary(AXO_OP_GELU, AXO_F32, n.data(), want.data(), R * C);
        double lit = 0;
        for (size_t i = 0; i < R * C; ++i) lit = std::max(lit, std::fabs(double(got[i]) - want[i]));
        std::printf("    distance to the literal CPU path (%s, %s): %.4f\n", dtype_name(dt).c_str(), rms ? "rms" : "layer", lit);
        EXPECT_LE(lit, 6e-2);
    }
}
GPU_TEST(FusedChain, GeluLayerNormBf16) { norm_chain_case(DType::BFloat16, false, 64, 4096); }
GPU_TEST(FusedChain, GeluRmsNormBf16) { norm_chain_case(DType::BFloat16, true, 64, 4096); }
GPU_TEST(FusedChain, GeluLayerNormF16OddWidth) { norm_chain_case(DType::Float16, false, 33, 1000); }
GPU_TEST(FusedChain, GeluLayerNormF32) { norm_chain_case(DType::Float32, false, 17, 768); }
GPU_TEST(FusedChain, GeluRmsNormF32Unaligned) { norm_chain_case(DType::Float32, true, 5, 37); }

GPU_TEST(Normalization, KnownAnswers) {
    // tests/test_tensor_normalization.cpp:80-141: [3,4] -> [3,4]/sqrt(12.5)
    float v[2] = {3.0f, 4.0f};
    auto x = Tensor::from_data(v, {1, 2}, Device::GPU);
    auto r = ops::rms_norm(x, Tensor::ones({2}, DType::Float32, Device::GPU), -1, 0.0f).cpu();
    EXPECT_NEAR(r.item<float>({0, 0}), 3.0f / std::sqrt(12.5f), 1e-5);
    EXPECT_NEAR(r.item<float>({0, 1}), 4.0f / std::sqrt(12.5f), 1e-5);
    // layer norm: mean ~ 0, var ~ 1 (tests/test_tensor_normalization.cpp:9-74)
    auto a = axtest::randn({8, 64}, 31);
    auto ln = host_floats(ops::layer_norm(a.gpu(), Tensor(), Tensor(), -1, 1e-5f));
    for (size_t i = 0; i < 8; ++i) {
        double m = 0, q = 0;
        for (size_t j = 0; j < 64; ++j) m += ln[i * 64 + j];
        m /= 64;
        for (size_t j = 0; j < 64; ++j) q += (ln[i * 64 + j] - m) * (ln[i * 64 + j] - m);
        EXPECT_NEAR(m, 0.0, 1e-5);
        EXPECT_NEAR(q / 64, 1.0, 1e-3);
    }
    // softmax rows sum to 1 (tests/test_tensor_activations.cpp:11-52); log_softmax = log(softmax)
    auto sm = host_floats(ops::softmax(a.gpu(), -1)), lsm = host_floats(ops::log_softmax(a.gpu(), -1));
    for (size_t i = 0; i < 8; ++i) {
        double s = 0;
        for (size_t j = 0; j < 64; ++j) s += sm[i * 64 + j];
        EXPECT_NEAR(s, 1.0, 1e-5);
    }
    for (size_t i = 0; i < sm.size(); ++i) EXPECT_NEAR(lsm[i], std::log(sm[i]), 1e-4);
    EXPECT_NEAR(ops::gelu(Tensor::zeros({4}, DType::Float32, Device::GPU)).cpu().item<float>({0}), 0.0f, 0); // :310-334
    { // over the first axis: columns sum to one (the axis and the last one change places around the row kernel)
        auto s0 = host_floats(ops::softmax(a.gpu(), 0));
        const size_t R = a.shape()[0], C = a.shape()[1];
        for (size_t j = 0; j < C; ++j) {
            double t = 0;
            for (size_t i = 0; i < R; ++i) t += s0[i * C + j];
            EXPECT_NEAR(t, 1.0, 1e-5);
        }
    }
}

// Rows whose length no 16-byte vector divides (Whisper's 1500 frames, an odd vocabulary) take the specialised
// kernels' ragged variant; the results are checked against a double-precision evaluation on the host.
GPU_TEST(FusedRows, OddRowLengthsRunOnTheRaggedKernels) {
    const size_t R = 37, C = 1501;
    auto a = axtest::randn({R, C}, 77);
    const float *x = a.typed_data<float>();
    auto sm = host_floats(ops::softmax(a.gpu() * 0.5f, -1));
    ASSERT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
    EXPECT_EQ(graph::last_gpu_plan_kernels()[0], std::string("rows_jit_muls_softmax_f32_g64_it6_grid"));
    auto ln = host_floats(ops::layer_norm(a.gpu(), Tensor(), Tensor(), -1, 1e-5f));
    EXPECT_EQ(graph::last_gpu_plan_kernels()[0], std::string("rows_jit_layernorm_f32_g64_it6_grid"));
    for (size_t i = 0; i < R; ++i) {
        double mx = -1e300, s = 0, mean = 0, var = 0;
        for (size_t j = 0; j < C; ++j) mx = std::max(mx, 0.5 * x[i * C + j]);
        for (size_t j = 0; j < C; ++j) s += std::exp(0.5 * x[i * C + j] - mx), mean += x[i * C + j];
        mean /= C;
        for (size_t j = 0; j < C; ++j) var += (x[i * C + j] - mean) * (x[i * C + j] - mean);
        var /= C;
        for (size_t j = 0; j < C; ++j) {
            EXPECT_NEAR(sm[i * C + j], std::exp(0.5 * x[i * C + j] - mx) / s, 1e-6);
            EXPECT_NEAR(ln[i * C + j], (x[i * C + j] - mean) / std::sqrt(var + 1e-5), 1e-4);
        }
    }
}

// Reductions and softmax over axes other than the last (tests/test_tensor_reductions.cpp: sum / mean / max along
// each axis and along pairs of axes, keep_dims): the kept axes move to the front, the reduced ones fold into the last,
// a row kernel reduces it.  Against double-precision loops on the host.
GPU_TEST(CpuGpuParity, ReductionsAndSoftmaxOverAnyAxis) {
    const Shape sh{5, 7, 6, 9};
    auto a = axtest::randn(sh, 4141);
    const float *x = a.typed_data<float>();
    auto ga = a.gpu();
    const size_t nd = sh.size();
    size_t strides[4] = {7 * 6 * 9, 6 * 9, 9, 1};
    const std::vector<std::vector<int>> axis_sets = {{0}, {1}, {2}, {3}, {0, 1}, {1, 3}, {0, 2, 3}, {-3}, {2, 0}, {0, 1, 2, 3}};
    for (const auto &axes : axis_sets) {
        bool red[4] = {false, false, false, false};
        for (int ax : axes) red[(ax + 4) % 4] = true;
        Shape kept_shape;
        for (size_t i = 0; i < nd; ++i)
            if (!red[i]) kept_shape.push_back(sh[i]);
        size_t kept = 1, count = 1;
        for (size_t i = 0; i < nd; ++i) (red[i] ? count : kept) *= sh[i];
        std::vector<double> sum(kept, 0.0), mx(kept, -1e300);
        for (size_t flat = 0; flat < a.size(); ++flat) {
            size_t out = 0, rest = flat;
            for (size_t i = 0; i < nd; ++i) {
                const size_t idx = rest / strides[i];
                rest %= strides[i];
                if (!red[i]) out = out * sh[i] + idx;
            }
            sum[out] += x[flat];
            mx[out] = std::max(mx[out], static_cast<double>(x[flat]));
        }
        auto gs = ops::sum(ga, axes, false), gm = ops::mean(ga, axes, true), gx = ops::max(ga, axes, false);
        if (!kept_shape.empty()) EXPECT_EQ(gs.shape(), kept_shape); // (over every axis: one element, shaped as the all-axes reduction always was)
        EXPECT_EQ(gm.ndim(), nd);
        auto hs = host_floats(gs), hm = host_floats(gm), hx = host_floats(gx);
        ASSERT_EQ(hs.size(), kept);
        ASSERT_EQ(hm.size(), kept);
        for (size_t i = 0; i < kept; ++i) {
            EXPECT_NEAR(hs[i], sum[i], 1e-4);
            EXPECT_NEAR(hm[i], sum[i] / static_cast<double>(count), 1e-5);
            EXPECT_NEAR(hx[i], mx[i], 0);
        }
    }
    // one run of neighbouring axes that ends before the last one is reduced in place: one kernel, no transposing copy
    {
        ops::sum(ga, {1, 2}, false).sync();
        ASSERT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
        EXPECT_EQ(graph::last_gpu_plan_kernels()[0], std::string("reduce_axis"));
        auto hb = a.astype(DType::BFloat16);
        auto mean16 = ops::mean(hb.gpu(), {0}, false);
        EXPECT_EQ(mean16.dtype(), DType::Float32); // graph_registry.cpp:278-287
        auto hm = host_floats(mean16);
        auto hb32 = hb.astype(DType::Float32);
        for (size_t k = 0; k < 7 * 6 * 9; ++k) {
            double t = 0;
            for (size_t i = 0; i < 5; ++i) t += hb32.typed_data<float>()[i * strides[0] + k];
            EXPECT_NEAR(hm[k], t / 5.0, 1e-5);
        }
    }
    // a chain below such a reduction is materialised first: sum(relu(x) * 2, axis 1)
    {
        auto got = host_floats(ops::sum(ops::relu(ga) * 2.0f, {1}, false));
        for (size_t i = 0; i < 5; ++i)
            for (size_t k = 0; k < 6 * 9; ++k) {
                double t = 0;
                for (size_t j = 0; j < 7; ++j) t += 2.0 * std::max(0.0f, x[i * strides[0] + j * strides[1] + k]);
                EXPECT_NEAR(got[i * 54 + k], t, 1e-4);
            }
    }
    // softmax over an inner axis is one kernel where the data lie, also below an elementwise chain
    {
        ops::softmax(ga, 1).sync();
        ASSERT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
        EXPECT_EQ(graph::last_gpu_plan_kernels()[0], std::string("softmax_axis"));
        auto b16 = axtest::randn({4, 10, 64}, 4242).astype(DType::BFloat16);
        auto got = host_floats((ops::softmax(b16.gpu(), 1) * 2.0f).astype(DType::Float32));
        auto b32 = b16.astype(DType::Float32);
        for (size_t o = 0; o < 4; ++o)
            for (size_t i = 0; i < 64; ++i) {
                double m = -1e300, z = 0;
                for (size_t k = 0; k < 10; ++k) m = std::max(m, static_cast<double>(b32.typed_data<float>()[(o * 10 + k) * 64 + i]));
                for (size_t k = 0; k < 10; ++k) z += std::exp(b32.typed_data<float>()[(o * 10 + k) * 64 + i] - m);
                for (size_t k = 0; k < 10; ++k)
                    EXPECT_NEAR(got[(o * 10 + k) * 64 + i], 2.0 * std::exp(b32.typed_data<float>()[(o * 10 + k) * 64 + i] - m) / z, 2e-2);
            }
    }
    // layer norm and RMS norm over an inner axis (weights along that axis)
    {
        auto xn = axtest::randn({3, 12, 20}, 4343), w = axtest::randn({12}, 4344), bb = axtest::randn({12}, 4345);
        auto ln = host_floats(ops::layer_norm(xn.gpu(), w.gpu(), bb.gpu(), 1, 1e-5f)), rn = host_floats(ops::rms_norm(xn.gpu(), w.gpu(), 1, 1e-5f));
        const float *p = xn.typed_data<float>(), *pw = w.typed_data<float>(), *pb = bb.typed_data<float>();
        for (size_t o = 0; o < 3; ++o)
            for (size_t i = 0; i < 20; ++i) {
                double mean = 0, sq = 0;
                for (size_t k = 0; k < 12; ++k) mean += p[(o * 12 + k) * 20 + i];
                mean /= 12;
                double var = 0;
                for (size_t k = 0; k < 12; ++k) {
                    const double d = p[(o * 12 + k) * 20 + i] - mean;
                    var += d * d;
                    sq += static_cast<double>(p[(o * 12 + k) * 20 + i]) * p[(o * 12 + k) * 20 + i];
                }
                var /= 12;
                sq /= 12;
                for (size_t k = 0; k < 12; ++k) {
                    const double v = p[(o * 12 + k) * 20 + i];
                    EXPECT_NEAR(ln[(o * 12 + k) * 20 + i], (v - mean) / std::sqrt(var + 1e-5) * pw[k] + pb[k], 1e-4);
                    EXPECT_NEAR(rn[(o * 12 + k) * 20 + i], v / std::sqrt(sq + 1e-5) * pw[k], 1e-4);
                }
            }
    }
    // softmax and log-softmax over each axis
    for (int axis = 0; axis < 4; ++axis) {
        auto sm = host_floats(ops::softmax(ga, axis)), lsm = host_floats(ops::log_softmax(ga, axis - 4));
        ASSERT_EQ(sm.size(), a.size());
        const size_t len = sh[static_cast<size_t>(axis)], st = strides[axis];
        for (size_t flat = 0; flat < a.size(); ++flat) {
            if ((flat / st) % len != 0) continue; // first element of each line along the axis
            double m = -1e300, z = 0;
            for (size_t k = 0; k < len; ++k) m = std::max(m, static_cast<double>(x[flat + k * st]));
            for (size_t k = 0; k < len; ++k) z += std::exp(x[flat + k * st] - m);
            for (size_t k = 0; k < len; ++k) {
                EXPECT_NEAR(sm[flat + k * st], std::exp(x[flat + k * st] - m) / z, 1e-5);
                EXPECT_NEAR(lsm[flat + k * st], x[flat + k * st] - m - std::log(z), 1e-4);
            }
        }
    }
}

// ---------------------------------------------------------------- parity ops
GPU_TEST(CpuGpuParity, ElementwiseReductionsMatmul) { // tests/test_cpu_gpu_parity.cpp:12-492 (hot-path ops)
    auto a = axtest::randn({4, 5}, 41), b = axtest::randn({4, 5}, 42);
    auto ga = a.gpu(), gb = b.gpu();
    std::vector<float> want(20);
    auto check_bin = [&](int op, const Tensor &got) {
        axo_binary(op, AXO_F32, a.data(), b.data(), want.data(), 4, 5, AXO_BK_FULL);
        auto g = host_floats(got);
        for (size_t i = 0; i < 20; ++i) EXPECT_NEAR(g[i], want[i], 1e-5 + 1e-5 * std::fabs(want[i]));
    };
    check_bin(AXO_OP_ADD, ga + gb);
    check_bin(AXO_OP_SUB, ga - gb);
    check_bin(AXO_OP_MUL, ga * gb);
    check_bin(AXO_OP_DIV, ga / gb);
    check_bin(AXO_OP_MAX, ops::maximum(ga, gb));
    auto check_un = [&](int op, const Tensor &got, const Tensor &src) {
        axo_unary(op, AXO_F32, src.data(), want.data(), 20);
        auto g = host_floats(got);
        for (size_t i = 0; i < 20; ++i) EXPECT_NEAR(g[i], want[i], 1e-5 + 1e-5 * std::fabs(want[i]));
    };
    check_un(AXO_OP_EXP, ops::exp(ga), a);
    check_un(AXO_OP_TANH, ops::tanh(ga), a);
    check_un(AXO_OP_SIGMOID, ops::sigmoid(ga), a);
    check_un(AXO_OP_SILU, ops::silu(ga), a);
    check_un(AXO_OP_GELU, ops::gelu(ga), a);
    check_un(AXO_OP_NEG, ops::negate(ga), a);
    std::vector<float> rs(4);
    axo_reduce_last(AXO_RED_SUM, AXO_F32, a.data(), rs.data(), 4, 5);
    auto gs = host_floats(ga.sum(-1));
    auto gm = host_floats(ga.mean(-1, true));
    EXPECT_EQ(ga.mean(-1, true).shape(), Shape({4, 1}));
    for (size_t i = 0; i < 4; ++i) {
        EXPECT_NEAR(gs[i], rs[i], 1e-5);
        EXPECT_NEAR(gm[i], rs[i] / 5, 1e-5);
    }
    axo_reduce_last(AXO_RED_MAX, AXO_F32, a.data(), rs.data(), 4, 5);
    auto gx = host_floats(ga.max(-1));
    for (size_t i = 0; i < 4; ++i) EXPECT_NEAR(gx[i], rs[i], 0);
    // matmul against the oracle's sgemm
    auto m1 = axtest::randn({7, 12}, 43), m2 = axtest::randn({12, 9}, 44);
    std::vector<float> mm(63);
    axo_matmul(AXO_F32, m1.data(), m2.data(), mm.data(), 7, 9, 12, 0, 0);
    auto gmm = host_floats(ops::matmul(m1.gpu(), m2.gpu()));
    for (size_t i = 0; i < 63; ++i) EXPECT_NEAR(gmm[i], mm[i], 1e-4 + 1e-4 * std::fabs(mm[i]));
    auto gmt = host_floats(ops::matmul(m1.gpu(), m2.transpose({1, 0}).ascontiguousarray().gpu(), false, true));
    for (size_t i = 0; i < 63; ++i) EXPECT_NEAR(gmt[i], mm[i], 1e-4 + 1e-4 * std::fabs(mm[i]));
    EXPECT_EQ(ops::sum(axtest::randn({3, 4, 5}, 1).gpu(), {1}).shape(), Shape({3, 5})); // (ReductionsAndSoftmaxOverAnyAxis checks the values)
}

// Products whose reduction length leaves the operands' rows off their 16-byte alignment (K = 301 fp32, 203 bf16), in
// both storage orders of the right operand: the planner pads both operands with zero columns and stays on the
// matrix-core kernels.  Against the oracle's sgemm.
GPU_TEST(CpuGpuParity, LargeMatmulWithUnalignedReductionLength) {
    const size_t M = 200, N = 160, K = 301;
    auto a = axtest::randn({M, K}, 51), b = axtest::randn({K, N}, 52);
    std::vector<float> want(M * N);
    axo_matmul(AXO_F32, a.data(), b.data(), want.data(), M, N, K, 0, 0);
    auto nn = host_floats(ops::matmul(a.gpu(), b.gpu()));
    auto nt = host_floats(ops::matmul(a.gpu(), b.transpose({1, 0}).ascontiguousarray().gpu(), false, true));
    for (size_t i = 0; i < M * N; ++i) {
        EXPECT_NEAR(nn[i], want[i], 2e-4 + 1e-4 * std::fabs(want[i]));
        EXPECT_NEAR(nt[i], want[i], 2e-4 + 1e-4 * std::fabs(want[i]));
    }
    ASSERT_TRUE(!graph::last_gpu_plan_kernels().empty());
    EXPECT_EQ(graph::last_gpu_plan_kernels().back(), std::string("gemm"));
    // bf16, batched, K = 203
    auto ab = axtest::randn({3, 128, 203}, 53).astype(DType::BFloat16), bb = axtest::randn({3, 96, 203}, 54).astype(DType::BFloat16);
    auto got = ops::matmul(ab.gpu(), bb.gpu(), false, true);
    EXPECT_EQ(got.shape(), Shape({3, 128, 96}));
    auto gh = host_floats(got.astype(DType::Float32));
    auto af = ab.astype(DType::Float32), bf = bb.astype(DType::Float32);
    std::vector<float> w2(128 * 96);
    for (size_t i = 0; i < 3; ++i) {
        axo_matmul(AXO_F32, af.typed_data<float>() + i * 128 * 203, bf.typed_data<float>() + i * 96 * 203, w2.data(), 128, 96, 203, 0, 1);
        for (size_t j = 0; j < w2.size(); ++j) EXPECT_NEAR(gh[i * w2.size() + j], w2[j], 0.15 + 0.01 * std::fabs(w2[j]));
    }
}

// Batch dimensions that broadcast in part (tests/test_tensor_matmul.cpp: batched products follow numpy's rules)
GPU_TEST(CpuGpuParity, MatmulBroadcastsBatchDimensions) {
    auto a = axtest::randn({3, 1, 20, 12}, 61), b = axtest::randn({1, 4, 12, 9}, 62);
    auto got = ops::matmul(a.gpu(), b.gpu());
    EXPECT_EQ(got.shape(), Shape({3, 4, 20, 9}));
    auto g = host_floats(got);
    std::vector<float> want(20 * 9);
    for (size_t i = 0; i < 3; ++i)
        for (size_t j = 0; j < 4; ++j) {
            axo_matmul(AXO_F32, a.typed_data<float>() + i * 20 * 12, b.typed_data<float>() + j * 12 * 9, want.data(), 20, 9, 12, 0, 0);
            for (size_t e = 0; e < want.size(); ++e) EXPECT_NEAR(g[(i * 4 + j) * want.size() + e], want[e], 1e-4 + 1e-4 * std::fabs(want[e]));
        }
    // equal batch counts in different shapes: [2,3,...] x [3,...] -> [2,3,...]
    auto c = axtest::randn({2, 3, 8, 5}, 63), d = axtest::randn({3, 5, 7}, 64);
    auto got2 = ops::matmul(c.gpu(), d.gpu());
    EXPECT_EQ(got2.shape(), Shape({2, 3, 8, 7}));
    auto g2 = host_floats(got2);
    std::vector<float> w2(8 * 7);
    for (size_t i = 0; i < 2; ++i)
        for (size_t j = 0; j < 3; ++j) {
            axo_matmul(AXO_F32, c.typed_data<float>() + (i * 3 + j) * 40, d.typed_data<float>() + j * 35, w2.data(), 8, 7, 5, 0, 0);
            for (size_t e = 0; e < w2.size(); ++e) EXPECT_NEAR(g2[(i * 3 + j) * w2.size() + e], w2[e], 1e-4 + 1e-4 * std::fabs(w2[e]));
        }
}

// tests/test_cpu_gpu_parity.cpp:348-370 (argmax / argmin along axis 1 against the CPU scan) and the known answers of
// tests/test_tensor_argmax_argmin.cpp:4-112
GPU_TEST(CpuGpuParity, ArgmaxArgminParity) {
    auto a = axtest::randn({37, 501}, 71);
    std::vector<int64_t> want(37);
    for (bool want_min : {false, true}) {
        auto got = want_min ? ops::argmin(a.gpu(), 1, false) : ops::argmax(a.gpu(), 1, false);
        EXPECT_EQ(got.dtype(), DType::Int64);
        EXPECT_EQ(got.shape(), Shape({37}));
        axo_argreduce(want_min, AXO_F32, a.typed_data<float>(), want.data(), 37, 501, 1);
        auto host = got.cpu();
        for (size_t i = 0; i < 37; ++i) EXPECT_EQ(host.typed_data<int64_t>()[i], want[i]);
    }
    // along axis 0 of a lazy chain's result, keep_dims
    auto lazy = ops::relu(a.gpu()) * 2.0f;
    auto got0 = lazy.argmax(0, true);
    EXPECT_EQ(got0.shape(), Shape({1, 501}));
    std::vector<float> chain(37 * 501);
    for (size_t i = 0; i < chain.size(); ++i) chain[i] = std::max(a.typed_data<float>()[i], 0.0f) * 2.0f;
    std::vector<int64_t> want0(501);
    axo_argreduce(0, AXO_F32, chain.data(), want0.data(), 1, 37, 501);
    auto host0 = got0.cpu();
    for (size_t i = 0; i < 501; ++i) EXPECT_EQ(host0.typed_data<int64_t>()[i], want0[i]);
    // known answers
    const float v5[5] = {1.0f, 5.0f, 3.0f, 9.0f, 2.0f};
    auto r = ops::argmax(Tensor::from_data(v5, {5}).gpu());
    EXPECT_EQ(r.ndim(), 0u);
    EXPECT_EQ(r.item<int64_t>(), 3);
    const float m4[4] = {1.0f, 5.0f, 3.0f, 2.0f};
    auto m = Tensor::from_data(m4, {2, 2}).gpu();
    auto c0 = ops::argmin(m, 0).cpu();
    EXPECT_EQ(c0.typed_data<int64_t>()[0], 0);
    EXPECT_EQ(c0.typed_data<int64_t>()[1], 1);
    // a transposed (non-contiguous) view gives what its contiguous copy gives (:117-131)
    auto t3 = axtest::randn({3, 4, 5}, 72).gpu().transpose({0, 2, 1});
    auto x1 = ops::argmax(t3, -1).cpu(), x2 = ops::argmax(t3.ascontiguousarray(), -1).cpu();
    for (size_t i = 0; i < 15; ++i) EXPECT_EQ(x1.typed_data<int64_t>()[i], x2.typed_data<int64_t>()[i]);
    EXPECT_THROW(ops::argmax(m, 2), ShapeError);
}

// ----------------------------------------------------------------- attention
static std::tuple<Tensor, Tensor, Tensor> make_inputs(size_t B, size_t H, size_t Sq, size_t Skv, size_t D, DType dt = DType::Float32, uint64_t seed = 42) {
    return {axtest::randn({B, H, Sq, D}, seed, dt), axtest::randn({B, H, Skv, D}, seed + 1, dt), axtest::randn({B, H, Skv, D}, seed + 2, dt)};
}

GPU_TEST(FlashAttentionGPU, ShapeCasesFloat32MatchCpuPath) { // tests/test_flash_attention.cpp:76-213, 219-277, 334-355
    struct Case { size_t B, H, Sq, Skv, D; bool causal; float scale; };
    const Case cases[] = {{1, 2, 8, 8, 32, false, -1}, {1, 2, 16, 32, 32, false, -1}, {1, 2, 16, 16, 32, true, -1}, {1, 1, 37, 37, 32, false, -1},
                          {1, 2, 256, 256, 64, false, -1}, {1, 1, 16, 16, 128, false, -1}, {1, 2, 16, 16, 32, false, 0.5f}, {4, 8, 16, 16, 32, false, -1},
                          {1, 1, 1, 1, 32, false, -1}, {1, 2, 16, 16, 48, false, -1}, {2, 4, 32, 32, 64, false, 0.125f}};
    for (const Case &c : cases) {
        auto [q, k, v] = make_inputs(c.B, c.H, c.Sq, c.Skv, c.D);
        auto cpu_result = axtest::oracle_sdpa(q, k, v, Tensor(), c.scale, c.causal);
        auto gpu_result = ops::scaled_dot_product_attention(q.gpu(), k.gpu(), v.gpu(), Tensor(), c.scale, c.causal);
        EXPECT_EQ(gpu_result.shape(), q.shape());
        ASSERT_TENSORS_CLOSE(gpu_result.cpu(), cpu_result, 1e-4, 1e-4);
    }
}
GPU_TEST(FlashAttentionGPU, BoolMasks) { // tests/test_flash_attention.cpp (mask (i+j)%3==0), tests/test_nn_attention.cpp:131-165
    auto [q, k, v] = make_inputs(2, 2, 16, 16, 32);
    Tensor m2({16, 16}, DType::Bool), m4({2, 1, 16, 16}, DType::Bool);
    for (size_t i = 0; i < 16; ++i)
        for (size_t j = 0; j < 16; ++j) {
            m2.set_item<int>({i, j}, (i + j) % 3 == 0);
            m4.set_item<int>({0, 0, i, j}, (i + j) % 3 == 0);
            m4.set_item<int>({1, 0, i, j}, j > i + 2);
        }
    ASSERT_TENSORS_CLOSE(ops::scaled_dot_product_attention(q.gpu(), k.gpu(), v.gpu(), m2.gpu(), -1, false).cpu(), axtest::oracle_sdpa(q, k, v, m2, -1, false), 1e-4, 1e-4);
    ASSERT_TENSORS_CLOSE(ops::scaled_dot_product_attention(q.gpu(), k.gpu(), v.gpu(), m4, -1, false).cpu(), axtest::oracle_sdpa(q, k, v, m4, -1, false), 1e-4, 1e-4); // host mask is moved over
    EXPECT_THROW(ops::scaled_dot_product_attention(q.gpu(), k.gpu(), v.gpu(), Tensor::zeros({8, 8}, DType::Bool), -1, false), ShapeError);
}
GPU_TEST(FlashAttentionGPU, HalfTypesRunOnMfma) { // tests/test_flash_attention.cpp:233-249 (vs f32 computation of the same inputs)
    for (DType dt : {DType::Float16, DType::BFloat16})
        for (size_t D : {size_t(32), size_t(64), size_t(128)})
            for (bool causal : {false, true}) {
                auto [q, k, v] = make_inputs(1, 2, 200, 200, D, dt);
                auto ref = axtest::oracle_sdpa(q.astype(DType::Float32), k.astype(DType::Float32), v.astype(DType::Float32), Tensor(), -1, causal);
                auto got = ops::scaled_dot_product_attention(q.gpu(), k.gpu(), v.gpu(), Tensor(), -1, causal);
                EXPECT_EQ(got.dtype(), dt);
                EXPECT_EQ(std::string(ops::last_sdpa_kernel()).substr(0, 5), std::string("mfma_"));
                EXPECT_LE(max_abs_diff(got, ref), 2e-2);
            }
}
GPU_TEST(FlashAttentionGPU, OddHeadSizesArePaddedOntoTheMatrixCores) {
    // large enough problems with head sizes no kernel takes as they are (fp32 50 / 90, bf16 100, f16 20) are padded to the next of
    // 32 / 64 / 128 by the host layer; multiples of 4 (fp32) or 8 (16-bit) go to the kernels unpadded; the result is the same
    struct Case { DType dt; size_t B, H, Sq, Skv, D; bool causal; const char *kernel; double tol; };
    const Case cases[] = {{DType::Float32, 1, 4, 300, 300, 50, false, "mfma_f32_d64", 1e-4}, {DType::Float32, 2, 2, 256, 200, 90, true, "mfma_f32_d128", 1e-4},
                          {DType::Float32, 1, 4, 300, 300, 48, false, "mfma_f32_d48", 1e-4}, {DType::BFloat16, 1, 4, 300, 300, 100, false, "mfma_bf16_d128", 2e-2},
                          {DType::BFloat16, 1, 4, 300, 300, 80, true, "mfma_bf16_d80", 2e-2}, {DType::Float16, 2, 4, 400, 400, 20, false, "mfma_f16_d32", 2e-2}};
    for (const Case &c : cases) {
        auto [q, k, v] = make_inputs(c.B, c.H, c.Sq, c.Skv, c.D, c.dt);
        auto ref = axtest::oracle_sdpa(q.astype(DType::Float32), k.astype(DType::Float32), v.astype(DType::Float32), Tensor(), -1, c.causal);
        auto got = ops::scaled_dot_product_attention(q.gpu(), k.gpu(), v.gpu(), Tensor(), -1, c.causal);
        EXPECT_EQ(got.shape(), q.shape());
        EXPECT_EQ(got.dtype(), c.dt);
        EXPECT_EQ(std::string(ops::last_sdpa_kernel()), std::string(c.kernel));
        EXPECT_LE(max_abs_diff(got, ref), c.tol);
    }
    // a small one stays on the kernel for arbitrary head sizes
    auto [q, k, v] = make_inputs(1, 2, 16, 16, 50);
    ops::scaled_dot_product_attention(q.gpu(), k.gpu(), v.gpu(), Tensor(), -1, false).sync();
    EXPECT_EQ(std::string(ops::last_sdpa_kernel()), std::string("generic"));
}
GPU_TEST(FlashAttentionGPU, Config1Float32) { // BASELINE configs[0]: B1 H8 S512 D64, no mask, scale 0.125
    auto [q, k, v] = make_inputs(1, 8, 512, 512, 64);
    auto got = ops::scaled_dot_product_attention(q.gpu(), k.gpu(), v.gpu(), Tensor(), 0.125f, false);
    ASSERT_TENSORS_CLOSE(got.cpu(), axtest::oracle_sdpa(q, k, v, Tensor(), 0.125f, false), 1e-4, 1e-4);
}

GPU_TEST(FlashAttentionGPU, ShapesNoKernelTakesAreComposedFromMatmulMaskAndSoftmax) { // flash_attention_dispatch.mm:125-162
    // head sizes above 256: plain, causal (query and key counts differ), and with a Bool mask shared by all heads
    auto [q, k, v] = make_inputs(1, 2, 40, 56, 320);
    for (bool causal : {false, true}) {
        auto got = ops::scaled_dot_product_attention(q.gpu(), k.gpu(), v.gpu(), Tensor(), -1, causal);
        EXPECT_EQ(std::string(ops::last_sdpa_kernel()), std::string("decomposed"));
        EXPECT_EQ(got.shape(), q.shape());
        ASSERT_TENSORS_CLOSE(got.cpu(), axtest::oracle_sdpa(q, k, v, Tensor(), -1, causal), 1e-4, 1e-4);
    }
    Tensor m2({40, 56}, DType::Bool);
    for (size_t i = 0; i < 40; ++i)
        for (size_t j = 0; j < 56; ++j) m2.set_item<int>({i, j}, (i + j) % 3 == 0);
    ASSERT_TENSORS_CLOSE(ops::scaled_dot_product_attention(q.gpu(), k.gpu(), v.gpu(), m2.gpu(), 0.05f, false).cpu(), axtest::oracle_sdpa(q, k, v, m2, 0.05f, false), 1e-4, 1e-4);
    EXPECT_EQ(std::string(ops::last_sdpa_kernel()), std::string("decomposed"));
    // bf16 at head size 512
    {
        auto [qh, kh, vh] = make_inputs(2, 3, 33, 33, 512, DType::BFloat16);
        auto ref = axtest::oracle_sdpa(qh.astype(DType::Float32), kh.astype(DType::Float32), vh.astype(DType::Float32), Tensor(), -1, true);
        auto got = ops::scaled_dot_product_attention(qh.gpu(), kh.gpu(), vh.gpu(), Tensor(), -1, true);
        EXPECT_EQ(std::string(ops::last_sdpa_kernel()), std::string("decomposed"));
        EXPECT_EQ(got.dtype(), DType::BFloat16);
        EXPECT_LE(max_abs_diff(got, ref), 3e-2); // the scores and the weights each pass through bf16 on the composed path
    }
    // fp32 head sizes 192 and 256 (only the FMA kernel takes them): composed once the problem is large enough to notice,
    // causal and not; 16-bit: 256 has a matrix-core kernel and 192 is padded onto it; a small fp32 problem of the same
    // head size stays on the FMA kernel
    for (size_t D : {192, 256}) {
        auto [qw, kw, vw] = make_inputs(1, 2, 256, 320, D);
        for (bool causal : {false, true}) {
            auto got = ops::scaled_dot_product_attention(qw.gpu(), kw.gpu(), vw.gpu(), Tensor(), -1, causal);
            EXPECT_EQ(std::string(ops::last_sdpa_kernel()), std::string("decomposed"));
            ASSERT_TENSORS_CLOSE(got.cpu(), axtest::oracle_sdpa(qw, kw, vw, Tensor(), -1, causal), 2e-4, 2e-4);
        }
        auto qb = qw.astype(DType::BFloat16), kb = kw.astype(DType::BFloat16), vb = vw.astype(DType::BFloat16);
        auto ref = axtest::oracle_sdpa(qb.astype(DType::Float32), kb.astype(DType::Float32), vb.astype(DType::Float32), Tensor(), -1, false);
        auto got = ops::scaled_dot_product_attention(qb.gpu(), kb.gpu(), vb.gpu(), Tensor(), -1, false);
        EXPECT_EQ(std::string(ops::last_sdpa_kernel()), std::string(D == 192 ? "mfma_bf16_d192" : "mfma_bf16_d256"));
        EXPECT_EQ(got.shape(), qb.shape());
        EXPECT_LE(max_abs_diff(got, ref), 2e-2);
        auto [q1, k1, v1] = make_inputs(1, 1, 8, 8, D);
        ops::scaled_dot_product_attention(q1.gpu(), k1.gpu(), v1.gpu(), Tensor(), -1, false).cpu();
        EXPECT_EQ(std::string(ops::last_sdpa_kernel()), std::string("generic"));
    }
    // 65 536 (batch, head) slices of a head size that only the FMA kernel takes
    {
        auto [qs, ks, vs] = make_inputs(256, 256, 4, 4, 6);
        auto got = ops::scaled_dot_product_attention(qs.gpu(), ks.gpu(), vs.gpu(), Tensor(), -1, false);
        EXPECT_EQ(std::string(ops::last_sdpa_kernel()), std::string("decomposed"));
        ASSERT_TENSORS_CLOSE(got.cpu(), axtest::oracle_sdpa(qs, ks, vs, Tensor(), -1, false), 1e-4, 1e-4);
    }
}

// ------------------------------------------------------------------------ nn
GPU_TEST(NNLayers, LinearKnownAnswers) { // tests/test_nn_layers.cpp:12-73
    nn::Linear lin;
    lin.load_state_dict({{"weight", Tensor::ones({2, 3})}, {"bias", Tensor::zeros({2})}});
    lin.to(Device::GPU);
    auto y = lin.forward(Tensor::ones({1, 3}, DType::Float32, Device::GPU)).cpu();
    EXPECT_EQ(y.shape(), Shape({1, 2}));
    EXPECT_NEAR(y.item<float>({0, 0}), 3.0f, 1e-5);
    lin.load_state_dict({{"weight", Tensor::ones({2, 3}, DType::Float32, Device::GPU)}, {"bias", Tensor::ones({2}, DType::Float32, Device::GPU)}});
    EXPECT_NEAR(lin.forward(Tensor::ones({1, 3}, DType::Float32, Device::GPU)).cpu().item<float>({0, 1}), 4.0f, 1e-5);
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u); // bias rides in the GEMM epilogue
    nn::Linear nob(false);
    nob.load_state_dict({{"weight", Tensor::ones({4, 2}, DType::Float32, Device::GPU)}});
    auto yb = nob.forward(Tensor::ones({5, 3, 2}, DType::Float32, Device::GPU)).cpu(); // batched input
    EXPECT_EQ(yb.shape(), Shape({5, 3, 4}));
    EXPECT_NEAR(yb.item<float>({4, 2, 3}), 2.0f, 1e-5);
}
GPU_TEST(NNLayers, NormModules) { // tests/test_nn_layers.cpp:191-207
    nn::RMSNorm rms;
    rms.load_state_dict({{"weight", Tensor::ones({4})}});
    rms.to(Device::GPU);
    float v[4] = {1, 2, 3, 4};
    auto y = rms.forward(Tensor::from_data(v, {1, 4}, Device::GPU)).cpu();
    EXPECT_NEAR(y.item<float>({0, 0}), 1.0f / std::sqrt(7.5f), 1e-4);
    nn::LayerNorm ln;
    ln.load_state_dict({{"weight", Tensor::ones({4})}, {"bias", Tensor::zeros({4})}});
    ln.to(Device::GPU).to(DType::Float32);
    auto z = host_floats(ln.forward(Tensor::from_data(v, {1, 4}, Device::GPU)));
    EXPECT_NEAR(z[0] + z[1] + z[2] + z[3], 0.0, 1e-5);
    EXPECT_NEAR(z[3], 1.5 / std::sqrt(1.25 + 1e-5), 1e-4);
}
GPU_TEST(FlashAttentionMHA, UniformInputIdentityProjections) { // tests/test_flash_attention.cpp:283-328, test_nn_attention.cpp:68-92
    nn::MultiHeadAttention mha(1);
    const size_t d = 2;
    std::map<std::string, Tensor> state;
    for (const char *p : {"q_proj", "k_proj", "v_proj", "out_proj"}) {
        state[std::string(p) + ".weight"] = Tensor::eye(d);
        state[std::string(p) + ".bias"] = Tensor::zeros({d});
    }
    mha.load_state_dict(state);
    mha.to(Device::GPU);
    auto input = Tensor::ones({1, 3, 2}, DType::Float32, Device::GPU);
    auto out = mha.forward(input, input, input).cpu();
    EXPECT_EQ(out.shape(), Shape({1, 3, 2}));
    for (size_t i = 0; i < 3; ++i)
        for (size_t j = 0; j < 2; ++j) EXPECT_NEAR(out.item<float>({0, i, j}), 1.0f, 1e-5);
    auto causal = mha.forward(input, input, input, Tensor(), true).cpu();
    EXPECT_NEAR(causal.item<float>({0, 2, 1}), 1.0f, 1e-5);
}

// BASELINE configs[4]: Whisper-style encoder self-attention block, at S=150 compared in full and at the full
// S=1500 on 48 sequence positions from the start, the middle and the end
static Tensor whisper_block(const Tensor &x, nn::MultiHeadAttention &mha, nn::LayerNorm &ln) { return ln.forward(x + mha.forward(x, x, x)); }

static void whisper_case(size_t S, bool /*compare*/) {
    const size_t Dm = 1280, H = 20, Dh = 64;
    const DType dt = DType::BFloat16;
    auto x = axtest::randn({1, S, Dm}, 51, dt);
    std::map<std::string, Tensor> w;
    uint64_t seed = 60;
    for (const char *p : {"q_proj", "k_proj", "v_proj", "out_proj"}) {
        w[std::string(p) + ".weight"] = axtest::randn({Dm, Dm}, seed++, dt, 0.02f);
        w[std::string(p) + ".bias"] = Tensor::zeros({Dm}, dt);
    }
    nn::MultiHeadAttention mha(static_cast<int>(H));
    mha.load_state_dict(w);
    mha.to(Device::GPU);
    nn::LayerNorm ln;
    ln.load_state_dict({{"weight", Tensor::ones({Dm}, dt)}, {"bias", Tensor::zeros({Dm}, dt)}});
    ln.to(Device::GPU);
    auto y = whisper_block(x.gpu(), mha, ln);
    EXPECT_EQ(y.dtype(), dt);
    EXPECT_EQ(y.shape(), Shape({1, S, Dm}));
    auto got = host_floats(y);
    EXPECT_EQ(std::string(ops::last_sdpa_kernel()), std::string("mfma_bf16_d64"));
    // layer-norm output: every row has mean ~ 0 and variance ~ 1
    for (size_t r : {size_t(0), S / 2, S - 1}) {
        double m = 0, q = 0;
        for (size_t j = 0; j < Dm; ++j) m += got[r * Dm + j];
        m /= Dm;
        for (size_t j = 0; j < Dm; ++j) q += (got[r * Dm + j] - m) * (got[r * Dm + j] - m);
        EXPECT_NEAR(m, 0.0, 2e-2);
        EXPECT_NEAR(q / Dm, 1.0, 5e-2);
    }
    // fp32 evaluation of the same bf16 inputs with the oracle's pieces, on a subset of the sequence positions: the
    // projections and the norm are row-wise, and a query row's attention needs every key and value but no other query
    std::vector<size_t> rows;
    if (S <= 256) {
        for (size_t r = 0; r < S; ++r) rows.push_back(r);
    } else {
        for (size_t r = 0; r < 16; ++r) rows.push_back(r);
        for (size_t r = S / 2 - 8; r < S / 2 + 8; ++r) rows.push_back(r);
        for (size_t r = S - 16; r < S; ++r) rows.push_back(r);
    }
    const size_t Q = rows.size();
    auto xf = x.astype(DType::Float32);
    Tensor x2 = xf.reshape({S, Dm});
    Tensor xq({Q, Dm}, DType::Float32);
    for (size_t i = 0; i < Q; ++i) std::memcpy(xq.typed_data<float>() + i * Dm, x2.typed_data<float>() + rows[i] * Dm, Dm * sizeof(float));
    auto proj = [&](const Tensor &in, size_t n, const char *name) {
        Tensor wf = w[std::string(name) + ".weight"].astype(DType::Float32), out({n, Dm}, DType::Float32);
        axo_matmul(AXO_F32, in.data(), wf.data(), out.data(), n, Dm, Dm, 0, 1);
        return out;
    };
    auto split = [&](const Tensor &t, size_t n) { return t.reshape({1, n, H, Dh}).transpose({0, 2, 1, 3}).ascontiguousarray(); };
    auto att = axtest::oracle_sdpa(split(proj(xq, Q, "q_proj"), Q), split(proj(x2, S, "k_proj"), S), split(proj(x2, S, "v_proj"), S), Tensor(), -1, false);
    Tensor merged = att.transpose({0, 2, 1, 3}).ascontiguousarray().reshape({Q, Dm});
    Tensor o = proj(merged, Q, "out_proj");
    std::vector<float> res(Q * Dm), want(Q * Dm);
    for (size_t i = 0; i < Q * Dm; ++i) res[i] = o.typed_data<float>()[i] + xq.typed_data<float>()[i];
    axo_layer_norm(AXO_F32, res.data(), nullptr, nullptr, want.data(), Q, Dm, 1e-5f);
    // The bar: 2e-2 absolute plus half a bf16 ulp of the expected value.  The block rounds to bf16 six times (q, k, v,
    // attention output, residual sum, norm output) where the fp32 evaluation rounds never; the last rounding alone
    // is up to 2^-8 |y|, i.e. 1.6e-2 at |y| = 4, so a flat 2e-2 cannot hold for the largest outputs of any bf16 pipeline.
    double worst = 0, worst_excess = 0;
    size_t beyond = 0;
    for (size_t i = 0; i < Q; ++i)
        for (size_t j = 0; j < Dm; ++j) {
            const double g0 = got[rows[i] * Dm + j], w0 = want[i * Dm + j], d = std::fabs(g0 - w0);
            worst = std::max(worst, d);
            worst_excess = std::max(worst_excess, d - (2e-2 + std::fabs(w0) * 0.00390625));
            beyond += d > 2e-2;
        }
    std::printf("    S=%zu: %zu rows compared, max |err| %.4f, %zu of %zu beyond 2e-2\n", S, Q, worst, beyond, Q * Dm);
    EXPECT_LE(worst_excess, 0.0);
    EXPECT_LE(double(beyond) / (Q * Dm), 0.002);
}
GPU_TEST(WhisperBlock, ReducedSequenceMatchesFp32Reference) { whisper_case(150, true); }
GPU_TEST(WhisperBlock, FullSizeMatchesFp32ReferenceOnSampledRows) { whisper_case(1500, true); }

// ---------------------------------------------------------------------------
// A whole pre-norm transformer encoder layer as in the reference's examples/whisper_poc.cpp:57-86
// (the module is written the way that file writes it), bf16 on the GPU against an fp32
// evaluation of the same bf16 parameters built from the oracle's pieces.
namespace {
struct WhisperEncoderLayer : nn::Module {
    nn::MultiHeadAttention self_attn_;
    nn::LayerNorm self_attn_layer_norm_;
    nn::Linear fc1_{true};
    nn::Linear fc2_{true};
    nn::LayerNorm final_layer_norm_;

    explicit WhisperEncoderLayer(int num_heads) : self_attn_(num_heads) {
        register_module("self_attn", self_attn_);
        register_module("self_attn_layer_norm", self_attn_layer_norm_);
        register_module("fc1", fc1_);
        register_module("fc2", fc2_);
        register_module("final_layer_norm", final_layer_norm_);
    }
    Tensor forward(const Tensor &x) const override {
        auto residual = x;
        auto h = self_attn_layer_norm_(x);
        h = self_attn_.forward(h, h, h);
        h = ops::add(residual, h);
        residual = h;
        h = final_layer_norm_(h);
        h = fc1_(h).gelu();
        h = fc2_(h);
        return ops::add(residual, h);
    }
};

// fp32 helpers over the oracle
Tensor ref_linear(const Tensor &x2d, const Tensor &w, const Tensor &b) { // x [S, in] f32, w [out, in], b [out]
    const size_t S = x2d.shape()[0], in = x2d.shape()[1], out = w.shape()[0];
    Tensor wf = w.astype(DType::Float32), bf = b.astype(DType::Float32), y({S, out}, DType::Float32);
    axo_matmul(AXO_F32, x2d.data(), wf.data(), y.data(), S, out, in, 0, 1);
    for (size_t i = 0; i < S; ++i)
        for (size_t j = 0; j < out; ++j) y.typed_data<float>()[i * out + j] += bf.typed_data<float>()[j];
    return y;
}
Tensor ref_layer_norm(const Tensor &x2d, const Tensor &w, const Tensor &b) {
    Tensor wf = w.astype(DType::Float32), bf = b.astype(DType::Float32), y(x2d.shape(), DType::Float32);
    axo_layer_norm(AXO_F32, x2d.data(), wf.data(), bf.data(), y.typed_data<float>(), x2d.shape()[0], x2d.shape()[1], 1e-5f);
    return y;
}
} // namespace

GPU_TEST(WhisperEncoderLayer, MatchesFp32ReferenceAndStaysFused) {
    const size_t S = 96, Dm = 1280, H = 20, Dh = 64, F = 5120;
    const DType dt = DType::BFloat16;
    std::map<std::string, Tensor> w;
    uint64_t seed = 100;
    auto mat = [&](size_t o, size_t i) { return axtest::randn({o, i}, seed++, dt, 0.02f); };
    auto vec = [&](size_t n, float lo, float hi) { return axtest::uniform({n}, seed++, lo, hi, dt); };
    for (const char *p : {"q_proj", "k_proj", "v_proj", "out_proj"}) {
        w[std::string("self_attn.") + p + ".weight"] = mat(Dm, Dm);
        w[std::string("self_attn.") + p + ".bias"] = vec(Dm, -0.05f, 0.05f);
    }
    w["self_attn_layer_norm.weight"] = vec(Dm, 0.8f, 1.2f);
    w["self_attn_layer_norm.bias"] = vec(Dm, -0.1f, 0.1f);
    w["final_layer_norm.weight"] = vec(Dm, 0.8f, 1.2f);
    w["final_layer_norm.bias"] = vec(Dm, -0.1f, 0.1f);
    w["fc1.weight"] = mat(F, Dm);
    w["fc1.bias"] = vec(F, -0.05f, 0.05f);
    w["fc2.weight"] = mat(Dm, F);
    w["fc2.bias"] = vec(Dm, -0.05f, 0.05f);
    WhisperEncoderLayer layer(static_cast<int>(H));
    layer.load_state_dict(w);
    layer.to(Device::GPU);
    EXPECT_EQ(layer.named_parameters().size(), 16u);

    auto x = axtest::randn({1, S, Dm}, 99, dt);
    auto y = layer.forward(x.gpu());
    EXPECT_EQ(y.dtype(), dt);
    auto got = host_floats(y);
    // the tail of the layer is one graph of four launches: out_proj+bias+residual (GEMM; its result is
    // shared by the norm and the last residual), LN, fc1+bias+gelu (GEMM), fc2+bias+residual (GEMM)
    const auto &ks = graph::last_gpu_plan_kernels();
    {
        std::string all;
        for (const auto &k : ks) all += " " + k;
        std::printf("    kernels of the last materialisation:%s\n", all.c_str());
    }
    ASSERT_EQ(ks.size(), 4u);
    EXPECT_EQ(ks[0], std::string("gemm"));
    EXPECT_EQ(ks[1].substr(0, 21), std::string("rows_static_layernorm"));
    EXPECT_EQ(ks[2], std::string("gemm"));
    EXPECT_EQ(ks[3], std::string("gemm"));

    // fp32 reference
    Tensor x2 = x.astype(DType::Float32).reshape({S, Dm});
    Tensor h = ref_layer_norm(x2, w["self_attn_layer_norm.weight"], w["self_attn_layer_norm.bias"]);
    auto split = [&](const Tensor &t) { return t.reshape({1, S, H, Dh}).transpose({0, 2, 1, 3}).ascontiguousarray(); };
    auto proj = [&](const Tensor &in, const char *n) { return ref_linear(in, w[std::string("self_attn.") + n + ".weight"], w[std::string("self_attn.") + n + ".bias"]); };
    Tensor att = axtest::oracle_sdpa(split(proj(h, "q_proj")), split(proj(h, "k_proj")), split(proj(h, "v_proj")), Tensor(), -1, false);
    Tensor merged = att.transpose({0, 2, 1, 3}).ascontiguousarray().reshape({S, Dm});
    Tensor o = proj(merged, "out_proj");
    Tensor r1({S, Dm}, DType::Float32);
    for (size_t i = 0; i < S * Dm; ++i) r1.typed_data<float>()[i] = x2.typed_data<float>()[i] + o.typed_data<float>()[i];
    Tensor h2 = ref_layer_norm(r1, w["final_layer_norm.weight"], w["final_layer_norm.bias"]);
    Tensor f1 = ref_linear(h2, w["fc1.weight"], w["fc1.bias"]);
    Tensor g1(f1.shape(), DType::Float32);
    axo_unary(AXO_OP_GELU, AXO_F32, f1.data(), g1.data(), f1.size());
    Tensor f2 = ref_linear(g1, w["fc2.weight"], w["fc2.bias"]);
    double worst = 0;
    size_t beyond = 0;
    for (size_t i = 0; i < S * Dm; ++i) {
        const double want = double(r1.typed_data<float>()[i]) + f2.typed_data<float>()[i];
        const double d = std::fabs(got[i] - want);
        worst = std::max(worst, d);
        beyond += d > 2e-2;
    }
    std::printf("    encoder layer: max |err| %.4f, %.3f %% of outputs beyond 2e-2\n", worst, 100.0 * beyond / (S * Dm));
    EXPECT_LE(worst, 8e-2);                         // several bf16 roundings of values up to |4|
    EXPECT_LE(double(beyond) / (S * Dm), 0.03);
}

// ---------------------------------------------------------------------------
// The remaining backend hooks: per-op registry, gpu_* free functions, CPU-planned fused steps
GPU_TEST(BackendHooks, OperationRegistryServesGpuOps) {
    using ops::OpType;
    ops::OperationRegistry::initialize_builtin_operations(); // tests/axiom_test_utils.hpp:17-22
    EXPECT_TRUE(ops::OperationRegistry::is_operation_available(OpType::Add, Device::GPU));
    EXPECT_TRUE(ops::OperationRegistry::get_operation(OpType::Add, Device::CPU) == nullptr); // no CPU backend in this library
    EXPECT_TRUE(ops::OperationRegistry::get_operation(OpType::Conv2D, Device::GPU) == nullptr);
    auto a = axtest::randn({4, 5}, 201), b = axtest::randn({5}, 202);
    const auto *add = ops::OperationRegistry::get_operation(OpType::Add, Device::GPU);
    ASSERT_TRUE(add != nullptr);
    EXPECT_EQ(add->name(), std::string("hip::add"));
    EXPECT_TRUE(add->supports_binary(a, b));
    EXPECT_FALSE(add->supports_binary(a, axtest::randn({4}, 1)));
    auto r = add->execute_binary(a.gpu(), b.gpu());
    EXPECT_FALSE(r.is_lazy() && !r.lazy_node()->is_materialized_); // registry ops run at once
    EXPECT_NEAR(r.cpu().item<float>({2, 3}), a.item<float>({2, 3}) + b.item<float>({3}), 0);
    auto sm = ops::OperationRegistry::get_operation(OpType::Softmax, Device::GPU)->execute_reduction(a.gpu(), {-1}, false).cpu();
    double s = 0;
    for (size_t j = 0; j < 5; ++j) s += sm.item<float>({1, j});
    EXPECT_NEAR(s, 1.0, 1e-5);
    auto mm = ops::OperationRegistry::get_operation(OpType::MatMul, Device::GPU)->execute_matmul(a.gpu(), a.gpu(), false, true).cpu();
    EXPECT_EQ(mm.shape(), Shape({4, 4}));
    EXPECT_THROW(add->execute_unary(a.gpu()).cpu(), AxiomError);
    auto devs = ops::OperationRegistry::available_devices_for_operation(OpType::ReLU);
    ASSERT_EQ(devs.size(), 1u);
    EXPECT_TRUE(devs[0] == Device::GPU);
}

GPU_TEST(BackendHooks, GpuFreeFunctions) {
    using namespace backends::hip;
    EXPECT_TRUE(is_hip_available());
    float v[4] = {1, 2, 3, 4};
    auto x = Tensor::from_data(v, {1, 4}, Device::GPU);
    auto r = gpu_rms_norm(x, Tensor::ones({4}, DType::Float32, Device::GPU), -1, 1e-5f);
    EXPECT_FALSE(r.is_lazy() && !r.lazy_node()->is_materialized_);
    EXPECT_NEAR(r.cpu().item<float>({0, 0}), 1.0f / std::sqrt(7.5f), 1e-4);
    auto ln = gpu_layer_norm(x, Tensor(), Tensor(), -1, 1e-5f).cpu();
    EXPECT_NEAR(ln.item<float>({0, 0}) + ln.item<float>({0, 3}), 0.0, 1e-5);
    EXPECT_NEAR(gpu_fill_constant({3, 3}, DType::BFloat16, 1.5).cpu().item<float>({2, 2}), 1.5f, 0);
    auto t = axtest::randn({6, 7}, 203).gpu().transpose({1, 0});
    auto c = gpu_make_contiguous(t);
    EXPECT_TRUE(c.is_contiguous());
    EXPECT_TRUE(c.cpu().allclose(t.cpu().ascontiguousarray(), 0, 0));
    auto y = gpu_linear(Tensor::ones({2, 3}, DType::Float32, Device::GPU), Tensor::ones({4, 3}, DType::Float32, Device::GPU), Tensor::ones({4}, DType::Float32, Device::GPU), true);
    EXPECT_NEAR(y.cpu().item<float>({1, 2}), 4.0f, 1e-5);
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
    auto [q, k, vv] = make_inputs(1, 2, 8, 8, 32);
    ASSERT_TENSORS_CLOSE(gpu_scaled_dot_product_attention(q.gpu(), k.gpu(), vv.gpu(), Tensor(), -1, true).cpu(), axtest::oracle_sdpa(q, k, vv, Tensor(), -1, true), 1e-4, 1e-4);
}

GPU_TEST(BackendHooks, CpuPlannedFusedSteps) { // include/axiom/graph/gpu_fusion.hpp:14-22
    using ops::OpType;
    // buffers: slot 0 = a, slot 1 = b, slot 2 = c (host-resident: moved over), slot 3 = output
    auto a = axtest::randn({8, 16}, 211), b = axtest::randn({8, 16}, 212), c = axtest::randn({16}, 213);
    std::vector<Tensor> buffers = {a.gpu(), b.gpu(), c, Tensor()};
    graph::FusedGenericStep step;
    step.output_slot = 3;
    step.output_shape = {8, 16};
    step.output_dtype = DType::Float32;
    step.device = Device::GPU;
    step.op_chain = {OpType::Multiply, OpType::Add, OpType::ReLU}; // relu(a * b + c)
    step.input_slot_indices = {{0, 1}, {-1, 2}, {-1}};
    ASSERT_TRUE(graph::execute_gpu_fused_chain(step, step.op_chain, buffers));
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u); // the whole step is one launch
    auto got = buffers[3].cpu();
    for (size_t i = 0; i < 8; ++i)
        for (size_t j = 0; j < 16; ++j)
            EXPECT_NEAR(got.item<float>({i, j}), std::max(a.item<float>({i, j}) * b.item<float>({i, j}) + c.item<float>({j}), 0.0f), 1e-6);
    // an op without a GPU kernel: the hook declines, the caller falls back
    graph::FusedGenericStep bad = step;
    bad.op_chain = {OpType::Multiply, OpType::Atan2};
    bad.input_slot_indices = {{0, 1}, {-1, 2}};
    EXPECT_FALSE(graph::execute_gpu_fused_chain(bad, bad.op_chain, buffers));
    // chain + full reduction: sum(a + b) (tests/test_fusion_extended.cpp:346-352)
    graph::FusedReductionStep red;
    red.output_slot = 3;
    red.output_shape = {1};
    red.output_dtype = DType::Float32;
    red.reduction_op = OpType::Sum;
    red.params = graph::ReductionParams{{}, false};
    red.op_chain = {OpType::Add};
    red.input_slot_indices = {{0, 1}};
    ASSERT_TRUE(graph::execute_gpu_fused_reduction(red, buffers));
    double want = 0;
    for (size_t i = 0; i < 8; ++i)
        for (size_t j = 0; j < 16; ++j) want += double(a.item<float>({i, j})) + b.item<float>({i, j});
    EXPECT_NEAR(buffers[3].cpu().item<float>(), want, 1e-3);
}

// ------------------------------------------------- remaining lazy node kinds
// Known answers of the reference's tests/test_conv1d.cpp, test_embedding.cpp,
// test_nn_ergonomics.cpp:41-90 (glu), test_shape_ops_extended.cpp:42-77 (pad) and
// test_tensor_where.cpp:212-218 (masked_fill), plus float64 loops on random inputs.
static Tensor gpu_f32(std::initializer_list<float> v, const Shape &shape) {
    std::vector<float> d(v);
    return Tensor::from_data(d.data(), shape, Device::GPU);
}

GPU_TEST(LazyNodes, Conv1dKnownAnswers) {
    auto x5 = gpu_f32({1, 2, 3, 4, 5}, {1, 1, 5});
    auto w3 = gpu_f32({1, 1, 1}, {1, 1, 3});
    auto r = ops::conv1d(x5, w3); // :3-16
    EXPECT_TRUE(r.shape() == Shape({1, 1, 3}));
    auto h = host_floats(r);
    EXPECT_NEAR(h[0], 6.0f, 0); EXPECT_NEAR(h[1], 9.0f, 0); EXPECT_NEAR(h[2], 12.0f, 0);
    h = host_floats(ops::conv1d(x5, w3, Tensor(), 1, 1)); // :18-33, pad 1
    ASSERT_EQ(h.size(), 5u);
    const float want_pad[5] = {3, 6, 9, 12, 9};
    for (int i = 0; i < 5; ++i) EXPECT_NEAR(h[i], want_pad[i], 0);
    r = ops::conv1d(gpu_f32({1, 2, 3, 4, 5, 6}, {1, 1, 6}), w3, Tensor(), 2); // :35-46, stride 2
    EXPECT_TRUE(r.shape() == Shape({1, 1, 2}));
    h = host_floats(r);
    EXPECT_NEAR(h[0], 6.0f, 0); EXPECT_NEAR(h[1], 12.0f, 0);
    r = ops::conv1d(x5, w3, Tensor(), 1, 0, 2); // :48-61, dilation 2
    EXPECT_TRUE(r.shape() == Shape({1, 1, 1}));
    EXPECT_NEAR(r.item<float>(), 9.0f, 0);
    EXPECT_NEAR(ops::conv1d(gpu_f32({1, 2, 3}, {1, 1, 3}), w3, gpu_f32({10}, {1})).item<float>(), 16.0f, 0); // :63-75, bias
    r = ops::conv1d(gpu_f32({1, 2, 3, 4, 5, 6, 7, 8}, {1, 2, 4}), gpu_f32({1, 0, 0, 1, 1, 0, 0, 1, 1, 1, 1, 1}, {3, 2, 2})); // :77-90
    EXPECT_TRUE(r.shape() == Shape({1, 3, 3}));
    h = host_floats(r); // out[co][l] = sum_ci,k w[co][ci][k] x[ci][l+k]
    const float want_mc[9] = {7, 9, 11, 7, 9, 11, 14, 18, 22};
    for (int i = 0; i < 9; ++i) EXPECT_NEAR(h[i], want_mc[i], 0);
    r = ops::conv1d(gpu_f32({1, 2, 3, 4, 5}, {1, 5}), w3); // :92-102, unbatched
    EXPECT_TRUE(r.shape() == Shape({1, 3}));
    EXPECT_NEAR(host_floats(r)[0], 6.0f, 0);
    EXPECT_THROW(ops::conv1d(x5, w3, Tensor(), 1, 0, 1, 2), ShapeError);                 // 1 channel cannot be cut into 2 groups
    EXPECT_THROW(ops::conv1d(x5, gpu_f32({1, 1, 1, 1, 1, 1}, {1, 2, 3})), ShapeError); // channel mismatch
}

static void conv1d_case(DType dt, size_t N, size_t Cin, size_t L, size_t Cout, size_t K, int stride, int padding, int dilation, bool gelu, double tol) {
    auto x = axtest::randn({N, Cin, L}, 70, dt), w = axtest::randn({Cout, Cin, K}, 71, dt, 0.2f), b = axtest::randn({Cout}, 72, dt, 0.5f);
    Tensor y = ops::conv1d(x.gpu(), w.gpu(), b.gpu(), stride, padding, dilation);
    if (gelu) y = y.gelu();
    const size_t Lout = (L + 2 * padding - dilation * (K - 1) - 1) / stride + 1;
    ASSERT_TRUE(y.shape() == Shape({N, Cout, Lout}));
    auto got = host_floats(y);
    if (gelu) { // pad (if any), window gather, one GEMM carrying bias and GELU: no separate elementwise pass, no transposing copy
        const auto &k = graph::last_gpu_plan_kernels();
        EXPECT_EQ(k.size(), padding > 0 ? 3u : 2u);
        EXPECT_EQ(k.back(), std::string("gemm"));
    }
    auto xf = host_floats(x), wf = host_floats(w), bf = host_floats(b);
    double worst = 0;
    for (size_t n = 0; n < N; ++n)
        for (size_t co = 0; co < Cout; ++co)
            for (size_t l = 0; l < Lout; ++l) {
                double acc = bf[co];
                for (size_t ci = 0; ci < Cin; ++ci)
                    for (size_t k = 0; k < K; ++k) {
                        const long pos = static_cast<long>(l * stride + k * dilation) - padding;
                        if (pos >= 0 && pos < static_cast<long>(L)) acc += double(wf[(co * Cin + ci) * K + k]) * xf[(n * Cin + ci) * L + pos];
                    }
                if (gelu) acc = 0.5 * acc * (1.0 + std::erf(acc / std::sqrt(2.0)));
                worst = std::max(worst, std::fabs(acc - got[(n * Cout + co) * Lout + l]));
            }
    EXPECT_LT(worst, tol);
}
GPU_TEST(LazyNodes, Conv1dMatchesFloat64Loops) {
    conv1d_case(DType::Float32, 2, 5, 37, 7, 3, 1, 1, 1, false, 1e-4);
    conv1d_case(DType::Float32, 1, 4, 50, 6, 4, 3, 2, 2, true, 1e-4);
    conv1d_case(DType::BFloat16, 2, 16, 64, 24, 3, 2, 1, 1, true, 2e-2);  // the Whisper stem pattern: conv, GELU
    conv1d_case(DType::Float16, 1, 8, 40, 8, 3, 1, 0, 1, false, 2e-2);
}

static std::string plan_kernels() {
    std::string s;
    for (const auto &k : graph::last_gpu_plan_kernels()) s += (s.empty() ? "" : " ") + k;
    return s;
}
// Every transpose combination of a product large enough for the matrix cores: operands stored the "wrong" way
// round are transposed once by a gather, a transposed view of contiguous memory is consumed as it lies.
static void matmul_layout_case(DType dt, double tol) {
    const size_t M = 300, K = 200, N = 260;
    auto a = axtest::randn({M, K}, 91).astype(dt), b = axtest::randn({K, N}, 92).astype(dt);
    const auto af = host_floats(a.astype(DType::Float32)), bf = host_floats(b.astype(DType::Float32));
    std::vector<double> want(M * N, 0.0);
    for (size_t i = 0; i < M; ++i)
        for (size_t k = 0; k < K; ++k)
            for (size_t j = 0; j < N; ++j) want[i * N + j] += double(af[i * K + k]) * double(bf[k * N + j]);
    auto check = [&](const Tensor &r, const char *what) {
        EXPECT_TRUE(r.shape() == Shape({M, N}));
        const auto h = host_floats(r);
        double worst = 0.0;
        for (size_t i = 0; i < M * N; ++i) worst = std::max(worst, std::abs(double(h[i]) - want[i]) / (1.0 + std::abs(want[i])));
        if (!(worst < tol)) std::fprintf(stderr, "    matmul layout case: %s\n", what);
        EXPECT_LT(worst, tol);
    };
    auto ag = a.gpu(), bg = b.gpu();
    auto at = ag.transpose({1, 0}).ascontiguousarray(), bt = bg.transpose({1, 0}).ascontiguousarray(); // stored [K, M] and [N, K]
    at.sync(); bt.sync();
    check(ops::matmul(ag, bg), "a b");
    EXPECT_EQ(plan_kernels(), std::string("strided_copy gemm")); // b transposed once
    check(ops::matmul(ag, bt, false, true), "a bT'");
    EXPECT_EQ(plan_kernels(), std::string("gemm"));
    check(ops::matmul(at, bg, true, false), "aT' b");
    EXPECT_EQ(plan_kernels(), std::string("strided_copy strided_copy gemm"));
    check(ops::matmul(at, bt, true, true), "aT' bT'");
    EXPECT_EQ(plan_kernels(), std::string("strided_copy gemm"));
    // views: the transposes below are strides over memory that already has the wanted layout
    check(ops::matmul(ag, bt.transpose({1, 0})), "a view(bT')");
    EXPECT_EQ(plan_kernels(), std::string("gemm"));
    check(ops::matmul(at.transpose({1, 0}), bt.transpose({1, 0})), "view(aT') view(bT')"); // a is stored [K, M]: one pass
    EXPECT_EQ(plan_kernels(), std::string("strided_copy gemm"));
    check(ops::matmul(ag, bg.transpose({1, 0}), false, true), "a view(b)T'");
    EXPECT_EQ(plan_kernels(), std::string("strided_copy gemm"));
}
GPU_TEST(LazyNodes, MatMulOperandLayouts) {
    matmul_layout_case(DType::Float32, 1e-4);
    matmul_layout_case(DType::BFloat16, 2e-2);
    // a small product stays as it is stored (FMA kernel, no transposing pass)
    auto x = axtest::randn({8, 16}, 93).gpu(), w = axtest::randn({16, 8}, 94).gpu();
    ops::matmul(x, w).sync();
    EXPECT_EQ(plan_kernels(), std::string("gemm"));
}

GPU_TEST(LazyNodes, EmbeddingLookup) { // tests/test_embedding.cpp:3-39
    std::vector<float> wd(12);
    for (int i = 0; i < 12; ++i) wd[i] = float(i);
    auto w = Tensor::from_data(wd.data(), {4, 3}, Device::GPU);
    std::vector<int64_t> id{0, 2};
    auto r = ops::embedding(w, Tensor::from_data(id.data(), {2}, Device::GPU));
    EXPECT_TRUE(r.shape() == Shape({2, 3}));
    auto h = host_floats(r);
    const float want[6] = {0, 1, 2, 6, 7, 8};
    for (int i = 0; i < 6; ++i) EXPECT_NEAR(h[i], want[i], 0);
    std::vector<int64_t> id2{0, 1, 2, 3, 4, 0};
    auto w2 = Tensor::from_data(wd.data(), {5, 2}, Device::GPU);
    r = ops::embedding(w2, Tensor::from_data(id2.data(), {2, 3})); // host indices are moved over
    EXPECT_TRUE(r.shape() == Shape({2, 3, 2}));
    h = host_floats(r);
    EXPECT_NEAR(h[0], 0.0f, 0); EXPECT_NEAR(h[1], 1.0f, 0); EXPECT_NEAR(h[10], 0.0f, 0); EXPECT_NEAR(h[11], 1.0f, 0);
    // positions = arange: the embedding table's leading rows, added to a sequence (the Whisper encoder's use)
    auto pos = Tensor::arange(0, 3).gpu();
    auto x = Tensor::full<float>({1, 3, 2}, 1.0f, Device::GPU);
    h = host_floats(ops::add(x, ops::embedding(w2, pos)));
    for (int i = 0; i < 6; ++i) EXPECT_NEAR(h[i], 1.0f + float(i), 0);
    std::vector<float> fidx{0.0f};
    EXPECT_THROW(ops::embedding(w, Tensor::from_data(fidx.data(), {1}, Device::GPU)), TypeError);
}

GPU_TEST(LazyNodes, GluSliceChunk) { // tests/test_nn_ergonomics.cpp:44-76
    auto in = gpu_f32({1, 2, 3, 0, 0, 0, 4, 5, 6, 0, 0, 0}, {2, 6});
    auto r = ops::glu(in, -1);
    EXPECT_TRUE(r.shape() == Shape({2, 3}));
    auto h = host_floats(r);
    const float want[6] = {0.5f, 1.0f, 1.5f, 2.0f, 2.5f, 3.0f}; // sigmoid(0) = 0.5
    for (int i = 0; i < 6; ++i) EXPECT_NEAR(h[i], want[i], 1e-5);
    auto x = axtest::randn({6, 4}, 80);
    auto g = x.gpu();
    EXPECT_TRUE(g.glu(0).shape() == Shape({3, 4}));
    auto xf = host_floats(x), g0 = host_floats(g.glu(0)), g1 = host_floats(ops::glu(ops::add(g, g), 1)); // the second on a lazy input
    for (size_t i = 0; i < 12; ++i) EXPECT_NEAR(g0[i], xf[i] / (1.0 + std::exp(-double(xf[12 + i]))), 1e-5);
    for (size_t r2 = 0; r2 < 6; ++r2)
        for (size_t c = 0; c < 2; ++c) EXPECT_NEAR(g1[r2 * 2 + c], 2 * xf[r2 * 4 + c] / (1.0 + std::exp(-2.0 * xf[r2 * 4 + 2 + c])), 1e-5);
    EXPECT_THROW(ops::glu(Tensor::zeros({2, 5}, DType::Float32, Device::GPU), -1), ValueError);
    // slices and chunks of device tensors are views; of lazy tensors, lazy Slice nodes
    auto parts = g.chunk(2, 1);
    ASSERT_EQ(parts.size(), 2u);
    EXPECT_EQ(parts[1].storage().get(), g.storage().get());
    auto ph = host_floats(parts[1]);
    for (size_t r2 = 0; r2 < 6; ++r2) EXPECT_NEAR(ph[r2 * 2], xf[r2 * 4 + 2], 0);
    auto lz = ops::relu(g).slice({Slice(1, 5, 2), Slice(-3)}); // rows 1 and 3, last three columns
    EXPECT_TRUE(lz.is_lazy());
    EXPECT_TRUE(lz.shape() == Shape({2, 3}));
    auto lh = host_floats(lz);
    for (size_t i = 0; i < 2; ++i)
        for (size_t c = 0; c < 3; ++c) EXPECT_NEAR(lh[i * 3 + c], std::max(0.0f, xf[(1 + 2 * i) * 4 + 1 + c]), 0);
}

GPU_TEST(LazyNodes, PadAndMaskedFill) { // tests/test_shape_ops_extended.cpp:42-67, tests/test_tensor_where.cpp:212-218
    auto p = ops::pad(Tensor::ones({3, 3}, DType::Float32, Device::GPU), {{1, 1}, {1, 1}}, "constant", 0.0);
    EXPECT_TRUE(p.shape() == Shape({5, 5}));
    auto h = host_floats(p);
    EXPECT_NEAR(h[0], 0.0f, 0); EXPECT_NEAR(h[2 * 5 + 2], 1.0f, 0);
    p = ops::pad(Tensor::ones({2, 2}, DType::Float32, Device::GPU), {{1, 2}, {0, 3}}, "constant", 5.0);
    EXPECT_TRUE(p.shape() == Shape({5, 5}));
    h = host_floats(p);
    EXPECT_NEAR(h[0], 5.0f, 0); EXPECT_NEAR(h[24], 5.0f, 0); EXPECT_NEAR(h[5], 1.0f, 0);
    EXPECT_THROW(ops::pad(p, {{1, 1}}), ShapeError);
    // ReLU through masked_fill, and the attention use: a (Sq, Skv) causal mask over (B, H, Sq, Skv) scores
    auto x = axtest::randn({2, 3, 4, 4}, 81);
    auto xf = host_floats(x);
    Tensor neg(x.shape(), DType::Bool), causal(Shape{4, 4}, DType::Bool);
    for (size_t i = 0; i < x.size(); ++i) static_cast<uint8_t *>(neg.data())[i] = xf[i] < 0;
    for (size_t i = 0; i < 4; ++i)
        for (size_t j = 0; j < 4; ++j) static_cast<uint8_t *>(causal.data())[i * 4 + j] = j > i;
    auto r1 = host_floats(x.gpu().masked_fill(neg.gpu(), 0.0f)), r2 = host_floats(ops::masked_fill(x.gpu() * 2.0f, causal, -1e9));
    for (size_t i = 0; i < x.size(); ++i) {
        EXPECT_NEAR(r1[i], std::max(0.0f, xf[i]), 0);
        EXPECT_NEAR(r2[i], (i % 4) > ((i / 4) % 4) ? -1e9f : 2 * xf[i], 0);
    }
    auto sm = host_floats(ops::softmax(ops::masked_fill(x.gpu(), causal.gpu(), -1e9f), -1)); // masked scores then softmax: row 0 keeps key 0 only
    EXPECT_NEAR(sm[0], 1.0f, 1e-6); EXPECT_NEAR(sm[1], 0.0f, 1e-6);
    std::vector<float> fm(16, 0.0f);
    EXPECT_THROW(ops::masked_fill(x.gpu(), Tensor::from_data(fm.data(), {4, 4}, Device::GPU), 0.0f), TypeError);
}

// The wider operator table: the reference's expectations (tests/test_tensor_comparisons.cpp:24-113,
// test_tensor_logical_bitwise.cpp:11-70 and :245-292, test_tensor_numpy_ops.cpp:13-104, test_tensor_where.cpp:26-205,
// test_tensor_activations.cpp:356-478, test_tensor_operations.cpp:107-121), result types, and what fuses.
static std::vector<int> host_truth(const Tensor &t) {
    EXPECT_TRUE(t.dtype() == DType::Bool);
    Tensor c = t.cpu().ascontiguousarray();
    const uint8_t *p = static_cast<const uint8_t *>(c.data());
    return std::vector<int>(p, p + c.size());
}

GPU_TEST(LazyNodes, ComparisonsLogicalOperationsAndWhere) {
    auto a = gpu_f32({0, 1, 2, 3, 4}, {5});
    auto two = Tensor::full({5}, 2.0f, Device::GPU);
    EXPECT_TRUE(host_truth(ops::less(a, two)) == std::vector<int>({1, 1, 0, 0, 0}));
    EXPECT_TRUE(host_truth(ops::less_equal(a, two)) == std::vector<int>({1, 1, 1, 0, 0}));
    EXPECT_TRUE(host_truth(ops::greater(a, two)) == std::vector<int>({0, 0, 0, 1, 1}));
    EXPECT_TRUE(host_truth(ops::greater_equal(a, two)) == std::vector<int>({0, 0, 1, 1, 1}));
    EXPECT_TRUE(host_truth(ops::equal(a, two)) == std::vector<int>({0, 0, 1, 0, 0}));
    EXPECT_TRUE(host_truth(a != two) == std::vector<int>({1, 1, 0, 1, 1}));
    EXPECT_TRUE(host_truth(2.5f > a + 0.0f) == std::vector<int>({1, 1, 1, 0, 0})); // the chain on the right-hand side
    EXPECT_TRUE((a < 2.0f).dtype() == DType::Bool);
    // broadcasting (test_tensor_comparisons.cpp:222-236): (3, 1) against (4) -> (3, 4)
    auto col = gpu_f32({0, 1, 2}, {3, 1}), row = gpu_f32({0, 1, 2, 3}, {4});
    auto lt = ops::less(col, row);
    EXPECT_TRUE(lt.shape() == Shape({3, 4}));
    EXPECT_TRUE(host_truth(lt) == std::vector<int>({0, 1, 1, 1, 0, 0, 1, 1, 0, 0, 0, 1}));

    bool la[] = {true, true, false, false}, lb[] = {true, false, true, false};
    auto ta = Tensor::from_data(la, {4}, Device::GPU), tb = Tensor::from_data(lb, {4}, Device::GPU);
    EXPECT_TRUE(host_truth(ops::logical_and(ta, tb)) == std::vector<int>({1, 0, 0, 0}));
    EXPECT_TRUE(host_truth(ops::logical_or(ta, tb)) == std::vector<int>({1, 1, 1, 0}));
    EXPECT_TRUE(host_truth(ops::logical_xor(ta, tb)) == std::vector<int>({0, 1, 1, 0}));
    EXPECT_TRUE(host_truth(ops::logical_not(ta)) == std::vector<int>({0, 0, 1, 1}));
    EXPECT_TRUE(host_truth(ops::logical_not(gpu_f32({1.0f, 0.0f, -3.5f, 0.0f}, {4}))) == std::vector<int>({0, 1, 0, 1}));

    // where
    auto cond = Tensor::from_data(lb, {4}, Device::GPU); // {1, 0, 1, 0}
    auto w = host_floats(ops::where(cond, Tensor::full({4}, 1.0f, Device::GPU), Tensor::full({4}, 0.0f, Device::GPU)));
    EXPECT_TRUE(w == std::vector<float>({1, 0, 1, 0}));
    auto x = gpu_f32({1, -2, 3, -4, 0}, {5});
    auto zero = Tensor::zeros({5}, DType::Float32, Device::GPU);
    EXPECT_TRUE(host_floats(ops::where(ops::greater(x, zero), x, zero)) == std::vector<float>({1, 0, 3, 0, 0})); // ReLU pattern
    EXPECT_TRUE(host_floats(x.where(x > 0.0f, zero - 1.0f)) == std::vector<float>({1, -1, 3, -1, -1}));
    // scalars broadcast on either branch; a (2, 1) condition against (2, 3) branches; mixed branch types promote
    auto m = gpu_f32({1, 2, 3, 4, 5, 6}, {2, 3});
    bool rows_on[] = {true, false};
    auto rc = Tensor::from_data(rows_on, {2, 1}, Device::GPU);
    EXPECT_TRUE(host_floats(ops::where(rc, m, Tensor::full({1}, -1.0f, Device::GPU))) == std::vector<float>({1, 2, 3, -1, -1, -1}));
    auto mixed = ops::where(rc, m.bfloat16(), m * 10.0f);
    EXPECT_TRUE(mixed.dtype() == DType::Float32);
    EXPECT_TRUE(host_floats(mixed) == std::vector<float>({1, 2, 3, 40, 50, 60}));
    // the attention use: where(mask, -1e9, scores) then softmax
    auto sc = gpu_f32({0.5f, 0.3f, 0.2f, 0.1f}, {2, 2});
    bool mk[] = {false, true, false, false};
    auto masked = ops::where(Tensor::from_data(mk, {2, 2}, Device::GPU), Tensor::full({2, 2}, -1e9f, Device::GPU), sc);
    auto sm = host_floats(ops::softmax(masked, -1));
    EXPECT_NEAR(sm[0], 1.0f, 1e-6); EXPECT_NEAR(sm[1], 0.0f, 1e-6);
    EXPECT_THROW(ops::less(Tensor::zeros({3}), Tensor::zeros({3})), RuntimeError); // CPU tensors: no CPU compute path here
}

GPU_TEST(LazyNodes, MathOperatorsRoundingTestsAndActivations) {
    EXPECT_TRUE(host_floats(gpu_f32({-3, -1, 0, 1, 3}, {5}).sign()) == std::vector<float>({-1, -1, 0, 1, 1}));
    auto x = gpu_f32({-2.7f, -0.5f, 0.5f, 2.7f}, {4});
    EXPECT_TRUE(host_floats(x.floor()) == std::vector<float>({-3, -1, 0, 2}));
    EXPECT_TRUE(host_floats(x.ceil()) == std::vector<float>({-2, 0, 1, 3}));
    EXPECT_TRUE(host_floats(x.trunc()) == std::vector<float>({-2, 0, 0, 2}));
    EXPECT_TRUE(host_floats(gpu_f32({0.5f, 1.5f, -0.5f, 2.4f}, {4}).round()) == std::vector<float>({1, 2, -1, 2}));
    auto r2 = host_floats(ops::round(gpu_f32({3.14159f, -2.71828f}, {2}), 2));
    EXPECT_NEAR(r2[0], 3.14f, 1e-5); EXPECT_NEAR(r2[1], -2.72f, 1e-5);
    auto cb = host_floats(gpu_f32({8, 27, 64}, {3}).cbrt());
    EXPECT_NEAR(cb[0], 2.0f, 1e-5); EXPECT_NEAR(cb[1], 3.0f, 1e-5); EXPECT_NEAR(cb[2], 4.0f, 1e-5);
    auto t = gpu_f32({1.0f, NAN, INFINITY, -INFINITY, 0.0f}, {5});
    EXPECT_TRUE(host_truth(t.isnan()) == std::vector<int>({0, 1, 0, 0, 0}));
    EXPECT_TRUE(host_truth(t.isinf()) == std::vector<int>({0, 0, 1, 1, 0}));
    EXPECT_TRUE(host_truth(t.isfinite()) == std::vector<int>({1, 0, 0, 0, 1}));
    EXPECT_TRUE(host_floats(gpu_f32({-5, -1, 0, 1, 5}, {5}).clip(-2.0, 2.0)) == std::vector<float>({-2, -1, 0, 1, 2}));
    auto p = host_floats(ops::power(Tensor::full({2, 2}, 3.0f, Device::GPU), Tensor::full({2, 2}, 4.0f, Device::GPU)));
    for (float v : p) EXPECT_NEAR(v, 81.0f, 1e-4);
    EXPECT_TRUE(host_floats(ops::modulo(gpu_f32({5.5f, -5.5f, 7.0f}, {3}), gpu_f32({2, 2, -3}, {3}))) == std::vector<float>({1.5f, -1.5f, 1.0f}));
    auto at = host_floats(ops::atan2(gpu_f32({1, 1, 0}, {3}), gpu_f32({1, 0, 1}, {3})));
    EXPECT_NEAR(at[0], M_PI / 4, 1e-6); EXPECT_NEAR(at[1], M_PI / 2, 1e-6); EXPECT_NEAR(at[2], 0.0, 1e-6);
    auto hy = host_floats(ops::hypot(gpu_f32({3, 0, 5}, {3}), gpu_f32({4, 5, 12}, {3})));
    EXPECT_NEAR(hy[0], 5.0f, 1e-5); EXPECT_NEAR(hy[1], 5.0f, 1e-5); EXPECT_NEAR(hy[2], 13.0f, 1e-5);
    auto e = host_floats(ops::erf(gpu_f32({0, 1, -1}, {3})));
    EXPECT_NEAR(e[0], 0.0f, 1e-6); EXPECT_NEAR(e[1], 0.8427f, 1e-4); EXPECT_NEAR(e[1] + e[2], 0.0f, 1e-6);
    auto lk = host_floats(gpu_f32({-2, 3, 0}, {3}).leaky_relu());
    EXPECT_NEAR(lk[0], -0.02f, 1e-8); EXPECT_NEAR(lk[1], 3.0f, 0); EXPECT_NEAR(lk[2], 0.0f, 0);
    EXPECT_NEAR(host_floats(gpu_f32({-2}, {1}).leaky_relu(0.2f))[0], -0.4f, 1e-7);

    // a long mixed chain is still ONE launch, float64 check on random data
    auto v = axtest::randn({33, 200}, 120);
    auto g = v.gpu();
    auto y = ops::sin(g) * ops::cos(g) + ops::floor(g * 2.0f) - ops::leaky_relu(g, 0.1f);
    auto got = host_floats(y), vf = host_floats(v);
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 4u); // sin, cos and leaky_relu of the shared input are chains of their own
    for (size_t i = 0; i < vf.size(); ++i) {
        const double d = vf[i];
        EXPECT_NEAR(got[i], std::sin(d) * std::cos(d) + std::floor(double(vf[i] * 2.0f)) - (d > 0 ? d : double(0.1f) * d), 1e-5);
    }
    auto z = host_floats(ops::tan(ops::sign(g) * ops::sqrt(ops::abs(g) + 1.0f) * 0.25f));
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 2u);
    for (size_t i = 0; i < vf.size(); i += 7) {
        const double d = vf[i], sg = d > 0 ? 1 : d < 0 ? -1 : 0;
        EXPECT_NEAR(z[i], std::tan(sg * std::sqrt(std::fabs(d) + 1.0) * 0.25), 1e-5);
    }
    // softmax(x) > 1/cols, in one kernel up to the Bool result; bf16 input
    auto pr = ops::greater(ops::softmax(g, -1), Tensor::full({1}, 1.0f / 200.0f, Device::GPU));
    auto truth = host_truth(pr);
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
    size_t ones = 0;
    for (int b : truth) ones += b;
    EXPECT_TRUE(ones > 33u * 20u && ones < 33u * 180u);
    auto hb = host_truth(ops::less(g.bfloat16(), Tensor::zeros({1}, DType::BFloat16, Device::GPU)));
    for (size_t i = 0; i < vf.size(); ++i) EXPECT_EQ(hb[i], float(bfloat16_t(vf[i])) < 0.0f ? 1 : 0);
}

GPU_TEST(LazyNodes, ProductsAnyAllAndCasts) {
    auto t = gpu_f32({1, 2, 3, 4}, {2, 2});
    EXPECT_NEAR(ops::prod(t).item<float>(), 24.0f, 1e-5);
    EXPECT_TRUE(host_floats(t.prod(0)) == std::vector<float>({3, 8}));
    EXPECT_TRUE(host_floats(t.prod(1)) == std::vector<float>({2, 12}));
    EXPECT_NEAR(ops::prod(ops::sqrt(gpu_f32({4, 9, 16}, {3}))).item<float>(), 24.0f, 1e-4); // tests/test_fusion_extended.cpp:376-385
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
    EXPECT_TRUE(host_truth(ops::any(gpu_f32({0, 0, 1, 0}, {4}))) == std::vector<int>({1}));
    EXPECT_TRUE(host_truth(ops::all(gpu_f32({1, 1, 1, 1}, {4}))) == std::vector<int>({1}));
    EXPECT_TRUE(host_truth(ops::all(gpu_f32({1, 0, 1, 1}, {4}))) == std::vector<int>({0}));
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u); // != 0 and the reduction in one launch
    auto m = gpu_f32({0, 0, 0, 1, 0, 2, 3, 4, 5}, {3, 3});
    EXPECT_TRUE(host_truth(m.any(1)) == std::vector<int>({0, 1, 1}));
    EXPECT_TRUE(host_truth(m.all(1)) == std::vector<int>({0, 0, 1}));
    EXPECT_TRUE(host_truth(m.any(0)) == std::vector<int>({1, 1, 1}));
    EXPECT_TRUE(host_truth(m.all(0)) == std::vector<int>({0, 0, 0}));
    EXPECT_TRUE(m.any(0, true).shape() == Shape({1, 3}));
    // all(isfinite(x)) as the reference's audio tests use it (tests/test_audio.cpp:118-123)
    auto v = axtest::randn({64, 100}, 121).gpu();
    EXPECT_TRUE(host_truth(ops::all(ops::isfinite(v))) == std::vector<int>({1}));
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
    EXPECT_TRUE(host_truth(ops::any(ops::isnan((v - v) / (v - v)))) == std::vector<int>({1}));
    // reductions over nothing: an empty result stays empty, an empty extent gives the identity
    auto z = Tensor::zeros({2, 0, 4}, DType::Float32, Device::GPU), z0 = Tensor::zeros({0, 3, 4}, DType::Float32, Device::GPU);
    EXPECT_TRUE(host_floats(ops::sum(z, {1})) == std::vector<float>(8, 0.0f));
    EXPECT_TRUE(host_floats(ops::prod(z, {1})) == std::vector<float>(8, 1.0f));
    EXPECT_TRUE(ops::sum(z, {1}).shape() == Shape({2, 4}));
    EXPECT_TRUE(ops::sum(z, {2}).shape() == Shape({2, 0}));
    EXPECT_EQ(ops::sum(z, {2}).size(), 0u);
    EXPECT_TRUE(ops::sum(z0, {1}).shape() == Shape({0, 4}));
    EXPECT_NEAR(ops::sum(z).item<float>(), 0.0f, 0);
    EXPECT_TRUE(std::isnan(host_floats(ops::mean(z, {1}))[0]));
    EXPECT_TRUE(host_truth(ops::any(z, {1})) == std::vector<int>(8, 0));
    EXPECT_TRUE(host_truth(ops::all(z, {1})) == std::vector<int>(8, 1));
    EXPECT_THROW(ops::max(z, {1}), ValueError);
    // products along a middle axis and over everything, against float64
    auto s = axtest::uniform({4, 9, 16}, 122, 0.9f, 1.1f);
    auto sf = host_floats(s), pm = host_floats(s.gpu().prod(1));
    for (size_t o = 0; o < 4; ++o)
        for (size_t i = 0; i < 16; ++i) {
            double want = 1;
            for (size_t a = 0; a < 9; ++a) want *= sf[(o * 9 + a) * 16 + i];
            EXPECT_NEAR(pm[o * 16 + i], want, 1e-5);
        }
    // casts: lazy nodes that fold into the neighbouring kernel
    auto c = (v * 2.0f).astype(DType::BFloat16);
    EXPECT_TRUE(c.dtype() == DType::BFloat16);
    auto cf = host_floats(c), vf = host_floats(v);
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u); // multiply and round in one launch
    for (size_t i = 0; i < vf.size(); ++i) EXPECT_NEAR(cf[i], float(bfloat16_t(vf[i] * 2.0f)), 0);
    auto widened = host_floats(ops::relu(c.to_float()) + 1.0f); // bf16 -> f32 in front of a chain: converted on load
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
    for (size_t i = 0; i < vf.size(); ++i) EXPECT_NEAR(widened[i], std::max(0.0f, float(bfloat16_t(vf[i] * 2.0f))) + 1.0f, 0);
    // a narrowing cast in mid-chain rounds there: relu(bf16(x * 3)) * 1.5 computed from the rounded value
    auto mid = host_floats(ops::relu((v * 3.0f).astype(DType::BFloat16)).to_float() * 1.5f);
    for (size_t i = 0; i < vf.size(); ++i) EXPECT_NEAR(mid[i], std::max(0.0f, float(bfloat16_t(vf[i] * 3.0f))) * 1.5f, 0);
    EXPECT_TRUE(host_truth(gpu_f32({0, 2, -1, 0}, {4}).to_bool()) == std::vector<int>({0, 1, 1, 0}));
    EXPECT_TRUE(host_floats(gpu_f32({0, 2, -1, 0}, {4}).to_bool().to_float() * 3.0f) == std::vector<float>({0, 3, 3, 0}));
    auto tv = v.transpose({1, 0}).astype(DType::Float16); // a strided view: one converting gather
    EXPECT_EQ(host_floats(tv).size(), vf.size());
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
    EXPECT_EQ(graph::last_gpu_plan_kernels()[0], std::string("strided_copy"));
    auto tvf = host_floats(tv);
    for (size_t i = 0; i < 64; ++i)
        for (size_t j = 0; j < 100; j += 9) EXPECT_NEAR(tvf[j * 64 + i], float(float16_t(vf[i * 100 + j])), 0);
}

// Grouped convolutions (tests/test_conv1d.cpp:104-119, tests/test_conv2d.cpp:113-127 give the shapes; the values are
// checked against float64 loops) and the pad modes other than "constant" (src/tensor/operations.cpp:2216-2246).
GPU_TEST(LazyNodes, GroupedConvolutions) {
    {
        auto input = gpu_f32({1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12}, {1, 4, 3});
        std::vector<float> ones(8, 1.0f);
        auto r = ops::conv1d(input, Tensor::from_data(ones.data(), {4, 2, 1}, Device::GPU), Tensor(), 1, 0, 1, 2);
        EXPECT_TRUE(r.shape() == Shape({1, 4, 3}));
        EXPECT_TRUE(host_floats(r) == std::vector<float>({5, 7, 9, 5, 7, 9, 17, 19, 21, 17, 19, 21})); // channel pairs summed
        std::vector<float> in2(36);
        for (int i = 0; i < 36; ++i) in2[i] = float(i + 1);
        auto r2 = ops::conv2d(Tensor::from_data(in2.data(), {1, 4, 3, 3}, Device::GPU), Tensor::from_data(ones.data(), {4, 2, 1, 1}, Device::GPU), Tensor(), {1, 1},
                              {0, 0}, {1, 1}, 2);
        EXPECT_TRUE(r2.shape() == Shape({1, 4, 3, 3}));
        auto h2 = host_floats(r2);
        for (int i = 0; i < 9; ++i) {
            EXPECT_NEAR(h2[i], in2[i] + in2[9 + i], 0); EXPECT_NEAR(h2[9 + i], in2[i] + in2[9 + i], 0);
            EXPECT_NEAR(h2[18 + i], in2[18 + i] + in2[27 + i], 0); EXPECT_NEAR(h2[27 + i], in2[18 + i] + in2[27 + i], 0);
        }
    }
    for (DType dt : {DType::Float32, DType::BFloat16}) {
        const size_t N = 2, Cin = 12, L = 37, Cout = 18, K = 3;
        for (int groups : {2, 3, 6}) {
            const size_t Cg = Cin / groups, Og = Cout / groups;
            const int stride = 2, padding = 1, dilation = 2;
            auto x = axtest::randn({N, Cin, L}, 130 + groups).astype(dt), w = axtest::randn({Cout, Cg, K}, 140 + groups).astype(dt), b = axtest::randn({Cout}, 150).astype(dt);
            auto xf = host_floats(x), wf = host_floats(w), bf = host_floats(b);
            auto y = ops::conv1d(x.gpu(), w.gpu(), b.gpu(), stride, padding, dilation, groups);
            const size_t Lout = (L + 2 * padding - dilation * (K - 1) - 1) / stride + 1;
            EXPECT_TRUE(y.shape() == Shape({N, Cout, Lout}));
            auto got = host_floats(y);
            const double tol = dt == DType::Float32 ? 1e-4 : 6e-2;
            for (size_t n = 0; n < N; ++n)
                for (size_t o = 0; o < Cout; ++o)
                    for (size_t l = 0; l < Lout; ++l) {
                        double acc = bf[o];
                        const size_t g = o / Og;
                        for (size_t c = 0; c < Cg; ++c)
                            for (size_t k = 0; k < K; ++k) {
                                const long pos = long(l * stride + k * dilation) - padding;
                                if (pos >= 0 && pos < long(L)) acc += double(xf[(n * Cin + g * Cg + c) * L + pos]) * wf[(o * Cg + c) * K + k];
                            }
                        EXPECT_NEAR(got[(n * Cout + o) * Lout + l], acc, tol * (1 + std::fabs(acc)));
                    }
        }
    }
    { // depthwise 2-D (groups == C_in == C_out), no bias
        const size_t N = 2, C = 5, H = 9, W = 11, KH = 3, KW = 2;
        auto x = axtest::randn({N, C, H, W}, 160), w = axtest::randn({C, 1, KH, KW}, 161);
        auto xf = host_floats(x), wf = host_floats(w);
        auto y = ops::conv2d(x.gpu(), w.gpu(), Tensor(), {1, 2}, {1, 0}, {1, 1}, static_cast<int>(C));
        const size_t Ho = H + 2 - KH + 1, Wo = (W - KW) / 2 + 1;
        EXPECT_TRUE(y.shape() == Shape({N, C, Ho, Wo}));
        auto got = host_floats(y);
        for (size_t n = 0; n < N; ++n)
            for (size_t c = 0; c < C; ++c)
                for (size_t i = 0; i < Ho; ++i)
                    for (size_t j = 0; j < Wo; ++j) {
                        double acc = 0;
                        for (size_t a = 0; a < KH; ++a)
                            for (size_t bb = 0; bb < KW; ++bb) {
                                const long r = long(i + a) - 1, q = long(j * 2 + bb);
                                if (r >= 0 && r < long(H)) acc += double(xf[((n * C + c) * H + r) * W + q]) * wf[(c * KH + a) * KW + bb];
                            }
                        EXPECT_NEAR(got[((n * C + c) * Ho + i) * Wo + j], acc, 1e-4);
                    }
    }
    EXPECT_THROW(ops::conv1d(Tensor::zeros({1, 4, 3}, DType::Float32, Device::GPU), Tensor::zeros({4, 2, 1}, DType::Float32, Device::GPU), Tensor(), 1, 0, 1, 0), ValueError);
    EXPECT_THROW(ops::conv1d(Tensor::zeros({1, 4, 3}, DType::Float32, Device::GPU), Tensor::zeros({4, 2, 1}, DType::Float32, Device::GPU), Tensor(), 1, 0, 1, 4), ShapeError);
    EXPECT_THROW(ops::conv1d(Tensor::zeros({1, 4, 3}, DType::Float32, Device::GPU), Tensor::zeros({3, 2, 1}, DType::Float32, Device::GPU), Tensor(), 1, 0, 1, 2), ShapeError);
}

GPU_TEST(LazyNodes, PadModes) {
    auto x = gpu_f32({1, 2, 3, 4}, {4});
    EXPECT_TRUE(host_floats(ops::pad(x, {{2, 3}}, "reflect")) == std::vector<float>({3, 2, 1, 2, 3, 4, 3, 2, 1}));
    EXPECT_TRUE(host_floats(ops::pad(x, {{2, 3}}, "replicate")) == std::vector<float>({1, 1, 1, 2, 3, 4, 4, 4, 4}));
    EXPECT_TRUE(host_floats(ops::pad(x, {{2, 5}}, "circular")) == std::vector<float>({3, 4, 1, 2, 3, 4, 1, 2, 3, 4, 1}));
    EXPECT_THROW(ops::pad(x, {{4, 0}}, "reflect"), ValueError);
    EXPECT_THROW(ops::pad(x, {{1, 1}}, "mirror"), ValueError);
    auto idx = [](long c, long n, int mode) { // the reference's get_source_idx
        if (c >= 0 && c < n) return c;
        if (mode == 1) return c < 0 ? -c : 2 * n - c - 2;
        if (mode == 2) return c < 0 ? 0L : n - 1;
        return ((c % n) + n) % n;
    };
    const char *names[4] = {"constant", "reflect", "replicate", "circular"};
    for (DType dt : {DType::Float32, DType::Float16}) {
        auto v = axtest::randn({3, 6, 40}, 170).astype(dt);
        auto vf = host_floats(v);
        for (int mode = 1; mode <= 3; ++mode) {
            auto got = host_floats(ops::pad(v.gpu().transpose({1, 0, 2}), {{1, 2}, {2, 0}, {3, 5}}, names[mode])); // a (6, 3, 40) view -> (9, 5, 48)
            ASSERT_EQ(got.size(), size_t(9 * 5 * 48));
            for (long a = 0; a < 9; ++a)
                for (long b = 0; b < 5; ++b)
                    for (long c = 0; c < 48; ++c) {
                        const long sa = idx(a - 1, 6, mode), sb = idx(b - 2, 3, mode), sc = idx(c - 3, 40, mode);
                        EXPECT_NEAR(got[(a * 5 + b) * 48 + c], vf[(sb * 6 + sa) * 40 + sc], 0);
                    }
        }
    }
}

GPU_TEST(LazyNodes, BatchNorm1dInference) {
    const size_t N = 3, C = 5, L = 7;
    auto w = axtest::uniform({C}, 90, 0.5f, 1.5f), b = axtest::randn({C}, 91), rm = axtest::randn({C}, 92), rv = axtest::uniform({C}, 93, 0.2f, 2.0f);
    std::map<std::string, Tensor> sd{{"weight", w.gpu()}, {"bias", b.gpu()}, {"running_mean", rm.gpu()}, {"running_var", rv.gpu()}};
    nn::BatchNorm1d bn;
    EXPECT_THROW(bn(Tensor::zeros({N, C}, DType::Float32, Device::GPU)), RuntimeError);
    bn.load_state_dict(sd);
    auto wf = host_floats(w), bf = host_floats(b), mf = host_floats(rm), vf = host_floats(rv);
    for (int nd = 2; nd <= 3; ++nd) {
        auto x = nd == 2 ? axtest::randn({N, C}, 94) : axtest::randn({N, C, L}, 95);
        auto xf = host_floats(x), got = host_floats(bn(x.gpu()));
        const size_t inner = nd == 2 ? 1 : L;
        for (size_t i = 0; i < xf.size(); ++i) {
            const size_t c = (i / inner) % C;
            EXPECT_NEAR(got[i], (double(xf[i]) - mf[c]) / std::sqrt(double(vf[c]) + 1e-5) * wf[c] + bf[c], 1e-4);
        }
    }
    EXPECT_THROW(bn(Tensor::zeros({N, C, L, 2}, DType::Float32, Device::GPU)), ShapeError);
}

GPU_TEST(LazyNodes, TransposeRewritesKeepFusion) {
    // unary over a pending transpose sinks below it; transposes compose, the identity disappears
    auto x = axtest::randn({8, 16, 32}, 96);
    auto g = x.gpu();
    auto y = (g + 1.0f).transpose({0, 2, 1}).gelu().transpose({0, 2, 1}); // == gelu(x + 1), no gather
    EXPECT_TRUE(y.shape() == x.shape());
    auto got = host_floats(y), xf = host_floats(x);
    EXPECT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
    for (size_t i = 0; i < xf.size(); ++i) {
        const double v = double(xf[i]) + 1.0;
        EXPECT_NEAR(got[i], 0.5 * v * (1.0 + std::erf(v / std::sqrt(2.0))), 1e-4);
    }
    auto z = host_floats(ops::relu(g.transpose({2, 0, 1})).transpose({1, 0, 2})); // composed permutation (0, 2, 1) of x
    for (size_t a = 0; a < 8; ++a)
        for (size_t c = 0; c < 32; ++c)
            for (size_t b2 = 0; b2 < 16; ++b2) EXPECT_NEAR(z[(a * 32 + c) * 16 + b2], std::max(0.0f, xf[(a * 16 + b2) * 32 + c]), 0);
}

// Self-attention stacks the three input projections into one product; passing the same values as
// three distinct tensor objects takes the projection-by-projection path.  Both must agree, before
// and after the parameters are replaced (the stacked weight is rebuilt), with and without biases.
GPU_TEST(FlashAttentionMHA, FusedQkvProjectionMatchesSeparateProjections) {
    const size_t B = 2, S = 70, Dm = 64;
    auto x = axtest::randn({B, S, Dm}, 300).gpu();
    for (bool with_bias : {true, false}) {
        nn::MultiHeadAttention mha(4, with_bias);
        for (uint64_t round = 0; round < 2; ++round) {
            std::map<std::string, Tensor> sd;
            uint64_t seed = 310 + 20 * round;
            for (const char *name : {"q_proj", "k_proj", "v_proj", "out_proj"}) {
                sd[std::string(name) + ".weight"] = axtest::randn({Dm, Dm}, seed++, DType::Float32, 0.125f).gpu();
                if (with_bias && std::string(name) != "k_proj") sd[std::string(name) + ".bias"] = axtest::randn({Dm}, seed++, DType::Float32, 0.1f).gpu(); // no key bias, as in Whisper
            }
            mha.load_state_dict(sd, "", /*strict=*/false);
            const Tensor x2 = x, x3 = x; // same storage, different objects
            auto fused = host_floats(mha.forward(x, x, x)), separate = host_floats(mha.forward(x, x2, x3));
            double worst = 0;
            for (size_t i = 0; i < fused.size(); ++i) worst = std::max(worst, std::fabs(double(fused[i]) - separate[i]));
            EXPECT_LT(worst, 1e-4);
        }
    }
}

// A projection weight replaced through the module's mutable parameter list (no load_state_dict, no to()): the old
// weight's device block is freed and the same-sized new one is likely to land at the same address, which an
// address comparison would take for "unchanged".  The stacked q/k/v weight must follow the new parameter.
GPU_TEST(FlashAttentionMHA, StackedProjectionFollowsAParameterSwappedInPlace) {
    const size_t B = 1, S = 40, Dm = 64;
    auto x = axtest::randn({B, S, Dm}, 400).gpu();
    nn::MultiHeadAttention mha(4);
    std::map<std::string, Tensor> sd;
    uint64_t seed = 410;
    for (const char *name : {"q_proj", "k_proj", "v_proj", "out_proj"}) {
        sd[std::string(name) + ".weight"] = axtest::randn({Dm, Dm}, seed++, DType::Float32, 0.125f).gpu();
        sd[std::string(name) + ".bias"] = axtest::randn({Dm}, seed++, DType::Float32, 0.1f).gpu();
    }
    mha.load_state_dict(sd);
    const Tensor x2 = x, x3 = x;
    auto before = host_floats(mha.forward(x, x, x));
    auto params = mha.named_parameters();
    bool swapped = false;
    for (auto &np : params)
        if (np.first == "q_proj.weight") {
            *np.second = Tensor(); // frees the old block first, so that the new weight can take its place
            *np.second = axtest::randn({Dm, Dm}, 999, DType::Float32, 0.125f).gpu();
            swapped = true;
        }
    ASSERT_TRUE(swapped);
    auto fused = host_floats(mha.forward(x, x, x)), separate = host_floats(mha.forward(x, x2, x3));
    double moved = 0, apart = 0;
    for (size_t i = 0; i < fused.size(); ++i) {
        moved = std::max(moved, std::fabs(double(fused[i]) - before[i]));
        apart = std::max(apart, std::fabs(double(fused[i]) - separate[i]));
    }
    EXPECT_GT(moved, 1e-3); // the output changed with the weight ...
    EXPECT_LT(apart, 1e-4); // ... to what the three separate projections give
}

// Lazy tensors handed in as parameters (a scaled, narrowed random matrix is the usual way to write one) are run once
// when the module takes them: forwards see memory, the stacked projection applies, and no forward repeats the
// parameter's own arithmetic.
GPU_TEST(FlashAttentionMHA, LazyParametersAreMaterialisedOnce) {
    const size_t S = 48, Dm = 64;
    auto x = axtest::randn({1, S, Dm}, 500, DType::Float32).gpu().astype(DType::BFloat16);
    x.sync();
    std::map<std::string, Tensor> sd;
    uint64_t seed = 510;
    for (const char *name : {"q_proj", "k_proj", "v_proj", "out_proj"}) {
        sd[std::string(name) + ".weight"] = (axtest::randn({Dm, Dm}, seed++, DType::Float32).gpu() * 0.125f).astype(DType::BFloat16);
        sd[std::string(name) + ".bias"] = (axtest::randn({Dm}, seed++, DType::Float32).gpu() * 0.1f).astype(DType::BFloat16);
        EXPECT_TRUE(sd[std::string(name) + ".weight"].is_lazy());
    }
    nn::MultiHeadAttention mha(4);
    mha.load_state_dict(sd);
    for (auto &np : mha.named_parameters()) EXPECT_FALSE(np.second->is_lazy());
    Tensor y = x + mha.forward(x, x, x);
    y.sync();
    ASSERT_EQ(graph::last_gpu_plan_kernels().size(), 1u);
    for (const auto &k : graph::last_gpu_plan_kernels()) EXPECT_EQ(k, std::string("gemm")); // the output projection with bias and residual, nothing else
    // a lazy weight assigned through the mutable parameter list is settled by the first forward
    for (auto &np : mha.named_parameters())
        if (np.first == "out_proj.weight") *np.second = (axtest::randn({Dm, Dm}, 599, DType::Float32).gpu() * 0.125f).astype(DType::BFloat16);
    (x + mha.forward(x, x, x)).sync();
    for (auto &np : mha.named_parameters()) EXPECT_FALSE(np.second->is_lazy());
}

GPU_TEST(LazyNodes, Conv2dKnownAnswers) { // tests/test_conv2d.cpp:3-111 of the reference
    auto x9 = gpu_f32({1, 2, 3, 4, 5, 6, 7, 8, 9}, {1, 1, 3, 3});
    auto w4 = gpu_f32({1, 1, 1, 1}, {1, 1, 2, 2});
    auto r = ops::conv2d(x9, w4);
    EXPECT_TRUE(r.shape() == Shape({1, 1, 2, 2}));
    auto h = host_floats(r);
    const float want[4] = {12, 16, 24, 28};
    for (int i = 0; i < 4; ++i) EXPECT_NEAR(h[i], want[i], 0);
    r = ops::conv2d(x9, Tensor::ones({1, 1, 3, 3}, DType::Float32, Device::GPU), Tensor(), {1, 1}, {1, 1}); // padding 1
    EXPECT_TRUE(r.shape() == Shape({1, 1, 3, 3}));
    EXPECT_NEAR(host_floats(r)[4], 45.0f, 0);
    std::vector<float> d16(16), d25(25);
    for (int i = 0; i < 16; ++i) d16[i] = float(i + 1);
    for (int i = 0; i < 25; ++i) d25[i] = float(i + 1);
    r = ops::conv2d(Tensor::from_data(d16.data(), {1, 1, 4, 4}, Device::GPU), w4, Tensor(), {2, 2}); // stride 2
    EXPECT_TRUE(r.shape() == Shape({1, 1, 2, 2}));
    h = host_floats(r);
    const float want_s[4] = {14, 22, 46, 54};
    for (int i = 0; i < 4; ++i) EXPECT_NEAR(h[i], want_s[i], 0);
    r = ops::conv2d(Tensor::from_data(d25.data(), {1, 1, 5, 5}, Device::GPU), w4, Tensor(), {1, 1}, {0, 0}, {2, 2}); // dilation 2
    EXPECT_TRUE(r.shape() == Shape({1, 1, 3, 3}));
    EXPECT_NEAR(host_floats(r)[0], 28.0f, 0);
    EXPECT_NEAR(ops::conv2d(gpu_f32({1, 2, 3, 4}, {1, 1, 2, 2}), w4, gpu_f32({10}, {1})).item<float>(), 20.0f, 0); // bias
    r = ops::conv2d(gpu_f32({1, 2, 3, 4, 5, 6, 7, 8, 9}, {1, 3, 3}), w4); // unbatched
    EXPECT_TRUE(r.shape() == Shape({1, 2, 2}));
    EXPECT_NEAR(host_floats(r)[0], 12.0f, 0);
    EXPECT_THROW(ops::conv2d(x9, w4, Tensor(), {1, 1}, {0, 0}, {1, 1}, 2), ShapeError); // 1 channel cannot be cut into 2 groups
}

GPU_TEST(LazyNodes, Conv2dMatchesFloat64Loops) {
    struct Case { DType dt; size_t N, C, H, W, Co, KH, KW; int sh, sw, ph, pw, dh, dw; bool relu; double tol; };
    const Case cases[] = {{DType::Float32, 2, 3, 9, 11, 5, 3, 3, 1, 1, 1, 1, 1, 1, false, 1e-4},
                          {DType::Float32, 1, 4, 12, 10, 6, 2, 3, 2, 1, 0, 2, 1, 2, true, 1e-4},
                          {DType::BFloat16, 2, 8, 16, 16, 16, 3, 3, 2, 2, 1, 1, 1, 1, true, 2e-2}};
    for (const Case &c : cases) {
        auto x = axtest::randn({c.N, c.C, c.H, c.W}, 400, c.dt), w = axtest::randn({c.Co, c.C, c.KH, c.KW}, 401, c.dt, 0.2f), b = axtest::randn({c.Co}, 402, c.dt, 0.5f);
        Tensor y = ops::conv2d(x.gpu(), w.gpu(), b.gpu(), {c.sh, c.sw}, {c.ph, c.pw}, {c.dh, c.dw});
        if (c.relu) y = y.relu();
        const size_t Ho = (c.H + 2 * c.ph - c.dh * (c.KH - 1) - 1) / c.sh + 1, Wo = (c.W + 2 * c.pw - c.dw * (c.KW - 1) - 1) / c.sw + 1;
        ASSERT_TRUE(y.shape() == Shape({c.N, c.Co, Ho, Wo}));
        auto got = host_floats(y);
        if (c.relu) EXPECT_EQ(graph::last_gpu_plan_kernels().back(), std::string("gemm")); // relu rode in the GEMM epilogue, through the reshape and the transpose
        auto xf = host_floats(x), wf = host_floats(w), bf = host_floats(b);
        double worst = 0;
        for (size_t n = 0; n < c.N; ++n)
            for (size_t co = 0; co < c.Co; ++co)
                for (size_t i = 0; i < Ho; ++i)
                    for (size_t j = 0; j < Wo; ++j) {
                        double acc = bf[co];
                        for (size_t ci = 0; ci < c.C; ++ci)
                            for (size_t a = 0; a < c.KH; ++a)
                                for (size_t bb = 0; bb < c.KW; ++bb) {
                                    const long hi = long(i * c.sh + a * c.dh) - c.ph, wi = long(j * c.sw + bb * c.dw) - c.pw;
                                    if (hi >= 0 && hi < long(c.H) && wi >= 0 && wi < long(c.W))
                                        acc += double(wf[((co * c.C + ci) * c.KH + a) * c.KW + bb]) * xf[((n * c.C + ci) * c.H + hi) * c.W + wi];
                                }
                        if (c.relu) acc = std::max(acc, 0.0);
                        worst = std::max(worst, std::fabs(acc - got[((n * c.Co + co) * Ho + i) * Wo + j]));
                    }
        EXPECT_LT(worst, c.tol);
    }
}

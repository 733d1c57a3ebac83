// Host-only cases: value types, views, dtype casts, errors, graph signatures.
// Mirrors tests/test_bfloat16.cpp, test_graph_compiler.cpp (signature part) and the
// error cases of tests/test_flash_attention.cpp / test_nn_attention.cpp / test_nn_layers.cpp.
#include <cstring>
#include <map>
#include <set>

#include "test_framework.hpp"

using namespace axiom;

TEST(BFloat16, RoundToNearestEvenAndNaN) { // tests/test_bfloat16.cpp:14-57
    EXPECT_EQ(bfloat16_t(1.0f).bits, 0x3F80);
    EXPECT_EQ(bfloat16_t(-2.0f).bits, 0xC000);
    EXPECT_EQ(bfloat16_t(0.0f).bits, 0x0000);
    EXPECT_NEAR(float(bfloat16_t(3.14159f)), 3.14159f, 0.02f);
    uint32_t tie_even = 0x3F808000u, tie_odd = 0x3F818000u, above = 0x3F808001u; // halfway cases
    float f;
    std::memcpy(&f, &tie_even, 4);
    EXPECT_EQ(bfloat16_t(f).bits, 0x3F80);
    std::memcpy(&f, &tie_odd, 4);
    EXPECT_EQ(bfloat16_t(f).bits, 0x3F82);
    std::memcpy(&f, &above, 4);
    EXPECT_EQ(bfloat16_t(f).bits, 0x3F81);
    EXPECT_EQ(bfloat16_t(std::nanf("")).bits, 0x7FC0);
    EXPECT_TRUE(std::isinf(float(bfloat16_t(INFINITY))));
    EXPECT_EQ(sizeof(bfloat16_t), 2u);
}

TEST(Float16, AllPatternsRoundTrip) {
    int bad = 0;
    for (uint32_t h = 0; h < 65536; ++h) {
        float16_t x;
        x.bits = static_cast<uint16_t>(h);
        const float f = float(x);
        if (std::isnan(f)) continue;
        if (float16_t(f).bits != h) ++bad;
    }
    EXPECT_EQ(bad, 0);
    EXPECT_EQ(float16_t(1.0f).bits, 0x3C00);
    EXPECT_EQ(float16_t(65504.0f).bits, 0x7BFF);
    EXPECT_EQ(float16_t(65520.0f).bits, 0x7C00);       // rounds to infinity
    EXPECT_EQ(float16_t(5.9604645e-8f).bits, 0x0001);  // smallest subnormal
    EXPECT_EQ(float16_t(2.9802322e-8f).bits, 0x0000);  // tie to even (zero)
    EXPECT_EQ(float16_t(1.0009765625f).bits, 0x3C01);
    EXPECT_EQ(float16_t(1.00048828125f).bits, 0x3C00); // tie to even
}

TEST(Tensor, ShapeStridesAndViews) {
    auto t = Tensor::zeros({2, 3, 4});
    EXPECT_EQ(t.ndim(), 3u);
    EXPECT_EQ(t.size(), 24u);
    EXPECT_EQ(t.strides()[0], 48); // bytes
    EXPECT_EQ(t.strides()[2], 4);
    EXPECT_TRUE(t.is_contiguous());
    for (size_t i = 0; i < 24; ++i) t.typed_data<float>()[i] = float(i);
    auto tr = t.transpose({0, 2, 1});
    EXPECT_EQ(tr.shape()[1], 4u);
    EXPECT_FALSE(tr.is_contiguous());
    EXPECT_EQ(tr.storage().get(), t.storage().get()); // a view
    EXPECT_NEAR(tr.item<float>({1, 3, 2}), t.item<float>({1, 2, 3}), 0);
    auto c = tr.ascontiguousarray();
    EXPECT_TRUE(c.is_contiguous());
    EXPECT_NEAR(c.item<float>({1, 3, 2}), 12 + 8 + 3, 0);
    auto r = t.reshape({6, 4});
    EXPECT_EQ(r.storage().get(), t.storage().get());
    EXPECT_NEAR(r.item<float>({5, 3}), 23, 0);
    EXPECT_THROW(t.reshape({5, 5}), ShapeError);
    EXPECT_EQ(t.unsqueeze(1).shape()[1], 1u);
    EXPECT_EQ(t.unsqueeze(1).squeeze(1).ndim(), 3u);
    EXPECT_THROW(t.transpose({0, 1}), ShapeError);
    EXPECT_THROW(t.item<float>({2, 0, 0}), IndexError);
}

TEST(Tensor, FactoriesSeedAndCasts) {
    Tensor::manual_seed(42);
    auto a = Tensor::randn({64, 64});
    Tensor::manual_seed(42);
    auto b = Tensor::randn({64, 64});
    EXPECT_TRUE(a.allclose(b, 0, 0));
    double s = 0, q = 0;
    for (size_t i = 0; i < a.size(); ++i) {
        s += a.typed_data<float>()[i];
        q += double(a.typed_data<float>()[i]) * a.typed_data<float>()[i];
    }
    EXPECT_NEAR(s / a.size(), 0.0, 0.06);
    EXPECT_NEAR(q / a.size(), 1.0, 0.08);
    auto u = Tensor::uniform(0.5, 1.5, {1000});
    for (size_t i = 0; i < u.size(); ++i) EXPECT_TRUE(u.typed_data<float>()[i] >= 0.5f && u.typed_data<float>()[i] < 1.5f);
    auto h = a.astype(DType::BFloat16);
    EXPECT_EQ(h.dtype(), DType::BFloat16);
    EXPECT_EQ(h.typed_data<bfloat16_t>()[5].bits, bfloat16_t(a.typed_data<float>()[5]).bits);
    EXPECT_TRUE(h.astype(DType::Float32).allclose(a, 1e-2, 1e-2));
    auto f = Tensor::full<float>({3, 3}, 2.5f);
    EXPECT_NEAR(f.item<float>({2, 2}), 2.5f, 0);
    EXPECT_NEAR(Tensor::eye(3).item<float>({1, 1}), 1.0f, 0);
    EXPECT_NEAR(Tensor::eye(3).item<float>({1, 2}), 0.0f, 0);
    EXPECT_THROW(Tensor::ones({2, 2}).item<float>(), ValueError);
    EXPECT_THROW(a.typed_data<double>(), TypeError);
}

TEST(Tensor, AllcloseFormula) { // |a-b| <= atol + rtol*|b|
    auto a = Tensor::full<float>({4}, 1.0f), b = Tensor::full<float>({4}, 1.001f);
    EXPECT_TRUE(a.allclose(b, 1e-2, 0));
    EXPECT_FALSE(a.allclose(b, 1e-5, 1e-8));
    EXPECT_TRUE(a.allclose(b, 0, 2e-3));
    EXPECT_FALSE(a.allclose(Tensor::full<float>({5}, 1.0f)));
}

TEST(Errors, OpsOnCpuTensorsAreRefused) {
    auto a = Tensor::ones({4, 4});
    EXPECT_THROW(ops::add(a, a), RuntimeError);  // no CPU compute path in this library
    EXPECT_THROW(ops::softmax(a), RuntimeError);
    auto q = Tensor::ones({1, 2, 8, 16});
    EXPECT_THROW(ops::scaled_dot_product_attention(q, q, q, Tensor()), RuntimeError);
}

TEST(Errors, AttentionShapeValidation) { // tests/test_flash_attention.cpp:357-371
    auto q3 = Tensor::ones({2, 8, 16});
    EXPECT_THROW(ops::scaled_dot_product_attention(q3, q3, q3, Tensor()), ShapeError);
    auto q = Tensor::ones({2, 2, 8, 16}), k = Tensor::ones({3, 2, 8, 16});
    EXPECT_THROW(ops::scaled_dot_product_attention(q, k, k, Tensor()), ShapeError);
    auto kd = Tensor::ones({2, 2, 8, 32});
    EXPECT_THROW(ops::scaled_dot_product_attention(q, kd, kd, Tensor()), ShapeError);
}

TEST(Errors, NoDeviceIsAnErrorNotAFallback) {
    if (system::is_gpu_available()) throw axtest::Skip("a GPU is present");
    EXPECT_THROW(make_storage(1024, Device::GPU), DeviceError); // src/tensor/storage.cpp:41-45
    EXPECT_THROW(Tensor::ones({4}).gpu(), DeviceError);
    EXPECT_FALSE(system::should_run_gpu_tests());
}

TEST(Module, ParameterOrderAndStateDict) { // tests/test_nn_attention.cpp:12-26
    nn::MultiHeadAttention mha(4);
    auto named = mha.named_parameters();
    ASSERT_EQ(named.size(), 8u);
    const char *want[] = {"q_proj.weight", "q_proj.bias", "k_proj.weight", "k_proj.bias", "v_proj.weight", "v_proj.bias", "out_proj.weight", "out_proj.bias"};
    for (size_t i = 0; i < 8; ++i) EXPECT_EQ(named[i].first, std::string(want[i]));
    nn::MultiHeadAttention nobias(2, false);
    EXPECT_EQ(nobias.named_parameters().size(), 4u);
    nn::Linear lin;
    EXPECT_THROW(lin.forward(Tensor::ones({1, 3})), RuntimeError); // forward before load (tests/test_nn_layers.cpp:83-104)
    std::map<std::string, Tensor> sd{{"weight", Tensor::ones({2, 3})}};
    EXPECT_THROW(lin.load_state_dict(sd), ValueError); // bias missing, strict
    EXPECT_NO_THROW(lin.load_state_dict(sd, "", false));
    EXPECT_EQ(lin.state_dict().count("weight"), 1u);
    nn::MultiHeadAttention m1(1);
    EXPECT_THROW(m1.forward(Tensor::ones({3, 2}), Tensor::ones({3, 2}), Tensor::ones({3, 2})), ShapeError); // tests/test_nn_attention.cpp:111-129
}

// ---- graph signatures on hand-built nodes (no device needed): tests/test_graph_compiler.cpp:20-76
namespace {
std::shared_ptr<graph::GraphNode> constant(const Shape &s, DType dt = DType::Float32) {
    auto n = std::make_shared<graph::GraphNode>();
    n->is_constant = true;
    n->output_shape = s;
    n->output_dtype = dt;
    n->target_device = Device::GPU;
    n->constant_strides = ShapeUtils::contiguous_strides(s, dtype_size(dt));
    return n;
}
std::shared_ptr<graph::GraphNode> node(ops::OpType op, std::vector<std::shared_ptr<graph::GraphNode>> in, const Shape &s, graph::OpParams p = graph::NoParams{}) {
    auto n = std::make_shared<graph::GraphNode>();
    n->op_type = op;
    n->inputs = std::move(in);
    n->output_shape = s;
    n->output_dtype = DType::Float32;
    n->target_device = Device::GPU;
    n->params = std::move(p);
    return n;
}
} // namespace

TEST(GraphSignature, DeterministicStructuralAndDataIndependent) {
    using ops::OpType;
    auto build = [&](OpType inner, const Shape &s) {
        auto a = constant(s), b = constant(s);
        return node(OpType::ReLU, {node(inner, {a, b}, s)}, s);
    };
    const Shape s{4, 8};
    const auto h1 = graph::compute_signature(build(OpType::Add, s).get());
    const auto h2 = graph::compute_signature(build(OpType::Add, s).get());
    EXPECT_TRUE(h1 == h2); // same structure, different node objects (and data)
    EXPECT_TRUE(h1 != graph::compute_signature(build(OpType::Multiply, s).get()));
    EXPECT_TRUE(h1 != graph::compute_signature(build(OpType::Add, Shape{8, 4}).get()));
    // parameters are part of the signature
    auto x = constant(s);
    auto r0 = node(OpType::Sum, {x}, {4}, graph::ReductionParams{{1}, false});
    auto r1 = node(OpType::Sum, {x}, {8}, graph::ReductionParams{{0}, false});
    EXPECT_TRUE(graph::compute_signature(r0.get()) != graph::compute_signature(r1.get()));
    // constant strides are part of it
    auto t = constant(s);
    t->constant_strides = {4, 16};
    auto v0 = node(OpType::ReLU, {constant(s)}, s), v1 = node(OpType::ReLU, {t}, s);
    EXPECT_TRUE(graph::compute_signature(v0.get()) != graph::compute_signature(v1.get()));
    // x+x (one shared input) differs from x+y
    auto sh = constant(s);
    auto same = node(OpType::Add, {sh, sh}, s), diff = node(OpType::Add, {constant(s), constant(s)}, s);
    EXPECT_TRUE(graph::compute_signature(same.get()) != graph::compute_signature(diff.get()));
    EXPECT_EQ(graph::topo_sort(same.get()).size(), 2u);
    EXPECT_EQ(graph::topo_sort(diff.get()).size(), 3u);
}

TEST(GraphInference, ShapesAndDtypes) {
    EXPECT_EQ(graph::infer_binary_shape({4, 1, 3}, {5, 1}).size(), 3u);
    EXPECT_EQ(graph::infer_binary_shape({4, 1, 3}, {5, 1})[1], 5u);
    EXPECT_THROW(graph::infer_binary_shape({4, 3}, {5, 2}), ShapeError);
    EXPECT_EQ(graph::infer_reduction_shape({4, 5}, {}, false), Shape({1})); // src/graph/graph_registry.cpp:102-111
    EXPECT_EQ(graph::infer_reduction_shape({4, 5}, {1}, false), Shape({4}));
    EXPECT_EQ(graph::infer_reduction_shape({4, 5}, {-1}, true), Shape({4, 1}));
    EXPECT_EQ(graph::infer_matmul_shape({2, 3, 4}, {5, 4}, false, true), Shape({2, 3, 5}));
    EXPECT_THROW(graph::infer_matmul_shape({3, 4}, {5, 6}, false, false), ShapeError);
    EXPECT_EQ(graph::infer_reduction_dtype(ops::OpType::Mean, DType::BFloat16), DType::Float32);
    EXPECT_EQ(graph::infer_reduction_dtype(ops::OpType::Sum, DType::BFloat16), DType::BFloat16);
    EXPECT_EQ(ops::promote_types(DType::BFloat16, DType::Float32), DType::Float32);
    EXPECT_EQ(ops::promote_types(DType::Float16, DType::BFloat16), DType::BFloat16);
    EXPECT_EQ(ops::promote_types(DType::UInt8, DType::Int8), DType::Int16);
}

TEST(EagerMode, ScopeNestsAndRestores) {
    const bool before = graph::is_eager_mode_enabled();
    {
        graph::EagerModeScope a;
        EXPECT_TRUE(graph::is_eager_mode_enabled());
        {
            graph::EagerModeScope b;
            EXPECT_TRUE(graph::is_eager_mode_enabled());
        }
        EXPECT_TRUE(graph::is_eager_mode_enabled());
    }
    EXPECT_EQ(graph::is_eager_mode_enabled(), before);
}

TEST(Random, Pcg64StreamIsFixed) {
    PCG64 g(42, 54);
    PCG64 h(42, 54);
    std::set<uint64_t> seen;
    for (int i = 0; i < 64; ++i) {
        const uint64_t v = g();
        EXPECT_EQ(v, h());
        seen.insert(v);
    }
    EXPECT_EQ(seen.size(), 64u);
    PCG64 other(43, 54);
    EXPECT_NE(other(), PCG64(42, 54)());
}

// ------------------------------------------------------------- safetensors
// tests/test_io_safetensors.cpp:31-141 of the reference, plus malformed files.
#include <cstdio>
#include <fstream>

namespace {
std::string st_path(const std::string &name) {
    const char *tmp = std::getenv("TMPDIR");
    return std::string(tmp && *tmp ? tmp : "/tmp") + "/axiom_hip_test_" + name + ".safetensors";
}
void write_st(const std::string &path, const std::string &header, const std::vector<uint8_t> &data, int64_t header_len_override = -1) {
    std::ofstream f(path, std::ios::binary);
    const uint64_t n = header_len_override >= 0 ? static_cast<uint64_t>(header_len_override) : header.size();
    f.write(reinterpret_cast<const char *>(&n), 8);
    f.write(header.data(), static_cast<std::streamsize>(header.size()));
    f.write(reinterpret_cast<const char *>(data.data()), static_cast<std::streamsize>(data.size()));
}
template <typename T> std::vector<uint8_t> bytes_of(const std::vector<T> &v) {
    std::vector<uint8_t> b(v.size() * sizeof(T));
    std::memcpy(b.data(), v.data(), b.size());
    return b;
}
} // namespace

TEST(SafeTensors, DetectionAndSingleTensor) { // :31-63
    namespace st = io::safetensors;
    EXPECT_TRUE(st::is_safetensors_file("model.safetensors"));
    EXPECT_TRUE(st::is_safetensors_file("/path/to/weights.safetensors"));
    EXPECT_FALSE(st::is_safetensors_file("model.bin"));
    EXPECT_FALSE(st::is_safetensors_file("model.npy"));
    const std::string path = st_path("single");
    write_st(path, R"({"weight":{"dtype":"F32","shape":[2,3],"data_offsets":[0,24]}})", bytes_of<float>({1, 2, 3, 4, 5, 6}));
    auto tensors = st::load(path);
    ASSERT_EQ(tensors.size(), 1u);
    ASSERT_TRUE(tensors.count("weight") > 0);
    auto &t = tensors["weight"];
    EXPECT_TRUE(t.shape() == Shape({2, 3}));
    EXPECT_EQ(t.dtype(), DType::Float32);
    EXPECT_TRUE(t.device() == Device::CPU);
    EXPECT_NEAR(t.item<float>({0, 0}), 1.0f, 0);
    EXPECT_NEAR(t.item<float>({1, 2}), 6.0f, 0);
    std::remove(path.c_str());
}

TEST(SafeTensors, SeveralTensorsListingMetadataAndDtypes) { // :65-141
    namespace st = io::safetensors;
    const std::string path = st_path("multi");
    std::vector<uint8_t> data = bytes_of<float>({1, 2, 3, 4});
    const auto i64 = bytes_of<int64_t>({10, 20, 30});
    data.insert(data.end(), i64.begin(), i64.end());
    const auto bf = bytes_of<uint16_t>({0x3F80, 0x4000}); // bf16 1.0, 2.0
    data.insert(data.end(), bf.begin(), bf.end());
    data.push_back(1); // BOOL
    data.push_back(0);
    write_st(path,
             "{ \"__metadata__\": {\"format\": \"pt\", \"note\": \"a \\\"quoted\\\" value\", \"nested\": {\"k\": [1, 2.5, true, null]}},\n"
             "  \"a\": {\"dtype\": \"F32\", \"shape\": [2, 2], \"data_offsets\": [0, 16]},\n"
             "  \"b\": {\"dtype\":\"I64\",\"shape\":[3],\"data_offsets\":[16,40]},\n"
             "  \"c.weight\": {\"shape\":[2],\"data_offsets\":[40,44],\"dtype\":\"BF16\"},\n"
             "  \"flag\": {\"dtype\":\"BOOL\",\"shape\":[2],\"data_offsets\":[44,46]},\n"
             "  \"empty\": {\"dtype\":\"F16\",\"shape\":[0,4],\"data_offsets\":[46,46]} }",
             data);
    auto names = st::list_tensors(path);
    ASSERT_EQ(names.size(), 5u); // __metadata__ is not a tensor
    std::set<std::string> ns(names.begin(), names.end());
    EXPECT_TRUE(ns.count("a") && ns.count("b") && ns.count("c.weight") && ns.count("flag") && ns.count("empty"));
    auto all = st::load(path);
    ASSERT_EQ(all.size(), 5u);
    EXPECT_NEAR(all["a"].item<float>({1, 1}), 4.0f, 0);
    EXPECT_EQ(all["b"].dtype(), DType::Int64);
    EXPECT_EQ(all["b"].item<int64_t>({2}), 30);
    EXPECT_EQ(all["c.weight"].dtype(), DType::BFloat16);
    EXPECT_NEAR(all["c.weight"].item<float>({1}), 2.0f, 0);
    EXPECT_EQ(all["flag"].dtype(), DType::Bool);
    EXPECT_EQ(all["flag"].item<int>({0}), 1);
    EXPECT_EQ(all["empty"].size(), 0u);
    auto one = st::load_tensor(path, "b");
    EXPECT_TRUE(one.shape() == Shape({3}));
    EXPECT_EQ(one.item<int64_t>({0}), 10);
    EXPECT_THROW(st::load_tensor(path, "missing"), io::SerializationError);
    std::remove(path.c_str());
}

TEST(SafeTensors, MalformedFilesAreRejected) {
    namespace st = io::safetensors;
    EXPECT_THROW(st::load(st_path("does_not_exist")), io::SerializationError);
    const std::string path = st_path("bad");
    const auto four = bytes_of<float>({1, 2, 3, 4});
    auto expect_format_error = [&](const std::string &header, const std::vector<uint8_t> &data, int64_t len = -1) {
        write_st(path, header, data, len);
        EXPECT_THROW(st::load(path), io::FileFormatError);
    };
    expect_format_error(R"({"w":{"dtype":"F32","shape":[2,2],"data_offsets":[0,16]}})", four, 1 << 30);           // header length beyond the file
    expect_format_error(R"({"w":{"dtype":"F32","shape":[2,2],"data_offsets":[0,32]}})", four);                    // byte range does not match the shape
    expect_format_error(R"({"w":{"dtype":"F32","shape":[4,2],"data_offsets":[0,32]}})", four);                    // range outside the file
    expect_format_error(R"({"w":{"dtype":"Q4","shape":[2,2],"data_offsets":[0,16]}})", four);                     // unknown dtype
    expect_format_error(R"({"w":{"dtype":"F32","shape":[2,2]}})", four);                                          // no offsets
    expect_format_error(R"({"w":{"dtype":"F32","shape":[2,-2],"data_offsets":[0,16]}})", four);                   // negative extent
    expect_format_error(R"({"w":{"dtype":"F32","shape":[2,2],"data_offsets":[16,0]}})", four);                    // reversed range
    expect_format_error(R"({"w":{"dtype":"F32","shape":[2,2],"data_offsets":[0,16]})", four);                     // unterminated object
    expect_format_error(R"({"w":{"dtype":"F32","shape":[4294967296,4294967296],"data_offsets":[0,0]}})", four);   // element count wraps to 0 in 64 bits
    expect_format_error(R"({"w":{"dtype":"F32","shape":[4611686018427387904,4],"data_offsets":[0,0]}})", four);   // byte count wraps to 0
    expect_format_error(R"({"__metadata__":)" + std::string(100000, '[') + std::string(100000, ']') + R"(,"w":{"dtype":"F32","shape":[2,2],"data_offsets":[0,16]}})",
                        four);                                                                                    // nesting that would exhaust the stack
    {
        std::ofstream f(path, std::ios::binary); // shorter than the length field
        f.write("abc", 3);
    }
    EXPECT_THROW(st::load(path), io::FileFormatError);
    std::remove(path.c_str());
}

// A file written by the safetensors Python package itself (tests/test_host_layer.py names it in
// AXIOM_TEST_SAFETENSORS): "ramp_<dtype>" tensors hold 0, 1, 2, ... in shape (3, 5); skipped when unset.
TEST(SafeTensors, ReadsFilesWrittenByTheReferenceImplementation) {
    const char *path = std::getenv("AXIOM_TEST_SAFETENSORS");
    if (!path || !*path) throw axtest::Skip("AXIOM_TEST_SAFETENSORS not set");
    auto all = io::safetensors::load(path);
    const std::pair<const char *, DType> want[] = {{"ramp_f32", DType::Float32}, {"ramp_f16", DType::Float16}, {"ramp_bf16", DType::BFloat16},
                                                   {"ramp_i64", DType::Int64},   {"ramp_i32", DType::Int32},   {"ramp_u8", DType::UInt8}};
    for (const auto &[name, dt] : want) {
        ASSERT_TRUE(all.count(name) > 0);
        const Tensor &t = all.at(name);
        EXPECT_EQ(t.dtype(), dt);
        EXPECT_TRUE(t.shape() == Shape({3, 5}));
        for (size_t i = 0; i < 3; ++i)
            for (size_t j = 0; j < 5; ++j) EXPECT_NEAR(t.item<double>({i, j}), double(i * 5 + j), 0);
    }
    ASSERT_TRUE(all.count("mask") > 0);
    EXPECT_EQ(all.at("mask").dtype(), DType::Bool);
    EXPECT_EQ(all.at("mask").item<int>({1}), 1);
    EXPECT_EQ(all.at("mask").item<int>({2}), 0);
    EXPECT_EQ(all.at("scalar").ndim(), 0u);
    EXPECT_NEAR(all.at("scalar").item<float>({}), 2.5f, 0);
}

// Differential test of the lazy-graph planner: seeded random expression DAGs over the op set
// of the fused path are built twice, as lazy GPU tensors and as float64 arrays evaluated by the
// plain loops below, and every root is compared.  The generator mixes what decides the plan:
// broadcast kinds (scalar, row vector, column vector, full), row ops with pre- and post-chains,
// reductions, matmul with epilogue candidates, transposes, reshapes, slices, nodes consumed
// several times and nodes whose handle is kept alive or dropped.
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <functional>

#include "oracle_util.hpp"
#include "test_framework.hpp"

using namespace axiom;

namespace {

struct Ref { // contiguous row-major float64 value
    Shape shape;
    std::vector<double> v;
    size_t size() const { return v.size(); }
};

struct Rng {
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed * 0x9E3779B97F4A7C15ull + 0x1234567ull) {}
    uint64_t next() {
        s ^= s << 13;
        s ^= s >> 7;
        s ^= s << 17;
        return s;
    }
    size_t below(size_t n) { return static_cast<size_t>(next() % n); }
    bool coin() { return next() & 1; }
};

size_t numel(const Shape &s) { return ShapeUtils::size(s); }

// value of `r` at the multi-index of flat position i of a tensor of shape `out` (numpy broadcasting)
double bcast_at(const Ref &r, const Shape &out, size_t i) {
    size_t off = 0, stride = 1;
    const size_t lead = out.size() - r.shape.size();
    for (size_t d = out.size(); d-- > 0;) {
        const size_t c = i % out[d];
        i /= out[d];
        if (d >= lead) {
            const size_t e = r.shape[d - lead];
            if (e != 1) off += c * stride;
            stride *= e;
        }
    }
    return r.v[off];
}

Ref unary(const Ref &a, const std::function<double(double)> &f) {
    Ref o{a.shape, a.v};
    for (double &x : o.v) x = f(x);
    return o;
}
Ref binary(const Ref &a, const Ref &b, const std::function<double(double, double)> &f) {
    Ref o;
    o.shape = ShapeUtils::broadcast(a.shape, b.shape);
    o.v.resize(numel(o.shape));
    for (size_t i = 0; i < o.v.size(); ++i) o.v[i] = f(bcast_at(a, o.shape, i), bcast_at(b, o.shape, i));
    return o;
}
// f over each row (last axis) of a
Ref rowwise(const Ref &a, const std::function<void(const double *, double *, size_t)> &f) {
    Ref o{a.shape, std::vector<double>(a.v.size())};
    const size_t cols = a.shape.back();
    for (size_t r = 0; r < a.v.size() / cols; ++r) f(&a.v[r * cols], &o.v[r * cols], cols);
    return o;
}
Ref reduce_last(const Ref &a, int kind, bool keep) { // 0 sum 1 mean 2 max 3 min
    const size_t cols = a.shape.back(), rows = a.v.size() / cols;
    Ref o;
    o.shape = Shape(a.shape.begin(), a.shape.end() - 1);
    if (keep) o.shape.push_back(1);
    if (o.shape.empty()) o.shape.push_back(1);
    o.v.resize(rows);
    for (size_t r = 0; r < rows; ++r) {
        const double *p = &a.v[r * cols];
        double acc = kind <= 1 ? 0.0 : p[0];
        for (size_t c = 0; c < cols; ++c) acc = kind <= 1 ? acc + p[c] : kind == 2 ? std::max(acc, p[c]) : std::min(acc, p[c]);
        o.v[r] = kind == 1 ? acc / double(cols) : acc;
    }
    return o;
}
Ref reduce_all(const Ref &a, int kind) {
    Ref flat{Shape{a.v.size()}, a.v};
    return reduce_last(flat, kind, false);
}
Ref transpose2(const Ref &a) { // swaps the last two axes
    Ref o;
    o.shape = a.shape;
    const size_t nd = a.shape.size(), R = a.shape[nd - 2], C = a.shape[nd - 1];
    std::swap(o.shape[nd - 2], o.shape[nd - 1]);
    o.v.resize(a.v.size());
    for (size_t b = 0; b < a.v.size() / (R * C); ++b)
        for (size_t r = 0; r < R; ++r)
            for (size_t c = 0; c < C; ++c) o.v[(b * C + c) * R + r] = a.v[(b * R + r) * C + c];
    return o;
}
Ref matmul_nt(const Ref &a, const Ref &w) { // a [.., M, K] times w [N, K] transposed
    const size_t K = a.shape.back(), N = w.shape[0], rows = a.v.size() / K;
    Ref o;
    o.shape = a.shape;
    o.shape.back() = N;
    o.v.resize(rows * N);
    for (size_t r = 0; r < rows; ++r)
        for (size_t n = 0; n < N; ++n) {
            double acc = 0;
            for (size_t k = 0; k < K; ++k) acc += a.v[r * K + k] * w.v[n * K + k];
            o.v[r * N + n] = acc;
        }
    return o;
}
Ref slice_cols(const Ref &a, size_t begin, size_t end, size_t step) {
    const size_t cols = a.shape.back(), rows = a.v.size() / cols, n = (end - begin + step - 1) / step;
    Ref o;
    o.shape = a.shape;
    o.shape.back() = n;
    o.v.resize(rows * n);
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < n; ++c) o.v[r * n + c] = a.v[r * cols + begin + c * step];
    return o;
}

struct Val {
    Tensor t; // lazy (or materialised) GPU tensor
    Ref r;
};

Val leaf(const Shape &shape, uint64_t seed, float scale = 1.0f, float shift = 0.0f) {
    Tensor h = axtest::randn(shape, seed, DType::Float32, scale);
    Ref r{shape, std::vector<double>(h.size())};
    for (size_t i = 0; i < h.size(); ++i) {
        h.typed_data<float>()[i] += shift;
        r.v[i] = h.typed_data<float>()[i];
    }
    return {h.gpu(), r};
}

double gelu_ref(double x) { return 0.5 * x * (1.0 + std::erf(x / std::sqrt(2.0))); }

// One random graph; returns the number of roots compared.
int run_graph(uint64_t seed, double tol) {
    Rng g(seed);
    const size_t R = 3 + g.below(40), C = 8 * (1 + g.below(9)) + (g.coin() ? 0 : g.below(7)); // aligned and ragged row lengths
    const bool batched = g.below(4) == 0;
    const Shape full = batched ? Shape{2, R, C} : Shape{R, C};
    std::vector<Val> pool;
    pool.push_back(leaf(full, seed * 11 + 1));
    pool.push_back(leaf(full, seed * 11 + 2));
    const Val rowvec = leaf({C}, seed * 11 + 3), rowvec_pos = leaf({C}, seed * 11 + 4, 0.2f, 1.0f);
    Shape col_shape = full;
    col_shape.back() = 1;
    const Val colvec = leaf(col_shape, seed * 11 + 5);
    const Val scalar = leaf({1}, seed * 11 + 6, 0.5f, 1.5f);
    const Val weight = leaf({C, C}, seed * 11 + 7, 1.0f / std::sqrt(float(C))); // square, so matmul keeps the shape

    auto full_shaped = [&]() -> const Val & { // a pool entry of the full shape
        for (int tries = 0; tries < 16; ++tries) {
            const Val &v = pool[g.below(pool.size())];
            if (v.r.shape == full) return v;
        }
        return pool[0];
    };
    const int steps = 4 + static_cast<int>(g.below(10));
    for (int s = 0; s < steps; ++s) {
        const Val &x = full_shaped();
        Val out;
        switch (g.below(12)) {
        case 0: { // unary
            static const struct { ops::OpType op; double (*f)(double); } table[] = {
                {ops::OpType::ReLU, [](double v) { return v > 0 ? v : 0.0; }}, {ops::OpType::Tanh, [](double v) { return std::tanh(v); }},
                {ops::OpType::Sigmoid, [](double v) { return 1.0 / (1.0 + std::exp(-v)); }}, {ops::OpType::Abs, [](double v) { return std::fabs(v); }},
                {ops::OpType::Negate, [](double v) { return -v; }}, {ops::OpType::GELU, gelu_ref},
                {ops::OpType::SiLU, [](double v) { return v / (1.0 + std::exp(-v)); }}};
            const auto &e = table[g.below(7)];
            out = {graph::GraphRegistry::create_lazy_unary(e.op, x.t), unary(x.r, e.f)};
            break;
        }
        case 1: case 2: case 3: { // binary against another full tensor or a broadcast operand
            const Val *ys[] = {&full_shaped(), &rowvec, &colvec, &scalar};
            const Val &y = *ys[g.below(4)];
            const bool swap = g.coin();
            const Val &l = swap ? y : x, &r = swap ? x : y;
            switch (g.below(5)) {
            case 0: out = {ops::add(l.t, r.t), binary(l.r, r.r, [](double a, double b) { return a + b; })}; break;
            case 1: out = {ops::subtract(l.t, r.t), binary(l.r, r.r, [](double a, double b) { return a - b; })}; break;
            case 2: out = {ops::multiply(l.t, r.t), binary(l.r, r.r, [](double a, double b) { return a * b; })}; break;
            case 3: out = {ops::maximum(l.t, r.t), binary(l.r, r.r, [](double a, double b) { return std::max(a, b); })}; break;
            default: out = {ops::minimum(l.t, r.t), binary(l.r, r.r, [](double a, double b) { return std::min(a, b); })}; break;
            }
            break;
        }
        case 4: { // division by something bounded away from zero
            const Val &d = full_shaped();
            const Val den{ops::add(ops::abs(d.t), scalar.t), binary(unary(d.r, [](double v) { return std::fabs(v); }), scalar.r, [](double a, double b) { return a + b; })};
            out = {ops::divide(x.t, den.t), binary(x.r, den.r, [](double a, double b) { return a / b; })};
            break;
        }
        case 5: { // softmax / log_softmax of a bounded input
            const bool lg = g.coin();
            Val in{ops::tanh(x.t), unary(x.r, [](double v) { return std::tanh(v); })};
            out = {lg ? ops::log_softmax(in.t, -1) : ops::softmax(in.t, -1), rowwise(in.r, [lg](const double *p, double *o, size_t n) {
                       double m = p[0], sum = 0;
                       for (size_t i = 0; i < n; ++i) m = std::max(m, p[i]);
                       for (size_t i = 0; i < n; ++i) sum += std::exp(p[i] - m);
                       for (size_t i = 0; i < n; ++i) o[i] = lg ? p[i] - m - std::log(sum) : std::exp(p[i] - m) / sum;
                   })};
            break;
        }
        case 6: { // layer norm / rms norm with weight (and bias)
            const bool rms = g.coin();
            const Ref &w = rowvec_pos.r, &b = rowvec.r;
            out = {rms ? ops::rms_norm(x.t, rowvec_pos.t, -1, 1e-5f) : ops::layer_norm(x.t, rowvec_pos.t, rowvec.t, -1, 1e-5f),
                   rowwise(x.r, [&, rms](const double *p, double *o, size_t n) {
                       double mean = 0, ss = 0;
                       for (size_t i = 0; i < n; ++i) mean += p[i] / double(n);
                       if (rms) mean = 0;
                       for (size_t i = 0; i < n; ++i) ss += (p[i] - mean) * (p[i] - mean) / double(n);
                       for (size_t i = 0; i < n; ++i) o[i] = (p[i] - mean) / std::sqrt(ss + 1e-5) * w.v[i] + (rms ? 0.0 : b.v[i]);
                   })};
            break;
        }
        case 7: { // reduction over the last axis, broadcast back against the full shape
            const int kind = static_cast<int>(g.below(4));
            Tensor red = kind == 0 ? ops::sum(x.t, {-1}, true) : kind == 1 ? ops::mean(x.t, {-1}, true) : kind == 2 ? ops::max(x.t, {-1}, true) : ops::min(x.t, {-1}, true);
            const Ref rr = reduce_last(x.r, kind, true);
            out = {ops::subtract(x.t, red), binary(x.r, rr, [](double a, double b) { return a - b; })};
            break;
        }
        case 8: { // matmul with the square weight, maybe bias, residual and activation behind it (epilogue candidates)
            Tensor t = ops::matmul(x.t, weight.t, false, true);
            Ref r = matmul_nt(x.r, weight.r);
            const auto plus = [](double a, double b) { return a + b; };
            if (g.coin()) {
                t = ops::add(t, rowvec.t);
                r = binary(r, rowvec.r, plus);
            }
            if (g.coin()) {
                const Val &res = full_shaped();
                t = ops::add(t, res.t);
                r = binary(r, res.r, plus);
            }
            if (g.coin()) {
                t = ops::gelu(t);
                r = unary(r, gelu_ref);
            }
            out = {t, r};
            break;
        }
        case 9: { // transpose of the last two axes, an elementwise op there, and back
            const std::vector<int> axes = batched ? std::vector<int>{0, 2, 1} : std::vector<int>{1, 0};
            Tensor t = x.t.transpose(axes);
            Ref tr = transpose2(x.r);
            t = ops::multiply(ops::tanh(t), scalar.t);
            tr = binary(unary(tr, [](double v) { return std::tanh(v); }), scalar.r, [](double a, double b) { return a * b; });
            out = {t.transpose(axes), transpose2(tr)};
            break;
        }
        case 10: { // reshape round trip through a flat view with an op in between
            Tensor t = ops::relu(x.t.reshape(Shape{numel(full)}));
            out = {t.reshape(full), unary(x.r, [](double v) { return v > 0 ? v : 0.0; })};
            break;
        }
        default: { // column slice (strided), used as a root of its own
            const size_t b0 = g.below(C / 2), step = 1 + g.below(2);
            std::vector<Slice> args(full.size());
            args.back() = Slice(static_cast<int64_t>(b0), static_cast<int64_t>(C), static_cast<int64_t>(step));
            Val sl{ops::abs(x.t).slice(args), slice_cols(unary(x.r, [](double v) { return std::fabs(v); }), b0, C, step)};
            pool.push_back(sl); // not of the full shape: only ever a root
            continue;
        }
        }
        pool.push_back(out);
        if (pool.size() > 6 && g.below(3) == 0) pool.erase(pool.begin() + 2 + static_cast<long>(g.below(pool.size() - 3))); // drop a handle
    }
    // roots: the last value, a full reduction of a random one, and one more random survivor
    std::vector<Val> roots{pool.back()};
    {
        const Val &x = pool[g.below(pool.size())];
        const int kind = static_cast<int>(g.below(4));
        roots.push_back({kind == 0 ? ops::sum(x.t) : kind == 1 ? ops::mean(x.t) : kind == 2 ? ops::max(x.t) : ops::min(x.t), reduce_all(x.r, kind)});
        roots.push_back(pool[g.below(pool.size())]);
    }
    int compared = 0;
    for (const Val &root : roots) {
        Tensor h = root.t.cpu().astype(DType::Float32).ascontiguousarray();
        if (!(h.shape() == root.r.shape)) {
            axtest::report(__FILE__, __LINE__, "seed " + std::to_string(seed) + ": shape " + ShapeUtils::to_string(h.shape()) + " vs " + ShapeUtils::to_string(root.r.shape), false);
            continue;
        }
        double worst = 0, scale = 1;
        for (double v : root.r.v) scale = std::max(scale, std::fabs(v));
        for (size_t i = 0; i < h.size(); ++i) {
            const double d = std::fabs(double(h.typed_data<float>()[i]) - root.r.v[i]);
            if (!(d <= worst)) worst = d;
        }
        if (std::getenv("AXIOM_TEST_SEED")) {
            std::printf("    seed %llu root: max |err| %g (scale %g), kernels:", static_cast<unsigned long long>(seed), worst, scale);
            for (const std::string &k : graph::last_gpu_plan_kernels()) std::printf(" %s", k.c_str());
            std::printf("\n");
        }
        if (!(worst <= tol * scale))
            axtest::report(__FILE__, __LINE__, "seed " + std::to_string(seed) + ": max |err| " + std::to_string(worst) + " (scale " + std::to_string(scale) + ")", false);
        ++compared;
    }
    return compared;
}

} // namespace

GPU_TEST(RandomGraphs, LazyPlansMatchFloat64Evaluation) {
    int compared = 0;
    if (const char *one = std::getenv("AXIOM_TEST_SEED")) { // a single graph, with the kernels of each root printed
        run_graph(std::strtoull(one, nullptr, 10), 2e-4);
        return;
    }
    for (uint64_t seed = 1; seed <= 120; ++seed) compared += run_graph(seed, 2e-4);
    std::printf("    %d roots of 120 random graphs compared\n", compared);
    EXPECT_EQ(compared, 360);
}

GPU_TEST(RandomGraphs, SameGraphsInEagerMode) { // every op its own graph: the plan per node kind, without fusion
    graph::EagerModeScope eager;
    int compared = 0;
    for (uint64_t seed = 1000; seed < 1030; ++seed) compared += run_graph(seed, 2e-4);
    EXPECT_EQ(compared, 90);
}

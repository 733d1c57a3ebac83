// Test-side bridge to the CPU oracle (oracle/axiom_oracle.h): expected values for the
// GPU cases come from the restatement of Axiom's CPU algorithms, computed here on the
// same host buffers that were uploaded.  Test infrastructure only.
#pragma once

#include <vector>

#include "axiom/axiom.hpp"
#include "axiom_oracle.h"

namespace axtest {

inline int oracle_dtype(axiom::DType d) {
    return d == axiom::DType::Float32 ? AXO_F32 : d == axiom::DType::Float16 ? AXO_F16 : AXO_BF16;
}

// deterministic N(0,1) host tensor from the oracle's generator, rounded to `dt`
inline axiom::Tensor randn(const axiom::Shape &shape, uint64_t seed, axiom::DType dt = axiom::DType::Float32, float scale = 1.0f) {
    axo_pcg64 g;
    axo_pcg64_seed(&g, seed, 0xda3e39cb94b95bdbULL);
    axiom::Tensor t(shape, axiom::DType::Float32);
    axo_fill_normal(&g, t.typed_data<float>(), t.size(), 0.0f, scale);
    return dt == axiom::DType::Float32 ? t : t.astype(dt);
}
inline axiom::Tensor uniform(const axiom::Shape &shape, uint64_t seed, float lo, float hi, axiom::DType dt = axiom::DType::Float32) {
    axo_pcg64 g;
    axo_pcg64_seed(&g, seed, 0xda3e39cb94b95bdbULL);
    axiom::Tensor t(shape, axiom::DType::Float32);
    axo_fill_uniform(&g, t.typed_data<float>(), t.size(), lo, hi);
    return dt == axiom::DType::Float32 ? t : t.astype(dt);
}

// CPU flash attention of the oracle on host tensors (any of the three dtypes); mask Bool or empty
inline axiom::Tensor oracle_sdpa(const axiom::Tensor &q, const axiom::Tensor &k, const axiom::Tensor &v, const axiom::Tensor &mask, float scale, bool causal) {
    const auto &s = q.shape();
    axiom::Tensor o(s, q.dtype());
    const uint8_t *m = mask.empty() ? nullptr : static_cast<const uint8_t *>(mask.data());
    const int nd = mask.empty() ? 0 : static_cast<int>(mask.ndim());
    axo_sdpa(oracle_dtype(q.dtype()), q.data(), k.data(), v.data(), o.data(), int(s[0]), int(s[1]), int(s[2]), int(k.shape()[2]), int(s[3]), scale, causal, m,
             nd, nd == 4 ? int(mask.shape()[0]) : 1, nd == 4 ? int(mask.shape()[1]) : 1, 0, int(s[0] * s[1]));
    return o;
}

inline double max_abs_diff(const axiom::Tensor &a, const axiom::Tensor &b) {
    axiom::Tensor x = a.cpu().astype(axiom::DType::Float32).ascontiguousarray(), y = b.cpu().astype(axiom::DType::Float32).ascontiguousarray();
    double m = 0;
    for (size_t i = 0; i < x.size(); ++i) {
        const double d = std::fabs(double(x.typed_data<float>()[i]) - double(y.typed_data<float>()[i]));
        if (!(d <= m)) m = d; // NaN propagates
    }
    return m;
}

} // namespace axtest

// ref_shim.cpp -- TEST INFRASTRUCTURE ONLY.
//
// C entry points over the two pieces of the Axiom reference that build from
// their own sources without third-party code: the native BLAS tier
// (src/backends/cpu/blas/blas_native.cpp, blas_backend.cpp) and the PCG64
// generator (include/axiom/random.hpp).  Compiled only where the reference
// tree is present; the result goes to oracle/_ref/ and is used to validate
// the C restatement in axiom_oracle.c.
#include <cstddef>
#include <cstdint>

#include "axiom/random.hpp"
#include "blas/blas_backend.hpp"

extern "C" {

void axref_sgemm(int transA, int transB, size_t M, size_t N, size_t K, float alpha,
                 const float *A, size_t lda, const float *B, size_t ldb, float beta,
                 float *C, size_t ldc) {
    axiom::backends::cpu::blas::get_blas_backend().sgemm(
        transA != 0, transB != 0, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
}

const char *axref_blas_name() {
    return axiom::backends::cpu::blas::get_blas_backend().name();
}

void axref_pcg64(uint64_t seed, uint64_t stream, uint64_t *out, size_t n) {
    axiom::PCG64 g(seed, stream);
    for (size_t i = 0; i < n; ++i) out[i] = g();
}

void axref_pcg64_default(uint64_t *out, size_t n) {
    axiom::PCG64 g;
    for (size_t i = 0; i < n; ++i) out[i] = g();
}
}

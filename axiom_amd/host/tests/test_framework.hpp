// Minimal test harness in the style of the reference's GoogleTest files
// (TEST / EXPECT_* / ASSERT_* / SKIP_IF_NO_GPU), so the cases read like
// tests/test_flash_attention.cpp, test_fusion_extended.cpp, test_cpu_gpu_parity.cpp.
//   host_tests [--cpu | --gpu] [--list] [substring-filter]
// TEST() cases need no device; GPU_TEST() cases are skipped (and reported as such)
// when no GPU is present and are the only ones run under --gpu.
#pragma once

#include <cmath>
#include <cstdio>
#include <functional>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "axiom/axiom.hpp"

namespace axtest {

struct Case {
    std::string suite, name;
    bool needs_gpu;
    std::function<void()> fn;
};
inline std::vector<Case> &registry() {
    static std::vector<Case> r;
    return r;
}
struct Registrar {
    Registrar(const char *s, const char *n, bool gpu, std::function<void()> f) { registry().push_back({s, n, gpu, std::move(f)}); }
};
struct Failure : std::runtime_error {
    using std::runtime_error::runtime_error;
};
struct Skip : std::runtime_error {
    using std::runtime_error::runtime_error;
};
inline int &soft_failures() {
    static int n = 0;
    return n;
}
inline void report(const char *file, int line, const std::string &msg, bool fatal) {
    std::fprintf(stderr, "  %s:%d: %s\n", file, line, msg.c_str());
    ++soft_failures();
    if (fatal) throw Failure(msg);
}

template <typename T> std::string show(const T &x) {
    std::ostringstream o;
    if constexpr (std::is_same_v<T, axiom::DType>) o << axiom::dtype_name(x);
    else if constexpr (std::is_same_v<T, axiom::Shape>) o << axiom::ShapeUtils::to_string(x);
    else if constexpr (std::is_enum_v<T>) o << static_cast<long long>(x);
    else o << x;
    return o.str();
}

} // namespace axtest

#define TEST(suite, name)                                                                                \
    static void axtest_##suite##_##name();                                                               \
    static axtest::Registrar axtest_reg_##suite##_##name(#suite, #name, false, axtest_##suite##_##name); \
    static void axtest_##suite##_##name()
#define GPU_TEST(suite, name)                                                                           \
    static void axtest_##suite##_##name();                                                              \
    static axtest::Registrar axtest_reg_##suite##_##name(#suite, #name, true, axtest_##suite##_##name); \
    static void axtest_##suite##_##name()

#define AXTEST_CHECK(cond, fatal, text)                                        \
    do {                                                                       \
        if (!(cond)) {                                                         \
            std::ostringstream axtest_os;                                      \
            axtest_os << text;                                                 \
            axtest::report(__FILE__, __LINE__, axtest_os.str(), fatal);        \
        }                                                                      \
    } while (0)
#define EXPECT_TRUE(c) AXTEST_CHECK((c), false, "expected true: " #c)
#define ASSERT_TRUE(c) AXTEST_CHECK((c), true, "expected true: " #c)
#define EXPECT_FALSE(c) AXTEST_CHECK(!(c), false, "expected false: " #c)
#define EXPECT_EQ(a, b) AXTEST_CHECK((a) == (b), false, #a " == " #b " failed: " << axtest::show(a) << " vs " << axtest::show(b))
#define ASSERT_EQ(a, b) AXTEST_CHECK((a) == (b), true, #a " == " #b " failed: " << axtest::show(a) << " vs " << axtest::show(b))
#define EXPECT_NE(a, b) AXTEST_CHECK((a) != (b), false, #a " != " #b " failed")
#define EXPECT_GT(a, b) AXTEST_CHECK((a) > (b), false, #a " > " #b " failed: " << (a) << " vs " << (b))
#define EXPECT_LT(a, b) AXTEST_CHECK((a) < (b), false, #a " < " #b " failed: " << (a) << " vs " << (b))
#define EXPECT_LE(a, b) AXTEST_CHECK((a) <= (b), false, #a " <= " #b " failed: " << (a) << " vs " << (b))
#define EXPECT_NEAR(a, b, tol) AXTEST_CHECK(std::fabs(double(a) - double(b)) <= (tol), false, #a " ~ " #b " failed: " << (a) << " vs " << (b) << " (tol " << (tol) << ")")
#define ASSERT_NEAR(a, b, tol) AXTEST_CHECK(std::fabs(double(a) - double(b)) <= (tol), true, #a " ~ " #b " failed: " << (a) << " vs " << (b) << " (tol " << (tol) << ")")
#define EXPECT_THROW(stmt, Exc)                                                              \
    do {                                                                                     \
        bool axtest_ok = false;                                                              \
        try {                                                                                \
            stmt;                                                                            \
        } catch (const Exc &) {                                                              \
            axtest_ok = true;                                                                \
        } catch (const std::exception &e) {                                                  \
            axtest::report(__FILE__, __LINE__, std::string(#stmt " threw a different exception: ") + e.what(), false); \
            axtest_ok = true;                                                                \
        }                                                                                    \
        if (!axtest_ok) axtest::report(__FILE__, __LINE__, #stmt " did not throw " #Exc, false); \
    } while (0)
#define EXPECT_NO_THROW(stmt)                                                                          \
    do {                                                                                               \
        try {                                                                                          \
            stmt;                                                                                      \
        } catch (const std::exception &e) {                                                            \
            axtest::report(__FILE__, __LINE__, std::string(#stmt " threw: ") + e.what(), false);       \
        }                                                                                              \
    } while (0)
#define SKIP_IF_NO_GPU()                                                                 \
    do {                                                                                 \
        if (!axiom::system::should_run_gpu_tests()) throw axtest::Skip("no GPU");        \
    } while (0)

namespace axtest {
// |a - b| <= atol + rtol * |b|, argument order (rtol, atol) as in the reference's AssertTensorsClose
inline void AssertTensorsClose(const axiom::Tensor &a, const axiom::Tensor &b, double rtol, double atol, const char *file, int line) {
    if (!a.allclose(b, rtol, atol)) report(file, line, "tensors differ beyond rtol=" + std::to_string(rtol) + " atol=" + std::to_string(atol), false);
}
} // namespace axtest
#define ASSERT_TENSORS_CLOSE(a, b, rtol, atol) axtest::AssertTensorsClose((a), (b), (rtol), (atol), __FILE__, __LINE__)

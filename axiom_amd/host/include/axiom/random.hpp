// PCG-XSH-RR generator producing 64 bits from two 32-bit steps, and the
// process-wide generator behind Tensor::randn / rand / uniform
// (include/axiom/random.hpp:12-92).
#pragma once

#include <cstdint>
#include <random>

namespace axiom {

class PCG64 {
  public:
    using result_type = uint64_t;
    explicit PCG64(uint64_t seed = 0x853c49e6748fea9bULL, uint64_t stream = 0xda3e39cb94b95bdbULL) { this->seed(seed, stream); }
    void seed(uint64_t seed, uint64_t stream = 0xda3e39cb94b95bdbULL) {
        state_ = 0;
        inc_ = (stream << 1) | 1u;
        (*this)();
        state_ += seed;
        (*this)();
    }
    result_type operator()() {
        const uint64_t hi = step32();
        const uint64_t lo = step32();
        return (hi << 32) | lo;
    }
    static constexpr result_type min() { return 0; }
    static constexpr result_type max() { return UINT64_MAX; }

  private:
    uint32_t step32() {
        const uint64_t old = state_;
        state_ = old * 6364136223846793005ULL + inc_;
        const uint32_t xs = static_cast<uint32_t>(((old >> 18) ^ old) >> 27);
        const uint32_t rot = static_cast<uint32_t>(old >> 59);
        return (xs >> rot) | (xs << ((32u - rot) & 31u));
    }
    uint64_t state_ = 0, inc_ = 1;
};

class RandomGenerator {
  public:
    static RandomGenerator &instance(); // thread-local
    void seed(uint64_t s) { gen_.seed(s); seed_ = s; }
    uint64_t get_seed() const { return seed_; }
    PCG64 &generator() { return gen_; }
    double random_double() { return static_cast<double>(gen_() >> 11) * (1.0 / 9007199254740992.0); }
    template <typename T> T normal(T mean = T(0), T stddev = T(1)) { return std::normal_distribution<T>(mean, stddev)(gen_); }
    template <typename T> T uniform(T lo = T(0), T hi = T(1)) { return std::uniform_real_distribution<T>(lo, hi)(gen_); }

  private:
    PCG64 gen_;
    uint64_t seed_ = 0;
};

} // namespace axiom

// thrust::random (thrust/random.h): the linear congruential engines (minstd_rand0, minstd_rand
// = default_random_engine) and the uniform_int / uniform_real / normal distributions, callable on
// host and device.  The arithmetic restates the reference's so that seeded streams agree number
// for number with thrust/random/detail/linear_congruential_engine.inl:31-63 (state update and
// the seed rule), linear_congruential_engine_discard.h:34-79 (discard by modular
// exponentiation when the increment is 0), uniform_real_distribution.inl:63-82,
// uniform_int_distribution.inl:67-85 (through a double-precision uniform_real over [a, b + 1))
// and normal_distribution_base.h:83-131 (the portable Box-Muller form with one cached value).
// The subtract-with-carry, shift-register and combining engines are not provided.
#pragma once
#include <cmath>
#include <cstdint>
#include <iostream>
#include <limits>
#include <thrust/functional.h>
#include <thrust/pair.h>

namespace thrust {
namespace random {

template <class UIntType, UIntType a, UIntType c, UIntType m>
class linear_congruential_engine {
 public:
  typedef UIntType result_type;
  static const result_type multiplier = a;
  static const result_type increment = c;
  static const result_type modulus = m;
  static const result_type min = c == 0u ? 1u : 0u;
  static const result_type max = m - 1u;
  static const result_type default_seed = 1u;

  THRUST_CDNA4_HD explicit linear_congruential_engine(result_type s = default_seed) { seed(s); }
  // a state of 0 would stay 0 when the increment is a multiple of the modulus: such a seed becomes 1
  THRUST_CDNA4_HD void seed(result_type s = default_seed) {
    if (reduce(c) == 0 && reduce(s) == 0) x_ = reduce(1u);
    else x_ = reduce(s);
  }
  THRUST_CDNA4_HD result_type operator()() {
    x_ = step(x_);
    return x_;
  }
  THRUST_CDNA4_HD void discard(unsigned long long z) {
    if (c == 0 && sizeof(UIntType) <= 4) {
      // x_z = a^z * x_0 (mod m), by square and multiply
      unsigned long long base = a, power = 1;
      while (z > 0) {
        if (z & 1) power = (power * base) % m;
        z >>= 1;
        base = (base * base) % m;
      }
      x_ = (result_type)((power * x_) % m);
    } else {
      for (; z > 0; --z) x_ = step(x_);
    }
  }
  THRUST_CDNA4_HD friend bool operator==(const linear_congruential_engine& l, const linear_congruential_engine& r) { return l.x_ == r.x_; }
  THRUST_CDNA4_HD friend bool operator!=(const linear_congruential_engine& l, const linear_congruential_engine& r) { return l.x_ != r.x_; }
  template <class Ch, class Tr> friend std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const linear_congruential_engine& e) { return os << e.x_; }
  template <class Ch, class Tr> friend std::basic_istream<Ch, Tr>& operator>>(std::basic_istream<Ch, Tr>& is, linear_congruential_engine& e) { return is >> e.x_; }

 private:
  THRUST_CDNA4_HD static result_type reduce(result_type v) { return m == 0 ? v : (result_type)(v % m); }
  THRUST_CDNA4_HD static result_type step(result_type x) {
    const unsigned long long t = (unsigned long long)a * x + c;  // wide enough for 32-bit engines
    return m == 0 ? (result_type)t : (result_type)(t % m);
  }
  result_type x_;
};
template <class U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::multiplier;
template <class U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::increment;
template <class U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::modulus;
template <class U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::min;
template <class U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::max;
template <class U, U a, U c, U m> const U linear_congruential_engine<U, a, c, m>::default_seed;

typedef linear_congruential_engine<std::uint32_t, 16807, 0, 2147483647> minstd_rand0;
typedef linear_congruential_engine<std::uint32_t, 48271, 0, 2147483647> minstd_rand;
typedef minstd_rand default_random_engine;

template <class RealType = double>
class uniform_real_distribution {
 public:
  typedef RealType result_type;
  typedef thrust::pair<RealType, RealType> param_type;
  THRUST_CDNA4_HD explicit uniform_real_distribution(RealType a = 0.0, RealType b = 1.0) : param_(a, b) {}
  THRUST_CDNA4_HD explicit uniform_real_distribution(const param_type& p) : param_(p) {}
  THRUST_CDNA4_HD void reset() {}
  template <class Urng> THRUST_CDNA4_HD result_type operator()(Urng& urng) { return (*this)(urng, param_); }
  // the engine's value mapped to [0, 1) — one more than its range in the denominator keeps 1 out —
  // then scaled to [a, b)
  template <class Urng> THRUST_CDNA4_HD result_type operator()(Urng& urng, const param_type& p) {
    result_type r = static_cast<result_type>(urng() - Urng::min);
    r /= (result_type(1) + static_cast<result_type>(Urng::max - Urng::min));
    return (r * (p.second - p.first)) + p.first;
  }
  THRUST_CDNA4_HD result_type a() const { return param_.first; }
  THRUST_CDNA4_HD result_type b() const { return param_.second; }
  THRUST_CDNA4_HD param_type param() const { return param_; }
  THRUST_CDNA4_HD void param(const param_type& p) { param_ = p; }
  THRUST_CDNA4_HD result_type(min)() const { return a(); }
  THRUST_CDNA4_HD result_type(max)() const { return b(); }
  THRUST_CDNA4_HD friend bool operator==(const uniform_real_distribution& l, const uniform_real_distribution& r) { return l.param_ == r.param_; }
  THRUST_CDNA4_HD friend bool operator!=(const uniform_real_distribution& l, const uniform_real_distribution& r) { return !(l == r); }

 private:
  param_type param_;
};

template <class IntType = int>
class uniform_int_distribution {
 public:
  typedef IntType result_type;
  typedef thrust::pair<IntType, IntType> param_type;
  THRUST_CDNA4_HD explicit uniform_int_distribution(IntType a = 0, IntType b = std::numeric_limits<IntType>::max()) : param_(a, b) {}
  THRUST_CDNA4_HD explicit uniform_int_distribution(const param_type& p) : param_(p) {}
  THRUST_CDNA4_HD void reset() {}
  template <class Urng> THRUST_CDNA4_HD result_type operator()(Urng& urng) { return (*this)(urng, param_); }
  // a double drawn from [a, b + 1), truncated
  template <class Urng> THRUST_CDNA4_HD result_type operator()(Urng& urng, const param_type& p) {
    uniform_real_distribution<double> real(static_cast<double>(p.first), static_cast<double>(p.second) + 1.0);
    return static_cast<result_type>(real(urng));
  }
  THRUST_CDNA4_HD result_type a() const { return param_.first; }
  THRUST_CDNA4_HD result_type b() const { return param_.second; }
  THRUST_CDNA4_HD param_type param() const { return param_; }
  THRUST_CDNA4_HD void param(const param_type& p) { param_ = p; }
  THRUST_CDNA4_HD result_type(min)() const { return a(); }
  THRUST_CDNA4_HD result_type(max)() const { return b(); }
  THRUST_CDNA4_HD friend bool operator==(const uniform_int_distribution& l, const uniform_int_distribution& r) { return l.param_ == r.param_; }
  THRUST_CDNA4_HD friend bool operator!=(const uniform_int_distribution& l, const uniform_int_distribution& r) { return !(l == r); }

 private:
  param_type param_;
};

template <class RealType = double>
class normal_distribution {
 public:
  typedef RealType result_type;
  typedef thrust::pair<RealType, RealType> param_type;
  THRUST_CDNA4_HD explicit normal_distribution(RealType mean = 0.0, RealType stddev = 1.0) : param_(mean, stddev), r1_(), r2_(), rho_(), valid_(false) {}
  THRUST_CDNA4_HD explicit normal_distribution(const param_type& p) : param_(p), r1_(), r2_(), rho_(), valid_(false) {}
  THRUST_CDNA4_HD void reset() { valid_ = false; }
  template <class Urng> THRUST_CDNA4_HD result_type operator()(Urng& urng) { return (*this)(urng, param_); }
  // Box-Muller: two uniforms give a radius and an angle; the cosine branch is returned first and
  // the sine branch, from the same pair, by the next call
  template <class Urng> THRUST_CDNA4_HD result_type operator()(Urng& urng, const param_type& p) {
    using std::cos; using std::log; using std::sin; using std::sqrt;
    if (!valid_) {
      uniform_real_distribution<RealType> u01;
      r1_ = u01(urng);
      r2_ = u01(urng);
      rho_ = sqrt(-RealType(2) * log(RealType(1) - r2_));
      valid_ = true;
    } else {
      valid_ = false;
    }
    const RealType pi = RealType(3.14159265358979323846);
    const RealType unit = rho_ * (valid_ ? cos(RealType(2) * pi * r1_) : sin(RealType(2) * pi * r1_));
    return p.first + p.second * unit;
  }
  THRUST_CDNA4_HD result_type mean() const { return param_.first; }
  THRUST_CDNA4_HD result_type stddev() const { return param_.second; }
  THRUST_CDNA4_HD param_type param() const { return param_; }
  THRUST_CDNA4_HD void param(const param_type& p) { param_ = p; }
  THRUST_CDNA4_HD result_type(min)() const { return -std::numeric_limits<RealType>::max(); }
  THRUST_CDNA4_HD result_type(max)() const { return std::numeric_limits<RealType>::max(); }

 private:
  param_type param_;
  RealType r1_, r2_, rho_;
  bool valid_;
};

}  // namespace random
using random::default_random_engine;
using random::linear_congruential_engine;
using random::minstd_rand;
using random::minstd_rand0;
using random::normal_distribution;
using random::uniform_int_distribution;
using random::uniform_real_distribution;
}  // namespace thrust

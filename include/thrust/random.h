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
#include <type_traits>
#include <cstddef>
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
  // saved and restored as its two parameters (thrust/random/detail/uniform_real_distribution.inl: stream_out, stream_in)
  template <class Ch, class Tr> friend std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const uniform_real_distribution& d) {
    return os << d.param_.first << os.widen(' ') << d.param_.second;
  }
  template <class Ch, class Tr> friend std::basic_istream<Ch, Tr>& operator>>(std::basic_istream<Ch, Tr>& is, uniform_real_distribution& d) {
    return is >> d.param_.first >> d.param_.second;
  }

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
  // saved and restored as its two parameters (thrust/random/detail/uniform_int_distribution.inl: stream_out, stream_in)
  template <class Ch, class Tr> friend std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const uniform_int_distribution& d) {
    return os << d.param_.first << os.widen(' ') << d.param_.second;
  }
  template <class Ch, class Tr> friend std::basic_istream<Ch, Tr>& operator>>(std::basic_istream<Ch, Tr>& is, uniform_int_distribution& d) {
    return is >> d.param_.first >> d.param_.second;
  }

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
  THRUST_CDNA4_HD friend bool operator==(const normal_distribution& l, const normal_distribution& r) { return l.param_ == r.param_; }
  THRUST_CDNA4_HD friend bool operator!=(const normal_distribution& l, const normal_distribution& r) { return !(l == r); }
  // saved and restored as mean and standard deviation (thrust/random/detail/normal_distribution.inl:206-231)
  template <class Ch, class Tr> friend std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const normal_distribution& d) {
    return os << d.param_.first << os.widen(' ') << d.param_.second;
  }
  template <class Ch, class Tr> friend std::basic_istream<Ch, Tr>& operator>>(std::basic_istream<Ch, Tr>& is, normal_distribution& d) {
    return is >> d.param_.first >> d.param_.second;
  }

 private:
  param_type param_;
  RealType r1_, r2_, rho_;
  bool valid_;
};

// ---- the other engines of the reference, restated so that every stream is identical number for
// number (the 10000th values of thrust/random.h:63-84 and subtract_with_carry_engine.h:226-239
// are the known answers)

// x_i = (x_{i-s} - x_{i-r} - carry) mod 2^w (thrust/random/detail/subtract_with_carry_engine.inl):
// seeded from linear_congruential_engine<result_type, 40014, 0, 2147483563>, one value per word
template <class UIntType, std::size_t w, std::size_t s, std::size_t r>
class subtract_with_carry_engine {
 public:
  typedef UIntType result_type;
  static const std::size_t word_size = w;
  static const std::size_t short_lag = s;
  static const std::size_t long_lag = r;
  static const result_type modulus = UIntType(1) << w;
  static const result_type min = 0;
  static const result_type max = modulus - 1;
  static const result_type default_seed = 19780503u;
  THRUST_CDNA4_HD explicit subtract_with_carry_engine(result_type value = default_seed) { seed(value); }
  THRUST_CDNA4_HD void seed(result_type value = default_seed) {
    linear_congruential_engine<result_type, 40014u, 0u, 2147483563u> e(value == 0u ? default_seed : value);
    for (std::size_t i = 0; i < long_lag; ++i) x_[i] = (result_type)(e() % modulus);
    carry_ = (x_[long_lag - 1] == 0);
    k_ = 0;
  }
  THRUST_CDNA4_HD result_type operator()() {
    int short_index = (int)k_ - (int)short_lag;
    if (short_index < 0) short_index += (int)long_lag;
    result_type xi;
    if (x_[short_index] >= x_[k_] + carry_) {
      xi = x_[short_index] - x_[k_] - carry_;
      carry_ = 0;
    } else {
      xi = modulus - x_[k_] - carry_ + x_[short_index];
      carry_ = 1;
    }
    x_[k_] = xi;
    ++k_;
    if (k_ >= long_lag) k_ = 0;
    return xi;
  }
  THRUST_CDNA4_HD void discard(unsigned long long z) {
    for (; z > 0; --z) (*this)();
  }
  THRUST_CDNA4_HD friend bool operator==(const subtract_with_carry_engine& a, const subtract_with_carry_engine& b) {
    bool same = a.carry_ == b.carry_;
    for (std::size_t i = 0; i < r; ++i) same &= a.x_[(i + a.k_) % r] == b.x_[(i + b.k_) % r];
    return same;
  }
  THRUST_CDNA4_HD friend bool operator!=(const subtract_with_carry_engine& a, const subtract_with_carry_engine& b) { return !(a == b); }
  template <class Ch, class Tr> friend std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const subtract_with_carry_engine& e) {
    for (std::size_t i = 0; i < r; ++i) os << e.x_[(i + e.k_) % r] << ' ';
    return os << e.carry_;
  }
  template <class Ch, class Tr> friend std::basic_istream<Ch, Tr>& operator>>(std::basic_istream<Ch, Tr>& is, subtract_with_carry_engine& e) {
    for (std::size_t i = 0; i < r; ++i) is >> e.x_[i];
    is >> e.carry_;
    e.k_ = 0;
    return is;
  }
 private:
  result_type x_[r];
  result_type carry_;
  unsigned int k_;
};
template <class U, std::size_t w, std::size_t s, std::size_t r> const U subtract_with_carry_engine<U, w, s, r>::modulus;
template <class U, std::size_t w, std::size_t s, std::size_t r> const U subtract_with_carry_engine<U, w, s, r>::min;
template <class U, std::size_t w, std::size_t s, std::size_t r> const U subtract_with_carry_engine<U, w, s, r>::max;
template <class U, std::size_t w, std::size_t s, std::size_t r> const U subtract_with_carry_engine<U, w, s, r>::default_seed;
typedef subtract_with_carry_engine<std::uint32_t, 24, 10, 24> ranlux24_base;
typedef subtract_with_carry_engine<std::uint64_t, 48, 5, 12> ranlux48_base;

// of every block of p values of the base engine the first r are used (thrust/random/detail/discard_block_engine.inl)
template <class Engine, std::size_t p, std::size_t r>
class discard_block_engine {
 public:
  typedef Engine base_type;
  typedef typename base_type::result_type result_type;
  static const std::size_t block_size = p;
  static const std::size_t used_block = r;
  static const result_type min = base_type::min;
  static const result_type max = base_type::max;
  THRUST_CDNA4_HD discard_block_engine() : e_(), n_(0) {}
  THRUST_CDNA4_HD explicit discard_block_engine(const base_type& urng) : e_(urng), n_(0) {}
  THRUST_CDNA4_HD explicit discard_block_engine(result_type s) : e_(s), n_(0) {}
  THRUST_CDNA4_HD void seed() { e_.seed(); n_ = 0; }
  THRUST_CDNA4_HD void seed(result_type s) { e_.seed(s); n_ = 0; }
  THRUST_CDNA4_HD result_type operator()() {
    if (n_ >= used_block) {
      e_.discard(block_size - n_);
      n_ = 0;
    }
    ++n_;
    return e_();
  }
  THRUST_CDNA4_HD void discard(unsigned long long z) {
    for (; z > 0; --z) (*this)();
  }
  THRUST_CDNA4_HD const base_type& base() const { return e_; }
  THRUST_CDNA4_HD friend bool operator==(const discard_block_engine& a, const discard_block_engine& b) { return a.e_ == b.e_ && a.n_ == b.n_; }
  THRUST_CDNA4_HD friend bool operator!=(const discard_block_engine& a, const discard_block_engine& b) { return !(a == b); }
  template <class Ch, class Tr> friend std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const discard_block_engine& e) { return os << e.e_ << ' ' << e.n_; }
  template <class Ch, class Tr> friend std::basic_istream<Ch, Tr>& operator>>(std::basic_istream<Ch, Tr>& is, discard_block_engine& e) { return is >> e.e_ >> e.n_; }
 private:
  base_type e_;
  unsigned int n_;
};
template <class E, std::size_t p, std::size_t r> const typename E::result_type discard_block_engine<E, p, r>::min;
template <class E, std::size_t p, std::size_t r> const typename E::result_type discard_block_engine<E, p, r>::max;
typedef discard_block_engine<ranlux24_base, 223, 23> ranlux24;
typedef discard_block_engine<ranlux48_base, 389, 11> ranlux48;

// Tausworthe generator (thrust/random/detail/linear_feedback_shift_engine.inl)
template <class UIntType, std::size_t w, std::size_t k, std::size_t q, std::size_t s>
class linear_feedback_shift_engine {
 public:
  typedef UIntType result_type;
  static const std::size_t word_size = w;
  static const std::size_t exponent1 = k;
  static const std::size_t exponent2 = q;
  static const std::size_t step_size = s;
  static const result_type wordmask = w >= 8 * sizeof(UIntType) ? ~UIntType(0) : (UIntType(1) << (w % (8 * sizeof(UIntType)))) - 1;
  static const result_type min = 0;
  static const result_type max = wordmask;
  static const result_type default_seed = 341u;
  THRUST_CDNA4_HD explicit linear_feedback_shift_engine(result_type value = default_seed) { seed(value); }
  THRUST_CDNA4_HD void seed(result_type value = default_seed) { value_ = value; }
  THRUST_CDNA4_HD result_type operator()() {
    const UIntType b = (((value_ << q) ^ value_) & wordmask) >> (k - s);
    const UIntType mask = ((~static_cast<UIntType>(0)) << (w - k)) & wordmask;
    value_ = ((value_ & mask) << s) ^ b;
    return value_;
  }
  THRUST_CDNA4_HD void discard(unsigned long long z) {
    for (; z > 0; --z) (*this)();
  }
  THRUST_CDNA4_HD friend bool operator==(const linear_feedback_shift_engine& a, const linear_feedback_shift_engine& b) { return a.value_ == b.value_; }
  THRUST_CDNA4_HD friend bool operator!=(const linear_feedback_shift_engine& a, const linear_feedback_shift_engine& b) { return a.value_ != b.value_; }
  template <class Ch, class Tr> friend std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const linear_feedback_shift_engine& e) { return os << e.value_; }
  template <class Ch, class Tr> friend std::basic_istream<Ch, Tr>& operator>>(std::basic_istream<Ch, Tr>& is, linear_feedback_shift_engine& e) { return is >> e.value_; }
 private:
  result_type value_;
};
template <class U, std::size_t w, std::size_t k, std::size_t q, std::size_t s> const U linear_feedback_shift_engine<U, w, k, q, s>::wordmask;
template <class U, std::size_t w, std::size_t k, std::size_t q, std::size_t s> const U linear_feedback_shift_engine<U, w, k, q, s>::min;
template <class U, std::size_t w, std::size_t k, std::size_t q, std::size_t s> const U linear_feedback_shift_engine<U, w, k, q, s>::max;
template <class U, std::size_t w, std::size_t k, std::size_t q, std::size_t s> const U linear_feedback_shift_engine<U, w, k, q, s>::default_seed;

// ((b1() - min1) << s1) ^ ((b2() - min2) << s2) (thrust/random/detail/xor_combine_engine.inl).  `max`
// is the exact maximum when both shifted ranges are bit masks (every engine combined in this
// library); otherwise the smallest all-ones value that covers both.
namespace detail {
template <class T> THRUST_CDNA4_HD constexpr T all_ones_covering(T v, T acc = 0) { return acc >= v ? acc : all_ones_covering<T>(v, (T)((acc << 1) | 1)); }
}  // namespace detail
template <class Engine1, std::size_t s1, class Engine2, std::size_t s2 = 0u>
class xor_combine_engine {
 public:
  typedef Engine1 base1_type;
  typedef Engine2 base2_type;
  typedef typename std::conditional<(sizeof(typename base2_type::result_type) > sizeof(typename base1_type::result_type)),
                                    typename base2_type::result_type, typename base1_type::result_type>::type result_type;
  static const std::size_t shift1 = s1;
  static const std::size_t shift2 = s2;
  static const result_type min = 0;
  static const result_type max = detail::all_ones_covering<result_type>(
      (result_type)((result_type)(base1_type::max - base1_type::min) << s1) | (result_type)((result_type)(base2_type::max - base2_type::min) << s2));
  THRUST_CDNA4_HD xor_combine_engine() : b1_(), b2_() {}
  THRUST_CDNA4_HD xor_combine_engine(const base1_type& urng1, const base2_type& urng2) : b1_(urng1), b2_(urng2) {}
  THRUST_CDNA4_HD explicit xor_combine_engine(result_type s) : b1_(s), b2_(s) {}
  THRUST_CDNA4_HD void seed() { b1_.seed(); b2_.seed(); }
  THRUST_CDNA4_HD void seed(result_type s) { b1_.seed(s); b2_.seed(s); }
  THRUST_CDNA4_HD result_type operator()() {
    return (result_type(b1_() - base1_type::min) << shift1) ^ (result_type(b2_() - base2_type::min) << shift2);
  }
  THRUST_CDNA4_HD void discard(unsigned long long z) {
    for (; z > 0; --z) (*this)();
  }
  THRUST_CDNA4_HD const base1_type& base1() const { return b1_; }
  THRUST_CDNA4_HD const base2_type& base2() const { return b2_; }
  THRUST_CDNA4_HD friend bool operator==(const xor_combine_engine& a, const xor_combine_engine& b) { return a.b1_ == b.b1_ && a.b2_ == b.b2_; }
  THRUST_CDNA4_HD friend bool operator!=(const xor_combine_engine& a, const xor_combine_engine& b) { return !(a == b); }
  template <class Ch, class Tr> friend std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const xor_combine_engine& e) { return os << e.b1_ << ' ' << e.b2_; }
  template <class Ch, class Tr> friend std::basic_istream<Ch, Tr>& operator>>(std::basic_istream<Ch, Tr>& is, xor_combine_engine& e) { return is >> e.b1_ >> e.b2_; }
 private:
  base1_type b1_;
  base2_type b2_;
};
template <class E1, std::size_t s1, class E2, std::size_t s2> const typename xor_combine_engine<E1, s1, E2, s2>::result_type xor_combine_engine<E1, s1, E2, s2>::min;
template <class E1, std::size_t s1, class E2, std::size_t s2> const typename xor_combine_engine<E1, s1, E2, s2>::result_type xor_combine_engine<E1, s1, E2, s2>::max;
// L'Ecuyer's three-component Tausworthe generator (thrust/random.h:85-93)
typedef xor_combine_engine<linear_feedback_shift_engine<std::uint32_t, 32u, 31u, 13u, 12u>, 0,
                           xor_combine_engine<linear_feedback_shift_engine<std::uint32_t, 32u, 29u, 2u, 4u>, 0,
                                              linear_feedback_shift_engine<std::uint32_t, 32u, 28u, 3u, 17u>, 0>,
                           0>
    taus88;

}  // namespace random
using random::discard_block_engine;
using random::linear_feedback_shift_engine;
using random::ranlux24;
using random::ranlux24_base;
using random::ranlux48;
using random::ranlux48_base;
using random::subtract_with_carry_engine;
using random::taus88;
using random::xor_combine_engine;
using random::default_random_engine;
using random::linear_congruential_engine;
using random::minstd_rand;
using random::minstd_rand0;
using random::normal_distribution;
using random::uniform_int_distribution;
using random::uniform_real_distribution;
}  // namespace thrust

// thrust::shuffle / shuffle_copy (thrust/shuffle.h): a pseudo-random permutation drawn from a
// uniform random bit generator.  The permutation is the reference's
// (thrust/system/detail/generic/shuffle.inl:33-105, :146-185): a 24-round Feistel network keyed by 24
// draws of the generator is a bijection on [0, 2^bits) with 2^bits >= m; output position p holds
// input element b(i) for the p-th index i (in increasing order) whose image b(i) falls below m.
// Host and device ranges give the same permutation for the same generator state.  On the device
// that is one stable compaction over the index range (the select engine).
#pragma once
#include <cstdint>
#include <utility>
#include <thrust/detail/iterator_util.h>
#include <thrust/device_vector.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

namespace thrust {
namespace detail {
class feistel_bijection {
 public:
  template <class URBG>
  feistel_bijection(std::uint64_t m, URBG&& g) {
    const std::uint64_t total_bits = cipher_bits(m);
    left_bits_ = total_bits / 2;
    left_mask_ = (1ull << left_bits_) - 1;
    right_bits_ = total_bits - left_bits_;
    right_mask_ = (1ull << right_bits_) - 1;
    for (std::uint32_t i = 0; i < kRounds; i++) key_[i] = (std::uint32_t)g();
  }
  THRUST_CDNA4_HD std::uint64_t nearest_power_of_two() const { return 1ull << (left_bits_ + right_bits_); }
  THRUST_CDNA4_HD std::uint64_t operator()(const std::uint64_t val) const {
    std::uint32_t left = (std::uint32_t)(val >> right_bits_), right = (std::uint32_t)(val & right_mask_);
    for (std::uint32_t i = 0; i < kRounds; i++) {
      const std::uint64_t product = 0xD2B74407B1CE6E93ull * (std::uint64_t)left;
      const std::uint32_t hi = (std::uint32_t)(product >> 32);
      std::uint32_t lo = (std::uint32_t)product;
      lo = (lo << (right_bits_ - left_bits_)) | right >> left_bits_;
      left = ((hi ^ key_[i]) ^ right) & (std::uint32_t)left_mask_;
      right = lo & (std::uint32_t)right_mask_;
    }
    return (std::uint64_t)(left << right_bits_) | (std::uint64_t)right;
  }
 private:
  static std::uint64_t cipher_bits(std::uint64_t m) {
    if (m <= 16) return 4;
    std::uint64_t bits = 0;
    for (m--; m != 0; m >>= 1) bits++;
    return bits;
  }
  static constexpr std::uint32_t kRounds = 24;
  std::uint64_t right_bits_, left_bits_, right_mask_, left_mask_;
  std::uint32_t key_[kRounds];
};
#if defined(__HIPCC__)
// index i of [0, 2^bits) is kept when its image is an input position; the item is that input
template <class In, class Out> struct shuffle_op {
  typedef typename std::iterator_traits<In>::value_type item;
  static constexpr bool rejects = false;
  In in; Out out; std::uint64_t m; feistel_bijection b;
  __device__ item load(std::int64_t i, bool& keep) const {
    const std::uint64_t from = b((std::uint64_t)i);
    keep = from < m;
    return in[keep ? from : 0];
  }
  __device__ void store(const item& x, std::int64_t pos) const { out[pos] = x; }
};
#endif
}  // namespace detail

}  // namespace thrust
#include <thrust/system/cdna4/detail/shuffle_copy.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/shuffle.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Out, class URBG>
void shuffle_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result, URBG&& g) {
  shuffle_copy(detail::derived_cast(detail::strip_const(exec)), first, last, result, g);
}
template <class In, class Out, class URBG>
void shuffle_copy(const system::cpp::detail::par_t&, In first, In last, Out result, URBG&& g) {
  const std::uint64_t m = (std::uint64_t)(last - first);
  if (m == 0) return;
  detail::feistel_bijection bijection(m, g);
  const std::uint64_t n = bijection.nearest_power_of_two();
  for (std::uint64_t i = 0; i < n; i++) {
    const std::uint64_t from = bijection(i);
    if (from < m) {
      *result = first[from];
      ++result;
    }
  }
}
}  // namespace thrust
#include <thrust/system/cdna4/detail/shuffle.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/shuffle.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class URBG>
void shuffle(const detail::execution_policy_base<D>& exec, It first, It last, URBG&& g) {
  shuffle(detail::derived_cast(detail::strip_const(exec)), first, last, g);
}
template <class It, class URBG>
void shuffle(const system::cpp::detail::par_t& exec, It first, It last, URBG&& g) {
  typedef typename std::iterator_traits<It>::value_type T;
  std::vector<T> copy(first, last);
  shuffle_copy(exec, copy.begin(), copy.end(), first, g);
}
template <class It, class URBG, detail::enable_if_device<It, URBG> = 0> void shuffle(It first, It last, URBG&& g) { shuffle(typename detail::implicit_policy<It, URBG>::type(), first, last, g); }
template <class It, class URBG, detail::enable_if_host<It, URBG> = 0> void shuffle(It first, It last, URBG&& g) { shuffle(host, first, last, g); }
template <class In, class Out, class URBG, detail::enable_if_device<In, Out, URBG> = 0> void shuffle_copy(In first, In last, Out result, URBG&& g) { shuffle_copy(typename detail::implicit_policy<In, Out, URBG>::type(), first, last, result, g); }
template <class In, class Out, class URBG, detail::enable_if_host<In, Out, URBG> = 0> void shuffle_copy(In first, In last, Out result, URBG&& g) { shuffle_copy(host, first, last, result, g); }
}  // namespace thrust

// thrust::generate / generate_n (thrust/generate.h): every element is assigned gen().
#pragma once
#include <algorithm>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

namespace thrust {
namespace detail {
template <class Out, class G> struct generate_body {
  Out out; G gen;
  THRUST_CDNA4_HD void operator()(std::int64_t i) { out[i] = gen(); }
};
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/generate.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/generate.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class G>
void generate(const detail::execution_policy_base<D>& exec, It first, It last, G gen) {
  generate(detail::derived_cast(detail::strip_const(exec)), first, last, gen);
}
template <class It, class G>
void generate(const system::cpp::detail::par_t&, It first, It last, G gen) { std::generate(first, last, gen); }
template <class Policy, class It, class Size, class G, detail::enable_if_policy<Policy> = 0>
It generate_n(const Policy& exec, It first, Size n, G gen) {
  generate(exec, first, first + n, gen);
  return first + n;
}
template <class It, class G, detail::enable_if_device<It, G> = 0> void generate(It f, It l, G g) { generate(device, f, l, g); }
template <class It, class G, detail::enable_if_host<It, G> = 0> void generate(It f, It l, G g) { generate(host, f, l, g); }
template <class It, class Size, class G, detail::enable_if_device<It, Size, G> = 0> It generate_n(It f, Size n, G g) { return generate_n(device, f, n, g); }
template <class It, class Size, class G, detail::enable_if_host<It, Size, G> = 0> It generate_n(It f, Size n, G g) { return generate_n(host, f, n, g); }
}  // namespace thrust

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
namespace detail {
template <class Policy, class It, class Size, class G>
It composed_generate_n(const Policy& exec, It first, Size n, G gen) {
  generate(exec, first, first + n, gen);
  return first + n;
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Size, class G>
It generate_n(execution_policy<D_>& exec, It first, Size n, G gen) { return thrust::detail::composed_generate_n(exec, first, n, gen); }
}}  // namespace system::cdna4
template <class D_, class It, class Size, class G>
It generate_n(const detail::execution_policy_base<D_>& exec, It first, Size n, G gen) { return generate_n(detail::derived_cast(detail::strip_const(exec)), first, n, gen); }
template <class It, class Size, class G>
It generate_n(const system::cpp::detail::par_t& exec, It first, Size n, G gen) { return detail::composed_generate_n(exec, first, n, gen); }
template <class It, class G, detail::enable_if_device<It, G> = 0> void generate(It f, It l, G g) { generate(typename detail::implicit_policy<It, G>::type(), f, l, g); }
template <class It, class G, detail::enable_if_host<It, G> = 0> void generate(It f, It l, G g) { generate(host, f, l, g); }
template <class It, class Size, class G, detail::enable_if_device<It, Size, G> = 0> It generate_n(It f, Size n, G g) { return generate_n(typename detail::implicit_policy<It, Size, G>::type(), f, n, g); }
template <class It, class Size, class G, detail::enable_if_host<It, Size, G> = 0> It generate_n(It f, Size n, G g) { return generate_n(host, f, n, g); }
}  // namespace thrust

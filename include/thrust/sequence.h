// thrust::sequence (thrust/sequence.h): first[i] = init + i * step.
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

#include <thrust/system/cdna4/detail/sequence.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/sequence.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class It, class T>
void sequence(const detail::execution_policy_base<D>& exec, It first, It last, T init, T step) {
  sequence(detail::derived_cast(detail::strip_const(exec)), first, last, init, step);
}
namespace detail {
// element i, computed in the type of init and step (thrust/system/detail/generic/sequence.inl:36-60)
template <class T> inline T sequence_value(const T& init, const T& step, std::size_t i, std::true_type) { return (T)(init + (T)i * step); }
template <class T> inline T sequence_value(const T& init, const T& step, std::size_t i, std::false_type) { return init + step * i; }
}  // namespace detail
template <class It, class T>
void sequence(const system::cpp::detail::par_t&, It first, It last, T init, T step) {
  std::size_t i = 0;
  for (; first != last; ++first, ++i) *first = detail::sequence_value(init, step, i, std::is_arithmetic<T>());
}
// the shorter forms dispatch on the policy like the full one (testing/sequence.cu:8-24 overloads the shortest)
template <class D, class It, class T>
void sequence(const detail::execution_policy_base<D>& exec, It first, It last, T init) {
  sequence(detail::derived_cast(detail::strip_const(exec)), first, last, init);
}
template <class D, class It, class = typename std::iterator_traits<It>::iterator_category>
void sequence(const detail::execution_policy_base<D>& exec, It first, It last) {
  sequence(detail::derived_cast(detail::strip_const(exec)), first, last);
}
template <class It, class T>
void sequence(const system::cpp::detail::par_t& exec, It first, It last, T init) { sequence(exec, first, last, init, T(1)); }
template <class It, class = typename std::iterator_traits<It>::iterator_category>
void sequence(const system::cpp::detail::par_t& exec, It first, It last) {
  typedef typename detail::value_of<It>::type V;
  sequence(exec, first, last, V(0), V(1));
}

template <class It, detail::enable_if_device<It> = 0> void sequence(It f, It l) { sequence(typename detail::implicit_policy<It>::type(), f, l); }
template <class It, detail::enable_if_host<It> = 0> void sequence(It f, It l) { sequence(host, f, l); }
template <class It, class T, detail::enable_if_device<It, T> = 0> void sequence(It f, It l, T init) { sequence(typename detail::implicit_policy<It, T>::type(), f, l, init); }
template <class It, class T, detail::enable_if_host<It, T> = 0> void sequence(It f, It l, T init) { sequence(host, f, l, init); }
template <class It, class T, detail::enable_if_device<It, T> = 0> void sequence(It f, It l, T init, T step) { sequence(typename detail::implicit_policy<It, T>::type(), f, l, init, step); }
template <class It, class T, detail::enable_if_host<It, T> = 0> void sequence(It f, It l, T init, T step) { sequence(host, f, l, init, step); }
}  // namespace thrust

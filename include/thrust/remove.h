// thrust::remove / remove_if / remove_copy / remove_copy_if (thrust/remove.h;
// thrust/system/cuda/detail/remove.h): stable; the in-place forms compact from a temporary copy.
#pragma once
#include <algorithm>
#include <thrust/count.h>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

#include <thrust/system/cdna4/detail/remove.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/remove.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Out, class Pred>
Out remove_copy_if(const detail::execution_policy_base<D>& exec, In first, In last, Out out, Pred pred) {
  return remove_copy_if(detail::derived_cast(detail::strip_const(exec)), first, last, out, pred);
}
template <class D, class In, class Pred>
In remove_if(const detail::execution_policy_base<D>& exec, In first, In last, Pred pred) {
  return remove_if(detail::derived_cast(detail::strip_const(exec)), first, last, pred);
}
template <class In, class Out, class Pred>
Out remove_copy_if(const system::cpp::detail::par_t&, In first, In last, Out out, Pred pred) { return std::remove_copy_if(first, last, out, pred); }
template <class In, class Pred>
In remove_if(const system::cpp::detail::par_t&, In first, In last, Pred pred) { return std::remove_if(first, last, pred); }

template <class Policy, class In, class Out, class V, class = typename std::iterator_traits<In>::iterator_category>
Out remove_copy(const Policy& exec, In first, In last, Out out, const V& value) {
  return remove_copy_if(exec, first, last, out, detail::equals_value<V>{value});
}
template <class Policy, class In, class V, class = typename std::iterator_traits<In>::iterator_category>
In remove(const Policy& exec, In first, In last, const V& value) { return remove_if(exec, first, last, detail::equals_value<V>{value}); }

template <class In, class Out, class Pred, detail::enable_if_device<In, Out, Pred> = 0> Out remove_copy_if(In f, In l, Out o, Pred p) { return remove_copy_if(typename detail::implicit_policy<In, Out, Pred>::type(), f, l, o, p); }
template <class In, class Out, class Pred, detail::enable_if_host<In, Out, Pred> = 0> Out remove_copy_if(In f, In l, Out o, Pred p) { return remove_copy_if(host, f, l, o, p); }
template <class In, class Pred, detail::enable_if_device<In, Pred> = 0> In remove_if(In f, In l, Pred p) { return remove_if(typename detail::implicit_policy<In, Pred>::type(), f, l, p); }
template <class In, class Pred, detail::enable_if_host<In, Pred> = 0> In remove_if(In f, In l, Pred p) { return remove_if(host, f, l, p); }
template <class In, class V, detail::enable_if_device<In, V> = 0> In remove(In f, In l, const V& v) { return remove(typename detail::implicit_policy<In, V>::type(), f, l, v); }
template <class In, class V, detail::enable_if_host<In, V> = 0> In remove(In f, In l, const V& v) { return remove(host, f, l, v); }
}  // namespace thrust

// thrust::remove / remove_if / remove_copy / remove_copy_if (thrust/remove.h;
// thrust/system/cuda/detail/remove.h): stable; the in-place forms compact from a temporary copy.
#pragma once
#include <algorithm>
#include <memory>
#include <thrust/copy.h>
#include <thrust/count.h>
#include <thrust/functional.h>
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

namespace detail {
template <class Policy, class In, class Out, class V>
Out composed_remove_copy(const Policy& exec, In first, In last, Out out, const V& value) {
  return remove_copy_if(exec, first, last, out, detail::equals_value<V>{value});
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class Out, class V>
Out remove_copy(execution_policy<D_>& exec, In first, In last, Out out, const V& value) { return thrust::detail::composed_remove_copy(exec, first, last, out, value); }
}}  // namespace system::cdna4
template <class D_, class In, class Out, class V>
Out remove_copy(const detail::execution_policy_base<D_>& exec, In first, In last, Out out, const V& value) { return remove_copy(detail::derived_cast(detail::strip_const(exec)), first, last, out, value); }
template <class In, class Out, class V>
Out remove_copy(const system::cpp::detail::par_t& exec, In first, In last, Out out, const V& value) { return detail::composed_remove_copy(exec, first, last, out, value); }
namespace detail {
template <class Policy, class In, class V>
In composed_remove(const Policy& exec, In first, In last, const V& value) { return remove_if(exec, first, last, detail::equals_value<V>{value}); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class V>
In remove(execution_policy<D_>& exec, In first, In last, const V& value) { return thrust::detail::composed_remove(exec, first, last, value); }
}}  // namespace system::cdna4
template <class D_, class In, class V>
In remove(const detail::execution_policy_base<D_>& exec, In first, In last, const V& value) { return remove(detail::derived_cast(detail::strip_const(exec)), first, last, value); }
template <class In, class V>
In remove(const system::cpp::detail::par_t& exec, In first, In last, const V& value) { return detail::composed_remove(exec, first, last, value); }
namespace detail {
// room for a copy of n elements in the memory a policy's algorithms work on
template <class Policy, class V> struct staged_range {
  template <class D> static void* stream(const system::cdna4::execution_policy<D>& e) { return system::cdna4::detail::stream_of(static_cast<const D&>(e)); }
  system::cdna4::detail::temporary_storage buf;
  staged_range(const Policy& exec, std::size_t n) : buf(n * sizeof(V), stream(exec)) {}
  device_ptr<V> begin() const { return device_ptr<V>(static_cast<V*>(buf.data())); }
};
template <class V> struct staged_range<system::cpp::detail::par_t, V> {
  std::unique_ptr<V[]> buf;
  staged_range(const system::cpp::detail::par_t&, std::size_t n) : buf(new V[n]) {}
  V* begin() const { return buf.get(); }
};
}  // namespace detail
// The forms with a stencil (thrust/remove.h:449-520, :700-780): element i goes when pred(stencil[i]).
namespace detail {
template <class Policy, class In, class St, class Out, class Pred>
Out composed_remove_copy_if(const Policy& exec, In first, In last, St stencil, Out out, Pred pred) {
  return thrust::copy_if(exec, first, last, stencil, out, thrust::not_fn(pred));
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class St, class Out, class Pred>
Out remove_copy_if(execution_policy<D_>& exec, In first, In last, St stencil, Out out, Pred pred) { return thrust::detail::composed_remove_copy_if(exec, first, last, stencil, out, pred); }
}}  // namespace system::cdna4
template <class D_, class In, class St, class Out, class Pred>
Out remove_copy_if(const detail::execution_policy_base<D_>& exec, In first, In last, St stencil, Out out, Pred pred) { return remove_copy_if(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, out, pred); }
template <class In, class St, class Out, class Pred>
Out remove_copy_if(const system::cpp::detail::par_t& exec, In first, In last, St stencil, Out out, Pred pred) { return detail::composed_remove_copy_if(exec, first, last, stencil, out, pred); }
namespace detail {
template <class Policy, class In, class St, class Pred>
In composed_remove_if(const Policy& exec, In first, In last, St stencil, Pred pred) {
  // in place: compacted from a copy of the range, in memory of the range's own system
  typedef typename std::iterator_traits<In>::value_type V;
  const std::size_t n = (std::size_t)(last - first);
  detail::staged_range<Policy, V> staged(exec, n);
  thrust::copy(exec, first, last, staged.begin());
  return thrust::copy_if(exec, staged.begin(), staged.begin() + n, stencil, first, thrust::not_fn(pred));
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class St, class Pred>
In remove_if(execution_policy<D_>& exec, In first, In last, St stencil, Pred pred) { return thrust::detail::composed_remove_if(exec, first, last, stencil, pred); }
}}  // namespace system::cdna4
template <class D_, class In, class St, class Pred>
In remove_if(const detail::execution_policy_base<D_>& exec, In first, In last, St stencil, Pred pred) { return remove_if(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, pred); }
template <class In, class St, class Pred>
In remove_if(const system::cpp::detail::par_t& exec, In first, In last, St stencil, Pred pred) { return detail::composed_remove_if(exec, first, last, stencil, pred); }

template <class In, class Out, class Pred, detail::enable_if_device<In, Out, Pred> = 0> Out remove_copy_if(In f, In l, Out o, Pred p) { return remove_copy_if(typename detail::implicit_policy<In, Out, Pred>::type(), f, l, o, p); }
template <class In, class Out, class Pred, detail::enable_if_host<In, Out, Pred> = 0> Out remove_copy_if(In f, In l, Out o, Pred p) { return remove_copy_if(host, f, l, o, p); }
template <class In, class Pred, detail::enable_if_device<In, Pred> = 0> In remove_if(In f, In l, Pred p) { return remove_if(typename detail::implicit_policy<In, Pred>::type(), f, l, p); }
template <class In, class Pred, detail::enable_if_host<In, Pred> = 0> In remove_if(In f, In l, Pred p) { return remove_if(host, f, l, p); }
template <class In, class V, detail::enable_if_device<In, V> = 0> In remove(In f, In l, const V& v) { return remove(typename detail::implicit_policy<In, V>::type(), f, l, v); }
template <class In, class V, detail::enable_if_host<In, V> = 0> In remove(In f, In l, const V& v) { return remove(host, f, l, v); }
template <class In, class Out, class V, detail::enable_if_device<In, Out, V> = 0,
          typename std::enable_if<!system::cdna4::detail::is_iterator_type<V>::value, int>::type = 0>
Out remove_copy(In f, In l, Out o, const V& v) { return remove_copy(typename detail::implicit_policy<In, Out, V>::type(), f, l, o, v); }
template <class In, class Out, class V, detail::enable_if_host<In, Out, V> = 0,
          typename std::enable_if<!system::cdna4::detail::is_iterator_type<V>::value, int>::type = 0>
Out remove_copy(In f, In l, Out o, const V& v) { return remove_copy(host, f, l, o, v); }
template <class In, class St, class Out, class Pred, detail::enable_if_device<In, St, Out, Pred> = 0>
Out remove_copy_if(In f, In l, St s, Out o, Pred p) { return remove_copy_if(typename detail::implicit_policy<In, St, Out, Pred>::type(), f, l, s, o, p); }
template <class In, class St, class Out, class Pred, detail::enable_if_host<In, St, Out, Pred> = 0>
Out remove_copy_if(In f, In l, St s, Out o, Pred p) { return remove_copy_if(host, f, l, s, o, p); }
template <class In, class St, class Pred, detail::enable_if_device<In, St, Pred> = 0,
          typename std::enable_if<system::cdna4::detail::is_iterator_type<St>::value, int>::type = 0>
In remove_if(In f, In l, St s, Pred p) { return remove_if(typename detail::implicit_policy<In, St, Pred>::type(), f, l, s, p); }
template <class In, class St, class Pred, detail::enable_if_host<In, St, Pred> = 0,
          typename std::enable_if<system::cdna4::detail::is_iterator_type<St>::value, int>::type = 0>
In remove_if(In f, In l, St s, Pred p) { return remove_if(host, f, l, s, p); }
}  // namespace thrust

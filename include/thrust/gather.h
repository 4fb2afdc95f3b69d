// thrust::gather / gather_if (thrust/gather.h): result[i] = input[map[i]].
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

namespace thrust {
namespace detail {
template <class Map, class In, class Out> struct gather_body {
  Map map; In in; Out out;
  THRUST_CDNA4_HD void operator()(std::int64_t i) { out[i] = in[map[i]]; }
};
template <class Map, class S, class In, class Out, class Pred> struct gather_if_body {
  Map map; S stencil; In in; Out out; Pred pred;
  THRUST_CDNA4_HD void operator()(std::int64_t i) {
    if (pred(stencil[i])) out[i] = in[map[i]];
  }
};
struct truthy {
  template <class T> THRUST_CDNA4_HD bool operator()(const T& x) const { return x ? true : false; }
};
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/gather.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/gather.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class Map, class In, class Out>
Out gather(const detail::execution_policy_base<D>& exec, Map map_first, Map map_last, In input, Out result) {
  return gather(detail::derived_cast(detail::strip_const(exec)), map_first, map_last, input, result);
}
template <class Map, class In, class Out>
Out gather(const system::cpp::detail::par_t&, Map map_first, Map map_last, In input, Out result) {
  for (; map_first != map_last; ++map_first, ++result) *result = input[*map_first];
  return result;
}
}  // namespace thrust
#include <thrust/system/cdna4/detail/gather_if.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/gather.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class Map, class S, class In, class Out, class Pred>
Out gather_if(const detail::execution_policy_base<D>& exec, Map map_first, Map map_last, S stencil, In input, Out result, Pred pred) {
  return gather_if(detail::derived_cast(detail::strip_const(exec)), map_first, map_last, stencil, input, result, pred);
}
template <class Map, class S, class In, class Out, class Pred>
Out gather_if(const system::cpp::detail::par_t&, Map map_first, Map map_last, S stencil, In input, Out result, Pred pred) {
  for (; map_first != map_last; ++map_first, ++stencil, ++result)
    if (pred(*stencil)) *result = input[*map_first];
  return result;
}
namespace detail {
template <class Policy, class Map, class S, class In, class Out>
Out composed_gather_if(const Policy& exec, Map mf, Map ml, S st, In in, Out out) { return gather_if(exec, mf, ml, st, in, out, detail::truthy()); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class Map, class S, class In, class Out>
Out gather_if(execution_policy<D_>& exec, Map mf, Map ml, S st, In in, Out out) { return thrust::detail::composed_gather_if(exec, mf, ml, st, in, out); }
}}  // namespace system::cdna4
template <class D_, class Map, class S, class In, class Out>
Out gather_if(const detail::execution_policy_base<D_>& exec, Map mf, Map ml, S st, In in, Out out) { return gather_if(detail::derived_cast(detail::strip_const(exec)), mf, ml, st, in, out); }
template <class Map, class S, class In, class Out>
Out gather_if(const system::cpp::detail::par_t& exec, Map mf, Map ml, S st, In in, Out out) { return detail::composed_gather_if(exec, mf, ml, st, in, out); }

template <class Map, class In, class Out, detail::enable_if_device<Map, In, Out> = 0>
Out gather(Map mf, Map ml, In in, Out out) { return gather(typename detail::implicit_policy<Map, In, Out>::type(), mf, ml, in, out); }
template <class Map, class In, class Out, detail::enable_if_host<Map, In, Out> = 0>
Out gather(Map mf, Map ml, In in, Out out) { return gather(host, mf, ml, in, out); }
template <class Map, class S, class In, class Out, detail::enable_if_device<Map, S, In, Out> = 0>
Out gather_if(Map mf, Map ml, S st, In in, Out out) { return gather_if(typename detail::implicit_policy<Map, S, In, Out>::type(), mf, ml, st, in, out); }
template <class Map, class S, class In, class Out, detail::enable_if_host<Map, S, In, Out> = 0>
Out gather_if(Map mf, Map ml, S st, In in, Out out) { return gather_if(host, mf, ml, st, in, out); }
template <class Map, class S, class In, class Out, class Pred, detail::enable_if_device<Map, S, In, Out, Pred> = 0>
Out gather_if(Map mf, Map ml, S st, In in, Out out, Pred p) { return gather_if(typename detail::implicit_policy<Map, S, In, Out, Pred>::type(), mf, ml, st, in, out, p); }
template <class Map, class S, class In, class Out, class Pred, detail::enable_if_host<Map, S, In, Out, Pred> = 0>
Out gather_if(Map mf, Map ml, S st, In in, Out out, Pred p) { return gather_if(host, mf, ml, st, in, out, p); }
}  // namespace thrust

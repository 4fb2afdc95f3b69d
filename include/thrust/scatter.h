// thrust::scatter / scatter_if (thrust/scatter.h): output[map[i]] = first[i].
#pragma once
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/gather.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

namespace thrust {
namespace detail {
template <class In, class Map, class Out> struct scatter_body {
  In in; Map map; Out out;
  THRUST_CDNA4_HD void operator()(std::int64_t i) { out[map[i]] = in[i]; }
};
template <class In, class Map, class S, class Out, class Pred> struct scatter_if_body {
  In in; Map map; S stencil; Out out; Pred pred;
  THRUST_CDNA4_HD void operator()(std::int64_t i) {
    if (pred(stencil[i])) out[map[i]] = in[i];
  }
};
}  // namespace detail
}  // namespace thrust
#include <thrust/system/cdna4/detail/scatter.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/scatter.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Map, class Out>
void scatter(const detail::execution_policy_base<D>& exec, In first, In last, Map map, Out output) {
  scatter(detail::derived_cast(detail::strip_const(exec)), first, last, map, output);
}
template <class In, class Map, class Out>
void scatter(const system::cpp::detail::par_t&, In first, In last, Map map, Out output) {
  for (; first != last; ++first, ++map) output[*map] = *first;
}
}  // namespace thrust
#include <thrust/system/cdna4/detail/scatter_if.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/scatter.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Map, class S, class Out, class Pred>
void scatter_if(const detail::execution_policy_base<D>& exec, In first, In last, Map map, S stencil, Out output, Pred pred) {
  scatter_if(detail::derived_cast(detail::strip_const(exec)), first, last, map, stencil, output, pred);
}
template <class In, class Map, class S, class Out, class Pred>
void scatter_if(const system::cpp::detail::par_t&, In first, In last, Map map, S stencil, Out output, Pred pred) {
  for (; first != last; ++first, ++map, ++stencil)
    if (pred(*stencil)) output[*map] = *first;
}
namespace detail {
template <class Policy, class In, class Map, class S, class Out>
void composed_scatter_if(const Policy& exec, In f, In l, Map m, S st, Out o) { scatter_if(exec, f, l, m, st, o, detail::truthy()); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class Map, class S, class Out>
void scatter_if(execution_policy<D_>& exec, In f, In l, Map m, S st, Out o) { return thrust::detail::composed_scatter_if(exec, f, l, m, st, o); }
}}  // namespace system::cdna4
template <class D_, class In, class Map, class S, class Out>
void scatter_if(const detail::execution_policy_base<D_>& exec, In f, In l, Map m, S st, Out o) { return scatter_if(detail::derived_cast(detail::strip_const(exec)), f, l, m, st, o); }
template <class In, class Map, class S, class Out>
void scatter_if(const system::cpp::detail::par_t& exec, In f, In l, Map m, S st, Out o) { return detail::composed_scatter_if(exec, f, l, m, st, o); }

template <class In, class Map, class Out, detail::enable_if_device<In, Map, Out> = 0> void scatter(In f, In l, Map m, Out o) { scatter(typename detail::implicit_policy<In, Map, Out>::type(), f, l, m, o); }
template <class In, class Map, class Out, detail::enable_if_host<In, Map, Out> = 0> void scatter(In f, In l, Map m, Out o) { scatter(host, f, l, m, o); }
template <class In, class Map, class S, class Out, detail::enable_if_device<In, Map, S, Out> = 0> void scatter_if(In f, In l, Map m, S st, Out o) { scatter_if(typename detail::implicit_policy<In, Map, S, Out>::type(), f, l, m, st, o); }
template <class In, class Map, class S, class Out, detail::enable_if_host<In, Map, S, Out> = 0> void scatter_if(In f, In l, Map m, S st, Out o) { scatter_if(host, f, l, m, st, o); }
template <class In, class Map, class S, class Out, class Pred, detail::enable_if_device<In, Map, S, Out, Pred> = 0>
void scatter_if(In f, In l, Map m, S st, Out o, Pred p) { scatter_if(typename detail::implicit_policy<In, Map, S, Out, Pred>::type(), f, l, m, st, o, p); }
template <class In, class Map, class S, class Out, class Pred, detail::enable_if_host<In, Map, S, Out, Pred> = 0>
void scatter_if(In f, In l, Map m, S st, Out o, Pred p) { scatter_if(host, f, l, m, st, o, p); }
}  // namespace thrust

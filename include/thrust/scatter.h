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
template <class D, class In, class Map, class Out>
void scatter(const system::cdna4::execution_policy<D>& exec, In first, In last, Map map, Out output) {
  system::cdna4::detail::for_each_index(
      exec.derived(), (std::int64_t)(last - first),
      detail::scatter_body<typename detail::unwrap_iterator<In>::type, typename detail::unwrap_iterator<Map>::type,
                           typename detail::unwrap_iterator<Out>::type>{detail::unwrap(first), detail::unwrap(map), detail::unwrap(output)},
      "scatter: failed to synchronize");
}
template <class In, class Map, class Out>
void scatter(const system::cpp::detail::par_t&, In first, In last, Map map, Out output) {
  for (; first != last; ++first, ++map) output[*map] = *first;
}
template <class D, class In, class Map, class S, class Out, class Pred>
void scatter_if(const system::cdna4::execution_policy<D>& exec, In first, In last, Map map, S stencil, Out output, Pred pred) {
  system::cdna4::detail::for_each_index(
      exec.derived(), (std::int64_t)(last - first),
      detail::scatter_if_body<typename detail::unwrap_iterator<In>::type, typename detail::unwrap_iterator<Map>::type,
                              typename detail::unwrap_iterator<S>::type, typename detail::unwrap_iterator<Out>::type, Pred>{
          detail::unwrap(first), detail::unwrap(map), detail::unwrap(stencil), detail::unwrap(output), pred},
      "scatter_if: failed to synchronize");
}
template <class In, class Map, class S, class Out, class Pred>
void scatter_if(const system::cpp::detail::par_t&, In first, In last, Map map, S stencil, Out output, Pred pred) {
  for (; first != last; ++first, ++map, ++stencil)
    if (pred(*stencil)) output[*map] = *first;
}
template <class Policy, class In, class Map, class S, class Out, detail::enable_if_policy<Policy> = 0>
void scatter_if(const Policy& exec, In f, In l, Map m, S st, Out o) { scatter_if(exec, f, l, m, st, o, detail::truthy()); }

template <class In, class Map, class Out, detail::enable_if_device<In> = 0> void scatter(In f, In l, Map m, Out o) { scatter(device, f, l, m, o); }
template <class In, class Map, class Out, detail::enable_if_host<In> = 0> void scatter(In f, In l, Map m, Out o) { scatter(host, f, l, m, o); }
template <class In, class Map, class S, class Out, detail::enable_if_device<In> = 0> void scatter_if(In f, In l, Map m, S st, Out o) { scatter_if(device, f, l, m, st, o); }
template <class In, class Map, class S, class Out, detail::enable_if_host<In> = 0> void scatter_if(In f, In l, Map m, S st, Out o) { scatter_if(host, f, l, m, st, o); }
template <class In, class Map, class S, class Out, class Pred, detail::enable_if_device<In> = 0>
void scatter_if(In f, In l, Map m, S st, Out o, Pred p) { scatter_if(device, f, l, m, st, o, p); }
template <class In, class Map, class S, class Out, class Pred, detail::enable_if_host<In> = 0>
void scatter_if(In f, In l, Map m, S st, Out o, Pred p) { scatter_if(host, f, l, m, st, o, p); }
}  // namespace thrust

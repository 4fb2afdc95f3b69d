// thrust::partition / stable_partition / partition_copy / stable_partition_copy, with and
// without a stencil (thrust/partition.h; thrust/system/cuda/detail/partition.h:138-606).
// All four are stable here: one pass of the select kernel writes the elements the predicate
// accepts and the ones it rejects, each in input order.  The in-place forms read a temporary
// copy and collect the rejected elements in a second temporary before appending them.
#pragma once
#include <thrust/copy.h>
#include <algorithm>
#include <vector>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/find.h>
#include <thrust/logical.h>
#include <thrust/pair.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

#include <thrust/system/cdna4/detail/partition.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/partition.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class St, class OutT, class OutF, class Pred>
pair<OutT, OutF> stable_partition_copy(const detail::execution_policy_base<D>& exec, In first, In last, St stencil, OutT out_true, OutF out_false, Pred pred) {
  return stable_partition_copy(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, out_true, out_false, pred);
}
template <class D, class In, class OutT, class OutF, class Pred, class = typename std::iterator_traits<OutF>::iterator_category>
pair<OutT, OutF> stable_partition_copy(const detail::execution_policy_base<D>& exec, In first, In last, OutT out_true, OutF out_false, Pred pred) {
  return stable_partition_copy(detail::derived_cast(detail::strip_const(exec)), first, last, out_true, out_false, pred);
}
template <class D, class It, class St, class Pred, class = typename std::iterator_traits<St>::iterator_category>
It stable_partition(const detail::execution_policy_base<D>& exec, It first, It last, St stencil, Pred pred) {
  return stable_partition(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, pred);
}
template <class D, class It, class Pred>
It stable_partition(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  return stable_partition(detail::derived_cast(detail::strip_const(exec)), first, last, pred);
}
// ---- host
template <class In, class St, class OutT, class OutF, class Pred>
pair<OutT, OutF> stable_partition_copy(const system::cpp::detail::par_t&, In first, In last, St stencil, OutT out_true, OutF out_false, Pred pred) {
  for (; first != last; ++first, ++stencil) {
    if (pred(*stencil)) { *out_true = *first; ++out_true; }
    else { *out_false = *first; ++out_false; }
  }
  return thrust::make_pair(out_true, out_false);
}
template <class In, class OutT, class OutF, class Pred, class = typename std::iterator_traits<OutF>::iterator_category>
pair<OutT, OutF> stable_partition_copy(const system::cpp::detail::par_t& e, In first, In last, OutT out_true, OutF out_false, Pred pred) {
  return stable_partition_copy(e, first, last, first, out_true, out_false, pred);
}
template <class It, class St, class Pred, class = typename std::iterator_traits<St>::iterator_category>
It stable_partition(const system::cpp::detail::par_t& e, It first, It last, St stencil, Pred pred) {
  typedef typename std::iterator_traits<It>::value_type V;
  std::vector<V> yes(last - first), no(last - first);
  auto ends = stable_partition_copy(e, first, last, stencil, yes.begin(), no.begin(), pred);
  It mid = std::copy(yes.begin(), ends.first, first);
  std::copy(no.begin(), ends.second, mid);
  return mid;
}
template <class It, class Pred>
It stable_partition(const system::cpp::detail::par_t&, It first, It last, Pred pred) { return std::stable_partition(first, last, pred); }

// ---- partition and partition_copy are the stable forms, any policy
namespace detail {
template <class Policy, class It, class Pred>
It composed_partition(const Policy& exec, It first, It last, Pred pred) { return stable_partition(exec, first, last, pred); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Pred>
It partition(execution_policy<D_>& exec, It first, It last, Pred pred) { return thrust::detail::composed_partition(exec, first, last, pred); }
}}  // namespace system::cdna4
template <class D_, class It, class Pred>
It partition(const detail::execution_policy_base<D_>& exec, It first, It last, Pred pred) { return partition(detail::derived_cast(detail::strip_const(exec)), first, last, pred); }
template <class It, class Pred>
It partition(const system::cpp::detail::par_t& exec, It first, It last, Pred pred) { return detail::composed_partition(exec, first, last, pred); }
namespace detail {
template <class Policy, class It, class St, class Pred, class = typename std::iterator_traits<St>::iterator_category>
It composed_partition(const Policy& exec, It first, It last, St stencil, Pred pred) { return stable_partition(exec, first, last, stencil, pred); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class St, class Pred, class = typename std::iterator_traits<St>::iterator_category>
It partition(execution_policy<D_>& exec, It first, It last, St stencil, Pred pred) { return thrust::detail::composed_partition(exec, first, last, stencil, pred); }
}}  // namespace system::cdna4
template <class D_, class It, class St, class Pred, class = typename std::iterator_traits<St>::iterator_category>
It partition(const detail::execution_policy_base<D_>& exec, It first, It last, St stencil, Pred pred) { return partition(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, pred); }
template <class It, class St, class Pred, class = typename std::iterator_traits<St>::iterator_category>
It partition(const system::cpp::detail::par_t& exec, It first, It last, St stencil, Pred pred) { return detail::composed_partition(exec, first, last, stencil, pred); }
namespace detail {
template <class Policy, class In, class OutT, class OutF, class Pred, class = typename std::iterator_traits<OutF>::iterator_category>
pair<OutT, OutF> composed_partition_copy(const Policy& exec, In first, In last, OutT out_true, OutF out_false, Pred pred) {
  return stable_partition_copy(exec, first, last, out_true, out_false, pred);
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class OutT, class OutF, class Pred, class = typename std::iterator_traits<OutF>::iterator_category>
pair<OutT, OutF> partition_copy(execution_policy<D_>& exec, In first, In last, OutT out_true, OutF out_false, Pred pred) { return thrust::detail::composed_partition_copy(exec, first, last, out_true, out_false, pred); }
}}  // namespace system::cdna4
template <class D_, class In, class OutT, class OutF, class Pred, class = typename std::iterator_traits<OutF>::iterator_category>
pair<OutT, OutF> partition_copy(const detail::execution_policy_base<D_>& exec, In first, In last, OutT out_true, OutF out_false, Pred pred) { return partition_copy(detail::derived_cast(detail::strip_const(exec)), first, last, out_true, out_false, pred); }
template <class In, class OutT, class OutF, class Pred, class = typename std::iterator_traits<OutF>::iterator_category>
pair<OutT, OutF> partition_copy(const system::cpp::detail::par_t& exec, In first, In last, OutT out_true, OutF out_false, Pred pred) { return detail::composed_partition_copy(exec, first, last, out_true, out_false, pred); }
namespace detail {
template <class Policy, class In, class St, class OutT, class OutF, class Pred>
pair<OutT, OutF> composed_partition_copy(const Policy& exec, In first, In last, St stencil, OutT out_true, OutF out_false, Pred pred) {
  return stable_partition_copy(exec, first, last, stencil, out_true, out_false, pred);
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class St, class OutT, class OutF, class Pred>
pair<OutT, OutF> partition_copy(execution_policy<D_>& exec, In first, In last, St stencil, OutT out_true, OutF out_false, Pred pred) { return thrust::detail::composed_partition_copy(exec, first, last, stencil, out_true, out_false, pred); }
}}  // namespace system::cdna4
template <class D_, class In, class St, class OutT, class OutF, class Pred>
pair<OutT, OutF> partition_copy(const detail::execution_policy_base<D_>& exec, In first, In last, St stencil, OutT out_true, OutF out_false, Pred pred) { return partition_copy(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, out_true, out_false, pred); }
template <class In, class St, class OutT, class OutF, class Pred>
pair<OutT, OutF> partition_copy(const system::cpp::detail::par_t& exec, In first, In last, St stencil, OutT out_true, OutF out_false, Pred pred) { return detail::composed_partition_copy(exec, first, last, stencil, out_true, out_false, pred); }
// ---- no policy
#define THRUST_CDNA4_PARTITION_NO_POLICY(NAME)                                                                          \
  template <class It, class Pred, detail::enable_if_device<It, Pred> = 0>                                                     \
  It NAME(It f, It l, Pred p) { return NAME(typename detail::implicit_policy<It, Pred>::type(), f, l, p); }                                                         \
  template <class It, class Pred, detail::enable_if_host<It, Pred> = 0>                                                       \
  It NAME(It f, It l, Pred p) { return NAME(host, f, l, p); }                                                           \
  template <class It, class St, class Pred, detail::enable_if_device<It, St, Pred> = 0,                                           \
            class = typename std::iterator_traits<St>::iterator_category>                                               \
  It NAME(It f, It l, St s, Pred p) { return NAME(typename detail::implicit_policy<It, St, Pred>::type(), f, l, s, p); }                                                \
  template <class It, class St, class Pred, detail::enable_if_host<It, St, Pred> = 0,                                             \
            class = typename std::iterator_traits<St>::iterator_category>                                               \
  It NAME(It f, It l, St s, Pred p) { return NAME(host, f, l, s, p); }
THRUST_CDNA4_PARTITION_NO_POLICY(partition)
THRUST_CDNA4_PARTITION_NO_POLICY(stable_partition)
#undef THRUST_CDNA4_PARTITION_NO_POLICY
#define THRUST_CDNA4_PARTITION_COPY_NO_POLICY(NAME)                                                                     \
  template <class In, class OutT, class OutF, class Pred, detail::enable_if_device<In, OutT, OutF, Pred> = 0>                             \
  pair<OutT, OutF> NAME(In f, In l, OutT t, OutF o, Pred p) { return NAME(typename detail::implicit_policy<In, OutT, OutF, Pred>::type(), f, l, t, o, p); }                     \
  template <class In, class OutT, class OutF, class Pred, detail::enable_if_host<In, OutT, OutF, Pred> = 0>                               \
  pair<OutT, OutF> NAME(In f, In l, OutT t, OutF o, Pred p) { return NAME(host, f, l, t, o, p); }                       \
  template <class In, class St, class OutT, class OutF, class Pred, detail::enable_if_device<In, St, OutT, OutF, Pred> = 0,                   \
            class = typename std::iterator_traits<OutF>::iterator_category>                                             \
  pair<OutT, OutF> NAME(In f, In l, St s, OutT t, OutF o, Pred p) { return NAME(typename detail::implicit_policy<In, St, OutT, OutF, Pred>::type(), f, l, s, t, o, p); }            \
  template <class In, class St, class OutT, class OutF, class Pred, detail::enable_if_host<In, St, OutT, OutF, Pred> = 0,                     \
            class = typename std::iterator_traits<OutF>::iterator_category>                                             \
  pair<OutT, OutF> NAME(In f, In l, St s, OutT t, OutF o, Pred p) { return NAME(host, f, l, s, t, o, p); }
THRUST_CDNA4_PARTITION_COPY_NO_POLICY(partition_copy)
THRUST_CDNA4_PARTITION_COPY_NO_POLICY(stable_partition_copy)
#undef THRUST_CDNA4_PARTITION_COPY_NO_POLICY

// ---- partition_point / is_partitioned (thrust/partition.h:1311-1435), on find_if_not and none_of as
//      the reference's generic layer has them (thrust/system/detail/generic/partition.inl:203-238)
namespace detail {
template <class Policy, class It, class Pred>
It composed_partition_point(const Policy& exec, It first, It last, Pred pred) { return thrust::find_if_not(exec, first, last, pred); }
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Pred>
It partition_point(execution_policy<D_>& exec, It first, It last, Pred pred) { return thrust::detail::composed_partition_point(exec, first, last, pred); }
}}  // namespace system::cdna4
template <class D_, class It, class Pred>
It partition_point(const detail::execution_policy_base<D_>& exec, It first, It last, Pred pred) { return partition_point(detail::derived_cast(detail::strip_const(exec)), first, last, pred); }
template <class It, class Pred>
It partition_point(const system::cpp::detail::par_t& exec, It first, It last, Pred pred) { return detail::composed_partition_point(exec, first, last, pred); }
namespace detail {
template <class Policy, class It, class Pred>
bool composed_is_partitioned(const Policy& exec, It first, It last, Pred pred) {
  return thrust::none_of(exec, thrust::find_if_not(exec, first, last, pred), last, pred);
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Pred>
bool is_partitioned(execution_policy<D_>& exec, It first, It last, Pred pred) { return thrust::detail::composed_is_partitioned(exec, first, last, pred); }
}}  // namespace system::cdna4
template <class D_, class It, class Pred>
bool is_partitioned(const detail::execution_policy_base<D_>& exec, It first, It last, Pred pred) { return is_partitioned(detail::derived_cast(detail::strip_const(exec)), first, last, pred); }
template <class It, class Pred>
bool is_partitioned(const system::cpp::detail::par_t& exec, It first, It last, Pred pred) { return detail::composed_is_partitioned(exec, first, last, pred); }
template <class It, class Pred, detail::enable_if_device<It, Pred> = 0> It partition_point(It f, It l, Pred p) { return partition_point(typename detail::implicit_policy<It, Pred>::type(), f, l, p); }
template <class It, class Pred, detail::enable_if_host<It, Pred> = 0> It partition_point(It f, It l, Pred p) { return partition_point(host, f, l, p); }
template <class It, class Pred, detail::enable_if_device<It, Pred> = 0> bool is_partitioned(It f, It l, Pred p) { return is_partitioned(typename detail::implicit_policy<It, Pred>::type(), f, l, p); }
template <class It, class Pred, detail::enable_if_host<It, Pred> = 0> bool is_partitioned(It f, It l, Pred p) { return is_partitioned(host, f, l, p); }
}  // namespace thrust

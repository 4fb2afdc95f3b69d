// thrust::unique / unique_copy / unique_by_key / unique_by_key_copy (thrust/unique.h;
// thrust/system/cuda/detail/unique.h, unique_by_key.h): the first element of every run of
// consecutive equal elements, in order; the in-place forms compact from a temporary copy.
#pragma once
#include <algorithm>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/pair.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/transform_reduce.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

#include <thrust/system/cdna4/detail/unique.h>
namespace thrust {
// The entry points dispatch on the policy's own type by an unqualified call (thrust/detail/unique.inl):
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class.
template <class D, class In, class Out, class Eq>
Out unique_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out out, Eq eq) {
  return unique_copy(detail::derived_cast(detail::strip_const(exec)), first, last, out, eq);
}
template <class D, class In, class Eq>
In unique(const detail::execution_policy_base<D>& exec, In first, In last, Eq eq) {
  return unique(detail::derived_cast(detail::strip_const(exec)), first, last, eq);
}
template <class D, class KIn, class VIn, class KOut, class VOut, class Eq>
pair<KOut, VOut> unique_by_key_copy(const detail::execution_policy_base<D>& exec, KIn kfirst, KIn klast, VIn vfirst, KOut kout, VOut vout, Eq eq) {
  return unique_by_key_copy(detail::derived_cast(detail::strip_const(exec)), kfirst, klast, vfirst, kout, vout, eq);
}
template <class D, class KIn, class VIn, class Eq>
pair<KIn, VIn> unique_by_key(const detail::execution_policy_base<D>& exec, KIn kfirst, KIn klast, VIn vfirst, Eq eq) {
  return unique_by_key(detail::derived_cast(detail::strip_const(exec)), kfirst, klast, vfirst, eq);
}
// ---- host
template <class In, class Out, class Eq>
Out unique_copy(const system::cpp::detail::par_t&, In first, In last, Out out, Eq eq) {
  // the last element kept is held in a variable, so that the output is only ever written
  // (thrust/system/detail/sequential/unique.h:38-66) — it may be a discard iterator
  if (first == last) return out;
  typename std::iterator_traits<In>::value_type kept = *first;
  *out = kept; ++out;
  for (++first; first != last; ++first) {
    typename std::iterator_traits<In>::value_type x = *first;
    if (!eq(kept, x)) { kept = x; *out = kept; ++out; }
  }
  return out;
}
template <class In, class Eq>
In unique(const system::cpp::detail::par_t&, In first, In last, Eq eq) { return std::unique(first, last, eq); }
template <class KIn, class VIn, class KOut, class VOut, class Eq>
pair<KOut, VOut> unique_by_key_copy(const system::cpp::detail::par_t&, KIn kfirst, KIn klast, VIn vfirst, KOut kout, VOut vout, Eq eq) {
  if (kfirst == klast) return thrust::make_pair(kout, vout);
  auto prev = *kfirst;
  *kout = prev; *vout = *vfirst; ++kout; ++vout;
  for (++kfirst, ++vfirst; kfirst != klast; ++kfirst, ++vfirst) {
    if (!eq(prev, *kfirst)) { *kout = *kfirst; *vout = *vfirst; ++kout; ++vout; }
    prev = *kfirst;
  }
  return thrust::make_pair(kout, vout);
}
template <class KIn, class VIn, class Eq>
pair<KIn, VIn> unique_by_key(const system::cpp::detail::par_t& e, KIn kfirst, KIn klast, VIn vfirst, Eq eq) {
  return unique_by_key_copy(e, kfirst, klast, vfirst, kfirst, vfirst, eq);  // outputs trail the inputs
}
// ---- default equality: the shorter forms dispatch on the policy like the full ones
// (testing/unique.cu and testing/unique_by_key.cu overload the shortest for their own policy)
template <class D, class In, class Out, class = typename std::iterator_traits<In>::iterator_category,
          class = typename std::iterator_traits<Out>::iterator_category>
Out unique_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out out) {
  return unique_copy(detail::derived_cast(detail::strip_const(exec)), first, last, out);
}
template <class D, class In, class = typename std::iterator_traits<In>::iterator_category>
In unique(const detail::execution_policy_base<D>& exec, In first, In last) {
  return unique(detail::derived_cast(detail::strip_const(exec)), first, last);
}
template <class D, class KIn, class VIn, class = typename std::iterator_traits<VIn>::iterator_category>
pair<KIn, VIn> unique_by_key(const detail::execution_policy_base<D>& exec, KIn kfirst, KIn klast, VIn vfirst) {
  return unique_by_key(detail::derived_cast(detail::strip_const(exec)), kfirst, klast, vfirst);
}
template <class D, class KIn, class VIn, class KOut, class VOut, class = typename std::iterator_traits<VOut>::iterator_category>
pair<KOut, VOut> unique_by_key_copy(const detail::execution_policy_base<D>& exec, KIn kfirst, KIn klast, VIn vfirst, KOut kout, VOut vout) {
  return unique_by_key_copy(detail::derived_cast(detail::strip_const(exec)), kfirst, klast, vfirst, kout, vout);
}
template <class In, class Out, class = typename std::iterator_traits<In>::iterator_category,
          class = typename std::iterator_traits<Out>::iterator_category>
Out unique_copy(const system::cpp::detail::par_t& exec, In first, In last, Out out) { return unique_copy(exec, first, last, out, equal_to<typename detail::value_of<In>::type>()); }
template <class In, class = typename std::iterator_traits<In>::iterator_category>
In unique(const system::cpp::detail::par_t& exec, In first, In last) { return unique(exec, first, last, equal_to<typename detail::value_of<In>::type>()); }
template <class KIn, class VIn, class = typename std::iterator_traits<VIn>::iterator_category>
pair<KIn, VIn> unique_by_key(const system::cpp::detail::par_t& exec, KIn kfirst, KIn klast, VIn vfirst) {
  return unique_by_key(exec, kfirst, klast, vfirst, equal_to<typename detail::value_of<KIn>::type>());
}
template <class KIn, class VIn, class KOut, class VOut, class = typename std::iterator_traits<VOut>::iterator_category>
pair<KOut, VOut> unique_by_key_copy(const system::cpp::detail::par_t& exec, KIn kfirst, KIn klast, VIn vfirst, KOut kout, VOut vout) {
  return unique_by_key_copy(exec, kfirst, klast, vfirst, kout, vout, equal_to<typename detail::value_of<KIn>::type>());
}
// ---- no policy
template <class In, detail::enable_if_device<In> = 0> In unique(In f, In l) { return unique(typename detail::implicit_policy<In>::type(), f, l); }
template <class In, detail::enable_if_host<In> = 0> In unique(In f, In l) { return unique(host, f, l); }
template <class In, class Eq, detail::enable_if_device<In, Eq> = 0> In unique(In f, In l, Eq eq) { return unique(typename detail::implicit_policy<In, Eq>::type(), f, l, eq); }
template <class In, class Eq, detail::enable_if_host<In, Eq> = 0> In unique(In f, In l, Eq eq) { return unique(host, f, l, eq); }
template <class In, class Out, detail::enable_if_device<In, Out> = 0> Out unique_copy(In f, In l, Out o) { return unique_copy(typename detail::implicit_policy<In, Out>::type(), f, l, o); }
template <class In, class Out, detail::enable_if_host<In, Out> = 0> Out unique_copy(In f, In l, Out o) { return unique_copy(host, f, l, o); }
template <class K, class V, detail::enable_if_device<K, V> = 0> pair<K, V> unique_by_key(K f, K l, V v) { return unique_by_key(typename detail::implicit_policy<K, V>::type(), f, l, v); }
template <class K, class V, detail::enable_if_host<K, V> = 0> pair<K, V> unique_by_key(K f, K l, V v) { return unique_by_key(host, f, l, v); }
template <class In, class Out, class Eq, detail::enable_if_device<In, Out, Eq> = 0, class = typename std::iterator_traits<Out>::iterator_category>
Out unique_copy(In f, In l, Out o, Eq eq) { return unique_copy(typename detail::implicit_policy<In, Out, Eq>::type(), f, l, o, eq); }
template <class In, class Out, class Eq, detail::enable_if_host<In, Out, Eq> = 0, class = typename std::iterator_traits<Out>::iterator_category>
Out unique_copy(In f, In l, Out o, Eq eq) { return unique_copy(host, f, l, o, eq); }
template <class K, class V, class Eq, detail::enable_if_device<K, V, Eq> = 0> pair<K, V> unique_by_key(K f, K l, V v, Eq eq) { return unique_by_key(typename detail::implicit_policy<K, V, Eq>::type(), f, l, v, eq); }
template <class K, class V, class Eq, detail::enable_if_host<K, V, Eq> = 0> pair<K, V> unique_by_key(K f, K l, V v, Eq eq) { return unique_by_key(host, f, l, v, eq); }
template <class K, class V, class KO, class VO, class Eq, detail::enable_if_device<K, V, KO, VO, Eq> = 0>
pair<KO, VO> unique_by_key_copy(K f, K l, V v, KO ko, VO vo, Eq eq) { return unique_by_key_copy(typename detail::implicit_policy<K, V, KO, VO, Eq>::type(), f, l, v, ko, vo, eq); }
template <class K, class V, class KO, class VO, class Eq, detail::enable_if_host<K, V, KO, VO, Eq> = 0>
pair<KO, VO> unique_by_key_copy(K f, K l, V v, KO ko, VO vo, Eq eq) { return unique_by_key_copy(host, f, l, v, ko, vo, eq); }
template <class K, class V, class KO, class VO, detail::enable_if_device<K, V, KO, VO> = 0>
pair<KO, VO> unique_by_key_copy(K f, K l, V v, KO ko, VO vo) { return unique_by_key_copy(typename detail::implicit_policy<K, V, KO, VO>::type(), f, l, v, ko, vo); }
template <class K, class V, class KO, class VO, detail::enable_if_host<K, V, KO, VO> = 0>
pair<KO, VO> unique_by_key_copy(K f, K l, V v, KO ko, VO vo) { return unique_by_key_copy(host, f, l, v, ko, vo); }

// ---- unique_count (thrust/unique.h:1022-1176): the number of runs of consecutive equivalent
//      elements, i.e. how many elements unique would keep — one plus the positions whose element is
//      not equivalent to the one before it, counted by a reduction over the positions
namespace detail {
template <class It, class Eq>
struct starts_a_run {
  It p; Eq eq;
  template <class Index> THRUST_CDNA4_HD std::int64_t operator()(Index i) { return eq(p[i], p[i + 1]) ? 0 : 1; }
};
}  // namespace detail
namespace detail {
template <class Policy, class It, class Eq>
typename std::iterator_traits<It>::difference_type composed_unique_count(const Policy& exec, It first, It last, Eq eq) {
  typedef typename std::iterator_traits<It>::difference_type D;
  const std::int64_t n = (std::int64_t)(last - first);
  if (n <= 0) return D(0);
  typedef detail::starts_a_run<typename detail::unwrap_iterator<It>::type, Eq> F;
  return D(1 + thrust::transform_reduce(exec, counting_iterator<std::int64_t>(0), counting_iterator<std::int64_t>(n - 1),
                                        F{detail::unwrap(first), eq}, std::int64_t(0), plus<std::int64_t>()));
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It, class Eq>
typename std::iterator_traits<It>::difference_type unique_count(execution_policy<D_>& exec, It first, It last, Eq eq) { return thrust::detail::composed_unique_count(exec, first, last, eq); }
}}  // namespace system::cdna4
template <class D_, class It, class Eq>
typename std::iterator_traits<It>::difference_type unique_count(const detail::execution_policy_base<D_>& exec, It first, It last, Eq eq) { return unique_count(detail::derived_cast(detail::strip_const(exec)), first, last, eq); }
template <class It, class Eq>
typename std::iterator_traits<It>::difference_type unique_count(const system::cpp::detail::par_t& exec, It first, It last, Eq eq) { return detail::composed_unique_count(exec, first, last, eq); }
namespace detail {
template <class Policy, class It>
typename std::iterator_traits<It>::difference_type composed_unique_count(const Policy& exec, It first, It last) {
  return unique_count(exec, first, last, equal_to<typename detail::value_of<It>::type>());
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class It>
typename std::iterator_traits<It>::difference_type unique_count(execution_policy<D_>& exec, It first, It last) { return thrust::detail::composed_unique_count(exec, first, last); }
}}  // namespace system::cdna4
template <class D_, class It>
typename std::iterator_traits<It>::difference_type unique_count(const detail::execution_policy_base<D_>& exec, It first, It last) { return unique_count(detail::derived_cast(detail::strip_const(exec)), first, last); }
template <class It>
typename std::iterator_traits<It>::difference_type unique_count(const system::cpp::detail::par_t& exec, It first, It last) { return detail::composed_unique_count(exec, first, last); }
template <class It, detail::enable_if_device<It> = 0> typename std::iterator_traits<It>::difference_type unique_count(It f, It l) { return unique_count(typename detail::implicit_policy<It>::type(), f, l); }
template <class It, detail::enable_if_host<It> = 0> typename std::iterator_traits<It>::difference_type unique_count(It f, It l) { return unique_count(host, f, l); }
template <class It, class Eq, detail::enable_if_device<It, Eq> = 0, typename std::enable_if<!detail::is_policy<It>::value, int>::type = 0>
typename std::iterator_traits<It>::difference_type unique_count(It f, It l, Eq eq) { return unique_count(typename detail::implicit_policy<It, Eq>::type(), f, l, eq); }
template <class It, class Eq, detail::enable_if_host<It, Eq> = 0, typename std::enable_if<!detail::is_policy<It>::value, int>::type = 0>
typename std::iterator_traits<It>::difference_type unique_count(It f, It l, Eq eq) { return unique_count(host, f, l, eq); }
}  // namespace thrust

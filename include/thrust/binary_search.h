// thrust::lower_bound / upper_bound / binary_search (thrust/binary_search.h;
// thrust/system/detail/generic/binary_search.inl): the vectorised forms run one search per
// thread over the sorted range; the scalar forms are a one-element vectorised search.
#pragma once
#include <algorithm>
#include <thrust/detail/iterator_util.h>
#include <thrust/device_vector.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/pair.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

namespace thrust {
namespace detail {
template <int MODE, class D, class Hay, class Needles, class Out, class Comp>
Out vector_search(const system::cdna4::execution_policy<D>& exec, Hay first, Hay last, Needles vfirst, Needles vlast, Out out, Comp comp) {
  const std::int64_t n = (std::int64_t)(vlast - vfirst);
  system::cdna4::detail::binary_search_n<MODE>(exec.derived(), unwrap(first), (std::int64_t)(last - first), unwrap(vfirst), unwrap(out), n, comp);
  return out + n;
}
template <int MODE, class Hay, class Needles, class Out, class Comp>
Out vector_search(const system::cpp::detail::par_t&, Hay first, Hay last, Needles vfirst, Needles vlast, Out out, Comp comp) {
  for (; vfirst != vlast; ++vfirst, ++out) {
    if (MODE == 0) *out = std::lower_bound(first, last, *vfirst, comp) - first;
    else if (MODE == 1) *out = std::upper_bound(first, last, *vfirst, comp) - first;
    else *out = std::binary_search(first, last, *vfirst, comp);
  }
  return out;
}
// one value: search from a one-element device vector, read the answer back
template <int MODE, class D, class Hay, class T, class Comp>
std::ptrdiff_t scalar_search(const system::cdna4::execution_policy<D>& exec, Hay first, Hay last, const T& value, Comp comp) {
  thrust::device_vector<T> needle(1, value);
  thrust::device_vector<std::ptrdiff_t> answer(1);
  vector_search<MODE>(exec, first, last, needle.begin(), needle.end(), answer.begin(), comp);
  system::cdna4::detail::throw_on_error(thrust_cdna4_stream_synchronize(system::cdna4::detail::stream_of(exec.derived())), "binary search");
  return answer[0];
}
template <int MODE, class Hay, class T, class Comp>
std::ptrdiff_t scalar_search(const system::cpp::detail::par_t&, Hay first, Hay last, const T& value, Comp comp) {
  if (MODE == 0) return std::lower_bound(first, last, value, comp) - first;
  if (MODE == 1) return std::upper_bound(first, last, value, comp) - first;
  return std::binary_search(first, last, value, comp);
}
}  // namespace detail

// Without a comparator the elements and the values are compared as they are, by the transparent
// less (thrust/system/detail/generic/binary_search.inl: `_1 < _2`), not converted to one type first.
#define THRUST_CDNA4_SEARCH(NAME, MODE)                                                                                  \
  namespace system { namespace cdna4 {                                                                                  \
  template <class D, class Hay, class Needles, class Out, class Comp>                                                    \
  Out NAME(execution_policy<D>& exec, Hay first, Hay last, Needles vfirst, Needles vlast, Out out, Comp comp) {          \
    return thrust::detail::vector_search<MODE>(exec.derived(), first, last, vfirst, vlast, out, comp);                   \
  }                                                                                                                      \
  template <class D, class Hay, class Needles, class Out>                                                                \
  Out NAME(execution_policy<D>& exec, Hay first, Hay last, Needles vfirst, Needles vlast, Out out) {                     \
    return NAME(exec, first, last, vfirst, vlast, out, thrust::less<>());                                                \
  }                                                                                                                      \
  }}                                                                                                                     \
  template <class D, class Hay, class Needles, class Out, class Comp>                                                    \
  Out NAME(const detail::execution_policy_base<D>& exec, Hay first, Hay last, Needles vfirst, Needles vlast, Out out, Comp comp) { \
    return NAME(detail::derived_cast(detail::strip_const(exec)), first, last, vfirst, vlast, out, comp);                 \
  }                                                                                                                      \
  template <class D, class Hay, class Needles, class Out>                                                                \
  Out NAME(const detail::execution_policy_base<D>& exec, Hay first, Hay last, Needles vfirst, Needles vlast, Out out) {  \
    return NAME(detail::derived_cast(detail::strip_const(exec)), first, last, vfirst, vlast, out);                       \
  }                                                                                                                      \
  template <class Hay, class Needles, class Out, class Comp>                                                             \
  Out NAME(const system::cpp::detail::par_t& exec, Hay first, Hay last, Needles vfirst, Needles vlast, Out out, Comp comp) { \
    return detail::vector_search<MODE>(exec, first, last, vfirst, vlast, out, comp);                                     \
  }                                                                                                                      \
  template <class Hay, class Needles, class Out>                                                                         \
  Out NAME(const system::cpp::detail::par_t& exec, Hay first, Hay last, Needles vfirst, Needles vlast, Out out) {        \
    return detail::vector_search<MODE>(exec, first, last, vfirst, vlast, out, less<>());                                 \
  }                                                                                                                      \
  template <class Hay, class Needles, class Out, detail::enable_if_device<Hay, Needles, Out> = 0,                                      \
            class = typename std::iterator_traits<Out>::iterator_category>                                               \
  Out NAME(Hay f, Hay l, Needles vf, Needles vl, Out o) { return NAME(typename detail::implicit_policy<Hay, Needles, Out>::type(), f, l, vf, vl, o); }                        \
  template <class Hay, class Needles, class Out, detail::enable_if_host<Hay, Needles, Out> = 0,                                        \
            class = typename std::iterator_traits<Out>::iterator_category>                                               \
  Out NAME(Hay f, Hay l, Needles vf, Needles vl, Out o) { return NAME(host, f, l, vf, vl, o); }                          \
  template <class Hay, class Needles, class Out, class Comp, detail::enable_if_device<Hay, Needles, Out, Comp> = 0,                          \
            class = typename std::iterator_traits<Out>::iterator_category>                                               \
  Out NAME(Hay f, Hay l, Needles vf, Needles vl, Out o, Comp c) { return NAME(typename detail::implicit_policy<Hay, Needles, Out, Comp>::type(), f, l, vf, vl, o, c); }             \
  template <class Hay, class Needles, class Out, class Comp, detail::enable_if_host<Hay, Needles, Out, Comp> = 0,                            \
            class = typename std::iterator_traits<Out>::iterator_category>                                               \
  Out NAME(Hay f, Hay l, Needles vf, Needles vl, Out o, Comp c) { return NAME(host, f, l, vf, vl, o, c); }
THRUST_CDNA4_SEARCH(lower_bound, 0)
THRUST_CDNA4_SEARCH(upper_bound, 1)
THRUST_CDNA4_SEARCH(binary_search, 2)
#undef THRUST_CDNA4_SEARCH

// scalar forms: an iterator for the bounds, a bool for binary_search
// (the forms with a policy dispatch on the policy's own type by an unqualified call, thrust/detail/binary_search.inl:
// a user's overload for a policy type derived from thrust::device_execution_policy is preferred to
// the device system's, which is found through the policy's base class)
#define THRUST_CDNA4_SCALAR_BOUND(NAME, MODE)                                                                            \
  namespace system { namespace cdna4 {                                                                                  \
  template <class D, class Hay, class T, class Comp>                                                                     \
  Hay NAME(execution_policy<D>& exec, Hay first, Hay last, const T& value, Comp comp) {                                  \
    return first + thrust::detail::scalar_search<MODE>(exec.derived(), first, last, value, comp);                        \
  }                                                                                                                      \
  template <class D, class Hay, class T>                                                                                 \
  Hay NAME(execution_policy<D>& exec, Hay first, Hay last, const T& value) { return NAME(exec, first, last, value, thrust::less<>()); } \
  }}                                                                                                                     \
  template <class D, class Hay, class T, class Comp>                                                                     \
  Hay NAME(const detail::execution_policy_base<D>& exec, Hay first, Hay last, const T& value, Comp comp) {               \
    return NAME(detail::derived_cast(detail::strip_const(exec)), first, last, value, comp);                              \
  }                                                                                                                      \
  template <class D, class Hay, class T>                                                                                 \
  Hay NAME(const detail::execution_policy_base<D>& exec, Hay first, Hay last, const T& value) {                          \
    return NAME(detail::derived_cast(detail::strip_const(exec)), first, last, value);                                    \
  }                                                                                                                      \
  template <class Hay, class T, class Comp>                                                                              \
  Hay NAME(const system::cpp::detail::par_t& exec, Hay first, Hay last, const T& value, Comp comp) {                     \
    return first + detail::scalar_search<MODE>(exec, first, last, value, comp);                                          \
  }                                                                                                                      \
  template <class Hay, class T>                                                                                          \
  Hay NAME(const system::cpp::detail::par_t& exec, Hay first, Hay last, const T& value) { return NAME(exec, first, last, value, less<>()); } \
  template <class Hay, class T, detail::enable_if_device<Hay, T> = 0> Hay NAME(Hay f, Hay l, const T& v) { return NAME(typename detail::implicit_policy<Hay, T>::type(), f, l, v); } \
  template <class Hay, class T, detail::enable_if_host<Hay, T> = 0> Hay NAME(Hay f, Hay l, const T& v) { return NAME(host, f, l, v); } \
  template <class Hay, class T, class Comp, detail::enable_if_device<Hay, T> = 0,                                        \
            typename std::enable_if<!detail::is_policy<Hay>::value, int>::type = 0>                                     \
  Hay NAME(Hay f, Hay l, const T& v, Comp c) { return NAME(typename detail::implicit_policy<Hay, T>::type(), f, l, v, c); } \
  template <class Hay, class T, class Comp, detail::enable_if_host<Hay, T> = 0,                                          \
            typename std::enable_if<!detail::is_policy<Hay>::value, int>::type = 0>                                     \
  Hay NAME(Hay f, Hay l, const T& v, Comp c) { return NAME(host, f, l, v, c); }
THRUST_CDNA4_SCALAR_BOUND(lower_bound, 0)
THRUST_CDNA4_SCALAR_BOUND(upper_bound, 1)
#undef THRUST_CDNA4_SCALAR_BOUND
namespace system { namespace cdna4 {
template <class D, class Hay, class T, class Comp>
bool binary_search(execution_policy<D>& exec, Hay first, Hay last, const T& value, Comp comp) {
  return thrust::detail::scalar_search<2>(exec.derived(), first, last, value, comp) != 0;
}
template <class D, class Hay, class T>
bool binary_search(execution_policy<D>& exec, Hay first, Hay last, const T& value) { return binary_search(exec, first, last, value, thrust::less<>()); }
}}  // namespace system::cdna4
template <class D, class Hay, class T, class Comp>
bool binary_search(const detail::execution_policy_base<D>& exec, Hay first, Hay last, const T& value, Comp comp) {
  return binary_search(detail::derived_cast(detail::strip_const(exec)), first, last, value, comp);
}
template <class D, class Hay, class T>
bool binary_search(const detail::execution_policy_base<D>& exec, Hay first, Hay last, const T& value) {
  return binary_search(detail::derived_cast(detail::strip_const(exec)), first, last, value);
}
template <class Hay, class T, class Comp>
bool binary_search(const system::cpp::detail::par_t& exec, Hay first, Hay last, const T& value, Comp comp) {
  return detail::scalar_search<2>(exec, first, last, value, comp) != 0;
}
template <class Hay, class T>
bool binary_search(const system::cpp::detail::par_t& exec, Hay first, Hay last, const T& value) { return binary_search(exec, first, last, value, less<>()); }
template <class Hay, class T, detail::enable_if_device<Hay, T> = 0> bool binary_search(Hay f, Hay l, const T& v) { return binary_search(typename detail::implicit_policy<Hay, T>::type(), f, l, v); }
template <class Hay, class T, detail::enable_if_host<Hay, T> = 0> bool binary_search(Hay f, Hay l, const T& v) { return binary_search(host, f, l, v); }
template <class Hay, class T, class Comp, detail::enable_if_device<Hay, T> = 0, typename std::enable_if<!detail::is_policy<Hay>::value, int>::type = 0>
bool binary_search(Hay f, Hay l, const T& v, Comp c) { return binary_search(typename detail::implicit_policy<Hay, T>::type(), f, l, v, c); }
template <class Hay, class T, class Comp, detail::enable_if_host<Hay, T> = 0, typename std::enable_if<!detail::is_policy<Hay>::value, int>::type = 0>
bool binary_search(Hay f, Hay l, const T& v, Comp c) { return binary_search(host, f, l, v, c); }

// ---- equal_range (thrust/binary_search.h:727-1017): the pair (lower_bound, upper_bound) of one value
namespace detail {
template <class Policy, class Hay, class T, class Comp>
pair<Hay, Hay> composed_equal_range(const Policy& exec, Hay first, Hay last, const T& value, Comp comp) {
  const Hay lo = thrust::lower_bound(exec, first, last, value, comp);
  return pair<Hay, Hay>(lo, thrust::upper_bound(exec, lo, last, value, comp));
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D, class Hay, class T, class Comp>
pair<Hay, Hay> equal_range(execution_policy<D>& exec, Hay first, Hay last, const T& value, Comp comp) {
  return thrust::detail::composed_equal_range(exec.derived(), first, last, value, comp);
}
template <class D, class Hay, class T>
pair<Hay, Hay> equal_range(execution_policy<D>& exec, Hay first, Hay last, const T& value) { return equal_range(exec, first, last, value, thrust::less<>()); }
}}  // namespace system::cdna4
template <class D, class Hay, class T, class Comp>
pair<Hay, Hay> equal_range(const detail::execution_policy_base<D>& exec, Hay first, Hay last, const T& value, Comp comp) {
  return equal_range(detail::derived_cast(detail::strip_const(exec)), first, last, value, comp);
}
template <class D, class Hay, class T>
pair<Hay, Hay> equal_range(const detail::execution_policy_base<D>& exec, Hay first, Hay last, const T& value) {
  return equal_range(detail::derived_cast(detail::strip_const(exec)), first, last, value);
}
template <class Hay, class T, class Comp>
pair<Hay, Hay> equal_range(const system::cpp::detail::par_t& exec, Hay first, Hay last, const T& value, Comp comp) {
  return detail::composed_equal_range(exec, first, last, value, comp);
}
template <class Hay, class T>
pair<Hay, Hay> equal_range(const system::cpp::detail::par_t& exec, Hay first, Hay last, const T& value) { return equal_range(exec, first, last, value, less<>()); }
template <class Hay, class T, detail::enable_if_device<Hay, T> = 0> pair<Hay, Hay> equal_range(Hay f, Hay l, const T& v) { return equal_range(typename detail::implicit_policy<Hay, T>::type(), f, l, v); }
template <class Hay, class T, detail::enable_if_host<Hay, T> = 0> pair<Hay, Hay> equal_range(Hay f, Hay l, const T& v) { return equal_range(host, f, l, v); }
template <class Hay, class T, class Comp, detail::enable_if_device<Hay, T, Comp> = 0, typename std::enable_if<!detail::is_policy<Hay>::value, int>::type = 0>
pair<Hay, Hay> equal_range(Hay f, Hay l, const T& v, Comp c) { return equal_range(typename detail::implicit_policy<Hay, T, Comp>::type(), f, l, v, c); }
template <class Hay, class T, class Comp, detail::enable_if_host<Hay, T, Comp> = 0, typename std::enable_if<!detail::is_policy<Hay>::value, int>::type = 0>
pair<Hay, Hay> equal_range(Hay f, Hay l, const T& v, Comp c) { return equal_range(host, f, l, v, c); }
}  // namespace thrust

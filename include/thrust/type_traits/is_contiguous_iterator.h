// thrust::is_contiguous_iterator, proclaim_contiguous_iterator and
// THRUST_PROCLAIM_CONTIGUOUS_ITERATOR (thrust/type_traits/is_contiguous_iterator.h): iterators
// whose elements lie next to each other in memory — raw pointers, thrust::device_ptr, the
// iterators of std::vector / std::string / thrust::host_vector / thrust::device_vector, and
// whatever a user proclaims.
#pragma once
#include <iterator>
#include <string>
#include <type_traits>
#include <vector>
#include <thrust/device_ptr.h>
#include <thrust/iterator/detail/normal_iterator.h>
namespace thrust {
template <class Iterator> struct proclaim_contiguous_iterator : std::false_type {};
#define THRUST_PROCLAIM_CONTIGUOUS_ITERATOR(Iterator) \
  namespace thrust { template <> struct proclaim_contiguous_iterator<Iterator> : std::true_type {}; }
namespace detail {
template <class It> struct is_contiguous_iterator_impl : proclaim_contiguous_iterator<It> {};
template <class T> struct is_contiguous_iterator_impl<T*> : std::true_type {};
template <class T> struct is_contiguous_iterator_impl<thrust::device_ptr<T>> : std::true_type {};
// libstdc++'s vector and string iterators wrap a raw pointer
template <class P, class C> struct is_contiguous_iterator_impl<__gnu_cxx::__normal_iterator<P, C>> : std::is_pointer<P> {};
// thrust::host_vector's iterators wrap a raw pointer too
template <class P> struct is_contiguous_iterator_impl<normal_iterator<P>> : std::is_pointer<P> {};
}  // namespace detail
template <class Iterator> struct is_contiguous_iterator : detail::is_contiguous_iterator_impl<typename std::remove_cv<Iterator>::type> {};
// the raw pointer behind a contiguous iterator, any other iterator as it is
// (thrust/type_traits/is_contiguous_iterator.h:160-230)
namespace detail {
template <class T> THRUST_CDNA4_HD inline T* contiguous_raw(T* p) { return p; }
template <class T> THRUST_CDNA4_HD inline T* contiguous_raw(thrust::device_ptr<T> p) { return p.get(); }
template <class P> THRUST_CDNA4_HD inline P contiguous_raw(normal_iterator<P> it) { return it.base(); }
template <class P, class C> inline P contiguous_raw(__gnu_cxx::__normal_iterator<P, C> it) { return it.base(); }
template <class It> struct contiguous_iterator_raw_pointer { typedef decltype(contiguous_raw(std::declval<It>())) type; };
template <class It> using contiguous_iterator_raw_pointer_t = typename contiguous_iterator_raw_pointer<It>::type;
template <class It> THRUST_CDNA4_HD inline contiguous_iterator_raw_pointer_t<It> contiguous_iterator_raw_pointer_cast(It it) { return contiguous_raw(it); }
template <class It, bool = thrust::is_contiguous_iterator<It>::value> struct try_unwrap_contiguous_iterator_return { typedef It type; };
template <class It> struct try_unwrap_contiguous_iterator_return<It, true> { typedef contiguous_iterator_raw_pointer_t<It> type; };
template <class It> using try_unwrap_contiguous_iterator_return_t = typename try_unwrap_contiguous_iterator_return<It>::type;
template <class It> THRUST_CDNA4_HD inline It try_unwrap_contiguous_iterator_impl(It it, std::false_type) { return it; }
template <class It> THRUST_CDNA4_HD inline contiguous_iterator_raw_pointer_t<It> try_unwrap_contiguous_iterator_impl(It it, std::true_type) { return contiguous_raw(it); }
template <class It> THRUST_CDNA4_HD inline try_unwrap_contiguous_iterator_return_t<It> try_unwrap_contiguous_iterator(It it) {
  return try_unwrap_contiguous_iterator_impl(it, std::integral_constant<bool, thrust::is_contiguous_iterator<It>::value>());
}
}  // namespace detail
#if __cplusplus >= 201402L
template <class Iterator> constexpr bool is_contiguous_iterator_v = is_contiguous_iterator<Iterator>::value;
#endif
}  // namespace thrust

// An allocator's own construct() (thrust/detail/allocator/allocator_traits.h: construct1 / construct2;
// testing/allocator.cu:10-63): device_vector moves bytes and constructs nothing by itself, but an
// allocator that DEFINES construct(T*) or construct(T*, const Arg&) is asked to construct every
// element the vector creates — on the device, where the elements live.  Allocators without such a
// member (the device system's own) cost nothing here.
#pragma once
#include <cstdint>
#include <type_traits>
#include <utility>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/index_algorithms.h>

namespace thrust {
namespace detail {
template <class A, class T, class = void> struct has_construct1 : std::false_type {};
template <class A, class T>
struct has_construct1<A, T, decltype(void(std::declval<A&>().construct(std::declval<T*>())))> : std::true_type {};
template <class A, class T, class Arg, class = void> struct has_construct2 : std::false_type {};
template <class A, class T, class Arg>
struct has_construct2<A, T, Arg, decltype(void(std::declval<A&>().construct(std::declval<T*>(), std::declval<const Arg&>())))> : std::true_type {};

template <class A, class T> struct construct1_body {
  mutable A alloc;
  T* p;
  THRUST_CDNA4_HD void operator()(std::int64_t i) const { alloc.construct(p + i); }
};
template <class A, class T, class Arg> struct construct2_body {
  mutable A alloc;
  T* p;
  const Arg* from;
  THRUST_CDNA4_HD void operator()(std::int64_t i) const { alloc.construct(p + i, from[i]); }
};

// elements [p, p + n) created without a value
template <class A, class T>
typename std::enable_if<has_construct1<A, T>::value>::type allocator_default_construct(A& alloc, T* p, std::size_t n) {
  if (n) system::cdna4::detail::for_each_index(thrust::device, (std::int64_t)n, construct1_body<A, T>{alloc, p}, "device_vector: construct");
}
template <class A, class T>
typename std::enable_if<!has_construct1<A, T>::value>::type allocator_default_construct(A&, T*, std::size_t) {}
// elements [p, p + n) created as copies of the device range [from, from + n)
template <class A, class T, class Arg>
typename std::enable_if<has_construct2<A, T, Arg>::value>::type allocator_copy_construct(A& alloc, T* p, const Arg* from, std::size_t n) {
  if (n) system::cdna4::detail::for_each_index(thrust::device, (std::int64_t)n, construct2_body<A, T, Arg>{alloc, p, from}, "device_vector: construct");
}
template <class A, class T, class Arg>
typename std::enable_if<!has_construct2<A, T, Arg>::value>::type allocator_copy_construct(A&, T*, const Arg*, std::size_t) {}
}  // namespace detail
}  // namespace thrust

// <thrust/detail/allocator/allocator_traits.h>: thrust::detail::allocator_traits — the standard
// allocator traits (nested types with their defaults, rebinding, allocate / deallocate /
// construct / destroy / max_size through the allocator's own members where it has them), plus
// allocator_system: the system of the memory an allocator hands out
// (thrust/detail/allocator/allocator_traits.h:248-440).
#pragma once
#include <memory>
#include <type_traits>
#include <thrust/detail/config.h>
#include <thrust/detail/type_traits/pointer_traits.h>
#include <thrust/iterator/iterator_traits.h>
namespace thrust { namespace detail {
template <class Alloc>
struct allocator_traits : std::allocator_traits<Alloc> {
  typedef std::allocator_traits<Alloc> base;
  typedef Alloc allocator_type;
  typedef typename base::value_type& reference;
  typedef const typename base::value_type& const_reference;
  template <class U> using rebind_alloc = typename base::template rebind_alloc<U>;
  // the traits of the rebound allocator; `other` names a traits class itself, so that both
  // rebind_traits<U> and the older spelling rebind_traits<U>::other give it
  template <class U> using rebind_traits = allocator_traits<typename base::template rebind_alloc<U>>;
  typedef allocator_traits other;
  // the allocator as it should be passed on: a reference when it has state, else a fresh object
  typedef typename std::conditional<std::is_empty<Alloc>::value, Alloc, Alloc&>::type get_result_type;
  static get_result_type get(Alloc& a) { return a; }
};
// the system of an allocator's pointer (device_ptr and tagged pointers: theirs; raw pointers: the host)
template <class Alloc>
struct allocator_system {
  typedef typename thrust::iterator_system<typename std::allocator_traits<Alloc>::pointer>::type type;
  typedef type get_result_type;
  static get_result_type get(Alloc&) { return type(); }
};
}}  // namespace thrust::detail

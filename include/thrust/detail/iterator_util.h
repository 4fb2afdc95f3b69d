// Helpers shared by the public algorithm headers: unwrap contiguous device iterators and
// classify an iterator as device or host.
#pragma once
#include <iterator>
#include <type_traits>
#include <thrust/device_ptr.h>
namespace thrust { namespace detail {
// What a kernel receives for an iterator: device_ptr<T> becomes T*, a fancy iterator the same
// iterator over unwrapped bases, anything else (a raw device pointer under an explicit device
// policy, a counting iterator, a user's own device iterator) itself.
template <class It> struct unwrap_iterator {
  typedef It type;
  static type apply(It it) { return it; }
};
template <class T> struct unwrap_iterator<thrust::device_ptr<T>> {
  typedef T* type;
  static type apply(thrust::device_ptr<T> p) { return p.get(); }
};
template <class It> inline typename unwrap_iterator<It>::type unwrap(It it) { return unwrap_iterator<It>::apply(it); }
template <class It> struct value_of { typedef typename std::iterator_traits<It>::value_type type; };
// Which overload of an algorithm called without a policy applies, from the types of its arguments:
// the first iterator that walks memory decides (counting / constant / discard iterators and
// arguments that are no iterators do not); with none, the device.
template <class... Args> using enable_if_device = typename std::enable_if<system::cdna4::detail::runs_on_device<Args...>::value, int>::type;
template <class... Args> using enable_if_host = typename std::enable_if<!system::cdna4::detail::runs_on_device<Args...>::value, int>::type;
// an execution policy of either system (tells policy-first overloads from iterator-first ones)
template <class P> struct is_policy {
  static constexpr bool value = std::is_base_of<system::cdna4::execution_policy<P>, P>::value || std::is_same<P, system::cpp::detail::par_t>::value;
};
template <class P> using enable_if_policy = typename std::enable_if<is_policy<P>::value, int>::type;
// The policy an algorithm called WITHOUT one runs under, from its first iterator's system
// (thrust/detail/sort.inl:202-215: `System system; sort(select_system(system), ...)`): the device
// system's default policy — or, for an iterator retagged with a user's policy type
// (thrust::retag<my_tag>(it), my_tag derived from thrust::device_execution_policy<my_tag>), a
// default-constructed object of that type, so that the user's overloads for it are found.
template <class Iterator, class Tag> class tagged_iterator;
template <class... Args> struct implicit_policy { typedef system::cdna4::detail::par_t type; };
template <class A, class... R> struct implicit_policy<A, R...> : implicit_policy<R...> {};
template <class I, class Tag, class... R> struct implicit_policy<tagged_iterator<I, Tag>, R...> {
  typedef typename std::conditional<std::is_base_of<system::cdna4::execution_policy<Tag>, Tag>::value, Tag,
                                    typename implicit_policy<R...>::type>::type type;
};
}}  // namespace thrust::detail
// For macros that stamp out the no-policy forms of an algorithm for both systems: the policy
// object of the form, from the types of its iterator arguments.
#define THRUST_CDNA4_DEVICE_SYS(...) typename ::thrust::detail::implicit_policy<__VA_ARGS__>::type()
#define THRUST_CDNA4_HOST_SYS(...) ::thrust::host

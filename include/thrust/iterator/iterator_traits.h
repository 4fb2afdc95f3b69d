// thrust::iterator_traits and friends (thrust/iterator/iterator_traits.h): the standard traits,
// plus iterator_system: the system tag of the memory an iterator walks.
#pragma once
#include <iterator>
#include <thrust/device_ptr.h>
namespace thrust {
// A class template of its own, so that user code can specialise it for an iterator of theirs
// (testing/scan.cu:649-656 does, for an output-only iterator); unspecialised it is the standard one.
template <class It> struct iterator_traits : std::iterator_traits<It> {};
template <class It> struct iterator_value { typedef typename iterator_traits<It>::value_type type; };
template <class It> struct iterator_pointer { typedef typename iterator_traits<It>::pointer type; };
template <class It> struct iterator_difference { typedef typename iterator_traits<It>::difference_type type; };
template <class It> struct iterator_reference { typedef typename iterator_traits<It>::reference type; };
template <class It> struct iterator_traversal { typedef typename iterator_traits<It>::iterator_category type; };
template <class It> using iterator_value_t = typename iterator_value<It>::type;
template <class It> using iterator_pointer_t = typename iterator_pointer<It>::type;
template <class It> using iterator_difference_t = typename iterator_difference<It>::type;
template <class It> using iterator_reference_t = typename iterator_reference<It>::type;
template <class It> using iterator_traversal_t = typename iterator_traversal<It>::type;
// device iterators (device_ptr and the fancy iterators over it) belong to the cdna4 system,
// everything else to the host (sequential) system
template <class It> struct iterator_system {
  typedef typename std::conditional<system::cdna4::detail::is_device_iterator<It>::value, device_system_tag, host_system_tag>::type type;
};
template <class It> using iterator_system_t = typename iterator_system<It>::type;
}  // namespace thrust

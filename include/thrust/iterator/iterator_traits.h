// thrust::iterator_traits and friends (thrust/iterator/iterator_traits.h): the standard traits.
#pragma once
#include <iterator>
namespace thrust {
template <class It> using iterator_traits = std::iterator_traits<It>;
template <class It> struct iterator_value { typedef typename std::iterator_traits<It>::value_type type; };
template <class It> struct iterator_difference { typedef typename std::iterator_traits<It>::difference_type type; };
template <class It> struct iterator_reference { typedef typename std::iterator_traits<It>::reference type; };
template <class It> using iterator_value_t = typename iterator_value<It>::type;
template <class It> using iterator_difference_t = typename iterator_difference<It>::type;
}  // namespace thrust

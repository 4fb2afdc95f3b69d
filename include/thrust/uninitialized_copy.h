// thrust::uninitialized_copy / uninitialized_copy_n (thrust/uninitialized_copy.h).  Device ranges
// hold trivially copyable elements, for which construction is assignment.
#pragma once
#include <memory>
#include <thrust/copy.h>
namespace thrust {
template <class D, class In, class Out>
Out uninitialized_copy(const system::cdna4::execution_policy<D>& exec, In first, In last, Out result) { return copy(exec, first, last, result); }
template <class In, class Out>
Out uninitialized_copy(const system::cpp::detail::par_t&, In first, In last, Out result) { return std::uninitialized_copy(first, last, result); }
template <class Policy, class In, class Size, class Out, detail::enable_if_policy<Policy> = 0>
Out uninitialized_copy_n(const Policy& exec, In first, Size n, Out result) { return uninitialized_copy(exec, first, first + n, result); }
template <class In, class Out> Out uninitialized_copy(In f, In l, Out o) { return copy(f, l, o); }
template <class In, class Size, class Out, class = typename std::iterator_traits<In>::iterator_category>
Out uninitialized_copy_n(In f, Size n, Out o) { return copy(f, f + n, o); }
}  // namespace thrust

// <thrust/detail/alignment.h>: alignment queries and aligned storage under thrust::detail
// (thrust/detail/alignment.h:44-230).
#pragma once
#include <thrust/detail/config.h>
#include <thrust/detail/type_traits.h>
#include <cstddef>
#include <type_traits>
namespace thrust { namespace detail {
template <class T> using alignment_of = std::alignment_of<T>;
// an empty type whose alignment is Align (a power of two)
template <std::size_t Align> struct aligned_type { struct alignas(Align) type {}; };
template <std::size_t Len, std::size_t Align> struct aligned_storage {
  union type { unsigned char bytes[Len]; typename aligned_type<Align>::type align; };
};
using max_align_t = std::max_align_t;
// reinterpret_cast through void*, for pointers the caller knows to be aligned for T
template <class T, class U> THRUST_HOST_DEVICE T aligned_reinterpret_cast(U u) {
  return reinterpret_cast<T>(reinterpret_cast<void*>(u));
}
THRUST_HOST_DEVICE inline std::size_t aligned_storage_size(std::size_t n, std::size_t align) {
  return ((n + align - 1) / align) * align;
}
}}  // namespace thrust::detail

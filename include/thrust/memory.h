// <thrust/memory.h>: pointer casts and raw memory helpers for the device system
// (raw_pointer_cast, raw_reference_cast, device_malloc / device_free through the pool).
#pragma once
#include <thrust/detail/raw_reference_cast.h>
#include <thrust/device_free.h>
#include <thrust/device_malloc.h>
#include <thrust/device_ptr.h>
#include <thrust/detail/pointer.h>
#include <cstdlib>
#include <thrust/pair.h>
#include <thrust/system/cdna4/detail/malloc_and_free.h>
#include <thrust/system/cdna4/detail/temporary_buffer.h>

// thrust::malloc / free / get_temporary_buffer / return_temporary_buffer with a policy
// (thrust/memory.h:203-395): memory of the policy's system.  They dispatch on the policy's own type,
// so a policy type derived from thrust::device_execution_policy can bring its own (the documented way
// to customise temporary allocation, examples/cuda/custom_temporary_allocation.cu:168-176 — the
// algorithms of this build take their temporaries through thrust::device(allocator) instead).
namespace thrust {
template <class D>
device_ptr<void> malloc(const detail::execution_policy_base<D>& exec, std::size_t n) {
  return device_ptr<void>(thrust::raw_pointer_cast(malloc(detail::derived_cast(detail::strip_const(exec)), n)));
}
template <class T, class D>
device_ptr<T> malloc(const detail::execution_policy_base<D>& exec, std::size_t n) {
  return device_ptr<T>(static_cast<T*>(thrust::raw_pointer_cast(thrust::malloc(exec, n * sizeof(T)))));
}
template <class D, class Pointer>
void free(const detail::execution_policy_base<D>& exec, Pointer ptr) { free(detail::derived_cast(detail::strip_const(exec)), ptr); }
template <class T, class D>
pair<device_ptr<T>, std::ptrdiff_t> get_temporary_buffer(const detail::execution_policy_base<D>& exec, std::ptrdiff_t n) {
  using system::cdna4::get_temporary_buffer;  // makes the name a template here; the call below still looks in the policy's namespaces
  return get_temporary_buffer<T>(detail::derived_cast(detail::strip_const(exec)), n);
}
template <class D, class Pointer>
void return_temporary_buffer(const detail::execution_policy_base<D>& exec, Pointer p, std::ptrdiff_t n) {
  return_temporary_buffer(detail::derived_cast(detail::strip_const(exec)), p, n);
}
// the host system
inline void* malloc(const system::cpp::detail::par_t&, std::size_t n) { return std::malloc(n); }
template <class T> inline T* malloc(const system::cpp::detail::par_t&, std::size_t n) { return static_cast<T*>(std::malloc(n * sizeof(T))); }
inline void free(const system::cpp::detail::par_t&, void* p) { std::free(p); }
template <class T>
inline pair<T*, std::ptrdiff_t> get_temporary_buffer(const system::cpp::detail::par_t&, std::ptrdiff_t n) {
  T* p = n > 0 ? static_cast<T*>(std::malloc((std::size_t)n * sizeof(T))) : nullptr;
  return pair<T*, std::ptrdiff_t>(p, p ? n : 0);
}
inline void return_temporary_buffer(const system::cpp::detail::par_t&, void* p, std::ptrdiff_t) { std::free(p); }
}  // namespace thrust

// Core of the cdna4 device system: execution policies, error mapping, element-type traits
// and temporary storage.  Everything here is host code that calls the C ABI of
// libthrust_cdna4.so; a translation unit that includes it builds with a plain C++14 host
// compiler, no device compiler needed.
//
// Mirrors, for this system:
//   thrust/system/cuda/detail/execution_policy.h:48-71   (tag, execution_policy<Derived>)
//   thrust/system/cuda/detail/par.h:44-238               (par, par.on(stream), par_nosync)
//   thrust/system/cuda/detail/util.h:46-140, :207-292    (stream(), synchronize_optional(), throw_on_error())
//   thrust/system/cuda/detail/malloc_and_free.h:53-116   (malloc / free)
//   thrust/detail/temporary_array.h:50-111               (algorithm-scoped temporary storage)
#pragma once

#include <cassert>
#include <cstddef>
#include <utility>
#include <cstdint>
#include <new>
#include <string>
#include <system_error>
#include <type_traits>

#include "thrust_cdna4.h"

#define THRUST_CDNA4_SYSTEM 1
// The version of the API surface this layer mirrors (Thrust 2.2.0).
#define THRUST_VERSION 200200
// Device system selection, as in thrust/detail/config/device_system.h:20-43: the reference's four
// ids keep their values, this system is the fifth and the default.  A build that names another
// device system with -DTHRUST_DEVICE_SYSTEM=... is refused: this tree holds one.
#define THRUST_DEVICE_SYSTEM_CUDA 1
#define THRUST_DEVICE_SYSTEM_OMP 2
#define THRUST_DEVICE_SYSTEM_TBB 3
#define THRUST_DEVICE_SYSTEM_CPP 4
#define THRUST_DEVICE_SYSTEM_CDNA4 5
#ifndef THRUST_DEVICE_SYSTEM
#define THRUST_DEVICE_SYSTEM THRUST_DEVICE_SYSTEM_CDNA4
#endif
#if THRUST_DEVICE_SYSTEM != THRUST_DEVICE_SYSTEM_CDNA4
#error "this Thrust tree provides the cdna4 device system only: build with -DTHRUST_DEVICE_SYSTEM=THRUST_DEVICE_SYSTEM_CDNA4 (5), or leave THRUST_DEVICE_SYSTEM undefined"
#endif
#define __THRUST_DEVICE_SYSTEM_NAMESPACE cdna4
#define __THRUST_DEVICE_SYSTEM_ROOT thrust/system/__THRUST_DEVICE_SYSTEM_NAMESPACE
// the host system is the sequential one (THRUST_HOST_SYSTEM_CPP of thrust/detail/config/host_system.h)
#define THRUST_HOST_SYSTEM_CPP 1
#define THRUST_HOST_SYSTEM_OMP 2
#define THRUST_HOST_SYSTEM_TBB 3
#ifndef THRUST_HOST_SYSTEM
#define THRUST_HOST_SYSTEM THRUST_HOST_SYSTEM_CPP
#endif
#if THRUST_HOST_SYSTEM != THRUST_HOST_SYSTEM_CPP
#error "this Thrust tree provides the sequential (CPP) host system only"
#endif

namespace thrust {

// ------------------------------------------------------------------------------------
// Errors: thrust::system_error with a hip error category; thrust::system::detail::bad_alloc
// for allocation failures (thrust/system/cuda/detail/malloc_and_free.h:79-83).
// ------------------------------------------------------------------------------------
using system_error = std::system_error;
using error_code = std::error_code;
using error_category = std::error_category;

namespace system {
namespace detail {
class bad_alloc : public std::bad_alloc {
 public:
  explicit bad_alloc(const std::string& w) : what_("std::bad_alloc: " + w) {}
  const char* what() const noexcept override { return what_.c_str(); }

 private:
  std::string what_;
};
}  // namespace detail

namespace cdna4 {
namespace detail {
class hip_error_category : public std::error_category {
 public:
  const char* name() const noexcept override { return "cdna4"; }
  std::string message(int ev) const override { return thrust_cdna4_error_string(ev); }
};
}  // namespace detail
}  // namespace cdna4
}  // namespace system

inline const error_category& cdna4_category() {
  static system::cdna4::detail::hip_error_category cat;
  return cat;
}

namespace detail {
// The element, key, value and accumulator types the device algorithms accept: those that may be
// moved as bytes between host and device and through kernel arguments.  A trivially copyable type
// is one; so is a number-like struct whose copy operations are written out but whose destructor is
// trivial (the reference's own tests use such a type, testing/unittest/testframework.h:128-232):
// its copy operations run where a kernel copies an element, and not where bytes are moved.
template <class T> struct is_bytewise_movable
    : std::integral_constant<bool, std::is_trivially_copyable<T>::value || std::is_trivially_destructible<T>::value> {};

// The root of every execution policy (thrust/detail/execution_policy.h): the public entry points
// that dispatch to a system's implementation take it, so that an overload for a nearer base — the
// system's own, or a user's for a policy type of their own — is the better match.
template <class Derived> struct execution_policy_base {};
// the policy as its own type, and without const: user overloads take their policy by reference
// (thrust/detail/execution_policy.h:50-75)
template <class Derived> inline execution_policy_base<Derived>& strip_const(const execution_policy_base<Derived>& x) {
  return const_cast<execution_policy_base<Derived>&>(x);
}
template <class Derived> inline Derived& derived_cast(execution_policy_base<Derived>& x) { return static_cast<Derived&>(x); }
template <class Derived> inline const Derived& derived_cast(const execution_policy_base<Derived>& x) { return static_cast<const Derived&>(x); }
}  // namespace detail

namespace system {
namespace cdna4 {

// ------------------------------------------------------------------------------------
// Execution policies
// ------------------------------------------------------------------------------------
struct tag {};

template <class Derived>
struct execution_policy : thrust::detail::execution_policy_base<Derived> {
  typedef tag tag_type;
  operator tag() const { return tag(); }
  const Derived& derived() const { return static_cast<const Derived&>(*this); }
};

namespace detail {

struct execute_on_stream : execution_policy<execute_on_stream> {
  void* stream_;
  bool sync_;
  execute_on_stream(void* s, bool sync) : stream_(s), sync_(sync) {}
};

// thrust::device / thrust::cdna4::par: work goes to the legacy default stream and the call
// returns after it has completed (thrust/system/cuda/detail/util.h:46-55, :113-140).
struct execute_after;  // thrust/event.h
template <class Alloc> struct execute_with_allocator;
template <class Alloc> struct execute_with_owned_allocator;
struct par_t : execution_policy<par_t> {
  execute_on_stream on(void* stream) const { return execute_on_stream(stream, true); }
  // thrust::device.after(events...): policy of an asynchronous algorithm that starts after them
  // (defined in thrust/event.h)
  template <class... Events> execute_after after(Events&&... events) const;
  template <class Alloc> execute_with_allocator<Alloc> operator()(Alloc& alloc) const;
  // an allocator passed as a temporary or a constant is copied into the policy
  // (thrust/detail/execute_with_allocator.h: the by-value form)
  template <class Alloc> execute_with_owned_allocator<Alloc> operator()(const Alloc& alloc) const;
};
// par_nosync: the call may return before the work has completed, except where a result has
// to be read back (thrust/system/cuda/detail/par.h:102-107, :181-186).
struct par_nosync_t : execution_policy<par_nosync_t> {
  execute_on_stream on(void* stream) const { return execute_on_stream(stream, false); }
};

// thrust::cdna4::par(alloc): temporary storage of the algorithm comes from the user's allocator
// (allocate(n) / deallocate(p, n) in units of its value_type) instead of the library's pool
// (thrust/system/cuda/detail/par.h:43-76, examples/cuda/custom_temporary_allocation.cu).
template <class Alloc>
struct execute_with_allocator : execution_policy<execute_with_allocator<Alloc>> {
  Alloc& alloc_;
  void* stream_;
  bool sync_;
  execute_with_allocator(Alloc& a, void* s, bool sync) : alloc_(a), stream_(s), sync_(sync) {}
  execute_with_allocator on(void* stream) const { return execute_with_allocator(alloc_, stream, sync_); }
};
template <class Alloc> struct owned_allocator { mutable Alloc owned_; explicit owned_allocator(const Alloc& a) : owned_(a) {} };
template <class Alloc>
struct execute_with_owned_allocator : private owned_allocator<Alloc>, execute_with_allocator<Alloc> {
  execute_with_owned_allocator(const Alloc& a, void* s, bool sync)
      : owned_allocator<Alloc>(a), execute_with_allocator<Alloc>(this->owned_, s, sync) {}
  execute_with_owned_allocator(const execute_with_owned_allocator& o)
      : owned_allocator<Alloc>(o.owned_), execute_with_allocator<Alloc>(this->owned_, o.stream_, o.sync_) {}
  execute_with_owned_allocator on(void* stream) const { return execute_with_owned_allocator(this->owned_, stream, this->sync_); }
};
template <class Alloc> inline void* stream_of(const execute_with_allocator<Alloc>& p) { return p.stream_; }
template <class Alloc> inline bool must_sync(const execute_with_allocator<Alloc>& p) { return p.sync_; }

// a policy of the user's own, derived from execution_policy<Derived> (thrust::device_execution_policy):
// the default stream, synchronous
template <class Derived> inline void* stream_of(const execution_policy<Derived>&) { return nullptr; }
template <class Derived> inline bool must_sync(const execution_policy<Derived>&) { return true; }
inline void* stream_of(const par_t&) { return nullptr; }
inline void* stream_of(const par_nosync_t&) { return nullptr; }
inline void* stream_of(const execute_on_stream& p) { return p.stream_; }
inline bool must_sync(const par_t&) { return true; }
inline bool must_sync(const par_nosync_t&) { return false; }
inline bool must_sync(const execute_on_stream& p) { return p.sync_; }

// Clears nothing on success; on failure throws thrust::system_error with the hip code
// (thrust/system/cuda/detail/util.h:207-292).
inline void throw_on_error(int status, const char* msg) {
  if (status != 0) throw thrust::system_error(status, thrust::cdna4_category(), msg);
}

template <class Policy>
inline void synchronize(const Policy& p, const char* msg) {
  throw_on_error(thrust_cdna4_stream_synchronize(stream_of(p)), msg);
}
template <class Policy>
inline void synchronize_optional(const Policy& p, const char* msg) {
  if (must_sync(p)) synchronize(p, msg);
}

// ------------------------------------------------------------------------------------
// Element types the kernels are built for.  Anything else is rejected at compile time:
// there is no fallback that would run a device algorithm on the host.
// ------------------------------------------------------------------------------------
template <class T, class = void>
struct dtype_of {
  static constexpr bool supported = false;
  static constexpr int value = -1;
};
template <class T>
struct dtype_of<T, typename std::enable_if<std::is_integral<T>::value && !std::is_same<T, bool>::value>::type> {
  static constexpr bool supported = sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8;
  static constexpr int value =
      sizeof(T) == 1 ? (std::is_signed<T>::value ? THRUST_CDNA4_I8 : THRUST_CDNA4_U8)
    : sizeof(T) == 2 ? (std::is_signed<T>::value ? THRUST_CDNA4_I16 : THRUST_CDNA4_U16)
    : sizeof(T) == 4 ? (std::is_signed<T>::value ? THRUST_CDNA4_I32 : THRUST_CDNA4_U32)
                     : (std::is_signed<T>::value ? THRUST_CDNA4_I64 : THRUST_CDNA4_U64);
};
template <>
struct dtype_of<float, void> {
  static constexpr bool supported = true;
  static constexpr int value = THRUST_CDNA4_F32;
};
template <>
struct dtype_of<double, void> {
  static constexpr bool supported = true;
  static constexpr int value = THRUST_CDNA4_F64;
};

// ------------------------------------------------------------------------------------
// Memory: cached, stream-ordered allocation through the library's pool.
// ------------------------------------------------------------------------------------
inline void* malloc_bytes(std::size_t bytes, void* stream) {
  void* p = nullptr;
  const int rc = thrust_cdna4_malloc(&p, bytes, stream);
  if (rc != 0) throw thrust::system::detail::bad_alloc(thrust_cdna4_error_string(rc));
  return p;
}
inline void free_bytes(void* p, void* stream) noexcept { (void)thrust_cdna4_free(p, stream); }

template <class Alloc>
execute_with_allocator<Alloc> par_t::operator()(Alloc& alloc) const { return execute_with_allocator<Alloc>(alloc, nullptr, true); }
template <class Alloc>
execute_with_owned_allocator<Alloc> par_t::operator()(const Alloc& alloc) const { return execute_with_owned_allocator<Alloc>(alloc, nullptr, true); }
// an allocator of void hands out bytes through its rebound form
template <class Alloc, class V = typename Alloc::value_type> struct storage_allocator {
  typedef Alloc type;
  static Alloc& get(Alloc& a) { return a; }
};
template <class Alloc> struct storage_allocator<Alloc, void> {
  typedef typename std::allocator_traits<Alloc>::template rebind_alloc<char> type;
  static type get(Alloc& a) { return type(a); }
};

// raw address of what an allocator returned (a raw pointer or a pointer-like object with get())
template <class T> inline void* address_of_allocation(T* p) { return const_cast<typename std::remove_const<T>::type*>(p); }
template <class P> inline auto address_of_allocation(const P& p) -> decltype((void*)p.get()) { return (void*)p.get(); }

// Byte buffer that lives for one algorithm call (thrust::detail::temporary_array<uint8_t>).
// It comes from the library's stream-ordered pool, or from the policy's allocator.
class temporary_storage {
 public:
  temporary_storage(std::size_t bytes, void* stream) : stream_(stream), bytes_(bytes), ptr_(nullptr), user_(nullptr), release_(nullptr) {
    if (bytes_) ptr_ = malloc_bytes(bytes_, stream_);
  }
  template <class Policy>
  temporary_storage(std::size_t bytes, const Policy& exec) : temporary_storage(bytes, stream_of(exec)) {}
  template <class Alloc>
  temporary_storage(std::size_t bytes, const execute_with_allocator<Alloc>& exec)
      : stream_(exec.stream_), bytes_(bytes), ptr_(nullptr), user_(&exec.alloc_), release_(nullptr) {
    typedef typename storage_allocator<Alloc>::type A;
    typedef typename A::value_type V;
    if (bytes_) {
      const std::size_t count = (bytes_ + sizeof(V) - 1) / sizeof(V);
      ptr_ = address_of_allocation(storage_allocator<Alloc>::get(exec.alloc_).allocate(count));
      release_ = [](void* alloc, void* p, std::size_t n, void* stream) {
        // the allocator may hand the block out again at once: wait for the work that uses it
        (void)thrust_cdna4_stream_synchronize(stream);
        typedef decltype(std::declval<A&>().allocate(1)) pointer;
        storage_allocator<Alloc>::get(*static_cast<Alloc*>(alloc)).deallocate(pointer(static_cast<V*>(p)), (n + sizeof(V) - 1) / sizeof(V));
      };
    }
  }
  ~temporary_storage() {
    if (!ptr_) return;
    if (release_) release_(user_, ptr_, bytes_, stream_);
    else free_bytes(ptr_, stream_);
  }
  temporary_storage(const temporary_storage&) = delete;
  temporary_storage& operator=(const temporary_storage&) = delete;
  void* data() const { return ptr_; }
  std::size_t size() const { return bytes_; }

 private:
  void* stream_;
  std::size_t bytes_;
  void* ptr_;
  void* user_;
  void (*release_)(void* alloc, void* p, std::size_t bytes, void* stream);
};

}  // namespace detail

static const detail::par_t par;
static const detail::par_nosync_t par_nosync;

}  // namespace cdna4
}  // namespace system

namespace cdna4 {
using thrust::system::cdna4::execution_policy;
using thrust::system::cdna4::par;
using thrust::system::cdna4::par_nosync;
using thrust::system::cdna4::tag;
}  // namespace cdna4

// Host system: the sequential implementations in this layer run for host_vector and raw
// host ranges under thrust::host (the counterpart of THRUST_HOST_SYSTEM_CPP).
namespace system {
namespace cpp {
struct tag {};
namespace detail {
struct par_t {};
}  // namespace detail
}  // namespace cpp
}  // namespace system

static const system::cdna4::detail::par_t device;
static const system::cpp::detail::par_t host;
// the system tags of device and host iterators (thrust/iterator/detail/device_system_tag.h:22-28)
typedef system::cdna4::tag device_system_tag;
typedef system::cpp::tag host_system_tag;

}  // namespace thrust

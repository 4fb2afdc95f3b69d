// <thrust/detail/config.h>: the configuration macros that user code and the reference's own tests
// read — namespace, compilers, language dialect, host/device decoration, small utilities
// (thrust/detail/config.h and thrust/detail/config/{namespace,compiler,cpp_dialect,host_device,
// cpp_compatibility,deprecated}.h).
#pragma once
#include <thrust/version.h>
#include <cstddef>
#include <utility>

// namespace (thrust/detail/config/namespace.h:18-120)
#ifndef THRUST_NAMESPACE_BEGIN
#define THRUST_NAMESPACE_BEGIN namespace thrust {
#define THRUST_NAMESPACE_END }
#endif
#ifndef THRUST_NS_QUALIFIER
#define THRUST_NS_QUALIFIER ::thrust
#endif
#ifndef THRUST_PREVENT_MACRO_SUBSTITUTION
#define THRUST_PREVENT_MACRO_SUBSTITUTION
#endif

// compilers (thrust/detail/config/compiler.h:24-110): hipcc and g++ are both "clang or gcc" hosts
#define THRUST_HOST_COMPILER_UNKNOWN 0
#define THRUST_HOST_COMPILER_MSVC 1
#define THRUST_HOST_COMPILER_GCC 2
#define THRUST_HOST_COMPILER_CLANG 3
#define THRUST_HOST_COMPILER_INTEL 4
#define THRUST_DEVICE_COMPILER_UNKNOWN 0
#define THRUST_DEVICE_COMPILER_MSVC 1
#define THRUST_DEVICE_COMPILER_GCC 2
#define THRUST_DEVICE_COMPILER_CLANG 3
#define THRUST_DEVICE_COMPILER_NVCC 4
#define THRUST_DEVICE_COMPILER_HIP 5
#if defined(__clang__)
#define THRUST_HOST_COMPILER THRUST_HOST_COMPILER_CLANG
#define THRUST_CLANG_VERSION (__clang_major__ * 10000 + __clang_minor__ * 100 + __clang_patchlevel__)
#elif defined(__GNUC__)
#define THRUST_HOST_COMPILER THRUST_HOST_COMPILER_GCC
#define THRUST_GCC_VERSION (__GNUC__ * 10000 + __GNUC_MINOR__ * 100 + __GNUC_PATCHLEVEL__)
#else
#define THRUST_HOST_COMPILER THRUST_HOST_COMPILER_UNKNOWN
#endif
#if defined(__HIPCC__)
#define THRUST_DEVICE_COMPILER THRUST_DEVICE_COMPILER_HIP
#elif defined(__clang__)
#define THRUST_DEVICE_COMPILER THRUST_DEVICE_COMPILER_CLANG
#else
#define THRUST_DEVICE_COMPILER THRUST_DEVICE_COMPILER_GCC
#endif

// language dialect (thrust/detail/config/cpp_dialect.h:60-80)
#if __cplusplus >= 202002L
#define THRUST_CPP_DIALECT 2020
#elif __cplusplus >= 201703L
#define THRUST_CPP_DIALECT 2017
#elif __cplusplus >= 201402L
#define THRUST_CPP_DIALECT 2014
#else
#define THRUST_CPP_DIALECT 2011
#endif
#define THRUST_CPP11
#define THRUST_CPP14

// decoration (thrust/detail/config/host_device.h, forceinline.h, exec_check_disable.h)
#if defined(__HIPCC__)
#define THRUST_HOST __host__
#define THRUST_DEVICE __device__
#define THRUST_HOST_DEVICE __host__ __device__
#define THRUST_FORCEINLINE __forceinline__
#else
#define THRUST_HOST
#define THRUST_DEVICE
#define THRUST_HOST_DEVICE
#define THRUST_FORCEINLINE inline __attribute__((always_inline))
// a host-only translation unit may still decorate its functors
#ifndef __host__
#define __host__
#endif
#ifndef __device__
#define __device__
#endif
#endif
#define THRUST_EXEC_CHECK_DISABLE

// small utilities (thrust/detail/config/cpp_compatibility.h:24-95)
#define THRUST_UNUSED_VAR(expr) do { (void)(expr); } while (0)
#if THRUST_CPP_DIALECT >= 2017
#define THRUST_IF_CONSTEXPR if constexpr
#define THRUST_INLINE_CONSTANT inline constexpr
#define THRUST_INLINE_INTEGRAL_MEMBER_CONSTANT inline constexpr
#define THRUST_NODISCARD [[nodiscard]]
#else
#define THRUST_IF_CONSTEXPR if
#define THRUST_INLINE_CONSTANT static constexpr
#define THRUST_INLINE_INTEGRAL_MEMBER_CONSTANT static constexpr
#define THRUST_NODISCARD
#endif
#define THRUST_CONSTEXPR constexpr
#define THRUST_OVERRIDE override
#define THRUST_DEFAULT = default;
#define THRUST_NOEXCEPT noexcept
#define THRUST_FINAL final
#define THRUST_TRIVIAL_ASSIGNMENT_OPERATOR_DEFAULT = default
#define THRUST_DEPRECATED [[deprecated]]
#define THRUST_DEPRECATED_BECAUSE(msg) [[deprecated(msg)]]
#define THRUST_ALIGNOF(x) alignof(x)

// warning brackets of other compilers expand to nothing here (thrust/detail/config/compiler.h:112-190)
#define THRUST_DISABLE_MSVC_WARNING_BEGIN(x)
#define THRUST_DISABLE_MSVC_WARNING_END(x)
#define THRUST_DISABLE_MSVC_POSSIBLE_LOSS_OF_DATA_WARNING_BEGIN
#define THRUST_DISABLE_MSVC_POSSIBLE_LOSS_OF_DATA_WARNING_END
#define THRUST_DISABLE_MSVC_POSSIBLE_LOSS_OF_DATA_WARNING(x) x
#define THRUST_DISABLE_MSVC_FORCING_VALUE_TO_BOOL_WARNING_BEGIN
#define THRUST_DISABLE_MSVC_FORCING_VALUE_TO_BOOL_WARNING_END
#define THRUST_DISABLE_MSVC_FORCING_VALUE_TO_BOOL_WARNING(x) x
#if defined(__clang__)
#define THRUST_DISABLE_CLANG_WARNING_BEGIN(x) _Pragma("clang diagnostic push") _Pragma(THRUST_CDNA4_PRAGMA_STR(clang diagnostic ignored #x))
#define THRUST_CDNA4_PRAGMA_STR(x) #x
#define THRUST_DISABLE_CLANG_WARNING_END(x) _Pragma("clang diagnostic pop")
#else
#define THRUST_DISABLE_CLANG_WARNING_BEGIN(x)
#define THRUST_DISABLE_CLANG_WARNING_END(x)
#endif
#define THRUST_DISABLE_CLANG_SELF_ASSIGNMENT_WARNING_BEGIN THRUST_DISABLE_CLANG_WARNING_BEGIN(-Wself-assign)
#define THRUST_DISABLE_CLANG_SELF_ASSIGNMENT_WARNING_END THRUST_DISABLE_CLANG_WARNING_END(-Wself-assign)
#define THRUST_DISABLE_CLANG_SELF_ASSIGNMENT_WARNING(x) \
  THRUST_DISABLE_CLANG_SELF_ASSIGNMENT_WARNING_BEGIN x; THRUST_DISABLE_CLANG_SELF_ASSIGNMENT_WARNING_END
#define THRUST_DISABLE_CLANG_AND_GCC_INITIALIZER_REORDERING_WARNING_BEGIN
#define THRUST_DISABLE_CLANG_AND_GCC_INITIALIZER_REORDERING_WARNING_END

// perfect forwarding and return-type deduction shorthands (thrust/detail/type_deduction.h:24-94)
#define THRUST_FWD(x) ::std::forward<decltype(x)>(x)
#define THRUST_MVCAP(x) x = ::std::move(x)
#define THRUST_RETURNS(...) noexcept(noexcept(__VA_ARGS__)) { return (__VA_ARGS__); }
#define THRUST_DECLTYPE_RETURNS(...) \
  noexcept(noexcept(__VA_ARGS__)) -> decltype(__VA_ARGS__) { return (__VA_ARGS__); }
#define THRUST_DECLTYPE_RETURNS_WITH_SFINAE_CONDITION(condition, ...)                                   \
  noexcept(noexcept(__VA_ARGS__)) -> typename ::std::enable_if<condition, decltype(__VA_ARGS__)>::type \
  { return (__VA_ARGS__); }

// deprecation brackets (thrust/detail/config/deprecated.h:24-60)
#if defined(__clang__)
#define THRUST_SUPPRESS_DEPRECATED_PUSH _Pragma("clang diagnostic push") _Pragma("clang diagnostic ignored \"-Wdeprecated-declarations\"")
#define THRUST_SUPPRESS_DEPRECATED_POP _Pragma("clang diagnostic pop")
#elif defined(__GNUC__)
#define THRUST_SUPPRESS_DEPRECATED_PUSH _Pragma("GCC diagnostic push") _Pragma("GCC diagnostic ignored \"-Wdeprecated-declarations\"")
#define THRUST_SUPPRESS_DEPRECATED_POP _Pragma("GCC diagnostic pop")
#else
#define THRUST_SUPPRESS_DEPRECATED_PUSH
#define THRUST_SUPPRESS_DEPRECATED_POP
#endif

// alignment of allocations made by the memory resources (thrust/mr/memory_resource.h:36-38)
#ifndef THRUST_MR_DEFAULT_ALIGNMENT
#define THRUST_MR_DEFAULT_ALIGNMENT alignof(::std::max_align_t)
#endif

// the token-pasting and argument-counting macros come with the configuration
#include <thrust/detail/preprocessor.h>
#include <thrust/detail/static_assert.h>

// <thrust/detail/cstdint.h>: the fixed-width integers under thrust::detail
// (thrust/detail/cstdint.h:30-85).
#pragma once
#include <thrust/detail/config.h>
#include <cstdint>
namespace thrust { namespace detail {
using ::std::int8_t;   using ::std::int16_t;   using ::std::int32_t;   using ::std::int64_t;
using ::std::uint8_t;  using ::std::uint16_t;  using ::std::uint32_t;  using ::std::uint64_t;
using ::std::intmax_t; using ::std::uintmax_t; using ::std::intptr_t;  using ::std::uintptr_t;
}}  // namespace thrust::detail

// thrust::mr::validator (thrust/mr/validator.h): a compile-time check that a type is a memory resource.
#pragma once
#include <type_traits>
#include <thrust/mr/memory_resource.h>
namespace thrust { namespace mr {
template <class MR>
struct validator {
  static_assert(std::is_base_of<memory_resource<typename MR::pointer>, MR>::value, "a type used as a memory resource must derive from memory_resource");
};
template <class T, class U> struct validator2 : private validator<T>, private validator<U> {};
template <class T> struct validator2<T, T> : private validator<T> {};
}}  // namespace thrust::mr

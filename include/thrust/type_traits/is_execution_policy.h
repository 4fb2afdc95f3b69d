// thrust::is_execution_policy (thrust/type_traits/is_execution_policy.h): whether a type is one
// of this build's execution policies (thrust::device, thrust::host, par.on(stream), par_nosync,
// par(alloc), or a policy a user derived from thrust::cdna4::execution_policy).
#pragma once
#include <type_traits>
#include <thrust/detail/iterator_util.h>
#include <thrust/execution_policy.h>
#include <thrust/type_traits/remove_cvref.h>
namespace thrust {
template <class T> struct is_execution_policy : std::integral_constant<bool, detail::is_policy<remove_cvref_t<T>>::value> {};
#if __cplusplus >= 201402L
template <class T> constexpr bool is_execution_policy_v = is_execution_policy<T>::value;
#endif
}  // namespace thrust

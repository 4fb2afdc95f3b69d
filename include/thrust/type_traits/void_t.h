// thrust::void_t (thrust/type_traits/void_t.h): maps any well-formed list of types to void.
#pragma once
namespace thrust {
template <class...> struct voider { typedef void type; };
template <class... Ts> using void_t = typename voider<Ts...>::type;
}  // namespace thrust

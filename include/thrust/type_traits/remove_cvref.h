// thrust::remove_cvref (thrust/type_traits/remove_cvref.h).
#pragma once
#include <type_traits>
namespace thrust {
template <class T> struct remove_cvref { typedef typename std::remove_cv<typename std::remove_reference<T>::type>::type type; };
template <class T> using remove_cvref_t = typename remove_cvref<T>::type;
}  // namespace thrust

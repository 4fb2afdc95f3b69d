// thrust::addressof (thrust/addressof.h): the address of an object even when operator& is overloaded.
#pragma once
#include <thrust/functional.h>
namespace thrust {
template <class T> THRUST_CDNA4_HD T* addressof(T& arg) {
  return reinterpret_cast<T*>(&const_cast<char&>(reinterpret_cast<const volatile char&>(arg)));
}
}  // namespace thrust

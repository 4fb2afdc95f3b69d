// thrust::complex<T> (thrust/complex.h): a complex number type whose every operation is callable
// in device code, layout-compatible with std::complex<T> and convertible from and to it.
// Arithmetic, comparison, stream I/O and the elementary functions of <complex>: abs, arg, norm,
// conj, polar, proj, exp, log, log10, pow, sqrt, the circular and hyperbolic functions and their
// inverses.  Division scales by the larger component of the divisor, sqrt and the inverse
// functions use the usual cancellation-free forms; results agree with std::complex to a few units
// in the last place for finite arguments of ordinary magnitude (tests/cpp/test_complex.cpp).
#pragma once
#include <cmath>
#include <complex>
#include <iostream>
#include <type_traits>
#include <thrust/detail/hd.h>

namespace thrust {

template <class T>
struct alignas(2 * sizeof(T)) complex {
  typedef T value_type;

  complex() = default;
  THRUST_CDNA4_HD complex(const T& re) : data_{re, T()} {}
  THRUST_CDNA4_HD complex(const T& re, const T& im) : data_{re, im} {}
  complex(const complex&) = default;
  template <class U> THRUST_CDNA4_HD complex(const complex<U>& z) : data_{T(z.real()), T(z.imag())} {}
  complex(const std::complex<T>& z) : data_{z.real(), z.imag()} {}
  template <class U> complex(const std::complex<U>& z) : data_{T(z.real()), T(z.imag())} {}

  complex& operator=(const complex&) = default;
  THRUST_CDNA4_HD complex& operator=(const T& re) { data_[0] = re; data_[1] = T(); return *this; }
  template <class U> THRUST_CDNA4_HD complex& operator=(const complex<U>& z) { data_[0] = T(z.real()); data_[1] = T(z.imag()); return *this; }
  complex& operator=(const std::complex<T>& z) { data_[0] = z.real(); data_[1] = z.imag(); return *this; }
  template <class U> complex& operator=(const std::complex<U>& z) { data_[0] = T(z.real()); data_[1] = T(z.imag()); return *this; }

  THRUST_CDNA4_HD T real() const { return data_[0]; }
  THRUST_CDNA4_HD T imag() const { return data_[1]; }
  THRUST_CDNA4_HD T real() const volatile { return data_[0]; }
  THRUST_CDNA4_HD T imag() const volatile { return data_[1]; }
  THRUST_CDNA4_HD void real(T re) { data_[0] = re; }
  THRUST_CDNA4_HD void imag(T im) { data_[1] = im; }
  THRUST_CDNA4_HD void real(T re) volatile { data_[0] = re; }
  THRUST_CDNA4_HD void imag(T im) volatile { data_[1] = im; }
  operator std::complex<T>() const { return std::complex<T>(real(), imag()); }

  template <class U> THRUST_CDNA4_HD complex& operator+=(const complex<U>& z) { data_[0] += T(z.real()); data_[1] += T(z.imag()); return *this; }
  template <class U> THRUST_CDNA4_HD complex& operator-=(const complex<U>& z) { data_[0] -= T(z.real()); data_[1] -= T(z.imag()); return *this; }
  template <class U> THRUST_CDNA4_HD complex& operator*=(const complex<U>& z) { *this = *this * complex<T>(z); return *this; }
  template <class U> THRUST_CDNA4_HD complex& operator/=(const complex<U>& z) { *this = *this / complex<T>(z); return *this; }
  THRUST_CDNA4_HD complex& operator+=(const T& x) { data_[0] += x; return *this; }
  THRUST_CDNA4_HD complex& operator-=(const T& x) { data_[0] -= x; return *this; }
  THRUST_CDNA4_HD complex& operator*=(const T& x) { data_[0] *= x; data_[1] *= x; return *this; }
  THRUST_CDNA4_HD complex& operator/=(const T& x) { data_[0] /= x; data_[1] /= x; return *this; }

 private:
  T data_[2];
};

// ---- arithmetic
template <class T> THRUST_CDNA4_HD complex<T> operator+(const complex<T>& a, const complex<T>& b) { return complex<T>(a.real() + b.real(), a.imag() + b.imag()); }
template <class T> THRUST_CDNA4_HD complex<T> operator+(const complex<T>& a, const T& b) { return complex<T>(a.real() + b, a.imag()); }
template <class T> THRUST_CDNA4_HD complex<T> operator+(const T& a, const complex<T>& b) { return complex<T>(a + b.real(), b.imag()); }
template <class T> THRUST_CDNA4_HD complex<T> operator-(const complex<T>& a, const complex<T>& b) { return complex<T>(a.real() - b.real(), a.imag() - b.imag()); }
template <class T> THRUST_CDNA4_HD complex<T> operator-(const complex<T>& a, const T& b) { return complex<T>(a.real() - b, a.imag()); }
template <class T> THRUST_CDNA4_HD complex<T> operator-(const T& a, const complex<T>& b) { return complex<T>(a - b.real(), -b.imag()); }
template <class T> THRUST_CDNA4_HD complex<T> operator*(const complex<T>& a, const complex<T>& b) {
  return complex<T>(a.real() * b.real() - a.imag() * b.imag(), a.real() * b.imag() + a.imag() * b.real());
}
template <class T> THRUST_CDNA4_HD complex<T> operator*(const complex<T>& a, const T& b) { return complex<T>(a.real() * b, a.imag() * b); }
template <class T> THRUST_CDNA4_HD complex<T> operator*(const T& a, const complex<T>& b) { return complex<T>(a * b.real(), a * b.imag()); }
// the divisor is scaled by its larger component first, so that c^2 + d^2 neither overflows nor underflows early
template <class T> THRUST_CDNA4_HD complex<T> operator/(const complex<T>& a, const complex<T>& b) {
  const T s = std::fabs(b.real()) > std::fabs(b.imag()) ? std::fabs(b.real()) : std::fabs(b.imag());
  if (s == T(0)) return complex<T>(a.real() / s, a.imag() / s);
  const T oos = T(1) / s;
  const T ars = a.real() * oos, ais = a.imag() * oos, brs = b.real() * oos, bis = b.imag() * oos;
  const T n = T(1) / (brs * brs + bis * bis);
  return complex<T>((ars * brs + ais * bis) * n, (ais * brs - ars * bis) * n);
}
template <class T> THRUST_CDNA4_HD complex<T> operator/(const complex<T>& a, const T& b) { return complex<T>(a.real() / b, a.imag() / b); }
template <class T> THRUST_CDNA4_HD complex<T> operator/(const T& a, const complex<T>& b) { return complex<T>(a) / b; }
template <class T> THRUST_CDNA4_HD complex<T> operator+(const complex<T>& a) { return a; }
template <class T> THRUST_CDNA4_HD complex<T> operator-(const complex<T>& a) { return complex<T>(-a.real(), -a.imag()); }
// mixed component types promote, as in the reference (complex<float> * complex<double> -> complex<double>)
template <class T, class U, class = typename std::enable_if<!std::is_same<T, U>::value>::type>
THRUST_CDNA4_HD complex<typename std::common_type<T, U>::type> operator+(const complex<T>& a, const complex<U>& b) {
  typedef typename std::common_type<T, U>::type R; return complex<R>(a) + complex<R>(b);
}
template <class T, class U, class = typename std::enable_if<!std::is_same<T, U>::value>::type>
THRUST_CDNA4_HD complex<typename std::common_type<T, U>::type> operator-(const complex<T>& a, const complex<U>& b) {
  typedef typename std::common_type<T, U>::type R; return complex<R>(a) - complex<R>(b);
}
template <class T, class U, class = typename std::enable_if<!std::is_same<T, U>::value>::type>
THRUST_CDNA4_HD complex<typename std::common_type<T, U>::type> operator*(const complex<T>& a, const complex<U>& b) {
  typedef typename std::common_type<T, U>::type R; return complex<R>(a) * complex<R>(b);
}
template <class T, class U, class = typename std::enable_if<!std::is_same<T, U>::value>::type>
THRUST_CDNA4_HD complex<typename std::common_type<T, U>::type> operator/(const complex<T>& a, const complex<U>& b) {
  typedef typename std::common_type<T, U>::type R; return complex<R>(a) / complex<R>(b);
}

// a scalar of another arithmetic type on either side (z * 2, 1 / z ...)
#define THRUST_CDNA4_COMPLEX_SCALAR_OP(OP)                                                                                              \
  template <class T, class U, class = typename std::enable_if<std::is_arithmetic<U>::value && !std::is_same<T, U>::value>::type>        \
  THRUST_CDNA4_HD complex<typename std::common_type<T, U>::type> operator OP(const complex<T>& a, const U& b) {                         \
    typedef typename std::common_type<T, U>::type R;                                                                                    \
    return complex<R>(a) OP R(b);                                                                                                       \
  }                                                                                                                                     \
  template <class T, class U, class = typename std::enable_if<std::is_arithmetic<U>::value && !std::is_same<T, U>::value>::type>        \
  THRUST_CDNA4_HD complex<typename std::common_type<T, U>::type> operator OP(const U& a, const complex<T>& b) {                         \
    typedef typename std::common_type<T, U>::type R;                                                                                    \
    return R(a) OP complex<R>(b);                                                                                                       \
  }
THRUST_CDNA4_COMPLEX_SCALAR_OP(+)
THRUST_CDNA4_COMPLEX_SCALAR_OP(-)
THRUST_CDNA4_COMPLEX_SCALAR_OP(*)
THRUST_CDNA4_COMPLEX_SCALAR_OP(/)
#undef THRUST_CDNA4_COMPLEX_SCALAR_OP

// ---- comparison
template <class T, class U> THRUST_CDNA4_HD bool operator==(const complex<T>& a, const complex<U>& b) { return a.real() == b.real() && a.imag() == b.imag(); }
template <class T, class U> THRUST_CDNA4_HD bool operator!=(const complex<T>& a, const complex<U>& b) { return !(a == b); }
template <class T> THRUST_CDNA4_HD bool operator==(const complex<T>& a, const T& b) { return a.real() == b && a.imag() == T(0); }
template <class T> THRUST_CDNA4_HD bool operator==(const T& a, const complex<T>& b) { return b == a; }
template <class T> THRUST_CDNA4_HD bool operator!=(const complex<T>& a, const T& b) { return !(a == b); }
template <class T> THRUST_CDNA4_HD bool operator!=(const T& a, const complex<T>& b) { return !(b == a); }
template <class T, class U> bool operator==(const complex<T>& a, const std::complex<U>& b) { return a.real() == b.real() && a.imag() == b.imag(); }
template <class T, class U> bool operator==(const std::complex<T>& a, const complex<U>& b) { return b == a; }
template <class T, class U> bool operator!=(const complex<T>& a, const std::complex<U>& b) { return !(a == b); }
template <class T, class U> bool operator!=(const std::complex<T>& a, const complex<U>& b) { return !(b == a); }

// ---- stream I/O in the standard's format: (re,im)
template <class T, class Ch, class Tr>
std::basic_ostream<Ch, Tr>& operator<<(std::basic_ostream<Ch, Tr>& os, const complex<T>& z) { return os << std::complex<T>(z.real(), z.imag()); }
template <class T, class Ch, class Tr>
std::basic_istream<Ch, Tr>& operator>>(std::basic_istream<Ch, Tr>& is, complex<T>& z) {
  std::complex<T> s;
  is >> s;
  z = s;
  return is;
}

// ---- value functions
template <class T> THRUST_CDNA4_HD T abs(const complex<T>& z) { return std::hypot(z.real(), z.imag()); }
template <class T> THRUST_CDNA4_HD T arg(const complex<T>& z) { return std::atan2(z.imag(), z.real()); }
template <class T> THRUST_CDNA4_HD T norm(const complex<T>& z) { return z.real() * z.real() + z.imag() * z.imag(); }
template <class T> THRUST_CDNA4_HD complex<T> conj(const complex<T>& z) { return complex<T>(z.real(), -z.imag()); }
template <class T> THRUST_CDNA4_HD complex<T> polar(const T& m, const T& theta = T()) { return complex<T>(m * std::cos(theta), m * std::sin(theta)); }
template <class T> THRUST_CDNA4_HD complex<T> proj(const complex<T>& z) {
  if (std::isinf(z.real()) || std::isinf(z.imag())) return complex<T>(INFINITY, std::copysign(T(0), z.imag()));
  return z;
}

// ---- exponential and logarithm
template <class T> THRUST_CDNA4_HD complex<T> exp(const complex<T>& z) {
  const T e = std::exp(z.real());
  if (z.imag() == T(0)) return complex<T>(e, z.imag());
  return complex<T>(e * std::cos(z.imag()), e * std::sin(z.imag()));
}
template <class T> THRUST_CDNA4_HD complex<T> log(const complex<T>& z) { return complex<T>(std::log(abs(z)), arg(z)); }
template <class T> THRUST_CDNA4_HD complex<T> log10(const complex<T>& z) { return log(z) / T(2.30258509299404568402); }

// ---- square root: the branch with a non-negative real part, without cancellation
template <class T> THRUST_CDNA4_HD complex<T> sqrt(const complex<T>& z) {
  const T x = z.real(), y = z.imag();
  if (x == T(0) && y == T(0)) return complex<T>(T(0), y);
  const T m = abs(z);
  if (x >= T(0)) {
    const T t = std::sqrt((m + x) * T(0.5));
    return complex<T>(t, y / (T(2) * t));
  }
  const T t = std::sqrt((m - x) * T(0.5));
  return complex<T>(std::fabs(y) / (T(2) * t), std::copysign(t, y));
}

// ---- powers
template <class T> THRUST_CDNA4_HD complex<T> pow(const complex<T>& x, const complex<T>& y) {
  if (x.real() == T(0) && x.imag() == T(0)) return (y.real() == T(0) && y.imag() == T(0)) ? complex<T>(T(1)) : complex<T>(T(0));
  return exp(log(x) * y);
}
template <class T> THRUST_CDNA4_HD complex<T> pow(const complex<T>& x, const T& y) { return pow(x, complex<T>(y)); }
template <class T> THRUST_CDNA4_HD complex<T> pow(const T& x, const complex<T>& y) { return pow(complex<T>(x), y); }
template <class T, class U, class = typename std::enable_if<!std::is_same<T, U>::value>::type>
THRUST_CDNA4_HD complex<typename std::common_type<T, U>::type> pow(const complex<T>& x, const complex<U>& y) {
  typedef typename std::common_type<T, U>::type R; return pow(complex<R>(x), complex<R>(y));
}

// ---- hyperbolic and circular functions
template <class T> THRUST_CDNA4_HD complex<T> sinh(const complex<T>& z) {
  return complex<T>(std::sinh(z.real()) * std::cos(z.imag()), std::cosh(z.real()) * std::sin(z.imag()));
}
template <class T> THRUST_CDNA4_HD complex<T> cosh(const complex<T>& z) {
  return complex<T>(std::cosh(z.real()) * std::cos(z.imag()), std::sinh(z.real()) * std::sin(z.imag()));
}
template <class T> THRUST_CDNA4_HD complex<T> tanh(const complex<T>& z) {
  // (sinh 2x + i sin 2y) / (cosh 2x + cos 2y); for large |x| the result is +-1 to working precision
  const T x2 = T(2) * z.real(), y2 = T(2) * z.imag();
  if (std::fabs(x2) > T(40)) return complex<T>(std::copysign(T(1), x2), std::copysign(T(0), std::sin(y2)));
  const T d = std::cosh(x2) + std::cos(y2);
  return complex<T>(std::sinh(x2) / d, std::sin(y2) / d);
}
template <class T> THRUST_CDNA4_HD complex<T> sin(const complex<T>& z) {
  return complex<T>(std::sin(z.real()) * std::cosh(z.imag()), std::cos(z.real()) * std::sinh(z.imag()));
}
template <class T> THRUST_CDNA4_HD complex<T> cos(const complex<T>& z) {
  return complex<T>(std::cos(z.real()) * std::cosh(z.imag()), -std::sin(z.real()) * std::sinh(z.imag()));
}
template <class T> THRUST_CDNA4_HD complex<T> tan(const complex<T>& z) {
  // tan z = -i tanh(iz)
  const complex<T> t = tanh(complex<T>(-z.imag(), z.real()));
  return complex<T>(t.imag(), -t.real());
}

// ---- inverse functions (principal values)
template <class T> THRUST_CDNA4_HD complex<T> asinh(const complex<T>& z) {
  // log(z + sqrt(z^2 + 1)), odd: computed for the half-plane where nothing cancels
  const bool flip = z.real() < T(0);
  const complex<T> w = flip ? -z : z;
  const complex<T> r = log(w + sqrt(w * w + T(1)));
  return flip ? -r : r;
}
template <class T> THRUST_CDNA4_HD complex<T> acosh(const complex<T>& z) {
  const complex<T> r = log(z + sqrt(z + T(1)) * sqrt(z - T(1)));
  return r;
}
template <class T> THRUST_CDNA4_HD complex<T> atanh(const complex<T>& z) {
  // 1/2 log((1 + z) / (1 - z)) with the real part from one log1p-free quotient of norms
  const T x = z.real(), y = z.imag();
  const T num = (T(1) + x) * (T(1) + x) + y * y, den = (T(1) - x) * (T(1) - x) + y * y;
  return complex<T>(T(0.25) * std::log(num / den), T(0.5) * std::atan2(T(2) * y, (T(1) - x) * (T(1) + x) - y * y));
}
template <class T> THRUST_CDNA4_HD complex<T> asin(const complex<T>& z) {
  // asin z = -i asinh(iz)
  const complex<T> t = asinh(complex<T>(-z.imag(), z.real()));
  return complex<T>(t.imag(), -t.real());
}
template <class T> THRUST_CDNA4_HD complex<T> acos(const complex<T>& z) {
  const complex<T> s = asin(z);
  return complex<T>(T(1.57079632679489661923) - s.real(), -s.imag());
}
template <class T> THRUST_CDNA4_HD complex<T> atan(const complex<T>& z) {
  // atan z = -i atanh(iz)
  const complex<T> t = atanh(complex<T>(-z.imag(), z.real()));
  return complex<T>(t.imag(), -t.real());
}

}  // namespace thrust

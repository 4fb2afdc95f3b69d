// thrust::complex: every operation against std::complex on the host over a grid of arguments
// (the shape of testing/complex.cu: arithmetic, abs / arg / norm / conj / polar, exp / log / pow /
// sqrt, the circular and hyperbolic functions and their inverses, stream I/O), and the same
// operations inside device kernels against the host results.  Tolerance: 4 units of 1e-6 (float) /
// 1e-13 (double) relative to max(1, |result|), stated where it is applied.
#include <thrust/complex.h>
#include <thrust/device_vector.h>
#include <thrust/host_vector.h>
#include <thrust/reduce.h>
#include <thrust/sort.h>
#include <thrust/transform.h>

#include <complex>
#include <sstream>

#include "testing.h"

template <class T> struct tol;
template <> struct tol<float> { static constexpr double value = 4e-6; };
template <> struct tol<double> { static constexpr double value = 4e-13; };

template <class T>
void near(thrust::complex<T> got, std::complex<T> want, const char* what, std::complex<T> at) {
  const double scale = std::max(1.0, (double)std::abs(want));
  const double err = std::max(std::fabs((double)got.real() - (double)want.real()), std::fabs((double)got.imag() - (double)want.imag()));
  if (!(err <= tol<T>::value * scale)) {
    std::ostringstream os;
    os << what << " at " << at << ": " << got << " vs " << want << " (error " << err << ")";
    unittest::fail(__FILE__, __LINE__, os.str());
  }
}

template <class T>
std::vector<std::complex<T>> grid() {
  std::vector<std::complex<T>> g;
  const T v[] = {T(-3.5), T(-1.25), T(-0.5), T(0), T(0.25), T(0.75), T(1), T(2.5), T(6)};
  for (T a : v)
    for (T b : v) g.push_back(std::complex<T>(a, b));
  return g;
}

template <class T>
void TestComplexAgainstStdComplex() {
  typedef thrust::complex<T> C;
  typedef std::complex<T> S;
  static_assert(sizeof(C) == sizeof(S) && alignof(C) >= alignof(S), "layout of std::complex");
  static_assert(std::is_trivially_copyable<C>::value && std::is_trivially_default_constructible<C>::value, "usable in device storage");
  for (S a : grid<T>()) {
    const C ta(a);
    near<T>(C(thrust::abs(ta)), S(std::abs(a)), "abs", a);
    near<T>(C(thrust::arg(ta)), S(std::arg(a)), "arg", a);
    near<T>(C(thrust::norm(ta)), S(std::norm(a)), "norm", a);
    near<T>(thrust::conj(ta), std::conj(a), "conj", a);
    near<T>(thrust::exp(ta), std::exp(a), "exp", a);
    near<T>(thrust::sinh(ta), std::sinh(a), "sinh", a);
    near<T>(thrust::cosh(ta), std::cosh(a), "cosh", a);
    near<T>(thrust::tanh(ta), std::tanh(a), "tanh", a);
    near<T>(thrust::sin(ta), std::sin(a), "sin", a);
    near<T>(thrust::cos(ta), std::cos(a), "cos", a);
    near<T>(thrust::sqrt(ta), std::sqrt(a), "sqrt", a);
    near<T>(-ta, -a, "negate", a);
    if (a != S(0)) {
      near<T>(thrust::log(ta), std::log(a), "log", a);
      near<T>(thrust::log10(ta), std::log10(a), "log10", a);
      near<T>(T(1) / ta, T(1) / a, "reciprocal", a);
      near<T>(thrust::pow(ta, T(2.5)), std::pow(a, T(2.5)), "pow(z, real)", a);
      near<T>(thrust::pow(T(2.5), ta), std::pow(T(2.5), a), "pow(real, z)", a);
    }
    // away from the branch cuts and poles of the inverse functions and of tan
    if (std::fabs(a.imag()) > T(0.1) || std::fabs(a.real()) < T(0.9)) {
      near<T>(thrust::asin(ta), std::asin(a), "asin", a);
      near<T>(thrust::acos(ta), std::acos(a), "acos", a);
      near<T>(thrust::atanh(ta), std::atanh(a), "atanh", a);
    }
    if (std::fabs(a.real()) > T(0.1) || std::fabs(a.imag()) < T(0.9)) {
      near<T>(thrust::atan(ta), std::atan(a), "atan", a);
      near<T>(thrust::asinh(ta), std::asinh(a), "asinh", a);
    }
    if (std::fabs(a.imag()) > T(0.1) || a.real() > T(1.1)) near<T>(thrust::acosh(ta), std::acosh(a), "acosh", a);
    if (std::abs(std::cos(a)) > T(0.05)) near<T>(thrust::tan(ta), std::tan(a), "tan", a);
    for (S b : grid<T>()) {
      const C tb(b);
      near<T>(ta + tb, a + b, "+", a);
      near<T>(ta - tb, a - b, "-", a);
      near<T>(ta * tb, a * b, "*", a);
      if (b != S(0)) near<T>(ta / tb, a / b, "/", a);
      if (a != S(0) && std::abs(b) < 4) near<T>(thrust::pow(ta, tb), std::pow(a, b), "pow", a);
    }
  }
  near<T>(thrust::polar(T(2), T(0.5)), std::polar(T(2), T(0.5)), "polar", S(2, 0.5));
  near<T>(thrust::pow(C(0), C(2)), S(0), "0^2", S(0));
  // compound assignment, scalars of another type, comparison, conversion
  C z(1, 2);
  z += C(2, 3);
  z -= T(1);
  z *= C(0, 1);
  z /= T(2);
  near<T>(z, (S(1, 2) + S(2, 3) - T(1)) * S(0, 1) / T(2), "compound", S(0));
  near<T>(C(1, 2) * 2, S(2, 4), "z * int", S(0));
  near<T>(1 / C(0, 1), S(0, -1), "int / z", S(0));
  ASSERT_TRUE(C(1, 2) == C(1, 2) && C(1, 2) != C(1, 3) && C(3, 0) == T(3) && C(1, 2) == S(1, 2));
  const S back = C(4, 5);
  ASSERT_TRUE(back == S(4, 5));
  const thrust::complex<double> wide = thrust::complex<float>(1.5f, -2.5f);
  ASSERT_TRUE(wide == thrust::complex<double>(1.5, -2.5));
  // stream format of the standard
  std::ostringstream os;
  os << C(1, -2);
  ASSERT_EQUAL(os.str(), std::string("(1,-2)"));
  std::istringstream is("(3,4)");
  C in;
  is >> in;
  ASSERT_TRUE(in == C(3, 4));
}
DECLARE_TYPED_UNITTEST(TestComplexAgainstStdComplex, float);
DECLARE_TYPED_UNITTEST(TestComplexAgainstStdComplex, double);

// the same functions evaluated in a kernel
template <class T>
struct every_function {
  __host__ __device__ thrust::complex<T> operator()(const thrust::complex<T>& z) const {
    typedef thrust::complex<T> C;
    const C w = z + C(T(0.3), T(-0.2));
    C acc = thrust::exp(z * T(0.1)) + thrust::sin(z) * thrust::cos(w) - thrust::sinh(z * T(0.2)) / (thrust::cosh(w * T(0.2)) + T(2));
    acc += thrust::sqrt(z) + thrust::log(w * w + T(1.5)) + thrust::tanh(z) + thrust::atan(z * T(0.1)) + thrust::asinh(w);
    acc += thrust::pow(w * w + T(2), C(T(0.5), T(0.25))) + thrust::conj(z) * thrust::polar(T(1), thrust::arg(w)) + C(thrust::abs(z), thrust::norm(w));
    return acc;
  }
};
template <class T>
void TestComplexInDeviceCode() {
  typedef thrust::complex<T> C;
  const std::size_t n = 100000;
  thrust::host_vector<C> h(n), want(n);
  std::uint64_t s = 99;
  for (auto& z : h) {
    const T re = (T)((double)(unittest::splitmix64(s) >> 11) / 9007199254740992.0 * 6.0 - 3.0);
    const T im = (T)((double)(unittest::splitmix64(s) >> 11) / 9007199254740992.0 * 6.0 - 3.0);
    z = C(re, im);
  }
  thrust::transform(h.begin(), h.end(), want.begin(), every_function<T>());
  thrust::device_vector<C> d = h, got(n);
  thrust::transform(d.begin(), d.end(), got.begin(), every_function<T>());
  thrust::host_vector<C> back = got;
  for (std::size_t i = 0; i < n; i++) {
    // device and host math libraries may differ in the last places: 20 x the per-function tolerance over the sum of 15 terms
    const double scale = std::max(1.0, (double)thrust::abs(want[i]));
    const double err = std::max(std::fabs((double)back[i].real() - (double)want[i].real()), std::fabs((double)back[i].imag() - (double)want[i].imag()));
    if (!(err <= 20 * tol<T>::value * scale)) {
      std::ostringstream os;
      os << "element " << i << " " << h[i] << ": " << back[i] << " vs " << want[i];
      unittest::fail(__FILE__, __LINE__, os.str());
    }
  }
  // reduction of complex numbers with the built-in plus
  thrust::device_vector<C> ones(4096, C(1, -2));
  const C total = thrust::reduce(ones.begin(), ones.end(), C(0, 0), thrust::plus<C>());
  ASSERT_TRUE(total == C(4096, -8192));
}
DECLARE_TYPED_UNITTEST(TestComplexInDeviceCode, float);
DECLARE_TYPED_UNITTEST(TestComplexInDeviceCode, double);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

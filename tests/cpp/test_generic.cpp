// for_each / transform / sequence / reduce / transform_reduce / count with user functors, in the
// shape of the reference's testing/for_each.cu, transform.cu, sequence.cu, reduce.cu,
// transform_reduce.cu and count.cu: known answers plus device vs host over the size ladder.
// User functors instantiate kernel templates, so this translation unit is compiled by hipcc.
#include <cmath>
#include <numeric>

#include <thrust/count.h>
#include <thrust/for_each.h>
#include <thrust/functional.h>
#include <thrust/reduce.h>
#include <thrust/sequence.h>
#include <thrust/transform.h>
#include <thrust/transform_reduce.h>

#include "testing.h"

template <class T>
struct times_two_plus_one {
  __host__ __device__ T operator()(const T& x) const { return (T)(2 * x + 1); }
};
template <class T>
struct add_in_place {
  T delta;
  __host__ __device__ void operator()(T& x) const { x = (T)(x + delta); }
};
struct saxpy {
  float a;
  __host__ __device__ float operator()(float x, float y) const { return a * x + y; }
};
struct is_even {
  __host__ __device__ bool operator()(int x) const { return (x & 1) == 0; }
};
template <class T>
struct max_of {
  __host__ __device__ T operator()(const T& a, const T& b) const { return a < b ? b : a; }
};

// testing/transform.cu:21-46 (unary known answer), :95-123 (binary)
void TestTransformSimple() {
  const int in[3] = {1, -2, 3};
  thrust::device_vector<int> d(in, in + 3), out(3);
  auto end = thrust::transform(d.begin(), d.end(), out.begin(), thrust::negate<int>());
  ASSERT_TRUE(end == out.end());
  const int expect[3] = {-1, 2, -3};
  ASSERT_EQUAL(out, thrust::host_vector<int>(expect, expect + 3));
  const int in2[3] = {-4, 5, 6};
  thrust::device_vector<int> d2(in2, in2 + 3);
  thrust::transform(d.begin(), d.end(), d2.begin(), out.begin(), thrust::minus<int>());
  const int expect2[3] = {5, -7, -3};
  ASSERT_EQUAL(out, thrust::host_vector<int>(expect2, expect2 + 3));
}
DECLARE_UNITTEST(TestTransformSimple);

template <class T>
void TestTransformLadder() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n), ho(n);
    thrust::device_vector<T> d = h, dout(n);
    thrust::transform(h.begin(), h.end(), ho.begin(), times_two_plus_one<T>());
    thrust::transform(d.begin(), d.end(), dout.begin(), times_two_plus_one<T>());
    ASSERT_EQUAL(ho, dout);
    thrust::transform(d.begin(), d.end(), d.begin(), times_two_plus_one<T>());  // in place
    ASSERT_EQUAL(ho, d);
  }
}
DECLARE_TYPED_UNITTEST(TestTransformLadder, int);
DECLARE_TYPED_UNITTEST(TestTransformLadder, uint8_t);
DECLARE_TYPED_UNITTEST(TestTransformLadder, int64_t);

void TestTransformBinarySaxpy() {
  const std::size_t n = 1000003;
  thrust::host_vector<float> x = unittest::random_samples<float>(n), y = unittest::random_samples<float>(n, 5), hz(n);
  thrust::device_vector<float> dx = x, dy = y, dz(n);
  thrust::transform(x.begin(), x.end(), y.begin(), hz.begin(), saxpy{2.5f});
  thrust::transform(thrust::device, dx.begin(), dx.end(), dy.begin(), dz.begin(), saxpy{2.5f});
  thrust::host_vector<float> got = dz;
  for (std::size_t i = 0; i < n; i++) ASSERT_TRUE(std::fabs(got[i] - hz[i]) <= 1e-5f * (1.0f + std::fabs(hz[i])));  // fma contraction differs
}
DECLARE_UNITTEST(TestTransformBinarySaxpy);

// testing/for_each.cu:45-83
void TestForEach() {
  for (std::size_t n : {std::size_t(0), std::size_t(1), std::size_t(1025), std::size_t(300001)}) {
    thrust::host_vector<int> h = unittest::random_integers<int>(n);
    thrust::device_vector<int> d = h;
    thrust::for_each(h.begin(), h.end(), add_in_place<int>{7});
    auto end = thrust::for_each(d.begin(), d.end(), add_in_place<int>{7});
    ASSERT_TRUE(end == d.end());
    ASSERT_EQUAL(h, d);
    thrust::for_each_n(h.begin(), n / 2, add_in_place<int>{-3});
    thrust::for_each_n(d.begin(), n / 2, add_in_place<int>{-3});
    ASSERT_EQUAL(h, d);
  }
}
DECLARE_UNITTEST(TestForEach);

// testing/sequence.cu:52-108
template <class T>
void TestSequence() {
  thrust::device_vector<T> d(5);
  thrust::sequence(d.begin(), d.end());
  const T e0[5] = {0, 1, 2, 3, 4};
  ASSERT_EQUAL(d, thrust::host_vector<T>(e0, e0 + 5));
  thrust::sequence(d.begin(), d.end(), T(10));
  const T e1[5] = {10, 11, 12, 13, 14};
  ASSERT_EQUAL(d, thrust::host_vector<T>(e1, e1 + 5));
  thrust::sequence(d.begin(), d.end(), T(10), T(2));
  const T e2[5] = {10, 12, 14, 16, 18};
  ASSERT_EQUAL(d, thrust::host_vector<T>(e2, e2 + 5));
  for (std::size_t n : {std::size_t(1023), std::size_t(100000)}) {
    thrust::host_vector<T> h(n);
    thrust::device_vector<T> dv(n);
    thrust::sequence(h.begin(), h.end(), T(3), T(2));
    thrust::sequence(dv.begin(), dv.end(), T(3), T(2));
    ASSERT_EQUAL(h, dv);
  }
}
DECLARE_TYPED_UNITTEST(TestSequence, int);
DECLARE_TYPED_UNITTEST(TestSequence, uint64_t);
DECLARE_TYPED_UNITTEST(TestSequence, float);

// testing/reduce.cu:29-49 (known answer), :67-84 (ladder)
void TestReduceSimple() {
  const int in[3] = {1, -2, 3};
  thrust::device_vector<int> d(in, in + 3);
  ASSERT_EQUAL(thrust::reduce(d.begin(), d.end()), 2);
  ASSERT_EQUAL(thrust::reduce(d.begin(), d.end(), 10), 12);
  ASSERT_EQUAL(thrust::reduce(d.begin(), d.end(), 0, max_of<int>()), 3);
  thrust::device_vector<int> empty;
  ASSERT_EQUAL(thrust::reduce(empty.begin(), empty.end(), 42), 42);
}
DECLARE_UNITTEST(TestReduceSimple);

template <class T>
void TestReduceLadder() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n);
    thrust::device_vector<T> d = h;
    // unsigned wrap-around arithmetic is exact and order-independent
    ASSERT_EQUAL(thrust::reduce(h.begin(), h.end(), T(13)), thrust::reduce(d.begin(), d.end(), T(13)));
    if (n) {
      ASSERT_EQUAL(thrust::reduce(h.begin(), h.end(), h[0], max_of<T>()),
                   thrust::reduce(thrust::device, d.begin(), d.end(), h[0], max_of<T>()));
    }
  }
}
DECLARE_TYPED_UNITTEST(TestReduceLadder, uint32_t);
DECLARE_TYPED_UNITTEST(TestReduceLadder, uint64_t);
DECLARE_TYPED_UNITTEST(TestReduceLadder, uint8_t);

void TestReduceFloat() {
  for (std::size_t n : {std::size_t(1000), std::size_t(1) << 20, (std::size_t(1) << 24) + 3}) {
    thrust::host_vector<float> h = unittest::random_samples<float>(n);
    thrust::device_vector<float> d = h;
    double ref = 0, l1 = 0;
    for (std::size_t i = 0; i < n; i++) { ref += h[i]; l1 += std::fabs(h[i]); }
    const float got = thrust::reduce(d.begin(), d.end(), 0.0f);
    ASSERT_TRUE(std::fabs((double)got - ref) <= 1e-5 * l1);  // tolerance relative to the L1 norm
  }
}
DECLARE_UNITTEST(TestReduceFloat);

// testing/transform_reduce.cu:20-38, testing/count.cu:20-60
void TestTransformReduceAndCount() {
  const int in[5] = {1, -2, 3, 4, 6};
  thrust::device_vector<int> d(in, in + 5);
  ASSERT_EQUAL(thrust::transform_reduce(d.begin(), d.end(), thrust::negate<int>(), 10, thrust::plus<int>()), -2);
  ASSERT_EQUAL(thrust::count_if(d.begin(), d.end(), is_even()), 3);
  ASSERT_EQUAL(thrust::count(d.begin(), d.end(), 3), 1);
  for (std::size_t n : {std::size_t(0), std::size_t(4097), std::size_t(2000001)}) {
    thrust::host_vector<int> h = unittest::random_integers<int>(n);
    thrust::device_vector<int> dv = h;
    ASSERT_EQUAL(thrust::count_if(h.begin(), h.end(), is_even()), thrust::count_if(dv.begin(), dv.end(), is_even()));
    ASSERT_EQUAL(thrust::transform_reduce(h.begin(), h.end(), times_two_plus_one<int>(), 5, max_of<int>()),
                 thrust::transform_reduce(dv.begin(), dv.end(), times_two_plus_one<int>(), 5, max_of<int>()));
  }
}
DECLARE_UNITTEST(TestTransformReduceAndCount);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

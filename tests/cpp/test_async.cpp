// thrust::async::* and device_event / device_future, in the shape of the reference's
// testing/async_copy.cu, async_for_each.cu, async_transform.cu, async_reduce.cu,
// async_reduce_into.cu, async_sort.cu and testing/async/{inclusive,exclusive}_scan: each
// asynchronous result equals the synchronous algorithm's; events become ready; dependencies
// given with thrust::device.after(...) are honoured.  Compiled by hipcc.
#include <algorithm>
#include <numeric>

#include <thrust/async/copy.h>
#include <thrust/async/for_each.h>
#include <thrust/async/reduce.h>
#include <thrust/async/scan.h>
#include <thrust/async/sort.h>
#include <thrust/async/transform.h>
#include <thrust/future.h>
#include <thrust/sequence.h>

#include "testing.h"

template <class T>
struct custom_plus {
  __host__ __device__ T operator()(T a, T b) const { return a + b; }
};
template <class T>
struct custom_greater {
  __host__ __device__ bool operator()(T a, T b) const { return a > b; }
};
template <class T>
struct twice {
  __host__ __device__ T operator()(T x) const { return (T)(2 * x); }
};
template <class T>
struct add_one_in_place {
  __host__ __device__ void operator()(T& x) const { x = (T)(x + 1); }
};

static const std::size_t kSizes[] = {0, 1, 2, 1000, 65537, 1048577};

// testing/async_copy.cu:22-120
template <class T>
void TestAsyncCopy() {
  for (std::size_t n : kSizes) {
    thrust::host_vector<T> h0 = unittest::random_integers<T>(n), h1(n);
    thrust::device_vector<T> d0(n), d1(n);
    auto e0 = thrust::async::copy(h0.begin(), h0.end(), d0.begin());             // host -> device
    auto e1 = thrust::async::copy(thrust::device.after(e0), d0.begin(), d0.end(), d1.begin());  // device -> device
    auto e2 = thrust::async::copy(thrust::device.after(e1), d1.begin(), d1.end(), h1.begin());  // device -> host
    e2.wait();
    ASSERT_TRUE(e2.ready());
    ASSERT_EQUAL(h0, h1);
    ASSERT_EQUAL(h0, d1);
  }
}
DECLARE_TYPED_UNITTEST(TestAsyncCopy, int);
DECLARE_TYPED_UNITTEST(TestAsyncCopy, double);
DECLARE_TYPED_UNITTEST(TestAsyncCopy, int8_t);

// testing/async_for_each.cu:60-110, async_transform.cu:60-120
template <class T>
void TestAsyncForEachTransform() {
  for (std::size_t n : kSizes) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n), ho(n);
    thrust::device_vector<T> d = h, dout(n);
    auto e = thrust::async::for_each(d.begin(), d.end(), add_one_in_place<T>());
    std::for_each(h.begin(), h.end(), add_one_in_place<T>());
    auto e2 = thrust::async::transform(thrust::device.after(e), d.begin(), d.end(), dout.begin(), twice<T>());
    std::transform(h.begin(), h.end(), ho.begin(), twice<T>());
    e2.wait();
    ASSERT_EQUAL(h, d);
    ASSERT_EQUAL(ho, dout);
  }
}
DECLARE_TYPED_UNITTEST(TestAsyncForEachTransform, int);
DECLARE_TYPED_UNITTEST(TestAsyncForEachTransform, uint16_t);
DECLARE_TYPED_UNITTEST(TestAsyncForEachTransform, int64_t);

// testing/async_reduce.cu:90-260, async_reduce_into.cu
template <class T>
void TestAsyncReduce() {
  for (std::size_t n : kSizes) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n);
    thrust::device_vector<T> d = h;
    const T want = std::accumulate(h.begin(), h.end(), T(0));
    auto f0 = thrust::async::reduce(d.begin(), d.end());
    auto f1 = thrust::async::reduce(thrust::device, d.begin(), d.end(), T(5));
    auto f2 = thrust::async::reduce(d.begin(), d.end(), T(7), custom_plus<T>());
    ASSERT_TRUE(f0.valid_stream());
    ASSERT_EQUAL(f0.get(), want);
    ASSERT_EQUAL(f0.get(), want);  // a second get returns the same value
    ASSERT_TRUE(f0.ready());
    ASSERT_EQUAL(f1.get(), (T)(want + T(5)));
    ASSERT_EQUAL(f2.extract(), (T)(want + T(7)));
    ASSERT_TRUE(!f2.valid_stream());
    ASSERT_EQUAL(thrust::reduce(d.begin(), d.end()), want);  // the synchronous one agrees
    thrust::device_vector<T> slot(1);
    auto e = thrust::async::reduce_into(d.begin(), d.end(), slot.begin(), T(3), custom_plus<T>());
    e.wait();
    ASSERT_EQUAL((T)slot[0], (T)(want + T(3)));
  }
}
DECLARE_TYPED_UNITTEST(TestAsyncReduce, int);
DECLARE_TYPED_UNITTEST(TestAsyncReduce, uint64_t);
DECLARE_TYPED_UNITTEST(TestAsyncReduce, int16_t);

// testing/async_sort.cu:20-160
template <class T>
void TestAsyncSort() {
  for (std::size_t n : kSizes) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n);
    thrust::device_vector<T> d0 = h, d1 = h, d2 = h;
    auto e0 = thrust::async::sort(d0.begin(), d0.end());
    auto e1 = thrust::async::sort(thrust::device, d1.begin(), d1.end(), thrust::greater<T>());
    auto e2 = thrust::async::stable_sort(d2.begin(), d2.end(), custom_greater<T>());  // comparison sort
    std::sort(h.begin(), h.end());
    e0.wait();
    ASSERT_EQUAL(h, d0);
    std::reverse(h.begin(), h.end());
    thrust::when_all(e1, e2).wait();
    ASSERT_EQUAL(h, d1);
    ASSERT_EQUAL(h, d2);
  }
}
DECLARE_TYPED_UNITTEST(TestAsyncSort, int);
DECLARE_TYPED_UNITTEST(TestAsyncSort, uint8_t);
DECLARE_TYPED_UNITTEST(TestAsyncSort, double);

// testing/async/inclusive_scan/simple.cu, exclusive_scan/simple.cu
template <class T>
void TestAsyncScan() {
  for (std::size_t n : kSizes) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n), hi(n), he(n);
    thrust::device_vector<T> d = h, di(n), de(n);
    auto e0 = thrust::async::inclusive_scan(d.begin(), d.end(), di.begin());
    auto e1 = thrust::async::exclusive_scan(thrust::device, d.begin(), d.end(), de.begin(), T(11), thrust::plus<T>());
    thrust::inclusive_scan(h.begin(), h.end(), hi.begin());
    thrust::exclusive_scan(h.begin(), h.end(), he.begin(), T(11), thrust::plus<T>());
    e0.wait();
    e1.wait();
    ASSERT_EQUAL(hi, di);
    ASSERT_EQUAL(he, de);
  }
}
DECLARE_TYPED_UNITTEST(TestAsyncScan, int);
DECLARE_TYPED_UNITTEST(TestAsyncScan, uint64_t);

// a chain across streams: fill -> sort -> scan -> reduce, every step after the one before
void TestAsyncDependencyChain() {
  const std::size_t n = 1 << 22;
  thrust::device_vector<int> a(n), b(n);
  thrust::sequence(a.begin(), a.end());
  auto e0 = thrust::async::transform(a.begin(), a.end(), a.begin(), twice<int>());           // 0, 2, 4, ...
  auto e1 = thrust::async::sort(thrust::device.after(e0), a.begin(), a.end(), thrust::greater<int>());
  auto e2 = thrust::async::inclusive_scan(thrust::device.after(e1), a.begin(), a.end(), b.begin(), thrust::maximum<int>());
  auto f = thrust::async::reduce(thrust::device.after(e2), b.begin(), b.end(), 0ll, thrust::plus<long long>());
  const long long top = 2ll * (long long)(n - 1);
  ASSERT_EQUAL(f.get(), top * (long long)n);  // the running maximum of a descending range is its first element
  ASSERT_TRUE(f.ready());
  // thrust::device.after(e) consumes e (testing/async_copy.cu:325-375): the chain ran on e0's stream
  ASSERT_TRUE(!e0.valid_stream() && !e1.valid_stream() && !e2.valid_stream());
  ASSERT_THROWS(thrust::device.after(e0), thrust::event_error);
  // an event moved from has no state; a default event neither
  thrust::device_event fresh = thrust::when_all();
  thrust::device_event moved = std::move(fresh);
  ASSERT_TRUE(!fresh.valid_stream());
  ASSERT_TRUE(moved.valid_stream());
  thrust::device_event none;
  ASSERT_TRUE(!none.valid_stream() && !none.ready());
  ASSERT_THROWS(none.wait(), std::logic_error);
  // the error carries the reference's code (testing/event.cu:39-50, testing/async_reduce.cu:797-821)
  try {
    none.wait();
    ASSERT_TRUE(false);
  } catch (const thrust::event_error& e) {
    ASSERT_TRUE(e == thrust::event_error(thrust::event_errc::no_state));
    ASSERT_TRUE(e.code().category() == thrust::event_category());
  }
  thrust::device_future<int> empty;
  ASSERT_THROWS(empty.get(), thrust::event_error);
  static_assert(std::is_same<thrust::device_unique_eager_event, thrust::device_event>::value, "");
  static_assert(std::is_same<thrust::unique_eager_future<thrust::device_system_tag, int>, thrust::device_future<int>>::value, "");
}
DECLARE_UNITTEST(TestAsyncDependencyChain);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

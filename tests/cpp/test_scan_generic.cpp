// scan / scan_by_key / reduce_by_key with user-defined operators and predicates, accumulator
// types that differ from the element type, struct elements and fancy iterators read in place: the
// kernel-template path (compiled by hipcc).  In the shape of the reference's testing/scan.cu:250-343,
// testing/scan_by_key.inclusive.cu:134-177, testing/reduce_by_key.cu:15-112 and
// testing/cuda/reduce_by_key.cu:339-400; device results are compared with the host path's.
#include <thrust/functional.h>
#include <thrust/iterator/constant_iterator.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/discard_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>

#include "testing.h"

template <class T>
thrust::host_vector<T> hv(std::initializer_list<double> v) {
  thrust::host_vector<T> r;
  for (double x : v) r.push_back((T)x);
  return r;
}

// ------------------------------------------------------------------ accumulator types
// testing/scan.cu:250-320
void TestScanMixedTypes() {
  thrust::device_vector<int> int_input = hv<int>({1, 2, 3, 4}), int_output(4);
  thrust::device_vector<float> float_input = hv<float>({1.5, 2.5, 3.5, 4.5}), float_output(4);

  // float -> int: plus<> and a float accumulator
  thrust::inclusive_scan(float_input.begin(), float_input.end(), int_output.begin());
  ASSERT_EQUAL(int_output, hv<int>({1, 4, 7, 12}));
  // float -> float with plus<int> (float accumulator, every sum truncated)
  thrust::inclusive_scan(float_input.begin(), float_input.end(), float_output.begin(), thrust::plus<int>());
  ASSERT_EQUAL(float_output, hv<float>({1.5, 3.0, 6.0, 10.0}));
  // float -> int, default init: float accumulator
  thrust::exclusive_scan(float_input.begin(), float_input.end(), int_output.begin());
  ASSERT_EQUAL(int_output, hv<int>({0, 1, 4, 7}));
  // float -> int with a float init
  thrust::exclusive_scan(float_input.begin(), float_input.end(), int_output.begin(), (float)5.5);
  ASSERT_EQUAL(int_output, hv<int>({5, 7, 9, 13}));
  // int -> float: int accumulator
  thrust::inclusive_scan(int_input.begin(), int_input.end(), float_output.begin());
  ASSERT_EQUAL(float_output, hv<float>({1, 3, 6, 10}));
  // int -> float with a float init: float accumulator
  thrust::exclusive_scan(int_input.begin(), int_input.end(), float_output.begin(), (float)5.5);
  ASSERT_EQUAL(float_output, hv<float>({5.5, 6.5, 8.5, 11.5}));
}
DECLARE_UNITTEST(TestScanMixedTypes);

// ------------------------------------------------------------------ user operators
template <class T>
struct max_functor {
  __host__ __device__ T operator()(T rhs, T lhs) const { return rhs < lhs ? lhs : rhs; }
};

// testing/scan.cu:324-343 over the size ladder
template <class T>
void TestScanWithOperator() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h_input = unittest::random_integers<T>(n);
    thrust::device_vector<T> d_input = h_input;
    thrust::host_vector<T> h_output(n);
    thrust::device_vector<T> d_output(n);
    thrust::inclusive_scan(h_input.begin(), h_input.end(), h_output.begin(), max_functor<T>());
    thrust::inclusive_scan(d_input.begin(), d_input.end(), d_output.begin(), max_functor<T>());
    ASSERT_EQUAL(d_output, h_output);
    thrust::exclusive_scan(h_input.begin(), h_input.end(), h_output.begin(), T(13), max_functor<T>());
    thrust::exclusive_scan(d_input.begin(), d_input.end(), d_output.begin(), T(13), max_functor<T>());
    ASSERT_EQUAL(d_output, h_output);
    // in place
    thrust::inclusive_scan(d_input.begin(), d_input.end(), d_input.begin(), max_functor<T>());
    thrust::inclusive_scan(h_input.begin(), h_input.end(), h_input.begin(), max_functor<T>());
    ASSERT_EQUAL(d_input, h_input);
  }
}
DECLARE_TYPED_UNITTEST(TestScanWithOperator, int8_t);
DECLARE_TYPED_UNITTEST(TestScanWithOperator, int16_t);
DECLARE_TYPED_UNITTEST(TestScanWithOperator, int32_t);
DECLARE_TYPED_UNITTEST(TestScanWithOperator, int64_t);

// an associative operator that does not commute: composition of affine maps x -> a*x + b
// (mod 2^32), each map a struct of two words
struct affine {
  unsigned a, b;
  __host__ __device__ bool operator==(const affine& o) const { return a == o.a && b == o.b; }
};
std::ostream& operator<<(std::ostream& os, const affine& f) { return os << "(" << f.a << "," << f.b << ")"; }
struct compose {  // first f, then g
  __host__ __device__ affine operator()(const affine& f, const affine& g) const { return affine{g.a * f.a, g.a * f.b + g.b}; }
};
void TestScanNonCommutativeStructOperator() {
  for (std::size_t n : {std::size_t(1), std::size_t(2), std::size_t(63), std::size_t(513), std::size_t(4097), std::size_t(100003), std::size_t(1) << 21}) {
    thrust::host_vector<affine> h(n);
    std::uint64_t s = 99 + n;
    for (auto& f : h) {
      const std::uint64_t r = unittest::splitmix64(s);
      f = affine{(unsigned)r | 1u, (unsigned)(r >> 32)};
    }
    thrust::device_vector<affine> d = h, d_out(n);
    thrust::host_vector<affine> h_out(n);
    thrust::inclusive_scan(h.begin(), h.end(), h_out.begin(), compose());
    thrust::inclusive_scan(d.begin(), d.end(), d_out.begin(), compose());
    ASSERT_EQUAL(d_out, h_out);
    const affine init{3u, 5u};
    thrust::exclusive_scan(h.begin(), h.end(), h_out.begin(), init, compose());
    thrust::exclusive_scan(d.begin(), d.end(), d_out.begin(), init, compose());
    ASSERT_EQUAL(d_out, h_out);
  }
}
DECLARE_UNITTEST(TestScanNonCommutativeStructOperator);

// scan of a counting / transform iterator (read in place) into a discard iterator and a vector
struct square {
  __host__ __device__ std::int64_t operator()(std::int64_t x) const { return x * x; }
};
void TestScanFancyIterators() {
  const std::int64_t n = 1234567;
  thrust::device_vector<std::int64_t> out(n);
  auto first = thrust::make_transform_iterator(thrust::counting_iterator<std::int64_t>(0), square());
  thrust::inclusive_scan(thrust::device, first, first + n, out.begin());
  thrust::host_vector<std::int64_t> h = out;
  for (std::int64_t i : {std::int64_t(0), std::int64_t(1), std::int64_t(4095), std::int64_t(4096), n - 1})
    ASSERT_EQUAL(h[i], i * (i + 1) * (2 * i + 1) / 6);  // sum of squares
  thrust::exclusive_scan(thrust::device, first, first + n, thrust::make_discard_iterator(), std::int64_t(0));  // compiles and runs
}
DECLARE_UNITTEST(TestScanFancyIterators);

// ------------------------------------------------------------------ scan_by_key
// testing/scan_by_key.inclusive.cu:134-177
struct head_flag_predicate {
  template <class T>
  __host__ __device__ bool operator()(const T&, const T& b) const { return b ? false : true; }
};
template <class T>
void TestScanByKeyHeadFlags() {
  thrust::device_vector<T> keys = hv<T>({0, 1, 0, 0, 1, 1, 0}), vals = hv<T>({1, 2, 3, 4, 5, 6, 7}), output(7, 0);
  thrust::inclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin(), head_flag_predicate(), thrust::plus<T>());
  ASSERT_EQUAL(output, hv<T>({1, 2, 5, 9, 5, 6, 13}));
  thrust::exclusive_scan_by_key(keys.begin(), keys.end(), vals.begin(), output.begin(), T(10), head_flag_predicate(), thrust::plus<T>());
  ASSERT_EQUAL(output, hv<T>({10, 10, 12, 15, 10, 10, 16}));
}
DECLARE_TYPED_UNITTEST(TestScanByKeyHeadFlags, int);
DECLARE_TYPED_UNITTEST(TestScanByKeyHeadFlags, float);
DECLARE_TYPED_UNITTEST(TestScanByKeyHeadFlags, int64_t);

template <class T>
struct is_equal_div_10 {
  __host__ __device__ bool operator()(const T x, const T& y) const { return ((int)x / 10) == ((int)y / 10); }
};
template <class T>
void TestScanByKeyWithPredicateAndOperatorLadder() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> hk(n), hvals = unittest::random_integers<T>(n, 5);
    std::uint64_t s = 7 + n;
    T cur = 0;
    for (std::size_t i = 0; i < n; i++) {  // runs of 1..40 equal tens
      if (unittest::splitmix64(s) % 17 == 0) cur = (T)((cur + 10) % 120);
      hk[i] = (T)(cur + (T)(unittest::splitmix64(s) % 10));
    }
    thrust::device_vector<T> dk = hk, dv = hvals, dout(n);
    thrust::host_vector<T> hout(n);
    thrust::inclusive_scan_by_key(hk.begin(), hk.end(), hvals.begin(), hout.begin(), is_equal_div_10<T>(), max_functor<T>());
    thrust::inclusive_scan_by_key(dk.begin(), dk.end(), dv.begin(), dout.begin(), is_equal_div_10<T>(), max_functor<T>());
    ASSERT_EQUAL(dout, hout);
    thrust::exclusive_scan_by_key(hk.begin(), hk.end(), hvals.begin(), hout.begin(), T(13), is_equal_div_10<T>(), max_functor<T>());
    thrust::exclusive_scan_by_key(dk.begin(), dk.end(), dv.begin(), dout.begin(), T(13), is_equal_div_10<T>(), max_functor<T>());
    ASSERT_EQUAL(dout, hout);
  }
}
DECLARE_TYPED_UNITTEST(TestScanByKeyWithPredicateAndOperatorLadder, int32_t);
DECLARE_TYPED_UNITTEST(TestScanByKeyWithPredicateAndOperatorLadder, int16_t);

// ------------------------------------------------------------------ reduce_by_key
// testing/reduce_by_key.cu:15-112
template <class T>
void TestReduceByKeySimple() {
  thrust::device_vector<T> keys = hv<T>({11, 11, 21, 20, 21, 21, 21, 37, 37}), values = hv<T>({0, 1, 2, 3, 4, 5, 6, 7, 8});
  thrust::device_vector<T> output_keys(9), output_values(9);
  auto new_last = thrust::reduce_by_key(keys.begin(), keys.end(), values.begin(), output_keys.begin(), output_values.begin(),
                                        is_equal_div_10<T>());
  ASSERT_EQUAL(new_last.first - output_keys.begin(), 3);
  ASSERT_EQUAL(new_last.second - output_values.begin(), 3);
  output_keys.resize(3);
  output_values.resize(3);
  ASSERT_EQUAL(output_keys, hv<T>({11, 21, 37}));
  ASSERT_EQUAL(output_values, hv<T>({1, 20, 15}));
}
DECLARE_TYPED_UNITTEST(TestReduceByKeySimple, int);
DECLARE_TYPED_UNITTEST(TestReduceByKeySimple, int8_t);
DECLARE_TYPED_UNITTEST(TestReduceByKeySimple, uint64_t);

template <class T>
void TestReduceByKeyWithPredicateAndOperatorLadder() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> hk(n), hvals = unittest::random_integers<T>(n, 6);
    std::uint64_t s = 11 + n;
    T cur = 0;
    for (std::size_t i = 0; i < n; i++) {
      if (unittest::splitmix64(s) % 5 == 0) cur = (T)((cur + 10) % 120);
      hk[i] = (T)(cur + (T)(unittest::splitmix64(s) % 10));
    }
    thrust::device_vector<T> dk = hk, dv = hvals, dko(n), dvo(n);
    thrust::host_vector<T> hko(n), hvo(n);
    auto hend = thrust::reduce_by_key(hk.begin(), hk.end(), hvals.begin(), hko.begin(), hvo.begin(), is_equal_div_10<T>(), max_functor<T>());
    auto dend = thrust::reduce_by_key(dk.begin(), dk.end(), dv.begin(), dko.begin(), dvo.begin(), is_equal_div_10<T>(), max_functor<T>());
    ASSERT_EQUAL(dend.first - dko.begin(), hend.first - hko.begin());
    ASSERT_EQUAL(dend.second - dvo.begin(), hend.second - hvo.begin());
    const std::size_t r = (std::size_t)(hend.first - hko.begin());
    dko.resize(r); dvo.resize(r); hko.resize(r); hvo.resize(r);
    ASSERT_EQUAL(dko, hko);
    ASSERT_EQUAL(dvo, hvo);
  }
}
DECLARE_TYPED_UNITTEST(TestReduceByKeyWithPredicateAndOperatorLadder, int32_t);
DECLARE_TYPED_UNITTEST(TestReduceByKeyWithPredicateAndOperatorLadder, int64_t);

// testing/cuda/reduce_by_key.cu:339-400: keys and values are transform iterators over a counting
// iterator (nothing is materialised), 2^magnitude items in 256 runs
struct div_op {
  std::int64_t d;
  __host__ __device__ std::int64_t operator()(std::int64_t x) const { return x / d; }
};
struct mod_op {
  std::int64_t d;
  __host__ __device__ std::int64_t operator()(std::int64_t x) const { return (x % d) + (x / d); }
};
void TestReduceByKeyWithBigIndexesHelper(int magnitude) {
  const std::int64_t num_items = 1ll << magnitude, num_unique_keys = 1ll << 8, key_size = num_items / num_unique_keys;
  thrust::counting_iterator<std::int64_t> count_begin(0ll);
  auto keys_begin = thrust::make_transform_iterator(count_begin, div_op{key_size});
  auto values_begin = thrust::make_transform_iterator(count_begin, mod_op{key_size});
  thrust::device_vector<std::int64_t> output_keys(num_unique_keys), output_values(num_unique_keys);
  auto end = thrust::reduce_by_key(thrust::device, keys_begin, keys_begin + num_items, values_begin, output_keys.begin(), output_values.begin());
  ASSERT_EQUAL(end.first - output_keys.begin(), num_unique_keys);
  thrust::host_vector<std::int64_t> keys = output_keys, result = output_values;
  const std::int64_t sum = (key_size - 1) * key_size / 2;
  for (std::int64_t key_id = 0; key_id < num_unique_keys; key_id++) {
    ASSERT_EQUAL(keys[key_id], key_id);
    ASSERT_EQUAL(result[key_id], sum + key_id * key_size);
  }
}
void TestReduceByKeyWithBigIndexes() {
  TestReduceByKeyWithBigIndexesHelper(30);
  TestReduceByKeyWithBigIndexesHelper(31);
  TestReduceByKeyWithBigIndexesHelper(32);
  TestReduceByKeyWithBigIndexesHelper(33);
}
DECLARE_UNITTEST(TestReduceByKeyWithBigIndexes);

// run-length encoding of a counting pattern through a constant iterator of ones
// (examples/run_length_encoding.cu pattern with fancy inputs and a user predicate)
void TestReduceByKeyConstantIteratorValues() {
  const std::int64_t n = 1 << 22;
  auto keys = thrust::make_transform_iterator(thrust::counting_iterator<std::int64_t>(0), div_op{1000});
  thrust::device_vector<std::int64_t> ko(n / 1000 + 1);
  thrust::device_vector<int> lengths(n / 1000 + 1);
  auto end = thrust::reduce_by_key(thrust::device, keys, keys + n, thrust::constant_iterator<int>(1), ko.begin(), lengths.begin());
  const std::int64_t r = end.first - ko.begin();
  ASSERT_EQUAL(r, n / 1000 + 1);
  thrust::host_vector<int> h = lengths;
  for (std::int64_t i = 0; i + 1 < r; i++) ASSERT_EQUAL(h[i], 1000);
  ASSERT_EQUAL(h[r - 1], (int)(n % 1000));
}
DECLARE_UNITTEST(TestReduceByKeyConstantIteratorValues);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

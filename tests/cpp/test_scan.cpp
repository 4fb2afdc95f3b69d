// Scan tests in the shape of the reference's testing/scan.cu.
#include <thrust/functional.h>
#include <thrust/scan.h>

#include "testing.h"

// testing/scan.cu:25-107
template <class T>
void TestScanSimple() {
  const T in[5] = {1, 3, (T)-2, 4, (T)-5};
  thrust::device_vector<T> input(in, in + 5), output(5);
  thrust::host_vector<T> input_copy(in, in + 5);
  auto expect = [](std::initializer_list<int> v) {
    thrust::host_vector<T> r;
    for (int x : v) r.push_back((T)x);
    return r;
  };
  auto it = thrust::inclusive_scan(input.begin(), input.end(), output.begin());
  ASSERT_EQUAL(std::size_t(it - output.begin()), input.size());
  ASSERT_EQUAL(input, input_copy);
  ASSERT_EQUAL(output, expect({1, 4, 2, 6, 1}));
  it = thrust::exclusive_scan(input.begin(), input.end(), output.begin(), T(0));
  ASSERT_EQUAL(std::size_t(it - output.begin()), input.size());
  ASSERT_EQUAL(output, expect({0, 1, 4, 2, 6}));
  thrust::exclusive_scan(input.begin(), input.end(), output.begin(), T(3));
  ASSERT_EQUAL(output, expect({3, 4, 7, 5, 9}));
  thrust::inclusive_scan(input.begin(), input.end(), output.begin(), thrust::plus<T>());
  ASSERT_EQUAL(output, expect({1, 4, 2, 6, 1}));
  thrust::exclusive_scan(input.begin(), input.end(), output.begin(), T(3), thrust::plus<T>());
  ASSERT_EQUAL(output, expect({3, 4, 7, 5, 9}));
  // in place
  thrust::inclusive_scan(input.begin(), input.end(), input.begin());
  ASSERT_EQUAL(input, expect({1, 4, 2, 6, 1}));
  input = input_copy;
  thrust::exclusive_scan(input.begin(), input.end(), input.begin(), T(3));
  ASSERT_EQUAL(input, expect({3, 4, 7, 5, 9}));
  input = input_copy;
  thrust::exclusive_scan(input.begin(), input.end(), input.begin());
  ASSERT_EQUAL(input, expect({0, 1, 4, 2, 6}));
}
DECLARE_TYPED_UNITTEST(TestScanSimple, int);
DECLARE_TYPED_UNITTEST(TestScanSimple, short);
DECLARE_TYPED_UNITTEST(TestScanSimple, int8_t);
DECLARE_TYPED_UNITTEST(TestScanSimple, int64_t);
DECLARE_TYPED_UNITTEST(TestScanSimple, float);
DECLARE_TYPED_UNITTEST(TestScanSimple, double);

// testing/scan.cu:378-415: host vs device over the size ladder, integral types (wraparound included)
template <class T>
void TestScan() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h_in = unittest::random_integers<T>(n);
    thrust::device_vector<T> d_in = h_in;
    thrust::host_vector<T> h_out(n);
    thrust::device_vector<T> d_out(n);
    thrust::inclusive_scan(h_in.begin(), h_in.end(), h_out.begin());
    thrust::inclusive_scan(d_in.begin(), d_in.end(), d_out.begin());
    ASSERT_EQUAL(d_out, h_out);
    thrust::exclusive_scan(h_in.begin(), h_in.end(), h_out.begin());
    thrust::exclusive_scan(d_in.begin(), d_in.end(), d_out.begin());
    ASSERT_EQUAL(d_out, h_out);
    thrust::exclusive_scan(h_in.begin(), h_in.end(), h_out.begin(), (T)11);
    thrust::exclusive_scan(d_in.begin(), d_in.end(), d_out.begin(), (T)11);
    ASSERT_EQUAL(d_out, h_out);
    // in place
    thrust::host_vector<T> h2 = h_in;
    thrust::device_vector<T> d2 = d_in;
    thrust::inclusive_scan(h2.begin(), h2.end(), h2.begin());
    thrust::inclusive_scan(d2.begin(), d2.end(), d2.begin());
    ASSERT_EQUAL(d2, h2);
  }
}
DECLARE_TYPED_UNITTEST(TestScan, int);
DECLARE_TYPED_UNITTEST(TestScan, uint32_t);
DECLARE_TYPED_UNITTEST(TestScan, int8_t);
DECLARE_TYPED_UNITTEST(TestScan, uint16_t);
DECLARE_TYPED_UNITTEST(TestScan, int64_t);

void TestScanOtherOperators() {
  const std::size_t n = 100003;
  thrust::host_vector<int> h = unittest::random_integers<int>(n);
  thrust::device_vector<int> d = h;
  thrust::host_vector<int> ho(n);
  thrust::device_vector<int> dout(n);
  thrust::inclusive_scan(h.begin(), h.end(), ho.begin(), thrust::maximum<int>());
  thrust::inclusive_scan(d.begin(), d.end(), dout.begin(), thrust::maximum<int>());
  ASSERT_EQUAL(dout, ho);
  thrust::exclusive_scan(h.begin(), h.end(), ho.begin(), 5, thrust::minimum<int>());
  thrust::exclusive_scan(d.begin(), d.end(), dout.begin(), 5, thrust::minimum<int>());
  ASSERT_EQUAL(dout, ho);
  thrust::inclusive_scan(h.begin(), h.end(), ho.begin(), thrust::multiplies<int>());
  thrust::inclusive_scan(d.begin(), d.end(), dout.begin(), thrust::multiplies<int>());
  ASSERT_EQUAL(dout, ho);
}
DECLARE_UNITTEST(TestScanOtherOperators);

// fp32: a reassociated sum; |gpu - serial| <= 1e-5 * running L1 norm
void TestScanFloatTolerance() {
  const std::size_t n = 1 << 20;
  thrust::host_vector<float> h = unittest::random_samples<float>(n);
  for (auto& x : h) x /= 100.0f;  // [-1, 1)
  thrust::device_vector<float> d = h;
  thrust::host_vector<float> ho(n);
  thrust::device_vector<float> dout(n);
  thrust::inclusive_scan(h.begin(), h.end(), ho.begin());
  thrust::inclusive_scan(d.begin(), d.end(), dout.begin());
  thrust::host_vector<float> got(dout);
  double l1 = 0;
  for (std::size_t i = 0; i < n; i++) {
    l1 += std::abs((double)h[i]);
    ASSERT_TRUE(std::abs((double)got[i] - (double)ho[i]) <= 1e-5 * l1);
  }
}
DECLARE_UNITTEST(TestScanFloatTolerance);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

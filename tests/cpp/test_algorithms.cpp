// generate / tabulate / gather / scatter / replace / reverse / find / mismatch / equal / logical /
// inner_product / extrema / transform_scan / swap_ranges / is_sorted / random / placeholders on
// device ranges against the same call on host ranges, over the reference's size ladder, plus the
// known answers of the reference's tests (testing/gather.cu:20-47, scatter.cu:19-45,
// replace.cu:23-46, reverse.cu:8-33, find.cu:33-62, mismatch.cu:6-33, equal.cu:8-40,
// logical.cu:9-54, inner_product.cu:10-24, min_element.cu:7-30, max_element.cu:7-30,
// minmax_element.cu:7-30, transform_scan.cu:60-120, is_sorted.cu:7-30, tabulate.cu:48-75).
#include <thrust/equal.h>
#include <thrust/extrema.h>
#include <thrust/find.h>
#include <thrust/functional.h>
#include <thrust/gather.h>
#include <thrust/generate.h>
#include <thrust/inner_product.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/logical.h>
#include <thrust/mismatch.h>
#include <thrust/optional.h>
#include <thrust/partition.h>
#include <thrust/binary_search.h>
#include <thrust/transform.h>
#include <thrust/unique.h>
#include <thrust/random.h>
#include <thrust/replace.h>
#include <thrust/reverse.h>
#include <thrust/scatter.h>
#include <thrust/sequence.h>
#include <thrust/shuffle.h>
#include <thrust/sort.h>
#include <thrust/swap.h>
#include <thrust/tabulate.h>
#include <thrust/transform_scan.h>

#include <random>

#include "testing.h"

template <class T>
thrust::host_vector<T> hv(std::initializer_list<double> v) {
  thrust::host_vector<T> r;
  for (double x : v) r.push_back((T)x);
  return r;
}
template <class T>
thrust::host_vector<T> small_values(std::size_t n, std::uint64_t seed, int range) {
  thrust::host_vector<T> v(n);
  std::uint64_t s = seed + n;
  for (auto& x : v) x = (T)(unittest::splitmix64(s) % (std::uint64_t)range);
  return v;
}

// ------------------------------------------------------------------ gather / scatter
void TestGatherScatterSimple() {
  thrust::device_vector<int> map = hv<int>({6, 2, 1, 7, 2}), src = hv<int>({0, 1, 2, 3, 4, 5, 6, 7}), dst(5, 0);
  thrust::gather(map.begin(), map.end(), src.begin(), dst.begin());
  ASSERT_EQUAL(dst, hv<int>({6, 2, 1, 7, 2}));
  thrust::device_vector<int> smap = hv<int>({6, 3, 1, 7, 2}), ssrc = hv<int>({0, 1, 2, 3, 4}), sdst(8, 0);
  thrust::scatter(ssrc.begin(), ssrc.end(), smap.begin(), sdst.begin());
  ASSERT_EQUAL(sdst, hv<int>({0, 2, 4, 1, 0, 0, 0, 3}));
  thrust::device_vector<int> flags = hv<int>({0, 1, 0, 1, 0}), gdst(5, 9);
  thrust::gather_if(map.begin(), map.end(), flags.begin(), src.begin(), gdst.begin());
  ASSERT_EQUAL(gdst, hv<int>({9, 2, 9, 7, 9}));
  thrust::device_vector<int> sdst2(8, 0);
  thrust::scatter_if(ssrc.begin(), ssrc.end(), smap.begin(), flags.begin(), sdst2.begin());
  ASSERT_EQUAL(sdst2, hv<int>({0, 0, 0, 1, 0, 0, 0, 3}));
}
DECLARE_UNITTEST(TestGatherScatterSimple);

template <class T>
void TestGatherScatterLadder() {
  for (std::size_t n : unittest::sizes()) {
    const std::size_t src_n = n ? 2 * n + 3 : 1;
    thrust::host_vector<T> h_src = unittest::random_integers<T>(src_n);
    thrust::host_vector<unsigned> h_map(n);
    std::uint64_t s = 3 + n;
    for (auto& m : h_map) m = (unsigned)(unittest::splitmix64(s) % src_n);
    thrust::device_vector<T> d_src = h_src, d_out(n);
    thrust::device_vector<unsigned> d_map = h_map;
    thrust::host_vector<T> h_out(n);
    thrust::gather(h_map.begin(), h_map.end(), h_src.begin(), h_out.begin());
    thrust::gather(d_map.begin(), d_map.end(), d_src.begin(), d_out.begin());
    ASSERT_EQUAL(d_out, h_out);
    // scatter through a permutation (a map with repeated targets would race, as in the reference)
    thrust::host_vector<unsigned> h_perm(n);
    for (std::size_t i = 0; i < n; i++) h_perm[i] = (unsigned)((i * 7919u + 13u) % (n ? n : 1));
    if (n % 7919 == 0 && n) continue;  // not a permutation then
    thrust::device_vector<unsigned> d_perm = h_perm;
    thrust::host_vector<T> h_in = unittest::random_integers<T>(n, 17), h_sc(n, T(0));
    thrust::device_vector<T> d_in = h_in, d_sc(n, T(0));
    thrust::scatter(h_in.begin(), h_in.end(), h_perm.begin(), h_sc.begin());
    thrust::scatter(d_in.begin(), d_in.end(), d_perm.begin(), d_sc.begin());
    ASSERT_EQUAL(d_sc, h_sc);
  }
}
DECLARE_TYPED_UNITTEST(TestGatherScatterLadder, int32_t);
DECLARE_TYPED_UNITTEST(TestGatherScatterLadder, int8_t);
DECLARE_TYPED_UNITTEST(TestGatherScatterLadder, int64_t);

// ------------------------------------------------------------------ replace / reverse / swap_ranges
template <class T>
struct less_than_five {
  __host__ __device__ bool operator()(const T& x) const { return x < T(5); }
};
template <class T>
void TestReplaceReverseSwapLadder() {
  ASSERT_EQUAL((thrust::device_vector<T>(hv<T>({1, 2, 1, 3, 2}))).size(), std::size_t(5));
  {
    thrust::device_vector<T> d = hv<T>({1, 2, 1, 3, 2});
    thrust::replace(d.begin(), d.end(), T(1), T(4));
    thrust::replace(d.begin(), d.end(), T(2), T(5));
    ASSERT_EQUAL(d, hv<T>({4, 5, 4, 3, 5}));  // testing/replace.cu:23-46
    thrust::reverse(d.begin(), d.end());
    ASSERT_EQUAL(d, hv<T>({5, 3, 4, 5, 4}));
  }
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h = small_values<T>(n, 1, 10), h2 = small_values<T>(n, 2, 10), ho(n);
    thrust::device_vector<T> d = h, d2 = h2, dout(n);
    thrust::replace_copy_if(h.begin(), h.end(), ho.begin(), less_than_five<T>(), T(7));
    thrust::replace_copy_if(d.begin(), d.end(), dout.begin(), less_than_five<T>(), T(7));
    ASSERT_EQUAL(dout, ho);
    thrust::replace_copy(h.begin(), h.end(), ho.begin(), T(3), T(9));
    thrust::replace_copy(d.begin(), d.end(), dout.begin(), T(3), T(9));
    ASSERT_EQUAL(dout, ho);
    thrust::replace_if(h.begin(), h.end(), h2.begin(), less_than_five<T>(), T(0));  // stencil form
    thrust::replace_if(d.begin(), d.end(), d2.begin(), less_than_five<T>(), T(0));
    ASSERT_EQUAL(d, h);
    thrust::reverse_copy(h.begin(), h.end(), ho.begin());
    thrust::reverse_copy(d.begin(), d.end(), dout.begin());
    ASSERT_EQUAL(dout, ho);
    thrust::reverse(h.begin(), h.end());
    thrust::reverse(d.begin(), d.end());
    ASSERT_EQUAL(d, h);
    thrust::swap_ranges(h.begin(), h.end(), h2.begin());
    thrust::swap_ranges(d.begin(), d.end(), d2.begin());
    ASSERT_EQUAL(d, h);
    ASSERT_EQUAL(d2, h2);
  }
}
DECLARE_TYPED_UNITTEST(TestReplaceReverseSwapLadder, int32_t);
DECLARE_TYPED_UNITTEST(TestReplaceReverseSwapLadder, int16_t);
DECLARE_TYPED_UNITTEST(TestReplaceReverseSwapLadder, double);

// ------------------------------------------------------------------ find / mismatch / equal / logical
template <class T>
struct equal_to_value_pred {
  T value;
  __host__ __device__ bool operator()(T v) const { return v == value; }
};
void TestFindSimple() {  // testing/find.cu:33-62
  thrust::device_vector<int> vec = hv<int>({1, 2, 3, 3, 5});
  ASSERT_EQUAL(thrust::find(vec.begin(), vec.end(), 0) - vec.begin(), 5);
  ASSERT_EQUAL(thrust::find(vec.begin(), vec.end(), 1) - vec.begin(), 0);
  ASSERT_EQUAL(thrust::find(vec.begin(), vec.end(), 3) - vec.begin(), 2);
  ASSERT_EQUAL(thrust::find(vec.begin(), vec.end(), 5) - vec.begin(), 4);
  ASSERT_EQUAL(thrust::find_if(vec.begin(), vec.end(), equal_to_value_pred<int>{3}) - vec.begin(), 2);
  ASSERT_EQUAL(thrust::find_if_not(vec.begin(), vec.end(), equal_to_value_pred<int>{1}) - vec.begin(), 1);
  thrust::device_vector<int> a = hv<int>({1, 2, 3, 4}), b = hv<int>({1, 2, 4, 3});
  ASSERT_EQUAL(thrust::mismatch(a.begin(), a.end(), b.begin()).first - a.begin(), 2);  // testing/mismatch.cu:6-33
  b = a;
  ASSERT_EQUAL(thrust::mismatch(a.begin(), a.end(), b.begin()).first - a.begin(), 4);
  ASSERT_TRUE(thrust::equal(a.begin(), a.end(), b.begin()));
  b[3] = 9;
  ASSERT_TRUE(!thrust::equal(a.begin(), a.end(), b.begin()));
  ASSERT_TRUE(thrust::equal(a.begin(), a.begin() + 3, b.begin()));
  thrust::device_vector<int> v3 = hv<int>({1, 1, 0});  // testing/logical.cu:9-54
  ASSERT_TRUE(thrust::all_of(v3.begin(), v3.begin(), thrust::identity<int>()));
  ASSERT_TRUE(thrust::all_of(v3.begin(), v3.begin() + 2, thrust::identity<int>()));
  ASSERT_TRUE(!thrust::all_of(v3.begin(), v3.end(), thrust::identity<int>()));
  ASSERT_TRUE(thrust::any_of(v3.begin(), v3.end(), thrust::identity<int>()));
  ASSERT_TRUE(!thrust::any_of(v3.begin() + 2, v3.end(), thrust::identity<int>()));
  ASSERT_TRUE(thrust::none_of(v3.begin() + 2, v3.end(), thrust::identity<int>()));
  ASSERT_TRUE(!thrust::none_of(v3.begin(), v3.end(), thrust::identity<int>()));
}
DECLARE_UNITTEST(TestFindSimple);

template <class T>
void TestFindMismatchLadder() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h = small_values<T>(n, 9, 1000);
    thrust::device_vector<T> d = h;
    for (T needle : {T(0), T(7), T(999), T(5000)}) {
      ASSERT_EQUAL(thrust::find(d.begin(), d.end(), needle) - d.begin(), thrust::find(h.begin(), h.end(), needle) - h.begin());
    }
    thrust::host_vector<T> h2 = h;
    if (n > 3) h2[n - 2] = T(h2[n - 2] + 1);
    thrust::device_vector<T> d2 = h2;
    ASSERT_EQUAL(thrust::mismatch(d.begin(), d.end(), d2.begin()).first - d.begin(),
                 thrust::mismatch(h.begin(), h.end(), h2.begin()).first - h.begin());
    ASSERT_EQUAL(thrust::equal(d.begin(), d.end(), d2.begin()), thrust::equal(h.begin(), h.end(), h2.begin()));
    thrust::host_vector<T> hs = h;
    std::sort(hs.begin(), hs.end());
    thrust::device_vector<T> ds = hs;
    ASSERT_TRUE(thrust::is_sorted(ds.begin(), ds.end()));
    ASSERT_EQUAL(thrust::is_sorted(d.begin(), d.end()), thrust::is_sorted(h.begin(), h.end()));
    ASSERT_EQUAL(thrust::is_sorted_until(d.begin(), d.end()) - d.begin(), thrust::is_sorted_until(h.begin(), h.end()) - h.begin());
  }
}
DECLARE_TYPED_UNITTEST(TestFindMismatchLadder, int32_t);
DECLARE_TYPED_UNITTEST(TestFindMismatchLadder, int16_t);

// ------------------------------------------------------------------ inner_product / extrema
void TestInnerProductSimple() {  // testing/inner_product.cu:10-24
  thrust::device_vector<int> v1 = hv<int>({1, -2, 3}), v2 = hv<int>({-4, 5, 6});
  ASSERT_EQUAL(thrust::inner_product(v1.begin(), v1.end(), v2.begin(), 3), 7);
  ASSERT_EQUAL(thrust::inner_product(v1.begin(), v1.end(), v2.begin(), 1, thrust::multiplies<int>(), thrust::plus<int>()), 1 * -3 * 3 * 9);
}
DECLARE_UNITTEST(TestInnerProductSimple);

template <class T>
void TestInnerProductExtremaLadder() {
  {  // testing/min_element.cu, max_element.cu, minmax_element.cu: the first of equal extrema
    thrust::device_vector<T> data = hv<T>({3, 5, 1, 2, 5, 1});
    ASSERT_EQUAL(thrust::min_element(data.begin(), data.end()) - data.begin(), 2);
    ASSERT_EQUAL(thrust::max_element(data.begin(), data.end()) - data.begin(), 1);
    ASSERT_EQUAL(thrust::min_element(data.begin(), data.end(), thrust::greater<T>()) - data.begin(), 1);
    ASSERT_EQUAL(thrust::max_element(data.begin(), data.end(), thrust::greater<T>()) - data.begin(), 2);
    auto mm = thrust::minmax_element(data.begin(), data.end());
    ASSERT_EQUAL(mm.first - data.begin(), 2);
    ASSERT_EQUAL(mm.second - data.begin(), 1);
    ASSERT_TRUE(thrust::min_element(data.begin(), data.begin()) == data.begin());
  }
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h1 = small_values<T>(n, 21, 50), h2 = small_values<T>(n, 22, 50);
    thrust::device_vector<T> d1 = h1, d2 = h2;
    ASSERT_EQUAL(thrust::inner_product(d1.begin(), d1.end(), d2.begin(), T(13)), thrust::inner_product(h1.begin(), h1.end(), h2.begin(), T(13)));
    if (n == 0) continue;
    ASSERT_EQUAL(thrust::min_element(d1.begin(), d1.end()) - d1.begin(), std::min_element(h1.begin(), h1.end()) - h1.begin());
    ASSERT_EQUAL(thrust::max_element(d1.begin(), d1.end()) - d1.begin(), std::max_element(h1.begin(), h1.end()) - h1.begin());
    auto dm = thrust::minmax_element(d1.begin(), d1.end());
    auto hm = thrust::minmax_element(h1.begin(), h1.end());
    ASSERT_EQUAL(dm.first - d1.begin(), hm.first - h1.begin());
    ASSERT_EQUAL(dm.second - d1.begin(), hm.second - h1.begin());
  }
}
DECLARE_TYPED_UNITTEST(TestInnerProductExtremaLadder, int32_t);
DECLARE_TYPED_UNITTEST(TestInnerProductExtremaLadder, int64_t);
DECLARE_TYPED_UNITTEST(TestInnerProductExtremaLadder, double);

// ------------------------------------------------------------------ transform_scan / tabulate / generate
void TestTransformScanSimple() {  // testing/transform_scan.cu:60-120
  thrust::device_vector<int> input = hv<int>({1, 3, -2, 4, -5}), output(5);
  thrust::transform_inclusive_scan(input.begin(), input.end(), output.begin(), thrust::negate<int>(), thrust::plus<int>());
  ASSERT_EQUAL(output, hv<int>({-1, -4, -2, -6, -1}));
  thrust::transform_exclusive_scan(input.begin(), input.end(), output.begin(), thrust::negate<int>(), 0, thrust::plus<int>());
  ASSERT_EQUAL(output, hv<int>({0, -1, -4, -2, -6}));
  thrust::transform_exclusive_scan(input.begin(), input.end(), output.begin(), thrust::negate<int>(), 3, thrust::plus<int>());
  ASSERT_EQUAL(output, hv<int>({3, 2, -1, 1, -3}));
  thrust::transform_inclusive_scan(input.begin(), input.end(), input.begin(), thrust::negate<int>(), thrust::plus<int>());  // in place
  ASSERT_EQUAL(input, hv<int>({-1, -4, -2, -6, -1}));
}
DECLARE_UNITTEST(TestTransformScanSimple);

struct constant_seven {
  __host__ __device__ int operator()() const { return 7; }
};
void TestTabulateGenerateSequenceOfRandoms() {
  using namespace thrust::placeholders;
  thrust::device_vector<int> v(5);
  thrust::tabulate(v.begin(), v.end(), thrust::identity<int>());
  ASSERT_EQUAL(v, hv<int>({0, 1, 2, 3, 4}));  // testing/tabulate.cu:48-75
  thrust::tabulate(v.begin(), v.end(), -_1);
  ASSERT_EQUAL(v, hv<int>({0, -1, -2, -3, -4}));
  thrust::tabulate(v.begin(), v.end(), _1 * _1 * _1);
  ASSERT_EQUAL(v, hv<int>({0, 1, 8, 27, 64}));
  thrust::generate(v.begin(), v.end(), constant_seven());
  ASSERT_EQUAL(v, hv<int>({7, 7, 7, 7, 7}));
  thrust::generate_n(v.begin(), 3, constant_seven());
  thrust::device_vector<int> a = hv<int>({1, 2, 3, 4}), b = hv<int>({10, 20, 30, 40}), c(4);
  thrust::transform(a.begin(), a.end(), b.begin(), c.begin(), 2 * _1 + _2);
  ASSERT_EQUAL(c, hv<int>({12, 24, 36, 48}));
  thrust::transform(a.begin(), a.end(), c.begin(), _1 % 2 == 0);
  ASSERT_EQUAL(c, hv<int>({0, 1, 0, 1}));
}
DECLARE_UNITTEST(TestTabulateGenerateSequenceOfRandoms);

// ------------------------------------------------------------------ random
// the engines are the standard's minstd generators: the streams must agree number for number
void TestRandomEnginesMatchTheStandardOnes() {
  thrust::minstd_rand a;
  std::minstd_rand b;
  for (int i = 0; i < 1000; i++) ASSERT_EQUAL((unsigned)a(), (unsigned)b());
  thrust::minstd_rand0 a0(12345);
  std::minstd_rand0 b0(12345);
  for (int i = 0; i < 1000; i++) ASSERT_EQUAL((unsigned)a0(), (unsigned)b0());
  // the 10000th value of a default-constructed engine (C++ standard, [rand.predef])
  thrust::minstd_rand c;
  c.discard(9999);
  ASSERT_EQUAL((unsigned)c(), 399268537u);
  thrust::minstd_rand0 c0;
  c0.discard(9999);
  ASSERT_EQUAL((unsigned)c0(), 1043618065u);
  // discard(z) equals z calls, also for large z (modular exponentiation)
  thrust::minstd_rand d1(77), d2(77);
  for (int i = 0; i < 54321; i++) d1();
  d2.discard(54321);
  ASSERT_TRUE(d1 == d2);
  ASSERT_EQUAL((unsigned)thrust::minstd_rand(0)(), (unsigned)thrust::minstd_rand(1)());  // a seed of 0 becomes 1
  thrust::default_random_engine rng;
  thrust::uniform_int_distribution<int> dist(10, 99);
  thrust::uniform_real_distribution<float> u01;
  thrust::normal_distribution<double> normal(5.0, 2.0);
  double mean = 0;
  for (int i = 0; i < 20000; i++) {
    const int x = dist(rng);
    ASSERT_TRUE(x >= 10 && x <= 99);
    const float u = u01(rng);
    ASSERT_TRUE(u >= 0.0f && u < 1.0f);
    mean += normal(rng);
  }
  mean /= 20000;
  ASSERT_TRUE(mean > 4.9 && mean < 5.1);
}
DECLARE_UNITTEST(TestRandomEnginesMatchTheStandardOnes);

// the same engine on the device: one value per element, each from its own position in the stream
struct draw {
  __host__ __device__ unsigned operator()(unsigned i) const {
    thrust::default_random_engine rng;
    rng.discard(i);
    thrust::uniform_int_distribution<unsigned> dist(0, 9999);
    return dist(rng);
  }
};
void TestRandomOnDeviceMatchesHost() {
  const unsigned n = 100000;
  thrust::device_vector<unsigned> d(n);
  thrust::tabulate(d.begin(), d.end(), draw());
  thrust::host_vector<unsigned> h(n);
  thrust::default_random_engine rng;
  thrust::uniform_int_distribution<unsigned> dist(0, 9999);
  for (unsigned i = 0; i < n; i++) h[i] = dist(rng);
  ASSERT_EQUAL(d, h);
}
DECLARE_UNITTEST(TestRandomOnDeviceMatchesHost);

// the other engines: the 10000th values the reference documents (thrust/random.h:63-84,
// thrust/random/subtract_with_carry_engine.h:226-239), and the standard's engines where the
// definitions coincide
void TestRandomOtherEnginesKnownAnswers() {
  thrust::ranlux24_base a;
  a.discard(9999);
  ASSERT_EQUAL((unsigned long long)a(), 7937952ull);
  thrust::ranlux48_base b;
  b.discard(9999);
  ASSERT_EQUAL((unsigned long long)b(), 192113843633948ull);
  thrust::ranlux24 c;
  c.discard(9999);
  ASSERT_EQUAL((unsigned long long)c(), 9901578ull);
  thrust::ranlux48 d;
  d.discard(9999);
  ASSERT_EQUAL((unsigned long long)d(), 88229545517833ull);
  thrust::taus88 e;
  e.discard(9999);
  ASSERT_EQUAL((unsigned long long)e(), 3535848941ull);
  ASSERT_EQUAL((unsigned long long)thrust::taus88::max, 4294967295ull);
  thrust::ranlux24 x(77), y(77);
  std::ranlux24 sx(77);
  for (int i = 0; i < 1000; i++) {
    const unsigned v = (unsigned)x();
    ASSERT_EQUAL(v, (unsigned)sx());  // 24-bit words: the same engine as the standard's
    ASSERT_EQUAL(v, (unsigned)y());
  }
  ASSERT_TRUE(x == y);
  y();
  ASSERT_TRUE(x != y);
}
DECLARE_UNITTEST(TestRandomOtherEnginesKnownAnswers);

// shuffle: a permutation, the same on host and device for the same generator state
// (testing/shuffle.cu:326-375), and the network is a bijection (:378-405)
void TestShuffle() {
  for (std::size_t n : {std::size_t(0), std::size_t(1), std::size_t(2), std::size_t(10), std::size_t(16), std::size_t(17), std::size_t(1000),
                        std::size_t(4096), std::size_t(4097), std::size_t(123457), std::size_t(1 << 20)}) {
    thrust::host_vector<int> h(n), hs(n);
    for (std::size_t i = 0; i < n; i++) h[i] = (int)i;
    thrust::device_vector<int> d = h, ds(n);
    thrust::default_random_engine gh(13), gd(13);
    thrust::shuffle_copy(h.begin(), h.end(), hs.begin(), gh);
    thrust::shuffle_copy(d.begin(), d.end(), ds.begin(), gd);
    ASSERT_EQUAL(ds, hs);
    ASSERT_TRUE(gh == gd);  // both drew the same 24 keys
    thrust::host_vector<int> sorted = hs;
    std::sort(sorted.begin(), sorted.end());
    ASSERT_EQUAL(sorted, h);  // a permutation
    if (n > 100) ASSERT_TRUE(!(hs == h));
    thrust::shuffle(d.begin(), d.end(), gd);  // in place, with the generator's next state
    thrust::shuffle(h.begin(), h.end(), gh);
    ASSERT_EQUAL(d, h);
    thrust::sort(d.begin(), d.end());
    ASSERT_EQUAL(d, sorted);
  }
  thrust::default_random_engine g(3);
  thrust::detail::feistel_bijection f(1000, g);
  ASSERT_EQUAL(f.nearest_power_of_two(), std::uint64_t(1024));
  std::vector<std::uint64_t> image(1024);
  for (std::uint64_t i = 0; i < 1024; i++) image[i] = f(i);
  std::sort(image.begin(), image.end());
  for (std::uint64_t i = 0; i < 1024; i++) ASSERT_EQUAL(image[i], i);
  ASSERT_EQUAL(thrust::detail::feistel_bijection(17, g).nearest_power_of_two(), std::uint64_t(32));  // testing/shuffle.cu:409-424
  ASSERT_EQUAL(thrust::detail::feistel_bijection(32, g).nearest_power_of_two(), std::uint64_t(32));
  ASSERT_EQUAL(thrust::detail::feistel_bijection(1, g).nearest_power_of_two(), std::uint64_t(16));
}
DECLARE_UNITTEST(TestShuffle);

// thrust::optional in device code and in device storage (trivially copyable for trivial T)
struct checked_root {
  __host__ __device__ thrust::optional<float> operator()(float x) const {
    if (x < 0) return thrust::nullopt;
    return thrust::optional<float>(x * 0.5f);
  }
};
struct value_or_minus_one {
  __host__ __device__ float operator()(const thrust::optional<float>& o) const {
    return o.map([](float v) { return v + 1.0f; }).value_or(-1.0f);
  }
};
void TestOptionalOnDevice() {
  static_assert(std::is_trivially_copyable<thrust::optional<float>>::value, "optional of a trivial type can live in device storage");
  const std::size_t n = 10000;
  thrust::host_vector<float> h(n);
  for (std::size_t i = 0; i < n; i++) h[i] = (float)((int)(i % 7) - 3);
  thrust::device_vector<float> d = h, out(n);
  thrust::device_vector<thrust::optional<float>> o(n);
  thrust::transform(d.begin(), d.end(), o.begin(), checked_root());
  thrust::transform(o.begin(), o.end(), out.begin(), value_or_minus_one());
  thrust::host_vector<thrust::optional<float>> ho = o;
  thrust::host_vector<float> hout = out;
  for (std::size_t i = 0; i < n; i++) {
    ASSERT_EQUAL(ho[i].has_value(), h[i] >= 0);
    if (h[i] >= 0) ASSERT_EQUAL(*ho[i], h[i] * 0.5f);
    ASSERT_EQUAL(hout[i], h[i] >= 0 ? h[i] * 0.5f + 1.0f : -1.0f);
  }
  thrust::optional<int> a(3), b;
  ASSERT_TRUE(b < a && a == 3 && b == thrust::nullopt && a.value_or(0) == 3 && b.value_or(9) == 9);
  ASSERT_THROWS(b.value(), thrust::bad_optional_access);
}
DECLARE_UNITTEST(TestOptionalOnDevice);

// ---- transform_if, partition_point, is_partitioned, equal_range, unique_count, and the function
//      objects they are tested with — after testing/transform.cu:169-194, :339-369,
//      partition_point.cu:14-48, is_partitioned.cu:14-60, binary_search.cu:217-249, unique.cu:143-147
template <class Vector>
void TestTransformIfSimple() {
  typedef typename Vector::value_type T;
  Vector input(3), input2(3), stencil(3), output(3), result(3);
  input[0] = 1; input[1] = -2; input[2] = 3;
  output[0] = 1; output[1] = 2; output[2] = 3;
  stencil[0] = 1; stencil[1] = 0; stencil[2] = 1;
  result[0] = -1; result[1] = 2; result[2] = -3;
  typename Vector::iterator iter = thrust::transform_if(input.begin(), input.end(), stencil.begin(), output.begin(), thrust::negate<T>(), thrust::identity<T>());
  ASSERT_EQUAL((std::size_t)(iter - output.begin()), input.size());
  ASSERT_EQUAL(output, result);
  // the predicate on the element itself
  output[0] = 7; output[1] = 8; output[2] = 9;
  iter = thrust::transform_if(input.begin(), input.end(), output.begin(), thrust::negate<T>(), thrust::not1(thrust::identity<T>()));
  result[0] = 7; result[1] = 8; result[2] = 9;  // no element is zero: nothing is written
  ASSERT_EQUAL(output, result);
  // binary, through a negated stencil
  input2[0] = -4; input2[1] = 5; input2[2] = 6;
  stencil[0] = 0; stencil[1] = 1; stencil[2] = 0;
  output[0] = 1; output[1] = 2; output[2] = 3;
  result[0] = 5; result[1] = 2; result[2] = -3;
  iter = thrust::transform_if(input.begin(), input.end(), input2.begin(), stencil.begin(), output.begin(), thrust::minus<T>(), thrust::not1(thrust::identity<T>()));
  ASSERT_EQUAL((std::size_t)(iter - output.begin()), input.size());
  ASSERT_EQUAL(output, result);
}
void TestTransformIfSimpleHost() { TestTransformIfSimple<thrust::host_vector<int>>(); }
void TestTransformIfSimpleDevice() { TestTransformIfSimple<thrust::device_vector<int>>(); }
DECLARE_UNITTEST(TestTransformIfSimpleHost);
DECLARE_UNITTEST(TestTransformIfSimpleDevice);

struct is_even_int { __host__ __device__ bool operator()(int x) const { return (x & 1) == 0; } };
void TestTransformIfLarge() {
  const int n = (1 << 18) + 5;
  thrust::host_vector<int> h(n), expect(n);
  for (int i = 0; i < n; i++) { h[i] = (i * 2654435761u) >> 20; expect[i] = (h[i] & 1) ? -7 : h[i] * 3; }
  thrust::device_vector<int> d = h, out(n, -7);
  thrust::transform_if(thrust::device, d.begin(), d.end(), out.begin(), [] __host__ __device__(int x) { return x * 3; }, is_even_int());
  ASSERT_EQUAL(thrust::host_vector<int>(out), expect);
}
DECLARE_UNITTEST(TestTransformIfLarge);

template <class Vector>
void TestPartitionPointAndIsPartitioned() {
  typedef typename Vector::value_type T;
  Vector v(4);
  v[0] = 1; v[1] = 1; v[2] = 1; v[3] = 0;
  ASSERT_TRUE(thrust::partition_point(v.begin(), v.end(), thrust::identity<T>()) == v.begin() + 3);
  ASSERT_TRUE(thrust::partition_point(v.begin(), v.begin() + 3, thrust::identity<T>()) == v.begin() + 3);
  ASSERT_EQUAL(true, thrust::is_partitioned(v.begin(), v.begin(), thrust::identity<T>()));      // empty
  ASSERT_EQUAL(true, thrust::is_partitioned(v.begin(), v.begin() + 1, thrust::identity<T>()));  // one true element
  ASSERT_EQUAL(true, thrust::is_partitioned(v.begin(), v.begin() + 2, thrust::identity<T>()));
  ASSERT_EQUAL(true, thrust::is_partitioned(v.begin(), v.end(), thrust::identity<T>()));
  ASSERT_EQUAL(true, thrust::is_partitioned(v.begin() + 3, v.end(), thrust::identity<T>()));    // one false element
  v[0] = 1; v[1] = 0; v[2] = 1; v[3] = 1;
  ASSERT_EQUAL(false, thrust::is_partitioned(v.begin(), v.end(), thrust::identity<T>()));
  const int n = (1 << 16) + 13;
  thrust::host_vector<int> h(n);
  for (int i = 0; i < n; i++) h[i] = (i * 2654435761u) >> 12;
  Vector big(h.begin(), h.end());
  ASSERT_EQUAL(false, thrust::is_partitioned(big.begin(), big.end(), is_even_int()));
  typename Vector::iterator ref = thrust::stable_partition(big.begin(), big.end(), is_even_int());
  ASSERT_EQUAL((long)(ref - big.begin()), (long)(thrust::partition_point(big.begin(), big.end(), is_even_int()) - big.begin()));
  ASSERT_EQUAL(true, thrust::is_partitioned(big.begin(), big.end(), is_even_int()));
}
void TestPartitionPointHost() { TestPartitionPointAndIsPartitioned<thrust::host_vector<int>>(); }
void TestPartitionPointDevice() { TestPartitionPointAndIsPartitioned<thrust::device_vector<int>>(); }
DECLARE_UNITTEST(TestPartitionPointHost);
DECLARE_UNITTEST(TestPartitionPointDevice);

template <class Vector>
void TestScalarEqualRangeSimple() {
  Vector vec(5);
  vec[0] = 0; vec[1] = 2; vec[2] = 5; vec[3] = 7; vec[4] = 8;
  const int first[10] = {0, 1, 1, 2, 2, 2, 3, 3, 4, 5}, second[10] = {1, 1, 2, 2, 2, 3, 3, 4, 5, 5};
  for (int x = 0; x < 10; x++) {
    ASSERT_EQUAL((int)(thrust::equal_range(vec.begin(), vec.end(), x).first - vec.begin()), first[x]);
    ASSERT_EQUAL((int)(thrust::equal_range(vec.begin(), vec.end(), x).second - vec.begin()), second[x]);
  }
  // descending order under greater
  Vector desc(6);
  desc[0] = 9; desc[1] = 7; desc[2] = 7; desc[3] = 7; desc[4] = 3; desc[5] = 1;
  auto r = thrust::equal_range(desc.begin(), desc.end(), 7, thrust::greater<int>());
  ASSERT_EQUAL((int)(r.first - desc.begin()), 1);
  ASSERT_EQUAL((int)(r.second - desc.begin()), 4);
}
void TestScalarEqualRangeHost() { TestScalarEqualRangeSimple<thrust::host_vector<int>>(); }
void TestScalarEqualRangeDevice() { TestScalarEqualRangeSimple<thrust::device_vector<int>>(); }
DECLARE_UNITTEST(TestScalarEqualRangeHost);
DECLARE_UNITTEST(TestScalarEqualRangeDevice);

struct is_equal_div_10 { __host__ __device__ bool operator()(int x, int y) const { return x / 10 == y / 10; } };
template <class Vector>
void TestUniqueCount() {
  Vector data(10);
  const int raw[10] = {11, 11, 12, 20, 29, 21, 21, 31, 31, 37};
  for (int i = 0; i < 10; i++) data[i] = raw[i];
  ASSERT_EQUAL((int)thrust::unique_count(data.begin(), data.end()), 7);
  ASSERT_EQUAL((int)thrust::unique_count(data.begin(), data.end(), is_equal_div_10()), 3);
  ASSERT_EQUAL((int)thrust::unique_count(data.begin(), data.begin()), 0);
  ASSERT_EQUAL((int)thrust::unique_count(data.begin(), data.begin() + 1), 1);
  const int n = (1 << 17) + 3;
  thrust::host_vector<int> h(n);
  for (int i = 0; i < n; i++) h[i] = ((i * 2654435761u) >> 28) / 3;
  Vector big(h.begin(), h.end());
  const long expect = (long)(std::unique(h.begin(), h.end()) - h.begin());
  ASSERT_EQUAL((long)thrust::unique_count(big.begin(), big.end()), expect);
  ASSERT_EQUAL((long)(thrust::unique(big.begin(), big.end()) - big.begin()), expect);
}
void TestUniqueCountHost() { TestUniqueCount<thrust::host_vector<int>>(); }
void TestUniqueCountDevice() { TestUniqueCount<thrust::device_vector<int>>(); }
DECLARE_UNITTEST(TestUniqueCountHost);
DECLARE_UNITTEST(TestUniqueCountDevice);

void TestFunctionObjects() {
  // adaptable typedefs, transparent forms, negators, projections (thrust/functional.h:129-1529)
  static_assert(std::is_same<thrust::plus<int>::result_type, int>::value && std::is_same<thrust::less<float>::result_type, bool>::value, "");
  static_assert(std::is_same<thrust::negate<int>::argument_type, int>::value && std::is_same<thrust::minus<long>::first_argument_type, long>::value, "");
  ASSERT_EQUAL(thrust::square<int>()(7), 49);
  ASSERT_EQUAL(thrust::square<>()(1.5), 2.25);
  ASSERT_EQUAL(thrust::minus<>()(7, 2.5), 4.5);
  ASSERT_EQUAL(thrust::bit_xor<>()(6, 3), 5);
  ASSERT_EQUAL(thrust::logical_not<>()(0), true);
  ASSERT_EQUAL((thrust::project1st<int, double>()(3, 4.5)), 3);
  ASSERT_EQUAL((thrust::project2nd<int, double>()(3, 4.5)), 4.5);
  ASSERT_EQUAL(thrust::project1st<>()(3, 4.5), 3);
  ASSERT_EQUAL(thrust::not1(thrust::identity<int>())(0), true);
  ASSERT_EQUAL(thrust::not2(thrust::less<int>())(1, 2), false);
  ASSERT_EQUAL(thrust::not_fn(is_even_int())(3), true);
  thrust::device_vector<int> v(100), sq(100);
  thrust::sequence(v.begin(), v.end());
  thrust::transform(v.begin(), v.end(), sq.begin(), thrust::square<int>());
  ASSERT_EQUAL((int)sq[9], 81);
  ASSERT_EQUAL((int)thrust::count_if(v.begin(), v.end(), thrust::not_fn(is_even_int())), 50);
  thrust::transform(v.begin(), v.end(), sq.begin(), sq.begin(), thrust::project1st<int, int>());
  ASSERT_EQUAL((int)sq[9], 9);
}
DECLARE_UNITTEST(TestFunctionObjects);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

// Fancy iterators as inputs and outputs of the device algorithms, adjacent_difference and the
// vectorised binary searches, in the shape of the reference's testing/counting_iterator.cu,
// constant_iterator.cu, transform_iterator.cu, zip_iterator.cu, permutation_iterator.cu,
// discard_iterator.cu, adjacent_difference.cu and binary_search_vector.cu, and the dense
// histogram of examples/histogram.cu (sort, upper_bound of a counting range, adjacent_difference).
// Compiled by hipcc.
#include <algorithm>
#include <cmath>
#include <numeric>

#include <thrust/adjacent_difference.h>
#include <thrust/binary_search.h>
#include <thrust/copy.h>
#include <thrust/for_each.h>
#include <thrust/functional.h>
#include <thrust/iterator/constant_iterator.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/discard_iterator.h>
#include <thrust/iterator/iterator_adaptor.h>
#include <thrust/iterator/iterator_facade.h>
#include <thrust/iterator/retag.h>
#include <thrust/iterator/permutation_iterator.h>
#include <thrust/iterator/reverse_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/sequence.h>
#include <thrust/sort.h>
#include <thrust/transform.h>
#include <thrust/transform_reduce.h>
#include <thrust/tuple.h>
#include <thrust/unique.h>

#include "testing.h"

template <class T>
thrust::host_vector<T> vec(std::initializer_list<int> l) {
  thrust::host_vector<T> h(l.size());
  std::size_t i = 0;
  for (int x : l) h[i++] = (T)x;
  return h;
}
struct square {
  __host__ __device__ long long operator()(long long x) const { return x * x; }
};
struct is_odd {
  __host__ __device__ bool operator()(int x) const { return x & 1; }
};
struct dot3 {
  __host__ __device__ float operator()(const thrust::tuple<float, float, float>& a) const {
    return thrust::get<0>(a) * thrust::get<0>(a) + thrust::get<1>(a) * thrust::get<1>(a) + thrust::get<2>(a) * thrust::get<2>(a);
  }
};
struct rotate_pair {
  template <class Tuple>
  __host__ __device__ void operator()(Tuple t) const {  // a tuple of references
    const int a = thrust::get<0>(t);
    thrust::get<0>(t) = thrust::get<1>(t);
    thrust::get<1>(t) = a;
  }
};
struct sum_pair {
  __host__ __device__ thrust::tuple<int, int> operator()(const thrust::tuple<int, int>& a, const thrust::tuple<int, int>& b) const {
    return thrust::make_tuple(thrust::get<0>(a) + thrust::get<0>(b), thrust::get<1>(a) + thrust::get<1>(b));
  }
};

// testing/adjacent_difference.cu:9-40
template <class T>
void TestAdjacentDifferenceSimple() {
  thrust::device_vector<T> input = vec<T>({1, 4, 6}), output(3);
  auto result = thrust::adjacent_difference(input.begin(), input.end(), output.begin());
  ASSERT_EQUAL(result - output.begin(), (std::ptrdiff_t)3);
  ASSERT_EQUAL(output, vec<T>({1, 3, 2}));
  result = thrust::adjacent_difference(input.begin(), input.end(), output.begin(), thrust::plus<T>());
  ASSERT_EQUAL(output, vec<T>({1, 5, 10}));
  result = thrust::adjacent_difference(input.begin(), input.end(), input.begin());  // in place
  ASSERT_EQUAL(result - input.begin(), (std::ptrdiff_t)3);
  ASSERT_EQUAL(input, vec<T>({1, 3, 2}));
}
DECLARE_TYPED_UNITTEST(TestAdjacentDifferenceSimple, int);
DECLARE_TYPED_UNITTEST(TestAdjacentDifferenceSimple, float);
DECLARE_TYPED_UNITTEST(TestAdjacentDifferenceSimple, int8_t);

// testing/adjacent_difference.cu:45-78
template <class T>
void TestAdjacentDifference() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n), ho(n);
    thrust::device_vector<T> d = h, dout(n);
    auto he = thrust::adjacent_difference(h.begin(), h.end(), ho.begin());
    auto de = thrust::adjacent_difference(d.begin(), d.end(), dout.begin());
    ASSERT_EQUAL(he - ho.begin(), de - dout.begin());
    ASSERT_EQUAL(ho, dout);
    thrust::adjacent_difference(h.begin(), h.end(), ho.begin(), thrust::plus<T>());
    thrust::adjacent_difference(d.begin(), d.end(), dout.begin(), thrust::plus<T>());
    ASSERT_EQUAL(ho, dout);
    thrust::adjacent_difference(h.begin(), h.end(), h.begin(), thrust::plus<T>());
    thrust::adjacent_difference(d.begin(), d.end(), d.begin(), thrust::plus<T>());  // in place
    ASSERT_EQUAL(h, d);
  }
}
DECLARE_TYPED_UNITTEST(TestAdjacentDifference, int);
DECLARE_TYPED_UNITTEST(TestAdjacentDifference, uint8_t);
DECLARE_TYPED_UNITTEST(TestAdjacentDifference, int64_t);

// testing/binary_search_vector.cu:26-76, :127-175, :226-276
template <class T>
void TestVectorSearchSimple() {
  thrust::device_vector<T> hay = vec<T>({0, 2, 5, 7, 8}), input(10);
  thrust::sequence(input.begin(), input.end());
  thrust::device_vector<std::ptrdiff_t> out(10);
  auto end = thrust::lower_bound(hay.begin(), hay.end(), input.begin(), input.end(), out.begin());
  ASSERT_EQUAL(end - out.begin(), (std::ptrdiff_t)10);
  ASSERT_EQUAL(out, vec<std::ptrdiff_t>({0, 1, 1, 2, 2, 2, 3, 3, 4, 5}));
  end = thrust::upper_bound(hay.begin(), hay.end(), input.begin(), input.end(), out.begin());
  ASSERT_EQUAL(end - out.begin(), (std::ptrdiff_t)10);
  ASSERT_EQUAL(out, vec<std::ptrdiff_t>({1, 1, 2, 2, 2, 3, 3, 4, 5, 5}));
  thrust::device_vector<int> found(10);
  auto fend = thrust::binary_search(hay.begin(), hay.end(), input.begin(), input.end(), found.begin());
  ASSERT_EQUAL(fend - found.begin(), (std::ptrdiff_t)10);
  ASSERT_EQUAL(found, vec<int>({1, 0, 1, 0, 0, 1, 0, 1, 1, 0}));
  // scalar forms (testing/binary_search.cu:21-120)
  ASSERT_EQUAL(thrust::lower_bound(hay.begin(), hay.end(), (T)3) - hay.begin(), (std::ptrdiff_t)2);
  ASSERT_EQUAL(thrust::upper_bound(hay.begin(), hay.end(), (T)5) - hay.begin(), (std::ptrdiff_t)3);
  ASSERT_EQUAL(thrust::lower_bound(hay.begin(), hay.end(), (T)9) - hay.begin(), (std::ptrdiff_t)5);
  ASSERT_TRUE(thrust::binary_search(hay.begin(), hay.end(), (T)7));
  ASSERT_TRUE(!thrust::binary_search(hay.begin(), hay.end(), (T)6));
}
DECLARE_TYPED_UNITTEST(TestVectorSearchSimple, int);
DECLARE_TYPED_UNITTEST(TestVectorSearchSimple, float);
DECLARE_TYPED_UNITTEST(TestVectorSearchSimple, int16_t);

// testing/binary_search_vector.cu:327-420: random sorted haystack, random needles, vs std
template <class T>
void TestVectorSearch() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n);
    for (std::size_t i = 0; i < n; i++) h[i] = (T)((long long)h[i] % 1000);
    std::sort(h.begin(), h.end());
    thrust::host_vector<T> q = unittest::random_integers<T>(2 * n + 3, 99);
    for (std::size_t i = 0; i < q.size(); i++) q[i] = (T)((long long)q[i] % 1100);
    thrust::device_vector<T> d = h, dq = q;
    thrust::host_vector<int> ho(q.size());
    thrust::device_vector<int> dout(q.size());
    thrust::lower_bound(h.begin(), h.end(), q.begin(), q.end(), ho.begin());
    thrust::lower_bound(d.begin(), d.end(), dq.begin(), dq.end(), dout.begin());
    ASSERT_EQUAL(ho, dout);
    thrust::upper_bound(h.begin(), h.end(), q.begin(), q.end(), ho.begin());
    thrust::upper_bound(thrust::device, d.begin(), d.end(), dq.begin(), dq.end(), dout.begin());
    ASSERT_EQUAL(ho, dout);
    thrust::binary_search(h.begin(), h.end(), q.begin(), q.end(), ho.begin());
    thrust::binary_search(d.begin(), d.end(), dq.begin(), dq.end(), dout.begin());
    ASSERT_EQUAL(ho, dout);
    // descending haystack with a comparator
    std::reverse(h.begin(), h.end());
    d = h;
    thrust::lower_bound(h.begin(), h.end(), q.begin(), q.end(), ho.begin(), thrust::greater<T>());
    thrust::lower_bound(d.begin(), d.end(), dq.begin(), dq.end(), dout.begin(), thrust::greater<T>());
    ASSERT_EQUAL(ho, dout);
  }
}
DECLARE_TYPED_UNITTEST(TestVectorSearch, int);
DECLARE_TYPED_UNITTEST(TestVectorSearch, int64_t);
DECLARE_TYPED_UNITTEST(TestVectorSearch, double);

// testing/counting_iterator.cu:96-140, constant_iterator.cu:60-120
void TestCountingAndConstantIterators() {
  thrust::counting_iterator<int> first(1);
  ASSERT_EQUAL(*first, 1);
  ASSERT_EQUAL(first[5], 6);
  ASSERT_EQUAL((first + 10) - first, (std::ptrdiff_t)10);
  thrust::device_vector<int> out(4);
  thrust::copy(first, first + 4, out.begin());
  ASSERT_EQUAL(out, vec<int>({1, 2, 3, 4}));
  thrust::host_vector<int> hout(4);
  thrust::copy(first + 10, first + 14, hout.begin());  // a device-side range copied to the host
  ASSERT_EQUAL(hout, vec<int>({11, 12, 13, 14}));
  const long long n = 1000003;
  thrust::counting_iterator<long long> c(0);
  ASSERT_EQUAL(thrust::reduce(c, c + n), n * (n - 1) / 2);
  ASSERT_EQUAL(thrust::transform_reduce(c, c + n, square(), 0ll, thrust::plus<long long>()), (n - 1) * n * (2 * n - 1) / 6);
  thrust::constant_iterator<int> k(7);
  ASSERT_EQUAL(k[123], 7);
  ASSERT_EQUAL(thrust::reduce(k, k + 1000), 7000);
  thrust::device_vector<int> d(1000, 1), sum(1000);
  thrust::transform(d.begin(), d.end(), k, sum.begin(), thrust::plus<int>());
  ASSERT_EQUAL(sum, thrust::host_vector<int>(1000, 8));
  // counting input to copy_if
  thrust::device_vector<int> odd(50);
  auto e = thrust::copy_if(thrust::device, first, first + 100, odd.begin(), is_odd());
  ASSERT_EQUAL(e - odd.begin(), (std::ptrdiff_t)50);
  thrust::host_vector<int> expect(50);
  for (int i = 0; i < 50; i++) expect[i] = 2 * i + 1;
  ASSERT_EQUAL(odd, expect);
}
DECLARE_UNITTEST(TestCountingAndConstantIterators);

// testing/transform_iterator.cu:20-60, :62-85
void TestTransformIterator() {
  const std::size_t n = 123457;
  thrust::host_vector<int> h = unittest::random_integers<int>(n);
  for (std::size_t i = 0; i < n; i++) h[i] %= 1000;
  thrust::device_vector<int> d = h;
  auto hneg = thrust::make_transform_iterator(h.begin(), thrust::negate<int>());
  auto dneg = thrust::make_transform_iterator(d.begin(), thrust::negate<int>());
  ASSERT_EQUAL(*dneg, -h[0]);  // host-side dereference of a device range
  ASSERT_EQUAL(thrust::reduce(hneg, hneg + n), thrust::reduce(dneg, dneg + n));
  thrust::device_vector<int> out(n);
  thrust::host_vector<int> hout(n);
  thrust::copy(dneg, dneg + n, out.begin());
  std::copy(hneg, hneg + n, hout.begin());
  ASSERT_EQUAL(hout, out);
  // a transform iterator over a counting iterator
  auto sq = thrust::make_transform_iterator(thrust::counting_iterator<long long>(0), square());
  ASSERT_EQUAL(thrust::reduce(sq, sq + 1000), 999ll * 1000 * 1999 / 6);
}
DECLARE_UNITTEST(TestTransformIterator);

// testing/zip_iterator.cu:20-90 (traversal), :300-345 (reduce), :347-400 (transform)
void TestZipIterator() {
  const std::size_t n = 100003;
  thrust::host_vector<float> hx = unittest::random_samples<float>(n), hy = unittest::random_samples<float>(n, 5), hz = unittest::random_samples<float>(n, 6);
  thrust::device_vector<float> x = hx, y = hy, z = hz, norm(n);
  auto first = thrust::make_zip_iterator(thrust::make_tuple(x.begin(), y.begin(), z.begin()));
  ASSERT_EQUAL((first + 5) - first, (std::ptrdiff_t)5);
  thrust::tuple<float, float, float> e0 = first[0];  // host-side read of three device elements
  ASSERT_EQUAL(thrust::get<1>(e0), hy[0]);
  thrust::transform(first, first + n, norm.begin(), dot3());
  thrust::host_vector<float> got = norm;
  for (std::size_t i = 0; i < n; i++) {
    const float want = hx[i] * hx[i] + hy[i] * hy[i] + hz[i] * hz[i];
    ASSERT_TRUE(std::fabs(got[i] - want) <= 1e-5f * (1.0f + want));
  }
  // writing through a zip iterator: swap the two members of every pair
  thrust::host_vector<int> ha = unittest::random_integers<int>(n), hb = unittest::random_integers<int>(n, 3);
  thrust::device_vector<int> a = ha, b = hb;
  auto pairs = thrust::make_zip_iterator(thrust::make_tuple(a.begin(), b.begin()));
  thrust::for_each(pairs, pairs + n, rotate_pair());
  ASSERT_EQUAL(a, hb);
  ASSERT_EQUAL(b, ha);
  // reducing tuples
  thrust::device_vector<int> ones(n, 1), twos(n, 2);
  auto ot = thrust::make_zip_iterator(thrust::make_tuple(ones.begin(), twos.begin()));
  thrust::tuple<int, int> s = thrust::reduce(ot, ot + n, thrust::make_tuple(0, 0), sum_pair());
  ASSERT_EQUAL(thrust::get<0>(s), (int)n);
  ASSERT_EQUAL(thrust::get<1>(s), (int)(2 * n));
  // a zip output: transform into two arrays at once
  thrust::device_vector<int> o1(n), o2(n);
  auto zout = thrust::make_zip_iterator(thrust::make_tuple(o1.begin(), o2.begin()));
  thrust::transform(ot, ot + n, ot, zout, sum_pair());
  ASSERT_EQUAL(o1, thrust::host_vector<int>(n, 2));
  ASSERT_EQUAL(o2, thrust::host_vector<int>(n, 4));
}
DECLARE_UNITTEST(TestZipIterator);

// testing/permutation_iterator.cu:20-110, reverse_iterator.cu:35-70, discard_iterator.cu
void TestPermutationReverseDiscard() {
  thrust::device_vector<int> source(8), indices = vec<int>({3, 0, 5, 7});
  thrust::sequence(source.begin(), source.end(), 1);
  auto p = thrust::make_permutation_iterator(source.begin(), indices.begin());
  ASSERT_EQUAL((int)p[2], 6);
  thrust::device_vector<int> gathered(4);
  thrust::copy(p, p + 4, gathered.begin());
  ASSERT_EQUAL(gathered, vec<int>({4, 1, 6, 8}));
  ASSERT_EQUAL(thrust::reduce(p, p + 4), 19);
  // scatter through a permutation output
  thrust::device_vector<int> target(8, 0), fours(4, 4);
  thrust::transform(fours.begin(), fours.end(), thrust::make_permutation_iterator(target.begin(), indices.begin()), thrust::negate<int>());
  ASSERT_EQUAL(target, vec<int>({-4, 0, 0, -4, 0, -4, 0, -4}));
  // reverse
  auto r = thrust::make_reverse_iterator(source.end());
  thrust::device_vector<int> reversed(8);
  thrust::copy(r, r + 8, reversed.begin());
  ASSERT_EQUAL(reversed, vec<int>({8, 7, 6, 5, 4, 3, 2, 1}));
  // discard: count runs without storing the values
  thrust::device_vector<int> keys = vec<int>({1, 1, 2, 2, 2, 3}), vals(6, 9), ukeys(6);
  auto ends = thrust::unique_by_key_copy(keys.begin(), keys.end(), vals.begin(), ukeys.begin(), thrust::make_discard_iterator());
  ASSERT_EQUAL(ends.first - ukeys.begin(), (std::ptrdiff_t)3);
  ukeys.resize(3);
  ASSERT_EQUAL(ukeys, vec<int>({1, 2, 3}));
}
DECLARE_UNITTEST(TestPermutationReverseDiscard);

// examples/histogram.cu:66-104 (dense histogram): sort, upper_bound of every bin index, differences
void TestDenseHistogramExample() {
  const std::size_t n = 400003;
  const int bins = 37;
  thrust::host_vector<int> h = unittest::random_integers<int>(n);
  for (std::size_t i = 0; i < n; i++) h[i] = (int)((unsigned)h[i] % bins);
  thrust::device_vector<int> data = h, histogram(bins);
  thrust::sort(data.begin(), data.end());
  thrust::counting_iterator<int> search_begin(0);
  thrust::upper_bound(data.begin(), data.end(), search_begin, search_begin + bins, histogram.begin());
  thrust::adjacent_difference(histogram.begin(), histogram.end(), histogram.begin());
  thrust::host_vector<int> expect(bins, 0);
  for (std::size_t i = 0; i < n; i++) expect[h[i]]++;
  ASSERT_EQUAL(histogram, expect);
}
DECLARE_UNITTEST(TestDenseHistogramExample);

// examples/histogram.cu:107-150 (sparse histogram): sort, then reduce_by_key of a constant 1
void TestSparseHistogramExample() {
  const std::size_t n = 300007;
  thrust::host_vector<int> h = unittest::random_integers<int>(n);
  for (std::size_t i = 0; i < n; i++) h[i] = (int)((unsigned)h[i] % 1000) * 3;  // only multiples of 3 occur
  thrust::device_vector<int> data = h, values(1000), counts(1000);
  thrust::sort(data.begin(), data.end());
  auto ends = thrust::reduce_by_key(data.begin(), data.end(), thrust::constant_iterator<int>(1), values.begin(), counts.begin());
  const std::size_t bins = ends.first - values.begin();
  std::vector<int> expect(3000, 0);
  for (std::size_t i = 0; i < n; i++) expect[h[i]]++;
  thrust::host_vector<int> ev, ec;
  for (int v = 0; v < 3000; v++)
    if (expect[v]) { ev.push_back(v); ec.push_back(expect[v]); }
  ASSERT_EQUAL(bins, ev.size());
  ASSERT_EQUAL((std::size_t)(ends.second - counts.begin()), ev.size());
  values.resize(bins); counts.resize(bins);
  ASSERT_EQUAL(values, ev);
  ASSERT_EQUAL(counts, ec);
  // the keys are not wanted: discard them
  thrust::device_vector<int> counts2(1000);
  auto ends2 = thrust::reduce_by_key(data.begin(), data.end(), thrust::constant_iterator<int>(1), thrust::make_discard_iterator(), counts2.begin());
  ASSERT_EQUAL((std::size_t)(ends2.second - counts2.begin()), bins);
  counts2.resize(bins);
  ASSERT_EQUAL(counts2, ec);
}
DECLARE_UNITTEST(TestSparseHistogramExample);

// fancy inputs and outputs of the scans (testing/scan.cu:480-520 uses transform and discard iterators)
void TestScanWithFancyIterators() {
  const std::size_t n = 200003;
  thrust::device_vector<long long> out(n);
  thrust::counting_iterator<long long> c(1);
  thrust::inclusive_scan(c, c + n, out.begin());
  thrust::host_vector<long long> got = out;
  for (std::size_t i = 0; i < n; i += 997) ASSERT_EQUAL(got[i], (long long)(i + 1) * (long long)(i + 2) / 2);
  auto sq = thrust::make_transform_iterator(c, square());
  thrust::exclusive_scan(sq, sq + n, out.begin(), 0ll);
  got = out;
  for (std::size_t i = 0; i < n; i += 997) ASSERT_EQUAL(got[i], (long long)i * (long long)(i + 1) * (long long)(2 * i + 1) / 6);
  // segment ranks: inclusive_scan_by_key of a constant 1
  thrust::host_vector<int> hk(n);
  for (std::size_t i = 0; i < n; i++) hk[i] = (int)(i / 7);
  thrust::device_vector<int> keys = hk, rank(n);
  thrust::inclusive_scan_by_key(keys.begin(), keys.end(), thrust::constant_iterator<int>(1), rank.begin());
  thrust::host_vector<int> hr = rank;
  for (std::size_t i = 0; i < n; i++) ASSERT_EQUAL(hr[i], (int)(i % 7) + 1);
  // scan into a permutation: the output lands reversed
  thrust::device_vector<int> ones(n, 1), rev(n);
  thrust::inclusive_scan(ones.begin(), ones.end(), thrust::make_reverse_iterator(rev.end()));
  thrust::host_vector<int> hrev = rev;
  for (std::size_t i = 0; i < n; i += 1013) ASSERT_EQUAL(hrev[i], (int)(n - i));
}
DECLARE_UNITTEST(TestScanWithFancyIterators);

// testing/zip_iterator_sort_by_key.cu, zip_iterator_sort.cu: zipped values follow their keys; a
// range of tuples sorts lexicographically
struct first_then_second {
  __host__ __device__ bool operator()(const thrust::tuple<int, int>& a, const thrust::tuple<int, int>& b) const {
    return thrust::get<0>(a) < thrust::get<0>(b) || (thrust::get<0>(a) == thrust::get<0>(b) && thrust::get<1>(a) < thrust::get<1>(b));
  }
};
void TestSortWithZipIterators() {
  for (std::size_t n : {std::size_t(0), std::size_t(1), std::size_t(1000), std::size_t(300007)}) {
    thrust::host_vector<int> hk = unittest::random_integers<int>(n);
    for (std::size_t i = 0; i < n; i++) hk[i] %= 97;  // many equal keys: stability shows
    thrust::host_vector<int> ha(n);
    thrust::host_vector<float> hb(n);
    for (std::size_t i = 0; i < n; i++) { ha[i] = (int)i; hb[i] = 0.5f * (float)i; }
    thrust::device_vector<int> k = hk, a = ha;
    thrust::device_vector<float> b = hb;
    thrust::stable_sort_by_key(k.begin(), k.end(), thrust::make_zip_iterator(thrust::make_tuple(a.begin(), b.begin())));
    std::vector<std::size_t> order(n);
    std::iota(order.begin(), order.end(), std::size_t(0));
    std::stable_sort(order.begin(), order.end(), [&](std::size_t x, std::size_t y) { return hk[x] < hk[y]; });
    thrust::host_vector<int> ek(n), ea(n);
    thrust::host_vector<float> eb(n);
    for (std::size_t i = 0; i < n; i++) { ek[i] = hk[order[i]]; ea[i] = ha[order[i]]; eb[i] = hb[order[i]]; }
    ASSERT_EQUAL(k, ek);
    ASSERT_EQUAL(a, ea);
    ASSERT_EQUAL(b, eb);
    // a range of (key, tiebreak) tuples, sorted lexicographically: with operator< and with a functor
    thrust::host_vector<int> h1 = unittest::random_integers<int>(n, 4);
    for (std::size_t i = 0; i < n; i++) h1[i] %= 1000;
    thrust::device_vector<int> p = hk, q = h1, p2 = hk, q2 = h1;
    auto zfirst = thrust::make_zip_iterator(thrust::make_tuple(p.begin(), q.begin()));
    thrust::sort(zfirst, zfirst + n);
    auto zfirst2 = thrust::make_zip_iterator(thrust::make_tuple(p2.begin(), q2.begin()));
    thrust::sort(thrust::device, zfirst2, zfirst2 + n, first_then_second());
    std::vector<std::pair<int, int>> pairs(n);
    for (std::size_t i = 0; i < n; i++) pairs[i] = std::make_pair((int)hk[i], (int)h1[i]);
    std::sort(pairs.begin(), pairs.end());
    thrust::host_vector<int> ep(n), eq(n);
    for (std::size_t i = 0; i < n; i++) { ep[i] = pairs[i].first; eq[i] = pairs[i].second; }
    ASSERT_EQUAL(p, ep);
    ASSERT_EQUAL(q, eq);
    ASSERT_EQUAL(p2, ep);
    ASSERT_EQUAL(q2, eq);
  }
}
DECLARE_UNITTEST(TestSortWithZipIterators);

// A user-defined iterator from iterator_adaptor (the example of thrust/iterator/iterator_adaptor.h:
// every element of the base range n times) and one from iterator_facade (squares of the index), used
// as inputs of device algorithms; retag declares a raw device pointer to be a device range.
template <class Iterator>
class repeat_iterator : public thrust::iterator_adaptor<repeat_iterator<Iterator>, Iterator> {
 public:
  typedef thrust::iterator_adaptor<repeat_iterator<Iterator>, Iterator> super_t;
  __host__ __device__ repeat_iterator(const Iterator& x, int n) : super_t(x), begin(x), n(n) {}
  friend class thrust::iterator_core_access;

 private:
  Iterator begin;
  int n;
  __host__ __device__ typename super_t::reference dereference() const { return *(begin + (this->base() - begin) / n); }
};
class squares_iterator
    : public thrust::iterator_facade<squares_iterator, long long, thrust::device_system_tag, thrust::random_access_traversal_tag, long long> {
 public:
  __host__ __device__ explicit squares_iterator(long long i = 0) : i_(i) {}
  friend class thrust::iterator_core_access;

 private:
  long long i_;
  __host__ __device__ long long dereference() const { return i_ * i_; }
  __host__ __device__ bool equal(const squares_iterator& o) const { return i_ == o.i_; }
  __host__ __device__ void increment() { ++i_; }
  __host__ __device__ void decrement() { --i_; }
  __host__ __device__ void advance(std::ptrdiff_t n) { i_ += n; }
  __host__ __device__ std::ptrdiff_t distance_to(const squares_iterator& o) const { return (std::ptrdiff_t)(o.i_ - i_); }
};
void TestUserIteratorsFromFacadeAndAdaptor() {
  thrust::host_vector<int> h = {1, 2, 3, 4};
  thrust::device_vector<int> d = h;
  typedef repeat_iterator<thrust::device_vector<int>::iterator> Rep;
  static_assert(thrust::system::cdna4::detail::is_device_iterator<Rep>::value, "an adaptor over a device iterator is a device iterator");
  static_assert(!thrust::system::cdna4::detail::is_device_iterator<repeat_iterator<thrust::host_vector<int>::iterator>>::value, "");
  Rep first(d.begin(), 3), last = first + 12;
  ASSERT_EQUAL(last - first, 12);
  ASSERT_EQUAL(thrust::reduce(first, last), 30);
  thrust::device_vector<int> out(12);
  thrust::copy(first, last, out.begin());
  ASSERT_EQUAL(out, (thrust::host_vector<int>{1, 1, 1, 2, 2, 2, 3, 3, 3, 4, 4, 4}));
  thrust::inclusive_scan(first, last, out.begin());
  ASSERT_EQUAL(out, (thrust::host_vector<int>{1, 2, 3, 5, 7, 9, 12, 15, 18, 22, 26, 30}));
  // the same adaptor over a host range runs on the host
  repeat_iterator<thrust::host_vector<int>::iterator> hf(h.begin(), 2);
  ASSERT_EQUAL(thrust::reduce(hf, hf + 8), 20);
  // a facade that computes its values: sum of i^2 below n
  const long long n = 100000;
  ASSERT_EQUAL(thrust::reduce(squares_iterator(0), squares_iterator(n), 0ll), (n - 1) * n * (2 * n - 1) / 6);
  ASSERT_EQUAL((long long)squares_iterator(3)[4], 49ll);
  ASSERT_TRUE(squares_iterator(3) < squares_iterator(5) && squares_iterator(5) - squares_iterator(3) == 2);
  // retag: a raw device pointer becomes a device range
  int* raw = thrust::raw_pointer_cast(d.data());
  auto tagged = thrust::retag<thrust::device_system_tag>(raw);
  ASSERT_EQUAL(thrust::reduce(tagged, tagged + 4), 10);
}
DECLARE_UNITTEST(TestUserIteratorsFromFacadeAndAdaptor);

// the accessors of the fancy iterators (base(), value(), functor(), get_iterator_tuple())
void TestIteratorAccessors() {
  thrust::counting_iterator<int> c(7);
  ASSERT_EQUAL((c + 3).base(), 10);
  thrust::constant_iterator<float> k(2.5f);
  ASSERT_EQUAL((k + 4).value(), 2.5f);
  ASSERT_EQUAL((int)*(k + 4).base(), 4);
  thrust::device_vector<int> data(4), idx(4);
  auto perm = thrust::make_permutation_iterator(data.begin(), idx.begin());
  ASSERT_TRUE((perm + 2).base() == idx.begin() + 2);
  auto d = thrust::make_discard_iterator(3);
  ASSERT_EQUAL((int)*(d + 2).base(), 5);
  auto r = thrust::make_reverse_iterator(data.end());
  ASSERT_TRUE((r + 1).base() == data.end() - 1);
  auto t = thrust::make_transform_iterator(data.begin(), thrust::negate<int>());
  ASSERT_TRUE((t + 1).base() == data.begin() + 1);
  auto z = thrust::make_zip_iterator(thrust::make_tuple(data.begin(), idx.begin()));
  ASSERT_TRUE(thrust::get<1>((z + 3).get_iterator_tuple()) == idx.begin() + 3);
}
DECLARE_UNITTEST(TestIteratorAccessors);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

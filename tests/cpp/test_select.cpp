// copy_if / remove_if / remove / unique / unique_by_key with user predicates, in the shape of the
// reference's testing/copy.cu (copy_if), remove.cu, unique.cu and unique_by_key.cu: their known
// answers plus device vs host over the size ladder.  User predicates instantiate kernel templates,
// so this translation unit is compiled by hipcc.
#include <algorithm>

#include <thrust/copy.h>
#include <thrust/remove.h>
#include <thrust/sequence.h>
#include <thrust/unique.h>

#include "testing.h"

template <class T>
struct is_even {
  __host__ __device__ bool operator()(T x) const { return ((int)x & 1) == 0; }
};
template <class T>
struct is_true {
  __host__ __device__ bool operator()(T x) const { return x ? true : false; }
};
template <class T>
struct is_equal_div_10_unique {
  __host__ __device__ bool operator()(const T x, const T& y) const { return ((int)x / 10) == ((int)y / 10); }
};
struct record {
  int id;
  float weight;
  bool operator==(const record& o) const { return id == o.id && weight == o.weight; }
};
std::ostream& operator<<(std::ostream& os, const record& r) { return os << "{" << r.id << "," << r.weight << "}"; }
struct heavy {
  __host__ __device__ bool operator()(const record& r) const { return r.weight > 0.5f; }
};
struct same_id {
  __host__ __device__ bool operator()(const record& a, const record& b) const { return a.id == b.id; }
};

template <class T>
thrust::host_vector<T> vec(std::initializer_list<int> l) {
  thrust::host_vector<T> h(l.size());
  std::size_t i = 0;
  for (int x : l) h[i++] = (T)x;
  return h;
}
// runs of random length up to max_run, values from a small alphabet
template <class T>
thrust::host_vector<T> random_runs(std::size_t n, int max_run, std::uint64_t seed = 99) {
  thrust::host_vector<T> h(n);
  std::uint64_t s = seed + n;
  std::size_t i = 0;
  while (i < n) {
    const T v = (T)(unittest::splitmix64(s) % 97);
    std::size_t len = 1 + unittest::splitmix64(s) % (std::uint64_t)max_run;
    for (; len && i < n; --len) h[i++] = v;
  }
  return h;
}

// testing/copy.cu:253-269
template <class T>
void TestCopyIfSimple() {
  thrust::device_vector<T> v = vec<T>({0, 1, 2, 3, 4}), dest(4);
  auto end = thrust::copy_if(v.begin(), v.end(), dest.begin(), is_true<T>());
  ASSERT_TRUE(end == dest.end());
  ASSERT_EQUAL(dest, vec<T>({1, 2, 3, 4}));
}
DECLARE_TYPED_UNITTEST(TestCopyIfSimple, int);
DECLARE_TYPED_UNITTEST(TestCopyIfSimple, float);
DECLARE_TYPED_UNITTEST(TestCopyIfSimple, int8_t);

// testing/copy.cu:379-397
template <class T>
void TestCopyIfStencilSimple() {
  thrust::device_vector<T> v = vec<T>({0, 1, 2, 3, 4}), s = vec<T>({1, 1, 0, 1, 0}), dest(3);
  auto end = thrust::copy_if(v.begin(), v.end(), s.begin(), dest.begin(), is_true<T>());
  ASSERT_TRUE(end == dest.end());
  ASSERT_EQUAL(dest, vec<T>({0, 1, 3}));
}
DECLARE_TYPED_UNITTEST(TestCopyIfStencilSimple, int);
DECLARE_TYPED_UNITTEST(TestCopyIfStencilSimple, double);

// testing/copy.cu:273-330: is_true and is_even over the size ladder, device vs host
template <class T>
void TestCopyIf() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n), hr(n);
    thrust::device_vector<T> d = h, dr(n);
    auto he = thrust::copy_if(h.begin(), h.end(), hr.begin(), is_true<T>());
    auto de = thrust::copy_if(d.begin(), d.end(), dr.begin(), is_true<T>());
    ASSERT_EQUAL(he - hr.begin(), de - dr.begin());
    hr.resize(he - hr.begin()); dr.resize(de - dr.begin());
    ASSERT_EQUAL(hr, dr);
    hr.resize(n); dr.resize(n);
    he = thrust::copy_if(h.begin(), h.end(), hr.begin(), is_even<T>());
    de = thrust::copy_if(thrust::device, d.begin(), d.end(), dr.begin(), is_even<T>());
    ASSERT_EQUAL(he - hr.begin(), de - dr.begin());
    hr.resize(he - hr.begin()); dr.resize(de - dr.begin());
    ASSERT_EQUAL(hr, dr);
  }
}
DECLARE_TYPED_UNITTEST(TestCopyIf, int);
DECLARE_TYPED_UNITTEST(TestCopyIf, uint8_t);
DECLARE_TYPED_UNITTEST(TestCopyIf, int64_t);
DECLARE_TYPED_UNITTEST(TestCopyIf, int16_t);

// testing/copy.cu:401-460: data = sequence, stencil random, a stencil type other than the data's
template <class T>
void TestCopyIfStencil() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h(n), hr(n);
    thrust::device_vector<T> d(n), dr(n);
    thrust::sequence(h.begin(), h.end());
    thrust::sequence(d.begin(), d.end());
    thrust::host_vector<uint16_t> hs = unittest::random_integers<uint16_t>(n);
    thrust::device_vector<uint16_t> ds = hs;
    auto he = thrust::copy_if(h.begin(), h.end(), hs.begin(), hr.begin(), is_even<uint16_t>());
    auto de = thrust::copy_if(d.begin(), d.end(), ds.begin(), dr.begin(), is_even<uint16_t>());
    ASSERT_EQUAL(he - hr.begin(), de - dr.begin());
    hr.resize(he - hr.begin()); dr.resize(de - dr.begin());
    ASSERT_EQUAL(hr, dr);
  }
}
DECLARE_TYPED_UNITTEST(TestCopyIfStencil, int);
DECLARE_TYPED_UNITTEST(TestCopyIfStencil, double);

// all kept / none kept: the tile offsets at both extremes
void TestCopyIfAllOrNothing() {
  const std::size_t n = 300001;
  thrust::device_vector<int> ones(n, 1), zeros(n, 0), out(n, -1);
  auto e = thrust::copy_if(ones.begin(), ones.end(), out.begin(), is_true<int>());
  ASSERT_EQUAL(e - out.begin(), (std::ptrdiff_t)n);
  ASSERT_EQUAL(out, ones);
  e = thrust::copy_if(zeros.begin(), zeros.end(), out.begin(), is_true<int>());
  ASSERT_EQUAL(e - out.begin(), (std::ptrdiff_t)0);
  ASSERT_EQUAL(out, ones);  // untouched
}
DECLARE_UNITTEST(TestCopyIfAllOrNothing);

// a struct element with a predicate on one member
void TestCopyIfStruct() {
  const std::size_t n = 123457;
  thrust::host_vector<record> h(n), hr(n);
  std::uint64_t s = 5;
  for (std::size_t i = 0; i < n; i++) h[i] = record{(int)i, (float)(unittest::splitmix64(s) % 1000) / 1000.0f};
  thrust::device_vector<record> d = h, dr(n);
  auto he = thrust::copy_if(h.begin(), h.end(), hr.begin(), heavy());
  auto de = thrust::copy_if(d.begin(), d.end(), dr.begin(), heavy());
  ASSERT_EQUAL(he - hr.begin(), de - dr.begin());
  hr.resize(he - hr.begin()); dr.resize(de - dr.begin());
  ASSERT_EQUAL(hr, dr);
}
DECLARE_UNITTEST(TestCopyIfStruct);

// testing/remove.cu:28-48, :184-204, :345-368 and remove_copy (:110-131)
template <class T>
void TestRemoveSimple() {
  thrust::device_vector<T> data = vec<T>({1, 2, 1, 3, 2});
  auto end = thrust::remove(data.begin(), data.end(), (T)2);
  ASSERT_EQUAL(end - data.begin(), (std::ptrdiff_t)3);
  data.resize(3);
  ASSERT_EQUAL(data, vec<T>({1, 1, 3}));

  data = vec<T>({1, 2, 1, 3, 2});
  data.erase(thrust::remove(data.begin(), data.end(), (T)2), data.end());  // the erase-remove idiom
  ASSERT_EQUAL(data, vec<T>({1, 1, 3}));

  data = vec<T>({1, 2, 1, 3, 2});
  end = thrust::remove_if(data.begin(), data.end(), is_even<T>());
  ASSERT_EQUAL(end - data.begin(), (std::ptrdiff_t)3);
  data.resize(3);
  ASSERT_EQUAL(data, vec<T>({1, 1, 3}));

  data = vec<T>({1, 2, 1, 3, 2});
  thrust::device_vector<T> result(5);
  end = thrust::remove_copy_if(data.begin(), data.end(), result.begin(), is_even<T>());
  ASSERT_EQUAL(end - result.begin(), (std::ptrdiff_t)3);
  result.resize(3);
  ASSERT_EQUAL(result, vec<T>({1, 1, 3}));

  result.resize(5);
  end = thrust::remove_copy(thrust::device, data.begin(), data.end(), result.begin(), (T)2);
  ASSERT_EQUAL(end - result.begin(), (std::ptrdiff_t)3);
  result.resize(3);
  ASSERT_EQUAL(result, vec<T>({1, 1, 3}));
}
DECLARE_TYPED_UNITTEST(TestRemoveSimple, int);
DECLARE_TYPED_UNITTEST(TestRemoveSimple, uint8_t);
DECLARE_TYPED_UNITTEST(TestRemoveSimple, int64_t);

// testing/remove.cu:465-560: remove / remove_if / remove_copy_if over the ladder, device vs host
template <class T>
void TestRemoveLadder() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h0 = unittest::random_samples<T>(n);
    for (std::size_t i = 0; i < n; i += 3) h0[i] = (T)0;
    {
      thrust::host_vector<T> h = h0;
      thrust::device_vector<T> d = h0;
      auto he = thrust::remove(h.begin(), h.end(), (T)0);
      auto de = thrust::remove(d.begin(), d.end(), (T)0);
      ASSERT_EQUAL(he - h.begin(), de - d.begin());
      h.resize(he - h.begin()); d.resize(de - d.begin());
      ASSERT_EQUAL(h, d);
    }
    {
      thrust::host_vector<T> h = h0;
      thrust::device_vector<T> d = h0;
      auto he = thrust::remove_if(h.begin(), h.end(), is_true<T>());
      auto de = thrust::remove_if(d.begin(), d.end(), is_true<T>());
      ASSERT_EQUAL(he - h.begin(), de - d.begin());
      h.resize(he - h.begin()); d.resize(de - d.begin());
      ASSERT_EQUAL(h, d);
    }
    {
      thrust::host_vector<T> h = h0, hr(n);
      thrust::device_vector<T> d = h0, dr(n);
      auto he = thrust::remove_copy_if(h.begin(), h.end(), hr.begin(), is_even<T>());
      auto de = thrust::remove_copy_if(d.begin(), d.end(), dr.begin(), is_even<T>());
      ASSERT_EQUAL(he - hr.begin(), de - dr.begin());
      hr.resize(he - hr.begin()); dr.resize(de - dr.begin());
      ASSERT_EQUAL(hr, dr);
      ASSERT_EQUAL(d, h0);  // the input is untouched
    }
  }
}
DECLARE_TYPED_UNITTEST(TestRemoveLadder, int);
DECLARE_TYPED_UNITTEST(TestRemoveLadder, float);
DECLARE_TYPED_UNITTEST(TestRemoveLadder, int8_t);

// testing/unique.cu:150-185 and unique_copy (:228-268)
template <class T>
void TestUniqueSimple() {
  thrust::device_vector<T> data = vec<T>({11, 11, 12, 20, 29, 21, 21, 31, 31, 37});
  auto new_last = thrust::unique(data.begin(), data.end());
  ASSERT_EQUAL(new_last - data.begin(), (std::ptrdiff_t)7);
  thrust::host_vector<T> got(data);
  got.resize(7);
  ASSERT_EQUAL(got, vec<T>({11, 12, 20, 29, 21, 31, 37}));
  new_last = thrust::unique(data.begin(), new_last, is_equal_div_10_unique<T>());
  ASSERT_EQUAL(new_last - data.begin(), (std::ptrdiff_t)3);
  got = data;
  got.resize(3);
  ASSERT_EQUAL(got, vec<T>({11, 20, 31}));

  data = vec<T>({11, 11, 12, 20, 29, 21, 21, 31, 31, 37});
  thrust::device_vector<T> output(10, (T)-1);
  auto out_last = thrust::unique_copy(data.begin(), data.end(), output.begin());
  ASSERT_EQUAL(out_last - output.begin(), (std::ptrdiff_t)7);
  got = output;
  got.resize(7);
  ASSERT_EQUAL(got, vec<T>({11, 12, 20, 29, 21, 31, 37}));
  out_last = thrust::unique_copy(thrust::device, output.begin(), out_last, data.begin(), is_equal_div_10_unique<T>());
  ASSERT_EQUAL(out_last - data.begin(), (std::ptrdiff_t)3);
  got = data;
  got.resize(3);
  ASSERT_EQUAL(got, vec<T>({11, 20, 31}));
}
DECLARE_TYPED_UNITTEST(TestUniqueSimple, int);
DECLARE_TYPED_UNITTEST(TestUniqueSimple, int8_t);
DECLARE_TYPED_UNITTEST(TestUniqueSimple, uint64_t);

// testing/unique.cu:189-226, :272-300: boolean-valued data (short runs) over the ladder, plus
// longer runs that straddle tiles
template <class T>
void TestUniqueLadder() {
  for (std::size_t n : unittest::sizes()) {
    for (int max_run : {2, 40, 5000}) {
      thrust::host_vector<T> h0 = random_runs<T>(n, max_run);
      thrust::host_vector<T> h = h0, hr(n);
      thrust::device_vector<T> d = h0, dr(n);
      auto hce = thrust::unique_copy(h.begin(), h.end(), hr.begin());
      auto dce = thrust::unique_copy(d.begin(), d.end(), dr.begin());
      ASSERT_EQUAL(hce - hr.begin(), dce - dr.begin());
      hr.resize(hce - hr.begin()); dr.resize(dce - dr.begin());
      ASSERT_EQUAL(hr, dr);
      auto he = thrust::unique(h.begin(), h.end());
      auto de = thrust::unique(d.begin(), d.end());
      ASSERT_EQUAL(he - h.begin(), de - d.begin());
      h.resize(he - h.begin()); d.resize(de - d.begin());
      ASSERT_EQUAL(h, d);
      ASSERT_EQUAL(h, hr);
    }
  }
}
DECLARE_TYPED_UNITTEST(TestUniqueLadder, int);
DECLARE_TYPED_UNITTEST(TestUniqueLadder, uint8_t);
DECLARE_TYPED_UNITTEST(TestUniqueLadder, double);

// testing/unique_by_key.cu:128-252
template <class T>
void TestUniqueByKeySimple() {
  const auto keys0 = vec<T>({11, 11, 21, 20, 21, 21, 21, 37, 37});
  const auto vals0 = vec<T>({0, 1, 2, 3, 4, 5, 6, 7, 8});
  thrust::device_vector<T> keys = keys0, values = vals0;
  auto new_last = thrust::unique_by_key(keys.begin(), keys.end(), values.begin());
  ASSERT_EQUAL(new_last.first - keys.begin(), (std::ptrdiff_t)5);
  ASSERT_EQUAL(new_last.second - values.begin(), (std::ptrdiff_t)5);
  keys.resize(5); values.resize(5);
  ASSERT_EQUAL(keys, vec<T>({11, 21, 20, 21, 37}));
  ASSERT_EQUAL(values, vec<T>({0, 2, 3, 4, 7}));

  keys = keys0; values = vals0;
  new_last = thrust::unique_by_key(keys.begin(), keys.end(), values.begin(), is_equal_div_10_unique<T>());
  ASSERT_EQUAL(new_last.first - keys.begin(), (std::ptrdiff_t)3);
  ASSERT_EQUAL(new_last.second - values.begin(), (std::ptrdiff_t)3);
  keys.resize(3); values.resize(3);
  ASSERT_EQUAL(keys, vec<T>({11, 21, 37}));
  ASSERT_EQUAL(values, vec<T>({0, 2, 7}));

  keys = keys0; values = vals0;
  thrust::device_vector<T> ok(9), ov(9);
  auto out_last = thrust::unique_by_key_copy(keys.begin(), keys.end(), values.begin(), ok.begin(), ov.begin());
  ASSERT_EQUAL(out_last.first - ok.begin(), (std::ptrdiff_t)5);
  ASSERT_EQUAL(out_last.second - ov.begin(), (std::ptrdiff_t)5);
  ok.resize(5); ov.resize(5);
  ASSERT_EQUAL(ok, vec<T>({11, 21, 20, 21, 37}));
  ASSERT_EQUAL(ov, vec<T>({0, 2, 3, 4, 7}));
  ok.resize(9); ov.resize(9);
  out_last = thrust::unique_by_key_copy(thrust::device, keys.begin(), keys.end(), values.begin(), ok.begin(), ov.begin(),
                                        is_equal_div_10_unique<T>());
  ASSERT_EQUAL(out_last.first - ok.begin(), (std::ptrdiff_t)3);
  ok.resize(3); ov.resize(3);
  ASSERT_EQUAL(ok, vec<T>({11, 21, 37}));
  ASSERT_EQUAL(ov, vec<T>({0, 2, 7}));
}
DECLARE_TYPED_UNITTEST(TestUniqueByKeySimple, int);
DECLARE_TYPED_UNITTEST(TestUniqueByKeySimple, int16_t);
DECLARE_TYPED_UNITTEST(TestUniqueByKeySimple, uint64_t);

// testing/unique_by_key.cu:256-330: keys with runs, unsigned int values, device vs host
template <class K>
void TestUniqueByKeyLadder() {
  typedef unsigned int V;
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<K> hk0 = random_runs<K>(n, n % 2 ? 3 : 300);
    thrust::host_vector<V> hv0 = unittest::random_integers<V>(n);
    thrust::host_vector<K> hk = hk0, hko(n);
    thrust::host_vector<V> hv = hv0, hvo(n);
    thrust::device_vector<K> dk = hk0, dko(n);
    thrust::device_vector<V> dv = hv0, dvo(n);
    auto hc = thrust::unique_by_key_copy(hk.begin(), hk.end(), hv.begin(), hko.begin(), hvo.begin());
    auto dc = thrust::unique_by_key_copy(dk.begin(), dk.end(), dv.begin(), dko.begin(), dvo.begin());
    ASSERT_EQUAL(hc.first - hko.begin(), dc.first - dko.begin());
    ASSERT_EQUAL(hc.second - hvo.begin(), dc.second - dvo.begin());
    const std::size_t c = hc.first - hko.begin();
    hko.resize(c); hvo.resize(c); dko.resize(c); dvo.resize(c);
    ASSERT_EQUAL(hko, dko);
    ASSERT_EQUAL(hvo, dvo);
    auto hl = thrust::unique_by_key(hk.begin(), hk.end(), hv.begin());
    auto dl = thrust::unique_by_key(dk.begin(), dk.end(), dv.begin());
    ASSERT_EQUAL(hl.first - hk.begin(), dl.first - dk.begin());
    ASSERT_EQUAL((std::size_t)(dl.second - dv.begin()), c);
    hk.resize(c); hv.resize(c); dk.resize(c); dv.resize(c);
    ASSERT_EQUAL(hk, dk);
    ASSERT_EQUAL(hv, dv);
    ASSERT_EQUAL(hk, hko);
  }
}
DECLARE_TYPED_UNITTEST(TestUniqueByKeyLadder, int);
DECLARE_TYPED_UNITTEST(TestUniqueByKeyLadder, uint8_t);
DECLARE_TYPED_UNITTEST(TestUniqueByKeyLadder, int64_t);

// struct keys with a user equivalence
void TestUniqueStruct() {
  const std::size_t n = 99991;
  thrust::host_vector<record> h(n);
  for (std::size_t i = 0; i < n; i++) h[i] = record{(int)(i / 7), (float)i};
  thrust::device_vector<record> d = h;
  auto he = thrust::unique(h.begin(), h.end(), same_id());
  auto de = thrust::unique(d.begin(), d.end(), same_id());
  ASSERT_EQUAL(he - h.begin(), de - d.begin());
  h.resize(he - h.begin()); d.resize(de - d.begin());
  ASSERT_EQUAL(h, d);
}
DECLARE_UNITTEST(TestUniqueStruct);

// 2^26 + 3 elements: more tiles than one scan tile of tile counts holds
void TestCopyIfLarge() {
  const std::size_t n = (std::size_t(1) << 26) + 3;
  thrust::host_vector<int> h = unittest::random_integers<int>(n), hr(n);
  thrust::device_vector<int> d = h, dr(n);
  auto he = thrust::copy_if(h.begin(), h.end(), hr.begin(), is_even<int>());
  auto de = thrust::copy_if(d.begin(), d.end(), dr.begin(), is_even<int>());
  ASSERT_EQUAL(he - hr.begin(), de - dr.begin());
  hr.resize(he - hr.begin()); dr.resize(de - dr.begin());
  ASSERT_EQUAL(hr, dr);
}
DECLARE_UNITTEST(TestCopyIfLarge);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

// Comparison-sort tests in the shape of the reference's testing/stable_sort.cu,
// stable_sort_by_key.cu and sort_by_key.cu (custom comparators, non-arithmetic keys): known
// answers plus device vs std::stable_sort on the host over the size ladder.  This translation
// unit instantiates kernel templates with user comparators, so it is compiled by hipcc.
#include <algorithm>
#include <cstring>
#include <numeric>

#include <thrust/functional.h>
#include <thrust/sort.h>

#include "testing.h"

// testing/stable_sort.cu:43-47
template <class T>
struct less_div_10 {
  __host__ __device__ bool operator()(const T& lhs, const T& rhs) const { return ((int)lhs) / 10 < ((int)rhs) / 10; }
};
template <class T>
struct greater_div_10 {
  __host__ __device__ bool operator()(const T& lhs, const T& rhs) const { return ((int)lhs) / 10 > ((int)rhs) / 10; }
};

// testing/stable_sort.cu:49-90: 9 keys whose tens digit is the sort key
template <class T>
void TestStableSortSimple() {
  const T unsorted[9] = {25, 14, 35, 16, 26, 34, 36, 24, 15};
  const T sorted[9] = {14, 16, 15, 25, 26, 24, 35, 34, 36};
  thrust::device_vector<T> d(unsorted, unsorted + 9);
  thrust::stable_sort(d.begin(), d.end(), less_div_10<T>());
  ASSERT_EQUAL(d, thrust::host_vector<T>(sorted, sorted + 9));
}
DECLARE_TYPED_UNITTEST(TestStableSortSimple, int);
DECLARE_TYPED_UNITTEST(TestStableSortSimple, short);
DECLARE_TYPED_UNITTEST(TestStableSortSimple, uint64_t);
DECLARE_TYPED_UNITTEST(TestStableSortSimple, float);

// testing/stable_sort_by_key.cu:43-95: same keys, values record the input position
void TestStableSortByKeySimple() {
  const int keys[9] = {25, 14, 35, 16, 26, 34, 36, 24, 15};
  const int sorted_keys[9] = {14, 16, 15, 25, 26, 24, 35, 34, 36};
  const int sorted_vals[9] = {1, 3, 8, 0, 4, 7, 2, 5, 6};
  thrust::device_vector<int> k(keys, keys + 9), v(9);
  for (int i = 0; i < 9; i++) v[i] = i;
  thrust::stable_sort_by_key(k.begin(), k.end(), v.begin(), less_div_10<int>());
  ASSERT_EQUAL(k, thrust::host_vector<int>(sorted_keys, sorted_keys + 9));
  ASSERT_EQUAL(v, thrust::host_vector<int>(sorted_vals, sorted_vals + 9));
}
DECLARE_UNITTEST(TestStableSortByKeySimple);

// testing/stable_sort.cu:93-124: device vs host over the size ladder, ties everywhere
template <class T>
void TestStableSortLadder() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<T> h = unittest::random_integers<T>(n);
    for (std::size_t i = 0; i < n; i++) h[i] = (T)(((unsigned)h[i]) % 1000u);
    thrust::device_vector<T> d = h;
    std::vector<T> ref(h.begin(), h.end());
    std::stable_sort(ref.begin(), ref.end(), less_div_10<T>());
    thrust::stable_sort(d.begin(), d.end(), less_div_10<T>());
    ASSERT_EQUAL(d, thrust::host_vector<T>(ref.begin(), ref.end()));
    d = h;
    ref.assign(h.begin(), h.end());
    std::stable_sort(ref.begin(), ref.end(), greater_div_10<T>());
    thrust::sort(d.begin(), d.end(), greater_div_10<T>());
    ASSERT_EQUAL(d, thrust::host_vector<T>(ref.begin(), ref.end()));
  }
}
DECLARE_TYPED_UNITTEST(TestStableSortLadder, int);
DECLARE_TYPED_UNITTEST(TestStableSortLadder, uint16_t);
DECLARE_TYPED_UNITTEST(TestStableSortLadder, int64_t);

// testing/stable_sort.cu:126-174: comparator that looks keys up in a device table
template <class T>
struct comp_mod3 {
  const T* table;
  explicit comp_mod3(const T* t) : table(t) {}
  __host__ __device__ bool operator()(T a, T b) const { return table[(int)a] < table[(int)b]; }
};
void TestStableSortWithIndirection() {
  const int table_h[6] = {0, 1, 2, 0, 1, 2};
  const int data_h[7] = {1, 3, 5, 3, 0, 2, 1};
  const int expect[7] = {3, 3, 0, 1, 1, 5, 2};
  thrust::device_vector<int> table(table_h, table_h + 6), data(data_h, data_h + 7);
  thrust::stable_sort(data.begin(), data.end(), comp_mod3<int>(thrust::raw_pointer_cast(table.data())));
  ASSERT_EQUAL(data, thrust::host_vector<int>(expect, expect + 7));
}
DECLARE_UNITTEST(TestStableSortWithIndirection);

// non-arithmetic keys: a 12-byte record ordered by one field (testing/zip_iterator_sort_by_key.cu
// sorts tuples; a struct key takes the same comparison-sort branch)
struct record {
  int group;
  float weight;
  unsigned id;
};
inline bool operator==(const record& a, const record& b) { return a.group == b.group && a.weight == b.weight && a.id == b.id; }
inline std::ostream& operator<<(std::ostream& os, const record& r) { return os << "(" << r.group << "," << r.weight << "," << r.id << ")"; }
struct by_group {
  __host__ __device__ bool operator()(const record& a, const record& b) const { return a.group < b.group; }
};
void TestSortStructKeys() {
  for (std::size_t n : {std::size_t(0), std::size_t(1), std::size_t(2047), std::size_t(2048), std::size_t(2049),
                        std::size_t(100003), std::size_t(1) << 20}) {
    thrust::host_vector<record> h(n);
    std::uint64_t s = 4242 + n;
    for (std::size_t i = 0; i < n; i++) {
      h[i].group = (int)(unittest::splitmix64(s) % 37);
      h[i].weight = (float)(unittest::splitmix64(s) % 1000) / 8.0f;
      h[i].id = (unsigned)i;
    }
    thrust::device_vector<record> d = h;
    std::vector<record> ref(h.begin(), h.end());
    std::stable_sort(ref.begin(), ref.end(), by_group());
    thrust::sort(d.begin(), d.end(), by_group());
    ASSERT_EQUAL(d, thrust::host_vector<record>(ref.begin(), ref.end()));
  }
}
DECLARE_UNITTEST(TestSortStructKeys);

// sort_by_key with a custom comparator and values of every width the kernels take
template <class V>
void TestStableSortByKeyLadder() {
  for (std::size_t n : unittest::sizes()) {
    thrust::host_vector<int> hk = unittest::random_integers<int>(n);
    for (std::size_t i = 0; i < n; i++) hk[i] = (int)(((unsigned)hk[i]) % 500u);
    thrust::host_vector<V> hv(n);
    for (std::size_t i = 0; i < n; i++) hv[i] = (V)i;
    thrust::device_vector<int> dk = hk;
    thrust::device_vector<V> dv = hv;
    std::vector<std::size_t> idx(n);
    std::iota(idx.begin(), idx.end(), std::size_t(0));
    std::stable_sort(idx.begin(), idx.end(), [&](std::size_t a, std::size_t b) { return less_div_10<int>()(hk[a], hk[b]); });
    thrust::host_vector<int> rk(n);
    thrust::host_vector<V> rv(n);
    for (std::size_t i = 0; i < n; i++) { rk[i] = hk[idx[i]]; rv[i] = hv[idx[i]]; }
    thrust::stable_sort_by_key(dk.begin(), dk.end(), dv.begin(), less_div_10<int>());
    ASSERT_EQUAL(dk, rk);
    ASSERT_EQUAL(dv, rv);
  }
}
DECLARE_TYPED_UNITTEST(TestStableSortByKeyLadder, uint8_t);
DECLARE_TYPED_UNITTEST(TestStableSortByKeyLadder, int);
DECLARE_TYPED_UNITTEST(TestStableSortByKeyLadder, double);

// testing/stable_sort_by_key_large_values.cu: values wider than the radix path's 8 bytes
struct wide_value {
  std::uint64_t a, b;
};
inline bool operator==(const wide_value& x, const wide_value& y) { return x.a == y.a && x.b == y.b; }
inline std::ostream& operator<<(std::ostream& os, const wide_value& v) { return os << "(" << v.a << "," << v.b << ")"; }
void TestSortByKeyLargeValues() {
  const std::size_t n = 300007;
  thrust::host_vector<unsigned> hk = unittest::random_integers<unsigned>(n);
  thrust::host_vector<wide_value> hv(n);
  for (std::size_t i = 0; i < n; i++) { hk[i] %= 4096u; hv[i].a = i; hv[i].b = ~(std::uint64_t)i; }
  thrust::device_vector<unsigned> dk = hk;
  thrust::device_vector<wide_value> dv = hv;
  std::vector<std::size_t> idx(n);
  std::iota(idx.begin(), idx.end(), std::size_t(0));
  std::stable_sort(idx.begin(), idx.end(), [&](std::size_t a, std::size_t b) { return hk[a] < hk[b]; });
  thrust::host_vector<unsigned> rk(n);
  thrust::host_vector<wide_value> rv(n);
  for (std::size_t i = 0; i < n; i++) { rk[i] = hk[idx[i]]; rv[i] = hv[idx[i]]; }
  thrust::sort_by_key(dk.begin(), dk.end(), dv.begin());  // thrust::less, but 16-byte values: comparison sort
  ASSERT_EQUAL(dk, rk);
  ASSERT_EQUAL(dv, rv);
}
DECLARE_UNITTEST(TestSortByKeyLargeValues);

// a sorted and a reversed input of 2^22 + 5 keys: many merge passes, ragged last tile
void TestStableSortLarge() {
  const std::size_t n = (std::size_t(1) << 22) + 5;
  thrust::host_vector<int> h(n);
  for (std::size_t i = 0; i < n; i++) h[i] = (int)(n - i);
  thrust::device_vector<int> d = h;
  thrust::stable_sort(d.begin(), d.end(), less_div_10<int>());
  std::vector<int> ref(h.begin(), h.end());
  std::stable_sort(ref.begin(), ref.end(), less_div_10<int>());
  ASSERT_EQUAL(d, thrust::host_vector<int>(ref.begin(), ref.end()));
}
DECLARE_UNITTEST(TestStableSortLarge);

// the same full-range random input sorted eight times in a row: the tile sort reads LDS into
// registers, passes a barrier and writes them back, which must not race between wavefronts
void TestStableSortRepeatable() {
  const std::size_t n = std::size_t(1) << 22;
  thrust::host_vector<unsigned> h = unittest::random_integers<unsigned>(n, 1337);
  std::vector<unsigned> ref(h.begin(), h.end());
  std::stable_sort(ref.begin(), ref.end());
  const thrust::host_vector<unsigned> expected(ref.begin(), ref.end());
  const thrust::device_vector<unsigned> src = h;
  for (int rep = 0; rep < 8; rep++) {
    thrust::device_vector<unsigned> d = src;
    thrust::sort(d.begin(), d.end(), less_div_10<unsigned>());  // ties by tens, then
    thrust::sort(d.begin(), d.end(), [] __host__ __device__(unsigned a, unsigned b) { return a < b; });
    ASSERT_EQUAL(d, expected);
  }
}
DECLARE_UNITTEST(TestStableSortRepeatable);

// Ranges that start a few elements into an allocation and end a few before its end: the tile
// sort and the merge passes move a thread's items as 16-byte blocks at the items' own alignment
// (2 bytes here for the pairs), whole tiles and the partial last one alike.
template <class K>
void TestStableSortOffsetRanges() {
  for (std::size_t n : {std::size_t(5000), std::size_t(4096 * 9 + 2), std::size_t(300007)}) {
    for (std::size_t skip : {std::size_t(1), std::size_t(3)}) {
      thrust::host_vector<K> h = unittest::random_integers<K>(n + skip + 2, 7 * n + skip);
      thrust::host_vector<K> hv(n + skip + 2);
      for (std::size_t i = 0; i < hv.size(); i++) hv[i] = (K)i;
      // keys alone
      thrust::device_vector<K> d = h;
      std::vector<K> ref(h.begin(), h.end());
      std::stable_sort(ref.begin() + skip, ref.begin() + skip + n, less_div_10<K>());
      thrust::stable_sort(d.begin() + skip, d.begin() + skip + n, less_div_10<K>());
      ASSERT_EQUAL(d, thrust::host_vector<K>(ref.begin(), ref.end()));  // the elements around the range are untouched
      // pairs: the values record where each key came from
      thrust::device_vector<K> dk = h, dv = hv;
      std::vector<std::size_t> order(n);
      std::iota(order.begin(), order.end(), skip);
      std::stable_sort(order.begin(), order.end(), [&](std::size_t a, std::size_t b) { return less_div_10<K>()(h[a], h[b]); });
      thrust::stable_sort_by_key(dk.begin() + skip, dk.begin() + skip + n, dv.begin() + skip, less_div_10<K>());
      thrust::host_vector<K> ek = h, ev = hv;
      for (std::size_t i = 0; i < n; i++) { ek[skip + i] = h[order[i]]; ev[skip + i] = hv[order[i]]; }
      ASSERT_EQUAL(dk, ek);
      ASSERT_EQUAL(dv, ev);
    }
  }
}
DECLARE_TYPED_UNITTEST(TestStableSortOffsetRanges, uint16_t);
DECLARE_TYPED_UNITTEST(TestStableSortOffsetRanges, unsigned);
DECLARE_TYPED_UNITTEST(TestStableSortOffsetRanges, int64_t);

// testing/stable_sort_large.cu, stable_sort_by_key_large_keys.cu, ..._large_keys_and_values.cu:
// keys and values of N ints, ordered by their first; N up to 2048 ints (8 KiB) an element.  Wider
// than an LDS tile allows, so positions are sorted and the elements gathered.
template <int N>
struct fixed_vector {
  int v[N];
  __host__ __device__ fixed_vector() { for (int i = 0; i < N; i++) v[i] = 0; }
  __host__ __device__ explicit fixed_vector(int x) { for (int i = 0; i < N; i++) v[i] = x; }
  __host__ __device__ bool operator<(const fixed_vector& o) const { return v[0] < o.v[0]; }
  __host__ __device__ bool operator==(const fixed_vector& o) const {
    for (int i = 0; i < N; i++) if (v[i] != o.v[i]) return false;
    return true;
  }
};
template <int N> inline std::ostream& operator<<(std::ostream& os, const fixed_vector<N>& f) { return os << "fixed_vector(" << f.v[0] << ")"; }
template <int N>
void TestStableSortWideKeysAndValues() {
  const std::size_t n = (128 * 1024) / sizeof(fixed_vector<N>) + 3;
  thrust::host_vector<fixed_vector<N>> hk(n), hv(n);
  thrust::host_vector<int> r = unittest::random_integers<int>(n);
  for (std::size_t i = 0; i < n; i++) { hk[i] = fixed_vector<N>((r[i] & 0x7fffffff) % 97); hv[i] = fixed_vector<N>((int)i); }
  std::vector<std::size_t> idx(n);
  std::iota(idx.begin(), idx.end(), std::size_t(0));
  std::stable_sort(idx.begin(), idx.end(), [&](std::size_t a, std::size_t b) { return hk[a] < hk[b]; });
  thrust::host_vector<fixed_vector<N>> rk(n), rv(n);
  for (std::size_t i = 0; i < n; i++) { rk[i] = hk[idx[i]]; rv[i] = hv[idx[i]]; }
  {  // keys only
    thrust::device_vector<fixed_vector<N>> dk = hk;
    thrust::stable_sort(dk.begin(), dk.end());
    ASSERT_EQUAL(dk == rk, true);
  }
  {  // wide keys, int values
    thrust::device_vector<fixed_vector<N>> dk = hk;
    thrust::device_vector<int> dv(n);
    thrust::sequence(dv.begin(), dv.end());
    thrust::stable_sort_by_key(dk.begin(), dk.end(), dv.begin());
    ASSERT_EQUAL(dk == rk, true);
    thrust::host_vector<int> ri(n);
    for (std::size_t i = 0; i < n; i++) ri[i] = (int)idx[i];
    ASSERT_EQUAL(dv, ri);
  }
  {  // wide keys and wide values
    thrust::device_vector<fixed_vector<N>> dk = hk, dv = hv;
    thrust::stable_sort_by_key(dk.begin(), dk.end(), dv.begin());
    ASSERT_EQUAL(dk == rk, true);
    ASSERT_EQUAL(dv == rv, true);
  }
}
void TestStableSortWide16() { TestStableSortWideKeysAndValues<16>(); }
void TestStableSortWide33() { TestStableSortWideKeysAndValues<33>(); }
void TestStableSortWide256() { TestStableSortWideKeysAndValues<256>(); }
void TestStableSortWide2048() { TestStableSortWideKeysAndValues<2048>(); }
DECLARE_UNITTEST(TestStableSortWide16);
DECLARE_UNITTEST(TestStableSortWide33);
DECLARE_UNITTEST(TestStableSortWide256);
DECLARE_UNITTEST(TestStableSortWide2048);

// a 4-byte key whose default constructor is written out (LDS arrays cannot hold it): the same path,
// over the size ladder and under a comparator of the user's
struct counted_key {
  int x;
  __host__ __device__ counted_key() : x(-1) {}
  __host__ __device__ explicit counted_key(int y) : x(y) {}
  __host__ __device__ bool operator==(const counted_key& o) const { return x == o.x; }
};
inline std::ostream& operator<<(std::ostream& os, const counted_key& k) { return os << k.x; }
struct counted_key_tens {
  __host__ __device__ bool operator()(const counted_key& a, const counted_key& b) const { return a.x / 10 < b.x / 10; }
};
void TestStableSortKeysWithConstructors() {
  for (std::size_t n : unittest::sizes()) {
    if (n > 300000) continue;
    thrust::host_vector<int> r = unittest::random_integers<int>(n);
    thrust::host_vector<counted_key> h(n);
    for (std::size_t i = 0; i < n; i++) h[i] = counted_key((r[i] & 0x7fffffff) % 1000);
    thrust::device_vector<counted_key> d = h;
    thrust::stable_sort(d.begin(), d.end(), counted_key_tens());
    std::vector<counted_key> ref(h.begin(), h.end());
    std::stable_sort(ref.begin(), ref.end(), counted_key_tens());
    ASSERT_EQUAL(d == thrust::host_vector<counted_key>(ref.begin(), ref.end()), true);
  }
}
DECLARE_UNITTEST(TestStableSortKeysWithConstructors);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

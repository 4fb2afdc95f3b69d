// thrust::host_vector as a container of its own — the cases of testing/vector.cu,
// vector_insert.cu and vector_manipulation.cu that need no device (construction, assignment between
// element types and from std containers, bool elements, insert / erase / resize / assign, iterators,
// comparison), checked against std::vector doing the same.  Runs on the CPU: nothing here touches
// device memory.
#include <list>
#include <string>
#include <vector>

#include <thrust/host_vector.h>

#include "testing.h"

template <class T>
static void expect_same(const thrust::host_vector<T>& h, const std::vector<T>& v) {
  ASSERT_EQUAL(h.size(), v.size());
  for (std::size_t i = 0; i < v.size(); i++) ASSERT_EQUAL(h[i] == v[i], true);
}

void TestHostVectorConstruction() {
  thrust::host_vector<int> a;
  ASSERT_EQUAL(a.empty(), true);
  thrust::host_vector<int> b(5);
  expect_same(b, std::vector<int>(5));
  thrust::host_vector<int> c(4, 7);
  expect_same(c, std::vector<int>(4, 7));
  thrust::host_vector<int> d{1, 2, 3};
  expect_same(d, std::vector<int>{1, 2, 3});
  thrust::host_vector<int> e(d);
  expect_same(e, std::vector<int>{1, 2, 3});
  thrust::host_vector<int> f(std::move(e));
  expect_same(f, std::vector<int>{1, 2, 3});
  ASSERT_EQUAL(e.size(), std::size_t(0));
  std::list<int> l{9, 8, 7};
  thrust::host_vector<int> g(l.begin(), l.end());
  expect_same(g, std::vector<int>{9, 8, 7});
  std::vector<short> sv{4, 5};
  thrust::host_vector<int> h(sv);
  expect_same(h, std::vector<int>{4, 5});
  thrust::host_vector<double> i(h);  // another element type
  ASSERT_EQUAL(i[1], 5.0);
  thrust::host_vector<int> j(10, 3);  // two integers are a count and a value, not a range
  ASSERT_EQUAL(j.size(), std::size_t(10));
  int raw[3] = {1, 2, 3};
  thrust::host_vector<int> k(raw, raw + 3);
  expect_same(k, std::vector<int>{1, 2, 3});
}
DECLARE_UNITTEST(TestHostVectorConstruction);

void TestHostVectorOfBoolIsAnArray() {
  thrust::host_vector<bool> b(70, false);
  b[3] = true; b[69] = true;
  bool* p = b.data();  // one object per element
  ASSERT_EQUAL(p[3], true);
  ASSERT_EQUAL(p[4], false);
  ASSERT_EQUAL(p[69], true);
  thrust::host_vector<unsigned char> u(b);
  ASSERT_EQUAL((int)u[3], 1);
  thrust::host_vector<bool> back(u);
  ASSERT_EQUAL(back == b, true);
}
DECLARE_UNITTEST(TestHostVectorOfBoolIsAnArray);

void TestHostVectorAssignment() {
  thrust::host_vector<int> a{1, 2, 3}, b;
  b = a;
  expect_same(b, std::vector<int>{1, 2, 3});
  b = {4, 5};
  expect_same(b, std::vector<int>{4, 5});
  b = std::vector<long>{7, 8, 9, 10};
  expect_same(b, std::vector<int>{7, 8, 9, 10});
  b = b;  // self
  expect_same(b, std::vector<int>{7, 8, 9, 10});
  b.assign(3, 1);
  expect_same(b, std::vector<int>{1, 1, 1});
  b.assign(a.begin() + 1, a.end());
  expect_same(b, std::vector<int>{2, 3});
  a.assign(a.begin() + 1, a.end());  // from itself
  expect_same(a, std::vector<int>{2, 3});
  thrust::host_vector<int> big(1000);
  for (int i = 0; i < 1000; i++) big[i] = i;
  a = big;  // grows
  ASSERT_EQUAL(a.size(), std::size_t(1000));
  ASSERT_EQUAL(a[999], 999);
  a = std::move(big);
  ASSERT_EQUAL(a[500], 500);
}
DECLARE_UNITTEST(TestHostVectorAssignment);

// testing/vector.cu:780-840: a moved-from vector is empty and the target has its storage
void TestHostVectorMove() {
  thrust::host_vector<int> v1{0, 1, 2};
  const int* p1 = v1.data();
  thrust::host_vector<int> v2(std::move(v1));
  ASSERT_EQUAL(v1.empty(), true);
  ASSERT_EQUAL(v2.data() == p1, true);
  thrust::host_vector<int> v3{3, 4, 5};
  const int* p3 = v3.data();
  v2 = std::move(v3);
  ASSERT_EQUAL(v3.empty(), true);
  ASSERT_EQUAL(v2.data() == p3, true);
  ASSERT_EQUAL(v2[2], 5);
  thrust::pair<int, float> z;
  ASSERT_EQUAL(z.first, 0);
  ASSERT_EQUAL(z.second, 0.0f);
}
DECLARE_UNITTEST(TestHostVectorMove);

void TestHostVectorGrowthAndShrinking() {
  thrust::host_vector<int> h;
  std::vector<int> v;
  for (int i = 0; i < 1000; i++) { h.push_back(i * 3); v.push_back(i * 3); }
  expect_same(h, v);
  ASSERT_EQUAL(h.capacity() >= h.size(), true);
  h.push_back(h[0]);  // an element of itself while growing
  v.push_back(v[0]);
  h.resize(10); v.resize(10);
  expect_same(h, v);
  h.resize(20, -1); v.resize(20, -1);
  expect_same(h, v);
  h.pop_back(); v.pop_back();
  expect_same(h, v);
  h.reserve(5000);
  ASSERT_EQUAL(h.capacity() >= std::size_t(5000), true);
  expect_same(h, v);
  h.shrink_to_fit();
  ASSERT_EQUAL(h.capacity(), h.size());
  expect_same(h, v);
  ASSERT_EQUAL(h.front(), v.front());
  ASSERT_EQUAL(h.back(), v.back());
  ASSERT_EQUAL(h.at(3), v.at(3));
  bool threw = false;
  try { h.at(1000); } catch (const std::out_of_range&) { threw = true; }
  ASSERT_EQUAL(threw, true);
  h.clear();
  ASSERT_EQUAL(h.empty(), true);
}
DECLARE_UNITTEST(TestHostVectorGrowthAndShrinking);

// testing/vector_insert.cu: every position, counts that do and do not force a reallocation
void TestHostVectorInsertAndErase() {
  for (std::size_t n : {0u, 1u, 2u, 7u, 64u}) {
    for (std::size_t at = 0; at <= n; at++) {
      for (std::size_t count : {0u, 1u, 3u, 100u}) {
        thrust::host_vector<int> h(n);
        std::vector<int> v(n);
        for (std::size_t i = 0; i < n; i++) h[i] = v[i] = (int)i;
        h.insert(h.begin() + at, count, 42);
        v.insert(v.begin() + at, count, 42);
        expect_same(h, v);
        std::vector<int> src(count);
        for (std::size_t i = 0; i < count; i++) src[i] = -(int)i;
        auto it = h.insert(h.begin() + at, src.begin(), src.end());
        v.insert(v.begin() + at, src.begin(), src.end());
        ASSERT_EQUAL((std::size_t)(it - h.begin()), at);
        expect_same(h, v);
        if (!h.empty()) {
          const std::size_t e = at < h.size() ? at : h.size() - 1;
          h.erase(h.begin() + e); v.erase(v.begin() + e);
          expect_same(h, v);
          const std::size_t last = e + count < h.size() ? e + count : h.size();
          auto r = h.erase(h.begin() + e, h.begin() + last);
          v.erase(v.begin() + e, v.begin() + last);
          ASSERT_EQUAL((std::size_t)(r - h.begin()), e);
          expect_same(h, v);
        }
      }
    }
  }
  thrust::host_vector<int> h{1, 2, 3, 4};
  h.insert(h.begin() + 1, h.begin(), h.end());  // a range of itself
  expect_same(h, std::vector<int>{1, 1, 2, 3, 4, 2, 3, 4});
  h.insert(h.begin(), h[7]);  // an element of itself
  ASSERT_EQUAL(h[0], 4);
}
DECLARE_UNITTEST(TestHostVectorInsertAndErase);

void TestHostVectorIteratorsAndComparison() {
  thrust::host_vector<int> h{3, 1, 2};
  thrust::host_vector<int>::const_iterator c = h.begin();  // iterator -> const_iterator
  ASSERT_EQUAL(*c, 3);
  ASSERT_EQUAL(h.end() - h.begin(), std::ptrdiff_t(3));
  ASSERT_EQUAL(h.begin()[2], 2);
  ASSERT_EQUAL(*(h.rbegin()), 2);
  ASSERT_EQUAL(*(h.crend() - 1), 3);
  std::sort(h.begin(), h.end());
  expect_same(h, std::vector<int>{1, 2, 3});
  ASSERT_EQUAL(h == (thrust::host_vector<int>{1, 2, 3}), true);
  ASSERT_EQUAL(h != (thrust::host_vector<int>{1, 2}), true);
  ASSERT_EQUAL(h == (std::vector<int>{1, 2, 3}), true);
  ASSERT_EQUAL((std::vector<long>{1, 2, 3}) == h, true);
  thrust::host_vector<int> o{9};
  swap(h, o);
  ASSERT_EQUAL(h.size(), std::size_t(1));
  ASSERT_EQUAL(o.size(), std::size_t(3));
  const thrust::host_vector<int>& k = o;
  ASSERT_EQUAL(*k.begin(), 1);
  ASSERT_EQUAL(k.data()[1], 2);
}
DECLARE_UNITTEST(TestHostVectorIteratorsAndComparison);

// elements that own memory: construction, destruction and moves are counted right
void TestHostVectorOfStrings() {
  thrust::host_vector<std::string> h;
  std::vector<std::string> v;
  for (int i = 0; i < 100; i++) { h.push_back(std::string(40, 'a' + i % 26)); v.push_back(std::string(40, 'a' + i % 26)); }
  h.insert(h.begin() + 5, 3, std::string("xyz")); v.insert(v.begin() + 5, 3, std::string("xyz"));
  h.erase(h.begin() + 10, h.begin() + 50); v.erase(v.begin() + 10, v.begin() + 50);
  h.resize(200, std::string("tail")); v.resize(200, std::string("tail"));
  h.resize(20); v.resize(20);
  thrust::host_vector<std::string> copy(h);
  h.clear();
  ASSERT_EQUAL(copy.size(), v.size());
  for (std::size_t i = 0; i < v.size(); i++) ASSERT_EQUAL(copy[i] == v[i], true);
  h.emplace_back(5, 'q');
  ASSERT_EQUAL(h.back() == std::string("qqqqq"), true);
}
DECLARE_UNITTEST(TestHostVectorOfStrings);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

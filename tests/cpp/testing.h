// Minimal unit-test harness for the C++ API tests, shaped after the reference's
// testing/unittest framework: tests register themselves, compare host and device results
// with ASSERT_EQUAL, and sweep the reference's size ladder
// (testing/unittest/testframework.cu:21-31).
#pragma once
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include <thrust/device_vector.h>
#include <thrust/host_vector.h>

namespace unittest {

struct failure : std::runtime_error {
  using std::runtime_error::runtime_error;
};

struct registry {
  static std::vector<std::pair<std::string, std::function<void()>>>& tests() {
    static std::vector<std::pair<std::string, std::function<void()>>> t;
    return t;
  }
};
struct registrar {
  registrar(const char* name, std::function<void()> f) { registry::tests().emplace_back(name, f); }
};

#define DECLARE_UNITTEST(NAME) static unittest::registrar reg_##NAME(#NAME, NAME)
#define DECLARE_TYPED_UNITTEST(NAME, T) static unittest::registrar reg_##NAME##_##T(#NAME "<" #T ">", NAME<T>)

inline void fail(const char* file, int line, const std::string& msg) {
  std::ostringstream os;
  os << file << ":" << line << ": " << msg;
  throw failure(os.str());
}

#define ASSERT_EQUAL(A, B) unittest::assert_equal((A), (B), #A " == " #B, __FILE__, __LINE__)
#define ASSERT_TRUE(A) do { if (!(A)) unittest::fail(__FILE__, __LINE__, "expected " #A); } while (0)
#define ASSERT_THROWS(EXPR, EXC) do { bool caught = false; try { EXPR; } catch (const EXC&) { caught = true; } \
  if (!caught) unittest::fail(__FILE__, __LINE__, #EXPR " did not throw " #EXC); } while (0)

template <class A, class B>
void assert_equal(const A& a, const B& b, const char* expr, const char* file, int line) {
  if (!(a == b)) {
    std::ostringstream os;
    os << expr << " failed: " << a << " vs " << b;
    fail(file, line, os.str());
  }
}
// characters print as numbers; everything else as it is
template <class T, typename std::enable_if<std::is_arithmetic<T>::value, int>::type = 0>
auto printable(const T& x) -> decltype(+x) { return +x; }
template <class T, typename std::enable_if<!std::is_arithmetic<T>::value, int>::type = 0>
const T& printable(const T& x) { return x; }

template <class T, class U, class VecA, class VecB>
void assert_equal_vec(const VecA& a, const VecB& b, const char* expr, const char* file, int line) {
  if (a.size() != b.size()) {
    std::ostringstream os;
    os << expr << " failed: sizes " << a.size() << " vs " << b.size();
    fail(file, line, os.str());
  }
  for (std::size_t i = 0; i < a.size(); i++) {
    if (!(a[i] == (T)b[i])) {
      std::ostringstream os;
      os << expr << " failed at [" << i << "] of " << a.size() << ": " << printable(a[i]) << " vs " << printable(b[i]);
      fail(file, line, os.str());
    }
  }
}
template <class T>
void assert_equal(const thrust::host_vector<T>& a, const thrust::host_vector<T>& b, const char* e, const char* f, int l) {
  assert_equal_vec<T, T>(a, b, e, f, l);
}
template <class T>
void assert_equal(const thrust::host_vector<T>& a, const thrust::device_vector<T>& b, const char* e, const char* f, int l) {
  assert_equal_vec<T, T>(a, thrust::host_vector<T>(b), e, f, l);
}
template <class T>
void assert_equal(const thrust::device_vector<T>& a, const thrust::host_vector<T>& b, const char* e, const char* f, int l) {
  assert_equal_vec<T, T>(thrust::host_vector<T>(a), b, e, f, l);
}
template <class T>
void assert_equal(const thrust::device_vector<T>& a, const thrust::device_vector<T>& b, const char* e, const char* f, int l) {
  assert_equal_vec<T, T>(thrust::host_vector<T>(a), thrust::host_vector<T>(b), e, f, l);
}

// sizes of the reference's variable-size tests up to 2^20+1
inline const std::vector<std::size_t>& sizes() {
  static const std::vector<std::size_t> s = {
      0, 1, 2, 3, 4, 5, 8, 10, 13, 16, 17, 19, 27, 30, 31, 32, 33, 35, 42, 53, 58, 63, 64, 65, 72, 97, 100, 127,
      128, 129, 142, 183, 192, 201, 240, 255, 256, 257, 302, 511, 512, 513, 687, 900, 1023, 1024, 1025, 1565,
      1786, 1973, 2047, 2048, 2049, 3050, 4095, 4096, 4097, 5030, 7791, 10000, 10027, 12345, 16384, 17354,
      26255, 32768, 43718, 65533, 65536, 65539, 123456, 131072, 731588, 1048575, 1048576, 1048577};
  return s;
}

inline std::uint64_t splitmix64(std::uint64_t& x) {
  std::uint64_t z = (x += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
// deterministic pseudo-random integers over the full range of T
template <class T>
thrust::host_vector<T> random_integers(std::size_t n, std::uint64_t seed = 12345) {
  thrust::host_vector<T> v(n);
  std::uint64_t s = seed + n;
  for (std::size_t i = 0; i < n; i++) v[i] = (T)splitmix64(s);
  return v;
}
template <class T>
thrust::host_vector<T> random_samples(std::size_t n, std::uint64_t seed = 777) {
  thrust::host_vector<T> v(n);
  std::uint64_t s = seed + n;
  for (std::size_t i = 0; i < n; i++) v[i] = (T)((double)(splitmix64(s) >> 11) / 9007199254740992.0 * 200.0 - 100.0);
  return v;
}

// `binary [substring]` runs the tests whose name contains the substring.  THRUST_CDNA4_TEST_SKIP
// holds comma-separated substrings of names to leave out (the emulated run skips the tests whose
// inputs only a device gets through in reasonable time).
inline bool skipped_by_environment(const std::string& name) {
  const char* skip = std::getenv("THRUST_CDNA4_TEST_SKIP");
  if (!skip) return false;
  std::string all(skip);
  std::size_t from = 0;
  while (from <= all.size()) {
    std::size_t to = all.find(',', from);
    if (to == std::string::npos) to = all.size();
    if (to > from && name.find(all.substr(from, to - from)) != std::string::npos) return true;
    from = to + 1;
  }
  return false;
}

inline int run_all(int argc, char** argv) {
  int failed = 0, ran = 0;
  for (auto& t : registry::tests()) {
    if (argc > 1 && t.first.find(argv[1]) == std::string::npos) continue;
    if (skipped_by_environment(t.first)) {
      std::printf("[SKIP] %s\n", t.first.c_str());
      continue;
    }
    ++ran;
    try {
      t.second();
      std::printf("[PASS] %s\n", t.first.c_str());
    } catch (const std::exception& e) {
      ++failed;
      std::printf("[FAIL] %s: %s\n", t.first.c_str(), e.what());
    }
    std::fflush(stdout);
  }
  std::printf("%d tests, %d failed\n", ran, failed);
  return failed ? 1 : 0;
}

}  // namespace unittest

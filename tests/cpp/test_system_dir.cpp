// The device system's own directory, used as the reference's is (thrust/system/cuda/vector.h,
// memory.h, pointer.h, execution_policy.h; testing/cuda/... include them first): thrust::cdna4::
// vector / pointer / malloc / free / allocator / par, the system's single-element primitives, and
// thrust::malloc / free / get_temporary_buffer / return_temporary_buffer with a policy, including a
// user's own for a policy type of theirs (thrust/memory.h:203-395; testing/allocator.cu and
// examples/cuda/custom_temporary_allocation.cu:168-176 use that customisation point).
#include <thrust/system/cdna4/execution_policy.h>
#include <thrust/system/cdna4/memory.h>
#include <thrust/system/cdna4/pointer.h>
#include <thrust/system/cdna4/vector.h>

#include <thrust/fill.h>
#include <thrust/memory.h>
#include <thrust/reduce.h>
#include <thrust/sort.h>

#include "testing.h"

void TestSystemVectorPointerAndMalloc() {
  thrust::cdna4::vector<int> v(100, 3);
  v[5] = 1;
  thrust::sort(thrust::cdna4::par, v.begin(), v.end());
  ASSERT_EQUAL((int)v[0], 1);
  ASSERT_EQUAL((int)v[99], 3);
  static_assert(std::is_same<thrust::cdna4::vector<int>, thrust::device_vector<int>>::value, "the system's vector");
  thrust::cdna4::pointer<int> p = thrust::cdna4::malloc<int>(10);
  ASSERT_TRUE(p.get() != nullptr);
  thrust::fill(thrust::device, p, p + 10, 7);
  ASSERT_EQUAL(thrust::reduce(thrust::cdna4::par, p, p + 10), 70);
  thrust::cdna4::free(thrust::cdna4::pointer<void>(static_cast<void*>(p.get())));
  thrust::cdna4::allocator<int> alloc;
  thrust::cdna4::pointer<int> q = alloc.allocate(4);
  alloc.deallocate(q, 4);
  thrust::cdna4::universal_vector<int> u(8, 2);
  ASSERT_EQUAL(thrust::raw_pointer_cast(u.data())[7], 2);  // host-addressable
}
DECLARE_UNITTEST(TestSystemVectorPointerAndMalloc);

void TestSingleElementPrimitives() {
  thrust::device_vector<int> v(4);
  v[0] = 10; v[1] = 20; v[2] = 30; v[3] = 40;
  ASSERT_EQUAL(thrust::system::cdna4::get_value(thrust::device, v.begin() + 2), 30);
  thrust::system::cdna4::assign_value(thrust::device, v.begin(), v.begin() + 3);  // device to device
  ASSERT_EQUAL((int)v[0], 40);
  const int from_host = 7;
  thrust::system::cdna4::assign_value(thrust::device, v.begin() + 1, &from_host);
  ASSERT_EQUAL((int)v[1], 7);
  thrust::system::cdna4::iter_swap(thrust::device, v.begin() + 1, v.begin() + 2);
  ASSERT_EQUAL((int)v[1], 30);
  ASSERT_EQUAL((int)v[2], 7);
}
DECLARE_UNITTEST(TestSingleElementPrimitives);

void TestMallocAndTemporaryBuffersWithAPolicy() {
  thrust::device_ptr<void> raw = thrust::malloc(thrust::device, 64);
  ASSERT_TRUE(raw.get() != nullptr);
  thrust::free(thrust::device, raw);
  thrust::device_ptr<double> d = thrust::malloc<double>(thrust::device, 8);
  thrust::fill(thrust::device, d, d + 8, 0.5);
  ASSERT_EQUAL(thrust::reduce(thrust::device, d, d + 8), 4.0);
  thrust::free(thrust::device, d);
  auto buf = thrust::get_temporary_buffer<int>(thrust::device, 50);
  ASSERT_EQUAL((int)buf.second, 50);
  thrust::fill(thrust::device, buf.first, buf.first + 50, 2);
  ASSERT_EQUAL(thrust::reduce(thrust::device, buf.first, buf.first + 50), 100);
  thrust::return_temporary_buffer(thrust::device, buf.first, buf.second);
  auto none = thrust::get_temporary_buffer<int>(thrust::device, 0);
  ASSERT_EQUAL((int)none.second, 0);
  // the host system
  int* hp = thrust::malloc<int>(thrust::host, 4);
  hp[3] = 9;
  thrust::free(thrust::host, hp);
  auto hb = thrust::get_temporary_buffer<int>(thrust::host, 5);
  ASSERT_EQUAL((int)hb.second, 5);
  thrust::return_temporary_buffer(thrust::host, hb.first, hb.second);
}
DECLARE_UNITTEST(TestMallocAndTemporaryBuffersWithAPolicy);

// a policy type that brings its own temporary buffers and malloc
struct my_memory_system : thrust::device_execution_policy<my_memory_system> {
  int mallocs = 0, frees = 0, gets = 0, returns = 0;
};
thrust::device_ptr<void> malloc(my_memory_system& s, std::size_t n) {
  s.mallocs++;
  return thrust::malloc(thrust::device, n);
}
template <class Pointer> void free(my_memory_system& s, Pointer p) {
  s.frees++;
  thrust::free(thrust::device, p);
}
template <class T> thrust::pair<thrust::device_ptr<T>, std::ptrdiff_t> get_temporary_buffer(my_memory_system& s, std::ptrdiff_t n) {
  s.gets++;
  return thrust::get_temporary_buffer<T>(thrust::device, n);
}
template <class Pointer> void return_temporary_buffer(my_memory_system& s, Pointer p, std::ptrdiff_t n) {
  s.returns++;
  thrust::return_temporary_buffer(thrust::device, p, n);
}
void TestUserPolicyBringsItsOwnMemory() {
  my_memory_system sys;
  thrust::device_ptr<void> p = thrust::malloc(sys, 128);
  thrust::free(sys, p);
  auto b = thrust::get_temporary_buffer<float>(sys, 16);
  ASSERT_EQUAL((int)b.second, 16);
  thrust::return_temporary_buffer(sys, b.first, b.second);
  ASSERT_EQUAL(sys.mallocs, 1);
  ASSERT_EQUAL(sys.frees, 1);
  ASSERT_EQUAL(sys.gets, 1);
  ASSERT_EQUAL(sys.returns, 1);
}
DECLARE_UNITTEST(TestUserPolicyBringsItsOwnMemory);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

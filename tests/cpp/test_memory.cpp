// device_new / device_delete, device_make_unique, allocate_unique, the device_malloc and
// device_new allocators, per-device resources, universal (host- and device-addressable) memory
// and the type traits headers — after testing/device_delete.cu, allocator.cu:170-230,
// universal_memory.cu:40-150 and testing/type_traits.cu.  Compiled by hipcc (reduce and sequence on device ranges are kernel templates).
#include <thrust/allocate_unique.h>
#include <thrust/device_delete.h>
#include <thrust/device_make_unique.h>
#include <thrust/device_malloc_allocator.h>
#include <thrust/device_new.h>
#include <thrust/device_new_allocator.h>
#include <thrust/mr/new.h>
#include <thrust/mr/universal_memory_resource.h>
#include <thrust/per_device_resource.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/sequence.h>
#include <thrust/sort.h>
#include <thrust/system/error_code.h>
#include <thrust/system/system_error.h>
#include <thrust/type_traits/integer_sequence.h>
#include <thrust/type_traits/is_contiguous_iterator.h>
#include <thrust/type_traits/is_execution_policy.h>
#include <thrust/type_traits/is_operator_less_or_greater_function_object.h>
#include <thrust/type_traits/is_operator_plus_function_object.h>
#include <thrust/type_traits/is_trivially_relocatable.h>
#include <thrust/type_traits/logical_metafunctions.h>
#include <thrust/type_traits/remove_cvref.h>
#include <thrust/type_traits/void_t.h>
#include <thrust/universal_vector.h>

#include <list>

#include "testing.h"

struct Foo {
  int set_me_upon_construction;
  Foo() : set_me_upon_construction(13) {}
};

void TestDeviceNewAndDelete() {
  // testing/device_delete.cu: the default constructor's effect is visible in device memory
  thrust::device_ptr<Foo> foo = thrust::device_new<Foo>();
  Foo back = *foo;
  ASSERT_EQUAL(back.set_me_upon_construction, 13);
  thrust::device_delete(foo);
  thrust::device_ptr<int> ints = thrust::device_new<int>(1000);
  ASSERT_EQUAL(thrust::reduce(ints, ints + 1000), 0);  // value-initialised
  thrust::device_ptr<void> raw(static_cast<void*>(ints.get()));
  thrust::device_ptr<int> again = thrust::device_new<int>(raw, 7, 1000);  // placement form with an exemplar
  ASSERT_TRUE(again == ints);
  ASSERT_EQUAL(thrust::reduce(ints, ints + 1000), 7000);
  thrust::device_delete(ints, 1000);
}
DECLARE_UNITTEST(TestDeviceNewAndDelete);

void TestAllocatorsOverDeviceMallocAndNew() {
  thrust::device_vector<int, thrust::device_malloc_allocator<int>> a(100, 3);
  ASSERT_EQUAL(thrust::reduce(a.begin(), a.end()), 300);
  thrust::device_vector<int, thrust::device_new_allocator<int>> b(100);
  thrust::sequence(b.begin(), b.end());
  ASSERT_EQUAL(thrust::reduce(b.begin(), b.end()), 4950);
  thrust::device_malloc_allocator<int> m1, m2;
  ASSERT_TRUE(m1 == m2);
}
DECLARE_UNITTEST(TestAllocatorsOverDeviceMallocAndNew);

void TestAllocateUnique() {
  {  // host memory
    thrust::mr::new_delete_resource res;
    thrust::mr::allocator<int, thrust::mr::new_delete_resource> alloc(&res);
    auto p = thrust::allocate_unique<int>(alloc, 42);
    ASSERT_EQUAL(*p, 42);
    auto arr = thrust::allocate_unique_n<int>(alloc, 10, 7);
    for (int i = 0; i < 10; i++) ASSERT_EQUAL(arr[i], 7);
    auto raw = thrust::uninitialized_allocate_unique_n<double>(alloc, 5);
    raw[4] = 1.5;
    ASSERT_EQUAL(raw[4], 1.5);
  }
  {  // device memory: the pointer is a device_ptr, the value is written through it
    auto p = thrust::allocate_unique<int>(thrust::device_allocator<int>(), 42);
    const int v = *p.get();
    ASSERT_EQUAL(v, 42);
    auto q = thrust::device_make_unique<Foo>();
    const Foo f = *q.get();
    ASSERT_EQUAL(f.set_me_upon_construction, 13);
    auto arr = thrust::allocate_unique_n<int>(thrust::device_allocator<int>(), 64, 5);
    ASSERT_EQUAL(thrust::reduce(arr.get(), arr.get() + 64), 320);
  }
}
DECLARE_UNITTEST(TestAllocateUnique);

void TestPerDeviceResource() {
  typedef thrust::system::cdna4::memory_resource MR;
  MR* a = thrust::get_per_device_resource<MR>(thrust::device);
  MR* b = thrust::get_per_device_resource<MR>(thrust::device);
  ASSERT_TRUE(a != nullptr && a == b);  // one instance per device
  thrust::per_device_allocator<int, MR, std::remove_const<decltype(thrust::device)>::type> alloc;
  thrust::device_ptr<int> p = alloc.allocate(10);
  ASSERT_TRUE(p.get() != nullptr);
  alloc.deallocate(p, 10);
}
DECLARE_UNITTEST(TestPerDeviceResource);

template <class Vector>
void exercise_universal(Vector& v) {
  const int n = (int)v.size();
  thrust::sequence(v.begin(), v.end());  // written by a kernel
  int* raw = thrust::raw_pointer_cast(v.data());
  long long host_sum = 0;
  for (int i = 0; i < n; i++) host_sum += raw[i];  // read by the host through the same address
  ASSERT_EQUAL(host_sum, (long long)n * (n - 1) / 2);
  for (int i = 0; i < n; i++) raw[i] = n - i;  // written by the host
  thrust::sort(v.begin(), v.end());            // sorted on the device
  ASSERT_EQUAL(raw[0], 1);
  ASSERT_EQUAL(raw[n - 1], n);
  thrust::inclusive_scan(v.begin(), v.end(), v.begin());
  ASSERT_EQUAL((long long)raw[n - 1], (long long)n * (n + 1) / 2);
}
void TestUniversalMemory() {
  thrust::universal_vector<int> v(10000);
  exercise_universal(v);
  thrust::device_vector<int, thrust::mr::stateless_resource_allocator<int, thrust::universal_host_pinned_memory_resource>> pinned(10000);
  exercise_universal(pinned);
  thrust::universal_ptr<int> p = v.data();
  ASSERT_EQUAL((int)*p, 1);
}
DECLARE_UNITTEST(TestUniversalMemory);

void TestTypeTraits() {
  static_assert(thrust::is_contiguous_iterator<int*>::value, "");
  static_assert(thrust::is_contiguous_iterator<thrust::device_ptr<int>>::value, "");
  static_assert(thrust::is_contiguous_iterator<std::vector<int>::iterator>::value, "");
  static_assert(thrust::is_contiguous_iterator<thrust::host_vector<int>::iterator>::value, "");
  static_assert(thrust::is_contiguous_iterator<thrust::device_vector<int>::iterator>::value, "");
  static_assert(!thrust::is_contiguous_iterator<std::list<int>::iterator>::value, "");
  static_assert(!thrust::is_contiguous_iterator<thrust::counting_iterator<int>>::value, "");
  static_assert(thrust::is_execution_policy<decltype(thrust::device)>::value, "");
  static_assert(thrust::is_execution_policy<decltype(thrust::host)>::value, "");
  static_assert(!thrust::is_execution_policy<int>::value, "");
  static_assert(thrust::is_operator_less_function_object<thrust::less<int>>::value, "");
  static_assert(thrust::is_operator_less_function_object<std::less<int>>::value, "");
  static_assert(thrust::is_operator_greater_function_object<thrust::greater<int>>::value, "");
  static_assert(thrust::is_operator_less_or_greater_function_object<std::greater<float>>::value, "");
  static_assert(!thrust::is_operator_less_or_greater_function_object<thrust::plus<int>>::value, "");
  static_assert(thrust::is_operator_plus_function_object<thrust::plus<int>>::value, "");
  static_assert(!thrust::is_operator_plus_function_object<thrust::minus<int>>::value, "");
  static_assert(thrust::is_trivially_relocatable<int>::value, "");
  static_assert(!thrust::is_trivially_relocatable<std::vector<int>>::value, "");
  static_assert(thrust::is_trivially_relocatable_to<int, const int>::value, "");
  static_assert(thrust::is_indirectly_trivially_relocatable_to<int*, thrust::device_ptr<int>>::value, "");
  static_assert(!thrust::is_indirectly_trivially_relocatable_to<int*, float*>::value, "");
  static_assert(thrust::conjunction<std::true_type, std::true_type>::value, "");
  static_assert(!thrust::conjunction<std::true_type, std::false_type>::value, "");
  static_assert(thrust::disjunction<std::false_type, std::true_type>::value, "");
  static_assert(thrust::negation<std::false_type>::value, "");
  static_assert(thrust::conjunction_value<true, true, true>::value && !thrust::disjunction_value<false, false>::value, "");
  static_assert(std::is_same<thrust::remove_cvref_t<const int&>, int>::value, "");
  static_assert(std::is_same<thrust::void_t<int, float>, void>::value, "");
  static_assert(std::is_same<thrust::make_reversed_integer_sequence<int, 4>, thrust::integer_sequence<int, 3, 2, 1, 0>>::value, "");
  static_assert(std::is_same<thrust::integer_sequence_push_front<int, 9, thrust::integer_sequence<int, 1, 2>>, thrust::integer_sequence<int, 9, 1, 2>>::value, "");
  static_assert(std::is_same<thrust::integer_sequence_push_back<int, 9, thrust::integer_sequence<int, 1, 2>>, thrust::integer_sequence<int, 1, 2, 9>>::value, "");
  static_assert(std::is_same<thrust::make_index_sequence<3>, thrust::index_sequence<0, 1, 2>>::value, "");
  // an error raised by the library carries the device category and is a thrust::system::system_error
  try {
    thrust::system::cdna4::detail::throw_on_error(1, "forced");
    ASSERT_TRUE(false);
  } catch (const thrust::system::system_error& e) {
    ASSERT_EQUAL(e.code().value(), 1);
    ASSERT_TRUE(e.code().category() == thrust::cdna4_category());
    thrust::system::error_code copy = e.code();
    ASSERT_TRUE(copy == e.code());
  }
}
DECLARE_UNITTEST(TestTypeTraits);

int main(int argc, char** argv) { return unittest::run_all(argc, argv); }

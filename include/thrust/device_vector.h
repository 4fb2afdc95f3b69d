// thrust::device_vector for trivially copyable element types (thrust/device_vector.h,
// thrust/detail/vector_base.h).  Storage comes from the library's cached allocator; value
// initialisation and fills run as typed fill kernels, transfers as async copies followed by
// a stream synchronise (thrust/system/cuda/detail/util.h:142-199), so a TU that uses
// device_vector needs no device compiler.
#pragma once
#include <algorithm>
#include <cstddef>
#include <initializer_list>
#include <memory>
#include <vector>

#include <thrust/device_allocator.h>
#include <thrust/device_ptr.h>
#include <thrust/host_vector.h>
#include <thrust/iterator/reverse_iterator.h>
#include <stdexcept>

namespace thrust {

template <class T, class Alloc>
class device_vector {
  // Elements travel between host and device, and within the device, as bytes — what the reference
  // does for the types it holds to be trivially relocatable (thrust/type_traits/is_trivially_relocatable.h).
  // A copy constructor or assignment operator written out by the user (a number-like struct with
  // __host__ __device__ members, say) is accepted and not run; a destructor with effects is refused.
  static_assert(detail::is_bytewise_movable<T>::value,
                "device_vector of the cdna4 system holds types that can be moved as bytes");

 public:
  typedef T value_type;
  typedef Alloc allocator_type;
  typedef std::size_t size_type;
  typedef device_ptr<T> iterator;
  typedef device_ptr<const T> const_iterator;
  typedef device_ptr<T> pointer;
  typedef device_reference<T> reference;
  typedef device_reference<const T> const_reference;
  typedef std::ptrdiff_t difference_type;
  typedef device_ptr<const T> const_pointer;
  typedef thrust::reverse_iterator<iterator> reverse_iterator;
  typedef thrust::reverse_iterator<const_iterator> const_reverse_iterator;

  device_vector() : p_(nullptr), n_(0), cap_(0), alloc_() {}
  explicit device_vector(const Alloc& alloc) : p_(nullptr), n_(0), cap_(0), alloc_(alloc) {}
  device_vector(size_type n, const T& v, const Alloc& alloc) : device_vector(alloc) { assign(n, v); }
  allocator_type get_allocator() const { return alloc_; }
  // (an allocator with a construct() of its own constructs the elements, thrust/detail/allocator_construct.h)
  explicit device_vector(size_type n) : device_vector() { resize(n); construct_default(0, n_); }
  device_vector(size_type n, const T& v) : device_vector() { assign(n, v); }
  device_vector(const device_vector& o) : device_vector(o.alloc_) { assign_device(o.p_, o.n_); }
  device_vector(device_vector&& o) noexcept : p_(o.p_), n_(o.n_), cap_(o.cap_), alloc_(o.alloc_) { o.p_ = nullptr; o.n_ = o.cap_ = 0; }
  // from a vector of either system, of this or a convertible element type
  template <class U, class A> device_vector(const std::vector<U, A>& h) : device_vector() { assign(h.begin(), h.end()); }
  template <class U, class A> device_vector(const host_vector<U, A>& h) : device_vector() { assign(h.begin(), h.end()); }
  template <class U, class A> device_vector(const device_vector<U, A>& d) : device_vector() { assign(d.begin(), d.end()); }
  device_vector(const device_vector& o, const Alloc& alloc) : device_vector(alloc) { assign_device(o.p_, o.n_); }
  device_vector(std::initializer_list<T> il, const Alloc& alloc) : device_vector(alloc) { assign_host(il.begin(), il.size()); }
  template <class It, class = typename std::iterator_traits<It>::iterator_category>
  device_vector(It first, It last, const Alloc& alloc) : device_vector(alloc) { assign(first, last); construct_copies(first); }
  device_vector(size_type n, const Alloc& alloc) : device_vector(alloc) { resize(n); construct_default(0, n_); }
  device_vector(std::initializer_list<T> il) : device_vector() { assign_host(il.begin(), il.size()); }
  template <class It, class = typename std::iterator_traits<It>::iterator_category>
  device_vector(It first, It last) : device_vector() { assign(first, last); construct_copies(first); }
  ~device_vector() { release(); }

  device_vector& operator=(const device_vector& o) { if (this != &o) assign_device(o.p_, o.n_); return *this; }
  // the source is left empty (testing/vector.cu:814-826)
  device_vector& operator=(device_vector&& o) noexcept {
    if (this != &o) {
      release();
      p_ = o.p_; n_ = o.n_; cap_ = o.cap_; alloc_ = o.alloc_;
      o.p_ = nullptr; o.n_ = o.cap_ = 0;
    }
    return *this;
  }
  template <class U, class A> device_vector& operator=(const std::vector<U, A>& h) { assign(h.begin(), h.end()); return *this; }
  template <class U, class A> device_vector& operator=(const host_vector<U, A>& h) { assign(h.begin(), h.end()); return *this; }
  template <class U, class A> device_vector& operator=(const device_vector<U, A>& d) { assign(d.begin(), d.end()); return *this; }
  device_vector& operator=(std::initializer_list<T> il) { assign_host(il.begin(), il.size()); return *this; }

  iterator begin() { return iterator(p_); }
  iterator end() { return iterator(p_ + n_); }
  const_iterator begin() const { return const_iterator(p_); }
  const_iterator end() const { return const_iterator(p_ + n_); }
  const_iterator cbegin() const { return begin(); }
  const_iterator cend() const { return end(); }
  reverse_iterator rbegin() { return reverse_iterator(end()); }
  reverse_iterator rend() { return reverse_iterator(begin()); }
  const_reverse_iterator rbegin() const { return const_reverse_iterator(end()); }
  const_reverse_iterator rend() const { return const_reverse_iterator(begin()); }
  const_reverse_iterator crbegin() const { return rbegin(); }
  const_reverse_iterator crend() const { return rend(); }
  pointer data() { return pointer(p_); }
  device_ptr<const T> data() const { return device_ptr<const T>(p_); }
  size_type size() const { return n_; }
  size_type capacity() const { return cap_; }
  bool empty() const { return n_ == 0; }
  reference operator[](size_type i) { return reference(p_ + i); }
  const_reference operator[](size_type i) const { return const_reference(p_ + i); }
  // checked access (thrust/detail/vector_base.h: at() throws std::out_of_range)
  reference at(size_type i) { if (i >= n_) throw std::out_of_range("thrust::device_vector::at"); return (*this)[i]; }
  const_reference at(size_type i) const { if (i >= n_) throw std::out_of_range("thrust::device_vector::at"); return (*this)[i]; }
  size_type max_size() const { return static_cast<size_type>(-1) / sizeof(T); }
  reference front() { return (*this)[0]; }
  reference back() { return (*this)[n_ - 1]; }
  const_reference front() const { return (*this)[0]; }
  const_reference back() const { return (*this)[n_ - 1]; }

  void clear() { n_ = 0; }
  void swap(device_vector& o) noexcept { std::swap(p_, o.p_); std::swap(n_, o.n_); std::swap(cap_, o.cap_); std::swap(alloc_, o.alloc_); }
  void reserve(size_type c) { if (c > cap_) regrow(c); }
  void resize(size_type n) { resize(n, T()); }
  void resize(size_type n, const T& v) {
    if (n > cap_) regrow(n);
    if (n > n_) fill_raw(p_ + n_, n - n_, v);
    n_ = n;
  }
  void assign(size_type n, const T& v) { n_ = 0; if (n > cap_) regrow(n); fill_raw(p_, n, v); n_ = n; }
  template <class It, class = typename std::iterator_traits<It>::iterator_category>
  void assign(It first, It last) {
    assign_range(first, last, std::integral_constant<bool, std::is_same<It, iterator>::value || std::is_same<It, const_iterator>::value>());
  }
  void pop_back() { --n_; }
  void shrink_to_fit() {
    if (n_ == cap_) return;
    device_vector tight(alloc_);
    tight.assign_device(p_, n_);
    swap(tight);
  }
  // erase [first, last): the tail moves down (the usual partner of remove_if / unique)
  iterator erase(iterator first, iterator last) {
    const size_type at = (size_type)(first - begin()), count = (size_type)(last - first), tail = n_ - at - count;
    if (count == 0) return first;
    if (tail) {
      // the ranges may overlap: go through a temporary
      device_vector moved(alloc_);
      moved.assign_device(p_ + at + count, tail);
      check(thrust_cdna4_memcpy_dtod(p_ + at, moved.p_, tail * sizeof(T), nullptr), "device_vector: erase");
      sync();
    }
    n_ -= count;
    return begin() + at;
  }
  iterator erase(iterator pos) { return erase(pos, pos + 1); }
  // insert [first, last) (a device or a host range) before pos
  template <class It, class = typename std::iterator_traits<It>::iterator_category>
  iterator insert(iterator pos, It first, It last) {
    const size_type at = (size_type)(pos - begin());
    device_vector added(alloc_);
    added.assign(first, last);
    device_vector tail(alloc_);
    tail.assign_device(p_ + at, n_ - at);
    const size_type total = n_ + added.n_;
    if (total > cap_) regrow(std::max(total, 2 * cap_));
    if (added.n_) check(thrust_cdna4_memcpy_dtod(p_ + at, added.p_, added.n_ * sizeof(T), nullptr), "device_vector: insert");
    if (tail.n_) check(thrust_cdna4_memcpy_dtod(p_ + at + added.n_, tail.p_, tail.n_ * sizeof(T), nullptr), "device_vector: insert");
    sync();
    n_ = total;
    return begin() + at;
  }
  iterator insert(iterator pos, const T& v) { return insert(pos, (size_type)1, v); }
  iterator insert(iterator pos, size_type n, const T& v) {
    const size_type at = (size_type)(pos - begin());
    device_vector added(n, v, alloc_);
    return insert(begin() + at, added.begin(), added.end());
  }
  void push_back(const T& v) {
    if (n_ == cap_) regrow(cap_ ? 2 * cap_ : 16);
    fill_raw(p_ + n_, 1, v);
    ++n_;
  }


 private:
  // the allocator's own construct(), where it has one: defined after the class, in allocator_construct.h
  void construct_default(size_type at, size_type count);
  template <class U> void construct_copies(device_ptr<U> from);
  template <class It> void construct_copies(It) {}  // a range outside device memory: the bytes are the copy
  static void check(int rc, const char* what) { system::cdna4::detail::throw_on_error(rc, what); }
  static void sync() { check(thrust_cdna4_stream_synchronize(nullptr), "device_vector: synchronize"); }
  void release() { if (p_) alloc_.deallocate(typename Alloc::pointer(p_), cap_); p_ = nullptr; n_ = cap_ = 0; }
  void regrow(size_type c) {
    T* q = alloc_.allocate(c).get();
    if (n_) { check(thrust_cdna4_memcpy_dtod(q, p_, n_ * sizeof(T), nullptr), "device_vector: copy"); sync(); }
    if (p_) alloc_.deallocate(typename Alloc::pointer(p_), cap_);
    p_ = q;
    cap_ = c;
  }
  static void fill_raw(T* dst, size_type n, const T& v) {
    if (!n) return;
    if (sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8) {
      check(thrust_cdna4_fill(dst, &v, (int)sizeof(T), (int64_t)n, nullptr), "device_vector: fill");
    } else {  // other element sizes (user structs): staged through the host
      const host_vector<T> tmp(n, v);
      check(thrust_cdna4_memcpy_htod(dst, tmp.data(), n * sizeof(T), nullptr), "device_vector: fill");
    }
    sync();
  }
  void assign_host(const T* h, size_type n) {
    n_ = 0;
    if (n > cap_) regrow(n);
    if (n) { check(thrust_cdna4_memcpy_htod(p_, h, n * sizeof(T), nullptr), "device_vector: copy from host"); sync(); }
    n_ = n;
  }
  void assign_device(const T* d, size_type n) {
    n_ = 0;
    if (n > cap_) regrow(n);
    if (n) { check(thrust_cdna4_memcpy_dtod(p_, d, n * sizeof(T), nullptr), "device_vector: copy"); sync(); }
    n_ = n;
  }
  template <class It> void assign_range(It first, It last, std::true_type) { assign_device(first.get(), (size_type)(last - first)); }
  // any other range, in host or in device memory, of this or a convertible element type: through
  // a host_vector, which reads a device range by the device system's copy
  template <class It> void assign_range(It first, It last, std::false_type) {
    const host_vector<T> tmp(first, last);
    assign_host(tmp.data(), tmp.size());
  }

  T* p_;
  size_type n_, cap_;
  Alloc alloc_;
};

// equality across the two vector kinds, element types and allocators (thrust/detail/vector_base.h:588-622)
template <class T1, class A1, class T2, class A2>
bool operator==(const device_vector<T1, A1>& a, const device_vector<T2, A2>& b) { return host_vector<T1>(a) == host_vector<T2>(b); }
template <class T1, class A1, class T2, class A2>
bool operator==(const device_vector<T1, A1>& a, const host_vector<T2, A2>& b) { return host_vector<T1>(a) == b; }
template <class T1, class A1, class T2, class A2>
bool operator==(const host_vector<T1, A1>& a, const device_vector<T2, A2>& b) { return a == host_vector<T2>(b); }
template <class T1, class A1, class T2, class A2>
bool operator==(const device_vector<T1, A1>& a, const std::vector<T2, A2>& b) { return host_vector<T1>(a) == b; }
template <class T1, class A1, class T2, class A2>
bool operator==(const std::vector<T1, A1>& a, const device_vector<T2, A2>& b) { return a == host_vector<T2>(b); }
template <class T1, class A1, class T2, class A2>
bool operator!=(const device_vector<T1, A1>& a, const device_vector<T2, A2>& b) { return !(a == b); }
template <class T1, class A1, class T2, class A2>
bool operator!=(const device_vector<T1, A1>& a, const host_vector<T2, A2>& b) { return !(a == b); }
template <class T1, class A1, class T2, class A2>
bool operator!=(const host_vector<T1, A1>& a, const device_vector<T2, A2>& b) { return !(a == b); }
template <class T1, class A1, class T2, class A2>
bool operator!=(const device_vector<T1, A1>& a, const std::vector<T2, A2>& b) { return !(a == b); }
template <class T1, class A1, class T2, class A2>
bool operator!=(const std::vector<T1, A1>& a, const device_vector<T2, A2>& b) { return !(a == b); }
template <class T, class A> void swap(device_vector<T, A>& a, device_vector<T, A>& b) noexcept { a.swap(b); }

}  // namespace thrust

namespace thrust {
namespace detail {
// thrust::detail::vector_base<T, Alloc> (thrust/detail/vector_base.h) as generic code names it when it
// derives a vector type from another vector's allocator (testing/binary_search_vector.cu:16-23): the
// vector of the system the allocator's pointer belongs to.
template <class T, class Alloc, class Pointer = typename std::allocator_traits<Alloc>::pointer>
struct vector_base_of { typedef host_vector<T, Alloc> type; };
template <class T, class Alloc, class U>
struct vector_base_of<T, Alloc, device_ptr<U>> { typedef device_vector<T, Alloc> type; };
template <class T, class Alloc> using vector_base = typename vector_base_of<T, Alloc>::type;
}  // namespace detail
}  // namespace thrust

#include <thrust/detail/vector_common.h>
#include <thrust/detail/allocator_construct.h>
namespace thrust {
template <class T, class Alloc>
void device_vector<T, Alloc>::construct_default(size_type at, size_type count) { detail::allocator_default_construct(alloc_, p_ + at, count); }
template <class T, class Alloc>
template <class U>
void device_vector<T, Alloc>::construct_copies(device_ptr<U> from) { detail::allocator_copy_construct(alloc_, p_, static_cast<const U*>(from.get()), n_); }
}  // namespace thrust

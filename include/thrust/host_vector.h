// thrust::host_vector (thrust/host_vector.h:45-520; thrust/detail/vector_base.h:40-630): a dynamic
// array in host memory with the interface of std::vector — elements of every type are stored one
// object each (bool too, unlike std::vector<bool>), and the iterators are thrust's own class, so
// that unqualified algorithm calls on them resolve to thrust's algorithms.
#pragma once
#include <algorithm>
#include <cstddef>
#include <initializer_list>
#include <iterator>
#include <limits>
#include <memory>
#include <stdexcept>
#include <type_traits>
#include <utility>
#include <vector>
#include <thrust/device_ptr.h>
#include <thrust/iterator/detail/normal_iterator.h>
#include <thrust/copy.h>
namespace thrust {
template <class T> class device_allocator;
template <class T, class Alloc = device_allocator<T>> class device_vector;

template <class T, class Alloc = std::allocator<T>>
class host_vector {
  typedef std::allocator_traits<Alloc> traits;
  template <class It> using if_iterator = typename std::enable_if<system::cdna4::detail::is_iterator_type<It>::value, int>::type;
  // a range in device memory (not a counting or constant iterator, which host code may read itself)
  template <class It> struct walks_device_memory
      : std::integral_constant<bool, system::cdna4::detail::is_device_iterator<It>::value &&
                                         !system::cdna4::detail::is_any_system_iterator<It>::value> {};

 public:
  typedef T value_type;
  typedef Alloc allocator_type;
  typedef T* pointer;
  typedef const T* const_pointer;
  typedef T& reference;
  typedef const T& const_reference;
  typedef std::size_t size_type;
  typedef std::ptrdiff_t difference_type;
  typedef detail::normal_iterator<T*> iterator;
  typedef detail::normal_iterator<const T*> const_iterator;
  typedef std::reverse_iterator<iterator> reverse_iterator;
  typedef std::reverse_iterator<const_iterator> const_reverse_iterator;

  host_vector() : p_(nullptr), n_(0), cap_(0), alloc_() {}
  explicit host_vector(const Alloc& alloc) : p_(nullptr), n_(0), cap_(0), alloc_(alloc) {}
  explicit host_vector(size_type n) : host_vector() { resize(n); }
  host_vector(size_type n, const Alloc& alloc) : host_vector(alloc) { resize(n); }
  host_vector(size_type n, const T& v) : host_vector() { assign(n, v); }
  host_vector(size_type n, const T& v, const Alloc& alloc) : host_vector(alloc) { assign(n, v); }
  host_vector(const host_vector& o) : host_vector(traits::select_on_container_copy_construction(o.alloc_)) { assign_range(o.p_, o.p_ + o.n_); }
  host_vector(const host_vector& o, const Alloc& alloc) : host_vector(alloc) { assign_range(o.p_, o.p_ + o.n_); }
  host_vector(host_vector&& o) noexcept : p_(o.p_), n_(o.n_), cap_(o.cap_), alloc_(std::move(o.alloc_)) { o.p_ = nullptr; o.n_ = o.cap_ = 0; }
  host_vector(std::initializer_list<T> il) : host_vector() { assign_range(il.begin(), il.end()); }
  host_vector(std::initializer_list<T> il, const Alloc& alloc) : host_vector(alloc) { assign_range(il.begin(), il.end()); }
  template <class U, class A2> host_vector(const host_vector<U, A2>& o) : host_vector() { assign_range(o.begin(), o.end()); }
  template <class U, class A2> host_vector(const std::vector<U, A2>& o) : host_vector() { assign_range(o.begin(), o.end()); }
  template <class U, class A2> host_vector(const device_vector<U, A2>& d) : host_vector() { assign(d.begin(), d.end()); }
  template <class It, if_iterator<It> = 0> host_vector(It first, It last) : host_vector() { assign(first, last); }
  template <class It, if_iterator<It> = 0> host_vector(It first, It last, const Alloc& alloc) : host_vector(alloc) { assign(first, last); }
  ~host_vector() { release(); }

  host_vector& operator=(const host_vector& o) { if (this != &o) assign_range(o.p_, o.p_ + o.n_); return *this; }
  // the source is left empty (thrust/detail/vector_base.inl: move assignment; testing/vector.cu:814-826)
  host_vector& operator=(host_vector&& o) noexcept {
    if (this != &o) {
      release();
      p_ = o.p_; n_ = o.n_; cap_ = o.cap_; alloc_ = std::move(o.alloc_);
      o.p_ = nullptr; o.n_ = o.cap_ = 0;
    }
    return *this;
  }
  host_vector& operator=(std::initializer_list<T> il) { assign_range(il.begin(), il.end()); return *this; }
  template <class U, class A2> host_vector& operator=(const host_vector<U, A2>& o) { assign_range(o.begin(), o.end()); return *this; }
  template <class U, class A2> host_vector& operator=(const std::vector<U, A2>& o) { assign_range(o.begin(), o.end()); return *this; }
  template <class U, class A2> host_vector& operator=(const device_vector<U, A2>& d) { assign(d.begin(), d.end()); return *this; }

  size_type size() const { return n_; }
  size_type max_size() const { return std::numeric_limits<difference_type>::max() / sizeof(T); }
  size_type capacity() const { return cap_; }
  bool empty() const { return n_ == 0; }
  void reserve(size_type n) { if (n > cap_) reallocate(n); }
  void shrink_to_fit() { if (cap_ > n_) reallocate(n_); }
  void resize(size_type n) {
    if (n < n_) destroy_from(n);
    else if (n > n_) { grow_to(n); for (; n_ < n; ++n_) traits::construct(alloc_, p_ + n_); }
  }
  void resize(size_type n, const T& v) {
    if (n < n_) destroy_from(n);
    else if (n > n_) { T copy(v); grow_to(n); for (; n_ < n; ++n_) traits::construct(alloc_, p_ + n_, copy); }
  }
  void clear() { destroy_from(0); }

  reference operator[](size_type i) { return p_[i]; }
  const_reference operator[](size_type i) const { return p_[i]; }
  reference at(size_type i) { if (i >= n_) throw std::out_of_range("host_vector::at"); return p_[i]; }
  const_reference at(size_type i) const { if (i >= n_) throw std::out_of_range("host_vector::at"); return p_[i]; }
  reference front() { return p_[0]; }
  const_reference front() const { return p_[0]; }
  reference back() { return p_[n_ - 1]; }
  const_reference back() const { return p_[n_ - 1]; }
  pointer data() { return p_; }
  const_pointer data() const { return p_; }

  iterator begin() { return iterator(p_); }
  const_iterator begin() const { return const_iterator(p_); }
  const_iterator cbegin() const { return const_iterator(p_); }
  iterator end() { return iterator(p_ + n_); }
  const_iterator end() const { return const_iterator(p_ + n_); }
  const_iterator cend() const { return const_iterator(p_ + n_); }
  reverse_iterator rbegin() { return reverse_iterator(end()); }
  const_reverse_iterator rbegin() const { return const_reverse_iterator(end()); }
  const_reverse_iterator crbegin() const { return const_reverse_iterator(end()); }
  reverse_iterator rend() { return reverse_iterator(begin()); }
  const_reverse_iterator rend() const { return const_reverse_iterator(begin()); }
  const_reverse_iterator crend() const { return const_reverse_iterator(begin()); }

  void push_back(const T& v) {
    if (n_ == cap_) { T copy(v); grow_to(n_ + 1); traits::construct(alloc_, p_ + n_, std::move(copy)); }
    else traits::construct(alloc_, p_ + n_, v);
    ++n_;
  }
  void push_back(T&& v) { grow_to(n_ + 1); traits::construct(alloc_, p_ + n_, std::move(v)); ++n_; }
  template <class... Args> reference emplace_back(Args&&... args) {
    grow_to(n_ + 1); traits::construct(alloc_, p_ + n_, std::forward<Args>(args)...); return p_[n_++];
  }
  void pop_back() { destroy_from(n_ - 1); }
  void swap(host_vector& o) noexcept { std::swap(p_, o.p_); std::swap(n_, o.n_); std::swap(cap_, o.cap_); std::swap(alloc_, o.alloc_); }

  iterator erase(const_iterator pos) { return erase(pos, pos + 1); }
  iterator erase(const_iterator first, const_iterator last) {
    const size_type i = (size_type)(first.base() - p_), j = (size_type)(last.base() - p_);
    if (j > i) { std::move(p_ + j, p_ + n_, p_ + i); destroy_from(n_ - (j - i)); }
    return iterator(p_ + i);
  }
  iterator insert(const_iterator pos, const T& v) {
    const size_type i = (size_type)(pos.base() - p_);
    T copy(v);
    open_gap(i, 1);
    p_[i] = std::move(copy);
    return iterator(p_ + i);
  }
  iterator insert(const_iterator pos, size_type n, const T& v) {
    const size_type i = (size_type)(pos.base() - p_);
    T copy(v);
    open_gap(i, n);
    std::fill(p_ + i, p_ + i + n, copy);
    return iterator(p_ + i);
  }
  template <class It, if_iterator<It> = 0>
  iterator insert(const_iterator pos, It first, It last) {
    const size_type i = (size_type)(pos.base() - p_);
    host_vector staged(first, last);  // the source may be this vector, or device memory
    open_gap(i, staged.n_);
    std::move(staged.p_, staged.p_ + staged.n_, p_ + i);
    return iterator(p_ + i);
  }
  iterator insert(const_iterator pos, std::initializer_list<T> il) { return insert(pos, il.begin(), il.end()); }

  void assign(size_type n, const T& v) { T copy(v); clear(); grow_to(n); for (; n_ < n; ++n_) traits::construct(alloc_, p_ + n_, copy); }
  void assign(std::initializer_list<T> il) { assign_range(il.begin(), il.end()); }
  // From a range in device memory: one copy when it is contiguous and of this element type,
  // otherwise through the device system's copy; from any other range element by element.
  template <class It, if_iterator<It> = 0>
  void assign(It first, It last) { assign_dispatch(first, last, walks_device_memory<It>()); }

  allocator_type get_allocator() const { return alloc_; }

 private:
  template <class It> void assign_dispatch(It first, It last, std::false_type) { assign_range(first, last); }
  template <class It> void assign_dispatch(It first, It last, std::true_type) {
    typedef typename std::iterator_traits<It>::value_type U;
    const size_type n = (size_type)(last - first);
    host_vector<typename std::remove_const<U>::type> staged;
    staged.resize(n);
    thrust::copy(first, last, staged.data());
    assign_range(staged.begin(), staged.end());
  }
  template <class U> void assign_dispatch(device_ptr<U> first, device_ptr<U> last, std::true_type) {
    typedef typename std::remove_const<U>::type V;
    const size_type n = (size_type)(last - first);
    if (std::is_same<V, T>::value) {
      resize(n);
      system::cdna4::detail::copy_bytes(p_, first.get(), n * sizeof(T), 1);
    } else {  // another element type: a host copy of the source, converted element by element
      host_vector<V> staged(first, last);
      assign_range(staged.begin(), staged.end());
    }
  }
  template <class It> void assign_range(It first, It last) { assign_range(first, last, typename std::iterator_traits<It>::iterator_category()); }
  template <class It> void assign_range(It first, It last, std::input_iterator_tag) {
    clear();
    for (; first != last; ++first) emplace_back(*first);
  }
  template <class It> void assign_range(It first, It last, std::forward_iterator_tag) {
    const size_type n = (size_type)std::distance(first, last);
    if (n > cap_) {  // the range cannot lie inside this vector then, unless it is the whole of it
      host_vector fresh(alloc_);
      fresh.grow_exactly(n);
      for (; first != last; ++first, ++fresh.n_) traits::construct(fresh.alloc_, fresh.p_ + fresh.n_, static_cast<T>(*first));
      swap(fresh);
      return;
    }
    size_type i = 0;
    for (; i < n_ && first != last; ++i, ++first) p_[i] = static_cast<T>(*first);
    if (first == last) destroy_from(i);
    else for (; first != last; ++first, ++n_) traits::construct(alloc_, p_ + n_, static_cast<T>(*first));
  }
  void destroy_from(size_type keep) { while (n_ > keep) traits::destroy(alloc_, p_ + --n_); }
  void release() {
    clear();
    if (p_) traits::deallocate(alloc_, typename traits::pointer(p_), cap_);
    p_ = nullptr; cap_ = 0;
  }
  static T* raw(T* p) { return p; }
  template <class P> static T* raw(P p) { return p.get(); }
  void reallocate(size_type cap) {
    T* fresh = cap ? raw(traits::allocate(alloc_, cap)) : nullptr;
    for (size_type i = 0; i < n_; ++i) { traits::construct(alloc_, fresh + i, std::move_if_noexcept(p_[i])); traits::destroy(alloc_, p_ + i); }
    if (p_) traits::deallocate(alloc_, typename traits::pointer(p_), cap_);
    p_ = fresh; cap_ = cap;
  }
  void grow_exactly(size_type n) { if (n > cap_) reallocate(n); }
  void grow_to(size_type n) { if (n > cap_) reallocate(std::max(n, 2 * cap_)); }
  // makes room for n elements at index i; the new slots hold moved-from or default values
  void open_gap(size_type i, size_type n) {
    if (!n) return;
    const size_type old = n_;
    grow_to(old + n);
    for (; n_ < old + n; ++n_) traits::construct(alloc_, p_ + n_);
    std::move_backward(p_ + i, p_ + old, p_ + old + n);
  }

  T* p_;
  size_type n_, cap_;
  Alloc alloc_;
  template <class, class> friend class host_vector;
};

template <class T, class A> void swap(host_vector<T, A>& a, host_vector<T, A>& b) noexcept { a.swap(b); }
template <class T1, class A1, class T2, class A2>
bool operator==(const host_vector<T1, A1>& a, const host_vector<T2, A2>& b) { return a.size() == b.size() && std::equal(a.begin(), a.end(), b.begin()); }
template <class T1, class A1, class T2, class A2>
bool operator==(const host_vector<T1, A1>& a, const std::vector<T2, A2>& b) { return a.size() == b.size() && std::equal(a.begin(), a.end(), b.begin()); }
template <class T1, class A1, class T2, class A2>
bool operator==(const std::vector<T1, A1>& a, const host_vector<T2, A2>& b) { return b == a; }
template <class T1, class A1, class T2, class A2>
bool operator!=(const host_vector<T1, A1>& a, const host_vector<T2, A2>& b) { return !(a == b); }
template <class T1, class A1, class T2, class A2>
bool operator!=(const host_vector<T1, A1>& a, const std::vector<T2, A2>& b) { return !(a == b); }
template <class T1, class A1, class T2, class A2>
bool operator!=(const std::vector<T1, A1>& a, const host_vector<T2, A2>& b) { return !(b == a); }
}  // namespace thrust
#include <thrust/detail/vector_common.h>

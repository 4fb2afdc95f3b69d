// thrust::optional<T> (thrust/optional.h): a value that may be absent, usable in device code.
// The interface of std::optional — nullopt, in_place, has_value / value / value_or / operator* /
// operator->, reset, emplace, swap, the comparisons, make_optional, bad_optional_access — plus
// the monadic helpers of the reference's implementation: map, and_then, or_else, map_or,
// disjunction, conjunction, take.
#pragma once
#include <exception>
#include <new>
#include <type_traits>
#include <utility>
#include <thrust/detail/hd.h>

namespace thrust {

// the value type of an optional that only says whether it is engaged (thrust/optional.h:171)
class monostate {};
THRUST_CDNA4_HD constexpr bool operator==(monostate, monostate) noexcept { return true; }
THRUST_CDNA4_HD constexpr bool operator!=(monostate, monostate) noexcept { return false; }
THRUST_CDNA4_HD constexpr bool operator<(monostate, monostate) noexcept { return false; }
struct nullopt_t {
  struct do_not_use {};
  THRUST_CDNA4_HD constexpr explicit nullopt_t(do_not_use, do_not_use) noexcept {}
};
static constexpr nullopt_t nullopt{nullopt_t::do_not_use{}, nullopt_t::do_not_use{}};
struct in_place_t {
  explicit in_place_t() = default;
};
static constexpr in_place_t in_place{};

class bad_optional_access : public std::exception {
 public:
  bad_optional_access() = default;
  const char* what() const noexcept override { return "Optional has no value"; }
};

namespace detail {
// Storage and special member functions.  For trivially copyable, trivially destructible T they
// are all defaulted, so optional<T> is trivially copyable too and may live in device storage.
template <class T, bool Trivial = std::is_trivially_copyable<T>::value && std::is_trivially_destructible<T>::value>
struct optional_base {
  struct empty {};
  union {
    empty dummy_;
    T value_;
  };
  bool has_;
  THRUST_CDNA4_HD constexpr optional_base() noexcept : dummy_(), has_(false) {}
  template <class... Args> THRUST_CDNA4_HD constexpr optional_base(in_place_t, Args&&... args) : value_(std::forward<Args>(args)...), has_(true) {}
  template <class... Args> THRUST_CDNA4_HD void construct(Args&&... args) {
    ::new (static_cast<void*>(&value_)) T(std::forward<Args>(args)...);
    has_ = true;
  }
  THRUST_CDNA4_HD void reset() noexcept { has_ = false; }
};
template <class T>
struct optional_base<T, false> {
  struct empty {};
  union {
    empty dummy_;
    T value_;
  };
  bool has_;
  THRUST_CDNA4_HD constexpr optional_base() noexcept : dummy_(), has_(false) {}
  template <class... Args> THRUST_CDNA4_HD constexpr optional_base(in_place_t, Args&&... args) : value_(std::forward<Args>(args)...), has_(true) {}
  THRUST_CDNA4_HD optional_base(const optional_base& o) : dummy_(), has_(false) {
    if (o.has_) construct(o.value_);
  }
  THRUST_CDNA4_HD optional_base(optional_base&& o) noexcept(std::is_nothrow_move_constructible<T>::value) : dummy_(), has_(false) {
    if (o.has_) construct(std::move(o.value_));
  }
  THRUST_CDNA4_HD optional_base& operator=(const optional_base& o) {
    if (this == &o) return *this;
    if (has_ && o.has_) value_ = o.value_;
    else if (o.has_) construct(o.value_);
    else reset();
    return *this;
  }
  THRUST_CDNA4_HD optional_base& operator=(optional_base&& o) noexcept(std::is_nothrow_move_assignable<T>::value && std::is_nothrow_move_constructible<T>::value) {
    if (has_ && o.has_) value_ = std::move(o.value_);
    else if (o.has_) construct(std::move(o.value_));
    else reset();
    return *this;
  }
  THRUST_CDNA4_HD ~optional_base() { reset(); }
  template <class... Args> THRUST_CDNA4_HD void construct(Args&&... args) {
    ::new (static_cast<void*>(&value_)) T(std::forward<Args>(args)...);
    has_ = true;
  }
  THRUST_CDNA4_HD void reset() noexcept {
    if (has_) {
      value_.~T();
      has_ = false;
    }
  }
};
}  // namespace detail

template <class T>
class optional : private detail::optional_base<T> {
  typedef detail::optional_base<T> base;
  using base::construct;
  using base::has_;
  using base::value_;
  static_assert(!std::is_reference<T>::value && !std::is_same<typename std::decay<T>::type, nullopt_t>::value &&
                    !std::is_same<typename std::decay<T>::type, in_place_t>::value,
                "thrust::optional of a reference, nullopt_t or in_place_t is ill-formed");

 public:
  typedef T value_type;

  constexpr optional() noexcept = default;
  THRUST_CDNA4_HD constexpr optional(nullopt_t) noexcept : base() {}
  optional(const optional&) = default;
  optional(optional&&) = default;
  optional& operator=(const optional&) = default;
  optional& operator=(optional&&) = default;
  ~optional() = default;
  template <class... Args>
  THRUST_CDNA4_HD constexpr explicit optional(in_place_t, Args&&... args) : base(in_place, std::forward<Args>(args)...) {}
  template <class U = T, typename std::enable_if<std::is_constructible<T, U&&>::value && !std::is_same<typename std::decay<U>::type, optional>::value &&
                                                     !std::is_same<typename std::decay<U>::type, in_place_t>::value, int>::type = 0>
  THRUST_CDNA4_HD constexpr optional(U&& u) : base(in_place, std::forward<U>(u)) {}
  template <class U, typename std::enable_if<std::is_constructible<T, const U&>::value && !std::is_same<U, T>::value, int>::type = 0>
  THRUST_CDNA4_HD optional(const optional<U>& o) : base() {
    if (o.has_value()) construct(*o);
  }

  THRUST_CDNA4_HD optional& operator=(nullopt_t) noexcept { reset(); return *this; }
  template <class U = T, typename std::enable_if<std::is_constructible<T, U&&>::value && !std::is_same<typename std::decay<U>::type, optional>::value, int>::type = 0>
  THRUST_CDNA4_HD optional& operator=(U&& u) {
    if (has_) value_ = std::forward<U>(u);
    else construct(std::forward<U>(u));
    return *this;
  }
  template <class... Args>
  THRUST_CDNA4_HD T& emplace(Args&&... args) {
    reset();
    construct(std::forward<Args>(args)...);
    return value_;
  }
  THRUST_CDNA4_HD void reset() noexcept { base::reset(); }
  THRUST_CDNA4_HD void swap(optional& o) {
    if (has_ && o.has_) {
      T t(std::move(value_));
      value_ = std::move(o.value_);
      o.value_ = std::move(t);
    } else if (has_) {
      o.construct(std::move(value_));
      reset();
    } else if (o.has_) {
      construct(std::move(o.value_));
      o.reset();
    }
  }

  THRUST_CDNA4_HD constexpr bool has_value() const noexcept { return has_; }
  THRUST_CDNA4_HD constexpr explicit operator bool() const noexcept { return has_; }
  THRUST_CDNA4_HD T& operator*() & { return value_; }
  THRUST_CDNA4_HD constexpr const T& operator*() const& { return value_; }
  THRUST_CDNA4_HD T&& operator*() && { return std::move(value_); }
  THRUST_CDNA4_HD T* operator->() { return &value_; }
  THRUST_CDNA4_HD constexpr const T* operator->() const { return &value_; }
  // value(): throws bad_optional_access on the host when empty (device code must check first)
  T& value() & {
    if (!has_) throw bad_optional_access();
    return value_;
  }
  const T& value() const& {
    if (!has_) throw bad_optional_access();
    return value_;
  }
  T&& value() && {
    if (!has_) throw bad_optional_access();
    return std::move(value_);
  }
  template <class U> THRUST_CDNA4_HD constexpr T value_or(U&& u) const& { return has_ ? value_ : static_cast<T>(std::forward<U>(u)); }
  template <class U> THRUST_CDNA4_HD T value_or(U&& u) && { return has_ ? std::move(value_) : static_cast<T>(std::forward<U>(u)); }

  // ---- monadic helpers: the result of f applied to the value, or an empty optional
  template <class F> THRUST_CDNA4_HD auto map(F&& f) const& -> optional<typename std::decay<decltype(f(std::declval<const T&>()))>::type> {
    typedef optional<typename std::decay<decltype(f(std::declval<const T&>()))>::type> R;
    return has_ ? R(f(value_)) : R(nullopt);
  }
  template <class F> THRUST_CDNA4_HD auto transform(F&& f) const& -> decltype(this->map(std::forward<F>(f))) { return map(std::forward<F>(f)); }
  // f returns an optional itself
  template <class F> THRUST_CDNA4_HD auto and_then(F&& f) const& -> typename std::decay<decltype(f(std::declval<const T&>()))>::type {
    typedef typename std::decay<decltype(f(std::declval<const T&>()))>::type R;
    return has_ ? f(value_) : R(nullopt);
  }
  // this when it holds a value, else what f returns
  template <class F> THRUST_CDNA4_HD optional or_else(F&& f) const& { return has_ ? *this : optional(f()); }
  template <class F, class U> THRUST_CDNA4_HD U map_or(F&& f, U&& u) const& { return has_ ? static_cast<U>(f(value_)) : std::forward<U>(u); }
  template <class U> THRUST_CDNA4_HD constexpr optional<typename std::decay<U>::type> conjunction(U&& u) const {
    typedef optional<typename std::decay<U>::type> R;
    return has_ ? R(std::forward<U>(u)) : R(nullopt);
  }
  THRUST_CDNA4_HD constexpr optional disjunction(const optional& rhs) const { return has_ ? *this : rhs; }
  THRUST_CDNA4_HD optional take() {
    optional ret = std::move(*this);
    reset();
    return ret;
  }

};

// ---- comparisons: an empty optional orders before any value
template <class T, class U> THRUST_CDNA4_HD constexpr bool operator==(const optional<T>& a, const optional<U>& b) {
  return a.has_value() == b.has_value() && (!a.has_value() || *a == *b);
}
template <class T, class U> THRUST_CDNA4_HD constexpr bool operator!=(const optional<T>& a, const optional<U>& b) { return !(a == b); }
template <class T, class U> THRUST_CDNA4_HD constexpr bool operator<(const optional<T>& a, const optional<U>& b) {
  return b.has_value() && (!a.has_value() || *a < *b);
}
template <class T, class U> THRUST_CDNA4_HD constexpr bool operator>(const optional<T>& a, const optional<U>& b) { return b < a; }
template <class T, class U> THRUST_CDNA4_HD constexpr bool operator<=(const optional<T>& a, const optional<U>& b) { return !(b < a); }
template <class T, class U> THRUST_CDNA4_HD constexpr bool operator>=(const optional<T>& a, const optional<U>& b) { return !(a < b); }
template <class T> THRUST_CDNA4_HD constexpr bool operator==(const optional<T>& a, nullopt_t) noexcept { return !a.has_value(); }
template <class T> THRUST_CDNA4_HD constexpr bool operator==(nullopt_t, const optional<T>& a) noexcept { return !a.has_value(); }
template <class T> THRUST_CDNA4_HD constexpr bool operator!=(const optional<T>& a, nullopt_t) noexcept { return a.has_value(); }
template <class T> THRUST_CDNA4_HD constexpr bool operator!=(nullopt_t, const optional<T>& a) noexcept { return a.has_value(); }
template <class T> THRUST_CDNA4_HD constexpr bool operator<(const optional<T>&, nullopt_t) noexcept { return false; }
template <class T> THRUST_CDNA4_HD constexpr bool operator<(nullopt_t, const optional<T>& a) noexcept { return a.has_value(); }
template <class T, class U, class = typename std::enable_if<!std::is_same<typename std::decay<U>::type, nullopt_t>::value>::type,
          class = decltype(std::declval<const T&>() == std::declval<const U&>())>
THRUST_CDNA4_HD constexpr bool operator==(const optional<T>& a, const U& b) { return a.has_value() && *a == b; }
template <class T, class U, class = typename std::enable_if<!std::is_same<typename std::decay<U>::type, nullopt_t>::value>::type,
          class = decltype(std::declval<const U&>() == std::declval<const T&>()), class = void>
THRUST_CDNA4_HD constexpr bool operator==(const U& b, const optional<T>& a) { return a.has_value() && b == *a; }
template <class T, class U, class = typename std::enable_if<!std::is_same<typename std::decay<U>::type, nullopt_t>::value>::type,
          class = decltype(std::declval<const T&>() == std::declval<const U&>())>
THRUST_CDNA4_HD constexpr bool operator!=(const optional<T>& a, const U& b) { return !(a == b); }
template <class T, class U, class = typename std::enable_if<!std::is_same<typename std::decay<U>::type, nullopt_t>::value>::type,
          class = decltype(std::declval<const T&>() < std::declval<const U&>())>
THRUST_CDNA4_HD constexpr bool operator<(const optional<T>& a, const U& b) { return !a.has_value() || *a < b; }

template <class T> THRUST_CDNA4_HD void swap(optional<T>& a, optional<T>& b) { a.swap(b); }
template <class T> THRUST_CDNA4_HD constexpr optional<typename std::decay<T>::type> make_optional(T&& v) {
  return optional<typename std::decay<T>::type>(std::forward<T>(v));
}
template <class T, class... Args> THRUST_CDNA4_HD constexpr optional<T> make_optional(Args&&... args) { return optional<T>(in_place, std::forward<Args>(args)...); }

}  // namespace thrust

// thrust::device_event / device_future / when_all (thrust/event.h, thrust/future.h;
// thrust/system/cuda/detail/future.inl:691-960, :1349-): the handle an asynchronous algorithm
// returns.  An event owns the stream its work was submitted to; ready() polls it, wait() blocks
// on it, and the destructor waits, so work never outlives the handle (as in the reference).  A
// future also owns the device storage of its result; get() waits and reads it back once.
#pragma once
#include <memory>
#include <stdexcept>
#include <type_traits>
#include <utility>
#include <vector>
#include <thrust/execution_policy.h>
#include <thrust/system/cdna4/detail/core.h>
#include <thrust/system/error_code.h>

namespace thrust {
// The errors of events and futures (thrust/detail/event_error.h:33-157): an operation on a handle
// without a stream (default constructed, moved from, consumed) raises event_error(no_state), one that
// needs a value on a future without one event_error(no_content).
enum class event_errc { unknown_event_error, no_state, no_content, last_event_error };
struct event_error_category : std::error_category {
  const char* name() const noexcept override { return "event"; }
  std::string message(int ev) const override {
    switch (static_cast<event_errc>(ev)) {
      case event_errc::no_state:
        return "no_state: an operation that requires an event or future to have a stream or content has been performed on an "
               "event or future without either, e.g. a moved-from or default constructed one";
      case event_errc::no_content:
        return "no_content: an operation that requires a future to have content has been performed on a future without any";
      default: return "unknown_event_error: an unknown error with a future object has occurred";
    }
  }
};
inline const std::error_category& event_category() {
  static const event_error_category result;
  return result;
}
inline std::error_code make_error_code(event_errc e) { return std::error_code(static_cast<int>(e), event_category()); }
inline std::error_condition make_error_condition(event_errc e) { return std::error_condition(static_cast<int>(e), event_category()); }
struct event_error : std::logic_error {
  explicit event_error(std::error_code ec) : std::logic_error(ec.message()), ec_(ec) {}
  explicit event_error(event_errc e) : event_error(make_error_code(e)) {}
  const std::error_code& code() const noexcept { return ec_; }
 private:
  std::error_code ec_;
};
inline bool operator==(const event_error& a, const event_error& b) noexcept { return a.code() == b.code(); }
inline bool operator<(const event_error& a, const event_error& b) noexcept { return a.code() < b.code(); }
namespace system { namespace cdna4 { namespace detail {
// The state shared by an event and the events that depend on it: a stream of its own, plus
// whatever must stay alive until the stream's work is done.
class async_signal {
 public:
  async_signal() : stream_(nullptr), submitted_(nullptr) { throw_on_error(thrust_cdna4_stream_create(&stream_), "async: stream"); }
  ~async_signal() {
    (void)thrust_cdna4_stream_synchronize(stream_);
    keep_.clear();
    if (submitted_) (void)thrust_cdna4_event_destroy(submitted_);
    (void)thrust_cdna4_stream_destroy(stream_);
  }
  async_signal(const async_signal&) = delete;
  async_signal& operator=(const async_signal&) = delete;
  void* stream() const { return stream_; }
  // Called once everything has been submitted: ready() then polls an event recorded behind the
  // work (a stream that holds only a wait on another stream's event does not answer a stream
  // query reliably).
  void mark_submitted() {
    if (!submitted_) throw_on_error(thrust_cdna4_event_create(&submitted_), "async: event");
    throw_on_error(thrust_cdna4_event_record(submitted_, stream_), "async: record");
  }
  bool ready() const {
    int done = 0;
    if (submitted_) throw_on_error(thrust_cdna4_event_query(submitted_, &done), "async: query");
    else throw_on_error(thrust_cdna4_stream_query(stream_, &done), "async: query");
    return done != 0;
  }
  void wait() const { throw_on_error(thrust_cdna4_stream_synchronize(stream_), "async: wait"); }
  // this stream's later work starts after everything submitted so far to `other`
  void depend_on(const async_signal& other) {
    void* e = nullptr;
    throw_on_error(thrust_cdna4_event_create(&e), "async: event");
    int rc = thrust_cdna4_event_record(e, other.stream_);
    if (rc == 0) rc = thrust_cdna4_stream_wait_event(stream_, e);
    (void)thrust_cdna4_event_destroy(e);  // the wait already holds what it needs
    throw_on_error(rc, "async: dependency");
  }
  void keep_alive(std::shared_ptr<void> p) { keep_.push_back(std::move(p)); }
 private:
  void* stream_;
  void* submitted_;
  std::vector<std::shared_ptr<void>> keep_;
};
}}}  // namespace system::cdna4::detail

struct new_stream_t {};
static const new_stream_t new_stream = {};

class device_event {
 public:
  device_event() = default;  // no state
  explicit device_event(new_stream_t) : signal_(std::make_shared<system::cdna4::detail::async_signal>()) {}
  // takes over a signal whose work has all been submitted
  explicit device_event(std::shared_ptr<system::cdna4::detail::async_signal> s) : signal_(std::move(s)) {
    if (signal_) signal_->mark_submitted();
  }
  device_event(device_event&&) = default;
  device_event& operator=(device_event&& o) {
    if (this != &o) {
      if (valid_stream()) wait();
      signal_ = std::move(o.signal_);
    }
    return *this;
  }
  device_event(const device_event&) = delete;
  device_event& operator=(const device_event&) = delete;
  ~device_event() {
    if (valid_stream()) (void)thrust_cdna4_stream_synchronize(signal_->stream());
  }
  bool valid_stream() const { return bool(signal_); }
  bool ready() const { return valid_stream() && signal_->ready(); }
  void wait() const { state().wait(); }
  // the stream the event's work was queued on: converts to the native handle, which
  // native_handle() names as the reference's unique_stream does (thrust/system/cuda/detail/future.inl)
  struct stream_reference {
    void* handle;
    void* native_handle() const { return handle; }
    operator void*() const { return handle; }
  };
  stream_reference stream() const { return stream_reference{state().stream()}; }
  const std::shared_ptr<system::cdna4::detail::async_signal>& signal() const { return signal_; }
  // gives the stream and its work away: the event is left without state
  std::shared_ptr<system::cdna4::detail::async_signal> release_signal() { return std::move(signal_); }
 protected:
  system::cdna4::detail::async_signal& state() const {
    if (!signal_) throw event_error(event_errc::no_state);
    return *signal_;
  }
  std::shared_ptr<system::cdna4::detail::async_signal> signal_;
};

template <class T>
class device_future : public device_event {
  static_assert(detail::is_bytewise_movable<T>::value, "device_future: the value type must be movable as bytes");
 public:
  typedef T value_type;
  device_future() : data_(nullptr), have_(false) {}
  // a stream of its own and no content yet (thrust/system/cuda/detail/future.inl: unique_eager_future(new_stream))
  explicit device_future(new_stream_t) : device_event(new_stream), data_(nullptr), have_(false) {}
  // the signal keeps the storage alive; data points into it
  device_future(std::shared_ptr<system::cdna4::detail::async_signal> s, T* data) : device_event(std::move(s)), data_(data), have_(false) {}
  device_future(device_future&&) = default;
  device_future& operator=(device_future&&) = default;
  bool valid_content() const { return data_ != nullptr || have_; }
  // waits for the work, reads the value back (once) and returns it
  T get() {
    if (!have_) {
      if (!data_) throw event_error(event_errc::no_content);  // with or without a stream (testing/future.cu:77-88)
      wait();
      system::cdna4::detail::throw_on_error(thrust_cdna4_read_back(&value_, data_, sizeof(T), stream()), "future: read back");
      have_ = true;
    }
    return value_;
  }
  T extract() {
    T v = get();
    data_ = nullptr;
    have_ = false;
    signal_.reset();
    return v;
  }
  T* raw_data() const { return data_; }  // the device address of the result
 private:
  T* data_;
  T value_;
  bool have_;
};

// the reference's names for the same handles (thrust/future.h:70-116): an event or future of a system
// is that system's unique eager one, and this build has one device system
template <class System> using unique_eager_event = device_event;
template <class System, class T> using unique_eager_future = device_future<T>;
// the default event and future of a system (thrust/event.h:21-26, thrust/future.h:150-160)
template <class System> using event = unique_eager_event<System>;
template <class System, class T> using future = unique_eager_future<System, T>;
typedef device_event device_unique_eager_event;
template <class T> using device_unique_eager_future = device_future<T>;

namespace system { namespace cdna4 { namespace detail {
// thrust::device.after(events...): the next asynchronous algorithm starts after these.  The events
// are consumed — afterwards they have no stream (thrust/system/cuda/detail/future.inl: the policy
// acquires the streams of its dependencies; testing/async_copy.cu:325-375) — and the algorithm
// continues the first one's stream.  An event without a stream, or a policy used a second time,
// is an event_error(no_state).
struct execute_after : execution_policy<execute_after> {
  struct state {
    std::vector<std::shared_ptr<async_signal>> deps;
    bool used = false;
  };
  std::shared_ptr<state> shared = std::make_shared<state>();  // copies of the policy are the same policy
};
inline void collect(execute_after&) {}
template <class E, class... Es>
void collect(execute_after& p, E&& e, Es&&... es) {
  if (!e.valid_stream()) throw event_error(event_errc::no_state);
  p.shared->deps.push_back(e.release_signal());
  collect(p, std::forward<Es>(es)...);
}
// the first dependency's signal, whose stream waits for the others and keeps them alive
inline std::shared_ptr<async_signal> make_signal(const execute_after& p) {
  if (p.shared->used) throw event_error(event_errc::no_state);
  p.shared->used = true;
  if (p.shared->deps.empty()) return std::make_shared<async_signal>();
  std::shared_ptr<async_signal> s = p.shared->deps[0];
  for (std::size_t i = 1; i < p.shared->deps.size(); i++) {
    s->depend_on(*p.shared->deps[i]);
    s->keep_alive(p.shared->deps[i]);
  }
  p.shared->deps.clear();
  return s;
}
inline std::shared_ptr<async_signal> make_signal(const par_t&) { return std::make_shared<async_signal>(); }
inline std::shared_ptr<async_signal> make_signal(const par_nosync_t&) { return std::make_shared<async_signal>(); }
// any other policy (the host system's, a user's): nothing to wait for
template <class Policy> inline std::shared_ptr<async_signal> make_signal(const Policy&) { return std::make_shared<async_signal>(); }
}}}  // namespace system::cdna4::detail

namespace system { namespace cdna4 { namespace detail {
template <class... Events>
execute_after par_t::after(Events&&... events) const {
  execute_after p;
  collect(p, std::forward<Events>(events)...);
  return p;
}
}}}  // namespace system::cdna4::detail
// an event that is ready when all of the given ones are
// The given events are consumed, lvalues too (testing/event.cu:72-110: afterwards they have no
// stream and are not ready), and the result continues the first one's stream, which waits for the
// others (thrust/system/cuda/detail/future.inl:1349-: when_all acquires the streams of its arguments).
namespace system { namespace cdna4 { namespace detail {
inline void consume(std::vector<std::shared_ptr<async_signal>>&) {}
template <class E, class... Es>
void consume(std::vector<std::shared_ptr<async_signal>>& taken, E&& e, Es&&... es) {
  if (e.valid_stream()) taken.push_back(e.release_signal());
  consume(taken, std::forward<Es>(es)...);
}
}}}  // namespace system::cdna4::detail
template <class... Events>
device_event when_all(Events&&... events) {
  std::vector<std::shared_ptr<system::cdna4::detail::async_signal>> taken;
  system::cdna4::detail::consume(taken, std::forward<Events>(events)...);
  if (taken.empty()) return device_event(std::make_shared<system::cdna4::detail::async_signal>());
  std::shared_ptr<system::cdna4::detail::async_signal> first = taken[0];
  for (std::size_t i = 1; i < taken.size(); i++) {
    first->depend_on(*taken[i]);
    first->keep_alive(taken[i]);
  }
  return device_event(std::move(first));
}
}  // namespace thrust

// <thrust/system/detail/internal/decompose.h>: uniform_decomposition — [0, N) cut into at most
// max_intervals ranges whose lengths are multiples of a granularity and differ by at most one
// granule, the longer ones first (thrust/system/detail/internal/decompose.h:28-108).
#pragma once
#include <thrust/detail/config.h>
namespace thrust { namespace system { namespace detail { namespace internal {
template <class IndexType>
class index_range {
 public:
  typedef IndexType index_type;
  THRUST_HOST_DEVICE index_range(index_type begin, index_type end) : begin_(begin), end_(end) {}
  THRUST_HOST_DEVICE index_type begin() const { return begin_; }
  THRUST_HOST_DEVICE index_type end() const { return end_; }
  THRUST_HOST_DEVICE index_type size() const { return end_ - begin_; }
 private:
  index_type begin_, end_;
};
template <class IndexType>
class uniform_decomposition {
 public:
  typedef IndexType index_type;
  typedef index_range<index_type> range_type;
  THRUST_HOST_DEVICE uniform_decomposition(index_type n, index_type granularity, index_type max_intervals)
      : n_(n), intervals_((n + granularity - 1) / granularity), longer_(0), short_(granularity), long_(0) {
    if (intervals_ > max_intervals) {  // granules are shared out; the first `longer_` ranges get one more
      short_ = granularity * (intervals_ / max_intervals);
      long_ = short_ + granularity;
      longer_ = intervals_ % max_intervals;
      intervals_ = max_intervals;
    }
  }
  THRUST_HOST_DEVICE range_type operator[](const index_type& i) const {
    if (i < longer_) return range_type(long_ * i, long_ * i + long_);
    const index_type begin = long_ * longer_ + short_ * (i - longer_);
    return range_type(begin, begin + short_ < n_ ? begin + short_ : n_);
  }
  THRUST_HOST_DEVICE index_type size() const { return intervals_; }
 private:
  index_type n_, intervals_, longer_, short_, long_;
};
}}}}  // namespace thrust::system::detail::internal

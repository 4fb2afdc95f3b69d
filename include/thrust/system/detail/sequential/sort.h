// Sequential stable sort, callable from host and device code (thrust::seq): the counterpart of
// thrust/system/detail/sequential/sort.inl:42-200 (stable_merge_sort / stable_radix_sort behind
// sequential::stable_sort and stable_sort_by_key).  The reference allocates a temporary array
// for its merges; a thread inside a kernel has no allocator to ask, so this sort works in place:
// runs of kRun elements by insertion, then bottom-up merges in which the two sorted halves are
// brought together by rotations (binary search for the cut, three reversals), which keeps equal
// elements in their order.  O(n log^2 n) moves, no storage beyond a fixed explicit stack.
#pragma once
#include <cstdint>
#include <iterator>
#include <thrust/detail/hd.h>

namespace thrust { namespace system { namespace detail { namespace sequential {

// the elements a sort moves: keys, or keys together with their values
template <class KIt>
struct keys_only {
  KIt k;
  THRUST_CDNA4_HD void swap(std::int64_t a, std::int64_t b) const {
    typename std::iterator_traits<KIt>::value_type t = k[a];  // (k[a] may be a proxy reference)
    k[a] = k[b];
    k[b] = t;
  }
};
template <class KIt, class VIt>
struct keys_and_values {
  KIt k;
  VIt v;
  THRUST_CDNA4_HD void swap(std::int64_t a, std::int64_t b) const {
    typename std::iterator_traits<KIt>::value_type t = k[a];
    k[a] = k[b];
    k[b] = t;
    typename std::iterator_traits<VIt>::value_type u = v[a];
    v[a] = v[b];
    v[b] = u;
  }
};

template <class Items>
THRUST_CDNA4_HD void reverse_range(const Items& x, std::int64_t first, std::int64_t last) {
  for (--last; first < last; ++first, --last) x.swap(first, last);
}
// [first, mid) and [mid, last) change places
template <class Items>
THRUST_CDNA4_HD void rotate_range(const Items& x, std::int64_t first, std::int64_t mid, std::int64_t last) {
  if (first == mid || mid == last) return;
  reverse_range(x, first, mid);
  reverse_range(x, mid, last);
  reverse_range(x, first, last);
}

// Merges the sorted ranges [first, mid) and [mid, last) in place, stably.  Each step cuts the
// longer range in the middle, finds the matching cut of the other by binary search, rotates the
// two inner pieces into place and is left with two smaller merges; the larger one waits on a
// stack while the smaller one is done, so the stack never holds more than 64 entries.
template <class Items, class KIt, class Compare>
THRUST_CDNA4_HD void merge_in_place(const Items& x, KIt k, std::int64_t first, std::int64_t mid, std::int64_t last, Compare comp) {
  std::int64_t stack[3 * 64];  // (first, mid, last) of the merges that wait
  int depth = 0;
  for (;;) {
    const std::int64_t n1 = mid - first, n2 = last - mid;
    bool done = n1 == 0 || n2 == 0;
    if (!done && n1 + n2 == 2) {
      if (comp(k[mid], k[first])) x.swap(first, mid);
      done = true;
    }
    if (done) {
      if (depth == 0) return;
      depth--;
      first = stack[3 * depth];
      mid = stack[3 * depth + 1];
      last = stack[3 * depth + 2];
      continue;
    }
    std::int64_t cut1, cut2;
    if (n1 > n2) {
      cut1 = first + n1 / 2;
      // the first element of the second range that is not before k[cut1]
      std::int64_t lo = mid, hi = last;
      while (lo < hi) {
        const std::int64_t m = lo + (hi - lo) / 2;
        if (comp(k[m], k[cut1])) lo = m + 1; else hi = m;
      }
      cut2 = lo;
    } else {
      cut2 = mid + n2 / 2;
      // the first element of the first range that k[cut2] is before
      std::int64_t lo = first, hi = mid;
      while (lo < hi) {
        const std::int64_t m = lo + (hi - lo) / 2;
        if (comp(k[cut2], k[m])) hi = m; else lo = m + 1;
      }
      cut1 = lo;
    }
    rotate_range(x, cut1, mid, cut2);
    const std::int64_t new_mid = cut1 + (cut2 - mid);
    // left: [first, cut1) with [cut1, new_mid); right: [new_mid, cut2) with [cut2, last)
    const bool left_is_smaller = new_mid - first <= last - new_mid;
    stack[3 * depth] = left_is_smaller ? new_mid : first;
    stack[3 * depth + 1] = left_is_smaller ? cut2 : cut1;
    stack[3 * depth + 2] = left_is_smaller ? last : new_mid;
    depth++;
    if (left_is_smaller) {
      mid = cut1;
      last = new_mid;
    } else {
      first = new_mid;
      mid = cut2;
    }
  }
}

template <class Items, class KIt, class Compare>
THRUST_CDNA4_HD void stable_sort_in_place(const Items& x, KIt k, std::int64_t n, Compare comp) {
  constexpr std::int64_t kRun = 16;
  for (std::int64_t r = 0; r < n; r += kRun) {
    const std::int64_t end = r + kRun < n ? r + kRun : n;
    for (std::int64_t i = r + 1; i < end; i++)
      for (std::int64_t j = i; j > r && comp(k[j], k[j - 1]); j--) x.swap(j, j - 1);
  }
  for (std::int64_t width = kRun; width < n; width *= 2)
    for (std::int64_t lo = 0; lo + width < n; lo += 2 * width)
      merge_in_place(x, k, lo, lo + width, lo + 2 * width < n ? lo + 2 * width : n, comp);
}

}}}}  // namespace thrust::system::detail::sequential

// merge / merge_by_key and the set operations of the cdna4 system, as kernel templates
// (thrust/system/cuda/detail/merge.h, set_operations.h).
//
// merge: the output is cut into tiles of 512 x IPT items; one thread per tile boundary finds by
// binary search along the merge path (in global memory) how many items of the first range lie
// before the boundary, then each workgroup loads its pieces of both ranges into LDS, every thread
// finds its own diagonal there and merges IPT outputs serially.  Ties take from the first range:
// the merge is stable, as the reference's (testing/merge.cu, merge_by_key.cu).  Values, if any,
// follow through LDS by source position.
//
// Set operations on sorted ranges with multiset semantics (an element that occurs m times in the
// first range and n times in the second occurs min(m, n) times in the intersection, max(m - n, 0)
// in the difference, max(m, n) in the union and |m - n| in the symmetric difference; the
// reference's tests pin this, testing/set_intersection.cu, set_union.cu ...).  Element i of a
// range is the r-th of its equivalents (r = i - lower_bound of itself in its own range); with c =
// the number of its equivalents in the other range it belongs to the intersection iff r < c and
// to the difference iff r >= c.  That is a predicate per element — three binary searches — so
// intersection and difference are one stable compaction (the select engine), the union is
// merge(first, second \ first) and the symmetric difference merge(first \ second, second \ first),
// where the stable merge puts the first range's elements before equivalent ones of the second,
// as the sequential algorithms do.
#pragma once
#if !defined(__HIPCC__)
#error "thrust/system/cdna4/detail/merge_engine.h holds device kernel templates: compile with hipcc"
#endif
#include <hip/hip_runtime.h>
#include <cstdint>
#include <type_traits>
#include <thrust/system/cdna4/detail/core.h>
#include <thrust/system/cdna4/detail/parallel_for.h>
#include <thrust/system/cdna4/detail/generic_algorithms.h>

namespace thrust { namespace system { namespace cdna4 { namespace detail { namespace merge2 {

constexpr int kBlock = 512;
using ::thrust::system::cdna4::detail::no_values;
template <class V> struct value_bytes { static constexpr std::size_t value = sizeof(V); };
template <> struct value_bytes<no_values> { static constexpr std::size_t value = 0; };
// items per thread by the LDS a tile of keys and values takes (at most 64 KiB of static LDS)
template <class K, std::size_t VB>
constexpr int items_per_thread() {
  return sizeof(K) + VB <= 8 ? 8 : sizeof(K) + VB <= 32 ? 4 : sizeof(K) + VB <= 64 ? 2 : 1;
}

// splits[t] = how many of the first t * TILE outputs (all of them for the last entry) come from a
template <int TILE, class KA, class KB, class Compare>
__global__ __launch_bounds__(256) void partition_kernel(KA a, std::int64_t na, KB b, std::int64_t nb, std::int64_t nsplits,
                                                        std::int64_t* splits, Compare comp) {
  const std::int64_t t = (std::int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= nsplits) return;
  const std::int64_t total = na + nb;
  const std::int64_t diag = t * TILE < total ? t * TILE : total;
  std::int64_t lo = diag > nb ? diag - nb : 0;
  std::int64_t hi = diag < na ? diag : na;
  while (lo < hi) {
    const std::int64_t mid = (lo + hi) >> 1;
    if (!comp(b[diag - 1 - mid], a[mid])) lo = mid + 1;  // a[mid] is not after b[...]: it is among the first diag
    else hi = mid;
  }
  splits[t] = lo;
}

template <int IPT, bool HAS_VALUES, class K, class V, class KA, class KB, class VA, class VB, class KO, class VO, class Compare>
__global__ __launch_bounds__(kBlock) void merge_kernel(KA a, std::int64_t na, KB b, std::int64_t nb, VA va, VB vb, KO kout, VO vout,
                                                       const std::int64_t* splits, Compare comp) {
  constexpr int kTile = kBlock * IPT;
  typedef typename std::aligned_storage<sizeof(K), alignof(K)>::type RawK;
  typedef typename std::aligned_storage<sizeof(V), alignof(V)>::type RawV;
  __shared__ RawK raw_keys[kTile];
  __shared__ RawV raw_vals[HAS_VALUES ? kTile : 1];
  K* s_keys = reinterpret_cast<K*>(raw_keys);
  V* s_vals = reinterpret_cast<V*>(raw_vals);
  const int tid = threadIdx.x;
  const std::int64_t tile = blockIdx.x;
  const std::int64_t out0 = tile * kTile;
  const std::int64_t total = na + nb;
  const int count = (int)(total - out0 < kTile ? total - out0 : kTile);  // >= 1
  const std::int64_t sa0 = splits[tile], sa1 = splits[tile + 1];
  const std::int64_t sb0 = out0 - sa0;
  const int cnt_a = (int)(sa1 - sa0), cnt_b = count - cnt_a;

  // independent loads with clamped indices (a load under a per-item branch waits for the one
  // before it); a piece that is empty is skipped as a whole
  if (cnt_a > 0) {
#pragma unroll
    for (int u = 0; u < IPT; u++) {
      const int i = tid + u * kBlock;
      const int ic = i < cnt_a ? i : cnt_a - 1;
      const K k = a[sa0 + ic];
      if (i < cnt_a) s_keys[i] = k;
      if constexpr (HAS_VALUES) {
        const V v = va[sa0 + ic];
        if (i < cnt_a) s_vals[i] = v;
      }
    }
  }
  if (cnt_b > 0) {
#pragma unroll
    for (int u = 0; u < IPT; u++) {
      const int i = tid + u * kBlock;
      const int ic = i < cnt_b ? i : cnt_b - 1;
      const K k = b[sb0 + ic];
      if (i < cnt_b) s_keys[cnt_a + i] = k;
      if constexpr (HAS_VALUES) {
        const V v = vb[sb0 + ic];
        if (i < cnt_b) s_vals[cnt_a + i] = v;
      }
    }
  }
  __syncthreads();

  const K* sa = s_keys;
  const K* sb = s_keys + cnt_a;
  int d = tid * IPT;
  if (d > count) d = count;
  int lo = d > cnt_b ? d - cnt_b : 0;
  int hi = d < cnt_a ? d : cnt_a;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (!comp(sb[d - 1 - mid], sa[mid])) lo = mid + 1;
    else hi = mid;
  }
  int pa = lo, pb = d - lo;
  // serial merge with both candidates in registers: one LDS read per output (the tile is never
  // empty, so slot 0 is always readable); outputs past `count` are computed and not stored
  K ka = s_keys[pa < cnt_a ? pa : 0], kb = s_keys[pb < cnt_b ? cnt_a + pb : 0];
#pragma unroll
  for (int j = 0; j < IPT; j++) {
    const bool take_a = pb >= cnt_b || (pa < cnt_a && !comp(kb, ka));
    const K k = take_a ? ka : kb;
    const int src = take_a ? pa : cnt_a + pb;
    pa += take_a ? 1 : 0;
    pb += take_a ? 0 : 1;
    const int next = take_a ? (pa < cnt_a ? pa : 0) : (pb < cnt_b ? cnt_a + pb : 0);
    const K kn = s_keys[next];
    ka = take_a ? kn : ka;
    kb = take_a ? kb : kn;
    if (d + j < count) {
      kout[out0 + d + j] = k;
      if constexpr (HAS_VALUES) vout[out0 + d + j] = s_vals[src];
    }
  }
}

// out[0, na + nb) = stable merge of a[0, na) and b[0, nb) under comp; values follow their keys
template <bool HAS_VALUES, class KA, class KB, class VA, class VB, class KO, class VO, class Compare>
void merge(void* stream_, KA a, std::int64_t na, KB b, std::int64_t nb, VA va, VB vb, KO kout, VO vout, Compare comp) {
  typedef typename std::iterator_traits<KA>::value_type K;
  typedef typename std::conditional<HAS_VALUES, typename std::iterator_traits<typename std::conditional<HAS_VALUES, VA, KA>::type>::value_type, char>::type V;
  static_assert(thrust::detail::is_bytewise_movable<K>::value && thrust::detail::is_bytewise_movable<V>::value,
                "cdna4 merge: keys and values must be movable as bytes");
  constexpr int IPT = items_per_thread<K, HAS_VALUES ? sizeof(V) : 0>();
  constexpr int kTile = kBlock * IPT;
  static_assert((sizeof(K) + (HAS_VALUES ? sizeof(V) : 0)) * kTile <= 65536, "cdna4 merge: an item is too large for a tile in LDS");
  const std::int64_t total = na + nb;
  if (total <= 0) return;
  hipStream_t s = static_cast<hipStream_t>(stream_);
  const std::int64_t tiles = (total + kTile - 1) / kTile;
  temporary_storage tmp((std::size_t)(tiles + 1) * sizeof(std::int64_t), stream_);
  std::int64_t* splits = static_cast<std::int64_t*>(tmp.data());
  hipLaunchKernelGGL((partition_kernel<kTile, KA, KB, Compare>), dim3((unsigned)((tiles + 1 + 255) / 256)), dim3(256), 0, s, a, na, b, nb,
                     tiles + 1, splits, comp);
  hipLaunchKernelGGL((merge_kernel<IPT, HAS_VALUES, K, V, KA, KB, VA, VB, KO, VO, Compare>), dim3((unsigned)tiles), dim3(kBlock), 0, s, a, na,
                     b, nb, va, vb, kout, vout, splits, comp);
  throw_on_error((int)hipGetLastError(), "merge: launch");
}

// ---- set operations: the per-element predicate ----------------------------------------------
// first position in r[0, n) whose element is not before x (UPPER: is after x); branch-free steps
template <bool UPPER, class R, class T, class Compare>
__device__ inline std::int64_t bound(R r, std::int64_t n, const T& x, Compare& comp) {
  std::int64_t lo = 0, len = n;
  while (len > 0) {
    const std::int64_t half = len >> 1;
    const bool right = UPPER ? !(bool)comp(x, r[lo + half]) : (bool)comp(r[lo + half], x);
    lo = right ? lo + half + 1 : lo;
    len = right ? len - half - 1 : half;
  }
  return lo;
}
// Keeps element i of `own` when it is (INTERSECT) / is not (!INTERSECT) matched by an equivalent
// element of `other`: the r-th of its equivalents is matched iff other holds more than r of them.
template <bool INTERSECT, bool HAS_VALUES, class Own, class Other, class Vals, class KOut, class VOut, class Compare>
struct set_keep_op {
  typedef typename std::iterator_traits<Own>::value_type K;
  typedef typename std::conditional<HAS_VALUES, typename std::iterator_traits<typename std::conditional<HAS_VALUES, Vals, Own>::type>::value_type, no_values>::type V;
  struct pair_item { K key; V value; };
  typedef typename std::conditional<HAS_VALUES, pair_item, K>::type item;
  static constexpr bool rejects = false;
  Own own; std::int64_t n_own; Other other; std::int64_t n_other; Vals vals; KOut kout; VOut vout; mutable Compare comp;
  __device__ static const K& key_of(const K& k) { return k; }
  __device__ static const K& key_of(const pair_item& p) { return p.key; }
  __device__ item make(const K& k, std::int64_t i, std::true_type) const { return pair_item{k, (V)vals[i]}; }
  __device__ item make(const K& k, std::int64_t, std::false_type) const { return k; }
  __device__ item load(std::int64_t i, bool& keep) const {
    const K x = own[i];
    const std::int64_t rank = i - bound<false>(own, i, x, comp);  // equivalents of x before position i
    const std::int64_t lb = bound<false>(other, n_other, x, comp);
    const std::int64_t ub = lb + bound<true>(other + lb, n_other - lb, x, comp);
    keep = (rank < ub - lb) == INTERSECT;
    return make(x, i, std::integral_constant<bool, HAS_VALUES>());
  }
  __device__ void store_one(const K& k, std::int64_t pos) const { kout[pos] = k; }
  __device__ void store_one(const pair_item& p, std::int64_t pos) const { kout[pos] = p.key; vout[pos] = p.value; }
  __device__ void store(const item& x, std::int64_t pos) const { store_one(x, pos); }
};

// kout[0, count) (and vout) = the elements of own[0, n_own) kept by the rule above, in order
template <bool INTERSECT, bool HAS_VALUES, class Own, class Other, class Vals, class KOut, class VOut, class Compare>
std::int64_t set_select(void* stream_, Own own, std::int64_t n_own, Other other, std::int64_t n_other, Vals vals, KOut kout, VOut vout,
                        Compare comp) {
  return generic::select(stream_, n_own,
                         set_keep_op<INTERSECT, HAS_VALUES, Own, Other, Vals, KOut, VOut, Compare>{own, n_own, other, n_other, vals, kout, vout, comp});
}

}}}}}  // namespace thrust::system::cdna4::detail::merge2

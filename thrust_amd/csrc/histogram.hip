// Even-bin histogram for gfx950: LDS-privatised counters, replicated per LANE, merged into
// global memory with atomics.  The reference has no histogram function; this is the device
// counterpart of the pattern in examples/histogram.cu:60-101.
//
// Bin mapping (identical on host and device, all in IEEE double without contraction):
//   v = (double)x;  dropped unless lower <= v < upper;
//   bin = (int)((v - lower) * scale), scale = num_bins / (upper - lower), clamped to num_bins-1.
//
// LDS layout: counter of (bin, copy) at word bin*copies + copy, copy = lane % copies, copies a
// power of two <= 32.  With 32 copies (up to 256 bins) lane l always hits bank l % 32: no bank
// conflicts and no two lanes of a half-wave on one address, whatever the data (uniform, a few
// hot bins, constant).  Fewer copies (more bins) get one padding word per 32 so that bins hit
// with a power-of-two stride do not fall into a few banks; there, samples that share a bin
// within one instruction still serialise, and when a quarter or more of a wave's lanes hit the
// bin of its first lane those lanes are counted with one ballot and a single atomic.
#include "common.h"

namespace tcd {

constexpr int kHistBlock = 512;
constexpr int kHistLdsWords = 16384;  // counters per workgroup (64 KiB); 16896 words with padding

template <class T>
__device__ inline int bin_of_sample(T x, double lower, double upper, double scale, int num_bins) {
  const double v = (double)x;
  if (!(v >= lower && v < upper)) return -1;
  int b = (int)((v - lower) * scale);
  return b >= num_bins ? num_bins - 1 : b;
}

// LDS > 0: counters live in LDS (LDS words, plus padding); LDS = 0: counters are the global
// array itself (more bins than fit in LDS).
// MODE 0: general mapping.  MODE 2 (1-byte samples): the workgroup counts the 256 raw byte
// values (always 32 copies, conflict-free) and maps each value's count to its bin only when it
// merges into global memory, so the per-sample work does not depend on the bin mapping at all.
template <class T, int LDS, int MODE>
__global__ __launch_bounds__(kHistBlock) void histogram_kernel(const T* __restrict__ samples, int64_t n,
                                                               uint32_t* counts, int num_bins, double lower,
                                                               double upper, double scale, int copies_log2,
                                                               int vec_ok) {
  constexpr int VEC = 16 / sizeof(T);
  // independent 128-bit loads in flight per thread.  1-byte samples: eight, with ONE workgroup
  // per CU — the per-sample LDS instruction (16 per load) is the scarce resource there, and few
  // wavefronts with deep queues of loads measured 25 % faster than many with shallow ones.
  constexpr int kHistUnroll = sizeof(T) == 1 ? 8 : sizeof(T) == 2 ? 4 : 2;
  __shared__ uint32_t s_hist[LDS > 0 ? LDS + LDS / 32 : 1];
  __shared__ uint32_t s_out[MODE == 2 ? 256 : 1];
  const int tid = threadIdx.x;
  const int lds_bins = MODE == 2 ? 256 : num_bins;  // counters kept per copy
  // byte counting (MODE 2) always has 32 unpadded copies: known at compile time, which keeps the
  // per-sample address arithmetic at one shift-or
  if constexpr (MODE == 2) copies_log2 = 5;
  const int copies = 1 << copies_log2;
  const bool padded = copies < 32;
  const uint32_t my_copy = (uint32_t)tid & (uint32_t)(copies - 1);

  if constexpr (LDS > 0) {
    const int words = (lds_bins << copies_log2) + (padded ? (lds_bins << copies_log2) >> 5 : 0);
    for (int i = tid; i < words; i += kHistBlock) s_hist[i] = 0;
  }
  __syncthreads();

  auto slot = [&](int b, uint32_t copy) -> uint32_t {
    const uint32_t a = ((uint32_t)b << copies_log2) + copy;
    return padded ? a + (a >> 5) : a;
  };
  auto bin_of = [&](T x) -> int {
    if constexpr (MODE == 2) {
      uint8_t raw;
      __builtin_memcpy(&raw, &x, 1);
      return (int)raw;
    } else {
      return bin_of_sample<T>(x, lower, upper, scale, num_bins);
    }
  };
  auto add = [&](int b, uint32_t v) {
    if constexpr (LDS > 0) atomicAdd(&s_hist[slot(b, my_copy)], v);
    else atomicAdd(&counts[b], v);
  };
  auto count_plain = [&](int b) {
    if (MODE == 2 || b >= 0) add(b, 1u);  // a raw byte value is always a valid counter
  };
  // counts the lanes sharing the first active lane's bin with one atomic, the rest one by one
  auto count_peeled = [&](int b) {
    const int hot = __builtin_amdgcn_readfirstlane(b);
    const uint64_t same = __builtin_amdgcn_ballot_w64(b == hot);
    if (b == hot) {
      if (hot >= 0 && lane_id() == (int)__builtin_ctzll(same)) add(hot, (uint32_t)__popcll(same));
    } else if (b >= 0) {
      add(b, 1u);
    }
  };
  auto count_group = [&](const T (&v)[VEC]) {
    int b[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) b[j] = bin_of(v[j]);
    // skew test on the first sample of the group: decides the path for all of them (not
    // needed with 16 or more copies, where lanes rarely share an address)
    const int hot = __builtin_amdgcn_readfirstlane(b[0]);
    if (copies_log2 < 4 && __popcll(__builtin_amdgcn_ballot_w64(b[0] == hot)) >= kWave / 4) {
#pragma unroll
      for (int j = 0; j < VEC; j++) count_peeled(b[j]);
    } else {
#pragma unroll
      for (int j = 0; j < VEC; j++) count_plain(b[j]);
    }
  };

  const int64_t gtid = (int64_t)blockIdx.x * kHistBlock + tid;
  const int64_t gstride = (int64_t)gridDim.x * kHistBlock;
  if (vec_ok) {
    struct alignas(16) V16 { T v[VEC]; };
    const int64_t nvec = n / VEC;
    const V16* sv = reinterpret_cast<const V16*>(samples);
    int64_t i = gtid;
    for (; i + (kHistUnroll - 1) * gstride < nvec; i += kHistUnroll * gstride) {
      V16 v[kHistUnroll];
#pragma unroll
      for (int u = 0; u < kHistUnroll; u++) v[u] = load16<V16>(&sv[i + u * gstride]);
#pragma unroll
      for (int u = 0; u < kHistUnroll; u++) count_group(v[u].v);
    }
    for (; i < nvec; i += gstride) {
      const V16 v = load16<V16>(&sv[i]);
      count_group(v.v);
    }
    for (int64_t i = nvec * VEC + gtid; i < n; i += gstride) count_plain(bin_of(samples[i]));
  } else {
    for (int64_t i = gtid; i < n; i += gstride) count_plain(bin_of(samples[i]));
  }

  if constexpr (LDS > 0) {
    __syncthreads();
    if constexpr (MODE == 2) {
      // counts of byte values -> bins.  Few bins: combine in LDS first, so that a workgroup
      // sends one atomic per bin (global atomics on one cache line serialise).
      const bool combine = num_bins <= 256;
      if (combine && tid < 256) s_out[tid] = 0;
      if (combine) __syncthreads();
      if (tid < 256) {
        uint32_t c = 0;
        for (int r = 0; r < 32; r++) c += s_hist[(tid << 5) + ((r + tid) & 31)];  // rotated: no bank conflicts
        T x;
        const uint8_t raw = (uint8_t)tid;
        __builtin_memcpy(&x, &raw, 1);
        const int bin = bin_of_sample<T>(x, lower, upper, scale, num_bins);
        if (c && bin >= 0) {
          if (combine) atomicAdd(&s_out[bin], c);
          else atomicAdd(&counts[bin], c);
        }
      }
      if (combine) {
        __syncthreads();
        if (tid < num_bins && s_out[tid]) atomicAdd(&counts[tid], s_out[tid]);
      }
    } else {
      for (int b = tid; b < num_bins; b += kHistBlock) {
        uint32_t c = 0;
        // rotated by the bin so that the threads of a wave read different banks
        for (int r = 0; r < copies; r++) c += s_hist[slot(b, (uint32_t)(r + b) & (uint32_t)(copies - 1))];
        if (c) atomicAdd(&counts[b], c);
      }
    }
  }
}

template <class T, int LDS, int MODE>
static void launch_hist(const T* samples, int64_t n, uint32_t* counts, int num_bins, double lower, double upper,
                        double scale, int vec_ok, int blocks_per_cu, hipStream_t s) {
  const int lds_bins = MODE == 2 ? 256 : num_bins;
  int copies_log2 = 0;
  if (LDS > 0)
    while (copies_log2 < 5 && ((int64_t)lds_bins << (copies_log2 + 1)) <= LDS) copies_log2++;
  int64_t blocks = ceil_div(n, (int64_t)kHistBlock * (16 / (int)sizeof(T)) * 4);
  const int64_t cap = (int64_t)device_cu_count() * blocks_per_cu;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  TCD_LAUNCH("histogram_kernel", (histogram_kernel<T, LDS, MODE>), dim3((unsigned)blocks), dim3(kHistBlock), s,
             samples, n, counts, num_bins, lower, upper, scale, copies_log2, vec_ok);
}

template <class T>
static hipError_t histogram_typed(const void* samples_, int64_t n, uint32_t* counts, int num_bins, double lower,
                                  double upper, hipStream_t s) {
  hipError_t e = zero_async(counts, (size_t)num_bins * 4, s);
  if (e != hipSuccess || n == 0) return e;
  const T* samples = static_cast<const T*>(samples_);
  const double scale = (double)num_bins / (upper - lower);
  const int vec_ok = (reinterpret_cast<uintptr_t>(samples) & (sizeof(T) - 1)) == 0;  // see load16
  // Two LDS footprints: 8192 counters (32 KiB, plus padding) up to 8192 bins — as many copies of
  // every counter as fit, 32 up to 256 bins, 2 at 4096 — and 16384 counters up to 16384 bins;
  // beyond that the counts go straight to global memory.  Workgroups per CU as measured on
  // MI355X at 2^30 samples: one for 1-byte samples (see kHistUnroll), three with the small
  // footprint (2^30 floats into 256 / 4096 bins: 0.66 ms against 0.74 ms with two workgroups of
  // the large one, Zipf or uniform; four are slower again), two with the large one.
  if constexpr (sizeof(T) == 1) {
    launch_hist<T, 8192, 2>(samples, n, counts, num_bins, lower, upper, scale, vec_ok, 1, s);
  } else if (num_bins <= 8192) {
    launch_hist<T, 8192, 0>(samples, n, counts, num_bins, lower, upper, scale, vec_ok, 3, s);
  } else if (num_bins <= kHistLdsWords) {
    launch_hist<T, kHistLdsWords, 0>(samples, n, counts, num_bins, lower, upper, scale, vec_ok, 2, s);
  } else {
    launch_hist<T, 0, 0>(samples, n, counts, num_bins, lower, upper, scale, vec_ok, 4, s);
  }
  return hipGetLastError();
}

}  // namespace tcd

extern "C" int thrust_cdna4_histogram_even(void* temp, size_t* temp_bytes, int sample_dtype,
                                           const void* samples, int64_t n, uint32_t* counts, int num_bins,
                                           double lower, double upper, void* stream) {
  using namespace tcd;
  if (!temp_bytes || n < 0 || num_bins <= 0 || !(upper > lower)) return hipErrorInvalidValue;
  if (!dtype_size(sample_dtype)) return hipErrorInvalidValue;
  if (temp == nullptr) {
    *temp_bytes = 256;  // nothing is needed; a non-zero size keeps the two-phase protocol uniform
    return hipSuccess;
  }
  if (!counts || (n > 0 && !samples)) return hipErrorInvalidValue;
  hipError_t rc = hipErrorInvalidValue;
  dispatch_dtype(sample_dtype, [&](auto t) {
    using T = decltype(t);
    rc = histogram_typed<T>(samples, n, counts, num_bins, lower, upper, static_cast<hipStream_t>(stream));
  });
  return (int)rc;
}

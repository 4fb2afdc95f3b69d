// Even-bin histogram for gfx950: LDS-privatised, per-wave replicated sub-histograms merged
// into global memory with atomics.  The reference has no histogram function; this is the
// device counterpart of the pattern in examples/histogram.cu:60-101.
//
// Bin mapping (identical on host and device, all in IEEE double without contraction):
//   v = (double)x;  dropped unless lower <= v < upper;
//   bin = (int)((v - lower) * scale), scale = num_bins / (upper - lower), clamped to num_bins-1.
//
// Contention: samples that share a bin within one wave instruction serialise in the LDS atomic
// unit.  When a quarter or more of a wave's lanes hit the bin of its first lane ("hot" bin:
// skewed data, e.g. Zipf ranks), those lanes are counted with one ballot and a single atomic,
// and only the remaining lanes issue their own.
#include "common.h"

namespace tcd {

constexpr int kHistBlock = 512;
constexpr int kHistWaves = kHistBlock / kWave;

// LDS slot of bin b: one padding word per 32 bins, so that bins hit with a power-of-two stride
// (e.g. 8-bit samples spread over 4096 bins: every 16th bin) do not all fall into two banks.
__host__ __device__ inline int lds_slot(int b) { return b + (b >> 5); }

template <class T>
__device__ inline int bin_of_sample(T x, double lower, double upper, double scale, int num_bins) {
  const double v = (double)x;
  if (!(v >= lower && v < upper)) return -1;
  int b = (int)((v - lower) * scale);
  return b >= num_bins ? num_bins - 1 : b;
}

// LDS_WORDS > 0: counters live in LDS (replicated `reps` times, replica = wave % reps);
//           = 0: counters are the global array itself (more bins than fit in LDS).
// MODE 0: general mapping; 1: 1-byte samples through a 256-entry table built per workgroup;
//      2: 1-byte unsigned samples whose bin is the sample value (lower 0, upper 256, 256 bins).
template <class T, int LDS_WORDS, int MODE>
__global__ __launch_bounds__(kHistBlock) void histogram_kernel(const T* __restrict__ samples, int64_t n,
                                                               uint32_t* counts, int num_bins, double lower,
                                                               double upper, double scale, int reps,
                                                               int vec_ok) {
  constexpr int VEC = 16 / sizeof(T);
  __shared__ uint32_t s_hist[LDS_WORDS > 0 ? LDS_WORDS + LDS_WORDS / 32 : 1];
  __shared__ int s_lut[MODE == 1 ? 256 : 1];
  const int tid = threadIdx.x;
  const int wave = tid / kWave;

  if constexpr (LDS_WORDS > 0) {
    for (int i = tid; i < reps * lds_slot(num_bins); i += kHistBlock) s_hist[i] = 0;
  }
  if constexpr (MODE == 1) {
    if (tid < 256) {
      T x;
      const uint8_t raw = (uint8_t)tid;
      __builtin_memcpy(&x, &raw, 1);
      s_lut[tid] = bin_of_sample<T>(x, lower, upper, scale, num_bins);
    }
  }
  __syncthreads();

  uint32_t* my = LDS_WORDS > 0 ? s_hist + (wave % reps) * lds_slot(num_bins) : counts;
  auto slot = [](int b) { return LDS_WORDS > 0 ? lds_slot(b) : b; };
  auto bin_of = [&](T x) -> int {
    if constexpr (MODE == 2) {
      uint8_t raw;
      __builtin_memcpy(&raw, &x, 1);
      return (int)raw;
    } else if constexpr (MODE == 1) {
      uint8_t raw;
      __builtin_memcpy(&raw, &x, 1);
      return s_lut[raw];
    } else {
      return bin_of_sample<T>(x, lower, upper, scale, num_bins);
    }
  };
  auto count_plain = [&](int b) {
    if (MODE == 2 || b >= 0) atomicAdd(&my[slot(b)], 1u);
  };
  // counts the lanes sharing the first active lane's bin with one atomic, the rest one by one
  auto count_peeled = [&](int b) {
    const int hot = __builtin_amdgcn_readfirstlane(b);
    const uint64_t same = __builtin_amdgcn_ballot_w64(b == hot);
    if (b == hot) {
      if (hot >= 0 && lane_id() == (int)__builtin_ctzll(same)) atomicAdd(&my[slot(hot)], (uint32_t)__popcll(same));
    } else if (b >= 0) {
      atomicAdd(&my[slot(b)], 1u);
    }
  };
  auto count_group = [&](const T (&v)[VEC]) {
    int b[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) b[j] = bin_of(v[j]);
    // skew test on the first sample of the group: decides the path for all of them
    const int hot = __builtin_amdgcn_readfirstlane(b[0]);
    if (__popcll(__builtin_amdgcn_ballot_w64(b[0] == hot)) >= kWave / 4) {
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
    for (int64_t i = gtid; i < nvec; i += gstride) {
      const V16 v = sv[i];
      count_group(v.v);
    }
    for (int64_t i = nvec * VEC + gtid; i < n; i += gstride) count_plain(bin_of(samples[i]));
  } else {
    for (int64_t i = gtid; i < n; i += gstride) count_plain(bin_of(samples[i]));
  }

  if constexpr (LDS_WORDS > 0) {
    __syncthreads();
    for (int b = tid; b < num_bins; b += kHistBlock) {
      uint32_t c = 0;
      for (int r = 0; r < reps; r++) c += s_hist[r * lds_slot(num_bins) + lds_slot(b)];
      if (c) atomicAdd(&counts[b], c);
    }
  }
}

template <class T, int LDS_WORDS, int MODE>
static void launch_hist(const T* samples, int64_t n, uint32_t* counts, int num_bins, double lower, double upper,
                        double scale, int vec_ok, int blocks_per_cu, hipStream_t s) {
  int reps = LDS_WORDS > 0 ? (LDS_WORDS + LDS_WORDS / 32) / lds_slot(num_bins) : 1;
  if (reps < 1) reps = 1;
  if (reps > kHistWaves) reps = kHistWaves;
  int64_t blocks = ceil_div(n, (int64_t)kHistBlock * (16 / (int)sizeof(T)) * 4);
  const int64_t cap = 256 * (int64_t)blocks_per_cu;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  TCD_LAUNCH("histogram_kernel", (histogram_kernel<T, LDS_WORDS, MODE>), dim3((unsigned)blocks), dim3(kHistBlock), s,
             samples, n, counts, num_bins, lower, upper, scale, reps, vec_ok);
}

template <class T>
static hipError_t histogram_typed(const void* samples_, int64_t n, uint32_t* counts, int num_bins, double lower,
                                  double upper, hipStream_t s) {
  hipError_t e = zero_async(counts, (size_t)num_bins * 4, s);
  if (e != hipSuccess || n == 0) return e;
  const T* samples = static_cast<const T*>(samples_);
  const double scale = (double)num_bins / (upper - lower);
  const int vec_ok = (reinterpret_cast<uintptr_t>(samples) & 15) == 0;
  constexpr bool kByte = sizeof(T) == 1;
  const bool identity8 = std::is_same<T, uint8_t>::value && num_bins == 256 && lower == 0.0 && upper == 256.0;
  // two LDS footprints: 8 KiB (four workgroups per CU) for up to 2048 counters, 64 KiB otherwise
  if (num_bins <= 2048) {  // (the LDS arrays carry the padding words on top of these sizes)
    if (identity8) launch_hist<T, 2048, kByte ? 2 : 0>(samples, n, counts, num_bins, lower, upper, scale, vec_ok, 4, s);
    else launch_hist<T, 2048, kByte ? 1 : 0>(samples, n, counts, num_bins, lower, upper, scale, vec_ok, 4, s);
  } else if (num_bins <= 16384) {
    launch_hist<T, 16384, kByte ? 1 : 0>(samples, n, counts, num_bins, lower, upper, scale, vec_ok, 2, s);
  } else {
    launch_hist<T, 0, kByte ? 1 : 0>(samples, n, counts, num_bins, lower, upper, scale, vec_ok, 4, s);
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

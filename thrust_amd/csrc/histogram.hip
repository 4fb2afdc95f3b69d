// Even-bin histogram for gfx950: LDS-privatised, per-wave replicated sub-histograms merged
// into global memory with atomics.  The reference has no histogram function; this is the
// device counterpart of the pattern in examples/histogram.cu:60-101.
//
// Bin mapping (identical on host and device, all in IEEE double without contraction):
//   v = (double)x;  dropped unless lower <= v < upper;
//   bin = (int)((v - lower) * scale), scale = num_bins / (upper - lower), clamped to num_bins-1.
#include "common.h"

namespace tcd {

constexpr int kHistBlock = 512;
constexpr int kHistWaves = kHistBlock / kWave;
constexpr int kHistLdsWords = 16384;  // 64 KiB of LDS counters per workgroup

template <class T>
__device__ inline int bin_of_sample(T x, double lower, double upper, double scale, int num_bins) {
  const double v = (double)x;
  if (!(v >= lower && v < upper)) return -1;
  int b = (int)((v - lower) * scale);
  return b >= num_bins ? num_bins - 1 : b;
}

// LDS_BINS: counters live in LDS (replicated `reps` times, replica = wave % reps).
// BYTE_LUT: 1-byte samples look their bin up in a 256-entry table built once per workgroup.
template <class T, bool LDS_BINS>
__global__ __launch_bounds__(kHistBlock) void histogram_kernel(const T* __restrict__ samples, int64_t n,
                                                               uint32_t* counts, int num_bins, double lower,
                                                               double upper, double scale, int reps,
                                                               int vec_ok) {
  constexpr bool BYTE_LUT = sizeof(T) == 1;
  constexpr int VEC = 16 / sizeof(T);
  __shared__ uint32_t s_hist[LDS_BINS ? kHistLdsWords : 1];
  __shared__ int s_lut[BYTE_LUT ? 256 : 1];
  const int tid = threadIdx.x;
  const int wave = tid / kWave;

  if constexpr (LDS_BINS) {
    for (int i = tid; i < reps * num_bins; i += kHistBlock) s_hist[i] = 0;
  }
  if constexpr (BYTE_LUT) {
    if (tid < 256) {
      T x;
      const uint8_t raw = (uint8_t)tid;
      __builtin_memcpy(&x, &raw, 1);
      s_lut[tid] = bin_of_sample<T>(x, lower, upper, scale, num_bins);
    }
  }
  __syncthreads();

  uint32_t* my = LDS_BINS ? s_hist + (wave % reps) * num_bins : counts;
  auto count = [&](T x) {
    int b;
    if constexpr (BYTE_LUT) {
      uint8_t raw;
      __builtin_memcpy(&raw, &x, 1);
      b = s_lut[raw];
    } else {
      b = bin_of_sample<T>(x, lower, upper, scale, num_bins);
    }
    if (b >= 0) atomicAdd(&my[b], 1u);
  };

  const int64_t gtid = (int64_t)blockIdx.x * kHistBlock + tid;
  const int64_t gstride = (int64_t)gridDim.x * kHistBlock;
  if (vec_ok) {
    struct alignas(16) V16 { T v[VEC]; };
    const int64_t nvec = n / VEC;
    const V16* sv = reinterpret_cast<const V16*>(samples);
    for (int64_t i = gtid; i < nvec; i += gstride) {
      const V16 v = sv[i];
#pragma unroll
      for (int j = 0; j < VEC; j++) count(v.v[j]);
    }
    for (int64_t i = nvec * VEC + gtid; i < n; i += gstride) count(samples[i]);
  } else {
    for (int64_t i = gtid; i < n; i += gstride) count(samples[i]);
  }

  if constexpr (LDS_BINS) {
    __syncthreads();
    for (int b = tid; b < num_bins; b += kHistBlock) {
      uint32_t c = 0;
      for (int r = 0; r < reps; r++) c += s_hist[r * num_bins + b];
      if (c) atomicAdd(&counts[b], c);
    }
  }
}

template <class T>
static hipError_t histogram_typed(const void* samples, int64_t n, uint32_t* counts, int num_bins, double lower,
                                  double upper, hipStream_t s) {
  hipError_t e = zero_async(counts, (size_t)num_bins * 4, s);
  if (e != hipSuccess || n == 0) return e;
  const double scale = (double)num_bins / (upper - lower);
  const int vec_ok = (reinterpret_cast<uintptr_t>(samples) & 15) == 0;
  int64_t blocks = ceil_div(n, (int64_t)kHistBlock * (16 / sizeof(T)) * 8);
  if (blocks > 1024) blocks = 1024;
  if (blocks < 1) blocks = 1;
  if (num_bins <= kHistLdsWords) {
    int reps = kHistLdsWords / num_bins;
    if (reps > kHistWaves) reps = kHistWaves;
    TCD_LAUNCH("histogram_kernel", (histogram_kernel<T, true>), dim3((unsigned)blocks), dim3(kHistBlock), s,
                       static_cast<const T*>(samples), n, counts, num_bins, lower, upper, scale, reps, vec_ok);
  } else {
    TCD_LAUNCH("histogram_kernel", (histogram_kernel<T, false>), dim3((unsigned)blocks), dim3(kHistBlock), s,
                       static_cast<const T*>(samples), n, counts, num_bins, lower, upper, scale, 1, vec_ok);
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

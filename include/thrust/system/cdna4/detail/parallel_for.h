// Generic-functor building blocks of the cdna4 system: parallel_for and reduce as kernel
// templates (thrust/system/cuda/detail/parallel_for.h:70-174, reduce.h:152-669, :947-971).
// They carry user functors, so the translation unit that instantiates them is compiled by
// hipcc (--offload-arch=gfx950) and the functors' operator() must be __host__ __device__.
// for_each, transform, sequence, transform_reduce, reduce and count_if in the public headers are
// thin wrappers over these two.
#pragma once
#if !defined(__HIPCC__)
#error "thrust/system/cdna4/detail/parallel_for.h holds device kernel templates: compile with hipcc"
#endif
#include <hip/hip_runtime.h>
#include <cstdint>
#include <type_traits>
#include <thrust/system/cdna4/detail/core.h>

namespace thrust { namespace system { namespace cdna4 { namespace detail { namespace generic {

constexpr int kBlock = 256;
constexpr int kItems = 4;  // indices per thread, strided by the workgroup size: a wave touches contiguous elements

// f(i) for every i in [0, n)
template <class F>
__global__ __launch_bounds__(kBlock) void parallel_for_kernel(std::int64_t n, F f) {
  const std::int64_t base = (std::int64_t)blockIdx.x * (kBlock * kItems) + threadIdx.x;
#pragma unroll
  for (int k = 0; k < kItems; k++) {
    const std::int64_t i = base + (std::int64_t)k * kBlock;
    if (i < n) f(i);
  }
}

template <class F>
void parallel_for(void* stream, std::int64_t n, F f) {
  if (n <= 0) return;
  const std::int64_t blocks = (n + kBlock * kItems - 1) / (kBlock * kItems);
  hipLaunchKernelGGL((parallel_for_kernel<F>), dim3((unsigned)blocks), dim3(kBlock), 0, static_cast<hipStream_t>(stream), n, f);
  throw_on_error((int)hipGetLastError(), "parallel_for: launch");
}

// ---------------------------------------------------------------------------------------
// reduce: workgroup partials, then one workgroup over the partials.  `op` must be associative
// and commutative (the order of combination is unspecified, as in the reference); no identity
// is needed: threads without an element do not take part.
// ---------------------------------------------------------------------------------------
template <class T, class Op>
__device__ inline T block_reduce(T v, int valid_threads, Op op) {
  __shared__ typename std::aligned_storage<sizeof(T), alignof(T)>::type raw[kBlock];
  T* s = reinterpret_cast<T*>(raw);
  const int tid = threadIdx.x;
  s[tid] = v;
  __syncthreads();
#pragma unroll
  for (int stride = kBlock / 2; stride > 0; stride >>= 1) {
    if (tid < stride && tid + stride < valid_threads) {
      v = op(v, s[tid + stride]);
      s[tid] = v;
    }
    __syncthreads();
  }
  return v;  // the total, in thread 0
}

// partial[b] = op-reduction of unary(i) over the indices of workgroup b; every workgroup owns at
// least one index (the host sizes the grid so)
template <class T, class Unary, class Op>
__global__ __launch_bounds__(kBlock) void reduce_partials_kernel(std::int64_t n, Unary unary, Op op, T* partial) {
  const std::int64_t stride = (std::int64_t)gridDim.x * kBlock;
  std::int64_t i = (std::int64_t)blockIdx.x * kBlock + threadIdx.x;
  const std::int64_t first = (std::int64_t)blockIdx.x * kBlock;
  const int valid = (int)(n - first < kBlock ? n - first : kBlock);
  T acc{};
  if (i < n) {
    acc = unary(i);
    i += stride;
    for (; i + 3 * stride < n; i += 4 * stride) {  // four independent loads in flight
      const T a = unary(i), b = unary(i + stride), c = unary(i + 2 * stride), d = unary(i + 3 * stride);
      acc = op(op(acc, a), op(op(b, c), d));
    }
    for (; i < n; i += stride) acc = op(acc, unary(i));
  }
  acc = block_reduce(acc, valid, op);
  if (threadIdx.x == 0) partial[blockIdx.x] = acc;
}

// out[0] = op(init, partial[0] (+) ... (+) partial[count-1])
template <class T, class Op>
__global__ __launch_bounds__(kBlock) void reduce_final_kernel(const T* partial, int count, T init, Op op, T* out) {
  T acc{};
  int i = threadIdx.x;
  if (i < count) {
    acc = partial[i];
    for (i += kBlock; i < count; i += kBlock) acc = op(acc, partial[i]);
  }
  acc = block_reduce(acc, count < kBlock ? count : kBlock, op);
  if (threadIdx.x == 0) out[0] = op(init, acc);
}

// Returns op(init, unary(0) (+) ... (+) unary(n-1)); blocks until the value is on the host
// (thrust/system/cuda/detail/reduce.h:947-971 does the same).
template <class T, class Unary, class Op>
T transform_reduce(void* stream_, std::int64_t n, Unary unary, T init, Op op) {
  static_assert(std::is_trivially_copyable<T>::value, "cdna4 reduce: the result type must be trivially copyable");
  if (n <= 0) return init;
  hipStream_t s = static_cast<hipStream_t>(stream_);
  std::int64_t blocks = (n + kBlock - 1) / kBlock;  // every workgroup gets at least one index
  const std::int64_t enough = 2048;                  // 8 workgroups per CU
  if (blocks > enough) blocks = enough;
  temporary_storage tmp((std::size_t)(blocks + 1) * sizeof(T), stream_);
  T* partial = static_cast<T*>(tmp.data());
  T* out = partial + blocks;
  hipLaunchKernelGGL((reduce_partials_kernel<T, Unary, Op>), dim3((unsigned)blocks), dim3(kBlock), 0, s, n, unary, op, partial);
  hipLaunchKernelGGL((reduce_final_kernel<T, Op>), dim3(1), dim3(kBlock), 0, s, partial, (int)blocks, init, op, out);
  throw_on_error((int)hipGetLastError(), "reduce: launch");
  T result;
  throw_on_error(thrust_cdna4_memcpy_dtoh(&result, out, sizeof(T), stream_), "reduce: read back");
  throw_on_error(thrust_cdna4_stream_synchronize(stream_), "reduce: failed to synchronize");
  return result;
}

}}}}}  // namespace thrust::system::cdna4::detail::generic

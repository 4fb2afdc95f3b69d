// Self-test of the race-detecting build of the emulator (make tsan): two kernels that differ in one
// barrier.  `selftest_race with_barrier` must run clean under ThreadSanitizer; `selftest_race
// without_barrier` (wavefront 1 reads what wavefront 0 wrote to LDS with nothing in between) and
// `selftest_race global` (the same through global memory) must be reported as data races, and so must
// `selftest_race across_workgroups` (workgroup 1 reads what workgroup 0 wrote) when several workgroups
// are in flight (THRUST_CDNA4_EMULATED_RESIDENT=2): one after the other, on one thread, the workgroups
// of a launch are ordered by the emulator itself and such a race goes unseen.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>

template <bool BARRIER>
__global__ void handoff_through_lds(int* out) {
  __shared__ int slot[64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x / 64;
  if (wave == 0) slot[lane] = lane + 1;
  if (BARRIER) __syncthreads();
  if (wave == 1) out[lane] = slot[lane];
}

__global__ void handoff_through_global(int* scratch, int* out) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x / 64;
  if (wave == 0) scratch[lane] = lane + 1;
  if (wave == 1) out[lane] = scratch[lane];
}

__global__ void handoff_across_workgroups(int* scratch, int* out) {
  // the barriers only give the other workgroup its turn in between
  if (blockIdx.x == 0) scratch[threadIdx.x] = (int)threadIdx.x + 1;
  __syncthreads();
  __syncthreads();
  if (blockIdx.x == 1) out[threadIdx.x] = scratch[threadIdx.x];
}

int main(int argc, char** argv) {
  static int out[64], scratch[64];
  const char* what = argc > 1 ? argv[1] : "with_barrier";
  if (!strcmp(what, "with_barrier")) hipLaunchKernelGGL((handoff_through_lds<true>), dim3(2), dim3(128), 0, 0, out);
  else if (!strcmp(what, "without_barrier")) hipLaunchKernelGGL((handoff_through_lds<false>), dim3(2), dim3(128), 0, 0, out);
  else if (!strcmp(what, "across_workgroups")) hipLaunchKernelGGL(handoff_across_workgroups, dim3(2), dim3(64), 0, 0, scratch, out);
  else hipLaunchKernelGGL(handoff_through_global, dim3(1), dim3(128), 0, 0, scratch, out);
  std::printf("%s: out[5] = %d\n", what, out[5]);
  return 0;
}

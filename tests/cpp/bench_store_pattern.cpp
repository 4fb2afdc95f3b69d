// What bounds a radix pass of the onesweep shape on this device, measured with a copy: one
// 1024-thread workgroup per CU, 32768 four-byte keys per tile, through LDS, 2^28 keys.  The variants
// add, one at a time, what the real pass does beyond a copy — a returning LDS atomic per key, a
// data-dependent LDS scatter, an idle stretch of the length of a look-back, stores in 256 per-digit
// runs per tile at different alignments — and hand the tiles out by ticket, by workgroup index, or so
// that consecutive tiles run on one XCD (workgroup i runs on XCD i mod 8).  No workgroup waits for
// another.  Prints one line per variant; bench.py --only store_probe runs it.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e)); exit(1); } } while (0)
constexpr int BLOCK = 1024, IPT = 32, TILE = BLOCK * IPT;
// STORES: 0 contiguous tile, 1 256 runs of 128 keys each at its digit's region (aligned), 2 the same shifted by 37 keys
template <int STORES, int RANK, int SLEEP, int SHIFT = 37, int MAP = 0>
__global__ __launch_bounds__(BLOCK) void probe(const unsigned* __restrict__ in, unsigned* __restrict__ out, unsigned* ticket, size_t n) {
  __shared__ unsigned s[TILE];
  __shared__ unsigned cnt[16][256];
  __shared__ unsigned s_tile;
  if (threadIdx.x == 0) s_tile = atomicAdd(ticket, 1u);
  if (RANK) for (int i = threadIdx.x; i < 16 * 256; i += BLOCK) (&cnt[0][0])[i] = 0;
  __syncthreads();
  unsigned tile = s_tile;
  if (MAP == 1) tile = blockIdx.x;
  if (MAP == 2) tile = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
  if (MAP == 3) { const unsigned x = blockIdx.x % 8, i = blockIdx.x / 8; tile = ((i / 8) * 8 + x) * 8 + (i % 8); }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t base = (size_t)tile * TILE;
  const int slab = wave * (64 * IPT) + lane;
  unsigned k[IPT];
#pragma unroll
  for (int i = 0; i < IPT; i++) k[i] = in[base + slab + i * 64];
  unsigned acc = 0;
  if (RANK) {
#pragma unroll
    for (int i = 0; i < IPT; i++) acc += atomicAdd(&cnt[wave][k[i] & 255u], 1u);  // returning LDS atomic per key
  }
  if (RANK == 2) {  // and the scatter into the exchange buffer goes to data-dependent slots
#pragma unroll
    for (int i = 0; i < IPT; i++) s[(slab + i * 64) ^ ((k[i] >> 8) & 0x7fc0u)] = k[i] + (acc & 1u);
  } else {
#pragma unroll
    for (int i = 0; i < IPT; i++) s[slab + i * 64] = k[i] + (acc & 1u);
  }
  __syncthreads();
  if (SLEEP > 0) {
    if (threadIdx.x < 256) for (int i = 0; i < SLEEP; i++) __builtin_amdgcn_s_sleep(127);
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < IPT; j++) {
    const int li = j * BLOCK + threadIdx.x;
    size_t o = base + li;
    if (STORES) {
      const size_t d = li >> 7, r = li & 127;
      o = d * (n / 256) + (size_t)tile * 128 + r + (STORES == 2 ? SHIFT : 0);
      if (o >= n) o -= n;
    }
    out[o] = s[li];
  }
}
template <int STORES, int RANK, int SLEEP, int SHIFT = 37, int MAP = 0>
float run(const unsigned* in, unsigned* out, unsigned* ticket, int tiles, size_t n) {
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a)); CHECK(hipEventCreate(&b));
  float best = 1e9;
  for (int r = 0; r < 6; r++) {
    CHECK(hipMemset(ticket, 0, 4));
    CHECK(hipEventRecord(a));
    hipLaunchKernelGGL((probe<STORES, RANK, SLEEP, SHIFT, MAP>), dim3(tiles), dim3(BLOCK), 0, 0, in, out, ticket, n);
    CHECK(hipEventRecord(b));
    CHECK(hipEventSynchronize(b));
    float ms; CHECK(hipEventElapsedTime(&ms, a, b));
    if (r > 0 && ms < best) best = ms;
  }
  return best;
}
__global__ void fill(unsigned* p, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    unsigned x = (unsigned)i * 2654435761u; x ^= x >> 15; x *= 2246822519u; x ^= x >> 13;
    p[i] = x;
  }
}
int main() {
  const size_t n = (size_t)1 << 28;
  unsigned *in, *out, *ticket;
  CHECK(hipMalloc(&in, n * 4)); CHECK(hipMalloc(&out, n * 4)); CHECK(hipMalloc(&ticket, 256));
  hipLaunchKernelGGL(fill, dim3(4096), dim3(256), 0, 0, in, n);
  CHECK(hipDeviceSynchronize());
  const int tiles = (int)(n / TILE);
  const double gb = 2.0 * n * 4 / 1e9;
  float t;
#define RUN(S, R, Z, SH, M, label) t = run<S, R, Z, SH, M>(in, out, ticket, tiles, n); printf("%-78s %.4f ms %.2f TB/s\n", label, t, gb / t);
  RUN(0, 0, 0, 0, 0, "contiguous stores, tiles by ticket")
  RUN(0, 1, 0, 0, 0, "  + a returning LDS atomic per key")
  RUN(0, 2, 0, 0, 0, "  + atomics + data-dependent LDS scatter")
  RUN(0, 2, 1, 0, 0, "  + atomics + scatter + 3.4 us idle per tile")
  RUN(2, 0, 0, 0, 0, "256 runs of 512 B per tile, runs start on 128-byte lines")
  RUN(2, 0, 0, 16, 0, "  runs shifted by 64 B")
  RUN(2, 0, 0, 8, 0, "  runs shifted by 32 B")
  RUN(2, 0, 0, 1, 0, "  runs shifted by 4 B")
  RUN(2, 0, 0, 37, 0, "  runs shifted by 148 B (any alignment), tiles by ticket")
  RUN(2, 0, 0, 37, 1, "  runs shifted by 148 B, tile = workgroup index")
  RUN(2, 0, 0, 37, 2, "  runs shifted by 148 B, each XCD a contiguous eighth of the tiles")
  RUN(2, 0, 0, 37, 3, "  runs shifted by 148 B, groups of 8 consecutive tiles per XCD")
  RUN(2, 2, 1, 37, 0, "  runs shifted by 148 B + atomics + scatter + idle, tiles by ticket")
  RUN(2, 2, 1, 37, 3, "  runs shifted by 148 B + atomics + scatter + idle, groups of 8 per XCD")
  return 0;
}

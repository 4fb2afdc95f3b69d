// Runtime services behind the C ABI: error text, the cached temporary-storage allocator,
// copies, fills and stream synchronisation.
#include <mutex>
#include <unordered_map>
#include <vector>

#include <cstring>
#include "common.h"
#include <atomic>

namespace tcd {

__global__ void zero_words_kernel(uint32_t* p, size_t nwords) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < nwords; i += stride) p[i] = 0u;
}

// bytes must be a multiple of 4 (all internal regions are 256-byte multiples)
hipError_t zero_async(void* p, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  const size_t nwords = bytes / 4;
  size_t blocks = (nwords + 1023) / 1024;
  if (blocks > 2048) blocks = 2048;
  TCD_LAUNCH("zero_words_kernel", zero_words_kernel, dim3((unsigned)blocks), dim3(256), stream,
             static_cast<uint32_t*>(p), nwords);
  return hipGetLastError();
}

int device_cu_count() {
  constexpr int kMaxDev = 64;
  static std::atomic<int> cached[kMaxDev];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) return 256;
  int c = cached[dev].load(std::memory_order_relaxed);
  if (c == 0) {
    if (hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || c <= 0) {
      (void)hipGetLastError();
      c = 256;
    }
    cached[dev].store(c, std::memory_order_relaxed);
  }
  return c;
}

// ---------------------------------------------------------------------------------------
// Launch profiling records
// ---------------------------------------------------------------------------------------
struct ProfileRecord {
  const char* name;
  hipEvent_t start, stop;
};
struct Profiler {
  std::mutex mu;
  bool on = false;
  std::vector<ProfileRecord> recs;
};
static Profiler& profiler() {
  static Profiler* p = new Profiler();
  return *p;
}
bool profile_enabled() { return profiler().on; }
void profile_begin(const char* name, hipStream_t stream) {
  Profiler& P = profiler();
  std::lock_guard<std::mutex> g(P.mu);
  if (P.recs.size() >= 65536) return;
  ProfileRecord r{name, nullptr, nullptr};
  if (hipEventCreate(&r.start) != hipSuccess || hipEventCreate(&r.stop) != hipSuccess) return;
  (void)hipEventRecord(r.start, stream);
  P.recs.push_back(r);
}
void profile_end(hipStream_t stream) {
  Profiler& P = profiler();
  std::lock_guard<std::mutex> g(P.mu);
  if (!P.recs.empty()) (void)hipEventRecord(P.recs.back().stop, stream);
}

template <class T>
__global__ void fill_kernel(T* p, T v, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}

template <class T>
static hipError_t fill_typed(void* dst, const void* value, int64_t n, hipStream_t s) {
  T v;
  memcpy(&v, value, sizeof(T));
  int64_t blocks = (n + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  TCD_LAUNCH("fill_kernel", fill_kernel<T>, dim3((unsigned)blocks), dim3(256), s, static_cast<T*>(dst), v, n);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------
// Temporary-storage pool.  Replaces the per-call cudaMalloc / cudaFree of
// thrust/system/cuda/detail/malloc_and_free.h:53-116.  Blocks are binned by size class:
// powers of two from 256 B to 1 MiB, eight classes per octave above (a request is rounded up by
// at most 12.5 %: the 1.02 GiB of a 2^28-key sort holds 1.125 GiB, not 2).  A free records an
// event on the freeing stream; the
// block is handed to a different stream only once that event has completed, and to the
// same stream immediately (stream order already serialises the two uses).
// ---------------------------------------------------------------------------------------
struct Block {
  void* ptr;
  size_t bytes;
  int device;
  hipStream_t stream;  // stream of the last free
  hipEvent_t event;    // recorded at the last free
};

struct Pool {
  std::mutex mu;
  std::unordered_map<void*, Block> live;              // handed out
  std::unordered_map<uint64_t, std::vector<Block>> cached;  // key: device << 56 | class size
  size_t bytes_held = 0;
};

static Pool& pool() {
  static Pool* p = new Pool();  // never destroyed: the HIP runtime may unload first
  return *p;
}

// the size class of a request: the bytes a block of that class holds
static size_t class_size(size_t bytes) {
  if (bytes <= 256) return 256;
  int top = 63 - __builtin_clzll((unsigned long long)(bytes - 1));  // 2^top < bytes <= 2^(top+1)
  if (top < 20) return (size_t)1 << (top + 1);
  const size_t step = (size_t)1 << (top - 3);  // an eighth of the octave's base
  return (bytes + step - 1) / step * step;
}
static uint64_t class_key(int device, size_t size) { return ((uint64_t)device << 56) | (uint64_t)size; }

}  // namespace tcd

using namespace tcd;

extern "C" int thrust_cdna4_abi_version(void) { return THRUST_CDNA4_ABI_VERSION; }

extern "C" const char* thrust_cdna4_error_string(int code) {
  return hipGetErrorString(static_cast<hipError_t>(code));
}

extern "C" int thrust_cdna4_profile_enable(int on) {
  Profiler& P = profiler();
  std::lock_guard<std::mutex> g(P.mu);
  for (auto& r : P.recs) {
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  P.recs.clear();
  P.on = on != 0;
  return hipSuccess;
}

extern "C" int thrust_cdna4_profile_count(void) {
  Profiler& P = profiler();
  std::lock_guard<std::mutex> g(P.mu);
  return (int)P.recs.size();
}

extern "C" int thrust_cdna4_profile_get(int index, const char** name, float* ms) {
  Profiler& P = profiler();
  ProfileRecord r;
  {
    std::lock_guard<std::mutex> g(P.mu);
    if (index < 0 || index >= (int)P.recs.size() || !name || !ms) return hipErrorInvalidValue;
    r = P.recs[(size_t)index];
  }
  hipError_t e = hipEventSynchronize(r.stop);
  if (e != hipSuccess) return e;
  *name = r.name;
  return hipEventElapsedTime(ms, r.start, r.stop);
}

extern "C" int thrust_cdna4_malloc(void** ptr, size_t bytes, void* stream) {
  if (!ptr) return hipErrorInvalidValue;
  *ptr = nullptr;
  if (bytes == 0) return hipSuccess;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const size_t size = class_size(bytes);
  const uint64_t key = class_key(dev, size);
  hipStream_t s = static_cast<hipStream_t>(stream);
  Pool& P = pool();
  {
    std::lock_guard<std::mutex> g(P.mu);
    auto it = P.cached.find(key);
    if (it != P.cached.end()) {
      auto& v = it->second;
      for (size_t i = v.size(); i-- > 0;) {
        Block b = v[i];
        const bool ready = (b.stream == s) || (hipEventQuery(b.event) == hipSuccess);
        if (ready) {
          v.erase(v.begin() + (long)i);
          P.live[b.ptr] = b;
          *ptr = b.ptr;
          return hipSuccess;
        }
      }
    }
  }
  Block b{};
  b.bytes = size;
  b.device = dev;
  e = hipMalloc(&b.ptr, b.bytes);
  if (e != hipSuccess) {
    // give cached memory back to the driver and retry once
    thrust_cdna4_pool_trim();
    e = hipMalloc(&b.ptr, b.bytes);
    if (e != hipSuccess) {
      (void)hipGetLastError();  // clear the sticky error, as the reference does before throwing
      return e;
    }
  }
  e = hipEventCreateWithFlags(&b.event, hipEventDisableTiming);
  if (e != hipSuccess) {
    (void)hipFree(b.ptr);
    return e;
  }
  std::lock_guard<std::mutex> g(P.mu);
  P.live[b.ptr] = b;
  P.bytes_held += b.bytes;
  *ptr = b.ptr;
  return hipSuccess;
}

extern "C" int thrust_cdna4_free(void* ptr, void* stream) {
  if (!ptr) return hipSuccess;
  Pool& P = pool();
  hipStream_t s = static_cast<hipStream_t>(stream);
  Block b;
  {
    std::lock_guard<std::mutex> g(P.mu);
    auto it = P.live.find(ptr);
    if (it == P.live.end()) return hipErrorInvalidValue;
    b = it->second;
    P.live.erase(it);
  }
  b.stream = s;
  hipError_t e = hipEventRecord(b.event, s);
  if (e != hipSuccess) return e;
  std::lock_guard<std::mutex> g(P.mu);
  P.cached[class_key(b.device, b.bytes)].push_back(b);
  return hipSuccess;
}

extern "C" int thrust_cdna4_pool_trim(void) {
  Pool& P = pool();
  std::vector<Block> victims;
  {
    std::lock_guard<std::mutex> g(P.mu);
    for (auto& kv : P.cached) {
      for (auto& b : kv.second) victims.push_back(b);
      kv.second.clear();
    }
    for (auto& b : victims) P.bytes_held -= b.bytes;
  }
  hipError_t rc = hipSuccess;
  for (auto& b : victims) {
    hipError_t e = hipEventSynchronize(b.event);
    if (e != hipSuccess) rc = e;
    (void)hipEventDestroy(b.event);
    e = hipFree(b.ptr);
    if (e != hipSuccess) rc = e;
  }
  return rc;
}

extern "C" size_t thrust_cdna4_pool_bytes(void) {
  Pool& P = pool();
  std::lock_guard<std::mutex> g(P.mu);
  return P.bytes_held;
}

extern "C" int thrust_cdna4_memcpy_htod(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return hipSuccess;
  return hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream));
}
extern "C" int thrust_cdna4_memcpy_dtoh(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return hipSuccess;
  return hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream));
}
namespace tcd {
// One pinned bounce buffer per host thread, allocated at its first read-back and kept until the
// process ends.
struct PinnedSlot {
  static constexpr size_t kBytes = 4096;
  void* p = nullptr;
  void* get() {
    if (!p && hipHostMalloc(&p, kBytes, hipHostMallocPortable) != hipSuccess) {
      (void)hipGetLastError();
      p = nullptr;
    }
    return p;
  }
};
static thread_local PinnedSlot t_slot;
}  // namespace tcd
extern "C" int thrust_cdna4_read_back(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return hipSuccess;
  if (!dst || !src) return hipErrorInvalidValue;
  hipStream_t s = static_cast<hipStream_t>(stream);
  void* slot = bytes <= tcd::PinnedSlot::kBytes ? tcd::t_slot.get() : nullptr;
  hipError_t e = hipMemcpyAsync(slot ? slot : dst, src, bytes, hipMemcpyDeviceToHost, s);
  if (e != hipSuccess) return (int)e;
  e = hipStreamSynchronize(s);
  if (e != hipSuccess) return (int)e;
  if (slot) std::memcpy(dst, slot, bytes);
  return hipSuccess;
}
// Device-to-device copy: one 16-byte load and store per thread, many small workgroups.  On
// MI355X this plain shape streams faster than longer per-thread loops and than the runtime's
// own copy (about 6 TB/s against 5 TB/s for 1 GiB).
namespace tcd {
__global__ __launch_bounds__(512) void copy16_kernel(const tcd_v4u* __restrict__ src, tcd_v4u* __restrict__ dst,
                                                     size_t nvec) {
  const size_t i = (size_t)blockIdx.x * 512 + threadIdx.x;
  if (i < nvec) dst[i] = src[i];
}

hipError_t copy_async(void* dst, const void* src, size_t bytes, hipStream_t s) {
  if (bytes == 0) return hipSuccess;
  const bool aligned = ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15) == 0;
  const size_t nvec = bytes / 16;
  if (!aligned || bytes < (size_t(1) << 20) || ceil_div((int64_t)nvec, (int64_t)512) > 0x7fffffff)
    return hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s);
  TCD_LAUNCH("copy16_kernel", copy16_kernel, dim3((unsigned)ceil_div((int64_t)nvec, (int64_t)512)), dim3(512), s,
             static_cast<const tcd_v4u*>(src), static_cast<tcd_v4u*>(dst), nvec);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess && (bytes & 15))
    e = hipMemcpyAsync(static_cast<char*>(dst) + nvec * 16, static_cast<const char*>(src) + nvec * 16, bytes & 15,
                       hipMemcpyDeviceToDevice, s);
  return e;
}
}  // namespace tcd

extern "C" int thrust_cdna4_memcpy_dtod(void* dst, const void* src, size_t bytes, void* stream) {
  return (int)tcd::copy_async(dst, src, bytes, static_cast<hipStream_t>(stream));
}

extern "C" int thrust_cdna4_fill(void* dst, const void* value, int elem_bytes, int64_t n, void* stream) {
  if (n < 0 || (n > 0 && (!dst || !value))) return hipErrorInvalidValue;
  if (n == 0) return hipSuccess;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (elem_bytes) {
    case 1: return fill_typed<uint8_t>(dst, value, n, s);
    case 2: return fill_typed<uint16_t>(dst, value, n, s);
    case 4: return fill_typed<uint32_t>(dst, value, n, s);
    case 8: return fill_typed<uint64_t>(dst, value, n, s);
  }
  return hipErrorInvalidValue;
}

namespace tcd {
static std::atomic<int> g_lookback_patience{kDefaultLookbackPatience};
int lookback_patience() { return g_lookback_patience.load(std::memory_order_relaxed); }
}  // namespace tcd
extern "C" int thrust_cdna4_set_lookback_patience(int polls) {
  return tcd::g_lookback_patience.exchange(polls < 0 ? tcd::kDefaultLookbackPatience : polls, std::memory_order_relaxed);
}

namespace tcd {
static std::atomic<int> g_publish_delay{0};
int lookback_test_publish_delay() { return g_publish_delay.load(std::memory_order_relaxed); }
}  // namespace tcd
extern "C" int thrust_cdna4_set_test_publish_delay(int sleeps) {
  if (sleeps < 0) sleeps = 0;
  if (sleeps > 100000) sleeps = 100000;  // bounded: a third of a second at most
  return tcd::g_publish_delay.exchange(sleeps, std::memory_order_relaxed);
}

extern "C" int thrust_cdna4_stream_synchronize(void* stream) {
  return hipStreamSynchronize(static_cast<hipStream_t>(stream));
}

// Streams and events for the asynchronous algorithms.  Streams are non-blocking (they do not
// synchronise with the legacy default stream) and keep the default priority; events carry no
// timing.
extern "C" int thrust_cdna4_stream_create(void** stream) {
  if (!stream) return hipErrorInvalidValue;
  hipStream_t s = nullptr;
  const hipError_t rc = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
  *stream = s;
  return rc;
}
extern "C" int thrust_cdna4_stream_destroy(void* stream) {
  if (!stream) return hipErrorInvalidValue;  // the default stream is not the library's to destroy
  return hipStreamDestroy(static_cast<hipStream_t>(stream));
}
extern "C" int thrust_cdna4_stream_query(void* stream, int* done) {
  if (!done) return hipErrorInvalidValue;
  const hipError_t rc = hipStreamQuery(static_cast<hipStream_t>(stream));
  *done = rc == hipSuccess;
  if (rc == hipErrorNotReady) {
    (void)hipGetLastError();  // not an error: work is still running
    return hipSuccess;
  }
  return rc;
}
extern "C" int thrust_cdna4_event_create(void** event) {
  if (!event) return hipErrorInvalidValue;
  hipEvent_t e = nullptr;
  const hipError_t rc = hipEventCreateWithFlags(&e, hipEventDisableTiming);
  *event = e;
  return rc;
}
extern "C" int thrust_cdna4_event_destroy(void* event) {
  if (!event) return hipErrorInvalidValue;
  return hipEventDestroy(static_cast<hipEvent_t>(event));
}
extern "C" int thrust_cdna4_event_record(void* event, void* stream) {
  if (!event) return hipErrorInvalidValue;
  return hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream));
}
extern "C" int thrust_cdna4_event_query(void* event, int* done) {
  if (!event || !done) return hipErrorInvalidValue;
  const hipError_t rc = hipEventQuery(static_cast<hipEvent_t>(event));
  *done = rc == hipSuccess;
  if (rc == hipErrorNotReady) {
    (void)hipGetLastError();
    return hipSuccess;
  }
  return rc;
}
extern "C" int thrust_cdna4_stream_wait_event(void* stream, void* event) {
  if (!event) return hipErrorInvalidValue;
  return hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0);
}
// Plain device memory from the driver, without the pool: the upstream of user-built pools.
extern "C" int thrust_cdna4_malloc_direct(void** ptr, size_t bytes) {
  if (!ptr) return hipErrorInvalidValue;
  *ptr = nullptr;
  if (bytes == 0) return hipSuccess;
  return hipMalloc(ptr, bytes);
}
extern "C" int thrust_cdna4_free_direct(void* ptr) {
  if (!ptr) return hipSuccess;
  return hipFree(ptr);
}
// Memory that host and device code can both address: managed memory (pages move to whoever
// touches them) or page-locked host memory that the device reaches over the bus.
extern "C" int thrust_cdna4_malloc_universal(void** ptr, size_t bytes, int host_pinned) {
  if (!ptr) return hipErrorInvalidValue;
  *ptr = nullptr;
  if (bytes == 0) return hipSuccess;
  return host_pinned ? hipHostMalloc(ptr, bytes, hipHostMallocDefault) : hipMallocManaged(ptr, bytes, hipMemAttachGlobal);
}
extern "C" int thrust_cdna4_free_universal(void* ptr, int host_pinned) {
  if (!ptr) return hipSuccess;
  return host_pinned ? hipHostFree(ptr) : hipFree(ptr);
}
extern "C" int thrust_cdna4_get_device(int* device) {
  if (!device) return hipErrorInvalidValue;
  return hipGetDevice(device);
}

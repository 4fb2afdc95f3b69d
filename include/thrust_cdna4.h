/*
 * thrust_cdna4.h — C ABI of libthrust_cdna4.so, the gfx950 (MI355X) device system for Thrust.
 *
 * This is the boundary the header-only C++ dispatch layer (include/thrust/system/cdna4/)
 * calls.  Every entry point is `extern "C"`, takes plain pointers and sizes, returns an
 * `int` that is a hipError_t value (0 = success), never throws, and enqueues its work on
 * `stream` (a hipStream_t passed as void*; NULL = the legacy default stream) without
 * waiting for it.  All data pointers are DEVICE pointers owned by the caller.
 *
 * Algorithms follow the two-phase temporary-storage protocol that the reference uses for
 * its own device primitives (thrust/system/cuda/detail/sort.h:330-365,
 * scan.h:80-117, reduce_by_key.h:1012-1031): call once with `temp == NULL` and the entry
 * point only writes the number of bytes it needs to `*temp_bytes`; call again with a
 * device buffer of at least that many bytes (256-byte aligned; an address that is not even a
 * multiple of 8 is refused with an invalid-value error) to run.  Data pointers need the
 * alignment of their element type and no more: a range that starts a few elements into an
 * allocation runs at the same speed as one that starts at it.
 *
 * Semantics are those of the reference's sequential system, which is what its tests
 * compare the device result against:
 *   sort          thrust/system/detail/sequential/stable_radix_sort.inl:43-596, sort.inl:54-105
 *   scan          thrust/system/detail/sequential/scan.h:47-114
 *   scan_by_key   thrust/system/detail/sequential/scan_by_key.h:46-142
 *   reduce_by_key thrust/system/detail/sequential/reduce_by_key.h:43-95
 */
#ifndef THRUST_CDNA4_H
#define THRUST_CDNA4_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define THRUST_CDNA4_ABI_VERSION 1

/* Element types.  The numeric values are part of the ABI. */
typedef enum thrust_cdna4_dtype {
  THRUST_CDNA4_I8 = 0,
  THRUST_CDNA4_U8 = 1,
  THRUST_CDNA4_I16 = 2,
  THRUST_CDNA4_U16 = 3,
  THRUST_CDNA4_I32 = 4,
  THRUST_CDNA4_U32 = 5,
  THRUST_CDNA4_I64 = 6,
  THRUST_CDNA4_U64 = 7,
  THRUST_CDNA4_F32 = 8,
  THRUST_CDNA4_F64 = 9
} thrust_cdna4_dtype;

/* Binary operators of thrust/functional.h that the kernels are specialised on. */
typedef enum thrust_cdna4_op {
  THRUST_CDNA4_PLUS = 0,       /* thrust::plus       */
  THRUST_CDNA4_MULTIPLIES = 1, /* thrust::multiplies */
  THRUST_CDNA4_MAXIMUM = 2,    /* thrust::maximum    */
  THRUST_CDNA4_MINIMUM = 3     /* thrust::minimum    */
} thrust_cdna4_op;

/* Returns THRUST_CDNA4_ABI_VERSION of the loaded library. */
int thrust_cdna4_abi_version(void);

/* Human-readable text for a return code (wraps hipGetErrorString). */
const char* thrust_cdna4_error_string(int code);

/*
 * Stable LSD radix sort of `n` keys in place.  Replaces
 * cuda_cub::__radix_sort::radix_sort<SORT_ITEMS=false> and the
 * cub::DeviceRadixSort::SortKeys / SortKeysDescending calls under it
 * (thrust/system/cuda/detail/sort.h:213-259, :306-380).  The alternate key buffer lives in
 * `temp`, as it does in the reference (:338-343); the result always ends in `keys`.
 * Order: ascending by the reference's RadixEncoder bit order
 * (sequential/stable_radix_sort.inl:43-139) — for floating-point keys that is the total
 * order -NaN < -inf < ... < -0 < +0 < ... < +inf < +NaN.  `descending != 0` gives the
 * order of thrust::greater (sequential/sort.inl:54-75).  n must be < 2^32 - 1.
 * A pass over a digit place at which all keys agree (64-bit keys holding small numbers, constant
 * fields, all keys equal) is skipped on the device; the result is the same, the call is faster.
 * One-byte keys are not moved at all: the sorted sequence is written from their histogram.
 */
int thrust_cdna4_sort_keys(void* temp, size_t* temp_bytes, int key_dtype, void* keys,
                           int64_t n, int descending, void* stream);

/*
 * Stable LSD radix sort of `n` (key, value) pairs in place; values are opaque items of
 * `value_bytes` bytes (1, 2, 4 or 8).  Replaces radix_sort<SORT_ITEMS=true> and
 * cub::DeviceRadixSort::SortPairs / SortPairsDescending
 * (thrust/system/cuda/detail/sort.h:261-304, :306-380).  Equal keys keep their input
 * order, also when `descending != 0` (sequential/sort.inl:78-105).
 */
int thrust_cdna4_sort_pairs(void* temp, size_t* temp_bytes, int key_dtype, void* keys,
                            int value_bytes, void* values, int64_t n, int descending,
                            void* stream);

/*
 * Prefix scan of `n` elements of type `dtype` under `op`.  Replaces
 * cuda_cub::detail::inclusive_scan_n_impl / exclusive_scan_n_impl and cub::DispatchScan
 * (thrust/system/cuda/detail/scan.h:57-204).  `exclusive == 0`: out[i] = in[0] op ... op
 * in[i].  `exclusive != 0`: out[0] = *init, out[i] = *init op in[0] op ... op in[i-1];
 * `init` is a HOST pointer to one element of `dtype` (NULL = value-initialised, the
 * reference's default, scan.h:347-348).  `in == out` is allowed
 * (testing/scan.cu:86-105).  Integer results are bit-exact (two's-complement wraparound);
 * floating-point sums and products are a reassociation of the serial left fold: they differ from
 * it, and from one run to the next (which tile's look-back sees which neighbour's aggregate
 * first depends on timing, and with it the grouping), by rounding only.  Floating-point
 * maximum and minimum select an input value and give the serial fold's bits, NaNs and signed
 * zeros included, in scan, scan_by_key (per segment) and reduce_by_key (per run): maximum
 * (a < b ? b : a) keeps a NaN that starts the fold (element 0, or *init) and skips NaNs met later,
 * and keeps the first of +0 and -0; minimum (a < b ? a : b) restarts at every NaN (the NaN
 * replaces the accumulator, the next element replaces the NaN) and keeps the last of +0 and -0.
 * The price of minimum's restarts: its floating-point instantiations publish one more word per
 * tile and always hand out tiles by ticket.
 */
int thrust_cdna4_scan(void* temp, size_t* temp_bytes, int dtype, int op, int exclusive,
                      const void* in, void* out, int64_t n, const void* init, void* stream);

/*
 * thrust_cdna4_scan for callers that cannot allocate: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference, whose scan
 * always takes caller-provided temporary storage (thrust/system/cuda/detail/scan.h:80-117).  Same
 * arguments, results and kernels as thrust_cdna4_scan without `temp` / `temp_bytes`: the ticket
 * and the tile descriptors live in a fixed array of 256 B + 256 KiB inside the library's device
 * image (one copy per GPU, held until the process ends), whose device address is looked up on the
 * first call on each device; no call allocates or frees memory.  That first call must be made
 * outside a stream capture: under capture on a device whose address is not known yet the call
 * returns hipErrorStreamCaptureUnsupported (900) and launches nothing.  Limit: at most 16384 tiles of 128 KiB, i.e. 2 GiB
 * of input (n <= 2^31 elements of 1 byte, 2^30 of 2 bytes, 2^29 of 4 bytes, 2^28 of 8 bytes;
 * 10922 tiles for minimum over 8-byte floating-point values, whose tiles publish three words);
 * a larger n returns hipErrorOutOfMemory (2) before anything else is looked
 * at, and launches nothing.  All calls on one GPU share the array: calls
 * that overlap in time on one GPU (different streams, or different host threads) race and must
 * be serialised by the caller; back-to-back calls on one stream are fine (each call clears the
 * descriptors it uses with a fill kernel, never hipMemsetAsync).
 */
int thrust_cdna4_scan_static(int dtype, int op, int exclusive, const void* in, void* out,
                             int64_t n, const void* init, void* stream);

/*
 * Segmented prefix scan: segments are maximal runs of consecutive equal keys
 * (thrust::equal_to on adjacent keys).  Replaces inclusive_scan_by_key_n /
 * exclusive_scan_by_key_n and cub::DispatchScanByKey
 * (thrust/system/cuda/detail/scan_by_key.h:69-282).  The exclusive form restarts from
 * `*init` at every segment head (sequential/scan_by_key.h:95-140).  `values == out` is
 * allowed, and so is an `out` that overlaps `keys` (testing/scan_by_key.inclusive.cu:325-334): the
 * keys are then read from a copy in the temporary storage, which is n keys larger for it — make
 * the size query with the pointers of the call.  n must be < 2^32 (32-bit head counts; the reference switches to 64-bit offsets there,
 * thrust/system/cuda/detail/dispatch.h:29-78 — the template layer's kernel templates take over).
 */
int thrust_cdna4_scan_by_key(void* temp, size_t* temp_bytes, int key_dtype, int value_dtype,
                             int op, int exclusive, const void* keys, const void* values,
                             void* out, int64_t n, const void* init, void* stream);

/*
 * Run-length segmented reduction.  Replaces __reduce_by_key::reduce_by_key_dispatch,
 * ReduceByKeyAgent and InitAgent (thrust/system/cuda/detail/reduce_by_key.h:204-1058).
 * For each maximal run of equal consecutive keys writes the run's first key to keys_out
 * and the left-to-right reduction of its values to values_out; writes the number of runs
 * (int64) to the DEVICE location `num_runs_out`, which the caller reads back after
 * synchronising (reduce_by_key.h:1049-1052).  An output may overlap an input it has the element
 * size of or begins at (the compaction only moves to the left); outputs over keys_in make the call
 * read the keys from a copy in the temporary storage, as in scan_by_key.  n must be < 2^32
 * (32-bit run positions; beyond, the template layer's kernel templates take over).
 */
int thrust_cdna4_reduce_by_key(void* temp, size_t* temp_bytes, int key_dtype, int value_dtype,
                               int op, const void* keys_in, const void* values_in,
                               void* keys_out, void* values_out, int64_t* num_runs_out,
                               int64_t n, void* stream);

/*
 * Histogram with `num_bins` equal-width bins over [lower, upper): sample x falls in bin
 * floor((x - lower) * num_bins / (upper - lower)); samples outside the range are not
 * counted.  counts[0..num_bins) are uint32 and are overwritten.  The reference has no such
 * function: this is the device counterpart of the dense-histogram pattern of
 * examples/histogram.cu:60-101 (sort + upper_bound + adjacent_difference), whose result
 * for integer-valued samples with unit-width bins it reproduces.
 */
int thrust_cdna4_histogram_even(void* temp, size_t* temp_bytes, int sample_dtype,
                                const void* samples, int64_t n, uint32_t* counts,
                                int num_bins, double lower, double upper, void* stream);

/*
 * Temporary-storage allocator.  Replaces cuda_cub::malloc / cuda_cub::free
 * (thrust/system/cuda/detail/malloc_and_free.h:53-116), which call cudaMalloc / cudaFree on
 * every algorithm invocation.  Blocks are cached per device in size classes (powers of two up
 * to 1 MiB, eight per octave above: at most 12.5 % more than asked for) and handed back without a
 * driver call; a block freed on one stream is reused on another
 * only after an event recorded at the free has completed.
 */
int thrust_cdna4_malloc(void** ptr, size_t bytes, void* stream);
int thrust_cdna4_free(void* ptr, void* stream);
/* Returns every cached block to the driver (hipFree). */
int thrust_cdna4_pool_trim(void);
/* Bytes currently held by the pool (cached + handed out) on the current device. */
size_t thrust_cdna4_pool_bytes(void);

/* Data movement used by device_vector and cross-system copy
 * (thrust/system/cuda/detail/util.h:142-199, internal/copy_cross_system.h:89-223). */
int thrust_cdna4_memcpy_htod(void* dst, const void* src, size_t bytes, void* stream);
int thrust_cdna4_memcpy_dtoh(void* dst, const void* src, size_t bytes, void* stream);
int thrust_cdna4_memcpy_dtod(void* dst, const void* src, size_t bytes, void* stream);
/* Copies `bytes` from device memory to host memory in stream order and returns when they have
 * arrived: the read-back of a result (a reduction's value, a count of kept elements, one element
 * behind a device_reference; cuda/detail/reduce.h:947-971, get_value.h:39-78).  Small results
 * (up to 4 KiB) travel through a pinned buffer of the calling thread, which spares the staging a
 * copy to pageable memory goes through (14 us instead of 23 us per read-back on MI355X). */
int thrust_cdna4_read_back(void* dst, const void* src, size_t bytes, void* stream);
/* Fills n elements of elem_bytes (1, 2, 4 or 8) with the pattern at HOST pointer `value`
 * (uninitialized_fill / fill for arithmetic types, cuda/detail/fill.h:61-75). */
int thrust_cdna4_fill(void* dst, const void* value, int elem_bytes, int64_t n, void* stream);
int thrust_cdna4_stream_synchronize(void* stream);

/*
 * Streams and events behind thrust::async::* / device_event / device_future
 * (thrust/system/cuda/detail/future.inl:60-300: unique_stream, unique_event, ready(), wait(),
 * depend_on(), record()).  A created stream does not synchronise with the default stream and
 * has the default priority.  stream_query / event_query store 1 in *done when all work submitted
 * to the stream / before the event's record has completed, else 0; work still running is not an
 * error.  (A stream that holds nothing but a wait on an event can keep answering 0 after it
 * has been synchronised; an event recorded behind the wait answers correctly, which is what
 * device_event::ready() polls.)
 */
int thrust_cdna4_stream_create(void** stream);
int thrust_cdna4_stream_destroy(void* stream);
int thrust_cdna4_stream_query(void* stream, int* done);
int thrust_cdna4_event_create(void** event);
int thrust_cdna4_event_destroy(void* event);
int thrust_cdna4_event_record(void* event, void* stream);
int thrust_cdna4_event_query(void* event, int* done);
int thrust_cdna4_stream_wait_event(void* stream, void* event);
/*
 * Device memory straight from the driver (hipMalloc / hipFree), bypassing the pool: the
 * upstream resource of thrust::mr pools built by users
 * (thrust/system/cuda/memory_resource.h:46-100, cuda_memory_resource<cudaMalloc, cudaFree>).
 */
int thrust_cdna4_malloc_direct(void** ptr, size_t bytes);
int thrust_cdna4_free_direct(void* ptr);
/*
 * Memory addressable from host and device code alike: managed memory (host_pinned = 0;
 * thrust/system/cuda/memory_resource.h:118-121, universal_memory_resource over cudaMallocManaged)
 * or page-locked host memory mapped into the device's address space (host_pinned = 1; :122-125,
 * universal_host_pinned_memory_resource over cudaMallocHost).  Free with the same flag.
 */
int thrust_cdna4_malloc_universal(void** ptr, size_t bytes, int host_pinned);
int thrust_cdna4_free_universal(void* ptr, int host_pinned);
/* The device that is current for the calling thread (cudaGetDevice in
 * thrust/system/cuda/detail/per_device_resource.h:46-62). */
int thrust_cdna4_get_device(int* device);

/*
 * Scan, scan_by_key and reduce_by_key chain their tiles by look-back.  When the output does not
 * overlap the input, a tile is the workgroup of the same index and a workgroup never waits
 * unboundedly for another: a tile descriptor that is still missing after `polls` polls is
 * recomputed from the input by the workgroup that needs it.  (With overlapping ranges tiles are
 * handed out by an atomic ticket instead, which makes every wait finite by construction; the
 * reference relies on cub's look-back, thrust/system/cuda/detail/scan.h:57-204.)  Sets the
 * number of polls for later launches and returns the previous value; a negative value restores
 * the default (256); 0 never waits, which the tests use to drive the recomputation path.
 * Results do not depend on it except for the rounding order of floating-point sums.
 */
int thrust_cdna4_set_lookback_patience(int polls);
/*
 * Test knob for that recomputation path; no counterpart in the reference.  Tile 0 of the
 * ticketless scan, scan_by_key and reduce_by_key kernels and of every pass of the sort sleeps `sleeps` times (a few
 * microseconds each, clamped to 100000) before it publishes its descriptor, so that with
 * patience 0 every later tile deterministically finds it missing, also at the second look.
 * Every kernel still runs to completion.  Returns the previous value; 0 (the default) switches
 * it off.
 */
int thrust_cdna4_set_test_publish_delay(int sleeps);

/*
 * Launch profiling.  While enabled, every kernel the library launches is bracketed by HIP
 * events recorded on the launch stream and logged under its kernel name; enable(…) also
 * clears the log.  get() waits for record `index` and returns its name and duration in
 * milliseconds.  This is the counterpart of the reference's compile-time launch log
 * (THRUST_DEBUG_SYNC, thrust/system/cuda/detail/core/agent_launcher.h:523-559); it is what
 * the benchmark uses to time one kernel inside a multi-kernel algorithm.
 */
int thrust_cdna4_profile_enable(int on);
int thrust_cdna4_profile_count(void);
int thrust_cdna4_profile_get(int index, const char** name, float* ms);

/*
 * The outcome of the sort whose temporary storage was `temp` (n items, enqueued on `stream`):
 * waits for the stream and returns hipSuccess, the stream's error, or hipErrorLaunchTimeOut (702)
 * when a wait inside the sort did not end.  Replaces the error path of the reference's
 * synchronous sort, which turns every runtime failure of its kernels into thrust::system_error
 * (thrust/system/cuda/detail/util.h:207-292, throw_on_error after cuda_cub::synchronize).
 *
 * Every wait of the sort's look-back is bounded: a thread that polls a missing tile descriptor
 * about 4 million times (seconds; a wait that ends takes microseconds) gives up and the kernels
 * still run to completion, with keys at wrong positions inside the output.  The sort records
 * that in the first word of its temporary storage, which this call reads; `temp` must still be
 * the storage the sort was given (call this before handing it to anything else).  After a
 * time-out, sorts on that device hand their tiles out from a single counter (the form whose
 * waits rest on nothing but running workgroups) for the rest of the process.
 *
 * The synchronous policies of the template layer (thrust::device, par, par.on(stream)) and
 * thrust_amd.sort call it in place of their synchronisation and throw.  A caller that does not
 * synchronise (par_nosync, or this C ABI used directly) calls it when it does, or reads
 * thrust_cdna4_lookback_timeouts: without one of the two a timed-out sort goes unnoticed.
 * Sorts of up to 4096 items are one workgroup, have no such wait, and use nothing of `temp`.
 */
int thrust_cdna4_sort_status(const void* temp, int64_t n, void* stream);
/*
 * Diagnostics; no counterpart in the reference.  Counts the waits that did not end (see
 * thrust_cdna4_sort_status) per device: blocks until the device is idle and stores the count
 * since the process started; anything but 0 means that some sort's result cannot be trusted.
 */
int thrust_cdna4_lookback_timeouts(unsigned long long* count);
/* The device address of that counter (a 32-bit unsigned word) on the current device, for kernels
 * built outside the library (the template layer's kernel templates add to it when one of their
 * own bounded waits gives up). */
int thrust_cdna4_lookback_timeout_counter(void** device_address);
/*
 * Test knob for that error path; no counterpart in the reference.  The number of polls after
 * which a wait inside the sort gives up (negative: the default, about 4 million); returns the
 * previous value.  With 0 and thrust_cdna4_set_test_publish_delay, tile 0 of a pass publishes
 * late, the tiles that look for it give up at once, every kernel still runs to completion, and
 * thrust_cdna4_sort_status reports the time-out.
 */
int thrust_cdna4_set_test_sort_spin_limit(long long polls);

/*
 * Hardware self-test.  The sort kernels rank keys with returning LDS atomics and rely on the
 * LDS unit serving the lanes of one instruction that hit the same address in lane order
 * (this is what makes the ranking stable, which cub::DeviceRadixSort obtains with warp match
 * operations, thrust/system/cuda/detail/sort.h:213-380).  Runs about 3*10^8 checked atomics
 * on the current device, waits for them, and stores the number of out-of-order results in
 * *mismatches (0 on a conforming device).  The library runs a short form of it by itself (10^7
 * atomics, about 0.1 ms): the first thrust_cdna4_sort_keys / sort_pairs call that does work on a
 * device waits for that check once — the only time a sort call blocks; a call under stream
 * capture leaves it to the next call — and on a device that fails it every sort returns
 * hipErrorNotSupported (801) instead of a result that may be unstable.
 */
int thrust_cdna4_selftest_lds_atomic_order(long long* mismatches, void* stream);

/*
 * Hardware self-test of what the sort's tile assignment relies on for speed.  Consecutive tiles of a
 * pass write the ends of their per-digit runs into the same cache lines; when one XCD processes
 * groups of consecutive tiles its L2 puts those lines together, which is worth 10 % of a pair sort.
 * That form is only used on a device where workgroup i runs on XCD i mod 8 and every XCD starts its
 * next workgroup independently of the others — otherwise a tile could wait for one that cannot start.
 * This call runs the probe that the library runs by itself before its first large sort on a device
 * (about 0.2 ms, workgroups that wait on nothing but the clock) and stores 1 in *grouped when the
 * device behaves that way, else 0 (its workgroups are not spread over 8 XCDs by index), -1 (the XCDs
 * were not seen to be served independently) or -2 (a CU count the probe does not fit); the sort then
 * hands tiles out from one counter in index order, the form that depends on nothing.  A sort call under stream capture never runs the probe.
 * The reference has no counterpart.
 */
int thrust_cdna4_selftest_xcd_dispatch(int* grouped, void* stream);

/* Test knob: non-zero makes every later sort hand its tiles out from one counter (the form used on
 * devices that fail the probe above); returns the previous setting. */
int thrust_cdna4_set_test_sort_plain_tickets(int on);
/* Which form the library has settled on for the current device: 0 not decided yet (no large sort
 * has run outside a stream capture), 1 groups of consecutive tiles per XCD, 2 the single counter
 * (the probe failed, or a wait timed out).  The probe's own verdict is asked for up to three times
 * when it rests on timing alone. */
int thrust_cdna4_sort_tile_assignment(int* form);

#ifdef __cplusplus
}
#endif
#endif /* THRUST_CDNA4_H */

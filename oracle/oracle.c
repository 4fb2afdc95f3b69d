/*
 * oracle.c — CPU restatement of the reference's sequential algorithms for the hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (libthrust_cdna4.so, the C++ dispatch
 * headers) links, loads or calls this file; only tests/, the smoke check and the
 * cpu_baseline leg of bench.py do, as the checker and as the timed CPU baseline.
 *
 * Each function restates, in plain C, the algorithm of the reference's sequential system
 * (what THRUST_DEVICE_SYSTEM_CPP runs and what the reference's own tests compare device
 * results against).  File:line citations are relative to the reference tree.
 *
 * Pinning status (see tests/test_oracle.py):
 *   sort / sort_pairs      pinned: reference KATs (testing/sort.cu:42-75,
 *                          sort_by_key.cu:46-85, example golden outputs), and equality with
 *                          numpy's stable sort on the encoded key for random inputs.
 *   scan                   pinned: testing/scan.cu:25-107 KAT, numpy cumsum (integers).
 *   scan_by_key            pinned: testing/scan_by_key.{inclusive,exclusive}.cu KATs, the
 *                          example golden output, brute force per segment.
 *   reduce_by_key          pinned: testing/reduce_by_key.cu:15-112 KAT, run_length_encoding
 *                          and mode example outputs, brute force per run.
 *   histogram_even         parity unpinned for the real-valued bin mapping (the reference
 *                          has no such function); pinned for unit-width integer bins by the
 *                          histogram example's golden output and numpy.bincount.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* dtype / op codes: identical to include/thrust_cdna4.h */
enum { I8, U8, I16, U16, I32, U32, I64, U64, F32, F64 };
enum { PLUS, MULTIPLIES, MAXIMUM, MINIMUM };

static int dtype_size(int dt) {
  switch (dt) {
    case I8: case U8: return 1;
    case I16: case U16: return 2;
    case I32: case U32: case F32: return 4;
    case I64: case U64: case F64: return 8;
  }
  return 0;
}

/* Key encoding class: 0 = unsigned (identity), 1 = signed (flip sign bit),
 * 2 = floating point (flip all bits of negatives, sign bit of non-negatives).
 * sequential/stable_radix_sort.inl:43-139 (RadixEncoder<T>). */
static int dtype_enc(int dt) {
  switch (dt) {
    case U8: case U16: case U32: case U64: return 0;
    case I8: case I16: case I32: case I64: return 1;
    default: return 2;
  }
}

/* ---------------------------------------------------------------------------------- */
/* Stable LSD radix sort: sequential/stable_radix_sort.inl:225-345 (radix_sort<>).     */
/* One histogram pass over all digits (:262-271), exclusive scan per digit with the    */
/* "one bin holds everything" skip (:274-289), then one stable scatter per digit       */
/* (:292-323), ping-ponging between the two buffers, and a final copy back (:326-).    */
/* The digit width is the reference's choice by key size, values and N                  */
/* (radix_sort_dispatcher, :345-515): it does not change the result of a stable LSD     */
/* sort, but it is what the timed CPU baseline pays for (eight 4-bit passes over 2^24   */
/* four-byte keys per thread, not four 8-bit ones).                                     */
/* ---------------------------------------------------------------------------------- */
static int reference_radix_bits(int key_bytes, int has_values, size_t n) {
  switch (key_bytes) {
    case 1: return 8;                                                   /* :345-372 */
    case 2: return n < ((size_t)1 << (has_values ? 15 : 16)) ? 8 : 16;  /* :375-428 */
    case 4: return n < ((size_t)1 << 22) ? 8 : (has_values ? 3 : 4);    /* :431-473 */
    default: return n < ((size_t)1 << 21) ? 8 : (has_values ? 3 : 4);   /* :476-518 */
  }
}

#define DEFINE_RADIX(W, UT)                                                              \
  static inline UT encode_##W(UT x, int enc) {                                           \
    const UT sign = (UT)((UT)1 << (W - 1));                                              \
    if (enc == 1) return (UT)(x ^ sign);                                                 \
    if (enc == 2) return (UT)(x ^ ((UT)(0 - (UT)(x >> (W - 1))) | sign));                \
    return x;                                                                            \
  }                                                                                      \
  static int radix_sort_##W(UT* keys1, UT* keys2, unsigned char* vals1,                  \
                            unsigned char* vals2, int vb, size_t n, int enc) {           \
    const int bits = reference_radix_bits(W / 8, vb != 0, n);                            \
    const int NH = (W + bits - 1) / bits; /* digits per key (:240) */                    \
    const size_t NB = (size_t)1 << bits;  /* bins per digit */                           \
    const UT mask = (UT)(NB - 1);                                                        \
    size_t* hist = calloc((size_t)NH * NB, sizeof(size_t));                              \
    int skip[64];                                                                        \
    if (!hist) return 1;                                                                 \
    for (size_t i = 0; i < n; i++) {                                                     \
      UT x = encode_##W(keys1[i], enc);                                                  \
      for (int j = 0; j < NH; j++) hist[(size_t)j * NB + ((x >> (bits * j)) & mask)]++;  \
    }                                                                                    \
    for (int j = 0; j < NH; j++) {                                                       \
      size_t sum = 0;                                                                    \
      skip[j] = 0;                                                                       \
      for (size_t b = 0; b < NB; b++) {                                                  \
        size_t c = hist[(size_t)j * NB + b];                                             \
        if (c == n) skip[j] = 1;                                                         \
        hist[(size_t)j * NB + b] = sum;                                                  \
        sum += c;                                                                        \
      }                                                                                  \
    }                                                                                    \
    int flip = 0;                                                                        \
    for (int j = 0; j < NH; j++) {                                                       \
      if (skip[j]) continue;                                                             \
      const UT* src = flip ? keys2 : keys1;                                              \
      UT* dst = flip ? keys1 : keys2;                                                    \
      const unsigned char* vsrc = flip ? vals2 : vals1;                                  \
      unsigned char* vdst = flip ? vals1 : vals2;                                        \
      size_t* h = hist + (size_t)j * NB;                                                 \
      for (size_t i = 0; i < n; i++) {                                                   \
        UT k = src[i];                                                                   \
        size_t pos = h[(encode_##W(k, enc) >> (bits * j)) & mask]++;                     \
        dst[pos] = k;                                                                    \
        switch (vb) {                                                                    \
          case 0: break;                                                                 \
          case 1: vdst[pos] = vsrc[i]; break;                                            \
          case 2: ((uint16_t*)vdst)[pos] = ((const uint16_t*)vsrc)[i]; break;            \
          case 4: ((uint32_t*)vdst)[pos] = ((const uint32_t*)vsrc)[i]; break;            \
          case 8: ((uint64_t*)vdst)[pos] = ((const uint64_t*)vsrc)[i]; break;            \
        }                                                                                \
      }                                                                                  \
      flip = !flip;                                                                      \
    }                                                                                    \
    if (flip) {                                                                          \
      memcpy(keys1, keys2, n * sizeof(UT));                                              \
      if (vb) memcpy(vals1, vals2, n * (size_t)vb);                                      \
    }                                                                                    \
    free(hist);                                                                          \
    return 0;                                                                            \
  }

DEFINE_RADIX(8, uint8_t)
DEFINE_RADIX(16, uint16_t)
DEFINE_RADIX(32, uint32_t)
DEFINE_RADIX(64, uint64_t)

static void reverse_bytes_n(void* p, size_t n, int eb) {
  unsigned char* a = p;
  unsigned char tmp[8];
  for (size_t i = 0, j = n ? n - 1 : 0; i < j; i++, j--) {
    memcpy(tmp, a + i * eb, eb);
    memcpy(a + i * eb, a + j * eb, eb);
    memcpy(a + j * eb, tmp, eb);
  }
}

static int radix_sort_any(int dt, void* keys, void* kalt, void* vals, void* valt, int vb,
                          size_t n) {
  int enc = dtype_enc(dt);
  switch (dtype_size(dt)) {
    case 1: return radix_sort_8(keys, kalt, vals, valt, vb, n, enc);
    case 2: return radix_sort_16(keys, kalt, vals, valt, vb, n, enc);
    case 4: return radix_sort_32(keys, kalt, vals, valt, vb, n, enc);
    case 8: return radix_sort_64(keys, kalt, vals, valt, vb, n, enc);
  }
  return 2;
}

/* sequential/sort.inl:54-75: primitive sort ascending, then reverse when the comparator is
 * thrust::greater. */
int oracle_sort_keys(int dt, void* keys, int64_t n, int descending) {
  int ks = dtype_size(dt);
  if (!ks || n < 0) return 2;
  if (n == 0) return 0;
  void* alt = malloc((size_t)n * ks);
  if (!alt) return 1;
  int rc = radix_sort_any(dt, keys, alt, NULL, NULL, 0, (size_t)n);
  free(alt);
  if (!rc && descending) reverse_bytes_n(keys, (size_t)n, ks);
  return rc;
}

/* sequential/sort.inl:78-105: for thrust::greater reverse keys and values, stable sort
 * ascending, reverse again — so equal keys keep their input order. */
int oracle_sort_pairs(int dt, void* keys, int vb, void* vals, int64_t n, int descending) {
  int ks = dtype_size(dt);
  if (!ks || n < 0 || !(vb == 1 || vb == 2 || vb == 4 || vb == 8)) return 2;
  if (n == 0) return 0;
  void* kalt = malloc((size_t)n * ks);
  void* valt = malloc((size_t)n * vb);
  if (!kalt || !valt) { free(kalt); free(valt); return 1; }
  if (descending) { reverse_bytes_n(keys, (size_t)n, ks); reverse_bytes_n(vals, (size_t)n, vb); }
  int rc = radix_sort_any(dt, keys, kalt, vals, valt, vb, (size_t)n);
  if (descending) { reverse_bytes_n(keys, (size_t)n, ks); reverse_bytes_n(vals, (size_t)n, vb); }
  free(kalt);
  free(valt);
  return rc;
}

/* ---------------------------------------------------------------------------------- */
/* Binary operators: thrust/functional.h plus / multiplies / maximum / minimum.        */
/* Integer arithmetic is done in the unsigned type of the same width so wraparound is   */
/* defined; maximum(a,b) = a < b ? b : a and minimum(a,b) = a < b ? a : b as in the      */
/* reference's functors.                                                               */
/* ---------------------------------------------------------------------------------- */
#define DEFINE_OPS_INT(N, T, UT)                                                         \
  static inline T apply_##N(int op, T a, T b) {                                          \
    switch (op) {                                                                        \
      case PLUS: return (T)((UT)a + (UT)b);                                              \
      case MULTIPLIES: return (T)((UT)a * (UT)b);                                        \
      case MAXIMUM: return a < b ? b : a;                                                \
      default: return a < b ? a : b;                                                     \
    }                                                                                    \
  }
#define DEFINE_OPS_FP(N, T)                                                              \
  static inline T apply_##N(int op, T a, T b) {                                          \
    switch (op) {                                                                        \
      case PLUS: return a + b;                                                           \
      case MULTIPLIES: return a * b;                                                     \
      case MAXIMUM: return a < b ? b : a;                                                \
      default: return a < b ? a : b;                                                     \
    }                                                                                    \
  }
DEFINE_OPS_INT(i8, int8_t, uint8_t)
DEFINE_OPS_INT(u8, uint8_t, uint8_t)
DEFINE_OPS_INT(i16, int16_t, uint16_t)
DEFINE_OPS_INT(u16, uint16_t, uint16_t)
DEFINE_OPS_INT(i32, int32_t, uint32_t)
DEFINE_OPS_INT(u32, uint32_t, uint32_t)
DEFINE_OPS_INT(i64, int64_t, uint64_t)
DEFINE_OPS_INT(u64, uint64_t, uint64_t)
DEFINE_OPS_FP(f32, float)
DEFINE_OPS_FP(f64, double)

/* ---------------------------------------------------------------------------------- */
/* Scan: sequential/scan.h:47-114.  Inclusive accumulates in the input value type       */
/* (:56-72); exclusive accumulates in the init type (:95-111), here the same type, and  */
/* reads in[i] into a temporary before writing out[i] so in == out works.               */
/* ---------------------------------------------------------------------------------- */
#define DEFINE_SCAN(N, T)                                                                \
  static void scan_##N(int op, int exclusive, const T* in, T* out, size_t n, T init) {   \
    if (!n) return;                                                                      \
    if (!exclusive) {                                                                    \
      T sum = in[0];                                                                     \
      out[0] = sum;                                                                      \
      for (size_t i = 1; i < n; i++) out[i] = sum = apply_##N(op, sum, in[i]);           \
    } else {                                                                             \
      T tmp = in[0];                                                                     \
      T sum = init;                                                                      \
      out[0] = sum;                                                                      \
      sum = apply_##N(op, sum, tmp);                                                     \
      for (size_t i = 1; i < n; i++) {                                                   \
        tmp = in[i];                                                                     \
        out[i] = sum;                                                                    \
        sum = apply_##N(op, sum, tmp);                                                   \
      }                                                                                  \
    }                                                                                    \
  }
DEFINE_SCAN(i8, int8_t)
DEFINE_SCAN(u8, uint8_t)
DEFINE_SCAN(i16, int16_t)
DEFINE_SCAN(u16, uint16_t)
DEFINE_SCAN(i32, int32_t)
DEFINE_SCAN(u32, uint32_t)
DEFINE_SCAN(i64, int64_t)
DEFINE_SCAN(u64, uint64_t)
DEFINE_SCAN(f32, float)
DEFINE_SCAN(f64, double)

#define FOR_DTYPE(dt, M, ERR)                                                               \
  switch (dt) {                                                                          \
    case I8: M(i8, int8_t) break;                                                        \
    case U8: M(u8, uint8_t) break;                                                       \
    case I16: M(i16, int16_t) break;                                                     \
    case U16: M(u16, uint16_t) break;                                                    \
    case I32: M(i32, int32_t) break;                                                     \
    case U32: M(u32, uint32_t) break;                                                    \
    case I64: M(i64, int64_t) break;                                                     \
    case U64: M(u64, uint64_t) break;                                                    \
    case F32: M(f32, float) break;                                                       \
    case F64: M(f64, double) break;                                                      \
    default: return ERR;                                                                 \
  }

int oracle_scan(int dt, int op, int exclusive, const void* in, void* out, int64_t n,
                const void* init) {
  if (n < 0 || op < 0 || op > MINIMUM) return 2;
#define M(N, T)                                                                          \
  {                                                                                      \
    T iv = init ? *(const T*)init : (T)0;                                                \
    scan_##N(op, exclusive, (const T*)in, (T*)out, (size_t)n, iv);                       \
  }
  FOR_DTYPE(dt, M, 2)
#undef M
  return 0;
}

/* ---------------------------------------------------------------------------------- */
/* Scan by key: sequential/scan_by_key.h:46-142.  Keys are compared with operator== on  */
/* ADJACENT elements (:75-78, :128-129).  Keys are handled by width for integers and as  */
/* real numbers for floating point (so -0 == +0 and NaN != NaN, as thrust::equal_to).   */
/* ---------------------------------------------------------------------------------- */
static inline int keys_equal(int kdt, const void* keys, size_t i, size_t j) {
  switch (kdt) {
    case I8: case U8: return ((const uint8_t*)keys)[i] == ((const uint8_t*)keys)[j];
    case I16: case U16: return ((const uint16_t*)keys)[i] == ((const uint16_t*)keys)[j];
    case I32: case U32: return ((const uint32_t*)keys)[i] == ((const uint32_t*)keys)[j];
    case I64: case U64: return ((const uint64_t*)keys)[i] == ((const uint64_t*)keys)[j];
    case F32: return ((const float*)keys)[i] == ((const float*)keys)[j];
    default: return ((const double*)keys)[i] == ((const double*)keys)[j];
  }
}

#define DEFINE_SCAN_BY_KEY(N, T)                                                         \
  static void scan_by_key_##N(int kdt, int op, int exclusive, const void* keys,          \
                              const T* vals, T* out, size_t n, T init) {                 \
    if (!n) return;                                                                      \
    if (!exclusive) {                                                                    \
      T prev = vals[0];                                                                  \
      out[0] = prev;                                                                     \
      for (size_t i = 1; i < n; i++) {                                                   \
        if (keys_equal(kdt, keys, i - 1, i))                                             \
          out[i] = prev = apply_##N(op, prev, vals[i]);                                  \
        else                                                                             \
          out[i] = prev = vals[i];                                                       \
      }                                                                                  \
    } else {                                                                             \
      T tmp = vals[0];                                                                   \
      T next = init;                                                                     \
      out[0] = next;                                                                     \
      next = apply_##N(op, next, tmp);                                                   \
      for (size_t i = 1; i < n; i++) {                                                   \
        tmp = vals[i];                                                                   \
        if (!keys_equal(kdt, keys, i - 1, i)) next = init;                               \
        out[i] = next;                                                                   \
        next = apply_##N(op, next, tmp);                                                 \
      }                                                                                  \
    }                                                                                    \
  }
DEFINE_SCAN_BY_KEY(i8, int8_t)
DEFINE_SCAN_BY_KEY(u8, uint8_t)
DEFINE_SCAN_BY_KEY(i16, int16_t)
DEFINE_SCAN_BY_KEY(u16, uint16_t)
DEFINE_SCAN_BY_KEY(i32, int32_t)
DEFINE_SCAN_BY_KEY(u32, uint32_t)
DEFINE_SCAN_BY_KEY(i64, int64_t)
DEFINE_SCAN_BY_KEY(u64, uint64_t)
DEFINE_SCAN_BY_KEY(f32, float)
DEFINE_SCAN_BY_KEY(f64, double)

int oracle_scan_by_key(int kdt, int vdt, int op, int exclusive, const void* keys,
                       const void* vals, void* out, int64_t n, const void* init) {
  if (n < 0 || op < 0 || op > MINIMUM || !dtype_size(kdt)) return 2;
#define M(N, T)                                                                          \
  {                                                                                      \
    T iv = init ? *(const T*)init : (T)0;                                                \
    scan_by_key_##N(kdt, op, exclusive, keys, (const T*)vals, (T*)out, (size_t)n, iv);   \
  }
  FOR_DTYPE(vdt, M, 2)
#undef M
  return 0;
}

/* ---------------------------------------------------------------------------------- */
/* Reduce by key: sequential/reduce_by_key.h:43-95.  Each key is compared with the      */
/* FIRST key of the current run (temp_key, :58, :68), the run's first key is what is     */
/* written (:74), values are folded left to right in the value type (:55, :70).          */
/* Returns the number of runs, or -2 on bad arguments.                                  */
/* ---------------------------------------------------------------------------------- */
#define DEFINE_RBK(N, T)                                                                 \
  static size_t rbk_##N(int kdt, int op, const void* keys, const T* vals, void* kout,    \
                        T* vout, size_t n) {                                             \
    if (!n) return 0;                                                                    \
    int ks = dtype_size(kdt);                                                            \
    size_t r = 0, head = 0;                                                              \
    T acc = vals[0];                                                                     \
    for (size_t i = 1; i < n; i++) {                                                     \
      if (keys_equal(kdt, keys, head, i)) {                                              \
        acc = apply_##N(op, acc, vals[i]);                                               \
      } else {                                                                           \
        memcpy((char*)kout + r * ks, (const char*)keys + head * ks, ks);                 \
        vout[r] = acc;                                                                   \
        r++;                                                                             \
        head = i;                                                                        \
        acc = vals[i];                                                                   \
      }                                                                                  \
    }                                                                                    \
    memcpy((char*)kout + r * ks, (const char*)keys + head * ks, ks);                     \
    vout[r] = acc;                                                                       \
    return r + 1;                                                                        \
  }
DEFINE_RBK(i8, int8_t)
DEFINE_RBK(u8, uint8_t)
DEFINE_RBK(i16, int16_t)
DEFINE_RBK(u16, uint16_t)
DEFINE_RBK(i32, int32_t)
DEFINE_RBK(u32, uint32_t)
DEFINE_RBK(i64, int64_t)
DEFINE_RBK(u64, uint64_t)
DEFINE_RBK(f32, float)
DEFINE_RBK(f64, double)

int64_t oracle_reduce_by_key(int kdt, int vdt, int op, const void* keys, const void* vals,
                             void* kout, void* vout, int64_t n) {
  if (n < 0 || op < 0 || op > MINIMUM || !dtype_size(kdt)) return -2;
  size_t r = 0;
#define M(N, T) r = rbk_##N(kdt, op, keys, (const T*)vals, kout, (T*)vout, (size_t)n);
  FOR_DTYPE(vdt, M, -2)
#undef M
  return (int64_t)r;
}

/* ---------------------------------------------------------------------------------- */
/* Even-bin histogram: a serial counting loop.  The reference has no histogram function; */
/* its example (examples/histogram.cu:60-101) sorts, then takes                         */
/* upper_bound(counting_iterator) and adjacent_difference, which for integer-valued      */
/* samples and unit-width bins gives exactly counts[b] = #{x : x == lower + b}.          */
/* Mapping (this build's definition): x is converted to double; x outside [lower,upper)  */
/* or NaN is dropped; bin = (int)((x - lower) * (num_bins / (upper - lower))), clamped   */
/* to num_bins-1.                                                                       */
/* ---------------------------------------------------------------------------------- */
int oracle_histogram_even(int dt, const void* samples, int64_t n, uint32_t* counts,
                          int num_bins, double lower, double upper) {
  if (n < 0 || num_bins <= 0 || !(upper > lower)) return 2;
  memset(counts, 0, (size_t)num_bins * sizeof(uint32_t));
  const double scale = (double)num_bins / (upper - lower);
#define M(N, T)                                                                          \
  for (int64_t i = 0; i < n; i++) {                                                      \
    double v = (double)((const T*)samples)[i];                                           \
    if (!(v >= lower && v < upper)) continue;                                            \
    int b = (int)((v - lower) * scale);                                                  \
    if (b >= num_bins) b = num_bins - 1;                                                 \
    counts[b]++;                                                                         \
  }
  FOR_DTYPE(dt, M, 2)
#undef M
  return 0;
}

/* ---------------------------------------------------------------------------------- */
/* CPU baseline: the reference's OpenMP sort (thrust/system/omp/detail/sort.inl:100-175) */
/* restated: the range is cut into one tile per thread                                  */
/* (omp/detail/default_decomposition.inl:36-55), each thread sorts its tile with the     */
/* sequential radix sort (:134-137), then log2(threads) rounds of pairwise stable merges */
/* combine neighbouring tiles through a temporary (:48-60, :143-172).  Only unsigned     */
/* and signed integer keys are merged here (the merge compares decoded keys with <, as   */
/* the reference does).  Used only as the timed cpu_baseline of the benchmark.           */
/* ---------------------------------------------------------------------------------- */
#define DEFINE_OMP_SORT(N, T, W)                                                         \
  static void merge_##N(const T* a, size_t na, const T* b, size_t nb, const uint32_t* va, \
                        const uint32_t* vb, T* out, uint32_t* vout) {                    \
    size_t i = 0, j = 0, k = 0;                                                          \
    while (i < na && j < nb) {                                                           \
      if (b[j] < a[i]) { out[k] = b[j]; if (vout) vout[k] = vb[j]; j++; }                \
      else { out[k] = a[i]; if (vout) vout[k] = va[i]; i++; }                            \
      k++;                                                                               \
    }                                                                                    \
    while (i < na) { out[k] = a[i]; if (vout) vout[k] = va[i]; i++; k++; }               \
    while (j < nb) { out[k] = b[j]; if (vout) vout[k] = vb[j]; j++; k++; }               \
  }                                                                                      \
  static int omp_sort_##N(int dt, T* keys, uint32_t* vals, size_t n, int threads) {      \
    T* tk = malloc(n * sizeof(T));                                                       \
    uint32_t* tv = vals ? malloc(n * sizeof(uint32_t)) : NULL;                           \
    if (!tk || (vals && !tv)) { free(tk); free(tv); return 1; }                          \
    size_t* begin = malloc((size_t)(threads + 1) * sizeof(size_t));                      \
    for (int t = 0; t <= threads; t++) begin[t] = n / threads * (size_t)t + ((size_t)t < n % threads ? (size_t)t : n % threads); \
    _Pragma("omp parallel num_threads(threads)")                                         \
    {                                                                                    \
      int t = 0;                                                                         \
      _Pragma("omp for schedule(static, 1)")                                             \
      for (t = 0; t < threads; t++) {                                                    \
        size_t b = begin[t], e = begin[t + 1];                                           \
        radix_sort_##W((void*)(keys + b), (void*)(tk + b),                               \
                       vals ? (unsigned char*)(vals + b) : NULL,                         \
                       vals ? (unsigned char*)(tv + b) : NULL, vals ? 4 : 0, e - b,      \
                       dtype_enc(dt));                                                   \
      }                                                                                  \
    }                                                                                    \
    for (int width = 1; width < threads; width *= 2) {                                   \
      _Pragma("omp parallel for schedule(static, 1) num_threads(threads)")               \
      for (int t = 0; t < threads; t += 2 * width) {                                     \
        int mid = t + width, end = t + 2 * width;                                        \
        if (mid >= threads) continue;                                                    \
        if (end > threads) end = threads;                                                \
        size_t b = begin[t], m = begin[mid], e = begin[end];                             \
        merge_##N(keys + b, m - b, keys + m, e - m, vals ? vals + b : NULL,              \
                  vals ? vals + m : NULL, tk + b, vals ? tv + b : NULL);                 \
        memcpy(keys + b, tk + b, (e - b) * sizeof(T));                                   \
        if (vals) memcpy(vals + b, tv + b, (e - b) * sizeof(uint32_t));                  \
      }                                                                                  \
    }                                                                                    \
    free(begin); free(tk); free(tv);                                                     \
    return 0;                                                                            \
  }
DEFINE_OMP_SORT(u32, uint32_t, 32)
DEFINE_OMP_SORT(i32, int32_t, 32)
DEFINE_OMP_SORT(u64, uint64_t, 64)
DEFINE_OMP_SORT(i64, int64_t, 64)

int oracle_omp_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* vals may be NULL (keys only) or n uint32 values sorted along with the keys. */
int oracle_omp_sort(int dt, void* keys, uint32_t* vals, int64_t n, int threads) {
  if (n < 0) return 2;
  if (threads <= 0) threads = oracle_omp_max_threads();
  if ((int64_t)threads > n) threads = n > 0 ? (int)n : 1;
  switch (dt) {
    case U32: return omp_sort_u32(dt, keys, vals, (size_t)n, threads);
    case I32: return omp_sort_i32(dt, keys, vals, (size_t)n, threads);
    case U64: return omp_sort_u64(dt, keys, vals, (size_t)n, threads);
    case I64: return omp_sort_i64(dt, keys, vals, (size_t)n, threads);
  }
  return 2;
}

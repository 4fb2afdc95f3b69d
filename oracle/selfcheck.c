/* Drives every entry point of the CPU oracle over small inputs of every element type, operator
 * and flag.  Meant to be built with -fsanitize=address,undefined (tests/test_cpp_api_build.py
 * does so): the checks here are only sanity (a sorted result, a count that adds up) — the point is
 * that the sanitizers see every code path of the oracle, which the parity tests trust as their
 * reference.  Test infrastructure like the oracle itself; never linked into the product. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

int oracle_sort_keys(int dt, void* keys, int64_t n, int descending);
int oracle_sort_pairs(int dt, void* keys, int vb, void* vals, int64_t n, int descending);
int oracle_scan(int dt, int op, int exclusive, const void* in, void* out, int64_t n, const void* init);
int oracle_scan_by_key(int kdt, int vdt, int op, int exclusive, const void* keys, const void* vals, void* out,
                       int64_t n, const void* init);
int64_t oracle_reduce_by_key(int kdt, int vdt, int op, const void* keys, const void* vals, void* kout, void* vout,
                             int64_t n);
int oracle_histogram_even(int dt, const void* samples, int64_t n, uint32_t* counts, int num_bins, double lower,
                          double upper);
int oracle_omp_sort(int dt, void* keys, uint32_t* vals, int64_t n, int threads);

enum { I8, U8, I16, U16, I32, U32, I64, U64, F32, F64, NDT };
static const int kSize[NDT] = {1, 1, 2, 2, 4, 4, 8, 8, 4, 8};

static uint64_t state = 88172645463325252ull;
static uint64_t rnd(void) {
  state ^= state << 13;
  state ^= state >> 7;
  state ^= state << 17;
  return state;
}

/* n elements of type dt holding small whole numbers in [-range/2, range/2) (unsigned: [0, range)) */
static void* small_numbers(int dt, int64_t n, int range) {
  char* p = malloc((size_t)(n ? n : 1) * kSize[dt]);
  for (int64_t i = 0; i < n; i++) {
    const int r = (int)(rnd() % (uint64_t)range);
    const int s = r - range / 2;
    switch (dt) {
      case I8: ((int8_t*)p)[i] = (int8_t)s; break;
      case U8: ((uint8_t*)p)[i] = (uint8_t)r; break;
      case I16: ((int16_t*)p)[i] = (int16_t)s; break;
      case U16: ((uint16_t*)p)[i] = (uint16_t)r; break;
      case I32: ((int32_t*)p)[i] = s; break;
      case U32: ((uint32_t*)p)[i] = (uint32_t)r; break;
      case I64: ((int64_t*)p)[i] = s; break;
      case U64: ((uint64_t*)p)[i] = (uint64_t)r; break;
      case F32: ((float*)p)[i] = (float)s; break;
      case F64: ((double*)p)[i] = (double)s; break;
    }
  }
  return p;
}
static void* random_bits(int dt, int64_t n) {
  char* p = malloc((size_t)(n ? n : 1) * kSize[dt]);
  for (int64_t i = 0; i < n * kSize[dt]; i++) p[i] = (char)rnd();
  return p;
}
static double as_double(int dt, const void* p, int64_t i) {
  switch (dt) {
    case I8: return ((const int8_t*)p)[i];
    case U8: return ((const uint8_t*)p)[i];
    case I16: return ((const int16_t*)p)[i];
    case U16: return ((const uint16_t*)p)[i];
    case I32: return ((const int32_t*)p)[i];
    case U32: return ((const uint32_t*)p)[i];
    case I64: return (double)((const int64_t*)p)[i];
    case U64: return (double)((const uint64_t*)p)[i];
    case F32: return ((const float*)p)[i];
    default: return ((const double*)p)[i];
  }
}

static int failures = 0;
#define CHECK(cond, ...)                                     \
  do {                                                       \
    if (!(cond)) {                                           \
      failures++;                                            \
      fprintf(stderr, "selfcheck: " __VA_ARGS__);            \
      fprintf(stderr, " (%s:%d)\n", __FILE__, __LINE__);     \
    }                                                        \
  } while (0)

int main(void) {
  static const int64_t sizes[] = {0, 1, 2, 3, 63, 64, 65, 255, 256, 257, 1000, 4099};
  const int nsizes = (int)(sizeof(sizes) / sizeof(sizes[0]));
  for (int si = 0; si < nsizes; si++) {
    const int64_t n = sizes[si];
    for (int dt = 0; dt < NDT; dt++) {
      /* sort: whole numbers (no NaN patterns, so the order is checkable as doubles) and raw bits */
      for (int desc = 0; desc < 2; desc++) {
        void* k = small_numbers(dt, n, 100);
        CHECK(oracle_sort_keys(dt, k, n, desc) == 0, "sort_keys dt=%d n=%ld", dt, (long)n);
        for (int64_t i = 1; i < n; i++) {
          const double a = as_double(dt, k, i - 1), b = as_double(dt, k, i);
          CHECK(desc ? a >= b : a <= b, "sort_keys order dt=%d n=%ld i=%ld", dt, (long)n, (long)i);
        }
        free(k);
        k = random_bits(dt, n);
        CHECK(oracle_sort_keys(dt, k, n, desc) == 0, "sort_keys bits dt=%d", dt);
        free(k);
        for (int vb = 1; vb <= 8; vb *= 2) {
          k = small_numbers(dt, n, 8);
          void* v = malloc((size_t)(n ? n : 1) * vb);
          for (int64_t i = 0; i < n; i++) {
            const uint64_t pos = (uint64_t)i;
            memcpy((char*)v + i * vb, &pos, (size_t)vb); /* little endian: the low bytes of the position */
          }
          CHECK(oracle_sort_pairs(dt, k, vb, v, n, desc) == 0, "sort_pairs dt=%d vb=%d", dt, vb);
          if (vb >= 2) /* stability: equal keys keep their positions ascending */
            for (int64_t i = 1; i < n; i++) {
              uint64_t p0 = 0, p1 = 0;
              memcpy(&p0, (char*)v + (i - 1) * vb, (size_t)vb);
              memcpy(&p1, (char*)v + i * vb, (size_t)vb);
              if (as_double(dt, k, i - 1) == as_double(dt, k, i))
                CHECK(p0 < p1, "sort_pairs stability dt=%d vb=%d n=%ld i=%ld", dt, vb, (long)n, (long)i);
            }
          free(k);
          free(v);
        }
      }
      /* scans and by-key algorithms: every operator, inclusive and exclusive */
      for (int op = 0; op < 4; op++) {
        void* in = small_numbers(dt, n, op == 1 ? 2 : 10); /* products of 0 / +-1 stay small */
        void* out = malloc((size_t)(n ? n : 1) * kSize[dt]);
        void* init = small_numbers(dt, 1, 4);
        for (int excl = 0; excl < 2; excl++) {
          CHECK(oracle_scan(dt, op, excl, in, out, n, excl ? init : NULL) == 0, "scan dt=%d op=%d", dt, op);
          if (op == 0 && n > 0 && !excl) {
            double sum = 0;
            for (int64_t i = 0; i < n; i++) sum += as_double(dt, in, i);
            if (dt >= I32) CHECK(as_double(dt, out, n - 1) == sum, "scan total dt=%d n=%ld", dt, (long)n);
          }
          CHECK(oracle_scan(dt, op, excl, in, in, n, excl ? init : NULL) == 0, "scan in place dt=%d", dt);
        }
        for (int kdt = 0; kdt < NDT; kdt++) {
          void* keys = small_numbers(kdt, n, 3);
          void* kout = malloc((size_t)(n ? n : 1) * kSize[kdt]);
          for (int excl = 0; excl < 2; excl++)
            CHECK(oracle_scan_by_key(kdt, dt, op, excl, keys, in, out, n, excl ? init : NULL) == 0,
                  "scan_by_key kdt=%d vdt=%d op=%d", kdt, dt, op);
          const int64_t runs = oracle_reduce_by_key(kdt, dt, op, keys, in, kout, out, n);
          int64_t expect = n > 0;
          for (int64_t i = 1; i < n; i++) expect += as_double(kdt, keys, i) != as_double(kdt, keys, i - 1);
          CHECK(runs == expect, "reduce_by_key runs kdt=%d vdt=%d op=%d n=%ld: %ld vs %ld", kdt, dt, op, (long)n,
                (long)runs, (long)expect);
          free(keys);
          free(kout);
        }
        free(in);
        free(out);
        free(init);
      }
      /* histogram: every sample of [0, 100) is counted once, those outside are dropped */
      for (int bins = 1; bins <= 4096; bins *= 16) {
        void* s = small_numbers(dt, n, 120);
        uint32_t* counts = malloc((size_t)bins * sizeof(uint32_t));
        CHECK(oracle_histogram_even(dt, s, n, counts, bins, 0.0, 100.0) == 0, "histogram dt=%d bins=%d", dt, bins);
        int64_t inside = 0, counted = 0;
        for (int64_t i = 0; i < n; i++) inside += as_double(dt, s, i) >= 0.0 && as_double(dt, s, i) < 100.0;
        for (int b = 0; b < bins; b++) counted += counts[b];
        CHECK(inside == counted, "histogram total dt=%d bins=%d n=%ld", dt, bins, (long)n);
        free(s);
        free(counts);
      }
    }
    /* the multi-threaded sort of the CPU baseline */
    static const int omp_types[] = {I32, U32, I64, U64};
    for (int t = 0; t < 4; t++) {
      const int dt = omp_types[t];
      for (int threads = 1; threads <= 5; threads += 2) {
        for (int with_vals = 0; with_vals < 2; with_vals++) {
          void* k = random_bits(dt, n);
          uint32_t* v = malloc((size_t)(n ? n : 1) * sizeof(uint32_t));
          for (int64_t i = 0; i < n; i++) v[i] = (uint32_t)i;
          CHECK(oracle_omp_sort(dt, k, with_vals ? v : NULL, n, threads) == 0, "omp_sort dt=%d", dt);
          for (int64_t i = 1; i < n; i++)
            CHECK(as_double(dt, k, i - 1) <= as_double(dt, k, i), "omp_sort order dt=%d n=%ld", dt, (long)n);
          free(k);
          free(v);
        }
      }
    }
  }
  /* refused arguments */
  CHECK(oracle_sort_keys(99, NULL, 4, 0) == 2, "unknown dtype");
  CHECK(oracle_scan(I32, 7, 0, NULL, NULL, 4, NULL) == 2, "unknown operator");
  CHECK(oracle_reduce_by_key(99, I32, 0, NULL, NULL, NULL, NULL, 4) == -2, "unknown key dtype");
  CHECK(oracle_histogram_even(I32, NULL, 4, NULL, 0, 0.0, 1.0) == 2, "no bins");
  if (failures) {
    fprintf(stderr, "selfcheck: %d failures\n", failures);
    return 1;
  }
  printf("selfcheck: ok\n");
  return 0;
}

// Public C-ABI entry points for scan_by_key and reduce_by_key: select the per-key-width
// build of bykey.hip.
#include "common.h"

#define TCD_DECL(K)                                                                                   \
  extern "C" int tcd_scan_by_key_k##K(void*, size_t*, int, int, int, int, const void*, const void*,   \
                                      void*, int64_t, const void*, void*);                            \
  extern "C" int tcd_reduce_by_key_k##K(void*, size_t*, int, int, int, const void*, const void*,      \
                                        void*, void*, int64_t*, int64_t, void*);
TCD_DECL(1)
TCD_DECL(2)
TCD_DECL(4)
TCD_DECL(8)

// head counts and run positions are 32-bit unsigned: n (hence the number of runs) must fit them
static const int64_t kByKeyMaxN = (int64_t(1) << 32) - 1;

static inline int is_float_dtype(int dt) { return dt == THRUST_CDNA4_F32 || dt == THRUST_CDNA4_F64; }

extern "C" int thrust_cdna4_scan_by_key(void* temp, size_t* temp_bytes, int key_dtype, int value_dtype,
                                        int op, int exclusive, const void* keys, const void* values,
                                        void* out, int64_t n, const void* init, void* stream) {
  if (!temp_bytes || n < 0 || n > kByKeyMaxN || tcd::temp_misaligned(temp) || (n > 0 && temp && (!keys || !values || !out)))
    return hipErrorInvalidValue;
  const int fk = is_float_dtype(key_dtype);
  switch (tcd::dtype_size(key_dtype)) {
    case 1: return tcd_scan_by_key_k1(temp, temp_bytes, fk, value_dtype, op, exclusive, keys, values, out, n, init, stream);
    case 2: return tcd_scan_by_key_k2(temp, temp_bytes, fk, value_dtype, op, exclusive, keys, values, out, n, init, stream);
    case 4: return tcd_scan_by_key_k4(temp, temp_bytes, fk, value_dtype, op, exclusive, keys, values, out, n, init, stream);
    case 8: return tcd_scan_by_key_k8(temp, temp_bytes, fk, value_dtype, op, exclusive, keys, values, out, n, init, stream);
  }
  return hipErrorInvalidValue;
}

extern "C" int thrust_cdna4_reduce_by_key(void* temp, size_t* temp_bytes, int key_dtype, int value_dtype,
                                          int op, const void* keys_in, const void* values_in,
                                          void* keys_out, void* values_out, int64_t* num_runs_out,
                                          int64_t n, void* stream) {
  if (!temp_bytes || n < 0 || n > kByKeyMaxN || tcd::temp_misaligned(temp) ||
      (temp && (!num_runs_out || (n > 0 && (!keys_in || !values_in || !keys_out || !values_out)))))
    return hipErrorInvalidValue;
  const int fk = is_float_dtype(key_dtype);
  switch (tcd::dtype_size(key_dtype)) {
    case 1: return tcd_reduce_by_key_k1(temp, temp_bytes, fk, value_dtype, op, keys_in, values_in, keys_out, values_out, num_runs_out, n, stream);
    case 2: return tcd_reduce_by_key_k2(temp, temp_bytes, fk, value_dtype, op, keys_in, values_in, keys_out, values_out, num_runs_out, n, stream);
    case 4: return tcd_reduce_by_key_k4(temp, temp_bytes, fk, value_dtype, op, keys_in, values_in, keys_out, values_out, num_runs_out, n, stream);
    case 8: return tcd_reduce_by_key_k8(temp, temp_bytes, fk, value_dtype, op, keys_in, values_in, keys_out, values_out, num_runs_out, n, stream);
  }
  return hipErrorInvalidValue;
}

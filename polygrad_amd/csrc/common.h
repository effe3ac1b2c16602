// Shared helpers for the HIP backend: error reporting in the reference's style
// ("polygrad: <area>: message" on stderr, negative int / NULL returns, never
// abort) and a tiny printf-style string builder.
#pragma once
#include <cstdlib>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "polygrad_abi.h"

namespace polyhip {

// Switches that change results (they skip work so that the rest can be timed), and the knobs
// of tuning experiments (a forced tile, pipeline depth, prefetch distance, ...), exist only
// in a measurement build of the library (make MEASURE=1); the default build ignores them.
// What the default build reads from the environment are the switches that the tests use
// for the other leg of a comparison (POLY_HIP_NO_...), the tuning switch POLY_BEAM, and the
// cache and debugging settings.
#ifdef POLY_HIP_MEASUREMENT_BUILD
inline const char *measurement_env(const char *name) { return getenv(name); }
#else
inline const char *measurement_env(const char *) { return nullptr; }
#endif


inline void log_err(const char *area, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  std::fprintf(stderr, "polygrad: %s: ", area);
  std::vfprintf(stderr, fmt, ap);
  std::fprintf(stderr, "\n");
  va_end(ap);
}

inline std::string strf(const char *fmt, ...) {
  va_list ap, ap2;
  va_start(ap, fmt);
  va_copy(ap2, ap);
  int n = std::vsnprintf(nullptr, 0, fmt, ap);
  va_end(ap);
  std::string s((size_t)(n > 0 ? n : 0), '\0');
  if (n > 0) std::vsnprintf(&s[0], (size_t)n + 1, fmt, ap2);
  va_end(ap2);
  return s;
}

// FNV-1a, 64 bit: keys the in-process and on-disk code-object caches.
inline uint64_t fnv1a(const void *data, size_t n, uint64_t h = 1469598103934665603ull) {
  const unsigned char *p = (const unsigned char *)data;
  for (size_t i = 0; i < n; i++) { h ^= p[i]; h *= 1099511628211ull; }
  return h;
}

// Scalar element types, classified from PolyDType (priority, bitsize).
enum DT : int {
  DT_VOID = POLYHIP_DT_VOID, DT_BOOL = POLYHIP_DT_BOOL, DT_I8 = POLYHIP_DT_INT8,
  DT_U8 = POLYHIP_DT_UINT8, DT_I16 = POLYHIP_DT_INT16, DT_U16 = POLYHIP_DT_UINT16,
  DT_I32 = POLYHIP_DT_INT32, DT_U32 = POLYHIP_DT_UINT32, DT_I64 = POLYHIP_DT_INT64,
  DT_U64 = POLYHIP_DT_UINT64, DT_F16 = POLYHIP_DT_FLOAT16, DT_BF16 = POLYHIP_DT_BFLOAT16,
  DT_F32 = POLYHIP_DT_FLOAT32, DT_F64 = POLYHIP_DT_FLOAT64, DT_INDEX = POLYHIP_DT_INDEX,
  DT_BAD = -1
};

inline DT classify_dtype(const PolyDType &d) {
  // Vector dtypes carry count*bitsize; scalar bitsize is bitsize / count.
  int bits = d.count > 1 ? d.bitsize / d.count : d.bitsize;
  switch (d.priority) {
    case -1: return bits == 0 ? DT_VOID : DT_INDEX;
    case 0: return DT_BOOL;
    case 1: return DT_I8;
    case 2: return DT_U8;
    case 3: return DT_I16;
    case 4: return DT_U16;
    case 5: return DT_I32;
    case 6: return DT_U32;
    case 7: return DT_I64;
    case 8: return DT_U64;
    case 11: return DT_F16;
    case 12: return DT_BF16;
    case 13: return DT_F32;
    case 14: return DT_F64;
    default: return DT_BAD;
  }
}

inline int dt_size(DT t) {
  switch (t) {
    case DT_BOOL: case DT_I8: case DT_U8: return 1;
    case DT_I16: case DT_U16: case DT_F16: case DT_BF16: return 2;
    case DT_I32: case DT_U32: case DT_F32: case DT_INDEX: return 4;
    case DT_I64: case DT_U64: case DT_F64: return 8;
    default: return 0;
  }
}
inline bool dt_is_float(DT t) { return t == DT_F16 || t == DT_BF16 || t == DT_F32 || t == DT_F64; }
inline bool dt_is_int(DT t) { return (t >= DT_I8 && t <= DT_U64) || t == DT_INDEX; }
inline bool dt_is_unsigned(DT t) { return t == DT_U8 || t == DT_U16 || t == DT_U32 || t == DT_U64; }

// HIP C spelling of each scalar type.
inline const char *dt_cname(DT t) {
  switch (t) {
    case DT_BOOL: return "bool";
    case DT_I8: return "signed char";
    case DT_U8: return "unsigned char";
    case DT_I16: return "short";
    case DT_U16: return "unsigned short";
    case DT_I32: case DT_INDEX: return "int";
    case DT_U32: return "unsigned int";
    case DT_I64: return "long long";
    case DT_U64: return "unsigned long long";
    case DT_F16: return "_Float16";
    case DT_BF16: return "__bf16";
    case DT_F32: return "float";
    case DT_F64: return "double";
    default: return "void";
  }
}

}  // namespace polyhip

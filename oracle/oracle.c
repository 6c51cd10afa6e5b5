/*
 * CPU oracle for the Aluminum combine hot path.  TEST INFRASTRUCTURE ONLY:
 * the checker for the GPU library, never a fallback for it.  See oracle.h for
 * what each function restates and what pins it.
 */
#include "oracle.h"

#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------ */
/* dtype table                                                              */
/* ------------------------------------------------------------------------ */

size_t alo_dtype_size(int dtype) {
  switch (dtype) {
  case ALO_I8: case ALO_U8: return 1;
  case ALO_I16: case ALO_U16: case ALO_F16: case ALO_BF16: return 2;
  case ALO_I32: case ALO_U32: case ALO_F32: return 4;
  case ALO_I64: case ALO_U64: case ALO_F64: return 8;
  default: return 0;
  }
}

static int is_float_dtype(int dtype) {
  return dtype == ALO_F16 || dtype == ALO_BF16 || dtype == ALO_F32 ||
         dtype == ALO_F64;
}

/* include/aluminum/mpi/utils.hpp:169-233: the generic map accepts sum..bxor;
 * the __half / bfloat specialisations accept only sum, prod, min, max.  MPI
 * itself defines the logical and bitwise ops for integer types only, so
 * fp32/fp64 with them is an error at the MPI call.  avg exists on the
 * reference's NCCL path only (include/aluminum/nccl_impl.hpp:176); the MPI and
 * host-transfer backends throw on it (mpi/utils.hpp:192-194).  Here it is
 * defined for every type as the sum followed by alo_divide. */
int alo_check_op(int dtype, int op) {
  if (alo_dtype_size(dtype) == 0) return 2;
  if (op < ALO_SUM || op > ALO_AVG) return 1;
  if (is_float_dtype(dtype) && op > ALO_MAX && op != ALO_AVG) return 1;
  return 0;
}

int alo_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void alo_set_num_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* ------------------------------------------------------------------------ */
/* 16-bit float conversions                                                 */
/* ------------------------------------------------------------------------ */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* __bfloat162float: the bf16 pattern is the top half of the fp32 pattern. */
float alo_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* __float2bfloat16 (src/mpi_impl.cpp:110): round to nearest, ties to even.
 * A NaN stays a NaN: quiet bit set, upper payload bits kept. */
uint16_t alo_f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* __half2float: exact widening, subnormals normalised. */
float alo_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0x1fu) /* inf, or NaN made quiet as a hardware conversion does */
    return bits_f32(sign | 0x7f800000u | (man ? 0x00400000u : 0u) | (man << 13));
  if (exp == 0) {
    if (man == 0) return bits_f32(sign);
    int e = -1;
    do { man <<= 1; e++; } while (!(man & 0x400u));
    man &= 0x3ffu;
    return bits_f32(sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13));
  }
  return bits_f32(sign | ((exp + 127 - 15) << 23) | (man << 13));
}

/* __float2half (src/mpi_impl.cpp:66): round to nearest, ties to even, with
 * gradual underflow and overflow to infinity. */
uint16_t alo_f32_to_f16(float f) {
  uint32_t u = f32_bits(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) /* NaN: quiet, keep upper payload */
    return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu));
  if (a >= 0x47800000u) { /* |f| >= 65536 (incl. inf) -> inf; 65520..65536 handled below */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (a >= 0x38800000u) { /* normal half range: |f| >= 2^-14 */
    uint32_t r = a - 0x38000000u; /* rebias exponent by 112 */
    uint32_t lsb = (r >> 13) & 1u;
    r += 0xfffu + lsb;
    return (uint16_t)(sign | (r >> 13)); /* may carry into exponent / infinity: correct */
  }
  if (a < 0x33000000u) return sign; /* |f| < 2^-25 -> 0 (2^-25 itself ties to even 0 below) */
  {
    /* subnormal half: value = man * 2^-24 */
    uint32_t e = a >> 23;               /* 102..112 */
    uint32_t m = (a & 0x7fffffu) | 0x800000u;
    uint32_t shift = 126u - e;          /* 14..24 : m >> shift gives units of 2^-24 */
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1u);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
  }
}

void alo_f32_to_bf16_array(uint16_t *dst, const float *src, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) dst[i] = alo_f32_to_bf16(src[i]);
}
void alo_f32_to_f16_array(uint16_t *dst, const float *src, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) dst[i] = alo_f32_to_f16(src[i]);
}
void alo_bf16_to_f32_array(float *dst, const uint16_t *src, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) dst[i] = alo_bf16_to_f32(src[i]);
}
void alo_f16_to_f32_array(float *dst, const uint16_t *src, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) dst[i] = alo_f16_to_f32(src[i]);
}

/* ------------------------------------------------------------------------ */
/* Counter-based input generator                                            */
/* ------------------------------------------------------------------------ */

#define ALO_GAMMA 0x9E3779B97F4A7C15ull

static inline uint64_t fin64(uint64_t z) {
  z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ull;
  z ^= z >> 27; z *= 0x94D049BB133111EBull;
  z ^= z >> 31;
  return z;
}

uint64_t alo_mix64(uint64_t seed, uint64_t idx) {
  return fin64(fin64(seed + ALO_GAMMA) + (idx + 1) * ALO_GAMMA);
}

/* Sum of the twelve 16-bit fields of three chained 64-bit words. */
static inline uint32_t ih12_sum(uint64_t b0) {
  uint64_t b1 = fin64(b0 + ALO_GAMMA), b2 = fin64(b1 + ALO_GAMMA);
  uint32_t s = 0;
  for (int k = 0; k < 4; k++) {
    s += (uint32_t)((b0 >> (16 * k)) & 0xffffu);
    s += (uint32_t)((b1 >> (16 * k)) & 0xffffu);
    s += (uint32_t)((b2 >> (16 * k)) & 0xffffu);
  }
  return s;
}

/* Real-valued draws are made in fp64 (every operation below is a single
 * correctly rounded IEEE operation, so host and device agree bit for bit) and
 * narrowed once, round-to-nearest-even, for the narrower types.  The uniform
 * draws keep full significands at every magnitude, so that different
 * summation orders really do round differently. */
static inline double gen_f64(uint64_t bits, int dist) {
  switch (dist) {
  case ALO_DIST_UNIFORM_09_11: {
    double u = (double)(bits >> 11) * 0x1p-53; /* exact */
    double t = u * 0.2;                        /* rounded product */
    return 0.9 + t;                            /* rounded sum, no fma */
  }
  case ALO_DIST_UNIFORM_01: return (double)(bits >> 11) * 0x1p-53;
  case ALO_DIST_BOOL01: return (double)(bits >> 63);
  case ALO_DIST_NORMAL: return (double)ih12_sum(bits) * 0x1p-16 - 6.0;
  case ALO_DIST_SMALLINT: return (double)((int)(bits >> 60) - 8);
  default:
    /* one rounding (int64 -> fp64, nearest-even), then an exact scaling */
    return (double)(int64_t)bits * 0x1p-63;
  }
}

static inline float gen_f32(uint64_t bits, int dist) {
  return (float)gen_f64(bits, dist);
}

static inline uint64_t gen_int(uint64_t bits, int dist, int is_signed) {
  switch (dist) {
  case ALO_DIST_FULLRANGE: return bits;
  case ALO_DIST_BOOL01: return bits >> 63;
  default:
    return is_signed ? (uint64_t)((int64_t)(bits >> 60) - 8) : (bits >> 60);
  }
}

static void fill_range(void *dst, size_t n, int dtype, int dist, uint64_t seed,
                       uint64_t idx0) {
  for (size_t i = 0; i < n; i++) {
    uint64_t bits = alo_mix64(seed, idx0 + i);
    switch (dtype) {
    case ALO_I8: ((int8_t *)dst)[i] = (int8_t)gen_int(bits, dist, 1); break;
    case ALO_U8: ((uint8_t *)dst)[i] = (uint8_t)gen_int(bits, dist, 0); break;
    case ALO_I16: ((int16_t *)dst)[i] = (int16_t)gen_int(bits, dist, 1); break;
    case ALO_U16: ((uint16_t *)dst)[i] = (uint16_t)gen_int(bits, dist, 0); break;
    case ALO_I32: ((int32_t *)dst)[i] = (int32_t)gen_int(bits, dist, 1); break;
    case ALO_U32: ((uint32_t *)dst)[i] = (uint32_t)gen_int(bits, dist, 0); break;
    case ALO_I64: ((int64_t *)dst)[i] = (int64_t)gen_int(bits, dist, 1); break;
    case ALO_U64: ((uint64_t *)dst)[i] = gen_int(bits, dist, 0); break;
    case ALO_F16: ((uint16_t *)dst)[i] = alo_f32_to_f16(gen_f32(bits, dist)); break;
    case ALO_BF16: ((uint16_t *)dst)[i] = alo_f32_to_bf16(gen_f32(bits, dist)); break;
    case ALO_F32: ((float *)dst)[i] = gen_f32(bits, dist); break;
    case ALO_F64: ((double *)dst)[i] = gen_f64(bits, dist); break;
    default: break;
    }
  }
}

void alo_fill(void *dst, size_t n, int dtype, int dist, uint64_t seed,
              uint64_t idx0) {
  const size_t es = alo_dtype_size(dtype);
  const size_t tile = 1u << 14;
  const size_t ntiles = (n + tile - 1) / tile;
  if (es == 0) return;
#pragma omp parallel for schedule(static)
  for (size_t t = 0; t < ntiles; t++) {
    size_t lo = t * tile, len = n - lo < tile ? n - lo : tile;
    fill_range((char *)dst + lo * es, len, dtype, dist, seed, idx0 + lo);
  }
}

/* ------------------------------------------------------------------------ */
/* The pairwise step: inout[i] = in[i] OP inout[i]                          */
/* ------------------------------------------------------------------------ */

/* Integers.  a = invec element, b = inoutvec element.  Sum and product wrap
 * (computed unsigned so the oracle itself has no undefined behaviour). */
#define DEF_INT_STEP(NAME, T)                                                   \
  static int step_##NAME(T *b, const T *a, size_t n, int op) {                  \
    size_t i;                                                                   \
    switch (op) {                                                               \
    case ALO_SUM: /* and avg: the sum comes first */                            \
    case ALO_AVG: for (i = 0; i < n; i++) b[i] = (T)((uint64_t)a[i] + (uint64_t)b[i]); break; \
    case ALO_PROD: for (i = 0; i < n; i++) b[i] = (T)((uint64_t)a[i] * (uint64_t)b[i]); break; \
    case ALO_MIN: for (i = 0; i < n; i++) b[i] = (b[i] < a[i]) ? b[i] : a[i]; break; \
    case ALO_MAX: for (i = 0; i < n; i++) b[i] = (b[i] > a[i]) ? b[i] : a[i]; break; \
    case ALO_LOR: for (i = 0; i < n; i++) b[i] = (T)(a[i] || b[i]); break;      \
    case ALO_LAND: for (i = 0; i < n; i++) b[i] = (T)(a[i] && b[i]); break;     \
    case ALO_LXOR: for (i = 0; i < n; i++) b[i] = (T)((a[i] && !b[i]) || (!a[i] && b[i])); break; \
    case ALO_BOR: for (i = 0; i < n; i++) b[i] = (T)(a[i] | b[i]); break;       \
    case ALO_BAND: for (i = 0; i < n; i++) b[i] = (T)(a[i] & b[i]); break;      \
    case ALO_BXOR: for (i = 0; i < n; i++) b[i] = (T)(a[i] ^ b[i]); break;      \
    default: return 1;                                                          \
    }                                                                           \
    return 0;                                                                   \
  }

DEF_INT_STEP(i8, int8_t)
DEF_INT_STEP(u8, uint8_t)
DEF_INT_STEP(i16, int16_t)
DEF_INT_STEP(u16, uint16_t)
DEF_INT_STEP(i32, int32_t)
DEF_INT_STEP(u32, uint32_t)
DEF_INT_STEP(i64, int64_t)
DEF_INT_STEP(u64, uint64_t)

/* fp32 / fp64: the MPI predefined ops, inoutvec[i] = OP(inoutvec[i], invec[i]):
 * MIN(x, y) is (x < y) ? x : y and MAX(x, y) is (x > y) ? x : y, so a tie or a
 * NaN on either side yields the invec element. */
#define DEF_FP_STEP(NAME, T)                                                    \
  static int step_##NAME(T *b, const T *a, size_t n, int op) {                  \
    size_t i;                                                                   \
    switch (op) {                                                               \
    case ALO_SUM: case ALO_AVG: for (i = 0; i < n; i++) b[i] = a[i] + b[i]; break; \
    case ALO_PROD: for (i = 0; i < n; i++) b[i] = a[i] * b[i]; break;           \
    case ALO_MIN: for (i = 0; i < n; i++) b[i] = (b[i] < a[i]) ? b[i] : a[i]; break; \
    case ALO_MAX: for (i = 0; i < n; i++) b[i] = (b[i] > a[i]) ? b[i] : a[i]; break; \
    default: return 1;                                                          \
    }                                                                           \
    return 0;                                                                   \
  }

DEF_FP_STEP(f32, float)
DEF_FP_STEP(f64, double)

/* fp16 / bf16: src/mpi_impl.cpp:61-145.  std::min(x, y) is (y < x) ? y : x
 * and std::max(x, y) is (x < y) ? y : x, called with x = float(invec[i]),
 * y = float(inoutvec[i]); the chosen fp32 value is narrowed again. */
#define DEF_H_STEP(NAME, WIDEN, NARROW)                                         \
  static int step_##NAME(uint16_t *b, const uint16_t *a, size_t n, int op) {    \
    size_t i;                                                                   \
    switch (op) {                                                               \
    case ALO_SUM: case ALO_AVG: for (i = 0; i < n; i++) b[i] = NARROW(WIDEN(a[i]) + WIDEN(b[i])); break; \
    case ALO_PROD: for (i = 0; i < n; i++) b[i] = NARROW(WIDEN(a[i]) * WIDEN(b[i])); break; \
    case ALO_MIN: for (i = 0; i < n; i++) { float x = WIDEN(a[i]), y = WIDEN(b[i]); b[i] = NARROW((y < x) ? y : x); } break; \
    case ALO_MAX: for (i = 0; i < n; i++) { float x = WIDEN(a[i]), y = WIDEN(b[i]); b[i] = NARROW((x < y) ? y : x); } break; \
    default: return 1;                                                          \
    }                                                                           \
    return 0;                                                                   \
  }

DEF_H_STEP(f16, alo_f16_to_f32, alo_f32_to_f16)
DEF_H_STEP(bf16, alo_bf16_to_f32, alo_f32_to_bf16)

static int step_serial(void *inout, const void *in, size_t n, int dtype, int op) {
  switch (dtype) {
  case ALO_I8: return step_i8((int8_t *)inout, (const int8_t *)in, n, op);
  case ALO_U8: return step_u8((uint8_t *)inout, (const uint8_t *)in, n, op);
  case ALO_I16: return step_i16((int16_t *)inout, (const int16_t *)in, n, op);
  case ALO_U16: return step_u16((uint16_t *)inout, (const uint16_t *)in, n, op);
  case ALO_I32: return step_i32((int32_t *)inout, (const int32_t *)in, n, op);
  case ALO_U32: return step_u32((uint32_t *)inout, (const uint32_t *)in, n, op);
  case ALO_I64: return step_i64((int64_t *)inout, (const int64_t *)in, n, op);
  case ALO_U64: return step_u64((uint64_t *)inout, (const uint64_t *)in, n, op);
  case ALO_F16: return step_f16((uint16_t *)inout, (const uint16_t *)in, n, op);
  case ALO_BF16: return step_bf16((uint16_t *)inout, (const uint16_t *)in, n, op);
  case ALO_F32: return step_f32((float *)inout, (const float *)in, n, op);
  case ALO_F64: return step_f64((double *)inout, (const double *)in, n, op);
  default: return 2;
  }
}

#define ALO_TILE 4096u

int alo_step(void *inout, const void *in, size_t n, int dtype, int op) {
  const size_t es = alo_dtype_size(dtype);
  int rc = alo_check_op(dtype, op);
  if (rc) return rc;
  const size_t ntiles = (n + ALO_TILE - 1) / ALO_TILE;
#pragma omp parallel for schedule(static)
  for (size_t t = 0; t < ntiles; t++) {
    size_t lo = t * ALO_TILE, len = n - lo < ALO_TILE ? n - lo : ALO_TILE;
    step_serial((char *)inout + lo * es, (const char *)in + lo * es, len, dtype, op);
  }
  return 0;
}

/* The division that ends an avg: x[i] /= ranks in the element type's own
 * arithmetic.  fp32 / fp64: IEEE division.  fp16 / bf16: widen, fp32 division,
 * narrow (one more step of the rule of src/mpi_impl.cpp:61-145).  Integers: C
 * division, which truncates toward zero. */
static void divide_serial(void *x, size_t n, int dtype, int ranks) {
  size_t i;
  switch (dtype) {
  case ALO_I8: { int8_t *p = (int8_t *)x; for (i = 0; i < n; i++) p[i] = (int8_t)(p[i] / ranks); } break;
  case ALO_U8: { uint8_t *p = (uint8_t *)x; for (i = 0; i < n; i++) p[i] = (uint8_t)(p[i] / ranks); } break;
  case ALO_I16: { int16_t *p = (int16_t *)x; for (i = 0; i < n; i++) p[i] = (int16_t)(p[i] / ranks); } break;
  case ALO_U16: { uint16_t *p = (uint16_t *)x; for (i = 0; i < n; i++) p[i] = (uint16_t)(p[i] / ranks); } break;
  case ALO_I32: { int32_t *p = (int32_t *)x; for (i = 0; i < n; i++) p[i] = p[i] / (int32_t)ranks; } break;
  case ALO_U32: { uint32_t *p = (uint32_t *)x; for (i = 0; i < n; i++) p[i] = p[i] / (uint32_t)ranks; } break;
  case ALO_I64: { int64_t *p = (int64_t *)x; for (i = 0; i < n; i++) p[i] = p[i] / (int64_t)ranks; } break;
  case ALO_U64: { uint64_t *p = (uint64_t *)x; for (i = 0; i < n; i++) p[i] = p[i] / (uint64_t)ranks; } break;
  case ALO_F16: { uint16_t *p = (uint16_t *)x; for (i = 0; i < n; i++) p[i] = alo_f32_to_f16(alo_f16_to_f32(p[i]) / (float)ranks); } break;
  case ALO_BF16: { uint16_t *p = (uint16_t *)x; for (i = 0; i < n; i++) p[i] = alo_f32_to_bf16(alo_bf16_to_f32(p[i]) / (float)ranks); } break;
  case ALO_F32: { float *p = (float *)x; for (i = 0; i < n; i++) p[i] = p[i] / (float)ranks; } break;
  case ALO_F64: { double *p = (double *)x; for (i = 0; i < n; i++) p[i] = p[i] / (double)ranks; } break;
  default: break;
  }
}

int alo_divide(void *x, size_t n, int dtype, int ranks) {
  const size_t es = alo_dtype_size(dtype);
  if (es == 0) return 2;
  if (ranks < 1) return 4;
  const size_t ntiles = (n + ALO_TILE - 1) / ALO_TILE;
#pragma omp parallel for schedule(static)
  for (size_t t = 0; t < ntiles; t++) {
    size_t lo = t * ALO_TILE, len = n - lo < ALO_TILE ? n - lo : ALO_TILE;
    divide_serial((char *)x + lo * es, len, dtype, ranks);
  }
  return 0;
}

/* ------------------------------------------------------------------------ */
/* Named orders as schedules of pairwise steps                              */
/* ------------------------------------------------------------------------ */

static int floor_pow2(int p) { int q = 1; while (2 * q <= p) q *= 2; return q; }

int alo_schedule(int P, int order, int start, int *pairs, int *result) {
  int np = 0;
  if (P < 1 || P > 1024) return -1;
  if (start < 0 || start >= P) return -1;
  switch (order) {
  case ALO_ORDER_RANK_ASC:
    for (int k = 1; k < P; k++) { pairs[2 * np] = 0; pairs[2 * np + 1] = k; np++; }
    *result = 0;
    return np;
  case ALO_ORDER_PAIRWISE_DESC:
    /* rank s keeps its own block as inoutvec and folds in the block received
     * from rank s-1, s-2, ... */
    for (int k = 1; k < P; k++) {
      pairs[2 * np] = start; pairs[2 * np + 1] = (start - k + P) % P; np++;
    }
    *result = start;
    return np;
  case ALO_ORDER_RING: {
    /* the partial travels: rank s+k receives it (invec) and folds it into
     * its own contribution (inoutvec) */
    int cur = start;
    for (int k = 1; k < P; k++) {
      int nxt = (start + k) % P;
      pairs[2 * np] = nxt; pairs[2 * np + 1] = cur; np++;
      cur = nxt;
    }
    *result = cur;
    return np;
  }
  case ALO_ORDER_TREE_BINOMIAL:
    /* binomial reduce to rank `start`, over ranks counted from it with wrap:
     * at distance d every relative rank that is a multiple of 2d folds in the
     * partial of relative rank + d, if that rank exists */
    for (int d = 1; d < P; d *= 2)
      for (int i = 0; i + d < P; i += 2 * d) {
        pairs[2 * np] = (i + start) % P; pairs[2 * np + 1] = (i + d + start) % P; np++;
      }
    *result = start;
    return np;
  case ALO_ORDER_TREE_RSG:
  case ALO_ORDER_TREE_RSG_SPREAD: {
    /* Reduce-scatter by recursive halving of the data at distance 1, 2, 4, ...
     * followed by a gather.  Non-power-of-two P: the odd ranks among the first
     * 2*rem send to the even rank below them, which keeps the result.  The
     * survivors then pair at distance d = 1, 2, 4, ...; of a pair, the one
     * whose bit d equals that bit of `start` keeps the result.  `start` is the
     * survivor that ends up owning the block the element lies in (see
     * alo_rsg_owner); only survivors that agree with it below bit d still
     * hold a partial of that block. */
    int pof2 = floor_pow2(P), rem = P - pof2;
    if (start >= pof2) return -1;
    int *L = (int *)malloc(sizeof(int) * (size_t)pof2);
    if (!L) return -1;
    for (int j = 0; j < rem; j++) {
      pairs[2 * np] = 2 * j; pairs[2 * np + 1] = 2 * j + 1; np++;
      L[j] = 2 * j;
    }
    for (int j = rem; j < pof2; j++) L[j] = j + rem;
    for (int d = 1; d < pof2; d *= 2)
      for (int i = 0; i < pof2; i++) {
        if ((i & d) || ((i ^ start) & (d - 1))) continue; /* i: lower of a pair of holders */
        int keep = (start & d) ? (i | d) : i, other = (start & d) ? i : (i | d);
        pairs[2 * np] = L[keep]; pairs[2 * np + 1] = L[other]; np++;
      }
    *result = L[start];
    free(L);
    return np;
  }
  case ALO_ORDER_TREE_DBL:
  case ALO_ORDER_TREE_HALV: {
    /* Non-power-of-two P: the first 2*rem ranks fold pairwise (even rank
     * sends to the odd rank above it, which keeps the result), leaving a
     * power-of-two set of survivors. */
    int pof2 = floor_pow2(P), rem = P - pof2;
    int *L = (int *)malloc(sizeof(int) * (size_t)pof2);
    if (!L) return -1;
    for (int j = 0; j < rem; j++) {
      pairs[2 * np] = 2 * j + 1; pairs[2 * np + 1] = 2 * j; np++;
      L[j] = 2 * j + 1;
    }
    for (int j = rem; j < pof2; j++) L[j] = j + rem;
    if (order == ALO_ORDER_TREE_DBL) {
      for (int d = 1; d < pof2; d *= 2)
        for (int i = 0; i + d < pof2; i += 2 * d) {
          pairs[2 * np] = L[i]; pairs[2 * np + 1] = L[i + d]; np++;
        }
      *result = L[0];
    } else {
      /* the result is for rank `start`: survivor o holds it in the end, and at
       * every distance the half that o lies in keeps its own data (inoutvec)
       * and folds in what the other half sends */
      int o = start < 2 * rem ? start / 2 : start - rem;
      for (int d = pof2 / 2; d >= 1; d /= 2)
        for (int i = 0; i < pof2; i++) {
          if ((i & d) != (o & d) || ((i ^ o) & ~(2 * d - 1))) continue; /* i: a holder on o's side */
          pairs[2 * np] = L[i]; pairs[2 * np + 1] = L[i ^ d]; np++;
        }
      *result = L[o];
    }
    free(L);
    return np;
  }
  default:
    return -1;
  }
}

/* TREE_RSG, TREE_RSG_SPREAD: the n elements are cut into pof2 blocks of
 * n / pof2; the n % pof2 elements left over go to the last block (TREE_RSG:
 * MPI_Ireduce, MPI_Iallreduce) or one each to the first n % pof2 blocks
 * (TREE_RSG_SPREAD: MPI_Reduce, MPI_Allreduce).  Block k ends up on survivor
 * bit_reverse(k): the first exchange, at distance 1, already halves the data,
 * the lower half staying with the survivors whose lowest bit is clear. */
int alo_rsg_blocks(int P) { return floor_pow2(P); }
void alo_rsg_block(int P, size_t n, int k, int spread, size_t *lo, size_t *hi, int *owner) {
  int pof2 = floor_pow2(P), bits = 0, o = 0;
  size_t b = n / (size_t)pof2, left = n % (size_t)pof2;
  while ((1 << bits) < pof2) bits++;
  for (int j = 0; j < bits; j++) if (k & (1 << j)) o |= 1 << (bits - 1 - j);
  if (spread) {
    *lo = (size_t)k * b + ((size_t)k < left ? (size_t)k : left);
    *hi = *lo + b + ((size_t)k < left ? 1 : 0);
  } else {
    *lo = (size_t)k * b;
    *hi = k == pof2 - 1 ? n : (size_t)(k + 1) * b;
  }
  *owner = o;
}

/* Run a schedule over P tiles held in `slots` (each `len` elements). */
static void run_schedule(char **slots, const int *pairs, int np, size_t len,
                         int dtype, int op) {
  for (int k = 0; k < np; k++)
    step_serial(slots[pairs[2 * k]], slots[pairs[2 * k + 1]], len, dtype, op);
}

static int combine_impl(void *out, const void *const *in, int P, size_t n,
                        int dtype, int op, int order, int start, int generated,
                        int dist, uint64_t seed_base, uint64_t idx0) {
  const size_t es = alo_dtype_size(dtype);
  int rc = alo_check_op(dtype, op);
  if (rc) return rc;
  int *pairs = (int *)malloc(sizeof(int) * 2 * (size_t)(P > 1 ? P : 1));
  if (!pairs) return 3;
  int fail = 0;
  /* one schedule for the whole range, except under TREE_RSG(_SPREAD): one per block */
  const int rsg = order == ALO_ORDER_TREE_RSG || order == ALO_ORDER_TREE_RSG_SPREAD;
  const int nblocks = rsg ? alo_rsg_blocks(P) : 1;
  if (rsg && start != 0) { free(pairs); return 4; }
  for (int k = 0; k < nblocks && !fail; k++) {
    size_t b_lo = 0, b_hi = n;
    int owner = start, result = 0;
    if (rsg) alo_rsg_block(P, n, k, order == ALO_ORDER_TREE_RSG_SPREAD, &b_lo, &b_hi, &owner);
    int np = alo_schedule(P, order, owner, pairs, &result);
    if (np < 0) { free(pairs); return 4; }
    const size_t bn = b_hi - b_lo, ntiles = (bn + ALO_TILE - 1) / ALO_TILE;
#pragma omp parallel
    {
      char *tiles = (char *)malloc((size_t)P * ALO_TILE * es);
      char **slots = (char **)malloc(sizeof(char *) * (size_t)P);
      if (!tiles || !slots) {
#pragma omp atomic write
        fail = 1;
      } else {
        for (int r = 0; r < P; r++) slots[r] = tiles + (size_t)r * ALO_TILE * es;
#pragma omp for schedule(static)
        for (size_t t = 0; t < ntiles; t++) {
          size_t lo = b_lo + t * ALO_TILE, len = b_hi - lo < ALO_TILE ? b_hi - lo : ALO_TILE;
          for (int r = 0; r < P; r++) {
            if (generated)
              fill_range(slots[r], len, dtype, dist, seed_base + (uint64_t)r, idx0 + lo);
            else
              memcpy(slots[r], (const char *)in[r] + lo * es, len * es);
          }
          run_schedule(slots, pairs, np, len, dtype, op);
          if (op == ALO_AVG) divide_serial(slots[result], len, dtype, P);
          memcpy((char *)out + lo * es, slots[result], len * es);
        }
      }
      free(tiles);
      free(slots);
    }
  }
  free(pairs);
  return fail ? 3 : 0;
}

int alo_combine(void *out, const void *const *in, int P, size_t n, int dtype,
                int op, int order, int start) {
  return combine_impl(out, in, P, n, dtype, op, order, start, 0, 0, 0, 0);
}

int alo_combine_generated(void *out, int P, size_t n, int dtype, int op,
                          int order, int start, int dist, uint64_t seed_base,
                          uint64_t idx0) {
  return combine_impl(out, NULL, P, n, dtype, op, order, start, 1, dist,
                      seed_base, idx0);
}

/* The `start` a Reduce_scatter passes for the block that rank b receives: the
 * orders whose result is "for" a rank take b, the others have no such notion. */
int alo_order_start(int order, int b) {
  return order == ALO_ORDER_PAIRWISE_DESC || order == ALO_ORDER_RING || order == ALO_ORDER_TREE_HALV ? b : 0;
}

int alo_reduce_scatter(void *const *recv, const void *const *send, int P,
                       size_t count, int dtype, int op, int order) {
  const size_t es = alo_dtype_size(dtype);
  int rc = alo_check_op(dtype, op);
  if (rc) return rc;
  const void **blk = (const void **)malloc(sizeof(void *) * (size_t)P);
  if (!blk) return 3;
  for (int b = 0; b < P && rc == 0; b++) {
    for (int r = 0; r < P; r++) blk[r] = (const char *)send[r] + (size_t)b * count * es;
    rc = alo_combine(recv[b], blk, P, count, dtype, op, order, alo_order_start(order, b));
  }
  free(blk);
  return rc;
}

int alo_allgather(void *const *recv, const void *const *send, int P,
                  size_t count, int dtype) {
  const size_t es = alo_dtype_size(dtype);
  if (es == 0) return 2;
  for (int r = 0; r < P; r++)
    for (int q = 0; q < P; q++) {
      char *dst = (char *)recv[r] + (size_t)q * count * es;
      if (dst != (const char *)send[q]) memmove(dst, send[q], count * es);
    }
  return 0;
}

int alo_reduce_scatterv(void *const *recv, const void *const *send, int P,
                        const size_t *counts, int dtype, int op, int order) {
  const size_t es = alo_dtype_size(dtype);
  int rc = alo_check_op(dtype, op);
  if (rc) return rc;
  const void **blk = (const void **)malloc(sizeof(void *) * (size_t)P);
  if (!blk) return 3;
  size_t displ = 0;
  for (int b = 0; b < P && rc == 0; b++) {
    for (int r = 0; r < P; r++) blk[r] = (const char *)send[r] + displ * es;
    if (counts[b]) rc = alo_combine(recv[b], blk, P, counts[b], dtype, op, order, alo_order_start(order, b));
    displ += counts[b];
  }
  free(blk);
  return rc;
}

int alo_allgatherv(void *const *recv, const void *const *send, int P,
                   const size_t *counts, const size_t *displs, int dtype) {
  const size_t es = alo_dtype_size(dtype);
  if (es == 0) return 2;
  for (int r = 0; r < P; r++)
    for (int q = 0; q < P; q++) {
      char *dst = (char *)recv[r] + displs[q] * es;
      if (counts[q] && dst != (const char *)send[q]) memmove(dst, send[q], counts[q] * es);
    }
  return 0;
}

/* ------------------------------------------------------------------------ */
/* Ring reduce-scatter + allgather, moved literally chunk by chunk           */
/* ------------------------------------------------------------------------ */

void alo_ring_segment(size_t n, int P, int s, size_t *offset, size_t *len) {
  size_t base = n / (size_t)P, rem = n % (size_t)P;
  *offset = (size_t)s * base + ((size_t)s < rem ? (size_t)s : rem);
  *len = base + ((size_t)s < rem ? 1 : 0);
}

int alo_ring_reduce_scatter(void *const *bufs, int P, size_t n, int dtype,
                            int op, size_t chunk_elems) {
  const size_t es = alo_dtype_size(dtype);
  int rc = alo_check_op(dtype, op);
  if (rc) return rc;
  if (P < 1 || chunk_elems == 0) return 4;
  char *wire = (char *)malloc(chunk_elems * es);
  if (!wire) return 3;
  for (int t = 0; t < P - 1; t++)
    for (int r = 0; r < P; r++) {
      int seg = ((r - t - 1) % P + P) % P, from = (r - 1 + P) % P;
      size_t off, len;
      alo_ring_segment(n, P, seg, &off, &len);
      for (size_t c = 0; c < len; c += chunk_elems) {
        size_t m = len - c < chunk_elems ? len - c : chunk_elems;
        memcpy(wire, (const char *)bufs[from] + (off + c) * es, m * es); /* the message */
        alo_step((char *)bufs[r] + (off + c) * es, wire, m, dtype, op);
        /* avg: the last step leaves the full sum in place; divide it there */
        if (op == ALO_AVG && t == P - 2)
          alo_divide((char *)bufs[r] + (off + c) * es, m, dtype, P);
      }
    }
  free(wire);
  return 0;
}

int alo_ring_allgather(void *const *bufs, int P, size_t n, int dtype,
                       size_t chunk_elems) {
  const size_t es = alo_dtype_size(dtype);
  if (es == 0) return 2;
  if (P < 1 || chunk_elems == 0) return 4;
  /* after the reduce-scatter rank r owns segment (r+1) mod P; at step t it
   * receives segment (r-t) mod P from rank r-1 */
  for (int t = 0; t < P - 1; t++)
    for (int r = 0; r < P; r++) {
      int seg = ((r - t) % P + P) % P, from = (r - 1 + P) % P;
      size_t off, len;
      alo_ring_segment(n, P, seg, &off, &len);
      for (size_t c = 0; c < len; c += chunk_elems) {
        size_t m = len - c < chunk_elems ? len - c : chunk_elems;
        memcpy((char *)bufs[r] + (off + c) * es,
               (const char *)bufs[from] + (off + c) * es, m * es);
      }
    }
  return 0;
}

int alo_ring_allreduce(void *const *bufs, int P, size_t n, int dtype, int op,
                       size_t chunk_elems) {
  int rc = alo_ring_reduce_scatter(bufs, P, n, dtype, op, chunk_elems);
  if (rc) return rc;
  return alo_ring_allgather(bufs, P, n, dtype, chunk_elems);
}

/* ------------------------------------------------------------------------ */
/* Halo faces                                                               */
/* ------------------------------------------------------------------------ */

/* Box of a face in allocation coordinates: lo[d] .. lo[d]+ext[d]. */
static int halo_box(size_t nx, size_t ny, size_t nz, size_t h, int face,
                    int ghost, size_t lo[3], size_t ext[3]) {
  size_t n[3] = {nx, ny, nz};
  if (face < 0 || face > 5) return 1;
  int axis = face / 2, plus = face % 2;
  for (int d = 0; d < 3; d++) { lo[d] = h; ext[d] = n[d]; }
  ext[axis] = h;
  if (ghost) lo[axis] = plus ? h + n[axis] : 0;
  else lo[axis] = plus ? n[axis] : h;
  return 0;
}

size_t alo_halo_face_elems(size_t nx, size_t ny, size_t nz, size_t h, int face) {
  size_t lo[3], ext[3];
  if (halo_box(nx, ny, nz, h, face, 0, lo, ext)) return 0;
  return ext[0] * ext[1] * ext[2];
}

static int halo_copy(void *grid, void *buf, size_t nx, size_t ny, size_t nz,
                     size_t h, int face, size_t es, int unpack) {
  size_t lo[3], ext[3];
  if (halo_box(nx, ny, nz, h, face, unpack, lo, ext)) return 1;
  if (h > nx || h > ny || h > nz) return 1;
  const size_t sx = nx + 2 * h, sy = ny + 2 * h;
  size_t k = 0;
  for (size_t z = 0; z < ext[2]; z++)
    for (size_t y = 0; y < ext[1]; y++)
      for (size_t x = 0; x < ext[0]; x++, k++) {
        size_t g = ((lo[2] + z) * sy + (lo[1] + y)) * sx + (lo[0] + x);
        if (unpack) memcpy((char *)grid + g * es, (char *)buf + k * es, es);
        else memcpy((char *)buf + k * es, (char *)grid + g * es, es);
      }
  return 0;
}

int alo_halo_pack(void *buf, const void *grid, size_t nx, size_t ny, size_t nz,
                  size_t h, int face, size_t elem_size) {
  return halo_copy((void *)grid, buf, nx, ny, nz, h, face, elem_size, 0);
}

int alo_halo_unpack(void *grid, const void *buf, size_t nx, size_t ny,
                    size_t nz, size_t h, int face, size_t elem_size) {
  return halo_copy(grid, (void *)buf, nx, ny, nz, h, face, elem_size, 1);
}

/* ------------------------------------------------------------------------ */

uint64_t alo_checksum(const void *buf, size_t nbytes) {
  const unsigned char *p = (const unsigned char *)buf;
  uint64_t h = 0xcbf29ce484222325ull;
  size_t i = 0;
  for (; i + 8 <= nbytes; i += 8) {
    uint64_t w;
    memcpy(&w, p + i, 8);
    h = fin64(h ^ w) + ALO_GAMMA;
  }
  for (; i < nbytes; i++) h = (h ^ p[i]) * 0x100000001b3ull;
  return h;
}

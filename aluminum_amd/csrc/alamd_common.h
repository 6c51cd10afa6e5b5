// Shared host/device helpers of the aluminum_amd library: error reporting,
// element tag types, the pairwise step of every (type, op) pair and the
// 128-bit vector load/store helpers.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include <atomic>
#include <type_traits>

#include "aluminum_amd.h"

namespace alamd {

// ---- errors ---------------------------------------------------------------

// Records the message for alamd_last_error() and returns `code`.
int set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

#define ALAMD_HIP(call)                                                        \
  do {                                                                         \
    hipError_t e_ = (call);                                                    \
    if (e_ != hipSuccess)                                                      \
      return ::alamd::set_error(ALAMD_ERR_HIP, "%s failed: %s", #call,         \
                                hipGetErrorString(e_));                        \
  } while (0)

// Number of compute units of the current device (cached per device); < 0 on
// error (message set).
int device_cus();

// The sizes the launch planners work with (what each one means, and the measurements behind its default,
// stands where it is used).  Defaults suit an MI355X; alamd_tune() changes them for comparisons.
// Process-wide; every field is an atomic, so that a setting changed while calls run is a clean old-or-new
// value for each of them, never a torn one.
constexpr size_t kBlockShapeFromBytes = (size_t)32 << 20, kBlockShapeBelowBytes = (size_t)384 << 20;
struct Tunables {
  std::atomic<size_t> launch_bytes{(size_t)4 << 30};            // bytes one fold / tree launch moves
  std::atomic<size_t> two_step_min_total_bytes{(size_t)128 << 20};  // fold + spread instead of one kernel: from this
                                                                    // many bytes written in all (outputs x bytes each) ...
  std::atomic<size_t> two_step_min_outputs{3};                  // ... and this many outputs up
  std::atomic<size_t> two_step_piece_bytes{(size_t)128 << 20};  // piece of the result the two steps alternate over
  std::atomic<size_t> ring_piece_bytes{(size_t)256 << 20};      // the same for the fused ring allreduce
  std::atomic<size_t> spread_launch_bytes{(size_t)288 << 20};   // bytes one spread launch moves
  std::atomic<size_t> spread_hbm_chunk_tiles{1024}, spread_hbm_launch_chunks{2};      // slices read from HBM
  std::atomic<size_t> spread_cache_chunk_tiles{512}, spread_cache_launch_chunks{16};  // a result just written
  std::atomic<size_t> stream_wgs_per_cu{0};  // workgroups per CU of a streaming fold / tree launch (0: the kernels' own)
  // a fold / tree launch that moves this much in all and less than that takes the block shape (alamd_tile.h)
  std::atomic<size_t> block_shape_from_bytes{kBlockShapeFromBytes}, block_shape_below_bytes{kBlockShapeBelowBytes};
  std::atomic<size_t> fold_front3_ranks{0};  // ranks from which a fold asks for three streams up front (0: by type)
  std::atomic<size_t> halo_load_policy{0};  // grid loads of a halo pack: 0 plain, 1 nt, 2 sc1, 3 sc0 sc1, 4 sc0 sc1 nt
};
Tunables &tunables();

// Checks (dtype, op) as alamd_check_op does, setting the error message.
int check_type_op(int dtype, int op);

inline bool is_float_dtype(int dt) {
  return dt == ALAMD_F16 || dt == ALAMD_BF16 || dt == ALAMD_F32 || dt == ALAMD_F64;
}

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// ---- element types --------------------------------------------------------

struct f16_t { uint16_t b; };   // IEEE binary16 bit pattern
struct bf16_t { uint16_t b; };  // bfloat16 bit pattern

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Exact widening of the 16-bit float types.
__device__ __forceinline__ float widen(f16_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, h.b));
}
__device__ __forceinline__ float widen(bf16_t h) {
  return __uint_as_float(static_cast<uint32_t>(h.b) << 16);
}

// Round-to-nearest-even narrowing.  A NaN stays a NaN with the quiet bit set.
template <typename H> __device__ __forceinline__ H narrow(float f);
template <> __device__ __forceinline__ f16_t narrow<f16_t>(float f) {
  f16_t r;
  r.b = __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
  return r;
}
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
// Two fp32 values to a packed pair of bf16 with the hardware conversion
// (v_cvt_pk_bf16_f32: nearest-even, NaN stays NaN).
__device__ __forceinline__ uint32_t narrow_bf16x2(float lo, float hi) {
  const f32x2_t f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}
template <> __device__ __forceinline__ bf16_t narrow<bf16_t>(float f) {
  bf16_t r;
  r.b = static_cast<uint16_t>(narrow_bf16x2(f, 0.0f) & 0xffffu);
  return r;
}

// ---- the pairwise step ----------------------------------------------------
//
// avg is sum followed by one division by the number of ranks (see Divisor
// below), so its pairwise step is the step of sum.
constexpr bool op_is_sum(int op) { return op == ALAMD_SUM || op == ALAMD_AVG; }
//
// step<T, OP>(in, inout) is one application of an MPI reduction function to
// one element: the value stored back to inoutvec.  For the native types it
// is OP(inout, in) with MIN(x, y) = (x < y) ? x : y and MAX(x, y) =
// (x > y) ? x : y, so a tie or a NaN operand yields `in`; for fp16 / bf16 it
// is narrow(OP(widen(in), widen(inout))) with std::min / std::max
// (reference: src/mpi_impl.cpp:61-145), which chooses the same operand.

template <typename T> struct unsigned_of { using type = T; };
template <> struct unsigned_of<int8_t> { using type = uint8_t; };
template <> struct unsigned_of<int16_t> { using type = uint16_t; };
template <> struct unsigned_of<int32_t> { using type = uint32_t; };
template <> struct unsigned_of<int64_t> { using type = uint64_t; };

template <typename T, int OP> struct Step {
  // integer types
  static __device__ __forceinline__ T apply(T in, T inout) {
    using U = typename unsigned_of<T>::type;
    if constexpr (op_is_sum(OP)) return static_cast<T>(static_cast<U>(static_cast<U>(inout) + static_cast<U>(in)));
    else if constexpr (OP == ALAMD_PROD) return static_cast<T>(static_cast<U>(static_cast<U>(inout) * static_cast<U>(in)));
    else if constexpr (OP == ALAMD_MIN) return (inout < in) ? inout : in;
    else if constexpr (OP == ALAMD_MAX) return (inout > in) ? inout : in;
    else if constexpr (OP == ALAMD_LOR) return static_cast<T>((inout != 0) || (in != 0));
    else if constexpr (OP == ALAMD_LAND) return static_cast<T>((inout != 0) && (in != 0));
    else if constexpr (OP == ALAMD_LXOR) return static_cast<T>((inout != 0) != (in != 0));
    else if constexpr (OP == ALAMD_BOR) return static_cast<T>(inout | in);
    else if constexpr (OP == ALAMD_BAND) return static_cast<T>(inout & in);
    else return static_cast<T>(inout ^ in);
  }
};

template <typename F, int OP> __device__ __forceinline__ F fp_step(F in, F inout) {
  if constexpr (op_is_sum(OP)) return inout + in;
  else if constexpr (OP == ALAMD_PROD) return inout * in;
  else if constexpr (OP == ALAMD_MIN) return (inout < in) ? inout : in;
  else return (inout > in) ? inout : in;
}

template <int OP> struct Step<float, OP> {
  static __device__ __forceinline__ float apply(float in, float inout) { return fp_step<float, OP>(in, inout); }
};
template <int OP> struct Step<double, OP> {
  static __device__ __forceinline__ double apply(double in, double inout) { return fp_step<double, OP>(in, inout); }
};
template <int OP> struct Step<f16_t, OP> {
  static __device__ __forceinline__ f16_t apply(f16_t in, f16_t inout) {
    return narrow<f16_t>(fp_step<float, OP>(widen(in), widen(inout)));
  }
};
template <int OP> struct Step<bf16_t, OP> {
  static __device__ __forceinline__ bf16_t apply(bf16_t in, bf16_t inout) {
    return narrow<bf16_t>(fp_step<float, OP>(widen(in), widen(inout)));
  }
};

// One 16-bit operation per byte of a dword: a byte of either operand selected as source and one byte of
// the result written, the first instruction clearing the others and the later ones keeping them.
// d = a NAME b, byte by byte; SRC0 / SRC1 are "%1" / "%2" or "sext(%1)" / "sext(%2)".
#define ALAMD_PER_BYTE(NAME, SRC0, SRC1)                                                                             \
asm(NAME " %0, " SRC0 ", " SRC1 " dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:BYTE_0 src1_sel:BYTE_0" : "=v"(d) : "v"(a), "v"(b)); \
asm(NAME " %0, " SRC0 ", " SRC1 " dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_1 src1_sel:BYTE_1" : "+v"(d) : "v"(a), "v"(b)); \
asm(NAME " %0, " SRC0 ", " SRC1 " dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_2 src1_sel:BYTE_2" : "+v"(d) : "v"(a), "v"(b)); \
asm(NAME " %0, " SRC0 ", " SRC1 " dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3 src1_sel:BYTE_3" : "+v"(d) : "v"(a), "v"(b));

// A logical operator on 8- or 16-bit elements, which step_vec takes a dword at a time: its result holds 0
// or 1 in every element, so a fold that has made its first operand so (truth_vec) can tell step_vec
// that `inout` needs no looking at again (INOUT_IS_TRUTH): eleven instructions per dword become six.
template <typename T, int OP> constexpr bool narrow_logical() {
  return sizeof(T) <= 2 && (OP == ALAMD_LOR || OP == ALAMD_LAND || OP == ALAMD_LXOR);
}
// 1 in every 8- or 16-bit element that is nonzero, 0 in the others (the carry of low bits + all-ones
// reaches the top bit iff a low bit is set).
template <typename T> __device__ __forceinline__ uint32_t truth_dword(uint32_t x) {
  constexpr uint32_t low = sizeof(T) == 1 ? 0x7f7f7f7fu : 0x7fff7fffu, top = ~low;
  constexpr int shift = 8 * (int)sizeof(T) - 1;
  return ((((x & low) + low) | x) & top) >> shift;
}
template <typename T> __device__ __forceinline__ u32x4 truth_vec(u32x4 v) {
  u32x4 r;
#pragma unroll
  for (int j = 0; j < 4; ++j) r[j] = truth_dword<T>(v[j]);
  return r;
}

// The step applied to every element of a 128-bit vector.
template <typename T, int OP, bool INOUT_IS_TRUTH = false>
__device__ __forceinline__ u32x4 step_vec(u32x4 in, u32x4 inout) {
  if constexpr (std::is_same<T, bf16_t>::value) {
    // two elements per dword: widen by shift / mask, one fp32 operation each,
    // narrow the pair with one packed conversion
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float a_lo = __uint_as_float(in[j] << 16), a_hi = __uint_as_float(in[j] & 0xffff0000u);
      const float b_lo = __uint_as_float(inout[j] << 16), b_hi = __uint_as_float(inout[j] & 0xffff0000u);
      r[j] = narrow_bf16x2(fp_step<float, OP>(a_lo, b_lo), fp_step<float, OP>(a_hi, b_hi));
    }
    return r;
  } else if constexpr (sizeof(T) == 1 && op_is_sum(OP)) {
    // four wrapping byte sums per dword: add the low seven bits of every byte
    // (no carry leaves a byte), then put the top bits back with an xor
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t a = in[j], b = inout[j];
      r[j] = ((a & 0x7f7f7f7fu) + (b & 0x7f7f7f7fu)) ^ ((a ^ b) & 0x80808080u);
    }
    return r;
  } else if constexpr (sizeof(T) == 1 && OP == ALAMD_PROD) {
    // wrapping byte products: the low byte of the 16-bit product of two bytes, one instruction per byte
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t a = in[j], b = inout[j];
      uint32_t d;
      ALAMD_PER_BYTE("v_mul_lo_u16_sdwa", "%1", "%2")
      r[j] = d;
    }
    return r;
  } else if constexpr (sizeof(T) == 1 && (OP == ALAMD_MIN || OP == ALAMD_MAX)) {
    // one instruction per byte: the 16-bit min / max with a byte of either operand selected as source
    // (sign-extended for signed bytes) and one byte of the result written, the others kept.  (Bytes
    // compared as packed 16-bit pairs took 11 instructions per dword, what the compiler makes of the
    // plain loop 9, this 4.)
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t a = in[j], b = inout[j];
      uint32_t d;
      if constexpr (std::is_signed<T>::value) {
        if constexpr (OP == ALAMD_MIN) { ALAMD_PER_BYTE("v_min_i16_sdwa", "sext(%1)", "sext(%2)") }
        else { ALAMD_PER_BYTE("v_max_i16_sdwa", "sext(%1)", "sext(%2)") }
      } else {
        if constexpr (OP == ALAMD_MIN) { ALAMD_PER_BYTE("v_min_u16_sdwa", "%1", "%2") }
        else { ALAMD_PER_BYTE("v_max_u16_sdwa", "%1", "%2") }
      }
      r[j] = d;
    }
    return r;
  } else if constexpr (narrow_logical<T, OP>()) {
    // a whole dword of bytes or halfwords at a time: a 1 in every element that is nonzero, then the
    // bitwise operator
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t a = in[j], b = inout[j];
      if constexpr (INOUT_IS_TRUTH) {
        const uint32_t ta = truth_dword<T>(a);
        r[j] = OP == ALAMD_LOR ? (b | ta) : OP == ALAMD_LAND ? (b & ta) : (b ^ ta);
      } else {
        r[j] = OP == ALAMD_LOR ? truth_dword<T>(b | a) : OP == ALAMD_LAND ? (truth_dword<T>(b) & truth_dword<T>(a))
                                                                           : (truth_dword<T>(b) ^ truth_dword<T>(a));
      }
    }
    return r;
  } else {
    constexpr int N = 16 / sizeof(T);
    union U { u32x4 v; T e[N]; __device__ U() {} } a, b;
    a.v = in;
    b.v = inout;
#pragma unroll
    for (int j = 0; j < N; ++j) b.e[j] = Step<T, OP>::apply(a.e[j], b.e[j]);
    return b.v;
  }
}

// ---- the division that ends an avg ------------------------------------------
//
// avg = the sum in the named order (rounded, or wrapped, after every step
// exactly as for sum), then one division by the number of ranks d in the
// element type's own arithmetic: IEEE division for fp32 / fp64; widen, fp32
// division, round-to-nearest-even narrowing for fp16 / bf16 (one more step of
// the rule of src/mpi_impl.cpp:61-145); C integer division (truncation toward
// zero) for the integer types.  The reference forwards avg to the
// communication library of its NCCL backend (include/aluminum/nccl_impl.hpp:176)
// and rejects it elsewhere.
//
// Integer division by the uniform d without a divide instruction (Granlund and
// Montgomery, "Division by invariant integers using multiplication"): with
// l = ceil(log2 d), m = floor(2^N (2^l - d) / d) + 1, t = mulhi(m, n),
// n / d = (t + ((n - t) >> min(l, 1))) >> max(l - 1, 0) for every N-bit n.
struct Divisor {
  unsigned long long m64;
  unsigned m32;
  unsigned sh1, sh2;
  float f;
  double d;
  // fp64: a power of two divides exactly by a multiplication - the same correctly rounded result as
  // the division, subnormal results included, without its two dozen instructions (P = 8: +5 %; the
  // same choice cost the fp32 kernel 3.5 %, whose division is short, so it divides)
  int pow2;
  double dinv;
};

inline Divisor make_divisor(int ranks) {
  Divisor dv;
  const unsigned d = ranks > 0 ? (unsigned)ranks : 1u;
  unsigned l = 0;
  while ((1u << l) < d) ++l;
  const unsigned long long k = (1ull << l) - d;
  dv.m32 = (unsigned)(((k << 32) / d) + 1);
  dv.m64 = (unsigned long long)((((unsigned __int128)k << 64) / d) + 1);
  dv.sh1 = l < 1 ? l : 1;
  dv.sh2 = l > 1 ? l - 1 : 0;
  dv.f = (float)d;
  dv.d = (double)d;
  dv.pow2 = (d & (d - 1)) == 0 ? 1 : 0;
  dv.dinv = 1.0 / dv.d;
  return dv;
}

__device__ __forceinline__ uint32_t udiv_by(uint32_t n, const Divisor &dv) {
  const uint32_t t = __umulhi(dv.m32, n);
  return (t + ((n - t) >> dv.sh1)) >> dv.sh2;
}
__device__ __forceinline__ uint64_t udiv_by(uint64_t n, const Divisor &dv) {
  const uint64_t t = __umul64hi(dv.m64, n);
  return (t + ((n - t) >> dv.sh1)) >> dv.sh2;
}

template <typename T> __device__ __forceinline__ T div_elem(T x, const Divisor &dv) {
  if constexpr (std::is_same<T, float>::value) return x / dv.f;
  else if constexpr (std::is_same<T, double>::value) return dv.pow2 ? x * dv.dinv : x / dv.d;
  else if constexpr (std::is_same<T, f16_t>::value || std::is_same<T, bf16_t>::value) return narrow<T>(widen(x) / dv.f);
  else {
    // magnitude in 32 or 64 bits, unsigned division, sign put back
    using W = typename std::conditional<sizeof(T) == 8, uint64_t, uint32_t>::type;
    using SW = typename std::make_signed<W>::type;
    const bool neg = std::is_signed<T>::value && x < 0;
    const W a = neg ? (W)0 - (W)(SW)x : (W)x;
    const W q = udiv_by(a, dv);
    return (T)(neg ? (W)0 - q : q);
  }
}

// The end of a combine: for avg every element of the folded vector is divided
// by the number of ranks; for every other operator nothing happens.
template <typename T, int OP> __device__ __forceinline__ u32x4 finish_vec(u32x4 acc, const Divisor &dv) {
  if constexpr (OP != ALAMD_AVG) return acc;
  else {
    constexpr int N = 16 / sizeof(T);
    union U { u32x4 v; T e[N]; __device__ U() {} } a;
    a.v = acc;
#pragma unroll
    for (int j = 0; j < N; ++j) a.e[j] = div_elem<T>(a.e[j], dv);
    return a.v;
  }
}
template <typename T, int OP> __device__ __forceinline__ T finish_elem(T acc, const Divisor &dv) {
  if constexpr (OP != ALAMD_AVG) return acc;
  else return div_elem<T>(acc, dv);
}

// ---- element access (any alignment) --------------------------------------

template <typename T> __device__ __forceinline__ T ld_elem(const void *p) {
  return *reinterpret_cast<const T *>(p);
}
template <typename T> __device__ __forceinline__ void st_elem(void *p, T v) {
  *reinterpret_cast<T *>(p) = v;
}

// The kernels issue 128-bit accesses at any element-aligned address (the
// device runs in unaligned access mode; see head_elems in alamd_tile.h for
// the one case that costs bandwidth).  A pointer that is not even aligned to
// its element type is refused.
inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// A byte range as the copy kernel walks it: `head` single bytes, `vec` bytes in
// whole 128-bit vectors, `tail` < 16.  The vectors start where the destination
// reaches a 64-byte boundary, so that every line is stored whole, if that
// leaves the loads 4-byte aligned (128-bit loads run at full rate from any
// 4-byte boundary and lose a fifth when they split dwords); otherwise at the
// source's next 4-byte boundary.
struct ByteSplit { size_t head, vec, tail; };
inline ByteSplit split_bytes(const void *dst, const void *src, size_t bytes) {
  const uintptr_t d = reinterpret_cast<uintptr_t>(dst), s = reinterpret_cast<uintptr_t>(src);
  ByteSplit b;
  b.head = ((d ^ s) & 3) == 0 ? (64 - (d & 63)) & 63 : (4 - (s & 3)) & 3;
  if (b.head > bytes) b.head = bytes;
  b.vec = (bytes - b.head) & ~(size_t)15;
  b.tail = bytes - b.head - b.vec;
  return b;
}

// Grid size for a streaming kernel over `work_items` items with `per_block`
// items per workgroup pass: enough workgroups to cover the work, capped at
// `waves` workgroups per compute unit.
unsigned stream_grid(size_t work_items, size_t per_block, int waves);

}  // namespace alamd

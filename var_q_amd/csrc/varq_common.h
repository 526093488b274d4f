// Shared host/device helpers for the gfx950 VAR-Q kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/varq.h"

#define VARQ_WAVE 64

// ---- host-side error plumbing -------------------------------------------
int varq_set_error(int code, const char *fmt, ...);

#define VARQ_CHECK_ARG(cond, ...)                                   \
  do {                                                              \
    if (!(cond)) return varq_set_error(VARQ_ERR_INVALID, __VA_ARGS__); \
  } while (0)

#define VARQ_CHECK_LAUNCH(what)                                              \
  do {                                                                       \
    hipError_t e_ = hipGetLastError();                                       \
    if (e_ != hipSuccess)                                                    \
      return varq_set_error(VARQ_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e_)); \
  } while (0)

// Row mapping {n0,n1,n2,os0,os1,os2,off,slot_dim}; see varq.h.
struct RowMap {
  int64_t n0, n1, n2;
  int64_t os0, os1, os2, off;
  int slot_dim;
};

static inline RowMap varq_dense_rowmap(int64_t n_rows) {
  RowMap m;
  m.n0 = 1; m.n1 = 1; m.n2 = n_rows;
  m.os0 = 0; m.os1 = 0; m.os2 = 1; m.off = 0;
  m.slot_dim = -1;
  return m;
}

static inline RowMap varq_rowmap_from_host(const int64_t *h, int64_t n_rows) {
  if (!h) return varq_dense_rowmap(n_rows);
  RowMap m;
  m.n0 = h[0]; m.n1 = h[1]; m.n2 = h[2];
  m.os0 = h[3]; m.os1 = h[4]; m.os2 = h[5]; m.off = h[6];
  m.slot_dim = (int)h[7];
  return m;
}

static inline int varq_log2_exact(int64_t v) {  // -1 unless v is a power of two
  if (v <= 0 || (v & (v - 1))) return -1;
  int s = 0;
  while ((1ll << s) < v) ++s;
  return s;
}

#ifdef __HIPCC__
// ---- device helpers -------------------------------------------------------
typedef unsigned int u32;

__device__ __forceinline__ float u2f(u32 u) { return __uint_as_float(u); }
__device__ __forceinline__ u32 f2u(float f) { return __float_as_uint(f); }

// Input element loaders: 8 consecutive elements starting at a 16-byte aligned
// (bf16/fp16) or 32-byte aligned (fp32) address, widened to fp32 exactly.
typedef __bf16 varq_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 varq_f16x8 __attribute__((ext_vector_type(8)));

// The 16-bit loaders widen with a language-level conversion (not bit tricks) so
// that the compiler knows the results are canonical floats and emits bare
// v_min/v_max for the reductions that follow.
template <int DT> struct In8;
template <> struct In8<VARQ_F32> {
  static constexpr int kBytes = 4;
  __device__ static __forceinline__ void load(const void *base, int64_t elem, float (&v)[8]) {
    const float4 *p = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(base) + elem);
    float4 a = p[0], b = p[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  __device__ static __forceinline__ float load1(const void *base, int64_t elem) {
    return reinterpret_cast<const float *>(base)[elem];
  }
};
template <> struct In8<VARQ_BF16> {
  static constexpr int kBytes = 2;
  __device__ static __forceinline__ void load(const void *base, int64_t elem, float (&v)[8]) {
    varq_bf16x8 a = *reinterpret_cast<const varq_bf16x8 *>(reinterpret_cast<const __bf16 *>(base) + elem);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)a[i];
  }
  __device__ static __forceinline__ float load1(const void *base, int64_t elem) {
    return (float)reinterpret_cast<const __bf16 *>(base)[elem];
  }
};
template <> struct In8<VARQ_F16> {
  static constexpr int kBytes = 2;
  __device__ static __forceinline__ void load(const void *base, int64_t elem, float (&v)[8]) {
    varq_f16x8 a = *reinterpret_cast<const varq_f16x8 *>(reinterpret_cast<const _Float16 *>(base) + elem);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)a[i];
  }
  __device__ static __forceinline__ float load1(const void *base, int64_t elem) {
    return (float)reinterpret_cast<const _Float16 *>(base)[elem];
  }
};

// Raw 8-element loads (no conversion) so that a kernel can issue the next
// tile's loads before converting the current one.  Streaming data: marked
// non-temporal, it is read exactly once.
typedef float varq_f32x4 __attribute__((ext_vector_type(4)));
template <int DT> struct Raw8;
template <> struct Raw8<VARQ_F32> {
  varq_f32x4 a, b;
  __device__ __forceinline__ void load(const void *base, int64_t elem) {
    const varq_f32x4 *p = reinterpret_cast<const varq_f32x4 *>(reinterpret_cast<const float *>(base) + elem);
    a = __builtin_nontemporal_load(p);
    b = __builtin_nontemporal_load(p + 1);
  }
  __device__ __forceinline__ void widen(float (&v)[8]) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
  }
};
template <> struct Raw8<VARQ_BF16> {
  varq_bf16x8 a;
  __device__ __forceinline__ void load(const void *base, int64_t elem) {
    a = __builtin_nontemporal_load(reinterpret_cast<const varq_bf16x8 *>(reinterpret_cast<const __bf16 *>(base) + elem));
  }
  __device__ __forceinline__ void widen(float (&v)[8]) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)a[i];
  }
};
template <> struct Raw8<VARQ_F16> {
  varq_f16x8 a;
  __device__ __forceinline__ void load(const void *base, int64_t elem) {
    a = __builtin_nontemporal_load(reinterpret_cast<const varq_f16x8 *>(reinterpret_cast<const _Float16 *>(base) + elem));
  }
  __device__ __forceinline__ void widen(float (&v)[8]) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)a[i];
  }
};

// fp32 -> output dtype, round to nearest even (what tensor.to(dtype) does).
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  u32 u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ uint16_t f32_to_f16_rne(float f) {
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}

// Cross-lane all-reduce over aligned groups of LANES lanes (power of two).
// Stages inside a 16-lane row use DPP, wider stages a lane permute.
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
  // (a lane whose partner is switched off keeps its own value)
  return u2f((u32)__builtin_amdgcn_update_dpp((int)f2u(v), (int)f2u(v), CTRL, 0xf, 0xf, false));
}

// A fold over aligned groups of up to 16 lanes as one DPP instruction per step, v = OP(v of
// the partner lane, v).  Written as assembly because the compiler's sequence for the same
// step through the intrinsic is four instructions (a copy, a DPP move, a canonicalising max
// of the moved value with itself, the operation).  A DPP read needs two idle cycles after a
// vector write of its source: the s_nop in front of every step provides them whatever wrote
// the source, the one at the end covers a DPP read of the result by whatever follows.
// v_max_f32 / v_min_f32 return the other operand when one is a quiet NaN, like fmaxf / fminf.
// A lane whose partner is switched off is not written by the step and so keeps its value.
#define VARQ_DPP_FOLD_STEP(op, ctrl) "s_nop 1\n\t" op "_dpp %0, %0, %0 " ctrl " row_mask:0xf bank_mask:0xf\n\t"
#define VARQ_DPP_FOLD(NAME, OP)                                                                     \
  template <int LANES> __device__ __forceinline__ float NAME(float v) {                             \
    static_assert(LANES == 1 || LANES == 2 || LANES == 4 || LANES == 8 || LANES == 16, "one row");  \
    if (LANES == 2) asm(VARQ_DPP_FOLD_STEP(OP, "quad_perm:[1,0,3,2]") "s_nop 1" : "+v"(v));         \
    if (LANES == 4)                                                                                 \
      asm(VARQ_DPP_FOLD_STEP(OP, "quad_perm:[1,0,3,2]") VARQ_DPP_FOLD_STEP(OP, "quad_perm:[2,3,0,1]") "s_nop 1" : "+v"(v)); \
    if (LANES == 8)                                                                                 \
      asm(VARQ_DPP_FOLD_STEP(OP, "quad_perm:[1,0,3,2]") VARQ_DPP_FOLD_STEP(OP, "quad_perm:[2,3,0,1]")  \
          VARQ_DPP_FOLD_STEP(OP, "row_half_mirror") "s_nop 1" : "+v"(v));                           \
    if (LANES == 16)                                                                                \
      asm(VARQ_DPP_FOLD_STEP(OP, "quad_perm:[1,0,3,2]") VARQ_DPP_FOLD_STEP(OP, "quad_perm:[2,3,0,1]")  \
          VARQ_DPP_FOLD_STEP(OP, "row_half_mirror") VARQ_DPP_FOLD_STEP(OP, "row_mirror") "s_nop 1" : "+v"(v)); \
    return v;                                                                                       \
  }
VARQ_DPP_FOLD(row_fold_max, "v_max_f32")
VARQ_DPP_FOLD(row_fold_min, "v_min_f32")
VARQ_DPP_FOLD(row_fold_add, "v_add_f32")
#undef VARQ_DPP_FOLD

template <int LANES, bool IS_MAX> __device__ __forceinline__ float group_allreduce(float v) {
#define VARQ_COMBINE(a, b) (IS_MAX ? fmaxf((a), (b)) : fminf((a), (b)))
  v = IS_MAX ? row_fold_max<(LANES < 16 ? LANES : 16)>(v) : row_fold_min<(LANES < 16 ? LANES : 16)>(v);
  if (LANES >= 32) v = VARQ_COMBINE(v, __shfl_xor(v, 16, 64));
  if (LANES >= 64) v = VARQ_COMBINE(v, __shfl_xor(v, 32, 64));
#undef VARQ_COMBINE
  return v;
}

template <int BITS> struct QRange {
  static constexpr int kMin = -(1 << (BITS - 1));
  static constexpr int kMax = (1 << (BITS - 1)) - 1;
  static constexpr int kLevels = (1 << BITS) - 1;
  static constexpr int kVals = 32 / BITS;
};
#endif  // __HIPCC__

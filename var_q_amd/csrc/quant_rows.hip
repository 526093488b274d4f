// One-pass quantize + pack for row-local groups (group = `group` contiguous
// channels of one row).  HBM-bound: every input byte is read once, every packed
// word, scale and zero-point written once.
//
// Arithmetic follows VAR_Q/quant.py:112-121 exactly (fp32, true division,
// round-half-to-even, clamp) and the packing layout of
// VAR_Q/pack_unpack.py:177-196; the affine (min/max) form is the extension
// documented in varq.h.
//
// Work decomposition: one lane owns an octet (8 consecutive channels, one
// 16-byte load for 16-bit inputs).  A group is LPG = group/8 adjacent lanes, so
// the min/max reduction is a DPP butterfly inside the wavefront and never
// touches LDS.  A block covers octets of one (i0,i1) pair of the row map so
// that the output row offset is block-uniform.
#include "varq_common.h"

namespace {

struct RowsParams {
  const void *x;
  int32_t *words;
  float *scale;
  float *zp;
  const int32_t *slot;
  RowMap map;
  int64_t octets_per_pair;   // n2 * c8
  int64_t blocks_per_pair;
  int c8;                    // octets per row
  int c8_shift;              // log2(c8) or -1
  int nseg;                  // groups per row
  float eps;
};

// Division x/s for a whole octet with the quotient's rounding verified:
// y = x * (1/s) differs from the correctly rounded quotient by at most
// 0.75 * 2^-22 * |x/s|, so round(y) == round(x/s) whenever y is farther than
// `thr` = 2^-21 * max|x/s| from every half-integer.  Lanes where that cannot be
// shown redo the octet with the IEEE division.  Result: identical integers to
// torch.round(x32 / scale), at a third of the VALU cost.
template <int BITS, bool ASYM>
__device__ __forceinline__ void quantize_octet(const float (&v)[8], float s, float zp, float amax,
                                               u32 &w0, u32 &w1) {
  constexpr float kMin = (float)QRange<BITS>::kMin, kMax = (float)QRange<BITS>::kMax;
  const float r = 1.0f / s;
  const float thr = amax * r * 0x1p-21f;
  const float lim = 0.5f - thr;
  float n[8];
  bool redo = !(s < 0x1p125f);  // 1/s would be subnormal: bound does not hold
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float y = v[j] * r;
    n[j] = rintf(y);
    float d = y - n[j];
    redo |= !(fabsf(d) < lim);  // also true for NaN/inf and for thr >= 0.5
  }
  if (redo) {
#pragma unroll
    for (int j = 0; j < 8; ++j) n[j] = rintf(v[j] / s);
  }
  u32 acc = 0;
  w0 = 0; w1 = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float u = ASYM ? (n[j] + zp) : n[j];
    u = __builtin_amdgcn_fmed3f(u, kMin, kMax);
    int q = (int)u;
    acc = __builtin_amdgcn_alignbit((u32)q, acc, BITS);
    if (BITS == 8 && j == 3) { w0 = acc; acc = 0; }
  }
  if (BITS == 8) w1 = acc;
  else if (BITS == 4) w0 = acc;
  else w0 = acc >> 16;  // 2-bit: this octet's 16 bits, low half
}

template <int DT, int BITS, bool ASYM, int LPG>
__global__ __launch_bounds__(256) void quant_pack_rows_kernel(RowsParams p) {
  // grid = (tiles of one pair, n1, n0): no division to find the pair
  const int64_t i0 = blockIdx.z, i1 = blockIdx.y;
  const int64_t pair = i0 * p.map.n1 + i1;
  const int tile = blockIdx.x;

  int64_t s0 = i0, s1 = i1;
  if (p.map.slot_dim == 0) s0 = p.slot[i0];
  if (p.map.slot_dim == 1) s1 = p.slot[i1];
  if (s0 < 0 || s1 < 0) return;  // block-uniform: this head is not in the class
  const int64_t out_base = s0 * p.map.os0 + s1 * p.map.os1 + p.map.off;

  const int o = tile * 256 + (int)threadIdx.x;      // octet index inside the pair
  const bool live = o < (int)p.octets_per_pair;
  const int oc = live ? o : 0;                        // clamp: dead lanes still join the DPP
  const int64_t in_elem = (pair * p.octets_per_pair + oc) * 8;

  float v[8];
  In8<DT>::load(p.x, in_elem, v);

  float mn, mx;
  if (ASYM) {
    mn = fminf(fminf(fminf(v[0], v[1]), fminf(v[2], v[3])), fminf(fminf(v[4], v[5]), fminf(v[6], v[7])));
    mx = fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7])));
    mn = group_allreduce<LPG, false>(mn);
    mx = group_allreduce<LPG, true>(mx);
  } else {
    mx = fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
               fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7]))));
    mx = group_allreduce<LPG, true>(mx);
    mn = 0.f;
  }

  float s, zp = 0.f, amax;
  if (ASYM) {
    s = fmaxf((mx - mn) / (float)QRange<BITS>::kLevels, p.eps);
    zp = (float)QRange<BITS>::kMin - rintf(mn / s);
    amax = fmaxf(fabsf(mn), fabsf(mx));
  } else {
    s = fmaxf(mx / (float)QRange<BITS>::kMax, p.eps);
    amax = mx;
  }

  u32 w0, w1;
  quantize_octet<BITS, ASYM>(v, s, zp, amax, w0, w1);
  if (BITS == 2) {
    // two adjacent lanes hold the halves of one word
    u32 other = (u32)__builtin_amdgcn_update_dpp(0, (int)w0, 0xB1, 0xf, 0xf, false);
    w0 |= other << 16;
  }
  if (!live) return;

  int i2, col;
  if (p.c8_shift >= 0) { i2 = oc >> p.c8_shift; col = oc & (p.c8 - 1); }
  else { i2 = oc / p.c8; col = oc - i2 * p.c8; }
  if (p.map.slot_dim == 2) {
    i2 = p.slot[i2];
    if (i2 < 0) return;
  }
  const int64_t out_row = out_base + (int64_t)i2 * p.map.os2;

  if (BITS == 8) {
    uint2 *dst = reinterpret_cast<uint2 *>(p.words + (out_row * p.c8 + col) * 2);
    *dst = make_uint2(w0, w1);
  } else if (BITS == 4) {
    p.words[out_row * p.c8 + col] = (int32_t)w0;
  } else {
    if ((threadIdx.x & 1) == 0) p.words[(out_row * p.c8 + col) >> 1] = (int32_t)w0;
  }
  if ((col & (LPG - 1)) == 0) {
    const int64_t g = out_row * p.nseg + col / LPG;
    p.scale[g] = s;
    if (ASYM) p.zp[g] = zp;
  }
}

template <int DT, int BITS, bool ASYM>
int launch_lpg(const RowsParams &p, int lpg, dim3 grid, hipStream_t st) {
  switch (lpg) {
#define VARQ_CASE(L)                                                                     \
  case L:                                                                                \
    hipLaunchKernelGGL((quant_pack_rows_kernel<DT, BITS, ASYM, L>), grid, dim3(256), 0, st, p); \
    return 0;
    VARQ_CASE(1) VARQ_CASE(2) VARQ_CASE(4) VARQ_CASE(8) VARQ_CASE(16) VARQ_CASE(32) VARQ_CASE(64)
#undef VARQ_CASE
  }
  return -1;
}

template <int DT>
int launch_dt(const RowsParams &p, int bits, int asym, int lpg, dim3 grid, hipStream_t st) {
  if (bits == 8) return asym ? launch_lpg<DT, 8, true>(p, lpg, grid, st) : launch_lpg<DT, 8, false>(p, lpg, grid, st);
  if (bits == 4) return asym ? launch_lpg<DT, 4, true>(p, lpg, grid, st) : launch_lpg<DT, 4, false>(p, lpg, grid, st);
  if (bits == 2) return asym ? launch_lpg<DT, 2, true>(p, lpg, grid, st) : launch_lpg<DT, 2, false>(p, lpg, grid, st);
  return -1;
}

}  // namespace

extern "C" int varq_quant_pack_rows(const void *x, int x_dtype, int64_t n_rows, int c, int group, int bits,
                                    int asym, float eps, const int64_t *host_rowmap, const int32_t *slot,
                                    int32_t *words, float *scale, float *zp, void *stream) {
  VARQ_CHECK_ARG(n_rows == 0 || (x && words && scale), "quant_pack_rows: null pointer");
  VARQ_CHECK_ARG(n_rows == 0 || !asym || zp, "quant_pack_rows: asym needs zp output");
  VARQ_CHECK_ARG(bits == 2 || bits == 4 || bits == 8, "quant_pack_rows: bits must be 2, 4 or 8 (got %d)", bits);
  VARQ_CHECK_ARG(x_dtype >= 0 && x_dtype <= 2, "quant_pack_rows: bad dtype %d", x_dtype);
  VARQ_CHECK_ARG(n_rows >= 0 && c > 0, "quant_pack_rows: bad shape");
  VARQ_CHECK_ARG(c % 8 == 0 && (c * bits) % 32 == 0, "quant_pack_rows: c=%d must be a multiple of 8 and fill whole words", c);
  VARQ_CHECK_ARG(group > 0 && group % 8 == 0 && c % group == 0, "quant_pack_rows: group=%d must be a multiple of 8 dividing c=%d", group, c);
  const int lpg = group / 8;
  VARQ_CHECK_ARG(varq_log2_exact(lpg) >= 0 && lpg <= 64, "quant_pack_rows: group/8=%d must be a power of two <= 64", lpg);
  RowMap m = varq_rowmap_from_host(host_rowmap, n_rows);
  VARQ_CHECK_ARG(m.n0 >= 0 && m.n1 >= 0 && m.n2 >= 0 && m.n0 * m.n1 * m.n2 == n_rows, "quant_pack_rows: row map does not cover n_rows");
  VARQ_CHECK_ARG(m.slot_dim >= -1 && m.slot_dim <= 2 && (m.slot_dim < 0 || slot), "quant_pack_rows: slot table missing");
  if (n_rows == 0) return VARQ_OK;

  RowsParams p;
  p.x = x; p.words = words; p.scale = scale; p.zp = zp; p.slot = slot; p.map = m;
  p.c8 = c / 8;
  p.c8_shift = varq_log2_exact(p.c8);
  p.nseg = c / group;
  p.eps = eps;
  p.octets_per_pair = m.n2 * p.c8;
  p.blocks_per_pair = (p.octets_per_pair + 255) / 256;
  VARQ_CHECK_ARG(p.octets_per_pair < (1ll << 31) - 256, "quant_pack_rows: more than 2^31 octets per (i0,i1) pair");
  VARQ_CHECK_ARG(m.n1 <= 65535 && m.n0 <= 65535, "quant_pack_rows: n0 and n1 of the row map must be <= 65535");
  dim3 grid((unsigned)p.blocks_per_pair, (unsigned)m.n1, (unsigned)m.n0);
  hipStream_t st = (hipStream_t)stream;
  int rc = -1;
  if (x_dtype == VARQ_F32) rc = launch_dt<VARQ_F32>(p, bits, asym, lpg, grid, st);
  else if (x_dtype == VARQ_BF16) rc = launch_dt<VARQ_BF16>(p, bits, asym, lpg, grid, st);
  else rc = launch_dt<VARQ_F16>(p, bits, asym, lpg, grid, st);
  if (rc) return varq_set_error(VARQ_ERR_UNSUPPORTED, "quant_pack_rows: no kernel for this configuration");
  VARQ_CHECK_LAUNCH("quant_pack_rows");
  return VARQ_OK;
}

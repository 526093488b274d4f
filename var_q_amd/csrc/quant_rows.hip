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
//
// Which of the map's inner two dims is the block-uniform one is the launcher's
// choice: the rows a block walks should be the ones that lie next to each other
// in the OUTPUT.  For K and V in [B, L, H, c] order going into a [B, H, Lmax]
// cache (VAR_Q/quant.py:196-201 after the transpose of
// Infinity/infinity/models/basic.py:330) a block therefore takes tokens l.. of
// one head - 2c-byte pieces H*2c bytes apart on the input side, whole
// contiguous stretches of packed words, scales and zero-points on the output
// side - instead of the H heads of one token, whose packed rows lie Lmax rows
// apart (64-byte stores all over the cache, a quarter of the lanes at work for
// H = 16: 0.34 of HBM peak where the other order reaches 0.72).
#include <type_traits>
#include "varq_common.h"

namespace {

struct RowsParams {
  const void *x;
  int32_t *words;
  float *scale;
  float *zp;
  // a second tensor of the same shape (K and V of one cache step in one launch), or NULLs;
  // it takes the upper half of grid.z
  const void *x1;
  int32_t *words1;
  float *scale1;
  float *zp1;
  const int32_t *slot;
  RowMap map;                // as the kernel walks it: n1 is uniform per workgroup, n2 the rows inside
  // element offset of row (i0, i1, i2) of the input: i0 * in_s0 + i1 * in_s1 + i2 * in_s2.  For an
  // input in the order of the map, in_s2 = c; when the launcher has swapped the roles of the map's
  // inner two dims (below), the rows of a workgroup lie in_s2 > c elements apart.
  int64_t in_s0, in_s1, in_s2;
  bool strided;              // in_s2 != c
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
  const bool second = blockIdx.z >= (unsigned)p.map.n0;   // block-uniform
  const void *px = second ? p.x1 : p.x;
  int32_t *pwords = second ? p.words1 : p.words;
  float *pscale = second ? p.scale1 : p.scale;
  float *pzp = second ? p.zp1 : p.zp;
  // (strided input: the pair index is the fastest grid dim, see the launcher)
  const int64_t i0 = blockIdx.z - (second ? (unsigned)p.map.n0 : 0u), i1 = p.strided ? blockIdx.x : blockIdx.y;
  const int tile = p.strided ? blockIdx.y : blockIdx.x;

  int64_t s0 = i0, s1 = i1;
  if (p.map.slot_dim == 0) s0 = p.slot[i0];
  if (p.map.slot_dim == 1) s1 = p.slot[i1];
  if (s0 < 0 || s1 < 0) return;  // block-uniform: this head is not in the class
  const int64_t out_base = s0 * p.map.os0 + s1 * p.map.os1 + p.map.off;

  const int o = tile * 256 + (int)threadIdx.x;      // octet index inside the pair
  const bool live = o < (int)p.octets_per_pair;
  const int oc = live ? o : 0;                        // clamp: dead lanes still join the DPP
  int64_t in_elem = i0 * p.in_s0 + i1 * p.in_s1;
  if (p.strided) in_elem += (oc >> p.c8_shift) * (int)p.in_s2 + (oc & (p.c8 - 1)) * 8;   // (c8 is a power of two, the extent fits 31 bits)
  else in_elem += (int64_t)oc * 8;

  float v[8];
  In8<DT>::load(px, in_elem, v);

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
    uint2 *dst = reinterpret_cast<uint2 *>(pwords + (out_row * p.c8 + col) * 2);
    *dst = make_uint2(w0, w1);
  } else if (BITS == 4) {
    pwords[out_row * p.c8 + col] = (int32_t)w0;
  } else {
    if ((threadIdx.x & 1) == 0) pwords[(out_row * p.c8 + col) >> 1] = (int32_t)w0;
  }
  if ((col & (LPG - 1)) == 0) {
    const int64_t g = out_row * p.nseg + col / LPG;
    pscale[g] = s;
    if (ASYM) pzp[g] = zp;
  }
}

// ---- wide variant: one lane owns 4 octets (32 channels) of one group ---------
// Used for groups of 32 channels and more.  The per-group work (one IEEE fp32
// division for the scale, one fp64 reciprocal, the cross-lane reduce) is
// amortized over 32 elements instead of 8.  A group is LPG4 = group/32 adjacent
// lanes; lane j owns octets j, j+LPG4, j+2*LPG4, j+3*LPG4 of its group.
//
// HBM side: every global load and (in the common dense-output case) every
// global store instruction of a wavefront touches 1 KiB of contiguous memory.
// The change of layout between "contiguous per instruction" and "32 channels of
// one group per lane" goes through a 4 KiB wave-private LDS window, so there is
// no workgroup barrier anywhere.
//
// Rounding: x/s is needed exactly as an IEEE fp32 division rounds it; see the
// two routes (fp32 correction step, fp64 product) in the kernel body.
template <int DT, int BITS, bool ASYM, int LPG4, bool DENSE>
__global__ __launch_bounds__(256) void quant_pack_rows32_kernel(RowsParams p) {
  __shared__ Raw8<DT> lds_stage[4][256];   // per wave: 256 octets in, then packed words out

  const bool second = blockIdx.z >= (unsigned)p.map.n0;   // block-uniform
  const void *px = second ? p.x1 : p.x;
  int32_t *pwords = second ? p.words1 : p.words;
  float *pscale = second ? p.scale1 : p.scale;
  float *pzp = second ? p.zp1 : p.zp;
  const int64_t i0 = blockIdx.z - (second ? (unsigned)p.map.n0 : 0u), i1 = p.strided ? blockIdx.x : blockIdx.y;
  const int tile = p.strided ? blockIdx.y : blockIdx.x;
  int64_t s0 = i0, s1 = i1;
  if (p.map.slot_dim == 0) s0 = p.slot[i0];
  if (p.map.slot_dim == 1) s1 = p.slot[i1];
  if (s0 < 0 || s1 < 0) return;
  const int64_t out_base = s0 * p.map.os0 + s1 * p.map.os1 + p.map.off;
  const int64_t pair_elem0 = i0 * p.in_s0 + i1 * p.in_s1;

  const int n_oct = (int)p.octets_per_pair;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  Raw8<DT> *stage = lds_stage[wv];
  constexpr float kMin = (float)QRange<BITS>::kMin, kMax = (float)QRange<BITS>::kMax;
  const int w0 = tile * 1024 + wv * 256;             // first octet of this wave's window, inside the pair

  // 1 KiB per load instruction: contiguous, or whole rows in_s2 elements apart.  Only the
  // offsets are formed under the (launch-uniform) branch; the four loads follow it together.
  int64_t e[4];
  if (!p.strided) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int o = w0 + k * 64 + lane;
      e[k] = (int64_t)(o < n_oct ? o : 0) * 8;          // past the end: re-read octet 0, never stored
    }
  } else {
    const int s2 = (int)p.in_s2;                        // (the pair's extent fits 31 bits: checked on the host)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      int o = w0 + k * 64 + lane;
      o = o < n_oct ? o : 0;
      e[k] = (o >> p.c8_shift) * s2 + (o & (p.c8 - 1)) * 8;
    }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    Raw8<DT> r;
    r.load(px, pair_elem0 + e[k]);
    stage[k * 64 + lane] = r;
  }
  __builtin_amdgcn_wave_barrier();

  // lane-owned octets inside the wave window
  const int j = lane & (LPG4 - 1);
  const int loc0 = ((lane - j) << 2) + j;
  float v[4][8];
#pragma unroll
  for (int k = 0; k < 4; ++k) stage[loc0 + k * LPG4].widen(v[k]);

  float mn = 0.f, mx;
  if (ASYM) {
    mn = v[0][0]; mx = v[0][0];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) { mn = fminf(mn, v[k][e]); mx = fmaxf(mx, v[k][e]); }
    mn = group_allreduce<LPG4, false>(mn);
    mx = group_allreduce<LPG4, true>(mx);
  } else {
    mx = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) mx = fmaxf(mx, fabsf(v[k][e]));
    mx = group_allreduce<LPG4, true>(mx);
  }

  float s, zp = 0.f;
  if (ASYM) s = fmaxf((mx - mn) / (float)QRange<BITS>::kLevels, p.eps);
  else s = fmaxf(mx / kMax, p.eps);

  // x/s exactly as an IEEE fp32 division rounds it, in three full-rate
  // instructions: with r = RN(1/s), q0 = RN(x*r) is within an ulp of the quotient,
  // e = x - q0*s is exact in one fma, and RN(q0 + e*r) is the correctly rounded
  // quotient (Markstein's correction step).  That holds for every finite x unless
  // the significand of s is all ones or the residual can underflow; such groups,
  // and zero-points beyond 2^21 (the clamped quotient, up to 128 beyond the zero-point, must stay
  // inside +-2^22 for the rounding trick below), take the fp64 route below.
  const float r = 1.0f / s;
  const bool plain = s > 0x1p-96f && s < 0x1p96f && (f2u(s) & 0x7fffffu) != 0x7fffffu;
  auto quotient = [&](float x) {
    const float q0 = x * r;
    const float e = __builtin_fmaf(-q0, s, x);
    return __builtin_fmaf(e, r, q0);
  };
  const bool wave_plain = __builtin_amdgcn_ballot_w64(!plain) == 0;
  if (ASYM) zp = kMin - rintf(wave_plain ? quotient(mn) : mn / s);
  const bool big_zp = ASYM && !(fabsf(zp) <= 0x1p21f);

  // Codes: clamp(rint(t) + zp, qmin, qmax) = rint(clamp(t, qmin - zp, qmax - zp)) + zp
  // (the bounds are integers).  Adding 1.5 * 2^23 rounds the clamped quotient to
  // nearest-even and leaves the integer in the low mantissa bits; the zero-point
  // is then added to all fields of a packed word at once, modulo the field width
  // (the sum is known to fit the field).
  const float lo = kMin - zp, hi = kMax - zp;
  constexpr u32 kFieldHi = BITS == 8 ? 0x80808080u : BITS == 4 ? 0x88888888u : 0xaaaaaaaau;
  constexpr u32 kFieldLsb = BITS == 8 ? 0x01010101u : BITS == 4 ? 0x11111111u : 0x55555555u;
  const u32 zrep = ((u32)(int)zp & ((1u << BITS) - 1u)) * kFieldLsb;
  const u32 zlo = zrep & ~kFieldHi, zhi = zrep & kFieldHi;
  auto add_zp = [&](u32 wd) { return ASYM ? (((wd & ~kFieldHi) + zlo) ^ (wd & kFieldHi) ^ zhi) : wd; };
  u32 w[4][2];
  auto quantize_all = [&](auto exact64) {
    double rinv = 0.0;
    if (decltype(exact64)::value) rinv = 1.0 / (double)s;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      u32 acc = 0;
      w[k][0] = 0; w[k][1] = 0;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        u32 q;
        if (decltype(exact64)::value) {
          // fp64 product x * RN64(1/s): within 2^-52 of the quotient, which is never that
          // close to a point where rounding to fp32 changes, so narrowing it is exact too
          const float t = rintf((float)((double)v[k][e] * rinv));
          q = (u32)(int)__builtin_amdgcn_fmed3f(ASYM ? t + zp : t, kMin, kMax);
        } else {
          q = f2u(__builtin_amdgcn_fmed3f(quotient(v[k][e]), lo, hi) + 12582912.f);
        }
        acc = __builtin_amdgcn_alignbit(q, acc, BITS);
        if (BITS == 8 && e == 3) { w[k][0] = acc; acc = 0; }
      }
      if (BITS == 8) w[k][1] = acc;
      else if (BITS == 4) w[k][0] = acc;
      else w[k][0] = acc >> 16;
      if (!decltype(exact64)::value) {
        w[k][0] = add_zp(w[k][0]);
        if (BITS == 8) w[k][1] = add_zp(w[k][1]);
        if (BITS == 2) w[k][0] &= 0xffffu;
      }
    }
  };
  if (!wave_plain || __builtin_amdgcn_ballot_w64(big_zp) != 0) quantize_all(std::true_type{});   // wave-uniform, rare
  else quantize_all(std::false_type{});
  if (BITS == 2 && LPG4 > 1) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      u32 other = (u32)__builtin_amdgcn_update_dpp(0, (int)w[k][0], 0xB1, 0xf, 0xf, false);
      w[k][0] |= other << 16;
    }
  }

  const int oct0 = w0 + loc0;                         // first owned octet, inside the pair
  const bool live = oct0 < n_oct;                     // groups never straddle the end

  if (DENSE) {
    // output rows of the pair are consecutive: word, scale and zp indices follow
    // the pair-local octet index directly
    if (BITS == 4) {
      // packed words back to global order through the same window, 16 B per lane
      typedef u32 u32x4 __attribute__((ext_vector_type(4)));
      u32 *wstage = reinterpret_cast<u32 *>(stage);
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int k = 0; k < 4; ++k) wstage[loc0 + k * LPG4] = w[k][0];
      __builtin_amdgcn_wave_barrier();
      const u32x4 out4 = reinterpret_cast<const u32x4 *>(wstage)[lane];
      const int o = w0 + 4 * lane;                    // octet == word index for 4-bit codes
      if (o < n_oct)
        __builtin_nontemporal_store(out4, reinterpret_cast<u32x4 *>(pwords + out_base * p.c8 + o));
    } else if (live) {
      const int64_t wbase = out_base * p.c8 + oct0;   // in octets
      if (BITS == 8) {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          *reinterpret_cast<uint2 *>(pwords + (wbase + k * LPG4) * 2) = make_uint2(w[k][0], w[k][1]);
      } else if (LPG4 == 1) {
        *reinterpret_cast<uint2 *>(pwords + (wbase >> 1)) =
            make_uint2(w[0][0] | (w[1][0] << 16), w[2][0] | (w[3][0] << 16));
      } else if ((j & 1) == 0) {
#pragma unroll
        for (int k = 0; k < 4; ++k) pwords[(wbase + k * LPG4) >> 1] = (int32_t)w[k][0];
      }
    }
    if (live && j == 0) {
      const int64_t g = out_base * p.nseg + oct0 / (4 * LPG4);
      pscale[g] = s;
      if (ASYM) pzp[g] = zp;
    }
    return;
  }

  if (!live) return;
  int i2, col;
  if (p.c8_shift >= 0) { i2 = oct0 >> p.c8_shift; col = oct0 & (p.c8 - 1); }
  else { i2 = oct0 / p.c8; col = oct0 - i2 * p.c8; }
  if (p.map.slot_dim == 2) i2 = p.slot[i2];
  if (i2 < 0) return;
  const int64_t out_row = out_base + (int64_t)i2 * p.map.os2;
  const int64_t wbase = out_row * p.c8 + col;            // in octets
  if (BITS == 8) {
#pragma unroll
    for (int k = 0; k < 4; ++k)
      *reinterpret_cast<uint2 *>(pwords + (wbase + k * LPG4) * 2) = make_uint2(w[k][0], w[k][1]);
  } else if (BITS == 4) {
    if (LPG4 == 1) {
      *reinterpret_cast<uint4 *>(pwords + wbase) = make_uint4(w[0][0], w[1][0], w[2][0], w[3][0]);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) pwords[wbase + k * LPG4] = (int32_t)w[k][0];
    }
  } else {
    if (LPG4 == 1) {
      *reinterpret_cast<uint2 *>(pwords + (wbase >> 1)) =
          make_uint2(w[0][0] | (w[1][0] << 16), w[2][0] | (w[3][0] << 16));
    } else if ((j & 1) == 0) {
#pragma unroll
      for (int k = 0; k < 4; ++k) pwords[(wbase + k * LPG4) >> 1] = (int32_t)w[k][0];
    }
  }
  if (j == 0) {
    const int64_t g = out_row * p.nseg + col / (4 * LPG4);
    pscale[g] = s;
    if (ASYM) pzp[g] = zp;
  }
}

template <int DT, int BITS, bool ASYM>
int launch_lpg(const RowsParams &p, int lpg, dim3 grid, hipStream_t st) {
  if (lpg >= 4) {   // groups of >= 32 channels: 4 octets per lane, 1024 octets per workgroup
    const unsigned t32 = (unsigned)((p.octets_per_pair + 1023) / 1024);
    dim3 g32(p.strided ? grid.x : t32, p.strided ? t32 : grid.y, grid.z);
    const bool dense = (p.map.os2 == 1) && (p.map.slot_dim != 2);
    switch (lpg / 4) {
#define VARQ_CASE32(L)                                                                                            \
  case L:                                                                                                         \
    if (dense) hipLaunchKernelGGL((quant_pack_rows32_kernel<DT, BITS, ASYM, L, true>), g32, dim3(256), 0, st, p); \
    else hipLaunchKernelGGL((quant_pack_rows32_kernel<DT, BITS, ASYM, L, false>), g32, dim3(256), 0, st, p);      \
    return 0;
      VARQ_CASE32(1) VARQ_CASE32(2) VARQ_CASE32(4) VARQ_CASE32(8) VARQ_CASE32(16)
#undef VARQ_CASE32
    }
    return -1;
  }
  switch (lpg) {
#define VARQ_CASE(L)                                                                     \
  case L:                                                                                \
    hipLaunchKernelGGL((quant_pack_rows_kernel<DT, BITS, ASYM, L>), grid, dim3(256), 0, st, p); \
    return 0;
    VARQ_CASE(1) VARQ_CASE(2)
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

static int quant_pack_rows_launch(const char *who, const void *x, const void *x1, int x_dtype, int64_t n_rows, int c,
                                  int group, int bits, int asym, float eps, const int64_t *host_rowmap,
                                  const int32_t *slot, int32_t *words, float *scale, float *zp, int32_t *words1,
                                  float *scale1, float *zp1, void *stream) {
  const bool two = x1 != nullptr;
  VARQ_CHECK_ARG(n_rows == 0 || (x && words && scale), "%s: null pointer", who);
  VARQ_CHECK_ARG(n_rows == 0 || !asym || zp, "%s: asym needs zp output", who);
  VARQ_CHECK_ARG(n_rows == 0 || !two || (words1 && scale1 && (!asym || zp1)), "%s: outputs of the second tensor missing", who);
  VARQ_CHECK_ARG(bits == 2 || bits == 4 || bits == 8, "%s: bits must be 2, 4 or 8 (got %d)", who, bits);
  VARQ_CHECK_ARG(x_dtype >= 0 && x_dtype <= 2, "%s: bad dtype %d", who, x_dtype);
  VARQ_CHECK_ARG(n_rows >= 0 && c > 0, "%s: bad shape", who);
  VARQ_CHECK_ARG(c % 8 == 0 && (c * bits) % 32 == 0, "%s: c=%d must be a multiple of 8 and fill whole words", who, c);
  VARQ_CHECK_ARG(group > 0 && group % 8 == 0 && c % group == 0, "%s: group=%d must be a multiple of 8 dividing c=%d", who, group, c);
  const int lpg = group / 8;
  VARQ_CHECK_ARG(varq_log2_exact(lpg) >= 0 && lpg <= 64, "%s: group/8=%d must be a power of two <= 64 (group <= 512)", who, lpg);
  RowMap m = varq_rowmap_from_host(host_rowmap, n_rows);
  VARQ_CHECK_ARG(m.n0 >= 0 && m.n1 >= 0 && m.n2 >= 0 && m.n0 * m.n1 * m.n2 == n_rows, "%s: row map does not cover n_rows", who);
  VARQ_CHECK_ARG(m.slot_dim >= -1 && m.slot_dim <= 2 && (m.slot_dim < 0 || slot), "%s: slot table missing", who);
  if (n_rows == 0) return VARQ_OK;

  RowsParams p;
  p.x = x; p.words = words; p.scale = scale; p.zp = zp; p.slot = slot;
  p.x1 = x1; p.words1 = words1; p.scale1 = scale1; p.zp1 = zp1;
  p.c8 = c / 8;
  p.c8_shift = varq_log2_exact(p.c8);
  p.in_s0 = m.n1 * m.n2 * c; p.in_s1 = m.n2 * c; p.in_s2 = c;
  // The rows a workgroup walks should be neighbours in the output: if those are the rows along
  // the map's middle dim (and there are at least as many of them as along the inner one), the
  // two dims change roles and the workgroup reads its rows n2 * c elements apart.
  if (m.os1 == 1 && m.os2 != 1 && m.slot_dim != 1 && p.c8_shift >= 0 && m.n1 >= m.n2 && m.n1 * m.n2 * c < (1ll << 31) &&
      (m.n1 * p.c8 + 255) / 256 <= 65535) {
    RowMap t = m;
    t.n1 = m.n2; t.n2 = m.n1; t.os1 = m.os2; t.os2 = m.os1;
    t.slot_dim = m.slot_dim == 2 ? 1 : m.slot_dim;
    p.in_s1 = c; p.in_s2 = m.n2 * c;
    m = t;
  }
  p.strided = p.in_s2 != c;
  p.map = m;
  p.nseg = c / group;
  p.eps = eps;
  p.octets_per_pair = m.n2 * p.c8;
  p.blocks_per_pair = (p.octets_per_pair + 255) / 256;
  VARQ_CHECK_ARG(p.octets_per_pair < (1ll << 31) - 256, "%s: more than 2^31 octets per (i0,i1) pair", who);
  VARQ_CHECK_ARG(m.n1 <= 65535 && m.n0 * (two ? 2 : 1) <= 65535, "%s: n0 (times the number of tensors) and n1 of the row map must be <= 65535", who);
  // strided input: the workgroups in flight together should read whole stretches of the input
  // between them, so the pair index (the head, for [B, L, H, c] input) is the fastest grid dim
  // and the tiles of tokens lie along y (their count was bounded where the roles were swapped)
  dim3 grid((unsigned)p.blocks_per_pair, (unsigned)m.n1, (unsigned)(m.n0 * (two ? 2 : 1)));
  if (p.strided) grid = dim3((unsigned)m.n1, (unsigned)p.blocks_per_pair, grid.z);
  hipStream_t st = (hipStream_t)stream;
  int rc = -1;
  if (x_dtype == VARQ_F32) rc = launch_dt<VARQ_F32>(p, bits, asym, lpg, grid, st);
  else if (x_dtype == VARQ_BF16) rc = launch_dt<VARQ_BF16>(p, bits, asym, lpg, grid, st);
  else rc = launch_dt<VARQ_F16>(p, bits, asym, lpg, grid, st);
  if (rc) return varq_set_error(VARQ_ERR_UNSUPPORTED, "%s: no kernel for this configuration", who);
  VARQ_CHECK_LAUNCH(who);
  return VARQ_OK;
}

extern "C" int varq_quant_pack_rows(const void *x, int x_dtype, int64_t n_rows, int c, int group, int bits,
                                    int asym, float eps, const int64_t *host_rowmap, const int32_t *slot,
                                    int32_t *words, float *scale, float *zp, void *stream) {
  return quant_pack_rows_launch("quant_pack_rows", x, nullptr, x_dtype, n_rows, c, group, bits, asym, eps, host_rowmap, slot,
                                words, scale, zp, nullptr, nullptr, nullptr, stream);
}

extern "C" int varq_quant_pack_rows2(const void *x0, const void *x1, int x_dtype, int64_t n_rows, int c, int group,
                                     int bits, int asym, float eps, const int64_t *host_rowmap, const int32_t *slot,
                                     int32_t *words0, float *scale0, float *zp0, int32_t *words1, float *scale1,
                                     float *zp1, void *stream) {
  VARQ_CHECK_ARG(n_rows == 0 || x1, "quant_pack_rows2: null pointer");
  return quant_pack_rows_launch("quant_pack_rows2", x0, x1, x_dtype, n_rows, c, group, bits, asym, eps, host_rowmap, slot,
                                words0, scale0, zp0, words1, scale1, zp1, stream);
}

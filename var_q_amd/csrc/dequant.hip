// Unpack + dequantize in one pass: what VAR_Q/quant.py:216-224 does with two
// unpack launches per field, a stack, a sign-extension and a multiply
// (VAR_Q/pack_unpack.py:198-211, VAR_Q/quant.py:123-124), plus the affine form
// (q - zp) * scale.  HBM-bound; the output (fp32 in the reference, 4 B/element)
// dominates the traffic, so bf16/fp16 outputs are offered too.
//
// One lane produces 8 consecutive channels.  A block stays inside one (i0,i1)
// pair so the scale base and the input-window row base are block-uniform.
#include "varq_common.h"

namespace {

struct DeqParams {
  const int32_t *words;
  const int8_t *codes;
  const float *scale;
  const float *zp;
  void *out;
  RowMap in_map;           // (i0,i1,i2) -> input row
  int64_t n1, n2;
  int64_t ss0, ss1, ss2, ss3;
  int64_t octets_per_pair;
  int c, c8, wpr, bits, group;
  int c8_shift;            // log2(c8) when c8 is a power of two, else -1
  int g8_shift;            // log2(group / 8) when group is 8 times a power of two, else -1
};

template <int ODT> __device__ __forceinline__ void store8(void *out, int64_t elem, const float (&f)[8], int n_valid) {
  if (ODT == VARQ_F32) {
    float *o = reinterpret_cast<float *>(out) + elem;
    if (n_valid == 8) {
      reinterpret_cast<float4 *>(o)[0] = make_float4(f[0], f[1], f[2], f[3]);
      reinterpret_cast<float4 *>(o)[1] = make_float4(f[4], f[5], f[6], f[7]);
    } else {
      for (int j = 0; j < n_valid; ++j) o[j] = f[j];
    }
  } else {
    uint16_t *o = reinterpret_cast<uint16_t *>(out) + elem;
    if (ODT == VARQ_BF16 && n_valid == 8) {
      // hardware round-to-nearest-even conversion, two values per instruction
      typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
      typedef float f2 __attribute__((ext_vector_type(2)));
      u32 w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f2 v = {f[2 * j], f[2 * j + 1]};
        w[j] = __builtin_bit_cast(u32, __builtin_convertvector(v, bf2));
      }
      *reinterpret_cast<uint4 *>(o) = make_uint4(w[0], w[1], w[2], w[3]);
      return;
    }
    uint16_t h[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) h[j] = (ODT == VARQ_BF16) ? f32_to_bf16_rne(f[j]) : f32_to_f16_rne(f[j]);
    if (n_valid == 8) {
      *reinterpret_cast<uint4 *>(o) = make_uint4(h[0] | ((u32)h[1] << 16), h[2] | ((u32)h[3] << 16),
                                                 h[4] | ((u32)h[5] << 16), h[6] | ((u32)h[7] << 16));
    } else {
      for (int j = 0; j < n_valid; ++j) o[j] = h[j];
    }
  }
}

// U items (octets) per lane, 256 lanes apart: all of a lane's loads are issued before the first
// of them is used, so a wavefront keeps U times the bytes in flight and the launch has a U-th of
// the wavefronts (with one item per lane the kernel is bound by wavefront turnover, not by
// bandwidth: 54-61 % of the HBM peak on the benchmark shapes against 62-70 % with four).
template <int ODT, int U>
__global__ __launch_bounds__(256) void dequant_kernel(DeqParams p) {
  // grid = (tiles of 256*U octets, i1, i0): no division to find the block's place
  const int64_t i0 = blockIdx.z, i1 = blockIdx.y;
  const int o0 = blockIdx.x * (256 * U) + threadIdx.x;   // first octet inside the (i0, i1) pair, < 2^31
  const int64_t sbase0 = i0 * p.ss0 + i1 * p.ss1;
  const int64_t in_base = i0 * p.in_map.os0 + i1 * p.in_map.os1 + p.in_map.off;
  const int64_t out_base = (i0 * p.n1 + i1) * p.n2;
  const bool words_ok = (p.c & 7) == 0 && p.words != nullptr &&
                        (p.bits != 8 || (reinterpret_cast<uintptr_t>(p.words) & 7) == 0);   // (block-uniform)
  // one scale per channel that does not depend on the token (a per-(head, channel) table), rows of
  // a power-of-two number of octets: the lane's U items are the same octet column of U tokens
  // and share one vector of 8 scales and 8 zero-points
  const bool chan = words_ok && p.group == 1 && p.ss3 == 1 && p.ss2 == 0 && p.c8_shift >= 0 && p.c8 <= 256 &&
                    ((sbase0 | (int64_t)(reinterpret_cast<uintptr_t>(p.scale) >> 2) |
                      (int64_t)(reinterpret_cast<uintptr_t>(p.zp) >> 2)) & 3) == 0;
  const bool fast = words_ok && (p.group & 7) == 0;
  if (fast || chan) {
    // packed words: one word (two for 8-bit codes) per item, and one scale and zero-point per
    // item (groups of whole octets) or the lane's vectors (per-channel tables)
    int w0[U], w1[U], i2v[U], colv[U];
    float sv[U], zv[U];
    bool live[U];
    float cs[8], cz[8];
    if (chan) {
      const int col = o0 & (p.c8 - 1);
      const float4 *sp = reinterpret_cast<const float4 *>(p.scale + sbase0 + col * 8);
      const float4 sa = sp[0], sb = sp[1];
      cs[0] = sa.x; cs[1] = sa.y; cs[2] = sa.z; cs[3] = sa.w; cs[4] = sb.x; cs[5] = sb.y; cs[6] = sb.z; cs[7] = sb.w;
#pragma unroll
      for (int j = 0; j < 8; ++j) cz[j] = 0.f;
      if (p.zp) {
        const float4 *zq = reinterpret_cast<const float4 *>(p.zp + sbase0 + col * 8);
        const float4 za = zq[0], zb = zq[1];
        cz[0] = za.x; cz[1] = za.y; cz[2] = za.z; cz[3] = za.w; cz[4] = zb.x; cz[5] = zb.y; cz[6] = zb.z; cz[7] = zb.w;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int o = o0 + u * 256;
      live[u] = o < p.octets_per_pair;
      const int oc = live[u] ? o : 0;
      int i2, col;
      if (p.c8_shift >= 0) { i2 = oc >> p.c8_shift; col = oc & (p.c8 - 1); }
      else { i2 = oc / p.c8; col = oc - i2 * p.c8; }
      i2v[u] = i2; colv[u] = col;
      const int32_t *src = p.words + (in_base + i2 * p.in_map.os2) * p.wpr;
      if (p.bits == 4) { w0[u] = src[col]; w1[u] = 0; }
      else if (p.bits == 8) { const int2 t = *reinterpret_cast<const int2 *>(src + col * 2); w0[u] = t.x; w1[u] = t.y; }
      else { w0[u] = src[col >> 1]; w1[u] = 0; }
      if (!chan) {
        const int gi = p.g8_shift >= 0 ? col >> p.g8_shift : col * 8 / p.group;   // (block-uniform choice)
        const int64_t g = sbase0 + i2 * p.ss2 + gi * p.ss3;
        sv[u] = p.scale[g];
        zv[u] = p.zp ? p.zp[g] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (!live[u]) continue;
      int q[8];
      if (p.bits == 4) {
#pragma unroll
        for (int j = 0; j < 8; ++j) q[j] = __builtin_amdgcn_sbfe(w0[u], 4 * j, 4);
      } else if (p.bits == 8) {
#pragma unroll
        for (int j = 0; j < 4; ++j) { q[j] = __builtin_amdgcn_sbfe(w0[u], 8 * j, 8); q[4 + j] = __builtin_amdgcn_sbfe(w1[u], 8 * j, 8); }
      } else {
        const int w = w0[u] >> ((colv[u] & 1) * 16);
#pragma unroll
        for (int j = 0; j < 8; ++j) q[j] = __builtin_amdgcn_sbfe(w, 2 * j, 2);
      }
      float f[8];
      if (chan) {
        // (the same two operations as the scalar form below, so the results are the same bits)
        if (p.zp) {
#pragma unroll
          for (int j = 0; j < 8; ++j) f[j] = ((float)q[j] - cz[j]) * cs[j];
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) f[j] = (float)q[j] * cs[j];
        }
      } else if (p.zp) {
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] = ((float)q[j] - zv[u]) * sv[u];
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] = (float)q[j] * sv[u];
      }
      store8<ODT>(p.out, (out_base + i2v[u]) * p.c + colv[u] * 8, f, 8);
    }
    return;
  }
#pragma unroll 1
  for (int u = 0; u < U; ++u) {
  const int o = o0 + u * 256;
  if (o >= p.octets_per_pair) return;
  int i2, col;
  if (p.c8_shift >= 0) { i2 = o >> p.c8_shift; col = o & (p.c8 - 1); }
  else { i2 = o / p.c8; col = o - i2 * p.c8; }
  const int ch0 = col * 8;
  const int n_valid = min(8, p.c - ch0);
  const int64_t in_row = in_base + i2 * p.in_map.os2;
  const int64_t out_row = out_base + i2;

  int q[8];
  if (p.codes) {
    const int8_t *src = p.codes + in_row * p.c + ch0;
    if (n_valid == 8 && (p.c & 7) == 0) {
      uint2 b = *reinterpret_cast<const uint2 *>(src);
#pragma unroll
      for (int j = 0; j < 4; ++j) { q[j] = __builtin_amdgcn_sbfe((int)b.x, 8 * j, 8); q[4 + j] = __builtin_amdgcn_sbfe((int)b.y, 8 * j, 8); }
    } else {
      for (int j = 0; j < 8; ++j) q[j] = j < n_valid ? src[j] : 0;
    }
  } else {
    const int32_t *src = p.words + in_row * p.wpr;
    if (p.bits == 4) {
      const int w = src[col];
#pragma unroll
      for (int j = 0; j < 8; ++j) q[j] = __builtin_amdgcn_sbfe(w, 4 * j, 4);
    } else if (p.bits == 8) {
      const int w0 = src[col * 2];
      const int w1 = (col * 2 + 1 < p.wpr) ? src[col * 2 + 1] : 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) { q[j] = __builtin_amdgcn_sbfe(w0, 8 * j, 8); q[4 + j] = __builtin_amdgcn_sbfe(w1, 8 * j, 8); }
    } else {
      const int w = src[col >> 1] >> ((col & 1) * 16);
#pragma unroll
      for (int j = 0; j < 8; ++j) q[j] = __builtin_amdgcn_sbfe(w, 2 * j, 2);
    }
  }

  const int64_t sbase = sbase0 + i2 * p.ss2;
  float f[8];
  if ((p.group & 7) == 0) {
    const int64_t g = sbase + (ch0 / p.group) * p.ss3;
    const float s = p.scale[g];
    if (p.zp) {
      const float z = p.zp[g];
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = ((float)q[j] - z) * s;
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = (float)q[j] * s;
    }
  } else if (p.group == 1 && p.ss3 == 1 && n_valid == 8 && ((sbase + ch0) & 3) == 0) {
    // one scale per channel, contiguous: two 16-byte loads
    const float4 *sp = reinterpret_cast<const float4 *>(p.scale + sbase + ch0);
    const float4 sa = sp[0], sb = sp[1];
    const float sv[8] = {sa.x, sa.y, sa.z, sa.w, sb.x, sb.y, sb.z, sb.w};
    if (p.zp) {
      const float4 *zq = reinterpret_cast<const float4 *>(p.zp + sbase + ch0);
      const float4 za = zq[0], zb = zq[1];
      const float zv[8] = {za.x, za.y, za.z, za.w, zb.x, zb.y, zb.z, zb.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = ((float)q[j] - zv[j]) * sv[j];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = (float)q[j] * sv[j];
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int ch = min(ch0 + j, p.c - 1);
      const int64_t g = sbase + (ch / p.group) * p.ss3;
      const float s = p.scale[g];
      f[j] = p.zp ? ((float)q[j] - p.zp[g]) * s : (float)q[j] * s;
    }
  }
  store8<ODT>(p.out, out_row * p.c + ch0, f, ((p.c & 7) == 0) ? 8 : n_valid);
  }
}

}  // namespace

extern "C" int varq_dequant(const int32_t *words, const int8_t *codes_i8, const float *scale, const float *zp,
                            const int64_t *host_shape4, const int64_t *host_scale_strides4, int group, int bits,
                            const int64_t *host_in_rowmap, void *out, int out_dtype, void *stream) {
  VARQ_CHECK_ARG(host_shape4 && host_scale_strides4, "dequant: null shape/strides");
  const int64_t *s = host_shape4;
  VARQ_CHECK_ARG(s[0] >= 0 && s[1] >= 0 && s[2] >= 0 && s[3] > 0 && s[3] <= (1 << 20), "dequant: bad shape");
  // (a tensor without rows may come as null pointers: nothing to do)
  if (s[0] * s[1] * s[2] == 0) return VARQ_OK;
  VARQ_CHECK_ARG((words != nullptr) != (codes_i8 != nullptr), "dequant: exactly one of words/codes must be given");
  VARQ_CHECK_ARG(!words || bits == 2 || bits == 4 || bits == 8, "dequant: bits must be 2, 4 or 8 (got %d)", bits);
  VARQ_CHECK_ARG(out_dtype >= 0 && out_dtype <= 2, "dequant: bad output dtype %d", out_dtype);
  VARQ_CHECK_ARG(group >= 1 && group <= s[3], "dequant: bad group %d", group);
  const int64_t rows = s[0] * s[1] * s[2];
  if (rows == 0) return VARQ_OK;
  VARQ_CHECK_ARG(scale && out, "dequant: null pointer");

  DeqParams p;
  p.words = words; p.codes = codes_i8; p.scale = scale; p.zp = zp; p.out = out;
  p.n1 = s[1]; p.n2 = s[2];
  p.c = (int)s[3];
  p.c8 = (p.c + 7) / 8;
  p.bits = bits; p.group = group;
  p.wpr = words ? (p.c + 32 / bits - 1) / (32 / bits) : 0;
  p.ss0 = host_scale_strides4[0]; p.ss1 = host_scale_strides4[1];
  p.ss2 = host_scale_strides4[2]; p.ss3 = host_scale_strides4[3];
  if (host_in_rowmap) {
    p.in_map = varq_rowmap_from_host(host_in_rowmap, rows);
    VARQ_CHECK_ARG(p.in_map.n0 == s[0] && p.in_map.n1 == s[1] && p.in_map.n2 == s[2], "dequant: row map dims differ from shape");
    VARQ_CHECK_ARG(p.in_map.slot_dim < 0, "dequant: slot tables are not supported on input maps");
  } else {
    p.in_map.n0 = s[0]; p.in_map.n1 = s[1]; p.in_map.n2 = s[2];
    p.in_map.os0 = s[1] * s[2]; p.in_map.os1 = s[2]; p.in_map.os2 = 1; p.in_map.off = 0; p.in_map.slot_dim = -1;
  }
  p.octets_per_pair = s[2] * p.c8;
  p.c8_shift = -1;
  p.g8_shift = -1;
  for (int sh = 0; sh < 20; ++sh) {
    if ((1 << sh) == p.c8) p.c8_shift = sh;
    if ((8 << sh) == group) p.g8_shift = sh;
  }
  // four items per lane where a pair has the work for it (the last block's idle lanes weigh less
  // than the wavefront turnover they save), one otherwise
  // (two where four would leave more than a twelfth of the last block's lanes idle; not for
  // per-channel tables, where a lane's pieces share one load of its eight scales and zero-points)
  int U = p.octets_per_pair >= 2048 ? 4 : 1;
  if (U == 4 && !(group == 1 && p.ss3 == 1 && p.ss2 == 0)) {
    const int64_t t4 = (p.octets_per_pair + 1023) / 1024;
    if ((t4 * 1024 - p.octets_per_pair) * 12 > t4 * 1024) U = 2;
  }
  const int64_t tiles = (p.octets_per_pair + 256 * U - 1) / (256 * U);
  // a pair with few rows wastes lanes of its last block only; pairs map to grid.y/z (limit 65535 each)
  VARQ_CHECK_ARG(p.octets_per_pair < (1ll << 31) - 1024 && s[1] <= 65535 && s[0] <= 65535, "dequant: shape exceeds the grid limits");
  dim3 grid((unsigned)tiles, (unsigned)s[1], (unsigned)s[0]);
  hipStream_t st = (hipStream_t)stream;
#define VARQ_DEQ(ODT_)                                                                       \
  do {                                                                                       \
    if (U == 4) hipLaunchKernelGGL((dequant_kernel<ODT_, 4>), grid, dim3(256), 0, st, p);    \
    else if (U == 2) hipLaunchKernelGGL((dequant_kernel<ODT_, 2>), grid, dim3(256), 0, st, p); \
    else hipLaunchKernelGGL((dequant_kernel<ODT_, 1>), grid, dim3(256), 0, st, p);           \
  } while (0)
  if (out_dtype == VARQ_F32) VARQ_DEQ(VARQ_F32);
  else if (out_dtype == VARQ_BF16) VARQ_DEQ(VARQ_BF16);
  else VARQ_DEQ(VARQ_F16);
#undef VARQ_DEQ
  VARQ_CHECK_LAUNCH("dequant");
  return VARQ_OK;
}

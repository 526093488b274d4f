// Producer side of the quantized KV cache in one pass.
//
// The Infinity attention block normalises q and k, rotates them, and only then
// hands k and v to the quantizer (Infinity/infinity/models/basic.py:316-330:
// F.normalize, .mul(scale_mul), apply_rotary_emb at :103-123, use_var_q); the
// VAR block does the same without the rotation
// (VAR/models/basic_var.py:137-147).  That is three elementwise passes over
// q and k in fp32 plus the quantizer's own.  This kernel reads the output of the
// qkv projection once, [B, L, 3, H, c], and writes
//   * q: l2-normalised, scaled per head, rotated, as bf16 [B, H, L, c];
//   * k (normalised, rotated) and v: group-wise quantized and packed straight into
//     their rows of the pre-allocated cache (same row map as varq_quant_pack_rows).
//
// Arithmetic, all fp32, every step rounded on its own (no fused multiply-add), in the
// order of the reference's tensor expressions:
//   ss   = sum of squares: 8 channels of an octet left to right, then octets pairwise
//          (o0+o1)+(o2+o3)...        [the reference leaves the order to the backend]
//   y    = x / max(sqrt(ss), norm_eps)                       (F.normalize)
//   y    = y * scale_mul[h]                                   (q only)
//   even = cos*y0 - sin*y1 ; odd = sin*y0 + cos*y1            (channel pairs 2i, 2i+1)
// followed by the group-wise quantizer of quant_rows.hip.
#include "varq_common.h"

namespace {

struct PrepParams {
  const void *qkv;
  const float *scale_mul;      // [H] or null
  const float *cos, *sin;      // [>= token_start + L, c/2] or null
  void *q_out;                 // bf16 [B, H, L, c]
  int32_t *k_words, *v_words;
  float *k_scale, *k_zp, *v_scale, *v_zp;
  const int32_t *slot;
  RowMap map;                  // (b, l, h) -> cache row
  int B, L, H, c, c8, c8_shift;
  int token_start, l2norm, nseg;
  float norm_eps, eps;
  int64_t rows;                // B*L*H
};

template <int LANES> __device__ __forceinline__ float group_allsum(float v) {
  // after each step the partners hold the same value, so the mirrored steps pair equal halves
  if (LANES >= 2) v = v + dpp_f<0xB1>(v);
  if (LANES >= 4) v = v + dpp_f<0x4E>(v);
  if (LANES >= 8) v = v + dpp_f<0x141>(v);
  if (LANES >= 16) v = v + dpp_f<0x140>(v);
  if (LANES >= 32) v = v + __shfl_xor(v, 16, 64);
  return v;
}

// x / d as IEEE division rounds it, for a divisor that passed plain_divisor (see
// quant_rows.hip for the argument); r = RN(1/d)
__device__ __forceinline__ float exact_div(float x, float d, float r) {
  const float q0 = x * r;
  return __builtin_fmaf(__builtin_fmaf(-q0, d, x), r, q0);
}
__device__ __forceinline__ bool plain_divisor(float d) {
  return d > 0x1p-96f && d < 0x1p96f && (f2u(d) & 0x7fffffu) != 0x7fffffu;
}

// group-wise quantize + pack of one octet held by each of LG adjacent lanes
template <int BITS, bool ASYM, int LG>
__device__ __forceinline__ void quant_octet(const float (&v)[8], float eps, float &s_out, float &zp_out, u32 &w0, u32 &w1) {
  constexpr float kMin = (float)QRange<BITS>::kMin, kMax = (float)QRange<BITS>::kMax;
  float mx, mn = 0.f;
  if (ASYM) {
    mx = v[0]; mn = v[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) { mx = fmaxf(mx, v[j]); mn = fminf(mn, v[j]); }
    mx = group_allreduce<LG, true>(mx);
    mn = group_allreduce<LG, false>(mn);
  } else {
    mx = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) mx = fmaxf(mx, fabsf(v[j]));
    mx = group_allreduce<LG, true>(mx);
  }
  const float s = ASYM ? fmaxf((mx - mn) / (float)QRange<BITS>::kLevels, eps) : fmaxf(mx / kMax, eps);
  const float r = 1.0f / s;
  const bool plain = plain_divisor(s);
  // the shortcut or the division for the whole wavefront: no per-element branches
  const bool wave_plain = __builtin_amdgcn_ballot_w64(!plain) == 0;
  const float zp = ASYM ? kMin - rintf(wave_plain ? exact_div(mn, s, r) : mn / s) : 0.f;
  float t[8];
  if (wave_plain) {
#pragma unroll
    for (int j = 0; j < 8; ++j) t[j] = exact_div(v[j], s, r);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) t[j] = v[j] / s;
  }
  u32 acc = 0;
  w0 = 0; w1 = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float n = rintf(t[j]);
    const int q = (int)__builtin_amdgcn_fmed3f(ASYM ? n + zp : n, kMin, kMax);
    acc = __builtin_amdgcn_alignbit((u32)q, acc, BITS);
    if (BITS == 8 && j == 3) { w0 = acc; acc = 0; }
  }
  if (BITS == 8) w1 = acc;
  else if (BITS == 4) w0 = acc;
  else w0 = acc >> 16;
  s_out = s; zp_out = zp;
}

// One lane = 8 channels of one (b, l, h); LR = c/8 lanes form the row, LG = group/8 a group.
template <int DT, int BITS, bool ASYM, int LR, int LG>
__global__ __launch_bounds__(256) void qkv_prepare_kernel(PrepParams p) {
  // Lanes walk the (b, h, l) order of the outputs, so the prepared q, the packed words and
  // the scales of a wavefront are contiguous; the reads are whole 16*LR-byte rows either way.
  const u32 o = blockIdx.x * 256u + threadIdx.x;      // < 2^31 (checked on the host)
  const u32 r = o / LR;
  const int col = (int)(o - r * LR);
  const bool live = r < (u32)p.rows;
  const u32 rc = live ? r : (u32)p.rows - 1u;         // idle lanes recompute the last row, never store
  const int l = (int)(rc % (u32)p.L);
  const u32 bh = rc / (u32)p.L;
  const int h = (int)(bh % (u32)p.H);
  const int b = (int)(bh / (u32)p.H);
  const int c = p.c;
  const int64_t bl = (int64_t)b * p.L + l;
  const int64_t base = (bl * 3) * (int64_t)p.H * c + (int64_t)h * c + col * 8;
  const int64_t tstride = (int64_t)p.H * c;

  float q[8], k[8], v[8];
  In8<DT>::load(p.qkv, base, q);
  In8<DT>::load(p.qkv, base + tstride, k);
  In8<DT>::load(p.qkv, base + 2 * tstride, v);

  if (p.l2norm) {
    float sq = q[0] * q[0], sk = k[0] * k[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) { sq = sq + q[j] * q[j]; sk = sk + k[j] * k[j]; }
    sq = group_allsum<LR>(sq);
    sk = group_allsum<LR>(sk);
    const float dq = fmaxf(__builtin_sqrtf(sq), p.norm_eps), dk = fmaxf(__builtin_sqrtf(sk), p.norm_eps);
    const float rq = 1.0f / dq, rk = 1.0f / dk;
    const bool pq = plain_divisor(dq), pk = plain_divisor(dk);
    const float mul = p.scale_mul ? p.scale_mul[h] : 1.f;
    if (__builtin_amdgcn_ballot_w64(!(pq && pk)) == 0) {
#pragma unroll
      for (int j = 0; j < 8; ++j) { q[j] = exact_div(q[j], dq, rq); k[j] = exact_div(k[j], dk, rk); }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) { q[j] = q[j] / dq; k[j] = k[j] / dk; }
    }
    if (p.scale_mul) {
#pragma unroll
      for (int j = 0; j < 8; ++j) q[j] = q[j] * mul;
    }
  }
  if (p.cos) {
    const int64_t t = (int64_t)(p.token_start + l) * (c / 2) + col * 4;
    const float4 cs = *reinterpret_cast<const float4 *>(p.cos + t);
    const float4 sn = *reinterpret_cast<const float4 *>(p.sin + t);
    const float cc[4] = {cs.x, cs.y, cs.z, cs.w}, ss[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float q0 = q[2 * i], q1 = q[2 * i + 1], k0 = k[2 * i], k1 = k[2 * i + 1];
      q[2 * i] = cc[i] * q0 - ss[i] * q1;
      q[2 * i + 1] = ss[i] * q0 + cc[i] * q1;
      k[2 * i] = cc[i] * k0 - ss[i] * k1;
      k[2 * i + 1] = ss[i] * k0 + cc[i] * k1;
    }
  }

  float ks, kz, vs, vz;
  u32 kw0, kw1, vw0, vw1;
  quant_octet<BITS, ASYM, LG>(k, p.eps, ks, kz, kw0, kw1);
  quant_octet<BITS, ASYM, LG>(v, p.eps, vs, vz, vw0, vw1);

  // cache row of (b, l, h)
  int64_t s0 = b, s1 = l, s2 = h;
  if (p.map.slot_dim == 0) s0 = p.slot[b];
  if (p.map.slot_dim == 1) s1 = p.slot[l];
  if (p.map.slot_dim == 2) s2 = p.slot[h];
  const bool stored = live && s0 >= 0 && s1 >= 0 && s2 >= 0;
  const int64_t row = s0 * p.map.os0 + s1 * p.map.os1 + s2 * p.map.os2 + p.map.off;

  // the 2-bit word is assembled from two lanes: every lane reaches the exchange
  if (BITS == 2) {
    const u32 ko = (u32)__builtin_amdgcn_update_dpp(0, (int)kw0, 0xB1, 0xf, 0xf, false);
    const u32 vo = (u32)__builtin_amdgcn_update_dpp(0, (int)vw0, 0xB1, 0xf, 0xf, false);
    kw0 |= ko << 16; vw0 |= vo << 16;
  }
  if (live) {
    __bf16 *qo = reinterpret_cast<__bf16 *>(p.q_out) + (((int64_t)b * p.H + h) * p.L + l) * c + col * 8;
    uint16_t hq[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) hq[j] = f32_to_bf16_rne(q[j]);
    *reinterpret_cast<uint4 *>(qo) = make_uint4(hq[0] | ((u32)hq[1] << 16), hq[2] | ((u32)hq[3] << 16),
                                                hq[4] | ((u32)hq[5] << 16), hq[6] | ((u32)hq[7] << 16));
  }
  if (!stored) return;
  if (BITS == 8) {
    *reinterpret_cast<uint2 *>(p.k_words + (row * p.c8 + col) * 2) = make_uint2(kw0, kw1);
    *reinterpret_cast<uint2 *>(p.v_words + (row * p.c8 + col) * 2) = make_uint2(vw0, vw1);
  } else if (BITS == 4) {
    p.k_words[row * p.c8 + col] = (int32_t)kw0;
    p.v_words[row * p.c8 + col] = (int32_t)vw0;
  } else if ((col & 1) == 0) {
    p.k_words[(row * p.c8 + col) >> 1] = (int32_t)kw0;
    p.v_words[(row * p.c8 + col) >> 1] = (int32_t)vw0;
  }
  if ((col & (LG - 1)) == 0) {
    const int64_t g = row * p.nseg + col / LG;
    p.k_scale[g] = ks; p.v_scale[g] = vs;
    if (ASYM) { p.k_zp[g] = kz; p.v_zp[g] = vz; }
  }
}

template <int DT, int BITS, bool ASYM, int LR>
int launch_lg(const PrepParams &p, int lg, dim3 grid, hipStream_t st) {
  switch (lg) {
#define VARQ_LG(G)                                                                                  \
  case G:                                                                                           \
    if constexpr (G <= LR) {                                                                        \
      hipLaunchKernelGGL((qkv_prepare_kernel<DT, BITS, ASYM, LR, G>), grid, dim3(256), 0, st, p);   \
      return 0;                                                                                     \
    }                                                                                               \
    return -1;
    VARQ_LG(1) VARQ_LG(2) VARQ_LG(4) VARQ_LG(8) VARQ_LG(16)
#undef VARQ_LG
  }
  return -1;
}

template <int DT, int BITS, bool ASYM>
int launch_lr(const PrepParams &p, int lr, int lg, dim3 grid, hipStream_t st) {
  if (lr == 4) return launch_lg<DT, BITS, ASYM, 4>(p, lg, grid, st);
  if (lr == 8) return launch_lg<DT, BITS, ASYM, 8>(p, lg, grid, st);
  if (lr == 16) return launch_lg<DT, BITS, ASYM, 16>(p, lg, grid, st);
  return -1;
}

template <int DT>
int launch_dt(const PrepParams &p, int bits, int asym, int lr, int lg, dim3 grid, hipStream_t st) {
  if (bits == 8) return asym ? launch_lr<DT, 8, true>(p, lr, lg, grid, st) : launch_lr<DT, 8, false>(p, lr, lg, grid, st);
  if (bits == 4) return asym ? launch_lr<DT, 4, true>(p, lr, lg, grid, st) : launch_lr<DT, 4, false>(p, lr, lg, grid, st);
  return asym ? launch_lr<DT, 2, true>(p, lr, lg, grid, st) : launch_lr<DT, 2, false>(p, lr, lg, grid, st);
}

}  // namespace

extern "C" int varq_qkv_prepare_append(const void *qkv, int x_dtype, int B, int L, int H, int c,
                                       const float *q_scale_mul, int l2norm, float norm_eps,
                                       const float *rope_cos, const float *rope_sin, int token_start,
                                       void *q_out, int group, int bits, int asym, float eps,
                                       const int64_t *host_rowmap, const int32_t *slot,
                                       int32_t *k_words, float *k_scale, float *k_zp,
                                       int32_t *v_words, float *v_scale, float *v_zp, void *stream) {
  VARQ_CHECK_ARG(B >= 0 && L >= 0 && H > 0, "qkv_prepare: bad sizes");
  VARQ_CHECK_ARG(c == 32 || c == 64 || c == 128, "qkv_prepare: head dim must be 32, 64 or 128 (got %d)", c);
  VARQ_CHECK_ARG(x_dtype >= 0 && x_dtype <= 2, "qkv_prepare: bad dtype %d", x_dtype);
  VARQ_CHECK_ARG(bits == 2 || bits == 4 || bits == 8, "qkv_prepare: bits must be 2, 4 or 8 (got %d)", bits);
  VARQ_CHECK_ARG(group >= 8 && group <= c && c % group == 0 && (group & (group - 1)) == 0,
                 "qkv_prepare: group must be a power of two in [8, c] (got %d)", group);
  VARQ_CHECK_ARG(bits != 2 || group >= 16, "qkv_prepare: 2-bit codes need groups of at least 16 channels");
  VARQ_CHECK_ARG((rope_cos == nullptr) == (rope_sin == nullptr), "qkv_prepare: give both rotary tables or neither");
  VARQ_CHECK_ARG(token_start >= 0, "qkv_prepare: bad token_start");
  const int64_t rows = (int64_t)B * L * H;
  if (rows == 0) return VARQ_OK;
  VARQ_CHECK_ARG(qkv && q_out && k_words && v_words && k_scale && v_scale && (!asym || (k_zp && v_zp)) && host_rowmap,
                 "qkv_prepare: null pointer");
  VARQ_CHECK_ARG(((uintptr_t)qkv & 15) == 0 && ((uintptr_t)q_out & 15) == 0, "qkv_prepare: qkv and q_out must be 16-byte aligned");
  VARQ_CHECK_ARG(rows * (c / 8) < (1ll << 31) - 256, "qkv_prepare: tensor too large");

  PrepParams p;
  p.qkv = qkv; p.scale_mul = q_scale_mul; p.cos = rope_cos; p.sin = rope_sin; p.q_out = q_out;
  p.k_words = k_words; p.v_words = v_words; p.k_scale = k_scale; p.k_zp = k_zp; p.v_scale = v_scale; p.v_zp = v_zp;
  p.slot = slot;
  p.map = varq_rowmap_from_host(host_rowmap, rows);
  VARQ_CHECK_ARG(p.map.n0 == B && p.map.n1 == L && p.map.n2 == H, "qkv_prepare: row map dims must be (B, L, H)");
  VARQ_CHECK_ARG(p.map.slot_dim < 0 || slot, "qkv_prepare: slot table missing");
  p.B = B; p.L = L; p.H = H; p.c = c; p.c8 = c / 8; p.c8_shift = 0;
  p.token_start = token_start; p.l2norm = l2norm ? 1 : 0; p.nseg = c / group;
  p.norm_eps = norm_eps; p.eps = eps; p.rows = rows;
  const int64_t blocks = (rows * p.c8 + 255) / 256;
  VARQ_CHECK_ARG(blocks < (1ll << 31), "qkv_prepare: too many blocks");
  dim3 grid((unsigned)blocks);
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (x_dtype == VARQ_F32) rc = launch_dt<VARQ_F32>(p, bits, asym, p.c8, group / 8, grid, st);
  else if (x_dtype == VARQ_BF16) rc = launch_dt<VARQ_BF16>(p, bits, asym, p.c8, group / 8, grid, st);
  else rc = launch_dt<VARQ_F16>(p, bits, asym, p.c8, group / 8, grid, st);
  if (rc) return varq_set_error(VARQ_ERR_UNSUPPORTED, "qkv_prepare: no kernel for c=%d group=%d", c, group);
  VARQ_CHECK_LAUNCH("qkv_prepare");
  return VARQ_OK;
}

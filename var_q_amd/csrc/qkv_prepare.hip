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
  bool slow_levels;            // eps so small that (max - min) / levels must be a true division
  int64_t rows;                // B*L*H
};

template <int LANES> __device__ __forceinline__ float group_allsum(float v) {
  // after each step the partners hold the same value, so the mirrored steps pair equal halves
  v = row_fold_add<(LANES < 16 ? LANES : 16)>(v);
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

// (max - min) / levels as IEEE division rounds it.  The divisor is a constant whose significand
// is not all ones, so the quotient shortcut applies whenever its residual cannot underflow:
// range >= 2^-90.  Below that the true quotient is below 2^-91 and any eps >= 2^-80 replaces it;
// smaller eps values take the division (`slow`, uniform for the launch).
template <int BITS> __device__ __forceinline__ float range_over_levels(float range, bool slow) {
  constexpr float kLv = (float)QRange<BITS>::kLevels;
  // (a range that overflowed to infinity takes the division too; the branch is wave-uniform)
  if (slow || __builtin_amdgcn_ballot_w64(!(range < 0x1p126f)) != 0) return range / kLv;
  return exact_div(range, kLv, 1.0f / kLv);
}

// Scale, reciprocal and the shortcut flag of one group from its max and min.
template <int BITS, bool ASYM>
__device__ __forceinline__ void group_scale(float mx, float mn, float eps, bool slow, float &s, float &r, bool &plain) {
  constexpr float kMax = (float)QRange<BITS>::kMax;
  s = ASYM ? fmaxf(range_over_levels<BITS>(mx - mn, slow), eps) : fmaxf(mx / kMax, eps);
  r = 1.0f / s;
  plain = plain_divisor(s);
}
// ... and its zero-point (wave_plain: every lane of the wavefront may take the shortcut)
template <int BITS, bool ASYM>
__device__ __forceinline__ float group_zp(float mn, float s, float r, bool wave_plain) {
  if (!ASYM) return 0.f;
  return (float)QRange<BITS>::kMin - rintf(wave_plain ? exact_div(mn, s, r) : mn / s);
}

// codes of one octet from the group's parameters, packed.
// fast (wave-uniform: every lane may take the quotient shortcut and no zero-point exceeds 2^22):
// clamp(rint(t) + zp, qmin, qmax) = rint(clamp(t, qmin - zp, qmax - zp)) + zp since the bounds
// are integers; adding 1.5 * 2^23 rounds the clamped quotient to nearest-even and leaves the
// integer in the low mantissa bits, and the zero-point is added to all fields of the finished
// word at once, modulo the field width (the sum is known to fit the field).
template <int BITS, bool ASYM>
__device__ __forceinline__ void pack_octet(const float (&v)[8], float s, float r, float zp, bool fast, u32 &w0, u32 &w1) {
  constexpr float kMin = (float)QRange<BITS>::kMin, kMax = (float)QRange<BITS>::kMax;
  u32 acc = 0;
  w0 = 0; w1 = 0;
  if (fast) {
    const float lo = kMin - zp, hi = kMax - zp;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const u32 q = f2u(__builtin_amdgcn_fmed3f(exact_div(v[j], s, r), lo, hi) + 12582912.f);
      acc = __builtin_amdgcn_alignbit(q, acc, BITS);
      if (BITS == 8 && j == 3) { w0 = acc; acc = 0; }
    }
    if (BITS == 8) w1 = acc;
    else if (BITS == 4) w0 = acc;
    else w0 = acc >> 16;
    if (ASYM) {
      constexpr u32 kFieldHi = BITS == 8 ? 0x80808080u : BITS == 4 ? 0x88888888u : 0xaaaaaaaau;
      constexpr u32 kFieldLsb = BITS == 8 ? 0x01010101u : BITS == 4 ? 0x11111111u : 0x55555555u;
      const u32 zrep = ((u32)(int)zp & ((1u << BITS) - 1u)) * kFieldLsb;
      const u32 zlo = zrep & ~kFieldHi, zhi = zrep & kFieldHi;
      w0 = ((w0 & ~kFieldHi) + zlo) ^ (w0 & kFieldHi) ^ zhi;
      if (BITS == 8) w1 = ((w1 & ~kFieldHi) + zlo) ^ (w1 & kFieldHi) ^ zhi;
      if (BITS == 2) w0 &= 0xffffu;
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float n = rintf(v[j] / s);
    const int q = (int)__builtin_amdgcn_fmed3f(ASYM ? n + zp : n, kMin, kMax);
    acc = __builtin_amdgcn_alignbit((u32)q, acc, BITS);
    if (BITS == 8 && j == 3) { w0 = acc; acc = 0; }
  }
  if (BITS == 8) w1 = acc;
  else if (BITS == 4) w0 = acc;
  else w0 = acc >> 16;
}

template <bool ASYM, int LG>
__device__ __forceinline__ void octet_minmax(const float (&v)[8], float &mx, float &mn) {
  mn = 0.f;
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
}

// the other lane of an aligned lane pair
__device__ __forceinline__ float pair_swap(float v) { return dpp_f<0xB1>(v); }

// One lane = 8 channels of one (b, l, h); LR = c/8 lanes form the row, LG = group/8 a group.
template <int DT, int BITS, bool ASYM, int LR, int LG>
__global__ __launch_bounds__(256) void qkv_prepare_kernel(PrepParams p) {
  // One workgroup = one tile of 256/LR tokens of one (b, h): lanes walk the (b, h, l) order of the
  // outputs, so the prepared q, the packed words and the scales of a wavefront are contiguous; the
  // reads are whole 16*LR-byte rows either way.  (b, h) is uniform for the workgroup: no vector
  // divisions.  Order of the workgroups (1-D grid; consecutive ids go to consecutive XCDs):
  // id = ((tile / 8) * B*H + bh) * 8 + tile % 8.  The workgroups in flight together then read all
  // heads of the same few tokens, whole 6*H*c-byte stretches of the input between them, instead
  // of one 2*c-byte piece out of every token row (8 % of the kernel's time at H=16, c=128), and
  // the B*H workgroups of one tile run on one XCD, whose L2 fetches that tile's rotary factors once.
  const u32 id = blockIdx.x, j = id >> 3;
  const u32 BH = (u32)(p.B * p.H);
  const u32 tile8 = j / BH;                           // (uniform: scalar arithmetic)
  const int bh = (int)(j - tile8 * BH);
  const int h = bh % p.H, b = bh / p.H;
  // a slot table over the heads (one launch per bit-width class of a mixed cache): the heads of
  // the other classes are theirs altogether, q included, so that the launches share out the work
  int head_slot = h;
  if (p.map.slot_dim == 2) {
    head_slot = p.slot[h];
    if (head_slot < 0) return;                        // (uniform for the workgroup)
  }
  const int o = (int)(tile8 * 8u + (id & 7u)) * 256 + threadIdx.x;
  const int lt = o / LR;                              // (LR is a power of two)
  const int col = o - lt * LR;
  const bool live = lt < p.L;
  const int l = live ? lt : p.L - 1;                  // idle lanes recompute the last token, never store
  const int c = p.c;
  // element offsets: the (b, h) part is uniform for the workgroup, the lane's part fits 32 bits
  // (L * 3 * H * c < 2^31, checked on the host)
  const int64_t base_bh = ((int64_t)b * p.L * 3) * (int64_t)p.H * c + (int64_t)h * c;
  const int tstride = p.H * c;
  const int lane_off = l * 3 * tstride + col * 8;
  const bool odd = col & 1;

  float q[8], k[8], v[8];
  // the rotation's factors are requested with the row, long before the rotation needs them;
  // without a table the requests read the first 16 bytes of the input and nothing uses them
  const float *cos_base = p.cos ? p.cos : reinterpret_cast<const float *>(p.qkv);
  const float *sin_base = p.cos ? p.sin : reinterpret_cast<const float *>(p.qkv);
  const int t = p.cos ? (p.token_start + l) * (c / 2) + col * 4 : 0;   // (fits 32 bits: checked on the host)
  const float4 cs = *reinterpret_cast<const float4 *>(cos_base + t);
  const float4 sn = *reinterpret_cast<const float4 *>(sin_base + t);
  In8<DT>::load(p.qkv, base_bh + lane_off, q);
  In8<DT>::load(p.qkv, base_bh + lane_off + tstride, k);
  In8<DT>::load(p.qkv, base_bh + lane_off + 2 * tstride, v);

  if (p.l2norm) {
    float sq = q[0] * q[0], sk = k[0] * k[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) { sq = sq + q[j] * q[j]; sk = sk + k[j] * k[j]; }
    sq = group_allsum<LR>(sq);
    sk = group_allsum<LR>(sk);
    // the two norms of a row are two jobs of one instruction stream: even lanes take q's, odd
    // lanes k's (square root, clamp, reciprocal, shortcut test), then the lanes of a pair swap
    const float ssum = odd ? sk : sq;
    const float dmine = fmaxf(__builtin_sqrtf(ssum), p.norm_eps);
    const float rmine = 1.0f / dmine;
    const bool pmine = plain_divisor(dmine);
    const float dother = pair_swap(dmine), rother = pair_swap(rmine);
    const float dq = odd ? dother : dmine, dk = odd ? dmine : dother;
    const float rq = odd ? rother : rmine, rk = odd ? rmine : rother;
    const float mul = p.scale_mul ? p.scale_mul[h] : 1.f;
    if (__builtin_amdgcn_ballot_w64(!pmine) == 0) {
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

  // group-wise quantizer of k and v
  float kmx, kmn, vmx, vmn;
  octet_minmax<ASYM, LG>(k, kmx, kmn);
  octet_minmax<ASYM, LG>(v, vmx, vmn);
  float ks, kr, kz, vs, vr, vz;
  bool wave_plain;   // the shortcut or the division for the whole wavefront: no per-element branches
  if constexpr (LG >= 2) {
    // a lane pair lies inside one group: the even lane derives k's parameters, the odd lane v's,
    // in one instruction stream, and the pair swaps
    float s, r;
    bool pl;
    const float mn = odd ? vmn : kmn;
    group_scale<BITS, ASYM>(odd ? vmx : kmx, mn, p.eps, p.slow_levels, s, r, pl);
    wave_plain = __builtin_amdgcn_ballot_w64(!pl) == 0;
    const float z = group_zp<BITS, ASYM>(mn, s, r, wave_plain);
    const float so = pair_swap(s), ro = pair_swap(r), zo = pair_swap(z);
    ks = odd ? so : s; kr = odd ? ro : r; kz = odd ? zo : z;
    vs = odd ? s : so; vr = odd ? r : ro; vz = odd ? z : zo;
  } else {
    bool kplain, vplain;
    group_scale<BITS, ASYM>(kmx, kmn, p.eps, p.slow_levels, ks, kr, kplain);
    group_scale<BITS, ASYM>(vmx, vmn, p.eps, p.slow_levels, vs, vr, vplain);
    wave_plain = __builtin_amdgcn_ballot_w64(!(kplain && vplain)) == 0;
    kz = group_zp<BITS, ASYM>(kmn, ks, kr, wave_plain);
    vz = group_zp<BITS, ASYM>(vmn, vs, vr, wave_plain);
  }
  u32 kw0, kw1, vw0, vw1;
  const bool fast = wave_plain && __builtin_amdgcn_ballot_w64(!(fabsf(kz) <= 0x1p21f && fabsf(vz) <= 0x1p21f)) == 0;
  pack_octet<BITS, ASYM>(k, ks, kr, kz, fast, kw0, kw1);
  pack_octet<BITS, ASYM>(v, vs, vr, vz, fast, vw0, vw1);

  // cache row of (b, l, h)
  int64_t s0 = b, s1 = l, s2 = head_slot;
  if (p.map.slot_dim == 0) s0 = p.slot[b];
  if (p.map.slot_dim == 1) s1 = p.slot[l];
  const bool stored = live && s0 >= 0 && s1 >= 0 && s2 >= 0;
  const int64_t row = s0 * p.map.os0 + s1 * p.map.os1 + s2 * p.map.os2 + p.map.off;

  // the 2-bit word is assembled from two lanes: every lane reaches the exchange
  if (BITS == 2) {
    const u32 ko = (u32)__builtin_amdgcn_update_dpp(0, (int)kw0, 0xB1, 0xf, 0xf, false);
    const u32 vo = (u32)__builtin_amdgcn_update_dpp(0, (int)vw0, 0xB1, 0xf, 0xf, false);
    kw0 |= ko << 16; vw0 |= vo << 16;
  }
  if (live) {
    __bf16 *qo = reinterpret_cast<__bf16 *>(p.q_out) + (int64_t)bh * p.L * c + (l * c + col * 8);
    // hardware round-to-nearest-even conversion, two values per instruction
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    u32 w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const f2 t = {q[2 * j], q[2 * j + 1]};
      w[j] = __builtin_bit_cast(u32, __builtin_convertvector(t, bf2));
    }
    *reinterpret_cast<uint4 *>(qo) = make_uint4(w[0], w[1], w[2], w[3]);
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
  VARQ_CHECK_ARG(rows * (c / 8) < (1ll << 31) - 256 && (int64_t)L * 3 * H * c < (1ll << 31) &&
                     ((int64_t)token_start + L) * (c / 2) < (1ll << 31), "qkv_prepare: tensor too large");

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
  p.slow_levels = !(eps >= 0x1p-80f);
  const int64_t tiles = ((int64_t)L * p.c8 + 255) / 256;
  // (tiles are dealt out in eights; those past the last token find no live lane and store nothing)
  const int64_t wgs = (tiles + 7) / 8 * 8 * ((int64_t)B * H);
  VARQ_CHECK_ARG(wgs < (1ll << 31), "qkv_prepare: tensor too large");
  dim3 grid((unsigned)wgs);
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (x_dtype == VARQ_F32) rc = launch_dt<VARQ_F32>(p, bits, asym, p.c8, group / 8, grid, st);
  else if (x_dtype == VARQ_BF16) rc = launch_dt<VARQ_BF16>(p, bits, asym, p.c8, group / 8, grid, st);
  else rc = launch_dt<VARQ_F16>(p, bits, asym, p.c8, group / 8, grid, st);
  if (rc) return varq_set_error(VARQ_ERR_UNSUPPORTED, "qkv_prepare: no kernel for c=%d group=%d", c, group);
  VARQ_CHECK_LAUNCH("qkv_prepare");
  return VARQ_OK;
}

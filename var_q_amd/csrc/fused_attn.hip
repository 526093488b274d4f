// Fused dequant flash-attention for gfx950.
//
//   out = softmax(scale * Q K^T + mask) V,   K = (kq - kzp) * ks,  V = (vq - vzp) * vs
//
// with K/V held as packed INT2/4/8 codes plus per-token group scales.  Replaces
// "unpack whole cache -> fp32 dequant -> external attention" of
// VAR_Q/quant.py:216-230 + VAR/models/basic_var.py:156-162 /
// Infinity/infinity/models/basic.py:339-351; the mask is the block-causal
// next-scale rule of VAR/models/var.py:110-114 expressed as a per-query key
// limit.
//
// Design (one workgroup = 4 wavefronts = 128 queries of one (batch, head)):
//  * Both contractions run on v_mfma_f32_32x32x16_bf16 in transposed form,
//    S^T = K Q^T and O^T = V^T P^T, so that a lane owns one query column: row
//    max/sum are per-lane (one cross-half exchange per tile) and the S^T
//    accumulator registers are directly the B operand of the second MFMA.
//  * Codes are never scaled before the MFMA.  They are widened to small exact
//    bf16 integers; the affine map is applied in fp32 to the 32x32 results:
//       S[l,q] = sum_seg  ks[l,seg] * (A_seg[l,q] - kzp'[l,seg] * qsum_seg[q])
//       O[q,:] = sum_l (p[l,q] * vs[l,seg]) * vraw[l,:]  -  sum_l p' * vzp'
//    which is cheaper than dequantizing every element and loses nothing to
//    bf16 rounding of K/V.
//  * K tile: packed words HBM -> LDS, expanded in registers by each wavefront
//    straight into MFMA A operands (8 codes of one word = one lane's operand).
//  * V tile: packed words HBM -> LDS -> expanded once per workgroup and written
//    transposed (V^T, bf16) to LDS, because the PV contraction runs over keys.
//  * Key rows are fed to the first MFMA in a permuted order chosen so that each
//    lane's accumulator registers hold 8 consecutive keys per 16-key chunk,
//    which makes the V^T operand a single 16-byte LDS read.
#include "varq_common.h"

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;
typedef __attribute__((__vector_size__(4 * sizeof(u32)))) u32 u32x4_t;

constexpr int BM = 128;  // queries per workgroup (32 per wavefront)
constexpr int BN = 64;   // keys per tile
constexpr float kLog2e = 1.4426950408889634f;

struct AttnParams {
  const __bf16 *q;
  __bf16 *out;
  const u32 *k_words, *v_words;
  const float *k_scale, *k_zp, *v_scale, *v_zp;
  const int32_t *head_map;
  const int32_t *kv_limit;
  int B, Hq, Hkv, Lq, Lk, Lstride;
  int q_tiles, bh_total;
  float scale_log2e;
};

// ---- code widening ---------------------------------------------------------
// K side: 8 codes of one octet -> 8 bf16 (4 dwords) holding code*kMul'+const,
// i.e. code = kMul * raw - kOff.  `slot_d(j)` is the channel (within the octet)
// that lands in operand slot j; the Q operand is gathered in the same order.
template <int BITS> struct KCodec;

template <> struct KCodec<4> {
  // nibble u = code+8 goes to the top 4 mantissa bits of bf16 1.0:
  // raw = 1 + u/16 = (code + 24)/16.
  static constexpr float kMul = 16.f, kOff = 24.f;
  __device__ static __forceinline__ int slot_d(int j) { return (j >> 1) + 4 * (j & 1); }
  __device__ static __forceinline__ void expand(const u32 *lds_row, int oct, u32 (&o)[4]) {
    const u32 w = lds_row[oct] ^ 0x88888888u;
    constexpr u32 M = 0x00780078u, B = 0x3f803f80u;
    o[0] = ((w << 3) & M) | B;   // nibbles 0,4
    o[1] = ((w >> 1) & M) | B;   // 1,5
    o[2] = ((w >> 5) & M) | B;   // 2,6
    o[3] = ((w >> 9) & M) | B;   // 3,7
  }
};

template <> struct KCodec<2> {
  // field u = code+2 goes to the top 2 mantissa bits: raw = 1 + u/4 = (code + 6)/4.
  static constexpr float kMul = 4.f, kOff = 6.f;
  // an octet is half a word: fields 0..7 of the half; dword m holds fields (m, m+4)
  __device__ static __forceinline__ int slot_d(int j) { return (j >> 1) + 4 * (j & 1); }
  __device__ static __forceinline__ void expand(const u32 *lds_row, int oct, u32 (&o)[4]) {
    const u32 w = ((lds_row[oct >> 1] >> ((oct & 1) * 16)) & 0xffffu) ^ 0xaaaau;
    // fields m (bits 2m) and m+4 (bits 2m+8): move to bits 5..6 and 21..22
    const u32 t = (w & 0xffu) | ((w & 0xff00u) << 8);  // low byte: fields 0-3, byte 2: fields 4-7
    constexpr u32 M = 0x00600060u, B = 0x3f803f80u;
    o[0] = ((t << 5) & M) | B;
    o[1] = ((t << 3) & M) | B;
    o[2] = ((t << 1) & M) | B;
    o[3] = ((t >> 1) & M) | B;
  }
};

template <> struct KCodec<8> {
  // bytes are widened through fp32 (exact), raw = code.
  static constexpr float kMul = 1.f, kOff = 0.f;
  __device__ static __forceinline__ int slot_d(int j) { return j; }
  __device__ static __forceinline__ void expand(const u32 *lds_row, int oct, u32 (&o)[4]) {
    const u32 w0 = lds_row[2 * oct], w1 = lds_row[2 * oct + 1];
    float f[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[j] = (float)(int)__builtin_amdgcn_sbfe((int)w0, 8 * j, 8);
      f[4 + j] = (float)(int)__builtin_amdgcn_sbfe((int)w1, 8 * j, 8);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = (f2u(f[2 * j]) >> 16) | (f2u(f[2 * j + 1]) & 0xffff0000u);
  }
};

// V side: the 8 codes of octet `oct` of one key as exact floats code + kOff.
template <int BITS> struct VCodec;
template <> struct VCodec<4> {
  static constexpr float kOff = 8.f;
  __device__ static __forceinline__ void codes(const u32 *lds_row, int oct, float (&f)[8]) {
    const u32 w = lds_row[oct] ^ 0x88888888u;
    const u32 e = w & 0x0f0f0f0fu, o = (w >> 4) & 0x0f0f0f0fu;
    f[0] = (float)(e & 0xffu); f[1] = (float)(o & 0xffu);
    f[2] = (float)((e >> 8) & 0xffu); f[3] = (float)((o >> 8) & 0xffu);
    f[4] = (float)((e >> 16) & 0xffu); f[5] = (float)((o >> 16) & 0xffu);
    f[6] = (float)(e >> 24); f[7] = (float)(o >> 24);
  }
};
template <> struct VCodec<2> {
  static constexpr float kOff = 0.f;
  __device__ static __forceinline__ void codes(const u32 *lds_row, int oct, float (&f)[8]) {
    const int w = (int)(lds_row[oct >> 1] >> ((oct & 1) * 16));
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = (float)(int)__builtin_amdgcn_sbfe(w, 2 * j, 2);
  }
};
template <> struct VCodec<8> {
  static constexpr float kOff = 0.f;
  __device__ static __forceinline__ void codes(const u32 *lds_row, int oct, float (&f)[8]) {
    const int w0 = (int)lds_row[2 * oct], w1 = (int)lds_row[2 * oct + 1];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[j] = (float)(int)__builtin_amdgcn_sbfe(w0, 8 * j, 8);
      f[4 + j] = (float)(int)__builtin_amdgcn_sbfe(w1, 8 * j, 8);
    }
  }
};

__device__ __forceinline__ u32 pack_bf16_hi(float lo, float hi) {  // exact for values with <= 8 significant bits
  return (f2u(lo) >> 16) | (f2u(hi) & 0xffff0000u);
}
__device__ __forceinline__ u32 pack_bf16_rne(float lo, float hi) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  f2 v = {lo, hi};
  bf2 b = __builtin_convertvector(v, bf2);
  return __builtin_bit_cast(u32, b);
}

// MFMA row r (0..31) of the S^T block carries key kperm(r) of the 32-key block
// (bits 2 and 3 of r swapped), so accumulator register i of a lane in half h
// holds key 16*(i/8) + 8*h + i%8.
__device__ __forceinline__ int kperm(int r) { return (r & 0x13) | ((r & 4) << 1) | ((r & 8) >> 1); }

// octet (8-channel unit) of K that lane-half h contracts in 16-channel chunk ch;
// chunks never straddle a scale group of `G` channels.
template <int G> __device__ __forceinline__ int k_octet(int ch, int h) {
  constexpr int CPS = G / 16;  // chunks per group
  const int seg = ch / CPS, cl = ch % CPS;
  return seg * (G / 8) + h * CPS + cl;
}

template <int D, int BITS, int GK, int GV>
__global__ __launch_bounds__(256, 2) void fused_attn_kernel(AttnParams p) {
  constexpr int NSK = D / GK, NSV = D / GV;
  constexpr int WPR = D * BITS / 32;        // packed words per key row
  constexpr int RS = WPR + 4;               // LDS row stride of packed tiles (words)
  constexpr int NCH = D / 16;               // contraction chunks of QK^T
  constexpr int NDB = D / 32;               // 32-row blocks of O^T
  constexpr int VTS = BN + 8;               // V^T row stride (bf16 elements)

  __shared__ u32 lds_k[BN * RS];
  __shared__ u32 lds_vp[BN * RS];
  __shared__ __attribute__((aligned(16))) uint16_t lds_vt[D * VTS];
  __shared__ __attribute__((aligned(16))) float lds_ck[NSK][BN];   // ks * scale * log2e * kMul
  __shared__ __attribute__((aligned(16))) float lds_dk[NSK][BN];   // -ks * scale * log2e * (kzp + kOff)
  __shared__ __attribute__((aligned(16))) float lds_sv[NSV][BN];   // vs
  __shared__ __attribute__((aligned(16))) float lds_zv[NSV][BN];   // vzp + vOff

  // XCD-aware decode: consecutive workgroup ids go to different XCDs (8 of
  // them), so ids congruent mod 8 share an L2.  All query tiles of one
  // (batch, head) are given ids of one residue class to keep its packed K/V in
  // that XCD's L2.
  const int wg = blockIdx.x;
  const int xcd = wg & 7, slot = wg >> 3;
  const int bh = (slot / p.q_tiles) * 8 + xcd;
  const int qt = slot % p.q_tiles;
  if (bh >= p.bh_total) return;
  const int b = bh / p.Hkv, hs = bh % p.Hkv;
  const int hq = p.head_map ? p.head_map[hs] : hs;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, half = lane >> 5;

  // ---- this lane's query ----------------------------------------------------
  const int qrow = qt * BM + wave * 32 + col;
  const bool q_live = qrow < p.Lq;
  const int qrow_c = q_live ? qrow : p.Lq - 1;
  const __bf16 *qptr = p.q + ((int64_t)(b * p.Hq + hq) * p.Lq + qrow_c) * D;
  int limit = p.kv_limit ? min(p.kv_limit[qrow_c], p.Lk) : p.Lk;
  if (limit < 0) limit = 0;

  // Q^T operands, gathered in the slot order of the K codec
  u32 qb[NCH][4];
  float qsum[NSK];
#pragma unroll
  for (int s = 0; s < NSK; ++s) qsum[s] = 0.f;
#pragma unroll
  for (int ch = 0; ch < NCH; ++ch) {
    const int oct = k_octet<GK>(ch, half);
    uint16_t e[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      e[j] = reinterpret_cast<const uint16_t *>(qptr)[oct * 8 + KCodec<BITS>::slot_d(j)];
      qsum[ch / (GK / 16)] += u2f((u32)e[j] << 16);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) qb[ch][j] = (u32)e[2 * j] | ((u32)e[2 * j + 1] << 16);
  }
#pragma unroll
  for (int s = 0; s < NSK; ++s) qsum[s] += __shfl_xor(qsum[s], 32, 64);

  // ---- tile range -------------------------------------------------------------
  // every lane of the workgroup must run the same number of tiles
  __shared__ int lds_maxlim;
  if (tid == 0) lds_maxlim = 0;
  __syncthreads();
  atomicMax(&lds_maxlim, q_live ? limit : 0);
  __syncthreads();
  const int kv_end = lds_maxlim;
  const int n_tiles = (kv_end + BN - 1) / BN;
  int wave_minlim = q_live ? limit : p.Lk;
  for (int off = 1; off < 64; off <<= 1) wave_minlim = min(wave_minlim, __shfl_xor(wave_minlim, off, 64));

  floatx16_t oacc[NDB];
#pragma unroll
  for (int i = 0; i < NDB; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) oacc[i][j] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  float r_run[NSV];
#pragma unroll
  for (int s = 0; s < NSV; ++s) r_run[s] = 0.f;

  const int64_t kv_row0 = (int64_t)(b * p.Hkv + hs) * p.Lstride;
  const u32 *kw = p.k_words + kv_row0 * WPR;
  const u32 *vw = p.v_words + kv_row0 * WPR;

  constexpr int QUADS = BN * WPR / 4;                 // 16-byte pieces per packed tile
  constexpr int LPT = (QUADS + 255) / 256;            // pieces per thread
  u32x4_t kreg[LPT], vreg[LPT];
  float ksc = 0.f, kzp = 0.f, vsc = 0.f, vzp = 0.f;

  auto prefetch = [&](int tile) {
    const int t0 = tile * BN;
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int piece = tid + i * 256;
      if (LPT * 256 == QUADS || piece < QUADS) {
        const int key = min(t0 + piece / (WPR / 4), p.Lk - 1);
        const int64_t off = (int64_t)key * WPR + (piece % (WPR / 4)) * 4;
        kreg[i] = *reinterpret_cast<const u32x4_t *>(kw + off);
        vreg[i] = *reinterpret_cast<const u32x4_t *>(vw + off);
      }
    }
    // scales: thread t < 64*NS handles (key = t % 64, seg = t / 64)
    {
      const int key = min(t0 + (tid & 63), p.Lk - 1), seg = tid >> 6;
      if (seg < NSK) {
        const int64_t g = (kv_row0 + key) * NSK + seg;
        ksc = p.k_scale[g];
        kzp = p.k_zp ? p.k_zp[g] : 0.f;
      }
      if (seg < NSV) {
        const int64_t g = (kv_row0 + key) * NSV + seg;
        vsc = p.v_scale[g];
        vzp = p.v_zp ? p.v_zp[g] : 0.f;
      }
    }
  };

  if (n_tiles > 0) prefetch(0);

  for (int tile = 0; tile < n_tiles; ++tile) {
    const int t0 = tile * BN;
    __syncthreads();  // previous tile's LDS reads are finished
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int piece = tid + i * 256;
      if (LPT * 256 == QUADS || piece < QUADS) {
        const int key = piece / (WPR / 4), w4 = (piece % (WPR / 4)) * 4;
        *reinterpret_cast<u32x4_t *>(&lds_k[key * RS + w4]) = kreg[i];
        *reinterpret_cast<u32x4_t *>(&lds_vp[key * RS + w4]) = vreg[i];
      }
    }
    {
      const int key = tid & 63, seg = tid >> 6;
      if (seg < NSK) {
        const float c = ksc * p.scale_log2e;
        lds_ck[seg][key] = c * KCodec<BITS>::kMul;
        lds_dk[seg][key] = -c * (kzp + KCodec<BITS>::kOff);
      }
      if (seg < NSV) {
        lds_sv[seg][key] = vsc;
        lds_zv[seg][key] = vzp + VCodec<BITS>::kOff;
      }
    }
    __syncthreads();
    if (tile + 1 < n_tiles) prefetch(tile + 1);

    // ---- V: packed -> V^T bf16 (each thread: 4 keys x 8 channels) ---------------
    for (int blk = tid; blk < (BN / 4) * (D / 8); blk += 256) {
      const int kq = blk & (BN / 4 - 1), oct = blk / (BN / 4);
      float f[4][8];
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) VCodec<BITS>::codes(&lds_vp[(kq * 4 + kk) * RS], oct, f[kk]);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        uint2 v = make_uint2(pack_bf16_hi(f[0][j], f[1][j]), pack_bf16_hi(f[2][j], f[3][j]));
        *reinterpret_cast<uint2 *>(&lds_vt[(oct * 8 + j) * VTS + kq * 4]) = v;
      }
    }
    __syncthreads();

    // ---- S^T = K Q^T for the two 32-key blocks -----------------------------------
    float x[2][16];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      floatx16_t sacc[NSK];
#pragma unroll
      for (int s = 0; s < NSK; ++s)
#pragma unroll
        for (int j = 0; j < 16; ++j) sacc[s][j] = 0.f;
      const u32 *krow = &lds_k[(kb * 32 + kperm(col)) * RS];
#pragma unroll
      for (int ch = 0; ch < NCH; ++ch) {
        u32 a[4];
        KCodec<BITS>::expand(krow, k_octet<GK>(ch, half), a);
        u32x4_t av = {a[0], a[1], a[2], a[3]};
        u32x4_t bv = {qb[ch][0], qb[ch][1], qb[ch][2], qb[ch][3]};
        sacc[ch / (GK / 16)] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            __builtin_bit_cast(bf16x8_t, av), __builtin_bit_cast(bf16x8_t, bv), sacc[ch / (GK / 16)], 0, 0, 0);
      }
      // affine map: register i <-> key kb*32 + 16*(i/8) + 8*half + i%8
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = kb * 32 + 16 * (i >> 3) + 8 * half + (i & 7);
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < NSK; ++s) v += lds_ck[s][key] * sacc[s][i] + lds_dk[s][key] * qsum[s];
        x[kb][i] = v;
      }
    }

    // ---- mask (block-causal key limit, and the ragged last tile) -----------------
    if (t0 + BN > wave_minlim) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = t0 + kb * 32 + 16 * (i >> 3) + 8 * half + (i & 7);
          if (key >= limit) x[kb][i] = -INFINITY;
        }
    }

    // ---- online softmax ---------------------------------------------------------
    float mt = x[0][0];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) mt = fmaxf(mt, x[kb][i]);
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = fmaxf(m_run, mt);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    m_run = m_new;
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int d = 0; d < NDB; ++d)
#pragma unroll
        for (int j = 0; j < 16; ++j) oacc[d][j] *= alpha;
#pragma unroll
      for (int s = 0; s < NSV; ++s) r_run[s] *= alpha;
      l_run *= alpha;
    }
    // P'^T operands: for each V scale group, p * vs as bf16; 8 registers -> 4 dwords per 16-key chunk
    u32 pop[NSV][4][4];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      float pv[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        pv[i] = __builtin_amdgcn_exp2f(x[kb][i] - m_use);
        l_run += pv[i];
      }
#pragma unroll
      for (int s = 0; s < NSV; ++s) {
        // The zero-point term must see the same bf16-rounded weights as the
        // MFMA does, or the constant offset of the raw codes stops cancelling.
#pragma unroll
        for (int i2 = 0; i2 < 8; ++i2) {
          const int i = 2 * i2;
          const int key = kb * 32 + 16 * (i >> 3) + 8 * half + (i & 7);
          const u32 pk = pack_bf16_rne(pv[i] * lds_sv[s][key], pv[i + 1] * lds_sv[s][key + 1]);
          pop[s][kb * 2 + (i >> 3)][(i & 7) >> 1] = pk;
          r_run[s] += u2f(pk << 16) * lds_zv[s][key];
          r_run[s] += u2f(pk & 0xffff0000u) * lds_zv[s][key + 1];
        }
      }
    }

    // ---- O^T += V^T P'^T -----------------------------------------------------------
#pragma unroll
    for (int d = 0; d < NDB; ++d) {
      constexpr int DBS = GV / 32;  // 32-row blocks per V scale group
      const int s = d / DBS;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const u32x4_t av = *reinterpret_cast<const u32x4_t *>(&lds_vt[(d * 32 + col) * VTS + c * 16 + half * 8]);
        u32x4_t bv = {pop[s][c][0], pop[s][c][1], pop[s][c][2], pop[s][c][3]};
        oacc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                          __builtin_bit_cast(bf16x8_t, bv), oacc[d], 0, 0, 0);
      }
    }
  }

  // ---- epilogue -------------------------------------------------------------------
  l_run += __shfl_xor(l_run, 32, 64);
#pragma unroll
  for (int s = 0; s < NSV; ++s) r_run[s] += __shfl_xor(r_run[s], 32, 64);
  const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
  if (q_live) {
    __bf16 *optr = p.out + ((int64_t)(b * p.Hq + hq) * p.Lq + qrow) * D;
#pragma unroll
    for (int d = 0; d < NDB; ++d) {
      constexpr int DBS = GV / 32;
      const float r = r_run[d / DBS];
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        // registers 4*g4 .. 4*g4+3 are rows d*32 + 8*g4 + 4*half + 0..3 of O^T
        const float o0 = (oacc[d][4 * g4 + 0] - r) * inv, o1 = (oacc[d][4 * g4 + 1] - r) * inv;
        const float o2 = (oacc[d][4 * g4 + 2] - r) * inv, o3 = (oacc[d][4 * g4 + 3] - r) * inv;
        uint2 v = make_uint2(pack_bf16_rne(o0, o1), pack_bf16_rne(o2, o3));
        *reinterpret_cast<uint2 *>(optr + d * 32 + 8 * g4 + 4 * half) = v;
      }
    }
  }
}

template <int D, int BITS, int GK, int GV>
void launch(const AttnParams &p, hipStream_t st) {
  const int bh_pad = (p.bh_total + 7) / 8 * 8;
  dim3 grid((unsigned)(bh_pad * p.q_tiles));
  hipLaunchKernelGGL((fused_attn_kernel<D, BITS, GK, GV>), grid, dim3(256), 0, st, p);
}

template <int D, int BITS>
int dispatch_groups(const AttnParams &p, int gk, int gv, hipStream_t st) {
#define VARQ_G(GK_, GV_)                                   \
  if (gk == GK_ && gv == GV_) {                            \
    if constexpr (GK_ <= D && GV_ <= D) {                  \
      launch<D, BITS, GK_, GV_>(p, st);                    \
      return 0;                                            \
    }                                                      \
  }
  VARQ_G(128, 128) VARQ_G(64, 64) VARQ_G(32, 32) VARQ_G(32, 64)
#undef VARQ_G
  return -1;
}

}  // namespace

extern "C" int varq_fused_attn(const void *q, void *out,
                               const int32_t *k_words, const float *k_scale, const float *k_zp, int k_bits, int k_group,
                               const int32_t *v_words, const float *v_scale, const float *v_zp, int v_bits, int v_group,
                               int B, int Hq, int Hkv, const int32_t *head_map,
                               int Lq, int Lk, int Lk_stride, int D,
                               const int32_t *kv_limit, float softmax_scale, void *stream) {
  VARQ_CHECK_ARG(q && out && k_words && v_words && k_scale && v_scale, "fused_attn: null pointer");
  VARQ_CHECK_ARG(B > 0 && Hq > 0 && Hkv > 0 && Lq >= 0 && Lk >= 0 && Lk_stride >= Lk, "fused_attn: bad sizes");
  VARQ_CHECK_ARG(head_map || Hkv == Hq, "fused_attn: Hkv != Hq needs a head map");
  VARQ_CHECK_ARG(D == 64 || D == 128, "fused_attn: D must be 64 or 128 (got %d)", D);
  VARQ_CHECK_ARG(k_bits == 2 || k_bits == 4 || k_bits == 8, "fused_attn: bits must be 2, 4 or 8 (got %d)", k_bits);
  if (k_bits != v_bits)
    return varq_set_error(VARQ_ERR_UNSUPPORTED, "fused_attn: K and V bit-widths must match (%d vs %d)", k_bits, v_bits);
  VARQ_CHECK_ARG(k_group > 0 && v_group > 0 && D % k_group == 0 && D % v_group == 0, "fused_attn: groups must divide D");
  if (Lq == 0 || Lk == 0) {
    if (Lq > 0) return varq_set_error(VARQ_ERR_INVALID, "fused_attn: no keys to attend");
    return VARQ_OK;
  }
  VARQ_CHECK_ARG((int64_t)B * Hkv * Lk_stride * D < (1ll << 40), "fused_attn: cache too large");

  AttnParams p;
  p.q = reinterpret_cast<const __bf16 *>(q);
  p.out = reinterpret_cast<__bf16 *>(out);
  p.k_words = reinterpret_cast<const u32 *>(k_words);
  p.v_words = reinterpret_cast<const u32 *>(v_words);
  p.k_scale = k_scale; p.k_zp = k_zp; p.v_scale = v_scale; p.v_zp = v_zp;
  p.head_map = head_map; p.kv_limit = kv_limit;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.Lq = Lq; p.Lk = Lk; p.Lstride = Lk_stride;
  p.q_tiles = (Lq + BM - 1) / BM;
  p.bh_total = B * Hkv;
  p.scale_log2e = softmax_scale * kLog2e;
  hipStream_t st = (hipStream_t)stream;
  int rc = -1;
  if (D == 128) {
    if (k_bits == 4) rc = dispatch_groups<128, 4>(p, k_group, v_group, st);
    else if (k_bits == 8) rc = dispatch_groups<128, 8>(p, k_group, v_group, st);
    else rc = dispatch_groups<128, 2>(p, k_group, v_group, st);
  } else {
    if (k_bits == 4) rc = dispatch_groups<64, 4>(p, k_group, v_group, st);
    else if (k_bits == 8) rc = dispatch_groups<64, 8>(p, k_group, v_group, st);
    else rc = dispatch_groups<64, 2>(p, k_group, v_group, st);
  }
  if (rc)
    return varq_set_error(VARQ_ERR_UNSUPPORTED, "fused_attn: no kernel for D=%d bits=%d k_group=%d v_group=%d", D, k_bits,
                          k_group, v_group);
  VARQ_CHECK_LAUNCH("fused_attn");
  return VARQ_OK;
}

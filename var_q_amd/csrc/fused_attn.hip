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
// Design (one workgroup = 8 wavefronts = 256 queries of one (batch, head)):
//  * Both contractions run on v_mfma_f32_32x32x16_bf16 in transposed form,
//    S^T = K Q^T and O^T = V^T P^T, so that a lane owns one query column: row
//    max/sum are per-lane (one cross-half exchange per tile) and the S^T
//    accumulator registers are directly the B operand of the second MFMA.
//  * Packed K and V tiles go HBM -> registers -> LDS (16-byte loads, issued one to three
//    tiles ahead, one workgroup barrier per tile).  K is widened once per workgroup,
//    straight from the registers it was loaded into, to LDS rows that are MFMA A operands;
//    V goes to LDS packed and is widened and transposed by 2 keys x 8 channels per thread
//    (the PV contraction runs over keys).  Widened tiles are double-buffered, packed V and
//    the per-key parameters triple-buffered.
//  * Key rows are fed to the first MFMA in a permuted order chosen so that each
//    lane's accumulator registers hold 8 consecutive keys per 16-key chunk,
//    which makes the V^T operand a single 16-byte LDS read.
//  * Online softmax in the log2 domain against a reference that is only moved when a logit
//    gets 16 octaves above the maximum it was set from, and that is found out from the weights
//    (their sum, or the exponent bits of the packed bf16 pairs), not by a search for the row
//    maximum: the common tile needs no maximum, no subtraction and no rescale of the output
//    accumulators; the rare one is computed twice.
//  * Two forms of the operands:
//    - dequantized (the default of every kernel): (code - zp) * scale in fp32, rounded to the
//      attention's 16-bit type (bf16, or fp16 for the VAR path) when a tile is widened -- the
//      operands the reference's attention sees -- and a plain flash attention behind it;
//    - exact codes (opt-in; one group per key of 4- or 2-bit codes at head dim 128, bf16): the MFMA operands
//      are exact small numbers derived from the codes, never scaled or rounded.  A code lands in
//      the top mantissa bits of a bf16 1.x (raw = (code + kOff) / kMul), which costs one shift and
//      one and-or per two elements.  Scales are applied in fp32, zero-points ride on extra MFMA
//      work:
//         S[l,q]  = ck[l] * ( sum_d rawK[l,d] q[d]  -  (kzp[l]+kOff)/kMul * sum_d q[d] )
//         O[q,:]  = ( kMul * sum_l p'[l,q] rawV[l,:]  -  sum_l p'[l,q] (vzp[l]+kOff) ) / sum_l p[l,q]
//      The second term of S is a rank-1 update: both factors are split into three bf16 pieces
//      and laid on the 16 contraction slots of one more MFMA per key block.  The second term of
//      O is one more row of V^T (one more 32-row MFMA block whose row 0 carries vzp+kOff).
//      p' = bf16(p * vs[l]): log2(vs)/ck is added to S through spare slots of the rank-1 MFMA,
//      so exp2 yields p * vs directly, and the denominator is accumulated as sum_l p'[l,q] / vs[l]
//      by rows 4..6 of the extra block (1/vs in three bf16 pieces): numerator and denominator
//      then use the same rounded weights.  V zero-points beyond +-kZmax (data offset by hundreds
//      of quantization steps) or with a fractional part are split zp = zp_c + zp_r; the remainder
//      goes through an fp32 correction term on tiles that have one.
#include <type_traits>

#include "varq_common.h"

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;
typedef __attribute__((__vector_size__(4 * sizeof(u32)))) u32 u32x4_t;

constexpr int NW = 8;          // wavefronts per workgroup
constexpr int BM = NW * 32;    // queries per workgroup (32 per wavefront)
// (The D=64 kernels also exist with four wavefronts per workgroup, for launches of many (batch,
// head) pairs with at most 128 queries each -- the first steps of a scale schedule at a large
// batch -- see launch().)
constexpr int BN = 64;   // keys per tile
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kHeadroom = 15.f;   // exact-code kernels: octaves between a fresh softmax reference and the row maximum

constexpr int kMaxSegments = 16;
constexpr int kMaxSplits_v = 8;        // shares of a query block's keys in the general kernel
constexpr int kMaxKeyShares_v = 64;    // ... and in the kernel for few queries
constexpr int kChanTableRows = 4;   // LDS rows per segment of the per-channel tables

struct AttnParams {
  const __bf16 *q;
  __bf16 *out;
  const u32 *k_words, *v_words;
  const float *k_scale, *k_zp, *v_scale, *v_zp;
  // per-(head, channel) quantization (CHAN kernels): fp32 [Hkv, D] tables shared by all
  // tokens and batch entries; the per-key pointers above are unused then
  const float *k_chan_scale, *k_chan_zp, *v_chan_scale, *v_chan_zp;
  // the tables may change along the keys: keys [seg_end[s-1], seg_end[s]) use table s
  // (fp32 [nseg, Hkv, D]); this is a cache that was quantized step by step
  int nseg;
  int seg_end[kMaxSegments];
  const int32_t *head_map;
  const int32_t *kv_limit;
  int B, Hq, Hkv, Lq, Lk, Lstride;
  int q_tiles, bh_total;
  float scale_log2e;
  // the keys of a query block may be shared out over nsplit workgroups; each leaves its
  // normalized output (fp32 [nsplit][B*Hkv*Lq][D]) and softmax statistics (reference,
  // denominator: fp32 [nsplit][B*Hkv*Lq][2]) for the combining kernel.  nsplit = 1: no
  // workspace, the output is written directly.
  int nsplit;
  float *ws_o, *ws_ml;
  // the caller asked for exact codes in the MFMA operands where such a kernel exists (host side only)
  int exact_codes;
  int f16;   // q, out and the MFMA operands are fp16 (host side only: it selects the instantiation)
  int fq_share_blocks;   // few-queries kernel: 32-key blocks per share of the keys
  // memory layout, in rows (a row = the D values of one token of one head):
  // q row = b*q_bs + h*q_hs + i*q_ts, out row likewise with o_*, key row = b*kv_bs + slot*kv_hs + j*kv_ts.
  // BHLc: (H*L, L, 1); BLHc (the layout of the flash-attention call): (L*H, 1, H).
  int64_t q_bs, q_hs, q_ts, o_bs, o_hs, o_ts, kv_bs, kv_hs, kv_ts;
};

__device__ __forceinline__ u32 pack_bf16_hi(float lo, float hi) {  // exact for values with <= 8 significant bits
  return __builtin_amdgcn_perm(f2u(hi), f2u(lo), 0x07060302u);   // {hi[31:16], lo[31:16]} in one v_perm_b32
}

// ---- V side code widening ----------------------------------------------------
// The V^T operand of the second MFMA holds, like the K operand of the first, an
// affine image `raw` of the code (code = kMul * raw - kOff) that costs one shift
// and one and-or per two elements.  `pairs` widens octet `oct` of two adjacent key
// rows at once: out[j] = {raw(row0, channel j), raw(row1, channel j)} as a bf16
// pair, which is one dword of the transposed tile.  The zero-point is not folded
// in here; it rides on an extra MFMA row (see the kernel).  kZmax bounds the
// part of the zero-point handled that way: kOff + zp must be a bf16-exact integer.
template <int BITS> struct VCodec;
template <> struct VCodec<4> {
  static constexpr float kMul = 16.f, kOff = 24.f, kZmax = 232.f;
  static constexpr u32 kStageXor = 0x88888888u;   // applied once when the tile is staged: nibble -> code + 8
  __device__ static __forceinline__ void pairs(const u32 *row0, const u32 *row1, int oct, u32 M, u32 (&o)[8]) {
    const u32 w0 = row0[oct], w1 = row1[oct];
    constexpr u32 B = 0x3f803f80u;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      // byte k of both rows, 16 bits apart: nibbles 2k and 2k+1
      const u32 x = __builtin_amdgcn_perm(w1, w0, 0x0c000c00u | (u32)k | ((u32)(4 + k) << 16));
      o[2 * k] = ((x << 3) & M) | B;
      o[2 * k + 1] = ((x >> 1) & M) | B;
    }
  }
};
template <> struct VCodec<2> {
  static constexpr float kMul = 4.f, kOff = 6.f, kZmax = 250.f;
  static constexpr u32 kStageXor = 0xaaaaaaaau;
  __device__ static __forceinline__ void pairs(const u32 *row0, const u32 *row1, int oct, u32 M, u32 (&o)[8]) {
    // the octet is half a word: put the two rows' halves side by side
    const u32 x = __builtin_amdgcn_perm(row1[oct >> 1], row0[oct >> 1], 0x05040100u + (u32)(oct & 1) * 0x02020202u);
    constexpr u32 B = 0x3f803f80u;
    o[0] = ((x << 5) & M) | B;
    o[1] = ((x << 3) & M) | B;
    o[2] = ((x << 1) & M) | B;
    o[3] = ((x >> 1) & M) | B;
    o[4] = ((x >> 3) & M) | B;
    o[5] = ((x >> 5) & M) | B;
    o[6] = ((x >> 7) & M) | B;
    o[7] = ((x >> 9) & M) | B;
  }
};
template <> struct VCodec<8> {
  static constexpr float kMul = 1.f, kOff = 0.f, kZmax = 256.f;
  static constexpr u32 kStageXor = 0u;
  __device__ static __forceinline__ void pairs(const u32 *row0, const u32 *row1, int oct, u32, u32 (&o)[8]) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int w0 = (int)row0[2 * oct + h], w1 = (int)row1[2 * oct + h];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        o[4 * h + j] = pack_bf16_hi((float)(int)__builtin_amdgcn_sbfe(w0, 8 * j, 8),
                                    (float)(int)__builtin_amdgcn_sbfe(w1, 8 * j, 8));
    }
  }
};
// The kernels that dequantize want the images as fp32 numbers: f0[j], f1[j] = raw of channel j of
// the octet in the two rows.  Bytes are converted once; the narrower fields come out of `pairs`.
template <int BITS>
__device__ __forceinline__ void v_pair_values(const u32 *row0, const u32 *row1, int oct, u32 M, float (&f0)[8], float (&f1)[8]) {
  if constexpr (BITS == 8) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int w0 = (int)row0[2 * oct + h], w1 = (int)row1[2 * oct + h];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        f0[4 * h + j] = (float)(int)__builtin_amdgcn_sbfe(w0, 8 * j, 8);
        f1[4 * h + j] = (float)(int)__builtin_amdgcn_sbfe(w1, 8 * j, 8);
      }
    }
  } else {
    u32 pr[8];
    VCodec<BITS>::pairs(row0, row1, oct, M, pr);
#pragma unroll
    for (int j = 0; j < 8; ++j) { f0[j] = __builtin_bit_cast(float, pr[j] << 16); f1[j] = __builtin_bit_cast(float, pr[j] & 0xffff0000u); }
  }
}

__device__ __forceinline__ u32 pack_bf16_rne(float lo, float hi) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  f2 v = {lo, hi};
  bf2 b = __builtin_convertvector(v, bf2);
  return __builtin_bit_cast(u32, b);
}
__device__ __forceinline__ u32 pack_f16_rne(float lo, float hi) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  f2 v = {lo, hi};
  h2 b = __builtin_convertvector(v, h2);
  return __builtin_bit_cast(u32, b);
}
// two fp32 values rounded to nearest-even into a pair of the attention's 16-bit type
template <bool F16> __device__ __forceinline__ u32 pack_io_rne(float lo, float hi) {
  if constexpr (F16) return pack_f16_rne(lo, hi);
  else return pack_bf16_rne(lo, hi);
}
// D (32x32 fp32) += A (32x16) B (16x32), operands in the attention's 16-bit type
template <bool F16> __device__ __forceinline__ floatx16_t mfma_32x32x16(u32x4_t a, u32x4_t b, floatx16_t c) {
  if constexpr (F16) {
    typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
}
// x = h0 + h1 + h2 exactly, each piece a bf16 (returned as its 16 bits): three
// 8-bit slices of the 24-bit significand
__device__ __forceinline__ void split3_bf16(float x, u32 &h0, u32 &h1, u32 &h2) {
  const float x0 = u2f(f2u(x) & 0xffff0000u);
  const float r1 = x - x0;
  const float x1 = u2f(f2u(r1) & 0xffff0000u);
  const float x2 = r1 - x1;
  h0 = f2u(x0) >> 16; h1 = f2u(x1) >> 16; h2 = f2u(x2) >> 16;
}

// MFMA row r (0..31) of the S^T block carries key kperm(r) of the 32-key block
// (bits 2 and 3 of r swapped), so accumulator register i of a lane in half h
// holds key 16*(i/8) + 8*h + i%8.
__device__ __forceinline__ int kperm(int r) { return (r & 0x13) | ((r & 4) << 1) | ((r & 8) >> 1); }

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
  static constexpr u32 kStageXor = 0x88888888u;   // applied once when the tile is staged
  static constexpr u32 kMask = 0x00780078u;
  // `M` is kMask held in a vector register, which lets each output be one shift and one v_and_or_b32
  __device__ static __forceinline__ void expand(const u32 *lds_row, int oct, u32 M, u32 (&o)[4]) {
    const u32 w = lds_row[oct];
    constexpr u32 B = 0x3f803f80u;
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
  static constexpr u32 kStageXor = 0xaaaaaaaau;
  static constexpr u32 kMask = 0x00600060u;
  __device__ static __forceinline__ void expand(const u32 *lds_row, int oct, u32 M, u32 (&o)[4]) {
    const u32 w = (lds_row[oct >> 1] >> ((oct & 1) * 16)) & 0xffffu;
    // fields m (bits 2m) and m+4 (bits 2m+8): move to bits 5..6 and 21..22
    const u32 t = (w & 0xffu) | ((w & 0xff00u) << 8);  // low byte: fields 0-3, byte 2: fields 4-7
    constexpr u32 B = 0x3f803f80u;
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
  static constexpr u32 kStageXor = 0u, kMask = 0u;
  __device__ static __forceinline__ void expand(const u32 *lds_row, int oct, u32, u32 (&o)[4]) {
    const u32 w0 = lds_row[2 * oct], w1 = lds_row[2 * oct + 1];
    float f[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[j] = (float)(int)__builtin_amdgcn_sbfe((int)w0, 8 * j, 8);
      f[4 + j] = (float)(int)__builtin_amdgcn_sbfe((int)w1, 8 * j, 8);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = pack_bf16_hi(f[2 * j], f[2 * j + 1]);
  }
};

// The kernels that dequantize want the images as fp32 numbers, in the operand's slot order.
template <int BITS> __device__ __forceinline__ void k_values(const u32 *q4, int oct, u32 M, float (&f)[8]) {
  if constexpr (BITS == 8) {
    const u32 w0 = q4[2 * oct], w1 = q4[2 * oct + 1];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[j] = (float)(int)__builtin_amdgcn_sbfe((int)w0, 8 * j, 8);
      f[4 + j] = (float)(int)__builtin_amdgcn_sbfe((int)w1, 8 * j, 8);
    }
  } else {
    u32 a[4];
    KCodec<BITS>::expand(q4, oct, M, a);
#pragma unroll
    for (int m = 0; m < 4; ++m) { f[2 * m] = __builtin_bit_cast(float, a[m] << 16); f[2 * m + 1] = __builtin_bit_cast(float, a[m] & 0xffff0000u); }
  }
}

// ---- dequantizing 4-bit codes through bytes (the kernel for few queries) ---------------------
// That kernel is bound by its vector instructions, most of them widening: field -> float, minus
// zero-point, times scale, round to bf16, 4.5 instructions per element.  For 4-bit codes there is a
// shorter way to the same bits.  A staged word holds u = code + 8 per nibble; two masks put the
// eight nibbles into the bytes of two dwords, one add per dword (no carries between bytes) makes
// every byte t = u + A with A = 120 - zp, i.e. t - 128 = code - zp, v_cvt_f32_ubyte turns a byte
// into a float in one instruction, and fma(t, s, -128 s) is RN((t - 128) s) = RN((code - zp) * scale),
// the very product the reference rounds (VAR_Q/quant.py:123-124 with a zero-point): -128 s is exact
// and an fma rounds once.  3 instructions per element.  It needs an integer zero-point with A in
// [0, 240] (|zp| <= 120: every zero-point the quantizer derives from data that straddles or lies
// near zero); a block with any other zero-point takes the general form, which computes the same
// values.  (In the kernels for many queries, which are not bound by the count of their vector
// instructions, the same change was measured: bit-identical results, no gain -- 752 against 745 us
// on the configuration-4 shape, 74.7 against 71.4 us on configuration 2 -- so they keep one form.)
__device__ __forceinline__ bool byte_bias4(float zp, u32 &a4) {
  const float a = 120.f - zp;
  const bool ok = a >= 0.f && a <= 240.f && a == __builtin_rintf(a);
  a4 = ok ? (u32)(int)a * 0x01010101u : 0u;
  return ok;
}
__device__ __forceinline__ float ubyte_f32(u32 x, int k) { return (float)((x >> (8 * k)) & 0xffu); }   // v_cvt_f32_ubyte<k>

// octet (8-channel unit) of K that lane-half h contracts in 16-channel chunk ch;
// chunks never straddle a scale group of `G` channels.
template <int G> __device__ __forceinline__ int k_octet(int ch, int h) {
  constexpr int CPS = G / 16;  // chunks per group
  const int seg = ch / CPS, cl = ch % CPS;
  return seg * (G / 8) + h * CPS + cl;
}

// LDS layout of the attention kernel (bytes), shared by kernel and launcher.
// kDeq: the kernel dequantizes when a tile is widened (see the kernel) and has no rank-1 operands.
// That is the form of every kernel unless the caller asks for exact codes (EXACT), which exist
// where they were measured to be the faster form: one group per key of 4- or 2-bit codes at
// D=128.  (Per-channel tables, more than one K or V group per key, every kernel at D=64 and the
// 8-bit kernels at D=128 are faster dequantizing, and have no exact-code instantiation.)
template <int D, int BITS, int GK, int GV, bool CHAN> struct AttnForms {
  static constexpr bool kHasExact = !CHAN && D / GK == 1 && D / GV == 1 && D == 128 && BITS != 8;
};
template <int D, int BITS, int GK, int GV, bool CHAN, bool EXACT = false> struct AttnLds {
  static_assert(!EXACT || AttnForms<D, BITS, GK, GV, CHAN>::kHasExact, "no exact-code form of this kernel");
  static constexpr bool kDeq = !EXACT;
  static constexpr int WPR = D * BITS / 32;
  static constexpr int RSV = WPR + 1;       // packed V row stride (words): odd, bank spread
  static constexpr bool kFoldSv = !kDeq && (D / GV == 1);   // one V group: its scale rides inside the logits
  static constexpr int kParFloats = ((D / GK) + (kFoldSv ? 1 : 2) * (D / GV)) * 64;
  static constexpr int RSR = 64 + 8;        // stride (bf16) of the rows feeding the extra PV MFMA
  static constexpr int KXS = D + 8;         // stride (bf16) of a widened K row: 16-byte rows, bank spread
  static constexpr int kKx = 0;             // widened K, two tiles
  static constexpr int kVp = kKx + 2 * 64 * KXS * 2;
  static constexpr int kVt = (kVp + 3 * 64 * RSV * 4 + 15) / 16 * 16;
  static constexpr int kKz = kVt + 2 * D * (64 + 8) * 2;          // rank-1 operands of S^T, 2 x 16 bytes per key and group
  static constexpr int kWz = kKz + (kDeq ? 0 : 3 * (D / GK) * 64 * 32);   // 8 rows per slot for the extra PV MFMA
  static constexpr int kPar = kWz + 3 * 8 * RSR * 2;
  static constexpr int kFlag = kPar + 3 * kParFloats * 4;
  static constexpr int kBytes = kFlag + 16;
};

// CHAN: scales and zero-points per (head, channel) instead of per (key, channel group), in up
// to 16 tables that change along the keys (a cache quantized step by step has one per step).
// Such a kernel dequantizes when a tile is widened, like the kernels for several groups per key
// (DEQ below): K[l,d] = (code[l,d] - zk_s[d]) * sk_s[d] with s the segment of key l, rounded to
// bf16 -- what the reference's attention sees -- and likewise V.  The tables of the head sit in
// LDS; a tile inside one segment reads that segment's rows, a tile that straddles segments
// looks the segment up per key.  Everything behind the widening is a plain bf16 flash attention
// that knows nothing of tables or segments.
// WPS: wavefronts per SIMD the register allocation aims at (2, or 4: two 8-wavefront workgroups
// per compute unit at 128 registers, which the D=64 kernels that dequantize afford)
// F16: q, out and the MFMA operands are fp16 instead of bf16 (dequantized K and V are rounded to
// fp16, as the reference's fp16 attention call sees them: VAR/models/basic_var.py:157-158 under the
// fp16 autocast of scripts/inference_multi_VAR.py:123); dequantizing kernels only.
template <int D, int BITS, int GK, int GV, bool CHAN, int NWV = 8, int WPS = 2, bool EXACT = false, bool F16 = false>
__global__ __launch_bounds__(NWV * 64, WPS) void fused_attn_kernel(AttnParams p) {
  static_assert(!(F16 && EXACT), "the exact-code form builds bf16 images of the codes");
  static_assert(!CHAN || (GK == D && GV == D), "per-channel tables go with the single-group kernels");
  constexpr int NW = NWV, NT = NWV * 64, BM = NWV * 32;   // (shadow the defaults of the file)
  constexpr int NSK = D / GK, NSV = D / GV;
  // DEQ: the kernel dequantizes when a tile is widened -- (code - zp) * scale in fp32, rounded to
  // bf16, the very values the reference's attention sees after its dequantize and downcast
  // (VAR_Q/quant.py:216-224, VAR/models/basic_var.py:158) -- and then runs like a plain bf16 flash
  // attention: one accumulator, one set of weights, whatever the group count, no rank-1 MFMA and
  // no extra O^T block (the softmax denominator is summed on the vector ALU).  With several K or
  // V groups per key, exact codes in the MFMAs would need one logit accumulator and one rank-1
  // MFMA per K group and one set of weights and one extra MFMA per V group (19 -> 28 MFMAs per
  // key block at four groups, and registers that do not exist); where there is one group, which
  // form is faster was measured (see AttnForms).
  constexpr bool DEQ = AttnLds<D, BITS, GK, GV, CHAN, EXACT>::kDeq;
  constexpr int NSKA = DEQ ? 1 : NSK, NSVA = DEQ ? 1 : NSV;   // accumulators / weight sets
  // (Exact codes are instantiated for one group per key only, so NSKA = NSVA = 1 in every kernel that
  // exists; the exact-code form is nevertheless written for any group count -- its loops over
  // groups are single passes today -- because AttnForms::kHasExact is a measured choice that may move.)
  static_assert(DEQ || (NSK == 1 && NSV == 1), "exact codes with several groups per key: AttnForms sends those to the dequantizing form");
  static_assert(NW >= NSK && NW >= NSV && NW >= 2, "one wavefront per K group and per V group stages the parameters");
  constexpr int WPR = D * BITS / 32;        // packed words per key row
  constexpr int NCH = D / 16;               // contraction chunks of QK^T
  constexpr int NDB = D / 32;               // 32-row blocks of O^T
  constexpr int VTS = BN + 8;               // V^T row stride (bf16 elements)
  using L = AttnLds<D, BITS, GK, GV, CHAN, EXACT>;

  // Pipelined LDS buffers (one workgroup barrier per tile):
  //   packed V and the per-key parameters of tile t live in slot t % 3, the
  //   widened K and the widened V^T of tile t in slot t % 2.
  // While tile t is being attended, K and V of tile t+1 are widened (K straight
  // from the registers it was loaded into one iteration earlier, once per
  // workgroup, so the eight wavefronts share the work) and packed V of tile t+2 is
  // written from its registers.
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  uint16_t *const lds_kx = reinterpret_cast<uint16_t *>(lds_raw + L::kKx);  // [2][BN][KXS] widened K codes (MFMA A operands)
  u32 *const lds_vp = reinterpret_cast<u32 *>(lds_raw + L::kVp);          // [3][BN][RSV]
  uint16_t *const lds_vt = reinterpret_cast<uint16_t *>(lds_raw + L::kVt);  // [2][D][VTS]  raw V codes, transposed
  u32x4_t *const lds_kz = reinterpret_cast<u32x4_t *>(lds_raw + L::kKz);  // [3][NSK][BN][2] rank-1 A operands (per lane half)
  // [3][8][RSR] bf16 rows of the extra PV MFMA: row s < NSV = vzp_c + kOff of group s,
  // rows 4..6 = the three bf16 pieces of 1/vs of group 0, row 7 = zeros
  uint16_t *const lds_wz = reinterpret_cast<uint16_t *>(lds_raw + L::kWz);
  float *const lds_par = reinterpret_cast<float *>(lds_raw + L::kPar);    // [3][L::kParFloats]
  int *const lds_flag = reinterpret_cast<int *>(lds_raw + L::kFlag);      // [3] tile+1 if that tile has a zero-point remainder
  // CHAN: the tables of this head for every segment, [nseg][4][D] fp32, filled once in the
  // prologue, as the widening steps use them: row 0 = kMul * sk and row 1 = (zk + kOff) / kMul in
  // the slot order of the K operand octets, row 2 = kMul * sv and row 3 = (zv + kOff) / kMul by
  // channel ((code - z) * s = (raw - z') * s' for the code image raw = (code + kOff) / kMul, both
  // rescalings exact)
  float *const lds_tab = reinterpret_cast<float *>(lds_raw + (L::kBytes + 15) / 16 * 16);
  constexpr int TR = kChanTableRows;
  constexpr int KXS = L::KXS, RSV = L::RSV;
  // parameter block of one tile: ck [NSK][BN]; vr [NSV][BN]; sv [NSV][BN] unless folded
  constexpr bool FOLD_SV = L::kFoldSv;
  constexpr int RSR = L::RSR;
  constexpr int P_CK = 0, P_VR = NSK * BN, P_SV = P_VR + NSV * BN;
  constexpr int P_VZ = P_VR;   // DEQ: per (V group, key) the zero-point image; P_SV holds the scale image

  // XCD-aware decode: consecutive workgroup ids go to different XCDs (8 of
  // them), so ids congruent mod 8 share an L2.  All query tiles of one
  // (batch, head) are given ids of one residue class to keep its packed K/V in
  // that XCD's L2.
  const int wg = blockIdx.x;
  const int xcd = wg & 7, slot_s = wg >> 3;
  const int split = p.nsplit > 1 ? slot_s % p.nsplit : 0;
  const int slot = p.nsplit > 1 ? slot_s / p.nsplit : slot_s;
  // (a token-major cache: the key rows of neighbouring heads share cache lines, so an XCD takes a
  // run of consecutive (batch, head) pairs there instead of every eighth)
  const int grp = slot / p.q_tiles;
  const int bh = p.kv_hs == 1 && p.kv_ts > 1 ? xcd * ((p.bh_total + 7) >> 3) + grp : grp * 8 + xcd;
  const int qt = slot % p.q_tiles;
  if (bh >= p.bh_total) return;
  const int b = bh / p.Hkv, hs = bh % p.Hkv;
  const int hq = p.head_map ? p.head_map[hs] : hs;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, half = lane >> 5;

  // ---- this lane's query ----------------------------------------------------
  const int qrow = qt * BM + wave * 32 + col;
  const bool q_live = qrow < p.Lq;
  const bool wave_live = qt * BM + wave * 32 < p.Lq;   // wave-uniform
  const int qrow_c = q_live ? qrow : p.Lq - 1;
  const __bf16 *qptr = p.q + (b * p.q_bs + hq * p.q_hs + qrow_c * p.q_ts) * D;
  int limit = p.kv_limit ? min(p.kv_limit[qrow_c], p.Lk) : p.Lk;
  if (limit < 0) limit = 0;

  // Q^T operands, gathered in the slot order of the K codec
  u32x4_t qb[NCH];
  u32x4_t bq[NSK];
  // The K zero-point term -(kzp+kOff)/kMul * sum(q) is a rank-1 update of S^T and
  // rides on one more MFMA per key block and group.  Both factors are split into
  // three bf16 pieces (a0+a1+a2, b0+b1+b2, exact) and the 9 products are laid on
  // the 16 contraction slots: slots 0..7 (lower lane half) carry
  // A = a0 a0 a0 a1 a1 a1 a2 a2 against B = b0 b1 b2 b0 b1 b2 b0 b1 (a2*b2, 2^-32 of
  // the term, is dropped).  With a single V group, slots 0..2 of the upper half add
  // log2(vs)/ck (three pieces against 1.0), which makes exp2(logit) come out as
  // p * vs without a multiplication; the other upper slots are zero.
  // (the raw values were requested into qb earlier -- the prologue does, to overlap the trip
  // with its other loads)
  auto load_q = [&]() {
    float qsum[NSK];
#pragma unroll
    for (int s = 0; s < NSK; ++s) qsum[s] = 0.f;
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
      // the octet's eight channels, loaded in one 16-byte piece, into the codec's slot order
      const u32x4_t raw = qb[ch];
#pragma unroll
      for (int j2 = 0; j2 < 4; ++j2) {
        // operand slots 2*j2 and 2*j2+1, one dword
        const int d0 = KCodec<BITS>::slot_d(2 * j2), d1 = KCodec<BITS>::slot_d(2 * j2 + 1);   // channels within the octet
        const u32 lo = (raw[d0 >> 1] >> (16 * (d0 & 1))) << 16, hi = (raw[d1 >> 1] >> (16 * (d1 & 1))) << 16;
        qb[ch][j2] = (lo >> 16) | hi;
        qsum[ch / (GK / 16)] += u2f(lo) + u2f(hi);
      }
    }
#pragma unroll
    for (int s = 0; s < NSK; ++s) qsum[s] += __shfl_xor(qsum[s], 32, 64);
#pragma unroll
    for (int s = 0; s < (DEQ ? 0 : NSK); ++s) {
      u32 b0, b1, b2;
      split3_bf16(qsum[s], b0, b1, b2);
      if (half == 0) bq[s] = u32x4_t{b0 | (b1 << 16), b2 | (b0 << 16), b1 | (b2 << 16), b0 | (b1 << 16)};
      else if (FOLD_SV && s == 0) bq[s] = u32x4_t{0x3f803f80u, 0x00003f80u, 0u, 0u};
      else bq[s] = u32x4_t{0u, 0u, 0u, 0u};
    }
  };
  // ---- tile range: every lane of the workgroup runs the same number of tiles ----
  __shared__ int lds_maxlim;
  int kv_end = p.Lk;   // without per-query limits every query sees all keys
  if (p.kv_limit) {
    if (tid == 0) lds_maxlim = 0;
    __syncthreads();
    atomicMax(&lds_maxlim, q_live ? limit : 0);
    __syncthreads();
    kv_end = lds_maxlim;
  }
  int n_tiles = (kv_end + BN - 1) / BN;
  // segment ends in LDS: indexing the kernel arguments with a run-time index would move
  // the whole argument block to scratch memory (literal indices only, for the same reason)
  __shared__ int lds_seg_end[kMaxSegments];
  if constexpr (CHAN) {
    if (p.nseg > 1 && tid == 0) {
#define VARQ_SEG(S) lds_seg_end[S] = p.seg_end[S];
      VARQ_SEG(0) VARQ_SEG(1) VARQ_SEG(2) VARQ_SEG(3) VARQ_SEG(4) VARQ_SEG(5) VARQ_SEG(6) VARQ_SEG(7)
      VARQ_SEG(8) VARQ_SEG(9) VARQ_SEG(10) VARQ_SEG(11) VARQ_SEG(12) VARQ_SEG(13) VARQ_SEG(14) VARQ_SEG(15)
#undef VARQ_SEG
      static_assert(kMaxSegments == 16, "the list above names every segment");
    }
    // (read behind the prologue's first barrier)
  }
  int tbase = 0;   // index of this workgroup's first tile in the block's tile sequence
  if (p.nsplit > 1) {
    // this workgroup's share of the tiles: [t_begin, t_end) of the block's tile sequence
    const int t_begin = n_tiles * split / p.nsplit, t_end = n_tiles * (split + 1) / p.nsplit;
    tbase = t_begin;
    n_tiles = t_end - t_begin;
  }
  const int tile_base = tbase * BN;   // first key of this workgroup's tiles
  // The K prefetch, the V prefetch and the widening each walk the tiles in order.
  int pk_tile = 0, pv_tile = 0;
  // CHAN: segment of the first key of the next tile to be widened, and where that segment ends
  // (wave-uniform; the tiles are widened in order, K and V of a tile one after the other)
  int wseg = 0, wseg_end = p.Lk;
  int wave_minlim = q_live ? limit : p.Lk;
  for (int off = 1; off < 64; off <<= 1) wave_minlim = min(wave_minlim, __shfl_xor(wave_minlim, off, 64));

  floatx16_t oacc[NDB];
#pragma unroll
  for (int i = 0; i < NDB; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) oacc[i][j] = 0.f;
  // extra O^T block: row s < NSV: sum_l p'_s * (vzp_c + kOff); rows 4..6: pieces of the
  // softmax denominator sum_l p'_0 / vs_0, i.e. the sum of the weights as rounded for the MFMA
  floatx16_t racc;
#pragma unroll
  for (int j = 0; j < 16; ++j) racc[j] = 0.f;
  // DEQ: no extra block; the softmax denominator is summed on the vector ALU from the weights as
  // rounded for the MFMA (this lane's keys; the two lane halves are added in the epilogue)
  float l_part = 0.f;
  float m_ref = 0.f;                 // softmax reference (log2 domain)
  float r_run[NSVA];                 // sum_l p' * vzp_r, only fed on tiles with a remainder
#pragma unroll
  for (int s = 0; s < NSVA; ++s) r_run[s] = 0.f;

  const int64_t kv_row0 = b * p.kv_bs + hs * p.kv_hs;
  const int64_t kv_ts = p.kv_ts;
  const u32 *kw = p.k_words + kv_row0 * WPR;
  const u32 *vw = p.v_words + kv_row0 * WPR;

  constexpr int QUADS = BN * WPR / 4;                 // 16-byte pieces per packed tile
  constexpr int LPT = (QUADS + NT - 1) / NT;          // pieces per thread
  // The K tile is loaded in pieces of KPW words, small enough that every thread of the workgroup
  // has one where the tile allows it (the thread that loads a piece widens it, so this spreads
  // the widening evenly: 2-bit codes at D=64 would otherwise occupy a single wavefront).
  // (the V tile is widened in (BN/2)*(D/8) items by the upper wavefronts; where those are fewer than
  // the threads, the K pieces go to the threads that are left)
  constexpr int K_THREADS = ((BN / 2) * (D / 8) < NT) ? NT - (BN / 2) * (D / 8) : NT;
  // (measured: 5-9 % faster for 2-bit codes and at D=64; 4-bit codes at D=128 are 5 % slower in
  // 8-byte pieces -- twice the per-piece parameter loads -- and keep 16-byte ones)
  constexpr int KPW = (DEQ && (D == 64 || BITS == 2) && BN * WPR / K_THREADS < 4) ? (BN * WPR / K_THREADS < 2 ? 1 : 2) : 4;
  constexpr int KPIECES = BN * WPR / KPW, KPPR = WPR / KPW;   // pieces per tile, per key row
  constexpr int KLPT = (KPIECES + NT - 1) / NT;
  u32x4_t kreg[KLPT], vreg[LPT];   // (a K piece uses the first KPW words of its register)
  float ksc = 0.f, kzp = 0.f, vsc = 0.f, vzp = 0.f, ksc0 = 0.f;
  // DEQ: scale and zero-point of the K groups that the thread's 16-byte pieces hold (a piece is
  // 128 / BITS channels of one key: one group, or two for 2-bit codes in groups of 32)
  constexpr int CPP = KPW * 32 / BITS;                  // channels per piece
  constexpr int GPP = (DEQ && CPP > GK) ? CPP / GK : 1; // groups per piece
  constexpr bool KGP = DEQ && !CHAN;                    // K group parameters travel with the pieces
  float kgs[KGP ? KLPT * GPP : 1], kgz[KGP ? KLPT * GPP : 1];

  auto prefetch_k = [&](int) {   // the next tile of the K stream
    const int t0 = tile_base + pk_tile * BN;
    ++pk_tile;
#pragma unroll
    for (int i = 0; i < KLPT; ++i) {
      const int piece = tid + i * NT;
      if (KLPT * NT == KPIECES || piece < KPIECES) {
        const int key = min(t0 + piece / KPPR, p.Lk - 1);
        const u32 *src = kw + key * kv_ts * WPR + (piece % KPPR) * KPW;
        if constexpr (KPW == 4) kreg[i] = *reinterpret_cast<const u32x4_t *>(src);
        else if constexpr (KPW == 2) { const uint2 t = *reinterpret_cast<const uint2 *>(src); kreg[i][0] = t.x; kreg[i][1] = t.y; }
        else kreg[i][0] = src[0];
        if constexpr (KGP) {
          const int g0 = (piece % KPPR) * CPP / GK;   // first group of the piece
#pragma unroll
          for (int j = 0; j < GPP; ++j) {
            const int64_t g = (kv_row0 + key * kv_ts) * NSK + g0 + j;
            kgs[i * GPP + j] = p.k_scale[g];
            kgz[i * GPP + j] = p.k_zp ? p.k_zp[g] : 0.f;
          }
        }
      }
    }
  };
  auto prefetch = [&](int) {   // the next tile of the V stream
    const int t0 = tile_base + pv_tile * BN;
    ++pv_tile;
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int piece = tid + i * NT;
      if (LPT * NT == QUADS || piece < QUADS) {
        const int key = min(t0 + piece / (WPR / 4), p.Lk - 1);
        vreg[i] = *reinterpret_cast<const u32x4_t *>(vw + key * kv_ts * WPR + (piece % (WPR / 4)) * 4);
      }
    }
    // scales: thread t handles key t % 64; wavefront w takes K group w and V group
    // 3 - w, which puts the K and the V arithmetic of the single-group case on
    // different wavefronts
    if constexpr (!CHAN) {   // (per-channel tables: no per-key parameters)
      const int key = min(t0 + (tid & 63), p.Lk - 1), seg = tid >> 6, vseg = NW - 1 - seg;
      if (!DEQ && seg < NSK) {
        const int64_t g = (kv_row0 + key * kv_ts) * NSK + seg;
        ksc = p.k_scale[g];
        kzp = p.k_zp ? p.k_zp[g] : 0.f;
      }
      if (vseg < NSV) {
        const int64_t g = (kv_row0 + key * kv_ts) * NSV + vseg;
        vsc = p.v_scale[g];
        vzp = p.v_zp ? p.v_zp[g] : 0.f;
        if (FOLD_SV) ksc0 = p.k_scale[(kv_row0 + key * kv_ts) * NSK];
      }
    }
  };

  // registers -> LDS slot of `tile` (packed words as they are, parameters precombined)
  auto stage = [&](int tile) {
    const int sl = tile % 3;
    u32 *vp = lds_vp + sl * BN * RSV;
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int piece = tid + i * NT;
      if (LPT * NT == QUADS || piece < QUADS) {
        const int key = piece / (WPR / 4), w4 = (piece % (WPR / 4)) * 4;
        constexpr u32 VX = VCodec<BITS>::kStageXor;
        // V rows use an odd stride (bank spread for the column reads of the widening step)
#pragma unroll
        for (int j = 0; j < 4; ++j) vp[key * RSV + w4 + j] = vreg[i][j] ^ VX;
      }
    }
    float *par = lds_par + sl * L::kParFloats;
    const int key = tid & 63, seg = tid >> 6, vseg = NW - 1 - seg;
    // |ck| is kept away from zero so that log2(vs)/ck stays finite for a constant group
    auto ck_of = [&](float ks) {
      const float c = ks * p.scale_log2e * KCodec<BITS>::kMul;
      return __builtin_fabsf(c) < 1e-30f ? 1e-30f : c;
    };
    if (!DEQ && seg < NSK) {
      par[P_CK + seg * BN + key] = ck_of(ksc);
      u32 a0, a1, a2;
      split3_bf16(-(kzp + KCodec<BITS>::kOff) * (1.f / KCodec<BITS>::kMul), a0, a1, a2);
      u32x4_t *dst = &lds_kz[((sl * NSK + seg) * BN + key) * 2];
      dst[0] = u32x4_t{a0 | (a0 << 16), a0 | (a1 << 16), a1 | (a1 << 16), a2 | (a2 << 16)};
      if (!(FOLD_SV && seg == 0)) dst[1] = u32x4_t{0u, 0u, 0u, 0u};
    }
    if (CHAN) {
      // (the tables are in LDS already)
    } else if (DEQ) {
      // (code - zp) * vs = (raw - (zp + kOff) / kMul) * (kMul * vs) for the code image `raw` the
      // widening step produces; both factors are exact rescalings by powers of two
      if (vseg < NSV) {
        par[P_VZ + vseg * BN + key] = (vzp + VCodec<BITS>::kOff) * (1.f / VCodec<BITS>::kMul);
        par[P_SV + vseg * BN + key] = vsc * VCodec<BITS>::kMul;
      }
    } else if (vseg < NSV) {
      const int seg = vseg;
      if (FOLD_SV) {
        u32 l0, l1, l2;
        split3_bf16(__builtin_amdgcn_logf(vsc) * __builtin_amdgcn_rcpf(ck_of(ksc0)), l0, l1, l2);
        lds_kz[(sl * NSK * BN + key) * 2 + 1] = u32x4_t{l0 | (l1 << 16), l2, 0u, 0u};
      }
      // integer part of the zero-point within +-kZmax rides on the MFMA, the rest (none
      // for zero-points produced by the quantizer of ordinary data) on the fp32 remainder
      const float zc = __builtin_amdgcn_fmed3f(__builtin_rintf(vzp), -VCodec<BITS>::kZmax, VCodec<BITS>::kZmax);
      const float zr = vzp - zc;
      if (!FOLD_SV) par[P_SV + seg * BN + key] = vsc;
      par[P_VR + seg * BN + key] = zr;
      uint16_t *rows = lds_wz + sl * 8 * RSR;
      rows[seg * RSR + key] = (uint16_t)(f2u(zc + VCodec<BITS>::kOff) >> 16);
      if (seg == 0) {
        u32 i0, i1, i2;
        split3_bf16(__builtin_amdgcn_rcpf(vsc), i0, i1, i2);
        rows[4 * RSR + key] = (uint16_t)i0;
        rows[5 * RSR + key] = (uint16_t)i1;
        rows[6 * RSR + key] = (uint16_t)i2;
      }
      if (!(zr == 0.f)) lds_flag[sl] = tile + 1;   // benign race: every writer stores the same tag
    }
  };

  u32 kmask = KCodec<BITS>::kMask;
  asm volatile("" : "+v"(kmask));   // keep the mask in a vector register (see KCodec::expand)

  // row of the extra PV block this lane feeds in the MFMA of V group s (as element offset)
  int rowsel[NSVA];
#pragma unroll
  for (int s = 0; s < NSVA; ++s) rowsel[s] = ((col == s) ? s : (s == 0 && col >= 4 && col < 7) ? col : 7) * RSR;

  // CHAN: the widening of `tile` begins: (wseg, wseg_end) follow the tile's first key
  auto widen_cursor = [&](int tile) {
    if constexpr (CHAN) {
      const int t0w = tile_base + tile * BN;
      while (wseg + 1 < p.nseg && t0w >= wseg_end) {
        ++wseg;
        wseg_end = __builtin_amdgcn_readfirstlane(lds_seg_end[wseg]);
      }
    }
  };
  // CHAN: segment of a key of the tile being widened, searched upwards from the tile's first
  auto key_segment = [&](int key) {
    int sg = wseg;
    while (sg + 1 < p.nseg && key >= lds_seg_end[sg]) ++sg;
    return sg;
  };
  // CHAN: all keys of the tile being widened belong to segment wseg (wave-uniform)
  auto tile_in_one_segment = [&](int tile) { return wseg + 1 >= p.nseg || tile_base + tile * BN + BN <= wseg_end; };

  // packed V of `tile` -> V^T bf16: a work item is 2 adjacent keys x 8 channels (one
  // packed word of each key), written as 8 dwords of the transposed tile
  auto widen_v = [&](int tile) {
    const u32 *vp = lds_vp + (tile % 3) * BN * RSV;
    uint16_t *vt = lds_vt + (tile & 1) * D * VTS;
    widen_cursor(tile);
    const bool one_seg = !CHAN || tile_in_one_segment(tile);
    // (where the tile has fewer items than the workgroup has threads, the upper wavefronts take
    // them: the K pieces are widened by the lower ones)
    constexpr int V_ITEMS = (BN / 2) * (D / 8);
    constexpr int V_ROT = V_ITEMS < NT ? NT - V_ITEMS : 0;
    for (int item = tid - V_ROT; item < V_ITEMS; item += NT) {
      if (V_ROT && item < 0) continue;
      const int kp2 = item & (BN / 2 - 1), oct = item / (BN / 2);
      const u32 *row = &vp[kp2 * 2 * RSV];
      u32 pr[8];
      float f0[8], f1[8];
      if constexpr (DEQ) v_pair_values<BITS>(row, row + RSV, oct, kmask, f0, f1);
      else VCodec<BITS>::pairs(row, row + RSV, oct, kmask, pr);
      if constexpr (CHAN) {
        // code images -> values, (raw - z') * s' per channel in fp32, rounded to bf16
        int sg0 = wseg, sg1 = wseg;
        if (!one_seg) {
          const int k0 = min(tile_base + tile * BN + 2 * kp2, p.Lk - 1);
          sg0 = key_segment(k0);
          sg1 = key_segment(min(k0 + 1, p.Lk - 1));
        }
        const float *t0s = lds_tab + (sg0 * TR + 2) * D + oct * 8;
        const float4 sa = *reinterpret_cast<const float4 *>(t0s), sb = *reinterpret_cast<const float4 *>(t0s + 4);
        const float4 za = *reinterpret_cast<const float4 *>(t0s + D), zb = *reinterpret_cast<const float4 *>(t0s + D + 4);
        const float s0[8] = {sa.x, sa.y, sa.z, sa.w, sb.x, sb.y, sb.z, sb.w}, z0[8] = {za.x, za.y, za.z, za.w, zb.x, zb.y, zb.z, zb.w};
        if (one_seg || sg1 == sg0) {
#pragma unroll
          for (int j = 0; j < 8; ++j) pr[j] = pack_io_rne<F16>((f0[j] - z0[j]) * s0[j], (f1[j] - z0[j]) * s0[j]);
        } else {
          const float *t1s = lds_tab + (sg1 * TR + 2) * D + oct * 8;
#pragma unroll
          for (int j = 0; j < 8; ++j) pr[j] = pack_io_rne<F16>((f0[j] - z0[j]) * s0[j], (f1[j] - t1s[D + j]) * t1s[j]);
        }
      } else if constexpr (DEQ) {
        // code images -> values of the two keys, (raw - z') * s' in fp32, rounded to bf16
        const float *pt = lds_par + (tile % 3) * L::kParFloats + (oct * 8 / GV) * BN + kp2 * 2;
        const float2 z2 = *reinterpret_cast<const float2 *>(pt + P_VZ), s2 = *reinterpret_cast<const float2 *>(pt + P_SV);
#pragma unroll
        for (int j = 0; j < 8; ++j) pr[j] = pack_io_rne<F16>((f0[j] - z2.x) * s2.x, (f1[j] - z2.y) * s2.y);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) *reinterpret_cast<u32 *>(&vt[(oct * 8 + j) * VTS + kp2 * 2]) = pr[j];
    }
  };

  // packed K of `tile` (in kreg) -> widened bf16 rows: each piece holds OPQ octets
  // of one key, every octet becomes one 16-byte MFMA A operand
  auto widen_k = [&](int tile) {
    uint16_t *kx = lds_kx + (tile & 1) * BN * KXS;
    constexpr int OPQ = KPW * 4 / BITS;       // octets per piece
    widen_cursor(tile);
    const bool one_seg = !CHAN || tile_in_one_segment(tile);
#pragma unroll
    for (int i = 0; i < KLPT; ++i) {
      const int piece = tid + i * NT;
      if (KLPT * NT == KPIECES || piece < KPIECES) {
        const int key = piece / KPPR, oct0 = (piece % KPPR) * OPQ;
        constexpr u32 KX = KCodec<BITS>::kStageXor;
        u32 q4[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) q4[w] = w < KPW ? kreg[i][w] ^ KX : 0u;
        int sg = wseg;
        if constexpr (CHAN) {
          if (!one_seg) sg = key_segment(min(tile_base + tile * BN + key, p.Lk - 1));
        }
#pragma unroll
        for (int j = 0; j < OPQ; ++j) {
          u32 a[4];
          float f[8];
          if constexpr (DEQ) k_values<BITS>(q4, j, kmask, f);
          else KCodec<BITS>::expand(q4, j, kmask, a);
          if constexpr (CHAN) {
            // code images -> values: (raw - z') * s' per channel (rows 0 and 1 of the segment's
            // tables, in the operand's slot order), the reference's (code - zp) * scale, rounded to bf16
            const float *tk = lds_tab + sg * TR * D + (oct0 + j) * 8;
            const float4 sa = *reinterpret_cast<const float4 *>(tk), sb = *reinterpret_cast<const float4 *>(tk + 4);
            const float4 za = *reinterpret_cast<const float4 *>(tk + D), zb = *reinterpret_cast<const float4 *>(tk + D + 4);
            const float sc[8] = {sa.x, sa.y, sa.z, sa.w, sb.x, sb.y, sb.z, sb.w}, zc[8] = {za.x, za.y, za.z, za.w, zb.x, zb.y, zb.z, zb.w};
#pragma unroll
            for (int m = 0; m < 4; ++m)
              a[m] = pack_io_rne<F16>((f[2 * m] - zc[2 * m]) * sc[2 * m], (f[2 * m + 1] - zc[2 * m + 1]) * sc[2 * m + 1]);
          } else if constexpr (DEQ) {
            // code images -> values: (raw - (zp + kOff) / kMul) * (kMul * ks), the reference's
            // (code - zp) * scale with both factors rescaled exactly, rounded to bf16
            const int gl = (j * 8) / GK < GPP ? (j * 8) / GK : GPP - 1;   // group of octet j inside the piece
            const float zk = (kgz[i * GPP + gl] + KCodec<BITS>::kOff) * (1.f / KCodec<BITS>::kMul);
            const float sk = kgs[i * GPP + gl] * KCodec<BITS>::kMul;
#pragma unroll
            for (int m = 0; m < 4; ++m) a[m] = pack_io_rne<F16>((f[2 * m] - zk) * sk, (f[2 * m + 1] - zk) * sk);
          }
          *reinterpret_cast<u32x4_t *>(&kx[key * KXS + (oct0 + j) * 8]) = u32x4_t{a[0], a[1], a[2], a[3]};
        }
      }
    }
  };

  // ---- prologue: V tiles 0 and 1 staged, K and V of tile 0 widened, K of tile 1 and V
  //      of tile 2 in registers ------------------------------------------------------------
  if (tid < 3) lds_flag[tid] = 0;
  for (int i = tid; i < 3 * RSR; i += NT) lds_wz[((i / RSR) * 8 + 7) * RSR + i % RSR] = 0;   // the all-zero row of each slot
  if (n_tiles > 0) { prefetch_k(0); prefetch(0); }
  // the query values, behind the first tile's requests and ahead of the table loads: one
  // round trip for all three
#pragma unroll
  for (int ch = 0; ch < NCH; ++ch) qb[ch] = *reinterpret_cast<const u32x4_t *>(qptr + k_octet<GK>(ch, half) * 8);
  if constexpr (CHAN) {
    // the head's tables, as the widening steps use them (see lds_tab above)
    for (int i = tid; i < p.nseg * TR * D; i += NT) {
      const int seg = i / (TR * D), which = (i / D) % TR, d = i % D;
      const bool is_k = which < 2, is_zp = which & 1;
      const float *src = which == 0 ? p.k_chan_scale : which == 1 ? p.k_chan_zp : which == 2 ? p.v_chan_scale : p.v_chan_zp;
      const int c = is_k ? (d & ~7) + KCodec<BITS>::slot_d(d & 7) : d;   // K rows: the operand's slot order inside an octet
      const float x = src ? src[((int64_t)seg * p.Hkv + hs) * D + c] : 0.f;
      const float mul = is_k ? KCodec<BITS>::kMul : VCodec<BITS>::kMul, off = is_k ? KCodec<BITS>::kOff : VCodec<BITS>::kOff;
      lds_tab[i] = is_zp ? (x + off) * (1.f / mul) : x * mul;
    }
  }
  __syncthreads();
  if constexpr (CHAN) {
    if (p.nseg > 1) {
      // the segment of this workgroup's first key (a share of the keys may begin mid-cache)
      wseg_end = __builtin_amdgcn_readfirstlane(lds_seg_end[0]);
      widen_cursor(0);
    }
  }
  load_q();
  if (n_tiles > 0) { stage(0); widen_k(0); }
  if (n_tiles > 1) { prefetch_k(1); prefetch(1); stage(1); }
  __syncthreads();
  if (n_tiles > 0) widen_v(0);
  if (n_tiles > 2) prefetch(2);
  __syncthreads();

  if (!wave_live) {
    // a wavefront without queries (short query blocks) only helps with staging and
    // widening, at the same barrier count as the others
    for (int tile = 0; tile < n_tiles; ++tile) {
      if (tile + 2 < n_tiles) stage(tile + 2);
      if (tile + 3 < n_tiles) prefetch(tile + 3);
      if (tile + 1 < n_tiles) { widen_v(tile + 1); widen_k(tile + 1); }
      if (tile + 2 < n_tiles) prefetch_k(tile + 2);
      __syncthreads();
    }
    return;
  }

  // ---- the three phases of one 32-key block, as lambdas over per-tile state --------
  // LDS operands are requested ahead of their use where the registers allow it (the
  // scheduling fences keep the requests where they are written).
  constexpr bool HOIST = (NSKA == 1 && NSVA == 1);
  int t0 = 0;
  const uint16_t *kx = nullptr, *vt = nullptr, *wz = nullptr;
  const float *par = nullptr;
  const u32x4_t *kz = nullptr;
  bool tile_rem = false, first = true;
  // register i of this lane <-> key kb*32 + 16*(i/8) + 8*half + i%8 of the tile
  floatx16_t sacc[2][NSKA];
  u32 pop[2][NSVA][2][4];          // P'^T operands: p * vs as bf16, [block][V group][16-key chunk][dword]
  float ckv[2][NSKA][16], svv[2][NSVA][16];
  u32x4_t vta[NDB], wza[NSVA];

  auto begin_tile = [&](int tile) {
    t0 = tile_base + tile * BN;
    kx = lds_kx + (tile & 1) * BN * KXS;
    par = lds_par + (tile % 3) * L::kParFloats;
    vt = lds_vt + (tile & 1) * D * VTS;
    kz = lds_kz + (tile % 3) * NSK * BN * 2;
    wz = lds_wz + (tile % 3) * 8 * RSR;
    tile_rem = lds_flag[tile % 3] == tile + 1;   // tagged with the tile, so stale tags never match
    // slot (tile+2)%3 was last read during tile-1 (before the barrier): refill it
    if (tile + 2 < n_tiles) stage(tile + 2);
    if (tile + 3 < n_tiles) prefetch(tile + 3);
  };
  // with the PV MFMAs of a block in flight: widen the next tile's K and V into the other slots
  auto widen_next = [&](int tile) {
    if (tile + 1 < n_tiles) {
      widen_v(tile + 1);
      widen_k(tile + 1);
      if (tile + 2 < n_tiles) prefetch_k(tile + 2);
    }
  };
  auto load_scales = [&](int kb) {
#pragma unroll
    for (int s = 0; s < ((HOIST && !DEQ) ? NSK : 0); ++s)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int key = kb * 32 + 16 * (i4 >> 1) + 8 * half + 4 * (i4 & 1);
        const float4 t = *reinterpret_cast<const float4 *>(&par[P_CK + s * BN + key]);
        ckv[kb][s][4 * i4] = t.x; ckv[kb][s][4 * i4 + 1] = t.y; ckv[kb][s][4 * i4 + 2] = t.z; ckv[kb][s][4 * i4 + 3] = t.w;
      }
#pragma unroll
    for (int s = 0; s < ((HOIST && !FOLD_SV && !DEQ) ? NSV : 0); ++s)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int key = kb * 32 + 16 * (i4 >> 1) + 8 * half + 4 * (i4 & 1);
        const float4 t = *reinterpret_cast<const float4 *>(&par[P_SV + s * BN + key]);
        svv[kb][s][4 * i4] = t.x; svv[kb][s][4 * i4 + 1] = t.y; svv[kb][s][4 * i4 + 2] = t.z; svv[kb][s][4 * i4 + 3] = t.w;
      }
  };
  auto load_v_operands = [&](int kb, int c) {
#pragma unroll
    for (int d = 0; d < NDB; ++d)
      vta[d] = *reinterpret_cast<const u32x4_t *>(&vt[(d * 32 + col) * VTS + (kb * 2 + c) * 16 + half * 8]);
#pragma unroll
    for (int s = 0; s < (DEQ ? 0 : NSV); ++s)
      wza[s] = *reinterpret_cast<const u32x4_t *>(&wz[rowsel[s] + (kb * 2 + c) * 16 + half * 8]);
  };

  // A wavefront raises its priority while it issues the MFMAs of a phase.  Measured per kernel
  // (same run, bit-identical results): at D=128 that is worth 5 % for 4-bit codes (0.725 against
  // 0.762 ms at the configuration-4 shape) and costs 1-3.5 % for 2-bit and 8-bit codes, whose
  // widening has more to do beside the MFMAs; at D=64 it makes no difference.
  constexpr bool MFMA_PRIO = !(D == 128 && BITS != 4);
  // S^T = K Q^T for one 32-key block; the A operands are the widened K rows in LDS
  auto qk = [&](int kb) {
    if constexpr (MFMA_PRIO) __builtin_amdgcn_s_setprio(1);
    const int krow_i = kb * 32 + kperm(col);
#pragma unroll
    for (int s = 0; s < NSKA; ++s) {
      floatx16_t zero;
#pragma unroll
      for (int j = 0; j < 16; ++j) zero[j] = 0.f;
      if constexpr (DEQ) {
        sacc[kb][s] = zero;   // (dequantized operands: no zero-point term)
      } else {
        // starts the accumulator with the zero-point term (see bq above)
        sacc[kb][s] = mfma_32x32x16<F16>(kz[(s * BN + krow_i) * 2 + half], bq[s], zero);
      }
    }
    const uint16_t *krow = &kx[krow_i * KXS];
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
      const u32x4_t av = *reinterpret_cast<const u32x4_t *>(&krow[k_octet<GK>(ch, half) * 8]);
      constexpr int kAcc = DEQ ? 0 : 1;
      sacc[kb][kAcc * (ch / (GK / 16))] = mfma_32x32x16<F16>(av, qb[ch], sacc[kb][kAcc * (ch / (GK / 16))]);
    }
    if constexpr (MFMA_PRIO) __builtin_amdgcn_s_setprio(0);
  };

  // logits -> P'^T operands of one block: online softmax against a lazily moved reference
  auto softmax = [&](int kb) {
    float z[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float v = -m_ref;
#pragma unroll
      for (int s = 0; s < NSKA; ++s) {
        const int key = kb * 32 + 16 * (i >> 3) + 8 * half + (i & 7);
        v = __builtin_fmaf(DEQ ? p.scale_log2e : HOIST ? ckv[kb][s][i] : par[P_CK + s * BN + key],
                           sacc[kb][s][i], v);
      }
      z[i] = v;
    }
    // mask: block-causal key limit and the ragged last tile
    const int lim_t = limit;
    if (t0 + BN > wave_minlim) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = t0 + kb * 32 + 16 * (i >> 3) + 8 * half + (i & 7);
        if (key >= lim_t) z[i] = -INFINITY;
      }
    }
    // Moves the softmax reference to the row's current maximum: up only (never down) once
    // something has been accumulated; the very first block takes its maximum as it is, negative
    // or not (the accumulators are still zero, so alpha = 1 is exact).
    auto move_reference = [&]() {
      float zmax = z[0];
#pragma unroll
      for (int i = 1; i < 16; ++i) zmax = fmaxf(zmax, z[i]);
      {
        // the other lane half of the same query, without a trip through LDS
        const auto sw = __builtin_amdgcn_permlane32_swap(f2u(zmax), f2u(zmax), false, false);
        zmax = fmaxf(u2f(sw[0]), u2f(sw[1]));
      }
      // exact codes: the reference goes kHeadroom octaves above the maximum (see below)
      constexpr float up = DEQ ? 0.f : kHeadroom;
      const float delta = first ? ((zmax == -INFINITY) ? 0.f : zmax + up) : fmaxf(zmax + up, 0.f);
      const float alpha = first ? 1.f : __builtin_amdgcn_exp2f(-delta);
      m_ref += delta;
#pragma unroll
      for (int i = 0; i < 16; ++i) z[i] -= delta;
#pragma unroll
      for (int d = 0; d < NDB; ++d)
#pragma unroll
        for (int j = 0; j < 16; ++j) oacc[d][j] *= alpha;
#pragma unroll
      for (int j = 0; j < (DEQ ? 0 : 16); ++j) racc[j] *= alpha;
      if constexpr (DEQ) l_part *= alpha;
#pragma unroll
      for (int s = 0; s < NSVA; ++s) r_run[s] *= alpha;
    };
    // exp2 of the logits, rounded to bf16 pairs for the MFMA; DEQ: also their sum (this lane's keys)
    float blk = 0.f;
    auto weights = [&]() {
      float pv[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) pv[i] = __builtin_amdgcn_exp2f(z[i]);
      blk = 0.f;
#pragma unroll
      for (int s = 0; s < NSVA; ++s)
#pragma unroll
        for (int i2 = 0; i2 < 8; ++i2) {
          const int i = 2 * i2;
          const int key = kb * 32 + 16 * (i >> 3) + 8 * half + (i & 7);
          if constexpr (FOLD_SV || DEQ) pop[kb][s][i >> 3][(i & 7) >> 1] = pack_io_rne<F16>(pv[i], pv[i + 1]);
          else if constexpr (HOIST)
            pop[kb][s][i >> 3][(i & 7) >> 1] = pack_bf16_rne(pv[i] * svv[kb][s][i], pv[i + 1] * svv[kb][s][i + 1]);
          else
            pop[kb][s][i >> 3][(i & 7) >> 1] =
                pack_bf16_rne(pv[i] * par[P_SV + s * BN + key], pv[i + 1] * par[P_SV + s * BN + key + 1]);
          if constexpr (DEQ) {   // += the two rounded weights (one v_dot2 against a pair of ones)
            if constexpr (F16) {
              typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
              blk = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, pop[kb][s][i >> 3][(i & 7) >> 1]),
                                           __builtin_bit_cast(f16x2_t, 0x3c003c00u), blk, false);
            } else {
              typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
              blk = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pop[kb][s][i >> 3][(i & 7) >> 1]),
                                                    __builtin_bit_cast(bf16x2_t, 0x3f803f80u), blk, false);
            }
          }
        }
    };
    if constexpr (DEQ) {
      // The reference has to move when a logit exceeds it by 2^16.  Rather than look for the
      // row maximum in every block (eleven instructions of sixty), the weights are computed
      // against the reference as it stands and their sum is looked at, which the denominator
      // needs anyway: a weight above 2^16 (or an overflow to infinity) shows in it, and the block
      // is then redone with the reference moved.  (A sum above 2^16 without such a weight moves
      // the reference too, which is harmless.)
      if (first) move_reference();
      weights();
      // (fp16 weights end at 65504: there the reference moves at a block sum of 2^15, which keeps
      // every weight of an accepted block finite; an overflowed one makes the sum infinite)
      constexpr float kMoveAt = F16 ? 32768.f : 65536.f;
      if (!first && __any(!(blk <= kMoveAt))) {
        move_reference();
        weights();
      }
      l_part += blk;
      first = false;
    } else {
      // Here the denominator is summed by the MFMA, so there is no sum to look at; the packed
      // weights themselves are: all are >= 0, so bit 14 of a bf16 (the top exponent bit) says
      // "this weight is 2 or more" (infinities included), and an OR over the block's eight words
      // finds one.  The reference is put kHeadroom octaves above the maximum when it moves, so
      // weights start at 2^-kHeadroom or below -- bf16 and the fp32 sums keep their relative
      // precision there -- and it moves again only for a logit 1 + kHeadroom octaves above that
      // maximum.
      if (first) move_reference();
      weights();
      if (!first) {
        u32 any_w = 0;
#pragma unroll
        for (int s = 0; s < NSVA; ++s)
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < 4; ++j) any_w |= pop[kb][s][h][j];
        if (__any((any_w & 0x40004000u) != 0)) {
          move_reference();
          weights();
        }
      }
      first = false;
    }
    if (!DEQ && tile_rem) {
      // the remainder term must see the same bf16-rounded weights as the MFMA
#pragma unroll
      for (int s = 0; s < NSVA; ++s)
#pragma unroll
        for (int i2 = 0; i2 < 8; ++i2) {
          const int i = 2 * i2;
          const int key = kb * 32 + 16 * (i >> 3) + 8 * half + (i & 7);
          const u32 pk = pop[kb][s][i >> 3][(i & 7) >> 1];
          r_run[s] = __builtin_fmaf(u2f(pk << 16), par[P_VR + s * BN + key], r_run[s]);
          r_run[s] = __builtin_fmaf(u2f(pk & 0xffff0000u), par[P_VR + s * BN + key + 1], r_run[s]);
        }
    }
  };

  // O^T += V^T P'^T for the 32 keys of one block; one more MFMA per chunk and V group
  // feeds the extra block: its row s collects the zero-point sum of group s and rows
  // 4..6 (group 0 only) the softmax denominator
  auto pv_mfma = [&](int kb, bool preloaded) {
    if constexpr (MFMA_PRIO) __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      u32x4_t av[NDB], aw[NSVA];
      if (!(preloaded && c == 0) && !(HOIST && c == 1)) load_v_operands(kb, c);
#pragma unroll
      for (int d = 0; d < NDB; ++d) av[d] = vta[d];
#pragma unroll
      for (int s = 0; s < (DEQ ? 0 : NSVA); ++s) aw[s] = wza[s];
      if (HOIST && c == 0) {
        load_v_operands(kb, 1);   // in flight under this chunk's MFMAs
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int d = 0; d < NDB; ++d) {
        constexpr int DBS = GV / 32;  // 32-row blocks per V scale group
        const int s = DEQ ? 0 : d / DBS;
        u32x4_t bv = {pop[kb][s][c][0], pop[kb][s][c][1], pop[kb][s][c][2], pop[kb][s][c][3]};
        oacc[d] = mfma_32x32x16<F16>(av[d], bv, oacc[d]);
      }
#pragma unroll
      for (int s = 0; s < (DEQ ? 0 : NSVA); ++s) {
        u32x4_t bv = {pop[kb][s][c][0], pop[kb][s][c][1], pop[kb][s][c][2], pop[kb][s][c][3]};
        racc = mfma_32x32x16<F16>(aw[s], bv, racc);
      }
    }
    if constexpr (MFMA_PRIO) __builtin_amdgcn_s_setprio(0);
  };

  for (int tile = 0; tile < n_tiles; ++tile) {
    begin_tile(tile);
    // a tile with at most 32 keys (the end of the cache) has nothing for the second key
    // block: every weight there would be exp2(-inf) = 0
    const bool half_tile = kv_end - t0 <= 32;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      if (kb == 1 && half_tile) continue;
      load_scales(kb);
      qk(kb);
      if constexpr (HOIST) {
        load_v_operands(kb, 0);   // used after the softmax arithmetic
        __builtin_amdgcn_sched_barrier(0);
      }
      softmax(kb);
      pv_mfma(kb, HOIST);
      if (kb == 0) widen_next(tile);
    }
    __syncthreads();   // the one barrier per tile
  }

  // ---- epilogue -------------------------------------------------------------------
#pragma unroll
  for (int s = 0; s < NSVA; ++s) r_run[s] += __shfl_xor(r_run[s], 32, 64);
  // rows 4..6 of racc are registers 0..2 of the upper lane half, rows 0..3 registers 0..3 of the lower
  // (DEQ: the denominator is row 0, the sum of the weights against the row of ones)
  const float l_sum = DEQ ? l_part + __shfl_xor(l_part, 32, 64) : __shfl(racc[0] + racc[1] + racc[2], col + 32, 64);
  const float inv = l_sum > 0.f ? 1.0f / l_sum : 0.f;
  float rq[NSVA];
#pragma unroll
  for (int s = 0; s < NSVA; ++s) rq[s] = DEQ ? 0.f : __shfl(racc[s], col, 64) + r_run[s];
  if (q_live) {
    __bf16 *optr = p.out + (b * p.o_bs + hq * p.o_hs + qrow * p.o_ts) * D;
    // with the keys shared out: the normalized fp32 output and (reference, denominator) of
    // this share, for the combining kernel
    const bool shared_out = p.nsplit > 1;
    const int64_t prow = ((int64_t)split * p.bh_total + bh) * p.Lq + qrow;
    float *wptr = p.ws_o + prow * D;
    if (shared_out && half == 0) *reinterpret_cast<float2 *>(p.ws_ml + prow * 2) = make_float2(m_ref, l_sum);
#pragma unroll
    for (int d = 0; d < NDB; ++d) {
      constexpr int DBS = GV / 32;
      const float r = rq[DEQ ? 0 : d / DBS];
      constexpr float VM = DEQ ? 1.f : VCodec<BITS>::kMul;   // (DEQ: the accumulators hold values already)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        // registers 4*g4 .. 4*g4+3 are rows d*32 + 8*g4 + 4*half + 0..3 of O^T
        float o0 = (VM * oacc[d][4 * g4 + 0] - r) * inv, o1 = (VM * oacc[d][4 * g4 + 1] - r) * inv;
        float o2 = (VM * oacc[d][4 * g4 + 2] - r) * inv, o3 = (VM * oacc[d][4 * g4 + 3] - r) * inv;
        if (shared_out) {
          *reinterpret_cast<float4 *>(wptr + d * 32 + 8 * g4 + 4 * half) = make_float4(o0, o1, o2, o3);
        } else {
          uint2 v = make_uint2(pack_io_rne<F16>(o0, o1), pack_io_rne<F16>(o2, o3));
          *reinterpret_cast<uint2 *>(optr + d * 32 + 8 * g4 + 4 * half) = v;
        }
      }
    }
  }
}

// The shares' outputs weighted by their softmax mass l * 2^(m - M), M the largest reference among
// the shares that saw a key.  A workgroup of 256 threads serves 2 query rows x (D/4) channel quads
// x G groups of shares (G = 4 at D=128, 8 at D=64: the threads of a quad split the shares among
// them): the weights of a row's shares are formed once, in LDS, and every thread then sums its
// shares' quads with nothing between the loads but the weights.
template <int D, bool F16>
__global__ __launch_bounds__(256) void combine_splits_kernel(AttnParams p) {
  constexpr int QUADS = D / 4, ROWS = 2, G = 256 / (ROWS * QUADS);
  constexpr int kMaxS = 64;
  static_assert(G >= 1 && kMaxS >= kMaxKeyShares_v && kMaxS >= kMaxSplits_v, "share counts");
  __shared__ float w_lds[ROWS][kMaxS];
  const int64_t rows = (int64_t)p.bh_total * p.Lq;
  const int tid = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.x * ROWS;
  // weights of the rows' shares
  __shared__ float2 ml_lds[ROWS][kMaxS];
  static_assert(ROWS * kMaxS <= 256, "one (row, share) per thread");
  const int wr = tid / kMaxS, wsh = tid % kMaxS;
  if (tid < ROWS * kMaxS) {
    float2 ml = make_float2(0.f, 0.f);   // (denominator 0: an empty share)
    if (wsh < p.nsplit && row0 + wr < rows) ml = *reinterpret_cast<const float2 *>(p.ws_ml + ((int64_t)wsh * rows + row0 + wr) * 2);
    ml_lds[wr][wsh] = ml;
  }
  __syncthreads();
  if (tid < ROWS * kMaxS) {
    float m_max = -INFINITY;
    for (int t = 0; t < p.nsplit; ++t)
      if (ml_lds[wr][t].y > 0.f) m_max = fmaxf(m_max, ml_lds[wr][t].x);
    const float2 ml = ml_lds[wr][wsh];
    w_lds[wr][wsh] = ml.y > 0.f ? ml.y * __builtin_amdgcn_exp2f(ml.x - m_max) : 0.f;
  }
  __syncthreads();
  const int r = tid / (QUADS * G), gq = tid % (QUADS * G), grp = gq / QUADS, c0 = (gq % QUADS) * 4;
  const int64_t row = row0 + r;
  float acc[4] = {0.f, 0.f, 0.f, 0.f}, wsum = 0.f;
  if (row < rows) {
#pragma unroll 4
    for (int s_ = grp; s_ < p.nsplit; s_ += G) {
      const float w = w_lds[r][s_];
      const float4 o = *reinterpret_cast<const float4 *>(p.ws_o + ((int64_t)s_ * rows + row) * D + c0);
      acc[0] = __builtin_fmaf(w, o.x, acc[0]); acc[1] = __builtin_fmaf(w, o.y, acc[1]);
      acc[2] = __builtin_fmaf(w, o.z, acc[2]); acc[3] = __builtin_fmaf(w, o.w, acc[3]);
      wsum += w;
    }
  }
  if constexpr (G > 1) {
    // the groups of a row's shares meet through LDS (group 0 collects)
    __shared__ float part[256][5];
    part[tid][0] = acc[0]; part[tid][1] = acc[1]; part[tid][2] = acc[2]; part[tid][3] = acc[3]; part[tid][4] = wsum;
    __syncthreads();
    if (grp != 0) return;
#pragma unroll
    for (int g2 = 1; g2 < G; ++g2) {
      const float *o = part[tid + g2 * QUADS];
      acc[0] += o[0]; acc[1] += o[1]; acc[2] += o[2]; acc[3] += o[3]; wsum += o[4];
    }
  }
  if (row >= rows) return;
  const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
  const int bh = (int)(row / p.Lq), qrow = (int)(row % p.Lq);
  const int b = bh / p.Hkv, hs = bh % p.Hkv;
  const int hq = p.head_map ? p.head_map[hs] : hs;
  __bf16 *optr = p.out + (b * p.o_bs + hq * p.o_hs + qrow * p.o_ts) * D + c0;
  *reinterpret_cast<uint2 *>(optr) = make_uint2(pack_io_rne<F16>(acc[0] * inv, acc[1] * inv), pack_io_rne<F16>(acc[2] * inv, acc[3] * inv));
}

int device_cus();

template <int D, int BITS, int GK, int GV, bool CHAN, int NWV, int WPS = 2, bool EXACT = false, bool F16 = false>
void launch_shape(const AttnParams &p, hipStream_t st) {
  // (the per-channel tables take LDS by the number of segments of the launch)
  constexpr int lds_base = (AttnLds<D, BITS, GK, GV, CHAN, EXACT>::kBytes + 15) / 16 * 16, lds_seg = CHAN ? kChanTableRows * D * 4 : 0;
  constexpr int lds_max = lds_base + kMaxSegments * lds_seg;
  static_assert(lds_max <= 160 * 1024, "LDS budget");
  const int lds_bytes = lds_base + p.nseg * lds_seg;
  // above 64 KiB the limit has to be raised, once per device the process launches on
  static bool configured[64] = {false};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
  if (dev < 0 || !configured[dev]) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&fused_attn_kernel<D, BITS, GK, GV, CHAN, NWV, WPS, EXACT, F16>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, lds_max);
    if (dev >= 0) configured[dev] = true;
  }
  const int bh_pad = (p.bh_total + 7) / 8 * 8;
  dim3 grid((unsigned)(bh_pad * p.q_tiles * p.nsplit));
  hipLaunchKernelGGL((fused_attn_kernel<D, BITS, GK, GV, CHAN, NWV, WPS, EXACT, F16>), grid, dim3(NWV * 64), lds_bytes, st, p);
  if (p.nsplit > 1) {
    const int64_t rows = (int64_t)p.bh_total * p.Lq;
    hipLaunchKernelGGL((combine_splits_kernel<D, F16>), dim3((unsigned)((rows + 1) / 2)), dim3(256), 0, st, p);
  }
}

template <int D, int BITS, int GK, int GV, bool CHAN = false>
void launch(const AttnParams &p, hipStream_t st) {
  if constexpr (D == 64) {
    // fp16 operands (the VAR path; every VAR model has head dim 64)
    if (p.f16) {
      if (p.Lq <= 128 && p.bh_total > device_cus()) launch_shape<D, BITS, GK, GV, CHAN, 4, 2, false, true>(p, st);
      else launch_shape<D, BITS, GK, GV, CHAN, 8, 4, false, true>(p, st);
      return;
    }
  }
  if constexpr (D == 64) {
    // more (batch, head) pairs than compute units, at most four wavefronts of queries each:
    // workgroups of four wavefronts (same arithmetic, same results).  Also for one or two
    // wavefronts of queries: the wavefronts without queries share the staging and the widening
    // of the tiles, which is what such a workgroup spends its time on (workgroups of two
    // wavefronts, also two to a compute unit by their LDS, took 20-35 % longer on 16-64 queries).
    if (p.Lq <= 128 && p.bh_total > device_cus()) {
      launch_shape<D, BITS, GK, GV, CHAN, 4>(p, st);
      return;
    }
  }
  if constexpr (D == 64) {
    // The kernels at D=64 fit 128 registers at the price of 24-48 bytes of spills,
    // and two resident workgroups per compute unit hide each other's prologue and barriers
    // (8-15 % faster than one workgroup at 140 registers).
    launch_shape<D, BITS, GK, GV, CHAN, 8, 4>(p, st);
  } else {
    if constexpr (AttnForms<D, BITS, GK, GV, CHAN>::kHasExact) {
      if (p.exact_codes) {
        launch_shape<D, BITS, GK, GV, CHAN, 8, 2, true>(p, st);
        return;
      }
    }
    launch_shape<D, BITS, GK, GV, CHAN, 8>(p, st);
  }
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

int set_layout(AttnParams &p, int layout, const char *who) {
  if (layout == VARQ_LAYOUT_BHLC || layout == VARQ_LAYOUT_BHLC_OUT_BLHC) {
    p.q_bs = (int64_t)p.Hq * p.Lq; p.q_hs = p.Lq; p.q_ts = 1;
    p.kv_bs = (int64_t)p.Hkv * p.Lstride; p.kv_hs = p.Lstride; p.kv_ts = 1;
  } else if (layout == VARQ_LAYOUT_BLHC) {
    p.q_bs = (int64_t)p.Lq * p.Hq; p.q_hs = 1; p.q_ts = p.Hq;
    p.kv_bs = (int64_t)p.Lstride * p.Hkv; p.kv_hs = 1; p.kv_ts = p.Hkv;
  } else {
    return varq_set_error(VARQ_ERR_INVALID, "%s: layout must be VARQ_LAYOUT_BHLC (0), VARQ_LAYOUT_BLHC (1) or VARQ_LAYOUT_BHLC_OUT_BLHC (2), got %d", who, layout);
  }
  p.o_bs = p.q_bs; p.o_hs = p.q_hs; p.o_ts = p.q_ts;
  if (layout == VARQ_LAYOUT_BHLC_OUT_BLHC) { p.o_bs = (int64_t)p.Lq * p.Hq; p.o_hs = 1; p.o_ts = p.Hq; }
  return VARQ_OK;
}

// ---- sharing the keys of a query block out over several workgroups ---------------------
constexpr int kMaxSplits = kMaxSplits_v;

int device_cus() {
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (!cus[dev]) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev] = n;
  }
  return cus[dev];
}

size_t split_workspace_bytes(int splits, int64_t rows, int D) {
  return splits > 1 ? (size_t)splits * (size_t)rows * (size_t)(D + 2) * sizeof(float) : 0;
}

// The split count that minimizes a launch's modelled time: workgroups run one per compute
// unit in rounds; a workgroup costs its tiles plus a fixed prologue and epilogue; shares
// cost a second pass over fp32 partial outputs.  Few query blocks on a long cache gain,
// a grid that already fills the device in whole rounds does not.
int choose_splits(int64_t wgs, int tiles, int64_t rows, int D) {
  const double cus = device_cus();
  const double tile_us = D == 128 ? 2.3 : 1.4, fixed_us = 9.0;
  double base = 0.0, best = 0.0;
  int best_s = 1;
  for (int s = 1; s <= kMaxSplits; ++s) {
    if (s > 1 && tiles / s < 2) break;
    const double rounds = (double)((wgs * s + (int64_t)cus - 1) / (int64_t)cus);
    double t = rounds * ((double)((tiles + s - 1) / s) * tile_us + fixed_us);
    if (s > 1) t += 4.0 + 2.0 * (double)split_workspace_bytes(s, rows, D) / 4.0e6;   // 4 TB/s, in us
    if (s == 1) base = best = t;
    else if (t < 0.9 * base && t < best) { best = t; best_s = s; }   // sharing must gain a tenth
  }
  return best_s;
}

// Fills the split fields of p from the caller's request.  splits: 0 = as the model above
// says, reduced to what the workspace holds; 1 = none; 2..8 = exactly that many.
int set_splits(AttnParams &p, int D, int tiles, int splits, void *workspace, size_t workspace_bytes, const char *who) {
  p.nsplit = 1; p.ws_o = nullptr; p.ws_ml = nullptr;
  if (splits < 0 || splits > kMaxSplits)
    return varq_set_error(VARQ_ERR_INVALID, "%s: splits must be 0 (automatic) or 1..%d (got %d)", who, kMaxSplits, splits);
  const int64_t rows = (int64_t)p.bh_total * p.Lq;
  int n = splits ? splits : choose_splits((int64_t)p.bh_total * p.q_tiles, tiles, rows, D);
  if (splits > 1 && (!workspace || workspace_bytes < split_workspace_bytes(n, rows, D)))
    return varq_set_error(VARQ_ERR_INVALID, "%s: %d splits need a workspace of %zu bytes (got %zu)", who, n,
                          split_workspace_bytes(n, rows, D), workspace ? workspace_bytes : (size_t)0);
  while (n > 1 && (!workspace || workspace_bytes < split_workspace_bytes(n, rows, D))) --n;
  if (n <= 1) return VARQ_OK;
  if ((uintptr_t)workspace & 15) return varq_set_error(VARQ_ERR_INVALID, "%s: the workspace must be 16-byte aligned", who);
  if ((int64_t)((p.bh_total + 7) / 8 * 8) * p.q_tiles * n >= (1ll << 31))
    return varq_set_error(VARQ_ERR_INVALID, "%s: grid too large for %d splits", who, n);
  p.nsplit = n;
  p.ws_o = reinterpret_cast<float *>(workspace);
  p.ws_ml = p.ws_o + (size_t)n * (size_t)rows * (size_t)D;
  return VARQ_OK;
}


// ---- few queries over a long cache (the regime bound by the reads of the packed cache) -----------
// With at most a few dozen queries per (batch, head) the arithmetic intensity of the attention,
// 32 * Lq / (bits_K + bits_V) flop per packed byte, is below the machine balance: the kernel above,
// built around 256 queries per workgroup, leaves seven of its eight wavefronts without queries and
// spends a workgroup barrier per 64 keys on the remaining one.  This kernel turns the work round:
// all wavefronts of a workgroup serve the SAME 32 queries and each takes its own 32-key blocks of
// the workgroup's share of the keys, from global memory straight to registers, with nothing shared
// between wavefronts inside the key loop and no workgroup barrier in it:
//  * K: a lane loads half a key row (the half its MFMA A operands come from), dequantizes it in
//    registers -- (code - zp) * scale in fp32, rounded to bf16, the operands the reference's
//    attention sees -- and feeds S^T = K Q^T directly; the Q^T operands sit in LDS, written once;
//  * V: a lane widens items of two adjacent keys x 8 channels into a wavefront-private V^T tile
//    in LDS (the second contraction runs over keys), read back as MFMA A operands by the same
//    wavefront -- LDS requests of one wavefront are served in order, so no barrier is needed;
//  * online softmax per lane against a reference that moves only when a weight would pass 2^16;
//  * a block runs S^T, then the V^T tile (under the S^T MFMAs), then the softmax, then O^T; the
//    wavefront's next block is requested piece by piece as the current one frees its registers
//    (K after S^T, V after the tile), each about a block's time ahead of its use.
// The wavefronts' partial results are merged through LDS (each wavefront ends up with a quarter
// of the channels), the workgroups' shares through the workspace and combine_splits_kernel, as
// for the kernel above.
// One scale group per key (group = D = 128), bf16, any layout, key limits, head maps.
constexpr int FQ_NW = 4;             // wavefronts per workgroup
constexpr int FQ_BK = 32;            // keys per block: one 32-row MFMA block
constexpr int FQ_VTS = FQ_BK + 8;    // V^T row stride (bf16): 16-byte rows, bank spread
constexpr int FQ_D = 128;
constexpr int kFewQueries = 64;      // launches with at most this many queries per (batch, head) ...
constexpr int kFewQMinKeys = 1024;   // ... over at least this many keys take this kernel
constexpr int kMaxKeyShares = kMaxKeyShares_v;
struct FewQLds {
  static constexpr int kVt = 0;                                        // [FQ_NW][D][FQ_VTS] bf16
  // the merge slots -- for every wavefront, a quarter of each other wavefront's accumulators --
  // start at the V^T tiles and need a little more
  static constexpr int kSlotBytes = FQ_NW * (FQ_NW - 1) * 16 * 64 * 4;
  static constexpr int kMl = kVt + (FQ_NW * FQ_D * FQ_VTS * 2 > kSlotBytes ? FQ_NW * FQ_D * FQ_VTS * 2 : kSlotBytes);   // [FQ_NW][32][2] fp32 (merge)
  static constexpr int kBytes = kMl + FQ_NW * 32 * 2 * 4;
};

template <int BITS>
__global__ __launch_bounds__(FQ_NW * 64, 2) void fused_attn_fewq_kernel(AttnParams p) {
  constexpr int D = FQ_D, WPR = D * BITS / 32, NCH = D / 16, NDB = D / 32;
  constexpr int HW = WPR / 2;                 // packed words of half a key row
  constexpr int KP = HW / 4;                  // 16-byte pieces of it
  constexpr int OPQ = 16 / BITS;              // octets per piece
  constexpr int UPR = BITS == 2 ? 8 : 16;     // V units per key row: a word, or the two words of an octet of bytes
  constexpr int WPU = BITS == 8 ? 2 : 1;      // words per unit
  constexpr int OPU = BITS == 2 ? 2 : 1;      // octets per unit
  constexpr int IPL = 16 * UPR / 64;          // V items (two keys x one unit) per lane and block
  static_assert(NDB == FQ_NW, "the merge gives every wavefront one 32-channel block of the output");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, half = lane >> 5;
  uint16_t *const vt = reinterpret_cast<uint16_t *>(lds_raw + FewQLds::kVt) + wave * D * FQ_VTS;
  float *const lds_ml = reinterpret_cast<float *>(lds_raw + FewQLds::kMl);

  // workgroup -> (batch * head, query tile, share) without a division: the grid is (8, shares,
  // groups of eight (batch, head) x query tiles); x runs fastest in the dispatch order, so the
  // workgroups of one (batch, head) sit on one XCD (one L2), as in the kernel above.
  static_assert(kFewQueries <= 64, "at most two query tiles");
  const int xcd = blockIdx.x, split = blockIdx.y, slot = blockIdx.z;
  const int qt = p.q_tiles == 2 ? (slot & 1) : 0;
  const int grp = p.q_tiles == 2 ? (slot >> 1) : slot;
  const int bh = p.kv_hs == 1 && p.kv_ts > 1 ? xcd * ((p.bh_total + 7) >> 3) + grp : grp * 8 + xcd;   // (as in the kernel above)
  if (bh >= p.bh_total) return;
  const int b = bh / p.Hkv, hs = bh % p.Hkv;
  const int hq = p.head_map ? p.head_map[hs] : hs;

  const int qrow = qt * 32 + col;
  const bool q_live = qrow < p.Lq;
  int limit = p.kv_limit ? min(p.kv_limit[min(qrow, p.Lq - 1)], p.Lk) : p.Lk;
  if (limit < 0) limit = 0;
  // every wavefront holds the same queries: the largest and smallest limit need no exchange between them
  int kv_end = q_live ? limit : 0, minlim = q_live ? limit : p.Lk;
  if (p.kv_limit) {
    for (int off = 1; off < 64; off <<= 1) {
      kv_end = max(kv_end, __shfl_xor(kv_end, off, 64));
      minlim = min(minlim, __shfl_xor(minlim, off, 64));
    }
  } else {
    kv_end = p.Lk; minlim = p.Lk;   // (some query of the tile is live)
  }
  // the share's blocks: a fixed number per share (set by the host from Lk), cut at the tile's last key
  const int nb = (kv_end + FQ_BK - 1) / FQ_BK;
  const int b_begin = split * p.fq_share_blocks, b_end = min(b_begin + p.fq_share_blocks, nb);
  // Block j of the share goes to wavefront (j + rot) % 4: the wavefront that gets the odd block
  // more differs between the workgroups that are likely to sit on one compute unit.  (A function
  // of the (batch, head) pair, the query tile and the share only, not of where the workgroup
  // sits in the grid: the two cache layouts add up in the same order.)
  const int slot_s = ((p.q_tiles == 2 ? ((bh >> 3) << 1) | qt : (bh >> 3))) * p.nsplit + split;
  const int rot = (slot_s + (slot_s >> 5)) & 3;
  const int blk0 = b_begin + ((wave - rot) & 3);

  u32 kmask = KCodec<BITS>::kMask;
  asm volatile("" : "+v"(kmask));

  // Packed words and parameters of a block as loaded.  The registers are refilled with the
  // wavefront's next block as soon as the current one has used them: K after S^T, V after the
  // V^T tile is written.  The requests are issued without conditions around them (past the end
  // they re-read the last key row; a missing zero-point array reads the scales instead): with a
  // branch around a load the compiler no longer knows how many loads are in flight and waits for
  // all of them where it needs the oldest.
  // Addresses: the (batch, head) bases are uniform; a lane keeps 32-bit byte offsets of its rows
  // from them, advanced by four blocks per request and clamped at the last key of the wavefront's
  // own last block (the host checks that they fit) -- an add and a min per stream instead of the
  // products of key and strides; the one request past the wavefront's blocks re-reads that row
  // instead of fetching a block of another wavefront's.
  const int64_t kv_row0 = b * p.kv_bs + hs * p.kv_hs;
  const char *const kw_base = reinterpret_cast<const char *>(p.k_words + kv_row0 * WPR);
  const char *const vw_base = reinterpret_cast<const char *>(p.v_words + kv_row0 * WPR);
  const char *const ks_base = reinterpret_cast<const char *>(p.k_scale + kv_row0);
  const char *const kz_base = reinterpret_cast<const char *>((p.k_zp ? p.k_zp : p.k_scale) + kv_row0);
  const char *const vs_base = reinterpret_cast<const char *>(p.v_scale + kv_row0);
  const char *const vz_base = reinterpret_cast<const char *>((p.v_zp ? p.v_zp : p.v_scale) + kv_row0);
  const bool has_kzp = p.k_zp != nullptr, has_vzp = p.v_zp != nullptr;
  const u32 row_b = (u32)p.kv_ts * (WPR * 4), par_b = (u32)p.kv_ts * 4;   // bytes from one key to the next
  static_assert(FQ_NW == 4, "a wavefront's blocks are four apart");
  const int last_blk = blk0 + ((max(b_end - 1 - blk0, 0) >> 2) << 2);   // (this wavefront's last block, if it has any)
  const u32 last_key = (u32)min(last_blk * FQ_BK + FQ_BK - 1, p.Lk - 1);
  const u32 par_last = last_key * par_b;
  const u32 k_lane = half * (HW * 4), v_lane = (lane >> 4) * (WPU * 4);     // this lane's place inside a row
  const u32 k_row_last = last_key * row_b + k_lane, v_row_last = last_key * row_b + v_lane;
  const u32 row_step = FQ_NW * FQ_BK * row_b, par_step = FQ_NW * FQ_BK * par_b;
  // MFMA row `col` carries key kperm(col) of the block; V: item = lane + 64 i covers keys 2 kp, 2 kp + 1
  // (kp = lane & 15: the lanes of a tile row write 16 adjacent banks) and unit (lane >> 4) + 4 i
  u32 ok_row = (u32)(blk0 * FQ_BK + kperm(col)) * row_b + k_lane, ok_par = (u32)(blk0 * FQ_BK + kperm(col)) * par_b;
  u32 ov_row = (u32)(blk0 * FQ_BK + 2 * (lane & 15)) * row_b + v_lane, ov_par = (u32)(blk0 * FQ_BK + 2 * (lane & 15)) * par_b;
  u32x4_t kraw[KP];
  u32 vraw[IPL][2][WPU];
  float ksc, kzp, vsc[2], vzp[2];   // (V: of this lane's two keys)
  auto umin = [](u32 x, u32 y) { return x < y ? x : y; };
  auto request_k = [&]() {   // the wavefront's next block
    const u32 orow = umin(ok_row, k_row_last), opar = umin(ok_par, par_last);
    ok_row += row_step; ok_par += par_step;
#pragma unroll
    for (int i = 0; i < KP; ++i) kraw[i] = *reinterpret_cast<const u32x4_t *>(kw_base + orow + 16 * i);
    ksc = *reinterpret_cast<const float *>(ks_base + opar);
    kzp = *reinterpret_cast<const float *>(kz_base + opar);
  };
  auto request_v = [&]() {
    const u32 orow[2] = {umin(ov_row, v_row_last), umin(ov_row + row_b, v_row_last)};
    const u32 opar[2] = {umin(ov_par, par_last), umin(ov_par + par_b, par_last)};
    ov_row += row_step; ov_par += par_step;
#pragma unroll
    for (int r = 0; r < 2; ++r) {   // (the parameters first: the block's V work starts with them)
      vsc[r] = *reinterpret_cast<const float *>(vs_base + opar[r]);
      vzp[r] = *reinterpret_cast<const float *>(vz_base + opar[r]);
    }
#pragma unroll
    for (int i = 0; i < IPL; ++i)
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const char *src = vw_base + orow[r] + i * (4 * WPU * 4);
        if constexpr (WPU == 2) { const uint2 t = *reinterpret_cast<const uint2 *>(src); vraw[i][r][0] = t.x; vraw[i][r][1] = t.y; }
        else vraw[i][r][0] = *reinterpret_cast<const u32 *>(src);
      }
  };
  // ---- this lane's query: the eight Q^T operands (channels in the slot order of the K codec)
  // stay in registers for the whole key loop; the loads go out ahead of the first block's ----
  u32x4_t qop[NCH];
  {
    const __bf16 *qp = p.q + (b * p.q_bs + hq * p.q_hs + min(qrow, p.Lq - 1) * p.q_ts) * D + half * 64;
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) qop[ch] = *reinterpret_cast<const u32x4_t *>(qp + ch * 8);
  }
  // (the loads keep this order -- queries, K, V: the compiler's count of loads in flight on the
  // way into the key loop becomes what it waits for inside it)
  __builtin_amdgcn_sched_barrier(0);
  request_k();
  __builtin_amdgcn_sched_barrier(0);
  request_v();
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int ch = 0; ch < NCH; ++ch) {
    const u32x4_t raw = qop[ch];
#pragma unroll
    for (int j2 = 0; j2 < 4; ++j2) {
      const int d0 = KCodec<BITS>::slot_d(2 * j2), d1 = KCodec<BITS>::slot_d(2 * j2 + 1);
      const u32 lo = (raw[d0 >> 1] >> (16 * (d0 & 1))) & 0xffffu, hi = (raw[d1 >> 1] >> (16 * (d1 & 1))) << 16;
      qop[ch][j2] = lo | hi;
    }
  }

  floatx16_t oacc[NDB];
#pragma unroll
  for (int d = 0; d < NDB; ++d)
#pragma unroll
    for (int j = 0; j < 16; ++j) oacc[d][j] = 0.f;
  float m_ref = 0.f, l_part = 0.f;
  bool first = true;

  // One block of 32 keys.  BYTES: 4-bit codes through bytes (see byte_bias4), with the bias ka4
  // of this lane's K row; V goes through bytes too if its zero-points fit.
  auto block = [&](const int blk, auto bytes_tag, const u32 ka4) {
    constexpr bool BYTES = decltype(bytes_tag)::value;
    const int t0 = blk * FQ_BK;
    // (code - zp) * scale = (raw - (zp + kOff) / kMul) * (kMul * scale) for the code image `raw`
    const float kz = has_kzp ? kzp : 0.f;
    const float zk = (kz + KCodec<BITS>::kOff) * (1.f / KCodec<BITS>::kMul), sk = ksc * KCodec<BITS>::kMul;
    const float ks_plain = ksc, kc = -128.f * ksc;

    // ---- S^T = K Q^T, K dequantized in registers ----
    floatx16_t sacc;
#pragma unroll
    for (int j = 0; j < 16; ++j) sacc[j] = 0.f;
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
      const int pc = ch / OPQ, j = ch % OPQ;
      u32 q4[4];
#pragma unroll
      for (int w = 0; w < 4; ++w) q4[w] = kraw[pc][w] ^ KCodec<BITS>::kStageXor;
      u32x4_t a;
      if constexpr (BYTES) {
        const u32 e = (q4[j] & 0x0f0f0f0fu) + ka4, o = ((q4[j] >> 4) & 0x0f0f0f0fu) + ka4;
        // operand slots (2m, 2m+1) hold channels (m, m+4): bytes 0 and 2 of e are channels 0 and 4, ...
        a[0] = pack_bf16_rne(__builtin_fmaf(ubyte_f32(e, 0), ks_plain, kc), __builtin_fmaf(ubyte_f32(e, 2), ks_plain, kc));
        a[1] = pack_bf16_rne(__builtin_fmaf(ubyte_f32(o, 0), ks_plain, kc), __builtin_fmaf(ubyte_f32(o, 2), ks_plain, kc));
        a[2] = pack_bf16_rne(__builtin_fmaf(ubyte_f32(e, 1), ks_plain, kc), __builtin_fmaf(ubyte_f32(e, 3), ks_plain, kc));
        a[3] = pack_bf16_rne(__builtin_fmaf(ubyte_f32(o, 1), ks_plain, kc), __builtin_fmaf(ubyte_f32(o, 3), ks_plain, kc));
      } else {
        float f[8];
        k_values<BITS>(q4, j, kmask, f);
#pragma unroll
        for (int m = 0; m < 4; ++m) a[m] = pack_bf16_rne((f[2 * m] - zk) * sk, (f[2 * m + 1] - zk) * sk);
      }
      sacc = mfma_32x32x16<false>(a, qop[ch], sacc);
    }
    request_k();

    // ---- V of the block -> V^T tile of this wavefront (bf16 values) ----
    // (z2, s2: byte biases and plain scales of the lane's two keys, or the general form's parameters)
    bool vbytes = false;
    float2 z2, s2;
    {
      u32 va0 = 0, va1 = 0;
      const float vz0 = has_vzp ? vzp[0] : 0.f, vz1 = has_vzp ? vzp[1] : 0.f;
      if constexpr (BYTES) {
        const bool ok0 = byte_bias4(vz0, va0), ok1 = byte_bias4(vz1, va1);
        vbytes = !__any(!(ok0 && ok1));
      }
      z2.x = vbytes ? u2f(va0) : (vz0 + VCodec<BITS>::kOff) * (1.f / VCodec<BITS>::kMul);
      z2.y = vbytes ? u2f(va1) : (vz1 + VCodec<BITS>::kOff) * (1.f / VCodec<BITS>::kMul);
      s2.x = vbytes ? vsc[0] : vsc[0] * VCodec<BITS>::kMul;
      s2.y = vbytes ? vsc[1] : vsc[1] * VCodec<BITS>::kMul;
    }
#pragma unroll
    for (int i = 0; i < IPL; ++i) {
      const int item = lane + 64 * i, kp = item & 15, u = item >> 4;   // (key pair fastest: the lanes of a row write 16 adjacent banks)
      u32 r0[WPU], r1[WPU];
#pragma unroll
      for (int w = 0; w < WPU; ++w) { r0[w] = vraw[i][0][w] ^ VCodec<BITS>::kStageXor; r1[w] = vraw[i][1][w] ^ VCodec<BITS>::kStageXor; }
      if (BYTES && vbytes) {
        // (z2 holds the two keys' byte biases, s2 their plain scales)
        const u32 e0 = (r0[0] & 0x0f0f0f0fu) + f2u(z2.x), o0 = ((r0[0] >> 4) & 0x0f0f0f0fu) + f2u(z2.x);
        const u32 e1 = (r1[0] & 0x0f0f0f0fu) + f2u(z2.y), o1 = ((r1[0] >> 4) & 0x0f0f0f0fu) + f2u(z2.y);
        const float c0 = -128.f * s2.x, c1 = -128.f * s2.y;
#pragma unroll
        for (int j2 = 0; j2 < 4; ++j2) {
          *reinterpret_cast<u32 *>(&vt[(u * 8 + 2 * j2) * FQ_VTS + kp * 2]) =
              pack_bf16_rne(__builtin_fmaf(ubyte_f32(e0, j2), s2.x, c0), __builtin_fmaf(ubyte_f32(e1, j2), s2.y, c1));
          *reinterpret_cast<u32 *>(&vt[(u * 8 + 2 * j2 + 1) * FQ_VTS + kp * 2]) =
              pack_bf16_rne(__builtin_fmaf(ubyte_f32(o0, j2), s2.x, c0), __builtin_fmaf(ubyte_f32(o1, j2), s2.y, c1));
        }
      } else {
#pragma unroll
        for (int o = 0; o < OPU; ++o) {
          float f0[8], f1[8];
          v_pair_values<BITS>(r0, r1, o, kmask, f0, f1);
          const int oct = u * OPU + o;
#pragma unroll
          for (int j = 0; j < 8; ++j)
            *reinterpret_cast<u32 *>(&vt[(oct * 8 + j) * FQ_VTS + kp * 2]) = pack_bf16_rne((f0[j] - z2.x) * s2.x, (f1[j] - z2.y) * s2.y);
        }
      }
    }
    request_v();

    // ---- softmax of the block: register i <-> key t0 + 16*(i/8) + 8*half + i%8 ----
    // The logits are taken against the reference as it stands (log2 domain) and the reference
    // moves only when a weight would exceed 2^16, which the block's sum of weights shows -- the
    // denominator needs that sum anyway, and the common block then has no search for the row
    // maximum and no rescaling of the 64 output accumulators.
    float z[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) z[i] = __builtin_fmaf(p.scale_log2e, sacc[i], -m_ref);
    if (t0 + FQ_BK > minlim) {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (t0 + 16 * (i >> 3) + 8 * half + (i & 7) >= limit) z[i] = -INFINITY;
    }
    // Moves the reference to the row's current maximum: up only once something has been
    // accumulated; the first block takes its maximum as it is (the accumulators are zero).
    auto move_reference = [&]() {
      float zmax = z[0];
#pragma unroll
      for (int i = 1; i < 16; ++i) zmax = fmaxf(zmax, z[i]);
      {
        const auto sw = __builtin_amdgcn_permlane32_swap(f2u(zmax), f2u(zmax), false, false);
        zmax = fmaxf(u2f(sw[0]), u2f(sw[1]));
      }
      const float delta = first ? ((zmax == -INFINITY) ? 0.f : zmax) : fmaxf(zmax, 0.f);
      const float alpha = first ? 1.f : __builtin_amdgcn_exp2f(-delta);
      m_ref += delta;
#pragma unroll
      for (int i = 0; i < 16; ++i) z[i] -= delta;
#pragma unroll
      for (int d = 0; d < NDB; ++d)
#pragma unroll
        for (int j = 0; j < 16; ++j) oacc[d][j] *= alpha;
      l_part *= alpha;
    };
    u32 pop[2][4];
    float bsum = 0.f;
    auto weights = [&]() {
      bsum = 0.f;
#pragma unroll
      for (int i2 = 0; i2 < 8; ++i2) {
        const int i = 2 * i2;
        const u32 w = pack_bf16_rne(__builtin_amdgcn_exp2f(z[i]), __builtin_amdgcn_exp2f(z[i + 1]));
        pop[i >> 3][(i & 7) >> 1] = w;
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
        bsum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), bsum, false);
      }
    };
    if (first) move_reference();
    weights();
    if (!first && __any(!(bsum <= 65536.f))) {
      move_reference();
      weights();
    }
    l_part += bsum;
    first = false;

    // ---- O^T += V^T P^T ----
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const u32x4_t bv = {pop[c][0], pop[c][1], pop[c][2], pop[c][3]};
#pragma unroll
      for (int d = 0; d < NDB; ++d) {
        const u32x4_t av = *reinterpret_cast<const u32x4_t *>(&vt[(d * 32 + col) * FQ_VTS + c * 16 + half * 8]);
        oacc[d] = mfma_32x32x16<false>(av, bv, oacc[d]);
      }
    }
  };

  // 4-bit codes go through bytes until a K zero-point of a block does not fit; from there on (and
  // for the other widths) the general form.  Two loops one after the other rather than two arms
  // inside one: arms that both update the output accumulators make the compiler copy them at
  // the join, twice per block.
  int blk = blk0;
  if constexpr (BITS == 4) {
    for (; blk < b_end; blk += FQ_NW) {
      u32 ka4 = 0;
      if (__any(!byte_bias4(has_kzp ? kzp : 0.f, ka4))) break;
      // Two workgroups share a compute unit and the SIMD's arbiter prefers the older wavefront:
      // left alone, the older workgroup finishes about a quarter earlier and the younger one
      // then runs its rest at one wavefront per SIMD.  Priority by the quarter of its own
      // blocks a wavefront is in lets the one that is behind catch up.
      {
        const int q4 = (blk - blk0) * 4 / max(b_end - blk0, 1);
        if (q4 == 0) __builtin_amdgcn_s_setprio(3);
        else if (q4 == 1) __builtin_amdgcn_s_setprio(2);
        else if (q4 == 2) __builtin_amdgcn_s_setprio(1);
        else __builtin_amdgcn_s_setprio(0);
      }
      block(blk, std::true_type{}, ka4);
    }
  }
  for (; blk < b_end; blk += FQ_NW) block(blk, std::false_type{}, 0u);

  // ---- merge the wavefronts' partial results: wavefront t ends up with channels 32t .. 32t+31 ----
  // Every wavefront hands the other three their quarters of its accumulators through LDS (one
  // barrier on each side), forms the four weights from everyone's (m, l) and sums its quarter.
  const float l_own = l_part + __shfl_xor(l_part, 32, 64);
  float *const slots = reinterpret_cast<float *>(lds_raw + FewQLds::kVt);   // [target][source - target - 1 mod 4][16 registers][64 lanes]
  __syncthreads();   // every wavefront is done with its V^T tile
#pragma unroll
  for (int t = 0; t < FQ_NW; ++t) {
    if (t == wave) continue;
    float *dst = slots + ((t * 3 + ((wave - t - 1) & 3)) * 16) * 64 + lane;
#pragma unroll
    for (int j = 0; j < 16; ++j) dst[j * 64] = oacc[t][j];
  }
  if (half == 0) *reinterpret_cast<float2 *>(lds_ml + (wave * 32 + col) * 2) = make_float2(m_ref, l_own);
  __syncthreads();
  // (the partial results are addressed through LDS, not through register arrays with a run-time index)
  float M = 0.f;
  bool any_live = false;
#pragma unroll
  for (int w = 0; w < FQ_NW; ++w) {
    const float2 ml = *reinterpret_cast<const float2 *>(lds_ml + (w * 32 + col) * 2);
    if (ml.y > 0.f) { M = any_live ? fmaxf(M, ml.x) : ml.x; any_live = true; }
  }
  auto weight_of = [&](int w, float &l_w) {
    const float2 ml = *reinterpret_cast<const float2 *>(lds_ml + (w * 32 + col) * 2);
    l_w = ml.y;
    return ml.y > 0.f ? __builtin_amdgcn_exp2f(ml.x - M) : 0.f;
  };
  float l_sum = 0.f;   // (summed in the same order by every wavefront)
#pragma unroll
  for (int w = 0; w < FQ_NW; ++w) {
    float l_w;
    const float wt = weight_of(w, l_w);
    l_sum = __builtin_fmaf(l_w, wt, l_sum);
  }
  float mine[16];
  {
    float l_w;
    const float w_own = weight_of(wave, l_w);
#pragma unroll
    for (int t = 0; t < FQ_NW; ++t)
      if (t == wave) {   // (a wavefront-uniform choice among the four accumulator blocks)
#pragma unroll
        for (int j = 0; j < 16; ++j) mine[j] = oacc[t][j] * w_own;
      }
  }
#pragma unroll
  for (int s = 0; s < FQ_NW - 1; ++s) {
    float l_w;
    const float ws = weight_of((wave + 1 + s) & 3, l_w);
    const float *src = slots + ((wave * 3 + s) * 16) * 64 + lane;
#pragma unroll
    for (int j = 0; j < 16; ++j) mine[j] = __builtin_fmaf(src[j * 64], ws, mine[j]);
  }
  if (!q_live) return;
  const float inv = l_sum > 0.f ? 1.0f / l_sum : 0.f;
  // registers 4*g4 .. 4*g4+3 are rows 32*wave + 8*g4 + 4*half + 0..3 of O^T
  if (p.nsplit > 1) {
    const int64_t prow = ((int64_t)split * p.bh_total + bh) * p.Lq + qrow;
    float *wptr = p.ws_o + prow * D + wave * 32 + 4 * half;
    if (wave == 0 && half == 0) *reinterpret_cast<float2 *>(p.ws_ml + prow * 2) = make_float2(M, l_sum);
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4)
      *reinterpret_cast<float4 *>(wptr + 8 * g4) = make_float4(mine[4 * g4] * inv, mine[4 * g4 + 1] * inv, mine[4 * g4 + 2] * inv, mine[4 * g4 + 3] * inv);
  } else {
    __bf16 *optr = p.out + (b * p.o_bs + hq * p.o_hs + qrow * p.o_ts) * D + wave * 32 + 4 * half;
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4)
      *reinterpret_cast<uint2 *>(optr + 8 * g4) =
          make_uint2(pack_bf16_rne(mine[4 * g4] * inv, mine[4 * g4 + 1] * inv), pack_bf16_rne(mine[4 * g4 + 2] * inv, mine[4 * g4 + 3] * inv));
  }
}

// Whether a launch takes the few-queries kernel, and over how many workgroups the keys of a
// (batch, head, 32 queries) are shared out then: enough for the two resident workgroups per
// compute unit (the kernel holds ~200 registers), at least eight blocks per workgroup.
bool fewq_eligible(int B, int Hkv, int Lq, int Lk, int D, int k_group, int v_group) {
  // (the kernel keeps 32-bit byte offsets inside one (batch, head): rows of up to D bytes, up to
  // Hkv rows from one key to the next, a few blocks of overshoot before the clamp)
  return D == FQ_D && k_group == D && v_group == D && Lq > 0 && Lq <= kFewQueries && Lk >= kFewQMinKeys &&
         ((int64_t)Lk + 8 * FQ_BK) * Hkv * D < (1ll << 32) &&
         ((int64_t)B * Hkv + 7) / 8 * ((Lq + 31) / 32) <= 65535;   // (the grid's z extent)
}
int fewq_shares(int bh_total, int Lq, int Lk) {
  const int64_t tiles = (int64_t)((bh_total + 7) / 8 * 8) * ((Lq + 31) / 32);
  int64_t s = (2 * (int64_t)device_cus() + tiles - 1) / tiles;
  const int64_t nb = (Lk + FQ_BK - 1) / FQ_BK;
  if (s > nb / 8) s = nb / 8;
  if (s > kMaxKeyShares) s = kMaxKeyShares;
  return s < 1 ? 1 : (int)s;
}

template <int BITS> void launch_fewq(const AttnParams &p, hipStream_t st) {
  const int bh_pad = (p.bh_total + 7) / 8 * 8;
  dim3 grid(8, (unsigned)p.nsplit, (unsigned)(bh_pad / 8 * p.q_tiles));
  hipLaunchKernelGGL((fused_attn_fewq_kernel<BITS>), grid, dim3(FQ_NW * 64), FewQLds::kBytes, st, p);
  if (p.nsplit > 1) {
    const int64_t rows = (int64_t)p.bh_total * p.Lq;
    hipLaunchKernelGGL((combine_splits_kernel<FQ_D, false>), dim3((unsigned)((rows + 1) / 2)), dim3(256), 0, st, p);
  }
}

}  // namespace

extern "C" size_t varq_fused_attn_workspace_bytes(int B, int Hkv, int Lq, int Lk, int D, int nseg, int splits) {
  if (B <= 0 || Hkv <= 0 || Lq <= 0 || Lk <= 0 || (D != 64 && D != 128) || splits < 0 || splits > kMaxSplits) return 0;
  const int64_t rows = (int64_t)B * Hkv * Lq;
  (void)nseg;   // (the tile count does not depend on the tables)
  const int tiles = (Lk + BN - 1) / BN;
  int n = splits ? splits : choose_splits((int64_t)B * Hkv * ((Lq + BM - 1) / BM), tiles, rows, D);
  // (the group sizes are not known here: room for the few-queries kernel's shares whenever the
  // other sizes would admit it)
  if (splits == 0 && fewq_eligible(B, Hkv, Lq, Lk, D, D, D)) n = max(n, fewq_shares(B * Hkv, Lq, Lk));
  return split_workspace_bytes(n, rows, D);
}

extern "C" int varq_fused_attn_key_shares(int B, int Hkv, int Lq, int Lk, int D, int k_group, int v_group) {
  if (B <= 0 || Hkv <= 0 || Lq <= 0 || Lk <= 0 || (D != 64 && D != 128)) return 0;
  if (fewq_eligible(B, Hkv, Lq, Lk, D, k_group, v_group)) return fewq_shares(B * Hkv, Lq, Lk);
  return choose_splits((int64_t)B * Hkv * ((Lq + BM - 1) / BM), (Lk + BN - 1) / BN, (int64_t)B * Hkv * Lq, D);
}

extern "C" int varq_fused_attn(const void *q, void *out,
                               const int32_t *k_words, const float *k_scale, const float *k_zp, int k_bits, int k_group,
                               const int32_t *v_words, const float *v_scale, const float *v_zp, int v_bits, int v_group,
                               int B, int Hq, int Hkv, const int32_t *head_map,
                               int Lq, int Lk, int Lk_stride, int D,
                               const int32_t *kv_limit, float softmax_scale, int layout, int io_dtype, int operand_form,
                               void *workspace, size_t workspace_bytes, int splits, void *stream) {
  VARQ_CHECK_ARG(B > 0 && Hq > 0 && Hkv > 0 && Lq >= 0 && Lk >= 0 && Lk_stride >= Lk, "fused_attn: bad sizes");
  VARQ_CHECK_ARG(io_dtype == VARQ_BF16 || io_dtype == VARQ_F16, "fused_attn: io_dtype must be VARQ_BF16 (1) or VARQ_F16 (2), got %d", io_dtype);
  VARQ_CHECK_ARG(operand_form == VARQ_ATTN_REFERENCE_ROUNDING || operand_form == VARQ_ATTN_EXACT_CODES,
                 "fused_attn: operand_form must be 0 (reference rounding) or 1 (exact codes), got %d", operand_form);
  if (io_dtype == VARQ_F16 && D != 64)
    return varq_set_error(VARQ_ERR_UNSUPPORTED, "fused_attn: fp16 queries need D = 64 (got %d); D = 128 is served in bf16", D);
  // (no queries: nothing to do, and q and out may be the null pointers of empty tensors)
  VARQ_CHECK_ARG(Lq == 0 || (q && out), "fused_attn: null pointer");
  VARQ_CHECK_ARG(Lq == 0 || Lk == 0 || (k_words && v_words && k_scale && v_scale), "fused_attn: null pointer");
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
  VARQ_CHECK_ARG(((uintptr_t)q & 15) == 0 && ((uintptr_t)out & 7) == 0, "fused_attn: q must be 16-byte and out 8-byte aligned");

  AttnParams p;
  p.q = reinterpret_cast<const __bf16 *>(q);
  p.out = reinterpret_cast<__bf16 *>(out);
  p.k_words = reinterpret_cast<const u32 *>(k_words);
  p.v_words = reinterpret_cast<const u32 *>(v_words);
  p.k_scale = k_scale; p.k_zp = k_zp; p.v_scale = v_scale; p.v_zp = v_zp;
  p.k_chan_scale = nullptr; p.k_chan_zp = nullptr; p.v_chan_scale = nullptr; p.v_chan_zp = nullptr;
  p.nseg = 1;
  for (int s = 0; s < kMaxSegments; ++s) p.seg_end[s] = Lk;
  p.head_map = head_map; p.kv_limit = kv_limit;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.Lq = Lq; p.Lk = Lk; p.Lstride = Lk_stride;
  p.q_tiles = (Lq + BM - 1) / BM;
  p.bh_total = B * Hkv;
  p.fq_share_blocks = 0;
  p.scale_log2e = softmax_scale * kLog2e;
  p.f16 = io_dtype == VARQ_F16;
  p.exact_codes = operand_form == VARQ_ATTN_EXACT_CODES && !p.f16;
  if (int e = set_layout(p, layout, "fused_attn")) return e;
  hipStream_t st = (hipStream_t)stream;
  // few queries over a long cache, left to the library: the kernel whose wavefronts share the keys
  if (splits == 0 && !p.f16 && !p.exact_codes && fewq_eligible(B, Hkv, Lq, Lk, D, k_group, v_group)) {
    const int64_t rows = (int64_t)p.bh_total * Lq;
    int n = fewq_shares(p.bh_total, Lq, Lk);
    while (n > 1 && (!workspace || ((uintptr_t)workspace & 15) || workspace_bytes < split_workspace_bytes(n, rows, D))) --n;
    p.q_tiles = (Lq + 31) / 32;
    p.nsplit = n;
    p.fq_share_blocks = ((Lk + FQ_BK - 1) / FQ_BK + n - 1) / n;
    p.ws_o = n > 1 ? reinterpret_cast<float *>(workspace) : nullptr;
    p.ws_ml = n > 1 ? p.ws_o + (size_t)n * (size_t)rows * (size_t)D : nullptr;
    if (k_bits == 4) launch_fewq<4>(p, st);
    else if (k_bits == 8) launch_fewq<8>(p, st);
    else launch_fewq<2>(p, st);
    VARQ_CHECK_LAUNCH("fused_attn");
    return VARQ_OK;
  }
  if (int e = set_splits(p, D, (Lk + BN - 1) / BN, splits, workspace, workspace_bytes, "fused_attn")) return e;
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

extern "C" int varq_fused_attn_channel(const void *q, void *out,
                                       const int32_t *k_words, const float *k_chan_scale, const float *k_chan_zp,
                                       const int32_t *v_words, const float *v_chan_scale, const float *v_chan_zp,
                                       int nseg, const int32_t *host_seg_end,
                                       int bits, int B, int Hq, int Hkv, const int32_t *head_map,
                                       int Lq, int Lk, int Lk_stride, int D,
                                       const int32_t *kv_limit, float softmax_scale, int layout, int io_dtype,
                                       void *workspace, size_t workspace_bytes, int splits, void *stream) {
  VARQ_CHECK_ARG(io_dtype == VARQ_BF16 || io_dtype == VARQ_F16, "fused_attn_channel: io_dtype must be VARQ_BF16 (1) or VARQ_F16 (2), got %d", io_dtype);
  if (io_dtype == VARQ_F16 && D != 64)
    return varq_set_error(VARQ_ERR_UNSUPPORTED, "fused_attn_channel: fp16 queries need D = 64 (got %d); D = 128 is served in bf16", D);
  // (no queries: nothing to do, and q and out may be the null pointers of empty tensors)
  VARQ_CHECK_ARG(Lq == 0 || (q && out), "fused_attn_channel: null pointer");
  VARQ_CHECK_ARG(Lq == 0 || Lk == 0 || (k_words && v_words && k_chan_scale && v_chan_scale), "fused_attn_channel: null pointer");
  VARQ_CHECK_ARG(nseg >= 1 && nseg <= kMaxSegments, "fused_attn_channel: nseg must be 1..%d (got %d)", kMaxSegments, nseg);
  VARQ_CHECK_ARG(nseg == 1 || host_seg_end, "fused_attn_channel: segment ends missing");
  VARQ_CHECK_ARG(B > 0 && Hq > 0 && Hkv > 0 && Lq >= 0 && Lk >= 0 && Lk_stride >= Lk, "fused_attn_channel: bad sizes");
  VARQ_CHECK_ARG(head_map || Hkv == Hq, "fused_attn_channel: Hkv != Hq needs a head map");
  VARQ_CHECK_ARG(D == 64 || D == 128, "fused_attn_channel: D must be 64 or 128 (got %d)", D);
  VARQ_CHECK_ARG(bits == 2 || bits == 4 || bits == 8, "fused_attn_channel: bits must be 2, 4 or 8 (got %d)", bits);
  if (Lq == 0 || Lk == 0) {
    if (Lq > 0) return varq_set_error(VARQ_ERR_INVALID, "fused_attn_channel: no keys to attend");
    return VARQ_OK;
  }
  VARQ_CHECK_ARG((int64_t)B * Hkv * Lk_stride * D < (1ll << 40), "fused_attn_channel: cache too large");
  VARQ_CHECK_ARG(((uintptr_t)q & 15) == 0 && ((uintptr_t)out & 7) == 0,
                 "fused_attn_channel: q must be 16-byte and out 8-byte aligned");
  VARQ_CHECK_ARG(((uintptr_t)k_chan_scale & 15) == 0 && ((uintptr_t)k_chan_zp & 15) == 0 &&
                     ((uintptr_t)v_chan_scale & 15) == 0 && ((uintptr_t)v_chan_zp & 15) == 0,
                 "fused_attn_channel: the tables must be 16-byte aligned");

  AttnParams p;
  p.q = reinterpret_cast<const __bf16 *>(q);
  p.out = reinterpret_cast<__bf16 *>(out);
  p.k_words = reinterpret_cast<const u32 *>(k_words);
  p.v_words = reinterpret_cast<const u32 *>(v_words);
  p.k_scale = nullptr; p.k_zp = nullptr; p.v_scale = nullptr; p.v_zp = nullptr;
  p.k_chan_scale = k_chan_scale; p.k_chan_zp = k_chan_zp; p.v_chan_scale = v_chan_scale; p.v_chan_zp = v_chan_zp;
  p.nseg = nseg;
  for (int s = 0, prev = 0; s < nseg; ++s) {
    // the last segment runs to the end of the keys whatever the caller's table says
    const int e = (s == nseg - 1 || !host_seg_end) ? Lk : host_seg_end[s];
    VARQ_CHECK_ARG(e > prev || (s == nseg - 1 && e >= prev), "fused_attn_channel: segment ends must increase");
    VARQ_CHECK_ARG(e <= Lk, "fused_attn_channel: segment end %d beyond Lk=%d", e, Lk);
    p.seg_end[s] = e;
    prev = e;
  }
  for (int s = nseg; s < kMaxSegments; ++s) p.seg_end[s] = Lk;
  p.head_map = head_map; p.kv_limit = kv_limit;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.Lq = Lq; p.Lk = Lk; p.Lstride = Lk_stride;
  p.q_tiles = (Lq + BM - 1) / BM;
  p.bh_total = B * Hkv;
  p.fq_share_blocks = 0;
  p.scale_log2e = softmax_scale * kLog2e;
  p.f16 = io_dtype == VARQ_F16;
  p.exact_codes = 0;
  if (int e = set_layout(p, layout, "fused_attn_channel")) return e;
  if (int e = set_splits(p, D, (Lk + BN - 1) / BN, splits, workspace, workspace_bytes, "fused_attn_channel"))
    return e;
  hipStream_t st = (hipStream_t)stream;
  if (D == 128) {
    if (bits == 4) launch<128, 4, 128, 128, true>(p, st);
    else if (bits == 8) launch<128, 8, 128, 128, true>(p, st);
    else launch<128, 2, 128, 128, true>(p, st);
  } else {
    if (bits == 4) launch<64, 4, 64, 64, true>(p, st);
    else if (bits == 8) launch<64, 8, 64, 64, true>(p, st);
    else launch<64, 2, 64, 64, true>(p, st);
  }
  VARQ_CHECK_LAUNCH("fused_attn_channel");
  return VARQ_OK;
}

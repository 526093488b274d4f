// Stand-alone bit packing and unpacking of int8 codes, the operations of
// VAR_Q/pack_unpack.py:107-162 (Triton wrappers) and 177-211 (layout
// definition).  Pure byte shuffling, HBM-bound: one thread per four 32-bit words
// (16 bytes of words, 16 to 64 bytes of codes, all in 16-byte accesses) when a row is a
// whole number of words and both buffers are 16-byte aligned; one thread per word
// otherwise, byte accesses for rows that do not fill their last word.
#include "varq_common.h"

namespace {

// 4 bytes -> their low `BITS` bits, concatenated (byte k -> field k).
template <int BITS> __device__ __forceinline__ u32 squeeze4(u32 b) {
  if (BITS == 8) return b;
  if (BITS == 4) {
    u32 t = b & 0x0f0f0f0fu;
    t = (t | (t >> 4)) & 0x00ff00ffu;
    return (t | (t >> 8)) & 0xffffu;
  }
  u32 t = b & 0x03030303u;
  t = (t | (t >> 6)) & 0x000f000fu;
  return (t | (t >> 12)) & 0xffu;
}

// field k of the low 4*BITS bits -> sign-extended byte k.
template <int BITS> __device__ __forceinline__ u32 spread4(u32 f) {
  if (BITS == 8) return f;
  u32 t;
  if (BITS == 4) {
    t = f & 0xffffu;
    t = (t | (t << 8)) & 0x00ff00ffu;
    t = (t | (t << 4)) & 0x0f0f0f0fu;
    const u32 s = t & 0x08080808u;       // sign bit of each field
    return t | ((s << 5) - (s << 1));     // fill bits 4..7 of negative fields
  }
  t = f & 0xffu;
  t = (t | (t << 12)) & 0x000f000fu;
  t = (t | (t << 6)) & 0x03030303u;
  const u32 s = t & 0x02020202u;
  return t | ((s << 7) - (s << 1));       // fill bits 2..7
}

template <int BITS> __device__ __forceinline__ u32 pack_word(const u32 *src) {   // 32/BITS codes -> one word
  if (BITS == 8) return src[0];
  if (BITS == 4) return squeeze4<4>(src[0]) | (squeeze4<4>(src[1]) << 16);
  return squeeze4<2>(src[0]) | (squeeze4<2>(src[1]) << 8) | (squeeze4<2>(src[2]) << 16) | (squeeze4<2>(src[3]) << 24);
}
template <int BITS> __device__ __forceinline__ void unpack_word(u32 x, u32 *dst) {   // one word -> 32/BITS codes
  if (BITS == 8) dst[0] = x;
  else if (BITS == 4) { dst[0] = spread4<4>(x); dst[1] = spread4<4>(x >> 16); }
  else { dst[0] = spread4<2>(x); dst[1] = spread4<2>(x >> 8); dst[2] = spread4<2>(x >> 16); dst[3] = spread4<2>(x >> 24); }
}

// Four words per thread: one 16-byte piece of words, DPW 16-byte pieces of codes.  (n_quads =
// n_words / 4; the host sends the words that are left to the per-word kernel.)
template <int BITS>
__global__ __launch_bounds__(256) void pack_quad_kernel(const int8_t *codes, int32_t *words, int64_t n_quads) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_quads) return;
  constexpr int DPW = 8 / BITS;   // dwords of codes per word: 1, 2 or 4
  const uint4 *src = reinterpret_cast<const uint4 *>(codes) + i * DPW;
  u32 q[4 * DPW];
#pragma unroll
  for (int k = 0; k < DPW; ++k) {
    const uint4 t = src[k];
    q[4 * k] = t.x; q[4 * k + 1] = t.y; q[4 * k + 2] = t.z; q[4 * k + 3] = t.w;
  }
  reinterpret_cast<uint4 *>(words)[i] =
      make_uint4(pack_word<BITS>(q), pack_word<BITS>(q + DPW), pack_word<BITS>(q + 2 * DPW), pack_word<BITS>(q + 3 * DPW));
}

// Unpacking writes most of the bytes, so there a thread owns one 16-byte piece of codes:
// BITS / 2 words (n_pieces = n_words / (BITS / 2)).
template <int BITS>
__global__ __launch_bounds__(256) void unpack_piece_kernel(const int32_t *words, int8_t *codes, int64_t n_pieces) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_pieces) return;
  constexpr int WPT = BITS / 2, DPW = 8 / BITS;   // words per thread, dwords of codes per word
  const u32 *src = reinterpret_cast<const u32 *>(words) + i * WPT;
  u32 x[WPT];
  if constexpr (WPT == 4) { const uint4 t = *reinterpret_cast<const uint4 *>(src); x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w; }
  else if constexpr (WPT == 2) { const uint2 t = *reinterpret_cast<const uint2 *>(src); x[0] = t.x; x[1] = t.y; }
  else x[0] = src[0];
  u32 q[4];
#pragma unroll
  for (int k = 0; k < WPT; ++k) unpack_word<BITS>(x[k], q + k * DPW);
  reinterpret_cast<uint4 *>(codes)[i] = make_uint4(q[0], q[1], q[2], q[3]);
}

// one word per thread, from word `w0` on
template <int BITS>
__global__ __launch_bounds__(256) void pack_flat_kernel(const int8_t *codes, int32_t *words, int64_t w0, int64_t n_words) {
  const int64_t w = w0 + (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (w >= n_words) return;
  constexpr int VALS = 32 / BITS;
  words[w] = (int32_t)pack_word<BITS>(reinterpret_cast<const u32 *>(codes + w * VALS));
}

template <int BITS>
__global__ __launch_bounds__(256) void unpack_flat_kernel(const int32_t *words, int8_t *codes, int64_t w0, int64_t n_words) {
  const int64_t w = w0 + (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (w >= n_words) return;
  constexpr int VALS = 32 / BITS;
  unpack_word<BITS>((u32)words[w], reinterpret_cast<u32 *>(codes + w * VALS));
}

// Any c: rows that do not fill their last word (zero padding on pack, dropped
// on unpack), byte accesses.
__global__ void pack_ragged_kernel(const int8_t *codes, int32_t *words, int64_t rows, int c, int bits, int wpr) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows * wpr) return;
  const int64_t r = t / wpr;
  const int wi = (int)(t - r * wpr);
  const int vals = 32 / bits;
  const u32 mask = (1u << bits) - 1u;
  u32 w = 0;
  for (int j = 0; j < vals; ++j) {
    const int ch = wi * vals + j;
    if (ch < c) w |= ((u32)(int)codes[r * c + ch] & mask) << (j * bits);
  }
  words[t] = (int32_t)w;
}

__global__ void unpack_ragged_kernel(const int32_t *words, int8_t *codes, int64_t rows, int c, int bits, int wpr) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows * wpr) return;
  const int64_t r = t / wpr;
  const int wi = (int)(t - r * wpr);
  const int vals = 32 / bits;
  const int x = words[t];
  for (int j = 0; j < vals; ++j) {
    const int ch = wi * vals + j;
    if (ch < c) codes[r * c + ch] = (int8_t)__builtin_amdgcn_sbfe(x, j * bits, bits);
  }
}

int check_common(const void *a, const void *b, int64_t rows, int c, int bits, const char *who) {
  if (!(bits == 2 || bits == 4 || bits == 8)) return varq_set_error(VARQ_ERR_INVALID, "%s: bits must be 2, 4 or 8 (got %d)", who, bits);
  if (rows < 0 || c <= 0) return varq_set_error(VARQ_ERR_INVALID, "%s: bad shape rows=%lld c=%d", who, (long long)rows, c);
  if (rows > 0 && (!a || !b)) return varq_set_error(VARQ_ERR_INVALID, "%s: null pointer", who);
  const int vals = 32 / bits;
  const int64_t wpr = (c + vals - 1) / vals;
  if (rows * wpr >= (1ll << 39)) return varq_set_error(VARQ_ERR_INVALID, "%s: too large", who);
  return 0;
}

}  // namespace

extern "C" int varq_pack(const int8_t *codes, int64_t rows, int c, int bits, int32_t *words, void *stream) {
  if (int rc = check_common(codes, words, rows, c, bits, "pack")) return rc;
  if (rows == 0) return VARQ_OK;
  hipStream_t st = (hipStream_t)stream;
  const int vals = 32 / bits;
  const int wpr = (c + vals - 1) / vals;
  const int64_t n_words = rows * wpr;
  dim3 grid((unsigned)((n_words + 255) / 256));
  if (c % vals == 0 && ((uintptr_t)codes % 16) == 0) {
    // whole words only: the tensor is one flat run of words; four per thread where the words are
    // 16-byte aligned too, the last 0..3 (or all of them) one per thread
    const int64_t n_quads = ((uintptr_t)words % 16) == 0 ? n_words / 4 : 0;
    const int64_t w0 = n_quads * 4;
    dim3 qgrid((unsigned)((n_quads + 255) / 256)), tgrid((unsigned)((n_words - w0 + 255) / 256));
#define VARQ_PACK(B_)                                                                                           \
  {                                                                                                             \
    if (n_quads) hipLaunchKernelGGL(pack_quad_kernel<B_>, qgrid, dim3(256), 0, st, codes, words, n_quads);      \
    if (w0 < n_words) hipLaunchKernelGGL(pack_flat_kernel<B_>, tgrid, dim3(256), 0, st, codes, words, w0, n_words); \
  }
    if (bits == 8) VARQ_PACK(8) else if (bits == 4) VARQ_PACK(4) else VARQ_PACK(2)
#undef VARQ_PACK
  } else {
    hipLaunchKernelGGL(pack_ragged_kernel, grid, dim3(256), 0, st, codes, words, rows, c, bits, wpr);
  }
  VARQ_CHECK_LAUNCH("pack");
  return VARQ_OK;
}

extern "C" int varq_unpack(const int32_t *words, int64_t rows, int c, int bits, int8_t *codes, void *stream) {
  if (int rc = check_common(words, codes, rows, c, bits, "unpack")) return rc;
  if (rows == 0) return VARQ_OK;
  hipStream_t st = (hipStream_t)stream;
  const int vals = 32 / bits;
  const int wpr = (c + vals - 1) / vals;
  const int64_t n_words = rows * wpr;
  dim3 grid((unsigned)((n_words + 255) / 256));
  if (c % vals == 0 && ((uintptr_t)codes % 16) == 0) {
    const int wpt = bits / 2;   // words per 16 bytes of codes
    const int64_t n_pieces = ((uintptr_t)words % 16) == 0 ? n_words / wpt : 0;
    const int64_t w0 = n_pieces * wpt;
    dim3 qgrid((unsigned)((n_pieces + 255) / 256)), tgrid((unsigned)((n_words - w0 + 255) / 256));
#define VARQ_UNPACK(B_)                                                                                           \
  {                                                                                                               \
    if (n_pieces) hipLaunchKernelGGL(unpack_piece_kernel<B_>, qgrid, dim3(256), 0, st, words, codes, n_pieces);   \
    if (w0 < n_words) hipLaunchKernelGGL(unpack_flat_kernel<B_>, tgrid, dim3(256), 0, st, words, codes, w0, n_words); \
  }
    if (bits == 8) VARQ_UNPACK(8) else if (bits == 4) VARQ_UNPACK(4) else VARQ_UNPACK(2)
#undef VARQ_UNPACK
  } else {
    hipLaunchKernelGGL(unpack_ragged_kernel, grid, dim3(256), 0, st, words, codes, rows, c, bits, wpr);
  }
  VARQ_CHECK_LAUNCH("unpack");
  return VARQ_OK;
}

// Stand-alone bit packing and unpacking of int8 codes, the operations of
// VAR_Q/pack_unpack.py:107-162 (Triton wrappers) and 177-211 (layout
// definition).  Pure byte shuffling, HBM-bound: one thread per 32-bit word,
// 16-byte code loads/stores when a row is a whole number of words.
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

template <int BITS>
__global__ __launch_bounds__(256) void pack_flat_kernel(const int8_t *codes, int32_t *words, int64_t n_words) {
  const int64_t w = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (w >= n_words) return;
  constexpr int VALS = 32 / BITS;
  const u32 *src = reinterpret_cast<const u32 *>(codes + w * VALS);
  u32 out;
  if (BITS == 8) out = src[0];
  else if (BITS == 4) {
    uint2 b = *reinterpret_cast<const uint2 *>(src);
    out = squeeze4<4>(b.x) | (squeeze4<4>(b.y) << 16);
  } else {
    uint4 b = *reinterpret_cast<const uint4 *>(src);
    out = squeeze4<2>(b.x) | (squeeze4<2>(b.y) << 8) | (squeeze4<2>(b.z) << 16) | (squeeze4<2>(b.w) << 24);
  }
  words[w] = (int32_t)out;
}

template <int BITS>
__global__ __launch_bounds__(256) void unpack_flat_kernel(const int32_t *words, int8_t *codes, int64_t n_words) {
  const int64_t w = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (w >= n_words) return;
  constexpr int VALS = 32 / BITS;
  const u32 x = (u32)words[w];
  u32 *dst = reinterpret_cast<u32 *>(codes + w * VALS);
  if (BITS == 8) dst[0] = x;
  else if (BITS == 4) *reinterpret_cast<uint2 *>(dst) = make_uint2(spread4<4>(x), spread4<4>(x >> 16));
  else *reinterpret_cast<uint4 *>(dst) = make_uint4(spread4<2>(x), spread4<2>(x >> 8), spread4<2>(x >> 16), spread4<2>(x >> 24));
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
    if (bits == 8) hipLaunchKernelGGL(pack_flat_kernel<8>, grid, dim3(256), 0, st, codes, words, n_words);
    else if (bits == 4) hipLaunchKernelGGL(pack_flat_kernel<4>, grid, dim3(256), 0, st, codes, words, n_words);
    else hipLaunchKernelGGL(pack_flat_kernel<2>, grid, dim3(256), 0, st, codes, words, n_words);
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
    if (bits == 8) hipLaunchKernelGGL(unpack_flat_kernel<8>, grid, dim3(256), 0, st, words, codes, n_words);
    else if (bits == 4) hipLaunchKernelGGL(unpack_flat_kernel<4>, grid, dim3(256), 0, st, words, codes, n_words);
    else hipLaunchKernelGGL(unpack_flat_kernel<2>, grid, dim3(256), 0, st, words, codes, n_words);
  } else {
    hipLaunchKernelGGL(unpack_ragged_kernel, grid, dim3(256), 0, st, words, codes, rows, c, bits, wpr);
  }
  VARQ_CHECK_LAUNCH("unpack");
  return VARQ_OK;
}

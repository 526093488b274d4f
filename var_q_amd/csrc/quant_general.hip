// General two-phase quantizer: groups that span rows (the six grouping methods
// of VAR_Q/quant.py:75-95, which all reduce over the batch dim, plus any other
// reduce set).  A single HBM read cannot serve such groups, so:
//   phase A  group min/max (or max-abs) -> workspace, via ordered-integer atomics
//   finalize workspace -> scale / zero-point           (VAR_Q/quant.py:112-116)
//   phase B  re-read input (L2 / Infinity-Cache resident for KV-sized tensors),
//            divide, round half-to-even, clamp, pack    (VAR_Q/quant.py:118-121,
//            VAR_Q/pack_unpack.py:177-196)
// min/max are exactly associative, so the result does not depend on the order
// in which partial results meet.
#include "varq_common.h"

namespace {

// Order-preserving float <-> uint map so that integer atomicMin/Max implement
// float min/max.
__device__ __forceinline__ u32 enc_ord(float f) {
  u32 u = f2u(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float dec_ord(u32 e) {
  return u2f((e & 0x80000000u) ? (e & 0x7fffffffu) : ~e);
}

struct GenParams {
  const void *x;
  u32 *ws_max;   // [n_groups] encoded max (or max-abs)
  u32 *ws_min;   // [n_groups] encoded min (asym only)
  float *scale, *zp;
  int32_t *words;
  int8_t *codes;
  int64_t n0, n1, n2;      // leading dims
  int64_t gs0, gs1, gs2;   // group-id stride of each leading dim (0 = reduced)
  int64_t rows;            // n0*n1*n2
  int64_t n_groups;
  int c, c8, c8p, c8p_shift; // channels, octets per row, lanes per row (pow2)
  int keepc;               // last dim kept (one group per channel) or reduced
  int rows_per_block;
  int bits, qmin, qmax, wpr; // wpr = words per row
  int asym;
  float eps;
};

__global__ void init_ws_kernel(u32 *ws_max, u32 *ws_min, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    ws_max[i] = 0u;
    if (ws_min) ws_min[i] = 0xffffffffu;
  }
}

__device__ __forceinline__ void row_to_idx(const GenParams &p, int64_t r, int64_t &i0, int64_t &i1, int64_t &i2) {
  i2 = r % p.n2;
  int64_t t = r / p.n2;
  i1 = t % p.n1;
  i0 = t / p.n1;
}

// ---- phase A, c % 8 == 0 ---------------------------------------------------
// Lane layout: c8p lanes per row (lanes >= c8 idle), 256/c8p rows per pass.
// Each thread walks rows r0 + k*rowlanes and keeps a running min/max for its
// current group, flushing with atomics when the group changes.  When the whole
// block stayed in one group the flush first goes through LDS so that only one
// thread per column issues atomics.
template <int DT, bool ASYM, bool KEEPC>
__global__ __launch_bounds__(256) void minmax_kernel(GenParams p) {
  constexpr int NV = KEEPC ? 8 : 1;
  __shared__ float lds_mx[256 * NV];
  __shared__ float lds_mn[ASYM ? 256 * NV : 1];

  const int lane_col = threadIdx.x & (p.c8p - 1);
  const int rowlane = threadIdx.x >> p.c8p_shift;
  const int rowlanes = 256 >> p.c8p_shift;
  const bool col_live = lane_col < p.c8;
  const int64_t r_begin = (int64_t)blockIdx.x * p.rows_per_block;
  const int64_t r_end = min(r_begin + p.rows_per_block, p.rows);

  float mx[NV], mn[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) { mx[j] = ASYM ? -INFINITY : 0.f; mn[j] = INFINITY; }
  int64_t cur = -1;
  bool flushed_midway = false;

  auto flush = [&](int64_t g) {
    if (KEEPC) {
      if (!col_live) return;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        atomicMax(&p.ws_max[g + lane_col * 8 + j], ASYM ? enc_ord(mx[j]) : f2u(mx[j]));
        if (ASYM) atomicMin(&p.ws_min[g + lane_col * 8 + j], enc_ord(mn[j]));
      }
    } else if (lane_col == 0) {
      atomicMax(&p.ws_max[g], ASYM ? enc_ord(mx[0]) : f2u(mx[0]));
      if (ASYM) atomicMin(&p.ws_min[g], enc_ord(mn[0]));
    }
  };

  for (int64_t r = r_begin + rowlane; r < r_end; r += rowlanes) {
    int64_t i0, i1, i2;
    row_to_idx(p, r, i0, i1, i2);
    const int64_t g = i0 * p.gs0 + i1 * p.gs1 + i2 * p.gs2;
    if (g != cur) {
      if (cur >= 0) { flush(cur); flushed_midway = true; }
      cur = g;
#pragma unroll
      for (int j = 0; j < NV; ++j) { mx[j] = ASYM ? -INFINITY : 0.f; mn[j] = INFINITY; }
    }
    float v[8];
    if (col_live) In8<DT>::load(p.x, r * p.c + lane_col * 8, v);
    else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = ASYM ? NAN : 0.f;  // fmin/fmax ignore NaN
    }
    if (KEEPC) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (ASYM) { mx[j] = fmaxf(mx[j], v[j]); mn[j] = fminf(mn[j], v[j]); }
        else mx[j] = fmaxf(mx[j], fabsf(v[j]));
      }
    } else {
      float a, b = INFINITY;
      if (ASYM) {
        a = fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7])));
        b = fminf(fminf(fminf(v[0], v[1]), fminf(v[2], v[3])), fminf(fminf(v[4], v[5]), fminf(v[6], v[7])));
      } else {
        a = fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
                  fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7]))));
      }
      // reduce over the lanes of this row (c8p <= 64: a row never spans wavefronts)
      for (int off = 1; off < p.c8p; off <<= 1) {
        a = fmaxf(a, __shfl_xor(a, off, 64));
        if (ASYM) b = fminf(b, __shfl_xor(b, off, 64));
      }
      mx[0] = fmaxf(mx[0], a);
      if (ASYM) mn[0] = fminf(mn[0], b);
    }
  }

  // Was the whole block one group?  (cur is -1 for threads that saw no row.)
  __shared__ long long first_g;
  if (threadIdx.x == 0) first_g = cur;
  __syncthreads();
  const bool uniform = __syncthreads_and(!flushed_midway && (cur == first_g || cur < 0)) && first_g >= 0;

  if (!uniform) {
    if (cur >= 0) flush(cur);
    return;
  }

  // block-uniform: tree through LDS, then one set of atomics
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    lds_mx[j * 256 + threadIdx.x] = (cur >= 0) ? mx[j] : (ASYM ? -INFINITY : 0.f);
    if (ASYM) lds_mn[j * 256 + threadIdx.x] = (cur >= 0) ? mn[j] : INFINITY;
  }
  __syncthreads();
  if (KEEPC) {
    // combine the rowlanes that share a column octet
    if (rowlane == 0 && col_live) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float a = lds_mx[j * 256 + lane_col], b = ASYM ? lds_mn[j * 256 + lane_col] : 0.f;
        for (int rl = 1; rl < rowlanes; ++rl) {
          a = fmaxf(a, lds_mx[j * 256 + rl * p.c8p + lane_col]);
          if (ASYM) b = fminf(b, lds_mn[j * 256 + rl * p.c8p + lane_col]);
        }
        atomicMax(&p.ws_max[first_g + lane_col * 8 + j], ASYM ? enc_ord(a) : f2u(a));
        if (ASYM) atomicMin(&p.ws_min[first_g + lane_col * 8 + j], enc_ord(b));
      }
    }
  } else {
    for (int s = 128; s > 0; s >>= 1) {
      if (threadIdx.x < s) {
        lds_mx[threadIdx.x] = fmaxf(lds_mx[threadIdx.x], lds_mx[threadIdx.x + s]);
        if (ASYM) lds_mn[threadIdx.x] = fminf(lds_mn[threadIdx.x], lds_mn[threadIdx.x + s]);
      }
      __syncthreads();
    }
    if (threadIdx.x == 0) {
      atomicMax(&p.ws_max[first_g], ASYM ? enc_ord(lds_mx[0]) : f2u(lds_mx[0]));
      if (ASYM) atomicMin(&p.ws_min[first_g], enc_ord(lds_mn[0]));
    }
  }
}

// ---- phase A, any c: one thread per element --------------------------------
template <int DT, bool ASYM>
__global__ void minmax_scalar_kernel(GenParams p) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= p.rows * p.c) return;
  const int64_t r = e / p.c;
  const int ch = (int)(e - r * p.c);
  int64_t i0, i1, i2;
  row_to_idx(p, r, i0, i1, i2);
  const int64_t g = i0 * p.gs0 + i1 * p.gs1 + i2 * p.gs2 + (p.keepc ? ch : 0);
  const float v = In8<DT>::load1(p.x, e);
  if (ASYM) {
    atomicMax(&p.ws_max[g], enc_ord(v));
    atomicMin(&p.ws_min[g], enc_ord(v));
  } else {
    atomicMax(&p.ws_max[g], f2u(fabsf(v)));
  }
}

// ---- finalize: min/max -> scale, zero-point --------------------------------
template <bool ASYM>
__global__ void finalize_kernel(GenParams p) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= p.n_groups) return;
  if (ASYM) {
    const float mx = dec_ord(p.ws_max[g]), mn = dec_ord(p.ws_min[g]);
    const float s = fmaxf((mx - mn) / (float)((1 << p.bits) - 1), p.eps);
    p.scale[g] = s;
    p.zp[g] = (float)p.qmin - rintf(mn / s);
  } else {
    p.scale[g] = fmaxf(u2f(p.ws_max[g]) / (float)p.qmax, p.eps);
  }
}

__device__ __forceinline__ int quant_one(float v, float s, float zp, bool asym, float qmin, float qmax) {
  float n = rintf(v / s);
  if (asym) n += zp;
  return (int)__builtin_amdgcn_fmed3f(n, qmin, qmax);
}

// ---- phase B, c % 8 == 0: one thread per octet -----------------------------
template <int DT, bool KEEPC>
__global__ __launch_bounds__(256) void quant_general_kernel(GenParams p) {
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= p.rows * p.c8) return;
  const int64_t r = o / p.c8;
  const int col = (int)(o - r * p.c8);
  int64_t i0, i1, i2;
  row_to_idx(p, r, i0, i1, i2);
  const int64_t g = i0 * p.gs0 + i1 * p.gs1 + i2 * p.gs2 + (KEEPC ? col * 8 : 0);

  float v[8];
  In8<DT>::load(p.x, o * 8, v);
  const float qmin = (float)p.qmin, qmax = (float)p.qmax;
  int q[8];
  if (KEEPC) {
    const float4 *sp = reinterpret_cast<const float4 *>(p.scale + g);  // g % 8 == 0 when c % 8 == 0
    float4 sa = sp[0], sb = sp[1];
    const float s[8] = {sa.x, sa.y, sa.z, sa.w, sb.x, sb.y, sb.z, sb.w};
    float z[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (p.asym) {
      const float4 *zp = reinterpret_cast<const float4 *>(p.zp + g);
      float4 za = zp[0], zb = zp[1];
      z[0] = za.x; z[1] = za.y; z[2] = za.z; z[3] = za.w; z[4] = zb.x; z[5] = zb.y; z[6] = zb.z; z[7] = zb.w;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = quant_one(v[j], s[j], z[j], p.asym, qmin, qmax);
  } else {
    const float s = p.scale[g];
    const float z = p.asym ? p.zp[g] : 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = quant_one(v[j], s, z, p.asym, qmin, qmax);
  }

  if (p.codes) {
    u32 lo = (q[0] & 0xff) | ((q[1] & 0xff) << 8) | ((q[2] & 0xff) << 16) | ((u32)q[3] << 24);
    u32 hi = (q[4] & 0xff) | ((q[5] & 0xff) << 8) | ((q[6] & 0xff) << 16) | ((u32)q[7] << 24);
    *reinterpret_cast<uint2 *>(p.codes + o * 8) = make_uint2(lo, hi);
  }
  if (p.words) {
    const u32 mask = (1u << p.bits) - 1u;
    if (p.bits == 8) {
      u32 lo = (q[0] & 0xff) | ((q[1] & 0xff) << 8) | ((q[2] & 0xff) << 16) | ((u32)q[3] << 24);
      u32 hi = (q[4] & 0xff) | ((q[5] & 0xff) << 8) | ((q[6] & 0xff) << 16) | ((u32)q[7] << 24);
      *reinterpret_cast<uint2 *>(p.words + r * p.wpr + col * 2) = make_uint2(lo, hi);
    } else {
      u32 w = 0;
#pragma unroll
      for (int j = 0; j < 8; ++j) w |= ((u32)q[j] & mask) << (j * p.bits);
      if (p.bits == 4) {
        p.words[r * p.wpr + col] = (int32_t)w;
      } else {  // 2 bits: 16 codes per word = two adjacent octets (c % 16 == 0 on this path)
        u32 other = __shfl_xor(w, 1, 64);
        if ((col & 1) == 0) p.words[r * p.wpr + (col >> 1)] = (int32_t)(w | (other << 16));
      }
    }
  }
}

// ---- phase B, any c: one thread per output word (or per code group) ---------
template <int DT>
__global__ void quant_scalar_kernel(GenParams p) {
  const int vals = p.words ? 32 / p.bits : 4;
  const int wpr = (p.c + vals - 1) / vals;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= p.rows * wpr) return;
  const int64_t r = t / wpr;
  const int wi = (int)(t - r * wpr);
  int64_t i0, i1, i2;
  row_to_idx(p, r, i0, i1, i2);
  const int64_t gb = i0 * p.gs0 + i1 * p.gs1 + i2 * p.gs2;
  const u32 mask = (p.bits == 32) ? ~0u : ((1u << p.bits) - 1u);
  u32 w = 0;
  for (int j = 0; j < vals; ++j) {
    const int ch = wi * vals + j;
    if (ch >= p.c) break;
    const int64_t g = gb + (p.keepc ? ch : 0);
    const int q = quant_one(In8<DT>::load1(p.x, r * p.c + ch), p.scale[g], p.asym ? p.zp[g] : 0.f, p.asym,
                            (float)p.qmin, (float)p.qmax);
    if (p.codes) p.codes[r * p.c + ch] = (int8_t)q;
    w |= ((u32)q & mask) << (j * p.bits);
  }
  if (p.words) p.words[r * wpr + wi] = (int32_t)w;
}

template <int DT>
int run_general(GenParams &p, hipStream_t st) {
  const int64_t ng = p.n_groups;
  hipLaunchKernelGGL(init_ws_kernel, dim3((unsigned)((ng + 255) / 256)), dim3(256), 0, st, p.ws_max,
                     p.asym ? p.ws_min : (u32 *)nullptr, ng);
  const bool fast = (p.c % 8 == 0) && p.c8p <= 64;
  if (fast) {
    const int rowlanes = 256 / p.c8p;
    // aim for a few thousand blocks, at least 8 passes each
    int64_t rpb = (p.rows + 4095) / 4096;
    rpb = ((rpb + rowlanes - 1) / rowlanes) * rowlanes;
    if (rpb < 8 * rowlanes) rpb = 8 * rowlanes;
    p.rows_per_block = (int)rpb;
    dim3 grid((unsigned)((p.rows + rpb - 1) / rpb));
    if (p.asym) {
      if (p.keepc) hipLaunchKernelGGL((minmax_kernel<DT, true, true>), grid, dim3(256), 0, st, p);
      else hipLaunchKernelGGL((minmax_kernel<DT, true, false>), grid, dim3(256), 0, st, p);
    } else {
      if (p.keepc) hipLaunchKernelGGL((minmax_kernel<DT, false, true>), grid, dim3(256), 0, st, p);
      else hipLaunchKernelGGL((minmax_kernel<DT, false, false>), grid, dim3(256), 0, st, p);
    }
  } else {
    const int64_t n = p.rows * p.c;
    dim3 grid((unsigned)((n + 255) / 256));
    if (p.asym) hipLaunchKernelGGL((minmax_scalar_kernel<DT, true>), grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((minmax_scalar_kernel<DT, false>), grid, dim3(256), 0, st, p);
  }
  {
    dim3 grid((unsigned)((ng + 255) / 256));
    if (p.asym) hipLaunchKernelGGL((finalize_kernel<true>), grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((finalize_kernel<false>), grid, dim3(256), 0, st, p);
  }
  const bool fast_b = (p.c % 8 == 0) && (!p.words || (p.c * p.bits) % 32 == 0);
  if (fast_b) {
    const int64_t n = p.rows * p.c8;
    dim3 grid((unsigned)((n + 255) / 256));
    if (p.keepc) hipLaunchKernelGGL((quant_general_kernel<DT, true>), grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((quant_general_kernel<DT, false>), grid, dim3(256), 0, st, p);
  } else {
    const int vals = p.words ? 32 / p.bits : 4;
    const int64_t n = p.rows * ((p.c + vals - 1) / vals);
    dim3 grid((unsigned)((n + 255) / 256));
    hipLaunchKernelGGL((quant_scalar_kernel<DT>), grid, dim3(256), 0, st, p);
  }
  return 0;
}

int64_t count_groups(const int64_t *s, int reduce_mask) {
  int64_t n = 1;
  for (int d = 0; d < 4; ++d)
    if (!(reduce_mask & (1 << d))) n *= s[d];
  return n;
}

}  // namespace

extern "C" size_t varq_quant_workspace_bytes(const int64_t *host_shape4, int reduce_mask) {
  if (!host_shape4) return 0;
  return (size_t)count_groups(host_shape4, reduce_mask) * 2 * sizeof(u32);
}

extern "C" int varq_quant_pack(const void *x, int x_dtype, const int64_t *host_shape4, int reduce_mask, int bits,
                               int asym, float eps, int32_t *words, int8_t *codes, float *scale, float *zp,
                               void *workspace, size_t workspace_bytes, void *stream) {
  VARQ_CHECK_ARG(host_shape4, "quant_pack: null shape");
  const int64_t *s = host_shape4;
  VARQ_CHECK_ARG(s[0] >= 0 && s[1] >= 0 && s[2] >= 0 && s[3] > 0 && s[3] <= (1 << 20), "quant_pack: bad shape");
  VARQ_CHECK_ARG(x_dtype >= 0 && x_dtype <= 2, "quant_pack: bad dtype %d", x_dtype);
  VARQ_CHECK_ARG(reduce_mask >= 0 && reduce_mask < 16, "quant_pack: bad reduce mask");
  VARQ_CHECK_ARG(bits > 1 && bits <= 8, "quant_pack: bits must be in 2..8 (got %d)", bits);
  VARQ_CHECK_ARG(!words || bits == 2 || bits == 4 || bits == 8, "quant_pack: packing implements 2/4/8 bits only (got %d)", bits);
  const int64_t rows = s[0] * s[1] * s[2];
  if (rows == 0) return VARQ_OK;
  VARQ_CHECK_ARG(words || codes, "quant_pack: no output requested");
  VARQ_CHECK_ARG(scale && (!asym || zp), "quant_pack: scale/zp output missing");
  VARQ_CHECK_ARG(x && workspace, "quant_pack: null pointer");
  const int64_t ng = count_groups(s, reduce_mask);
  if (workspace_bytes < (size_t)ng * 2 * sizeof(u32))
    return varq_set_error(VARQ_ERR_WORKSPACE, "quant_pack: workspace %zu < %zu bytes", workspace_bytes,
                          (size_t)ng * 2 * sizeof(u32));
  VARQ_CHECK_ARG(rows * s[3] < (1ll << 40), "quant_pack: tensor too large");

  GenParams p;
  p.x = x;
  p.ws_max = reinterpret_cast<u32 *>(workspace);
  p.ws_min = p.ws_max + ng;
  p.scale = scale; p.zp = zp; p.words = words; p.codes = codes;
  p.n0 = s[0]; p.n1 = s[1]; p.n2 = s[2];
  p.c = (int)s[3];
  p.keepc = !(reduce_mask & 8);
  // group-id strides of the kept leading dims, row-major over the kept dims
  int64_t stride = p.keepc ? p.c : 1;
  p.gs2 = (reduce_mask & 4) ? 0 : stride; if (!(reduce_mask & 4)) stride *= s[2];
  p.gs1 = (reduce_mask & 2) ? 0 : stride; if (!(reduce_mask & 2)) stride *= s[1];
  p.gs0 = (reduce_mask & 1) ? 0 : stride;
  p.rows = rows;
  p.n_groups = ng;
  p.c8 = (p.c + 7) / 8;
  int c8p = 1, sh = 0;
  while (c8p < p.c8) { c8p <<= 1; ++sh; }
  p.c8p = c8p; p.c8p_shift = sh;
  p.rows_per_block = 0;
  p.bits = bits; p.qmin = -(1 << (bits - 1)); p.qmax = (1 << (bits - 1)) - 1;
  p.wpr = words ? (p.c + 32 / bits - 1) / (32 / bits) : 0;
  p.asym = asym ? 1 : 0;
  p.eps = eps;
  hipStream_t st = (hipStream_t)stream;
  if (x_dtype == VARQ_F32) run_general<VARQ_F32>(p, st);
  else if (x_dtype == VARQ_BF16) run_general<VARQ_BF16>(p, st);
  else run_general<VARQ_F16>(p, st);
  VARQ_CHECK_LAUNCH("quant_pack");
  return VARQ_OK;
}

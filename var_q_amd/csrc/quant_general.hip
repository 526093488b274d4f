// General two-phase quantizer: groups that span rows (the six grouping methods
// of VAR_Q/quant.py:75-95, which all reduce over the batch dim, plus any other
// reduce set).  A single HBM read cannot serve such groups, so:
//   phase A  group min/max (or max-abs): one partial per (chunk, group) in the
//            workspace, no atomics (tiled path below)
//   finalize fold the partials -> scale / zero-point      (VAR_Q/quant.py:112-116)
//   phase B  re-read input (L2 / Infinity-Cache resident for KV-sized tensors),
//            divide, round half-to-even, clamp, pack    (VAR_Q/quant.py:118-121,
//            VAR_Q/pack_unpack.py:177-196)
// min/max are exactly associative, so the result does not depend on the order
// in which partial results meet.  Channel counts that are not a multiple of 8 and
// rows wider than 512 channels take scalar kernels with ordered-integer atomics.
#include "varq_common.h"
#include <mutex>

#ifndef VARQ_GEN_NRO_MIN
#define VARQ_GEN_NRO_MIN 256
#endif
#ifndef VARQ_FIN_THREADS
#define VARQ_FIN_THREADS 65536
#endif
#ifndef VARQ_GEN_BLOCKS
#define VARQ_GEN_BLOCKS 2048
#endif

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
  // Output rows (codes / words) may land in a larger buffer: input row r goes to output row
  // r + (r / out_inner) * out_delta + out_off -- a step [B,H,n,c] into tokens len.. of a cache
  // [B,H,cap,..] is (n, cap - n, len), a step [B,n,H,c] into [B,cap,H,..] is (n*H, (cap - n)*H, len*H).
  int out_mapped;
  int64_t out_inner, out_delta, out_off;
  // a second tensor of the same shape in the same launches (blockIdx.y == 1): its input,
  // its outputs and the distance (in 4-byte words) to its part of the workspace
  const void *x1;
  float *scale1, *zp1;
  int32_t *words1;
  int8_t *codes1;
  int64_t ws1;
};

// the tensor a workgroup of the tiled kernels works on
__device__ __forceinline__ bool take_second(GenParams &p) {
  if (blockIdx.y == 0) return false;
  p.x = p.x1; p.scale = p.scale1; p.zp = p.zp1; p.words = p.words1; p.codes = p.codes1;
  return true;
}

__device__ __forceinline__ int64_t out_row(const GenParams &p, int64_t row) {
  return p.out_mapped ? row + (row / p.out_inner) * p.out_delta + p.out_off : row;
}
// (rows of the tiled kernels fit 31 bits)
__device__ __forceinline__ int64_t out_row32(const GenParams &p, int64_t row) {
  return p.out_mapped ? row + (int64_t)((u32)row / (u32)p.out_inner) * p.out_delta + p.out_off : row;
}

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

// ---- fast path (c % 8 == 0, at most 512 channels): tiled, atomic-free -------------
// The leading dims are brought to a canonical form on the host (Plan): a linear
// index `ko` over kept outer dims, a linear index `ro` over reduced outer dims,
// and along contiguous rows either a kept extent Q (d2 kept) or a reduced extent
// RI (d2 reduced):
//     row   = ko*ko_rs + ro*ro_rs + (q | ri)
//     group = ko*ko_gs + q*q_gs  (+ channel when the channel dim is kept)
// A workgroup is 256 threads = R row lanes x c8p column lanes (8 channels each) and
// owns one (ko, tile of Q, chunk z of the reduced steps).  Every thread sees a
// single group (per channel) for its whole life: no group lookups and no integer
// divisions in the loop.  Phase A leaves one partial min/max per (z, group) in the
// workspace (plain stores, each written exactly once), the finalize kernel folds
// the Z partials, phase B walks the same decomposition with the group's scale,
// reciprocal and zero-point in registers.
struct Plan {
  int64_t ko_rs, ro_rs, ko_gs, q_gs;
  int nko, nro, Q, RI;
  int lanesQ, sub, tilesQ;     // row lanes spent on q; positions folded into the rest; tiles over Q
  int fold_ro;                 // 1: the spare row lanes fold consecutive ro (RI == 1), 0: consecutive rows of RI
  int T;                       // steps per ro along RI (inner reduced), 1 when d2 is kept
  int steps, Z, steps_per_chunk;
  int R, c8, c8p, shift;
};

// decode the workgroup and lane; returns false for an idle lane
struct Lane {
  int ko, q, f, col, z;
  bool live;
};
__device__ __forceinline__ Lane decode(const Plan &pl) {
  Lane l;
  const int bid = blockIdx.x;
  l.z = bid % pl.Z;
  const int kb = bid / pl.Z;
  const int tq = kb % pl.tilesQ;
  l.ko = kb / pl.tilesQ;
  l.col = threadIdx.x & (pl.c8p - 1);
  const int rowlane = threadIdx.x >> pl.shift;
  const int lq = rowlane % pl.lanesQ;
  l.f = rowlane / pl.lanesQ;
  l.q = tq * pl.lanesQ + lq;
  l.live = l.col < pl.c8 && l.f < pl.sub && l.q < pl.Q;
  return l;
}

// Calls body(row, v) for every row of this thread, in step order, with the row's 8 values of
// this lane's octet.
template <int DT, typename F>
__device__ __forceinline__ void for_rows(const GenParams &p, const Plan &pl, const Lane &l, F body) {
  const int s0 = l.z * pl.steps_per_chunk, s1 = min(s0 + pl.steps_per_chunk, pl.steps);
  const int64_t base = (int64_t)l.ko * pl.ko_rs + l.q;
  const int64_t col8 = l.col * 8;
  // (one load in flight per lane: issuing two steps' loads before either is used, or the next
  // row's load ahead of the current row's arithmetic, was measured 5-15 % slower on both phases)
  if (pl.fold_ro) {
    // d2 kept: a step is `sub` consecutive reduced positions
    for (int s = s0; s < s1; ++s) {
      const int ro = s * pl.sub + l.f;
      if (ro < pl.nro) {
        const int64_t r = base + (int64_t)ro * pl.ro_rs;
        float v[8];
        In8<DT>::load(p.x, r * p.c + col8, v);
        body(r, v);
      }
    }
  } else {
    // d2 reduced: a step is `sub` (= R) consecutive rows of one ro
    int ro = s0 / pl.T, t = s0 - ro * pl.T;
    for (int s = s0; s < s1; ++s) {
      const int ri = t * pl.sub + l.f;
      if (ri < pl.RI) {
        const int64_t r = base + (int64_t)ro * pl.ro_rs + ri;
        float v[8];
        In8<DT>::load(p.x, r * p.c + col8, v);
        body(r, v);
      }
      if (++t == pl.T) { t = 0; ++ro; }
    }
  }
}

template <int DT, bool ASYM, bool KEEPC>
__global__ __launch_bounds__(256) void minmax_tiled_kernel(GenParams p, Plan pl, float *part_max, float *part_min) {
  constexpr int NV = KEEPC ? 8 : 1;
  __shared__ float lds_mx[256 * NV];
  __shared__ float lds_mn[ASYM ? 256 * NV : 1];
  if (take_second(p)) { part_max += p.ws1; part_min += p.ws1; }
  const Lane l = decode(pl);
  float mx[NV], mn[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) { mx[j] = ASYM ? -INFINITY : 0.f; mn[j] = INFINITY; }
  if (l.live) {
    for_rows<DT>(p, pl, l, [&](int64_t, const float (&v)[8]) {
      if (KEEPC) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (ASYM) { mx[j] = fmaxf(mx[j], v[j]); mn[j] = fminf(mn[j], v[j]); }
          else mx[j] = fmaxf(mx[j], fabsf(v[j]));
        }
      } else if (ASYM) {
        mx[0] = fmaxf(mx[0], fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7]))));
        mn[0] = fminf(mn[0], fminf(fminf(fminf(v[0], v[1]), fminf(v[2], v[3])), fminf(fminf(v[4], v[5]), fminf(v[6], v[7]))));
      } else {
        mx[0] = fmaxf(mx[0], fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
                                   fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7])))));
      }
    });
  }
  if (!KEEPC) {
    // fold the column lanes of a row (c8p <= 64: a row never spans wavefronts; idle lanes hold the identity)
    for (int off = 1; off < pl.c8p; off <<= 1) {
      mx[0] = fmaxf(mx[0], __shfl_xor(mx[0], off, 64));
      if (ASYM) mn[0] = fminf(mn[0], __shfl_xor(mn[0], off, 64));
    }
  }
  // fold the `sub` row lanes that share q (lane index = (f*lanesQ + lq)*c8p + col, so the
  // positions f of one (q, col) lie `stride` lanes apart): inside a wavefront by lane exchanges
  // when the stride is a power of two below 64, the rest -- at most one value per wavefront
  // then -- through LDS.  (Idle lanes hold the identity of max / min.)
  if (pl.sub > 1) {
    const int stride = pl.lanesQ * pl.c8p;
    int fstep = 1;                       // distance in f between the values still to fold
    if (stride < 64 && (stride & (stride - 1)) == 0) {
      for (int off = stride; off < 64; off <<= 1) {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
          mx[j] = fmaxf(mx[j], __shfl_xor(mx[j], off, 64));
          if (ASYM) mn[j] = fminf(mn[j], __shfl_xor(mn[j], off, 64));
        }
      }
      fstep = 64 / stride;
    }
    if (fstep < pl.sub) {
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        lds_mx[j * 256 + threadIdx.x] = mx[j];
        if (ASYM) lds_mn[j * 256 + threadIdx.x] = mn[j];
      }
      __syncthreads();
      if (l.f == 0) {
        for (int f = fstep; f < pl.sub; f += fstep)
#pragma unroll
          for (int j = 0; j < NV; ++j) {
            mx[j] = fmaxf(mx[j], lds_mx[j * 256 + threadIdx.x + f * stride]);
            if (ASYM) mn[j] = fminf(mn[j], lds_mn[j * 256 + threadIdx.x + f * stride]);
          }
      }
    }
  }
  if (l.f != 0 || l.q >= pl.Q || l.col >= pl.c8 || (!KEEPC && l.col != 0)) return;
  const int64_t g = (int64_t)l.ko * pl.ko_gs + (int64_t)l.q * pl.q_gs + (KEEPC ? l.col * 8 : 0);
  float *dmx = part_max + (int64_t)l.z * p.n_groups + g;
  float *dmn = part_min + (int64_t)l.z * p.n_groups + g;
  if (KEEPC) {
    reinterpret_cast<float4 *>(dmx)[0] = make_float4(mx[0], mx[1], mx[2], mx[3]);
    reinterpret_cast<float4 *>(dmx)[1] = make_float4(mx[4 % NV], mx[5 % NV], mx[6 % NV], mx[7 % NV]);
    if (ASYM) {
      reinterpret_cast<float4 *>(dmn)[0] = make_float4(mn[0], mn[1], mn[2], mn[3]);
      reinterpret_cast<float4 *>(dmn)[1] = make_float4(mn[4 % NV], mn[5 % NV], mn[6 % NV], mn[7 % NV]);
    }
  } else {
    dmx[0] = mx[0];
    if (ASYM) dmn[0] = mn[0];
  }
}

// partials -> scale, zero-point, reciprocal and the flag of the exact-quotient shortcut.
// 256 threads = ZL z-lanes x 256/ZL adjacent groups; the z-lanes of a group meet in LDS.
template <bool ASYM>
__global__ __launch_bounds__(256) void finalize_tiled_kernel(GenParams p, int Z, int ZL, const float *part_max,
                                                             const float *part_min, float *rinv, u32 *plain) {
  __shared__ float lds_mx[256];
  __shared__ float lds_mn[256];
  if (take_second(p)) { part_max += p.ws1; part_min += p.ws1; rinv += p.ws1; plain += p.ws1; }
  const int gpb = 256 / ZL;                       // groups per block
  const int gl = threadIdx.x % gpb, zl = threadIdx.x / gpb;
  const int64_t g = (int64_t)blockIdx.x * gpb + gl;
  float mx = ASYM ? -INFINITY : 0.f, mn = INFINITY;
  if (g < p.n_groups) {
    for (int z = zl; z < Z; z += ZL) {
      mx = fmaxf(mx, part_max[(int64_t)z * p.n_groups + g]);
      if (ASYM) mn = fminf(mn, part_min[(int64_t)z * p.n_groups + g]);
    }
  }
  lds_mx[threadIdx.x] = mx;
  lds_mn[threadIdx.x] = mn;
  __syncthreads();
  for (int h = ZL >> 1; h > 0; h >>= 1) {
    if (zl < h) {
      lds_mx[threadIdx.x] = fmaxf(lds_mx[threadIdx.x], lds_mx[threadIdx.x + h * gpb]);
      lds_mn[threadIdx.x] = fminf(lds_mn[threadIdx.x], lds_mn[threadIdx.x + h * gpb]);
    }
    __syncthreads();
  }
  if (zl != 0 || g >= p.n_groups) return;
  mx = lds_mx[threadIdx.x];
  mn = lds_mn[threadIdx.x];
  float s;
  if (ASYM) {
    s = fmaxf((mx - mn) / (float)((1 << p.bits) - 1), p.eps);
    p.zp[g] = (float)p.qmin - rintf(mn / s);
  } else {
    s = fmaxf(mx / (float)p.qmax, p.eps);
  }
  p.scale[g] = s;
  rinv[g] = 1.0f / s;
  // x/s == RN(q0 + (x - q0*s)*r) with q0 = RN(x*r), r = RN(1/s), for every finite x unless the
  // significand of s is all ones or the residual can underflow
  plain[g] = (s > 0x1p-96f && s < 0x1p96f && (f2u(s) & 0x7fffffu) != 0x7fffffu) ? 1u : 0u;
}

template <int DT, bool KEEPC>
__global__ __launch_bounds__(256) void quant_tiled_kernel(GenParams p, Plan pl, const float *rinv, const u32 *plain) {
  constexpr int NV = KEEPC ? 8 : 1;
  if (take_second(p)) { rinv += p.ws1; plain += p.ws1; }
  const Lane l = decode(pl);
  // 2-bit words are assembled from two adjacent column lanes: idle lanes must still reach the shuffle
  const bool live = l.live;
  const int64_t g = (int64_t)l.ko * pl.ko_gs + (int64_t)(live ? l.q : 0) * pl.q_gs + (KEEPC ? (live ? l.col : 0) * 8 : 0);
  float s[NV], r[NV], z[NV];
  bool all_plain = true;
  if constexpr (KEEPC) {
    // the lane's eight groups are adjacent and start at a multiple of 8: 16-byte loads (the
    // workspace and the outputs are 16-byte aligned; checked on the host)
    auto ld8 = [&](const float *src, float (&dst)[NV]) {
      const float4 a = reinterpret_cast<const float4 *>(src + g)[0], b = reinterpret_cast<const float4 *>(src + g)[1];
      dst[0] = a.x; dst[1] = a.y; dst[2] = a.z; dst[3] = a.w; dst[4 % NV] = b.x; dst[5 % NV] = b.y; dst[6 % NV] = b.z; dst[7 % NV] = b.w;
    };
    ld8(p.scale, s);
    ld8(rinv, r);
    if (p.asym) ld8(p.zp, z);
    else {
#pragma unroll
      for (int j = 0; j < NV; ++j) z[j] = 0.f;
    }
    const uint4 pa = reinterpret_cast<const uint4 *>(plain + g)[0], pb = reinterpret_cast<const uint4 *>(plain + g)[1];
    all_plain = (pa.x & pa.y & pa.z & pa.w & pb.x & pb.y & pb.z & pb.w) != 0u;
  } else {
    s[0] = p.scale[g];
    r[0] = rinv[g];
    z[0] = p.asym ? p.zp[g] : 0.f;
    all_plain = plain[g] != 0u;
  }
  const float qmin = (float)p.qmin, qmax = (float)p.qmax;
  const u32 mask = (1u << p.bits) - 1u;
  if (!live) return;   // (only the 2-bit path shuffles, and there c8 is even: partners are live together)
  for_rows<DT>(p, pl, l, [&](int64_t row, const float (&v)[8]) {
    int q[8];
    if (all_plain) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float sj = s[j % NV], rj = r[j % NV];
        const float q0 = v[j] * rj;
        const float t = __builtin_fmaf(__builtin_fmaf(-q0, sj, v[j]), rj, q0);
        q[j] = (int)__builtin_amdgcn_fmed3f(rintf(t) + z[j % NV], qmin, qmax);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) q[j] = (int)__builtin_amdgcn_fmed3f(rintf(v[j] / s[j % NV]) + z[j % NV], qmin, qmax);
    }
    const int64_t orow = out_row32(p, row);
    const int64_t o = orow * p.c8 + l.col;
    if (p.codes) {
      u32 lo = (q[0] & 0xff) | ((q[1] & 0xff) << 8) | ((q[2] & 0xff) << 16) | ((u32)q[3] << 24);
      u32 hi = (q[4] & 0xff) | ((q[5] & 0xff) << 8) | ((q[6] & 0xff) << 16) | ((u32)q[7] << 24);
      *reinterpret_cast<uint2 *>(p.codes + o * 8) = make_uint2(lo, hi);
    }
    if (p.words) {
      if (p.bits == 8) {
        u32 lo = (q[0] & 0xff) | ((q[1] & 0xff) << 8) | ((q[2] & 0xff) << 16) | ((u32)q[3] << 24);
        u32 hi = (q[4] & 0xff) | ((q[5] & 0xff) << 8) | ((q[6] & 0xff) << 16) | ((u32)q[7] << 24);
        *reinterpret_cast<uint2 *>(p.words + orow * p.wpr + l.col * 2) = make_uint2(lo, hi);
      } else {
        u32 w = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) w |= ((u32)q[j] & mask) << (j * p.bits);
        if (p.bits == 4) {
          p.words[orow * p.wpr + l.col] = (int32_t)w;
        } else {  // 2 bits: 16 codes per word = two adjacent octets (c % 16 == 0 on this path)
          u32 other = __shfl_xor(w, 1, 64);
          if ((l.col & 1) == 0) p.words[orow * p.wpr + (l.col >> 1)] = (int32_t)(w | (other << 16));
        }
      }
    }
  });
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
    if (p.codes) p.codes[out_row(p, r) * p.c + ch] = (int8_t)q;
    w |= ((u32)q & mask) << (j * p.bits);
  }
  if (p.words) p.words[out_row(p, r) * wpr + wi] = (int32_t)w;
}

// Host side of the tiled path: canonical form of the leading dims and the launch shape.
// Returns false when the shape needs the scalar kernels.
bool make_plan(const int64_t *sh, int reduce_mask, int64_t n_groups, Plan &pl) {
  const int64_t n0 = sh[0], n1 = sh[1], n2 = sh[2], c = sh[3];
  const int64_t rows = n0 * n1 * n2;
  if (c % 8 != 0 || rows <= 0 || rows >= (1ll << 31) - 512) return false;
  pl.c8 = (int)(c / 8);
  int c8p = 1, shl = 0;
  while (c8p < pl.c8) { c8p <<= 1; ++shl; }
  if (c8p > 64) return false;
  pl.c8p = c8p; pl.shift = shl; pl.R = 256 / c8p;
  const bool k0 = !(reduce_mask & 1), k1 = !(reduce_mask & 2), k2 = !(reduce_mask & 4), kc = !(reduce_mask & 8);
  int64_t stride = kc ? c : 1;
  const int64_t gs2 = k2 ? stride : 0; if (k2) stride *= n2;
  const int64_t gs1 = k1 ? stride : 0; if (k1) stride *= n1;
  const int64_t gs0 = k0 ? stride : 0;
  int64_t nko = 1, nro = 1, Q = 1, RI = 1;
  pl.ko_rs = pl.ro_rs = pl.ko_gs = pl.q_gs = 0;
  if (k2) {
    Q = n2; pl.q_gs = gs2;
    if (k1) {
      Q = n1 * n2;                                   // gs1 == gs2 * n2: q runs over (i1, i2)
      if (k0) Q = rows;                              // every row its own group
      else { nro = n0; pl.ro_rs = n1 * n2; }
    } else if (k0) { nko = n0; pl.ko_rs = n1 * n2; pl.ko_gs = gs0; nro = n1; pl.ro_rs = n2; }
    else { nro = n0 * n1; pl.ro_rs = n2; }
  } else {
    RI = n2;
    if (!k1) {
      RI = n1 * n2;
      if (!k0) RI = rows;
      else { nko = n0; pl.ko_rs = n1 * n2; pl.ko_gs = gs0; }
    } else if (k0) { nko = n0 * n1; pl.ko_rs = n2; pl.ko_gs = gs1; }     // gs0 == gs1 * n1
    else { nko = n1; pl.ko_rs = n2; pl.ko_gs = gs1; nro = n0; pl.ro_rs = n1 * n2; }
  }
  pl.nko = (int)nko; pl.nro = (int)nro; pl.Q = (int)Q; pl.RI = (int)RI;
  pl.lanesQ = (int)(Q < pl.R ? Q : pl.R);
  if (RI == 1 && nro >= VARQ_GEN_NRO_MIN) {
    // Groups indexed by the innermost leading dim, many reduced rows each (the reference's default
    // method in layout BLHc): few row lanes on q -- rows of at least 128 channels per wavefront
    // segment -- and the others on consecutive reduced rows, which fold inside the workgroup.  More
    // tiles over q, hence fewer chunks and fewer partials for the finalize kernel to fold.
    int cap = 1;
    while (cap * 2 * c <= 128) cap *= 2;
    if (pl.lanesQ > cap) pl.lanesQ = cap;
  }
  pl.sub = pl.R / pl.lanesQ;
  pl.tilesQ = (int)((Q + pl.lanesQ - 1) / pl.lanesQ);
  pl.fold_ro = (RI == 1);
  int64_t steps;
  if (pl.fold_ro) { pl.T = 1; steps = (nro + pl.sub - 1) / pl.sub; }
  else { pl.T = (int)((RI + pl.sub - 1) / pl.sub); steps = nro * pl.T; }
  const int64_t kept_blocks = nko * pl.tilesQ;
  int64_t Z = (VARQ_GEN_BLOCKS + kept_blocks - 1) / kept_blocks;
  const int64_t zcap = (8ll << 20) / (n_groups > 0 ? n_groups : 1);   // partials stay below 64 MiB
  if (Z > zcap) Z = zcap;
  // ... and below a sixteenth of the input: with few kept blocks (groups indexed by the
  // innermost leading dim only, the BLHc layouts) thousands of chunks would write and re-read
  // as many partials as half the tensor
  const int64_t zvol = rows * c / (16 * (n_groups > 0 ? n_groups : 1));
  if (Z > zvol) Z = zvol;
  if (Z > steps) Z = steps;
  if (Z < 1) Z = 1;
  const int64_t spc = (steps + Z - 1) / Z;
  Z = (steps + spc - 1) / spc;                     // no empty chunk: every (z, group) partial gets written
  if (steps >= (1ll << 31) || kept_blocks * Z >= (1ll << 31)) return false;
  pl.steps = (int)steps; pl.Z = (int)Z; pl.steps_per_chunk = (int)spc;
  return true;
}

size_t plan_workspace_bytes(const Plan &pl, int64_t n_groups) {
  return (size_t)n_groups * (2 + 2 * (size_t)pl.Z) * sizeof(float);
}

template <int DT>
int run_tiled(GenParams &p, const Plan &pl, void *workspace, hipStream_t st) {
  const int64_t ng = p.n_groups;
  float *rinv = reinterpret_cast<float *>(workspace);
  u32 *plain = reinterpret_cast<u32 *>(rinv + ng);
  float *part_max = rinv + 2 * ng;
  float *part_min = part_max + (int64_t)pl.Z * ng;
  const unsigned nt = p.x1 ? 2u : 1u;   // tensors per launch (grid.y)
  p.ws1 = (int64_t)(plan_workspace_bytes(pl, ng) / sizeof(float));
  dim3 grid((unsigned)((int64_t)pl.nko * pl.tilesQ * pl.Z), nt);
  if (p.asym) {
    if (p.keepc) hipLaunchKernelGGL((minmax_tiled_kernel<DT, true, true>), grid, dim3(256), 0, st, p, pl, part_max, part_min);
    else hipLaunchKernelGGL((minmax_tiled_kernel<DT, true, false>), grid, dim3(256), 0, st, p, pl, part_max, part_min);
  } else {
    if (p.keepc) hipLaunchKernelGGL((minmax_tiled_kernel<DT, false, true>), grid, dim3(256), 0, st, p, pl, part_max, part_min);
    else hipLaunchKernelGGL((minmax_tiled_kernel<DT, false, false>), grid, dim3(256), 0, st, p, pl, part_max, part_min);
  }
  // z-lanes per group in the finalize kernel: enough threads in total, no more lanes than partials
  int ZL = 1;
  while (ZL < 256 && ZL < pl.Z && ng * ZL < VARQ_FIN_THREADS) ZL <<= 1;
  dim3 fgrid((unsigned)((ng + 256 / ZL - 1) / (256 / ZL)), nt);
  if (p.asym)
    hipLaunchKernelGGL((finalize_tiled_kernel<true>), fgrid, dim3(256), 0, st, p, pl.Z, ZL, part_max, part_min, rinv, plain);
  else
    hipLaunchKernelGGL((finalize_tiled_kernel<false>), fgrid, dim3(256), 0, st, p, pl.Z, ZL, part_max, part_min, rinv, plain);
  // phase B walks the same chunks (its per-thread parameters are eight 16-byte loads; chunks of 4 to 8 steps
  // per thread measured alike, longer ones slower)
  const Plan &pb = pl;
  dim3 bgrid((unsigned)((int64_t)pb.nko * pb.tilesQ * pb.Z), nt);
  if (p.keepc) hipLaunchKernelGGL((quant_tiled_kernel<DT, true>), bgrid, dim3(256), 0, st, p, pb, rinv, plain);
  else hipLaunchKernelGGL((quant_tiled_kernel<DT, false>), bgrid, dim3(256), 0, st, p, pb, rinv, plain);
  return 0;
}

// any shape: one thread per element / per output word, group min/max by ordered-integer atomics
template <int DT>
int run_general(GenParams &p, hipStream_t st) {
  const int64_t ng = p.n_groups;
  hipLaunchKernelGGL(init_ws_kernel, dim3((unsigned)((ng + 255) / 256)), dim3(256), 0, st, p.ws_max,
                     p.asym ? p.ws_min : (u32 *)nullptr, ng);
  {
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
  {
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
  const int64_t ng = count_groups(host_shape4, reduce_mask);
  Plan pl;
  if (make_plan(host_shape4, reduce_mask, ng, pl)) return plan_workspace_bytes(pl, ng);
  return (size_t)ng * 2 * sizeof(u32);
}

namespace {
// x1 != NULL: a second tensor of the same shape with its own outputs, in the same launches
// where the tiled kernels apply, one after the other through the same workspace otherwise
int quant_pack_impl(const void *x, const void *x1, int x_dtype, const int64_t *host_shape4, int reduce_mask, int bits,
                    int asym, float eps, int32_t *words, int8_t *codes, float *scale, float *zp,
                    int32_t *words1, int8_t *codes1, float *scale1, float *zp1,
                    const int64_t *host_out_map, void *workspace, size_t workspace_bytes, void *stream) {
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
  if (x1) {
    VARQ_CHECK_ARG((!words == !words1) && (!codes == !codes1) && scale1 && (!asym || zp1),
                   "quant_pack: the second tensor needs the same kinds of output as the first");
  }
  const int64_t ng = count_groups(s, reduce_mask);
  Plan pl;
  // the tiled kernels pack whole words per octet: c*bits must fill words (always true for 4 and 8 bits)
  const bool tiled = make_plan(s, reduce_mask, ng, pl) && (!words || (s[3] * bits) % 32 == 0);
  const size_t need = tiled ? plan_workspace_bytes(pl, ng) * (x1 ? 2 : 1) : (size_t)ng * 2 * sizeof(u32);
  if (workspace_bytes < need)
    return varq_set_error(VARQ_ERR_WORKSPACE, "quant_pack: workspace %zu < %zu bytes", workspace_bytes, need);
  VARQ_CHECK_ARG(rows * s[3] < (1ll << 40), "quant_pack: tensor too large");
  // only the tiled kernels that keep the channel dim move scales, zero-points and partials in
  // 16-byte pieces; every other path reads and writes them one word at a time
  const uintptr_t par_align = (tiled && !(reduce_mask & 8)) ? 15 : 3;
  VARQ_CHECK_ARG((((uintptr_t)workspace | (uintptr_t)scale | (uintptr_t)zp | (uintptr_t)scale1 | (uintptr_t)zp1) & par_align) == 0,
                 "quant_pack: scale, zp and workspace must be %d-byte aligned for this shape", (int)par_align + 1);

  GenParams p;
  p.x = x;
  p.ws_max = reinterpret_cast<u32 *>(workspace);
  p.ws_min = p.ws_max + ng;
  p.scale = scale; p.zp = zp; p.words = words; p.codes = codes;
  p.x1 = nullptr; p.scale1 = nullptr; p.zp1 = nullptr; p.words1 = nullptr; p.codes1 = nullptr; p.ws1 = 0;
  p.out_mapped = 0; p.out_inner = 1; p.out_delta = 0; p.out_off = 0;
  if (host_out_map) {
    VARQ_CHECK_ARG(host_out_map[0] > 0 && host_out_map[1] >= 0 && host_out_map[2] >= 0 && rows % host_out_map[0] == 0,
                   "quant_pack: output map {rows per block, extra rows per block, first row} = {%lld, %lld, %lld} does not fit %lld rows",
                   (long long)host_out_map[0], (long long)host_out_map[1], (long long)host_out_map[2], (long long)rows);
    p.out_mapped = 1; p.out_inner = host_out_map[0]; p.out_delta = host_out_map[1]; p.out_off = host_out_map[2];
  }
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
  if (tiled) {
    if (x1) { p.x1 = x1; p.scale1 = scale1; p.zp1 = zp1; p.words1 = words1; p.codes1 = codes1; }
    if (x_dtype == VARQ_F32) run_tiled<VARQ_F32>(p, pl, workspace, st);
    else if (x_dtype == VARQ_BF16) run_tiled<VARQ_BF16>(p, pl, workspace, st);
    else run_tiled<VARQ_F16>(p, pl, workspace, st);
  } else {
    for (int t = 0; t < (x1 ? 2 : 1); ++t) {   // stream order keeps the shared workspace safe
      if (t == 1) { p.x = x1; p.scale = scale1; p.zp = zp1; p.words = words1; p.codes = codes1; }
      if (x_dtype == VARQ_F32) run_general<VARQ_F32>(p, st);
      else if (x_dtype == VARQ_BF16) run_general<VARQ_BF16>(p, st);
      else run_general<VARQ_F16>(p, st);
    }
  }
  VARQ_CHECK_LAUNCH("quant_pack");
  return VARQ_OK;
}
}  // namespace

extern "C" int varq_quant_pack(const void *x, int x_dtype, const int64_t *host_shape4, int reduce_mask, int bits,
                               int asym, float eps, int32_t *words, int8_t *codes, float *scale, float *zp,
                               const int64_t *host_out_map, void *workspace, size_t workspace_bytes, void *stream) {
  return quant_pack_impl(x, nullptr, x_dtype, host_shape4, reduce_mask, bits, asym, eps, words, codes, scale, zp,
                         nullptr, nullptr, nullptr, nullptr, host_out_map, workspace, workspace_bytes, stream);
}

extern "C" int varq_quant_pack2(const void *x0, const void *x1, int x_dtype, const int64_t *host_shape4, int reduce_mask,
                                int bits, int asym, float eps, int32_t *words0, int8_t *codes0, float *scale0, float *zp0,
                                int32_t *words1, int8_t *codes1, float *scale1, float *zp1,
                                const int64_t *host_out_map, void *workspace, size_t workspace_bytes, void *stream) {
  // (tensors without rows may come as null pointers: nothing to do, as in varq_quant_pack)
  if (host_shape4 && host_shape4[0] >= 0 && host_shape4[1] >= 0 && host_shape4[2] >= 0 &&
      host_shape4[0] * host_shape4[1] * host_shape4[2] == 0 && host_shape4[3] > 0)
    return VARQ_OK;
  VARQ_CHECK_ARG(x1, "quant_pack2: null second tensor");
  return quant_pack_impl(x0, x1, x_dtype, host_shape4, reduce_mask, bits, asym, eps, words0, codes0, scale0, zp0,
                         words1, codes1, scale1, zp1, host_out_map, workspace, workspace_bytes, stream);
}

// ---- the entry point that allocates nothing ------------------------------------------
// Its workspace is this array, which every device the library runs on holds from the load
// of the code object to the end of the process.  Host code never uses the array's name as
// an address: scratch_for_current_device() asks the runtime once per device where that
// device's copy lives and hands out that pointer.
static __device__ __align__(256) unsigned char scratch[VARQ_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void *g_scratch_ptr[kMaxDevices] = {};

int scratch_for_current_device(void **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return varq_set_error(VARQ_ERR_LAUNCH, "quant_pack_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return varq_set_error(VARQ_ERR_UNSUPPORTED, "quant_pack_static: device index %d beyond %d", dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return varq_set_error(VARQ_ERR_LAUNCH, "quant_pack_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return VARQ_OK;
}
}  // namespace

// Also the warm-up call: it looks the current device's copy of the array up (a runtime query that
// must not happen while a stream is being captured into a graph), so that the entry point below
// finds the address already there.  Without a usable device it only reports the size.
extern "C" size_t varq_quant_static_scratch_bytes(void) {
  void *ws = nullptr;
  (void)scratch_for_current_device(&ws);
  return (size_t)VARQ_STATIC_SCRATCH_BYTES;
}

extern "C" int varq_quant_pack_static(const void *x, int x_dtype, const int64_t *host_shape4, int reduce_mask, int bits,
                                      int asym, float eps, int32_t *words, int8_t *codes, float *scale, float *zp,
                                      const int64_t *host_out_map, void *stream) {
  VARQ_CHECK_ARG(host_shape4, "quant_pack_static: null shape");
  VARQ_CHECK_ARG(reduce_mask >= 0 && reduce_mask < 16, "quant_pack_static: bad reduce mask");
  const size_t need = varq_quant_workspace_bytes(host_shape4, reduce_mask);
  if (need > (size_t)VARQ_STATIC_SCRATCH_BYTES)
    return varq_set_error(VARQ_ERR_WORKSPACE,
                          "quant_pack_static: this shape and grouping need %zu bytes of partial results, the static "
                          "scratch holds %zu; use varq_quant_pack with a workspace of the caller's",
                          need, (size_t)VARQ_STATIC_SCRATCH_BYTES);
  void *ws = nullptr;
  const int rc = scratch_for_current_device(&ws);
  if (rc != VARQ_OK) return rc;
  // every partial and parameter the kernels read is written earlier in the same call (plain
  // stores, or the fill kernel of the scalar path), so what an earlier call left behind is
  // never seen and nothing needs clearing here
  return quant_pack_impl(x, nullptr, x_dtype, host_shape4, reduce_mask, bits, asym, eps, words, codes, scale, zp,
                         nullptr, nullptr, nullptr, nullptr, host_out_map, ws, (size_t)VARQ_STATIC_SCRATCH_BYTES, stream);
}

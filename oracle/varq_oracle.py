"""CPU oracle for the VAR-Q KV-cache quantization hot path.

TEST INFRASTRUCTURE ONLY.  This module is the checker that the HIP kernels are
compared against and the CPU baseline that the benchmark times.  Nothing in the
shipped package imports it; only tests, the smoke entry and the benchmark's CPU
leg do.

Every function restates, in plain torch on CPU tensors, what the reference
computes; the reference lines each one follows are cited in its docstring.
Functions marked EXTENSION have no counterpart in the reference (it is
symmetric-only, one bit-width per quantizer, no fused attention): for them this
file is the definition, and the reference cannot pin them ("parity unpinned by
reference").  They are pinned instead by closed forms and invariants in
tests/test_oracle_*.py.

Pinning status
  pack_last_dim / unpack_last_dim     pinned: hand-computed known-answer words,
                                      numpy brute force, bijection/round-trip
  scale_sym / codes_sym / dequant_sym pinned: closed forms (arg-max -> +-qmax,
                                      half-to-even ties, all-zero group, 2-bit)
  OracleVARQ state machine            pinned: length/shape invariants and the
                                      "append == concat of independent steps"
                                      identity; quirks of the reference kept
  asym_* (EXTENSION)                  pinned by invariants only (min -> qmin,
                                      constant group, error bound scale/2)
  attention_ref (EXTENSION)           torch SDPA (library) on bf16 operands;
                                      checked against an fp64 softmax formula
  prepare_qkv (EXTENSION)             parity unpinned by reference (its norm's
                                      summation order is the backend's); checked
                                      against torch's F.normalize / scale /
                                      rotation to rounding, norm-preservation
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

METHODS = ('G_TENSOR', 'G_SCALE_HEAD_DIM', 'G_HEAD_DIM', 'G_SCALE', 'G_TOKEN', 'G_TOKEN_HEAD')

# Token counts per scale (side length squared).
# VAR: VAR/models/var.py:27 -> L = 680.
VAR_PATCH_NUMS = (1, 2, 3, 4, 5, 6, 8, 10, 13, 16)
# Infinity ratio 1.0 / '1M': Infinity/infinity/utils/dynamic_resolution.py:7 -> L = 10521.
INFINITY_PATCH_NUMS = (1, 2, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 64)


def qrange(bits: int) -> Tuple[int, int]:
    """Signed code range, VAR_Q/quant.py:97-98."""
    return -(2 ** (bits - 1)), (2 ** (bits - 1)) - 1


def reduce_dims(method: str, qkv_format: str) -> Tuple[int, ...]:
    """Dims reduced per grouping method, VAR_Q/quant.py:75-95.  Dim 0 (batch) is
    always reduced."""
    if qkv_format == 'BLHc':
        return {
            'G_TENSOR': (0, 1, 2, 3), 'G_SCALE_HEAD_DIM': (0, 1), 'G_HEAD_DIM': (0, 1),
            'G_TOKEN': (0, 2, 3), 'G_TOKEN_HEAD': (0, 3), 'G_SCALE': (0, 1, 2, 3),
        }[method]
    return {
        'G_TENSOR': (0, 1, 2, 3), 'G_SCALE_HEAD_DIM': (0, 2), 'G_HEAD_DIM': (0, 2),
        'G_TOKEN': (0, 1, 3), 'G_TOKEN_HEAD': (0, 3), 'G_SCALE': (0, 1, 2, 3),
    }[method]


# --------------------------------------------------------------------------
# symmetric max-abs quantizer (the reference's only arithmetic)
# --------------------------------------------------------------------------
def scale_sym(x: torch.Tensor, dims: Sequence[int], bits: int, eps: float = 1e-12) -> torch.Tensor:
    """VAR_Q/quant.py:112-116: amax(|x|)/qmax in fp32, clamped below at eps."""
    _, qmax = qrange(bits)
    x32 = x.to(torch.float32)
    return (x32.abs().amax(dim=tuple(dims), keepdim=True) / float(qmax)).clamp_min(eps)


def codes_sym(x: torch.Tensor, scale: torch.Tensor, bits: int) -> torch.Tensor:
    """VAR_Q/quant.py:118-121: true fp32 division, round-half-to-even, clamp, int8."""
    qmin, qmax = qrange(bits)
    return torch.round(x.to(torch.float32) / scale).clamp(qmin, qmax).to(torch.int8)


def dequant_sym(q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """VAR_Q/quant.py:123-124: one fp32 multiply, fp32 result."""
    return q.to(torch.float32) * scale


# --------------------------------------------------------------------------
# EXTENSION: asymmetric min-max quantizer and group-wise-along-D reductions
# --------------------------------------------------------------------------
def asym_params(x: torch.Tensor, dims: Sequence[int], bits: int, eps: float = 1e-12):
    """EXTENSION.  scale=(max-min)/(2^b-1) clamped at eps; zp=qmin-round(min/scale),
    fp32, integer valued, not clamped.  Same fp32/true-division/half-to-even
    conventions as VAR_Q/quant.py:112-121."""
    qmin, _ = qrange(bits)
    x32 = x.to(torch.float32)
    mn = x32.amin(dim=tuple(dims), keepdim=True)
    mx = x32.amax(dim=tuple(dims), keepdim=True)
    scale = ((mx - mn) / float(2 ** bits - 1)).clamp_min(eps)
    zp = float(qmin) - torch.round(mn / scale)
    return scale, zp


def codes_asym(x: torch.Tensor, scale: torch.Tensor, zp: torch.Tensor, bits: int) -> torch.Tensor:
    """EXTENSION.  q = clamp(round(x/scale) + zp, qmin, qmax) as int8."""
    qmin, qmax = qrange(bits)
    return (torch.round(x.to(torch.float32) / scale) + zp).clamp(qmin, qmax).to(torch.int8)


def dequant_asym(q: torch.Tensor, scale: torch.Tensor, zp: torch.Tensor) -> torch.Tensor:
    """EXTENSION.  (q - zp) * scale in fp32."""
    return (q.to(torch.float32) - zp) * scale


def quant_groupwise(x: torch.Tensor, group: int, bits: int, asym: bool, eps: float = 1e-12):
    """EXTENSION.  Groups are `group` contiguous channels of one row of the last
    dim; batch and token dims are NOT reduced.  Returns (codes int8 like x,
    scale [..., C/group] fp32, zp [..., C/group] fp32 or None)."""
    *lead, c = x.shape
    assert c % group == 0
    xg = x.reshape(*lead, c // group, group)
    if asym:
        s, z = asym_params(xg, (-1,), bits, eps)
        q = codes_asym(xg, s, z, bits)
        return q.reshape(*lead, c), s.squeeze(-1), z.squeeze(-1)
    s = scale_sym(xg, (-1,), bits, eps)
    q = codes_sym(xg, s, bits)
    return q.reshape(*lead, c), s.squeeze(-1), None


def dequant_groupwise(q: torch.Tensor, scale: torch.Tensor, zp: Optional[torch.Tensor], group: int) -> torch.Tensor:
    """EXTENSION.  Inverse of quant_groupwise, fp32 result."""
    *lead, c = q.shape
    qg = q.reshape(*lead, c // group, group)
    if zp is None:
        return dequant_sym(qg, scale.unsqueeze(-1)).reshape(*lead, c)
    return dequant_asym(qg, scale.unsqueeze(-1), zp.unsqueeze(-1)).reshape(*lead, c)


def quant_reduce(x: torch.Tensor, dims: Sequence[int], bits: int, asym: bool, eps: float = 1e-12):
    """Quantize with one (scale[, zp]) per group, a group being all elements that
    share the indices of the non-reduced dims.  asym=False is exactly
    VAR_Q/quant.py:112-121; asym=True is the EXTENSION above."""
    if asym:
        s, z = asym_params(x, dims, bits, eps)
        return codes_asym(x, s, z, bits), s, z
    s = scale_sym(x, dims, bits, eps)
    return codes_sym(x, s, bits), s, None


# --------------------------------------------------------------------------
# bit packing (layout is defined by the reference's pure-PyTorch fallback)
# --------------------------------------------------------------------------
def pack_last_dim(q_int8: torch.Tensor, bits: int) -> Tuple[torch.Tensor, Dict[str, int]]:
    """VAR_Q/pack_unpack.py:177-196.  32/bits two's-complement fields per int32
    word, field j of a word at bit j*bits (little-endian), last dim zero-padded
    to a whole word."""
    assert bits in (2, 4, 8), "bit-pack only implements 2/4/8 bits"
    vals = 32 // bits
    *lead, c = q_int8.shape
    pad_len = (-c) % vals
    if pad_len:
        q_int8 = torch.cat([q_int8, q_int8.new_zeros((*lead, pad_len))], dim=-1)
    n_words = (c + pad_len) // vals
    u = (q_int8.to(torch.int32) & ((1 << bits) - 1)).view(*lead, n_words, vals)
    shifts = (torch.arange(vals, dtype=torch.int32) * bits).view(*([1] * (u.dim() - 1)), vals)
    words = (u << shifts).sum(dim=-1).to(torch.int32)
    meta = {'orig_c': int(c), 'vals_per_word': int(vals), 'pad_len': int(pad_len), 'bits': int(bits)}
    return words, meta


def unpack_last_dim(words: torch.Tensor, meta: Dict[str, int]) -> torch.Tensor:
    """VAR_Q/pack_unpack.py:198-211 (+171-175): shift, mask, drop padding,
    sign-extend each field to int8."""
    bits, vals, orig_c = int(meta['bits']), int(meta['vals_per_word']), int(meta['orig_c'])
    mask, sign = (1 << bits) - 1, 1 << (bits - 1)
    pieces = [(words >> (j * bits)) & mask for j in range(vals)]
    u = torch.stack(pieces, dim=-1).reshape(*words.shape[:-1], words.shape[-1] * vals)[..., :orig_c]
    return torch.where((u & sign) != 0, u - (1 << bits), u).to(torch.int8)


# --------------------------------------------------------------------------
# the quantizer's per-step cache state machine
# --------------------------------------------------------------------------
class OracleVARQ:
    """VAR_Q/quant.py:52-230 restated on CPU tensors, quirks included:

    * batch dim is reduced by every method (quant.py:78-95);
    * G_HEAD_DIM and G_TENSOR re-quantize cat(dequant_all(), item) when a cache
      exists (quant.py:149-159);
    * G_TENSOR is matched by the *append* branch of cache() first
      (quant.py:196-201), so from the second step on the cache holds the
      re-quantized concatenation appended after the old cache;
    * the first cached scale is a stride-0 expand along L (quant.py:180-188,198).

    Unlike the reference class (whose packing path asserts a CUDA tensor,
    pack_unpack.py:109), packing here uses the reference's CPU layout functions,
    so pack_to_int32=True works on CPU tensors.
    """

    def __init__(self, quant_bits=8, qkv_format='BLHc', quant_method='G_SCALE_HEAD_DIM', blk_idx=0,
                 pack_to_int32=True, eps=1e-12, debug=False):
        assert qkv_format in ('BLHc', 'BHLc'), f"Invalid qkv_format: {qkv_format}"
        assert quant_method in METHODS, f"Invalid quant_method: {quant_method}"
        assert 1 < quant_bits <= 8
        self.quant_bits, self.quant_method, self.cur_blk_idx = quant_bits, quant_method, blk_idx
        self.qkv_format, self.pack_to_int32, self.eps, self.debug = qkv_format, pack_to_int32, eps, debug
        self.dim_cat = 1 if qkv_format == 'BLHc' else 2
        self.dim_map = {m: reduce_dims(m, qkv_format) for m in METHODS}
        self.bound_min, self.bound_max = qrange(quant_bits)
        self.cached_item = self.cached_scale = self.quantized_item = self.scale = None
        self._pack_meta = None

    def _q(self, x):
        s = scale_sym(x, self.dim_map[self.quant_method], self.quant_bits, self.eps)
        return s, codes_sym(x, s, self.quant_bits)

    def quant(self, item):
        m = self.quant_method
        if m in ('G_HEAD_DIM', 'G_TENSOR') and self.cached_item is not None and self.cached_scale is not None:
            item = torch.cat([self.dequant_all(), item], dim=self.dim_cat)
        scale, q = self._q(item)
        if self.pack_to_int32:
            q, meta = pack_last_dim(q, self.quant_bits)
            if self._pack_meta is not None:
                assert meta == self._pack_meta
            self._pack_meta = meta
        self.quantized_item, self.scale = q, scale

    def _expand_scale_like_L(self, q, scale):
        d = self.dim_cat
        if scale.size(d) == 1 and q.size(d) > 1:
            shape = [-1, -1, -1, -1]
            shape[d] = q.size(d)
            scale = scale.expand(*shape)
        return scale

    def cache(self):
        m = self.quant_method
        q_cur = self.quantized_item
        s_cur = self._expand_scale_like_L(q_cur, self.scale)
        if m in ('G_SCALE_HEAD_DIM', 'G_SCALE', 'G_TOKEN', 'G_TOKEN_HEAD', 'G_TENSOR'):
            if self.cached_item is None:
                self.cached_item, self.cached_scale = q_cur, s_cur
            else:
                self.cached_item = torch.cat([self.cached_item, q_cur], dim=self.dim_cat)
                self.cached_scale = torch.cat([self.cached_scale, s_cur], dim=self.dim_cat)
        elif m == 'G_HEAD_DIM':
            self.cached_item, self.cached_scale = q_cur, s_cur
        else:
            raise ValueError(f"[VAR-Q]: Invalid quantization method: {m}")

    def _deq(self, q, s):
        if self.pack_to_int32:
            assert self._pack_meta is not None, "pack meta is missing"
            q = unpack_last_dim(q, self._pack_meta)
        return dequant_sym(q, s)

    def dequant_current(self):
        return self._deq(self.quantized_item, self.scale)

    def dequant_all(self):
        if self.cached_item is None:
            return self.dequant_current()
        return self._deq(self.cached_item, self.cached_scale)

    def use_var_q(self, item):
        self.quant(item)
        self.cache()
        return self.dequant_all()


# --------------------------------------------------------------------------
# scale schedule, block-causal next-scale mask, attention
# --------------------------------------------------------------------------
def level_of_token(patch_nums: Sequence[int]) -> torch.Tensor:
    """Scale index of every token, VAR/models/var.py:110 (`d`)."""
    return torch.cat([torch.full((pn * pn,), i, dtype=torch.int64) for i, pn in enumerate(patch_nums)])


def block_causal_bias(patch_nums: Sequence[int], q_start: int = 0, q_len: Optional[int] = None) -> torch.Tensor:
    """Additive mask rows q_start..q_start+q_len of VAR/models/var.py:110-114:
    0 where lvl(q) >= lvl(k), -inf elsewhere.  Shape [q_len, L] fp32."""
    lvl = level_of_token(patch_nums)
    q_len = lvl.numel() - q_start if q_len is None else q_len
    lq = lvl[q_start:q_start + q_len].view(-1, 1)
    return torch.where(lq >= lvl.view(1, -1), 0.0, float('-inf')).to(torch.float32)


def kv_limit_from_schedule(patch_nums: Sequence[int], q_start: int = 0, q_len: Optional[int] = None) -> torch.Tensor:
    """Number of visible keys for each query row under the block-causal rule:
    the end offset of the query's own scale.  Equivalent to block_causal_bias
    because levels are non-decreasing in token index.  int32 [q_len]."""
    lvl = level_of_token(patch_nums)
    ends = torch.cumsum(torch.tensor([pn * pn for pn in patch_nums]), 0)
    q_len = lvl.numel() - q_start if q_len is None else q_len
    return ends[lvl[q_start:q_start + q_len]].to(torch.int32)


def attention_ref(q: torch.Tensor, k_deq: torch.Tensor, v_deq: torch.Tensor, softmax_scale: float,
                  bias: Optional[torch.Tensor] = None, dtype=torch.bfloat16) -> torch.Tensor:
    """EXTENSION oracle for the fused kernel: the reference feeds *dequantized*
    K/V to its attention backend after a downcast (VAR/models/basic_var.py:156-162,
    Infinity/infinity/models/basic.py:339-351); here that backend is torch SDPA in
    `dtype` with an explicit additive mask.  q [B,H,Lq,D], k/v [B,H,Lk,D]."""
    attn_mask = None if bias is None else bias.to(dtype)
    return F.scaled_dot_product_attention(q.to(dtype), k_deq.to(dtype), v_deq.to(dtype),
                                          attn_mask=attn_mask, scale=softmax_scale)


def attention_exact(q, k_deq, v_deq, softmax_scale, bias=None):
    """fp64 softmax(QK^T*scale+bias)V, the ground truth both the oracle and the
    kernel approximate.  Used to bound their errors, not as a parity target."""
    s = torch.einsum('bhqd,bhkd->bhqk', q.double(), k_deq.double()) * softmax_scale
    if bias is not None:
        s = s + bias.double()
    return torch.einsum('bhqk,bhkd->bhqd', torch.softmax(s, dim=-1), v_deq.double())


# --------------------------------------------------------------------------
# synthetic inputs of the benchmark configurations
# --------------------------------------------------------------------------
def synth_kv(shape: Sequence[int], seed: int, dist: str = 'normal', outlier_frac: float = 0.02,
             outlier_mul: float = 15.0, dtype=torch.float32, outlier_seed: Optional[int] = None) -> torch.Tensor:
    """Seeded K/V-like tensor [B,H,L,D]: N(0,1) or Student-t(nu=4) values with
    max(1, round(frac*D)) channels of the last dim scaled by `outlier_mul`."""
    g = torch.Generator().manual_seed(seed)
    if dist == 'normal':
        x = torch.randn(*shape, generator=g, dtype=torch.float32)
    elif dist == 'student4':
        n = torch.randn(*shape, generator=g, dtype=torch.float32)
        chi = torch.randn(4, *shape, generator=g, dtype=torch.float32).square_().sum(0)
        x = n / torch.sqrt(chi / 4.0)
    else:
        raise ValueError(dist)
    d = shape[-1]
    n_out = max(1, round(outlier_frac * d))
    go = torch.Generator().manual_seed(seed + 3000 if outlier_seed is None else outlier_seed)
    ch = torch.randperm(d, generator=go)[:n_out]
    x[..., ch] *= outlier_mul
    return x.to(dtype)


def prepare_qkv(qkv: torch.Tensor, scale_mul: Optional[torch.Tensor] = None, l2norm: bool = False,
                norm_eps: float = 1e-12, rope=None, token_start: int = 0):
    """EXTENSION (parity unpinned by reference: the reference leaves the summation order of
    the norm to the backend).  The producer side of Infinity/infinity/models/basic.py:316-330
    (F.normalize, .mul(scale_mul), apply_rotary_emb at :103-123) and
    VAR/models/basic_var.py:137-141 restated for a qkv projection output [B,L,3,H,c]:
    returns q [B,H,L,c] bf16, k [B,H,L,c] fp32, v [B,H,L,c] in the input dtype.

    All arithmetic fp32, each operation rounded on its own.  Sum of squares: the 8
    channels of an octet left to right, then octets pairwise ((o0+o1)+(o2+o3))+...;
    y = x / max(sqrt(ss), norm_eps) with correctly rounded sqrt and true division; q times scale_mul[h]; rotation
    of the pairs (2i, 2i+1): even = cos*y0 - sin*y1, odd = sin*y0 + cos*y1."""
    B, L, three, H, c = qkv.shape
    assert three == 3 and c % 8 == 0 and (c // 8) & (c // 8 - 1) == 0
    q, k, v = (qkv[:, :, t].permute(0, 2, 1, 3).contiguous() for t in range(3))      # [B,H,L,c]
    qf, kf = q.float(), k.float()

    def normalize(x):
        sq = x * x
        o = sq.reshape(*sq.shape[:-1], c // 8, 8)
        acc = o[..., 0]
        for j in range(1, 8):
            acc = acc + o[..., j]
        while acc.shape[-1] > 1:
            acc = acc[..., 0::2] + acc[..., 1::2]
        # correctly rounded fp32 square root: through fp64 (53 >= 2*24+2 bits, so the second rounding
        # cannot change the result); torch's vectorized fp32 sqrt on CPU is off by an ulp now and then
        denom = torch.sqrt(acc.double()).float().clamp_min(norm_eps)                  # [..., 1]
        return x / denom

    if l2norm:
        qf, kf = normalize(qf), normalize(kf)
        if scale_mul is not None:
            qf = qf * scale_mul.float().view(1, H, 1, 1)
    if rope is not None:
        cos, sin = rope
        cs = cos[token_start:token_start + L].float().view(1, 1, L, c // 2)
        sn = sin[token_start:token_start + L].float().view(1, 1, L, c // 2)

        def rotate(x):
            x2 = x.reshape(*x.shape[:-1], c // 2, 2)
            even = cs * x2[..., 0] - sn * x2[..., 1]
            odd = sn * x2[..., 0] + cs * x2[..., 1]
            return torch.stack([even, odd], dim=-1).reshape(x.shape)

        qf, kf = rotate(qf), rotate(kf)
    return qf.to(torch.bfloat16), kf, v

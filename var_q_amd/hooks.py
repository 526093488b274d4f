"""Self-attention modules that carry the VAR-Q hook, on random weights.

They reproduce the inference-time contract of the two call sites of the
reference quantizer,

  * VAR:       VAR/models/basic_var.py:70-165  (`SelfAttention`)
  * Infinity:  Infinity/infinity/models/basic.py:205-351 (`SelfAttention`),
               2-D rotary embedding basic.py:44-123

i.e. `kv_caching(True)` creates one K and one V quantizer, `forward` projects
x to q/k/v, normalises (and rotates) q and k, pushes k and v through the
quantized cache and attends with the current scale's queries over everything
cached.  Three backends behind the same interface:

  * `fused=False`: the drop-in `VAR_Q.use_var_q` (dequantized full-length K/V
    out) followed by scaled-dot-product attention, which is what the reference
    modules do with flash-attn / xformers / their `slow_attn`;
  * `fused=True`: `PackedKVCache.append` + `PackedKVCache.attend`: the step is
    quantized in place into a pre-allocated packed cache and attention reads the
    packed codes; no dequantized K/V exists.  Needs a row-local quantizer
    (`quant_method='G_GROUP'`).  With `fused_producer=True` the normalisation,
    the per-head scale of q, the rotation and the quantization of k and v run as
    one kernel on the qkv projection output (`PackedKVCache.append_from_qkv`);
  * `fused='quantizer'`: the drop-in quantizers of any rule of the JSON files (the shipped
    G_SCALE_HEAD_DIM rule included) do `quant` + `cache` as in the first backend, and
    `var_q_amd.quant.fused_attention` attends over their packed caches, so the
    dequantized full-length K/V of `dequant_all` is never built.  Either layout.

The transformer blocks around the attention (AdaLN, FFN, cross-attention) are
outside this package.
"""
import math
from typing import Callable, Optional, Sequence, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .kv_cache import PackedKVCache
from .quant import VAR_Q, fused_step


def rope2d_tables(head_dim: int, scale_hw: Sequence[Tuple[int, int]], normalized_by_hw: int = 2,
                  base: float = 10000.0, max_hw: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos, sin [sum(h*w), head_dim/2] of the 2-D rotary embedding for a scale
    schedule [(h, w), ...]: the first half of the rotated pairs turns with the
    token's row, the second half with its column, frequencies
    base^(-2j/(head_dim/2)) (Infinity/infinity/models/basic.py:44-97).
    normalized_by_hw = 0: grid coordinates as they are; 2: coordinates scaled to
    the last scale's grid and rounded (the released models' setting); 1
    (bilinear resampling of the table) is not provided."""
    assert head_dim % 4 == 0
    if normalized_by_hw not in (0, 2):
        raise ValueError('normalized_by_hw must be 0 or 2 (got %r)' % (normalized_by_hw,))
    half = head_dim // 2
    inv_freq = 1.0 / (base ** (torch.arange(0, half, 2, dtype=torch.int64).float() / half))   # [half/2]
    pos = torch.arange(max_hw, dtype=torch.int64).float()
    ang = torch.outer(pos, inv_freq)                                                         # [max_hw, half/2]
    uh, uw = scale_hw[-1]
    cos, sin = [], []
    for h, w in scale_hw:
        if normalized_by_hw == 2:
            ys = (torch.arange(h) * (uh / h)).round().long()
            xs = (torch.arange(w) * (uw / w)).round().long()
        else:
            ys, xs = torch.arange(h), torch.arange(w)
        a = torch.cat([ang[ys][:, None, :].expand(h, w, -1), ang[xs][None, :, :].expand(h, w, -1)], dim=-1)
        a = a.reshape(h * w, half)
        cos.append(torch.cos(a))
        sin.append(torch.sin(a))
    return torch.cat(cos), torch.cat(sin)


def apply_rope2d(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, start: int, l_dim: int) -> torch.Tensor:
    """Rotate adjacent channel pairs (2i, 2i+1) of x (fp32) by the angles of tokens
    start..start+L (basic.py:103-123).  l_dim is the token axis of x."""
    L = x.shape[l_dim]
    shape = [1] * x.dim()
    shape[l_dim], shape[-1] = L, x.shape[-1] // 2
    c = cos[start:start + L].to(x.device).view(shape)
    s = sin[start:start + L].to(x.device).view(shape)
    x2 = x.float().reshape(*x.shape[:-1], -1, 2)
    out = torch.stack([c * x2[..., 0] - s * x2[..., 1], s * x2[..., 0] + c * x2[..., 1]], dim=-1)
    return out.reshape(x.shape)


class _QuantizedSelfAttention(nn.Module):
    """Common part: qkv projection, quantized cache, attention, output projection."""

    def __init__(self, embed_dim: int, num_heads: int, layout: str, q_bits, quant_method: str, enable_quantization: bool,
                 fused: bool, group_size: Optional[int], symmetric: bool, max_tokens: int, block_idx: int,
                 quantizer_factory: Optional[Callable] = None, fused_producer: bool = False):
        super().__init__()
        assert embed_dim % num_heads == 0 and layout in ('BLHc', 'BHLc')
        self.num_heads, self.head_dim = num_heads, embed_dim // num_heads
        self.layout, self.block_idx = layout, block_idx
        self.q_bits, self.quant_method, self.enable_quantization = q_bits, quant_method, enable_quantization
        self.fused, self.group_size, self.symmetric, self.max_tokens = fused, group_size, symmetric, max_tokens
        self.fused_producer = fused_producer
        assert fused is True or not fused_producer, 'fused_producer needs the packed-cache backend (fused=True)'
        self._quantizer_factory = quantizer_factory or VAR_Q
        assert fused in (False, True, 'quantizer'), "fused: False, True or 'quantizer'"
        if fused is True:
            assert enable_quantization and quant_method == 'G_GROUP' and group_size, \
                'the fused backend needs the row-local group-wise quantizer (quant_method="G_GROUP", group_size=g)'
        if fused == 'quantizer':
            assert enable_quantization, "fused='quantizer' needs quantization"
        self.mat_qkv = nn.Linear(embed_dim, embed_dim * 3, bias=False)
        self.q_bias, self.v_bias = nn.Parameter(torch.zeros(embed_dim)), nn.Parameter(torch.zeros(embed_dim))
        self.register_buffer('zero_k_bias', torch.zeros(embed_dim))
        self.proj = nn.Linear(embed_dim, embed_dim)
        self.caching, self.cached_k, self.cached_v = False, None, None
        self.k_quant = self.v_quant = None
        self.packed_cache: Optional[PackedKVCache] = None

    # -- cache life cycle (basic_var.py:104-117, basic.py:254-271) ---------------------
    def kv_caching(self, enable: bool):
        self.caching, self.cached_k, self.cached_v = enable, None, None
        self.k_quant = self.v_quant = None
        self.packed_cache = None
        self._session = {}          # tensors derived from the parameters alone, kept while a schedule is cached
        if enable and self.enable_quantization and self.fused is not True:
            kw = dict(quant_bits=self.q_bits, qkv_format=self.layout, quant_method=self.quant_method, blk_idx=self.block_idx)
            if self.quant_method == 'G_GROUP' or not self.symmetric:
                kw.update(group_size=self.group_size, symmetric=self.symmetric)
            self.k_quant = self._quantizer_factory(**kw)
            self.v_quant = self._quantizer_factory(**kw)
            for quantizer in (self.k_quant, self.v_quant):
                if self.max_tokens and hasattr(quantizer, 'reserve_tokens'):
                    quantizer.reserve_tokens(self.max_tokens)     # no buffer growth during a schedule

    def _qkv(self, x):
        B, L, _ = x.shape
        bias = self._per_session(('qkv bias', x.dtype),
                                 lambda: torch.cat((self.q_bias, self.zero_k_bias, self.v_bias)).to(x.dtype))
        return F.linear(x, self.mat_qkv.weight.to(x.dtype), bias).view(B, L, 3, self.num_heads, self.head_dim)

    def _per_session(self, key, make):
        """make() once per cached schedule (kv_caching(True) .. kv_caching(False): inference, the
        parameters do not change under it), every time otherwise, as the reference's modules do
        (VAR/models/basic_var.py:122, :138): a handful of tiny launches per call that cost the
        small scales more host time than their attention takes."""
        if not self.caching or torch.is_grad_enabled():
            return make()
        session = self.__dict__.setdefault('_session', {})
        if key not in session:
            session[key] = make()
        return session[key]

    def _project(self, x):
        qkv = self._qkv(x)
        if self.layout == 'BLHc':
            return qkv.unbind(dim=2)                       # each [B,L,H,c]
        return qkv.permute(2, 0, 3, 1, 4).unbind(dim=0)     # each [B,H,L,c]

    def _attend(self, q, k, v, scale: float, attn_bias, out_dtype):
        """q, k, v in self.layout (k, v full length); returns [B,L,C]."""
        B = q.shape[0]
        if self.layout == 'BLHc':
            q, k, v = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
        L = q.shape[2]
        o = F.scaled_dot_product_attention(q.to(out_dtype), k.to(out_dtype), v.to(out_dtype), scale=scale,
                                           attn_mask=None if attn_bias is None else attn_bias.to(out_dtype))
        return o.transpose(1, 2).reshape(B, L, self.num_heads * self.head_dim)

    def _fused_from_qkv(self, x, scale: float, scale_mul, l2norm: bool, rope, token_start, attn_bias):
        """qkv projection -> one producer kernel (normalise, scale, rotate, quantize into the
        cache) -> fused attention; returns [B,L,C]."""
        if attn_bias is not None:
            raise ValueError('the fused backend takes the mask as a key limit per query, not as a bias tensor')
        qkv = self._qkv(x)
        B, L = qkv.shape[:2]
        if self.packed_cache is None:
            self.packed_cache = PackedKVCache(B, self.num_heads, self.max_tokens, self.head_dim, self.q_bits,
                                              self.group_size, qkv.device, symmetric=self.symmetric)
        mul = None if scale_mul is None else self._per_session('scale_mul fp32', lambda: scale_mul().detach().float().reshape(-1).contiguous())
        q = self.packed_cache.append_from_qkv(qkv, mul, l2norm, 1e-12, rope, token_start)
        o = self.packed_cache.attend(q, scale, out_layout='BLHc')                       # [B,L,H,c]
        return o.reshape(B, L, self.num_heads * self.head_dim).to(x.dtype)

    def _attn_dtype(self, main_type):
        """dtype of the fused attention: the module's compute dtype where the kernels have it
        (fp16 at head dim 64, the VAR models), bf16 otherwise."""
        return torch.float16 if (main_type == torch.float16 and self.head_dim == 64) else torch.bfloat16

    def _cache_and_attend(self, q, k, v, scale: float, attn_bias, out_dtype):
        B = q.shape[0]
        l_dim = 1 if self.layout == 'BLHc' else 2
        L = q.shape[l_dim]
        if self.caching and self.fused == 'quantizer':
            if attn_bias is not None:
                raise ValueError('the fused backend takes the mask as a key limit per query, not as a bias tensor')
            # the attention runs in the module's compute dtype, like the reference's call
            # (q.to(dtype=main_type), VAR/models/basic_var.py:158): fp16 for VAR, bf16 for Infinity
            o = fused_step(q.to(self._attn_dtype(out_dtype)), k, v, self.k_quant, self.v_quant, scale)   # in the layout of q
            if self.layout == 'BHLc':
                o = o.transpose(1, 2)
            return o.reshape(B, L, self.num_heads * self.head_dim).to(out_dtype)
        if self.caching and self.fused:
            if attn_bias is not None:
                raise ValueError('the fused backend takes the mask as a key limit per query, not as a bias tensor')
            if self.packed_cache is None:
                self.packed_cache = PackedKVCache(B, self.num_heads, self.max_tokens, self.head_dim, self.q_bits,
                                                  self.group_size, q.device, symmetric=self.symmetric)
            self.packed_cache.append(k, v, layout=self.layout)
            qh = q if self.layout == 'BHLc' else q.transpose(1, 2)
            o = self.packed_cache.attend(qh.to(self._attn_dtype(out_dtype)).contiguous(), scale, out_layout='BLHc')   # [B,L,H,c]
            return o.reshape(B, L, self.num_heads * self.head_dim).to(out_dtype)
        if self.caching:
            if self.enable_quantization:
                # (dequantized straight into the attention's dtype: the values `.to(out_dtype)` of
                # the reference's fp32 result would have)
                # (only this package's quantizer takes the argument; any other factory's is called
                # as the reference calls it)
                if out_dtype in (torch.bfloat16, torch.float16) and isinstance(self.k_quant, VAR_Q):
                    k = self.k_quant.use_var_q(k, out_dtype=out_dtype)
                    v = self.v_quant.use_var_q(v, out_dtype=out_dtype)
                else:
                    k = self.k_quant.use_var_q(k)
                    v = self.v_quant.use_var_q(v)
            elif self.cached_k is None:
                self.cached_k, self.cached_v = k, v
            else:
                k = self.cached_k = torch.cat((self.cached_k, k), dim=l_dim)
                v = self.cached_v = torch.cat((self.cached_v, v), dim=l_dim)
        return self._attend(q, k, v, scale, attn_bias, out_dtype)


class VarSelfAttention(_QuantizedSelfAttention):
    """VAR/models/basic_var.py:70-165.  attn_l2_norm=True (the released VAR-d16..d30
    setting): q and k are l2-normalised, q is multiplied by a per-head
    exp(min(param, ln 100)), softmax scale 1; else scale 0.25/sqrt(c)."""

    def __init__(self, block_idx: int, embed_dim: int = 1024, num_heads: int = 16, attn_l2_norm: bool = True,
                 layout: str = 'BLHc', q_bits=8, quant_method: str = 'G_SCALE_HEAD_DIM', enable_quantization: bool = False,
                 fused: bool = False, group_size: Optional[int] = None, symmetric: bool = True, max_tokens: int = 680,
                 quantizer_factory: Optional[Callable] = None, fused_producer: bool = False):
        super().__init__(embed_dim, num_heads, layout, q_bits, quant_method, enable_quantization, fused, group_size,
                         symmetric, max_tokens, block_idx, quantizer_factory, fused_producer)
        self.attn_l2_norm = attn_l2_norm
        if attn_l2_norm:
            self.scale = 1.0
            self.scale_mul_1H11 = nn.Parameter(torch.full((1, num_heads, 1, 1), 4.0).log())
            self.max_scale_mul = math.log(100.0)
        else:
            self.scale = 0.25 / math.sqrt(self.head_dim)

    def forward(self, x: torch.Tensor, attn_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        if self.caching and self.fused_producer:
            mul = (lambda: self.scale_mul_1H11.clamp_max(self.max_scale_mul).exp()) if self.attn_l2_norm else None
            o = self._fused_from_qkv(x, self.scale, mul, self.attn_l2_norm, None, None, attn_bias)
            return self.proj(o.to(self.proj.weight.dtype))
        q, k, v = self._project(x)
        main_type = x.dtype
        if self.attn_l2_norm:
            scale_mul = self.scale_mul_1H11.clamp_max(self.max_scale_mul).exp()
            if self.layout == 'BLHc':
                scale_mul = scale_mul.transpose(1, 2)
            q = F.normalize(q.float(), dim=-1).mul(scale_mul)
            k = F.normalize(k.float(), dim=-1)
        o = self._cache_and_attend(q, k, v, self.scale, attn_bias, main_type)
        return self.proj(o.to(self.proj.weight.dtype))


class InfinitySelfAttention(_QuantizedSelfAttention):
    """Infinity/infinity/models/basic.py:205-351: cos_attn (l2-normalised q, k with
    a per-head multiplier, scale 1) or scale 1/sqrt(c)/tau; 2-D rotary embedding of
    q and k before the cache; K reaches the quantizer in fp32, V in the compute
    dtype."""

    def __init__(self, embed_dim: int = 2048, num_heads: int = 16, tau: float = 1.0, cos_attn: bool = True,
                 layout: str = 'BHLc', q_bits=8, quant_method: str = 'G_SCALE_HEAD_DIM', enable_quantization: bool = False,
                 fused: bool = False, group_size: Optional[int] = None, symmetric: bool = True, max_tokens: int = 10521,
                 block_idx: int = 0, quantizer_factory: Optional[Callable] = None, fused_producer: bool = False):
        super().__init__(embed_dim, num_heads, layout, q_bits, quant_method, enable_quantization, fused, group_size,
                         symmetric, max_tokens, block_idx, quantizer_factory, fused_producer)
        self.tau, self.cos_attn = tau, cos_attn
        if cos_attn:
            self.scale = 1.0
            size = (1, 1, num_heads, 1) if layout == 'BLHc' else (1, num_heads, 1, 1)
            self.scale_mul_1H11 = nn.Parameter(torch.full(size, 4.0).log())
            self.max_scale_mul = math.log(100.0)
        else:
            self.scale = 1.0 / math.sqrt(self.head_dim) / tau

    def forward(self, x: torch.Tensor, attn_bias: Optional[torch.Tensor] = None,
                rope: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, token_start: int = 0) -> torch.Tensor:
        """rope = (cos, sin) from rope2d_tables for the whole schedule; token_start =
        number of tokens of the scales before this one."""
        if self.caching and self.fused_producer:
            mul = (lambda: self.scale_mul_1H11.clamp_max(self.max_scale_mul).exp()) if self.cos_attn else None
            rope_dev = None
            if rope is not None:
                rope_dev = tuple(t.to(x.device, torch.float32).contiguous() for t in rope)   # (no copies for fp32 tables on the device)
            o = self._fused_from_qkv(x, self.scale, mul, self.cos_attn, rope_dev, token_start, attn_bias)
            return self.proj(o.to(self.proj.weight.dtype))
        q, k, v = self._project(x)
        main_type = x.dtype
        if self.cos_attn:
            scale_mul = self.scale_mul_1H11.clamp_max(self.max_scale_mul).exp()
            q = F.normalize(q.float(), dim=-1, eps=1e-12).mul(scale_mul).contiguous()
            k = F.normalize(k.float(), dim=-1, eps=1e-12).contiguous()
            v = v.contiguous()
        else:
            q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        if rope is not None:
            l_dim = 1 if self.layout == 'BLHc' else 2
            q = apply_rope2d(q, rope[0], rope[1], token_start, l_dim)
            k = apply_rope2d(k, rope[0], rope[1], token_start, l_dim)
        o = self._cache_and_attend(q, k, v, self.scale, attn_bias, main_type)
        return self.proj(o.to(self.proj.weight.dtype))

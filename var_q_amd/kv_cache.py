"""Pre-allocated packed KV cache with in-place append and fused attention.

Functionally the append-type cache of the reference quantizer
(VAR_Q/quant.py:191-205: concatenate each step's codes and scales) for the
group-wise asymmetric quantizer, but a step costs O(new tokens): it is
quantized straight into its slot of the cache.  Heads may carry different
bit-widths; heads of equal width share one dense buffer ("class") and a table
maps each head to (class, slot).  Layout BHLc: K/V steps are [B, H, n, D].
"""
from typing import List, Optional, Sequence, Union

import torch

from . import ops


class _BitClass:
    def __init__(self, bits, heads, B, H, Lmax, D, group, device):
        self.bits, self.heads = bits, list(heads)
        hc, w, ns = len(self.heads), D * bits // 32, D // group
        slot = torch.full((H,), -1, dtype=torch.int32)
        slot[self.heads] = torch.arange(hc, dtype=torch.int32)
        self.slot = slot.to(device)
        self.head_map = torch.tensor(self.heads, dtype=torch.int32, device=device)
        mk = lambda last, dt: torch.zeros((B, hc, Lmax, last), dtype=dt, device=device)
        self.k_words, self.v_words = mk(w, torch.int32), mk(w, torch.int32)
        self.k_scale, self.v_scale = mk(ns, torch.float32), mk(ns, torch.float32)
        self.k_zp, self.v_zp = mk(ns, torch.float32), mk(ns, torch.float32)


class PackedKVCache:
    def __init__(self, B: int, H: int, Lmax: int, D: int, bits: Union[int, Sequence[int]], group_size: int,
                 device, symmetric: bool = False, eps: float = 1e-12):
        per_head = [int(bits)] * H if isinstance(bits, int) else [int(b) for b in bits]
        assert len(per_head) == H and all(b in (2, 4, 8) for b in per_head)
        assert D % group_size == 0
        self.B, self.H, self.Lmax, self.D, self.group = B, H, Lmax, D, group_size
        self.per_head_bits, self.symmetric, self.eps = per_head, symmetric, eps
        self.len = 0
        self.classes: List[_BitClass] = [
            _BitClass(b, [h for h in range(H) if per_head[h] == b], B, H, Lmax, D, group_size, device)
            for b in sorted(set(per_head))]

    def reset(self):
        self.len = 0

    def append(self, k: torch.Tensor, v: torch.Tensor, layout: str = 'BHLc'):
        """Quantize + pack one step into tokens len..len+n of the cache.  The step is
        [B,H,n,D] (layout 'BHLc') or [B,n,H,D] ('BLHc', the flash-attention layout of
        VAR/models/basic_var.py:127-131); either is read where it lies."""
        assert layout in ('BHLc', 'BLHc')
        if layout == 'BHLc':
            B, H, n, D = k.shape
        else:
            B, n, H, D = k.shape
        assert (B, H, D) == (self.B, self.H, self.D) and v.shape == k.shape
        assert self.len + n <= self.Lmax, 'cache overflow'
        k, v = k.contiguous(), v.contiguous()
        for c in self.classes:
            hc = len(c.heads)
            # input rows in memory order -> output row b*hc*Lmax + slot(h)*Lmax + len + l
            if layout == 'BHLc':
                rowmap = [B, H, n, hc * self.Lmax, self.Lmax, 1, self.len, 1]
            else:
                rowmap = [B, n, H, hc * self.Lmax, 1, self.Lmax, self.len, 2]
            asym = not self.symmetric
            ops.quant_pack_rows_into(k, self.group, c.bits, asym, self.eps, c.k_words, c.k_scale,
                                     c.k_zp if asym else None, rowmap, c.slot)
            ops.quant_pack_rows_into(v, self.group, c.bits, asym, self.eps, c.v_words, c.v_scale,
                                     c.v_zp if asym else None, rowmap, c.slot)
        self.len += n

    def attend(self, q: torch.Tensor, softmax_scale: float, kv_limit: Optional[torch.Tensor] = None,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Fused dequant attention of q [B,H,Lq,D] (bf16) over the cached tokens."""
        assert self.len > 0
        if out is None:
            out = torch.empty_like(q)
        asym = not self.symmetric
        for c in self.classes:
            ops.fused_attn(q, c.k_words, c.k_scale, c.k_zp if asym else None,
                           c.v_words, c.v_scale, c.v_zp if asym else None,
                           c.bits, c.bits, self.len, softmax_scale, kv_limit=kv_limit,
                           head_map=c.head_map if len(self.classes) > 1 else None, out=out)
        return out

    def dequant(self, which: str = 'k', out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """Dequantized [B,H,len,D] copy of the cached K or V (for checking)."""
        out = torch.empty((self.B, self.H, self.len, self.D), dtype=out_dtype, device=self.classes[0].k_words.device)
        asym = not self.symmetric
        for c in self.classes:
            words = c.k_words if which == 'k' else c.v_words
            scale = c.k_scale if which == 'k' else c.v_scale
            zp = (c.k_zp if which == 'k' else c.v_zp) if asym else None
            hc, ns = len(c.heads), self.D // self.group
            rowmap = [self.B, hc, self.len, hc * self.Lmax, self.Lmax, 1, 0, -1]
            strides = [hc * self.Lmax * ns, self.Lmax * ns, ns, 1]
            part = ops.dequant_window(words, scale, zp, (self.B, hc, self.len, self.D), strides, self.group,
                                      c.bits, rowmap, out_dtype)
            out[:, c.heads] = part
        return out

"""Pre-allocated packed KV cache with in-place append and fused attention.

Functionally the append-type cache of the reference quantizer
(VAR_Q/quant.py:191-205: concatenate each step's codes and scales) for the
group-wise asymmetric quantizer, but a step costs O(new tokens): it is
quantized straight into its slot of the cache.  Heads may carry different
bit-widths; heads of equal width share one dense buffer ("class") and a table
maps each head to (class, slot).  Layout BHLc: K/V steps are [B, H, n, D].
"""
import json
from typing import Any, Dict, List, Optional, Sequence, Union

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
        self.concurrent_classes = True   # attend(): one stream per bit-width class ...
        # ... once the call is large enough: forking and joining the streams costs the host about
        # 50 us, more than the classes of a small step gain by running side by side (measured on
        # the 13-scale schedule at B=8, H=16: side streams win from 576 queries over 1 497 keys
        # on).  While a graph is being recorded there is no such cost and the streams are always used.
        self.concurrent_min_flops = 4e10
        self.splits = 0                  # attend() on one stream: shares of a query block's keys (0 = library's choice)
        self._side = self._fork = self._join = None
        self.classes: List[_BitClass] = [
            _BitClass(b, [h for h in range(H) if per_head[h] == b], B, H, Lmax, D, group_size, device)
            for b in sorted(set(per_head))]

    def reset(self):
        self.len = 0

    # -- hand-over format ---------------------------------------------------------------
    FORMAT_VERSION = 1

    def descriptor(self) -> Dict[str, Any]:
        """JSON-serialisable description of the packed cache: everything a consumer
        needs to address and decode the buffers of `tensors()`.  Per bit-width class it
        repeats the `meta` dictionary of the reference's pack functions
        (VAR_Q/pack_unpack.py:133: orig_c, vals_per_word, pad_len, bits)."""
        ns = self.D // self.group
        return {
            'format': 'varq-packed-kv', 'version': self.FORMAT_VERSION, 'layout': 'BHLc',
            'B': self.B, 'H': self.H, 'Lmax': self.Lmax, 'D': self.D, 'len': self.len,
            'group_size': self.group, 'symmetric': self.symmetric, 'eps': self.eps,
            'per_head_bits': list(self.per_head_bits),
            'field_order': 'code j of a word at bits [j*bits, (j+1)*bits), two\'s complement',
            'dequant': '(code - zp) * scale' if not self.symmetric else 'code * scale',
            'classes': [{
                'bits': c.bits, 'heads': list(c.heads),
                'words': {'name': f'b{c.bits}.{{k,v}}_words', 'dtype': 'int32',
                          'shape': [self.B, len(c.heads), self.Lmax, self.D * c.bits // 32]},
                'scale': {'name': f'b{c.bits}.{{k,v}}_scale', 'dtype': 'float32',
                          'shape': [self.B, len(c.heads), self.Lmax, ns]},
                'zp': None if self.symmetric else {'name': f'b{c.bits}.{{k,v}}_zp', 'dtype': 'float32',
                                                   'shape': [self.B, len(c.heads), self.Lmax, ns]},
                'meta': {'orig_c': self.D, 'vals_per_word': 32 // c.bits, 'pad_len': 0, 'bits': c.bits},
            } for c in self.classes],
        }

    def tensors(self) -> Dict[str, torch.Tensor]:
        """The cache buffers under the names the descriptor uses (no copies)."""
        out = {}
        for c in self.classes:
            for kv in 'kv':
                out[f'b{c.bits}.{kv}_words'] = getattr(c, f'{kv}_words')
                out[f'b{c.bits}.{kv}_scale'] = getattr(c, f'{kv}_scale')
                if not self.symmetric:
                    out[f'b{c.bits}.{kv}_zp'] = getattr(c, f'{kv}_zp')
        return out

    def save(self, path: str):
        """Write the filled part of the cache (tokens 0..len-1) as one safetensors
        file; the descriptor travels in the file's metadata."""
        from safetensors.torch import save_file
        desc = self.descriptor()
        desc['Lmax_saved'] = self.len
        data = {k: t[:, :, :self.len].contiguous().cpu() for k, t in self.tensors().items()}
        save_file(data, path, metadata={'varq': json.dumps(desc)})

    @classmethod
    def load(cls, path: str, device, Lmax: Optional[int] = None) -> 'PackedKVCache':
        """Rebuild a cache from `save`'s file (room for Lmax tokens, default: as saved
        cache's capacity)."""
        from safetensors import safe_open
        with safe_open(path, framework='pt', device='cpu') as f:
            desc = json.loads(f.metadata()['varq'])
            if desc.get('format') != 'varq-packed-kv' or desc.get('version') != cls.FORMAT_VERSION:
                raise ValueError('not a version-%d varq packed cache: %r' % (cls.FORMAT_VERSION, desc.get('format')))
            cache = cls(desc['B'], desc['H'], Lmax or desc['Lmax'], desc['D'], desc['per_head_bits'], desc['group_size'],
                        device, symmetric=desc['symmetric'], eps=desc['eps'])
            n = desc['len']
            assert n <= cache.Lmax, 'saved cache longer than the requested capacity'
            for name, dst in cache.tensors().items():
                dst[:, :, :n].copy_(f.get_tensor(name))
            cache.len = n
        return cache

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
            if k.dtype == v.dtype and 2 * rowmap[0] <= 65535:
                ops.quant_pack_rows_pair_into(k, v, self.group, c.bits, asym, self.eps,
                                              (c.k_words, c.k_scale, c.k_zp if asym else None),
                                              (c.v_words, c.v_scale, c.v_zp if asym else None), rowmap, c.slot)
            else:   # K and V of different dtypes (Infinity: fp32 K after cos-norm, bf16 V)
                ops.quant_pack_rows_into(k, self.group, c.bits, asym, self.eps, c.k_words, c.k_scale,
                                         c.k_zp if asym else None, rowmap, c.slot)
                ops.quant_pack_rows_into(v, self.group, c.bits, asym, self.eps, c.v_words, c.v_scale,
                                         c.v_zp if asym else None, rowmap, c.slot)
        self.len += n

    def append_from_qkv(self, qkv: torch.Tensor, q_scale_mul: Optional[torch.Tensor] = None, l2norm: bool = False,
                        norm_eps: float = 1e-12, rope=None, token_start: Optional[int] = None) -> torch.Tensor:
        """One pass from the qkv projection output [B,n,3,H,D] to the cache: k (l2-normalised and
        rotated if asked) and v are quantized into tokens len..len+n, the prepared q comes back
        as bf16 [B,H,n,D] (Infinity/infinity/models/basic.py:316-330 in one kernel).
        token_start (default: the cache length) selects the rotary table rows."""
        B, n, three, H, D = qkv.shape
        assert three == 3 and (B, H, D) == (self.B, self.H, self.D)
        assert self.len + n <= self.Lmax, 'cache overflow'
        qkv = qkv.contiguous()
        q_out = torch.empty((B, H, n, D), dtype=torch.bfloat16, device=qkv.device)
        asym = not self.symmetric
        start = self.len if token_start is None else token_start
        for c in self.classes:
            hc = len(c.heads)
            rowmap = [B, n, H, hc * self.Lmax, 1, self.Lmax, self.len, 2]
            ops.qkv_prepare_append(qkv, q_out, self.group, c.bits, asym, self.eps, c.k_words, c.k_scale,
                                   c.k_zp if asym else None, c.v_words, c.v_scale, c.v_zp if asym else None,
                                   rowmap, c.slot, q_scale_mul, l2norm, norm_eps, rope, start)
        self.len += n
        return q_out

    def attend(self, q: torch.Tensor, softmax_scale: float, kv_limit: Optional[torch.Tensor] = None,
               out: Optional[torch.Tensor] = None, exact_codes: bool = False, out_layout: str = 'BHLc') -> torch.Tensor:
        """Fused dequant attention of q [B,H,Lq,D] (bf16; fp16 at D=64) over the cached tokens.
        K and V enter the products rounded to q's dtype, as in the reference; exact_codes=True
        selects the form that does not round them where it exists (see ops.fused_attn).
        out_layout 'BLHc': the result as [B,Lq,H,D], the order an attention module reshapes to
        [B,Lq,C] for its output projection (no transposing copy)."""
        assert self.len > 0, 'attend on an empty cache: append keys and values first'
        assert out_layout in ('BHLc', 'BLHc')
        if out is None:
            B_, H_, Lq_, D_ = q.shape
            out = torch.empty((B_, Lq_, H_, D_) if out_layout == 'BLHc' else q.shape, dtype=q.dtype, device=q.device)
        asym = not self.symmetric
        many = len(self.classes) > 1
        # side streams for the bit-width classes only where the call is large enough to gain from
        # them (or a graph is being recorded); small calls stay on the caller's stream and skip
        # every stream lookup
        side = None
        if many and self.concurrent_classes and (
                4.0 * q.shape[0] * q.shape[1] * q.shape[2] * self.len * self.D >= self.concurrent_min_flops
                or torch.cuda.is_current_stream_capturing()):
            side = self._side_streams(q.device)
            main = torch.cuda.current_stream(q.device)
            self._fork.record(main)
        splits = 1 if many and self.concurrent_classes else self.splits   # classes side by side fill the device already;
        for i, c in enumerate(self.classes):                              # the same rule on one stream, so both ways add up alike
            # classes cover disjoint heads and disjoint rows of `out`: with side streams their
            # launches share the GPU instead of queueing behind each other half-empty
            args = (q, c.k_words, c.k_scale, c.k_zp if asym else None, c.v_words, c.v_scale, c.v_zp if asym else None,
                    c.bits, c.bits, self.len, softmax_scale)
            kw = dict(kv_limit=kv_limit, head_map=c.head_map if many else None, out=out, splits=splits, exact_codes=exact_codes,
                      out_layout=out_layout)
            if side and i:
                stream = side[i - 1]
                stream.wait_event(self._fork)
                with torch.cuda.stream(stream):
                    ops.fused_attn(*args, **kw)
                self._join[i - 1].record(stream)
                main.wait_event(self._join[i - 1])
            else:
                ops.fused_attn(*args, **kw)
        return out

    def _side_streams(self, device):
        """One extra stream (default priority) per bit-width class beyond the first, with the
        events that order them after and before the caller's stream."""
        if self._side is None:
            n = len(self.classes) - 1
            self._side = [torch.cuda.Stream(device=device) for _ in range(n)]
            self._fork = torch.cuda.Event()
            self._join = [torch.cuda.Event() for _ in range(n)]
        return self._side

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

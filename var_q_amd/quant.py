"""Drop-in for the reference class VAR_Q (VAR_Q/quant.py:52-230): quantizer plus
per-step KV cache state machine, on HIP kernels.

Same constructor arguments, methods (`quant`, `cache`, `dequant_current`,
`dequant_all`, `use_var_q`), readable attributes and error behaviour.  What
changes underneath:

* scale + codes + packing is one kernel chain (ops.quant_pack /
  ops.quant_pack_rows) instead of ~15 torch launches with fp32 temporaries;
* unpack + dequant is one kernel (ops.dequant_window);
* the cache lives in pre-allocated buffers that grow geometrically; a step is
  written in place instead of re-copying the whole cache with torch.cat
  (VAR_Q/quant.py:200-201).  `cached_item` / `cached_scale` are views of the
  valid part and hold the same values the reference's concatenations hold.

Behaviour kept on purpose, because callers can observe it:
* every method reduces over the batch dim (VAR_Q/quant.py:78-95);
* G_HEAD_DIM and G_TENSOR re-quantize cat(dequant_all(), item)
  (VAR_Q/quant.py:149-159); G_TENSOR then *appends* that re-quantized
  concatenation (the first branch of cache() matches it, VAR_Q/quant.py:196-201);
* dequantized tensors are fp32 (VAR_Q/quant.py:123-124).

Extensions (absent from the reference): `symmetric=False` selects the min/max
affine quantizer (attributes `zp`, `cached_zp`); quant_method 'G_GROUP' with
`group_size=g` quantizes g contiguous channels of each token independently
(batch and tokens not reduced); 'G_HEAD' keeps one scale per head;
`fused_attention(q, k_quant, v_quant, scale)` attends over two packed caches
without dequantizing them.
GPU tensors only.
"""
from typing import Dict, List, Optional, Tuple

import torch

from . import _lib, ops
from ._lib import VarqError, check, i64arr

_REF_METHODS = ('G_TENSOR', 'G_SCALE_HEAD_DIM', 'G_HEAD_DIM', 'G_SCALE', 'G_TOKEN', 'G_TOKEN_HEAD')
_EXT_METHODS = ('G_GROUP', 'G_HEAD')


def _dim_map(qkv_format: str) -> Dict[str, Tuple[int, ...]]:
    if qkv_format == 'BLHc':
        return {'G_TENSOR': (0, 1, 2, 3), 'G_SCALE_HEAD_DIM': (0, 1), 'G_HEAD_DIM': (0, 1), 'G_TOKEN': (0, 2, 3),
                'G_TOKEN_HEAD': (0, 3), 'G_SCALE': (0, 1, 2, 3), 'G_HEAD': (0, 1, 3), 'G_GROUP': (3,)}
    return {'G_TENSOR': (0, 1, 2, 3), 'G_SCALE_HEAD_DIM': (0, 2), 'G_HEAD_DIM': (0, 2), 'G_TOKEN': (0, 1, 3),
            'G_TOKEN_HEAD': (0, 3), 'G_SCALE': (0, 1, 2, 3), 'G_HEAD': (0, 2, 3), 'G_GROUP': (3,)}


class _Growable:
    """Buffer that grows along one dim; `view()` is the valid prefix."""

    def __init__(self, dim: int, min_capacity: int = 64):
        self.dim, self.buf, self.len = dim, None, 0
        self.min_capacity = min_capacity       # room of the first allocation (tokens)
        self._pending = []

    def append_later(self, t: torch.Tensor):
        """Append when the buffer is next looked at.  The cached scales of the reference are
        each step's scale expanded over the step's tokens (VAR_Q/quant.py:196-201): fp32 per
        code, four times the bytes of the 8-bit codes themselves; a caller that attends the packed
        cache through the tables never reads them."""
        self._pending.append(t)

    def _flush(self):
        pending, self._pending = self._pending, []
        for t in pending:
            self.append(t() if callable(t) else t)     # (a callable builds the expanded view when asked)

    def append(self, t: torch.Tensor):
        n = t.size(self.dim)
        if self.buf is None or self.len + n > self.buf.size(self.dim):
            cap = max(2 * (self.len + n), self.min_capacity)
            shape = list(t.shape)
            shape[self.dim] = cap
            new = torch.empty(shape, dtype=t.dtype, device=t.device)
            if self.buf is not None and self.len:
                new.narrow(self.dim, 0, self.len).copy_(self.buf.narrow(self.dim, 0, self.len))
            self.buf = new
        self.buf.narrow(self.dim, self.len, n).copy_(t)
        self.len += n

    def reserve(self, step_shape, dtype, device) -> Optional[torch.Tensor]:
        """Room for one more step of this shape behind the valid prefix (growing like append);
        the buffer, or None if it holds tensors of another shape or type."""
        n = step_shape[self.dim]
        if self.buf is not None:
            other = [i for i in range(len(step_shape)) if i != self.dim]
            if self.buf.dtype != dtype or self.buf.dim() != len(step_shape) or \
                    any(self.buf.size(i) != step_shape[i] for i in other):
                return None
        if self.buf is None or self.len + n > self.buf.size(self.dim):
            shape = list(step_shape)
            shape[self.dim] = max(2 * (self.len + n), self.min_capacity)
            new = torch.empty(shape, dtype=dtype, device=device)
            if self.buf is not None and self.len:
                new.narrow(self.dim, 0, self.len).copy_(self.buf.narrow(self.dim, 0, self.len))
            self.buf = new
        return self.buf

    def replace(self, t: torch.Tensor):
        self._pending = []
        self.buf, self.len = t, t.size(self.dim)

    def view(self) -> Optional[torch.Tensor]:
        self._flush()
        return None if self.buf is None else self.buf.narrow(self.dim, 0, self.len)


class VAR_Q:
    def __init__(self, quant_bits: int = 8, qkv_format: str = 'BLHc', quant_method: str = 'G_SCALE_HEAD_DIM',
                 blk_idx: int = 0, pack_to_int32: bool = True, eps: float = 1e-12, debug: bool = False,
                 symmetric: bool = True, group_size: Optional[int] = None, keep_dequantized: bool = False):
        assert qkv_format in ('BLHc', 'BHLc'), f"Invalid qkv_format: {qkv_format}"
        assert quant_method in _REF_METHODS + _EXT_METHODS, f"Invalid quant_method: {quant_method}"
        assert 1 < quant_bits <= 8, "Only support (2..8] bits (common 2/4/8 bits); bit-pack implementation covers 2/4/8 bits"
        if quant_method == 'G_GROUP':
            assert group_size is not None and group_size > 0, "G_GROUP needs group_size"
            assert pack_to_int32, "G_GROUP always packs"
        self.quant_bits = quant_bits
        self.quant_method = quant_method
        self.cur_blk_idx = blk_idx
        self.pack_to_int32 = pack_to_int32
        self.eps = eps
        self.debug = debug
        self.symmetric = symmetric
        self.group_size = group_size
        # use_var_q keeps the fp32 values it handed out from step to step (see use_var_q): faster,
        # and 4 bytes per cached element resident for the life of the quantizer.  Off unless asked for.
        self.keep_dequantized = keep_dequantized
        self.qkv_format = qkv_format   # property: also derives dim_cat / dim_map
        self.bound_min = -(2 ** (quant_bits - 1))
        self.bound_max = (2 ** (quant_bits - 1)) - 1

        self.quantized_item: Optional[torch.Tensor] = None
        self.scale: Optional[torch.Tensor] = None
        self.zp: Optional[torch.Tensor] = None
        self._pack_meta: Optional[Dict[str, int]] = None
        self._staged = None
        self._fast_plans: Dict[Tuple[int, int, int, int], tuple] = {}
        self._reset_cache()

    # The reference derives dim_cat/dim_map once in __init__ and callers later
    # assign `qkv_format` (Infinity/infinity/models/basic.py:309,314) without the
    # derived fields following.  Here the assignment re-derives them.
    @property
    def qkv_format(self) -> str:
        return self._qkv_format

    @qkv_format.setter
    def qkv_format(self, fmt: str):
        assert fmt in ('BLHc', 'BHLc'), f"Invalid qkv_format: {fmt}"
        self._qkv_format = fmt
        self.dim_cat = 1 if fmt == 'BLHc' else 2
        self.dim_map = _dim_map(fmt)

    # ---------------- cache views ----------------
    def _reset_cache(self):
        # what the fused attention reads, kept up to date by cache(): the end of every cached
        # step with its (head, channel) tables for the methods whose scale is shared by the
        # tokens of a step, a full-size copy of the per-token scales (shaped like the code buffer,
        # [.., capacity, .., groups]) for the others
        self._staged = None
        self._seg_ends: List[int] = []
        self._tab_scale: Optional[torch.Tensor] = None      # [MAX_TABLE_STEPS, H, c]
        self._tab_zp: Optional[torch.Tensor] = None
        room = max(64, getattr(self, '_reserved_tokens', 0))
        self._tok_scale = _Growable(self.dim_cat, room)
        self._tok_zp = _Growable(self.dim_cat, room)
        self._c_item = _Growable(self.dim_cat, room)
        self._c_scale = _Growable(self.dim_cat, room)
        self._c_zp = _Growable(self.dim_cat, room)
        # the dequantized cache as use_var_q hands it out, kept from step to step (see use_var_q)
        self._c_deq = _Growable(self.dim_cat, room)

    def reserve_tokens(self, n_tokens: int):
        """Size the cache buffers for n_tokens at their first allocation (an extension: the
        reference grows its cache by torch.cat, VAR_Q/quant.py:200-201; here the buffers double
        when they run out, and a caller that knows the schedule's length avoids those copies).
        Takes effect for buffers not allocated yet."""
        self._reserved_tokens = int(n_tokens)
        for g in (self._tok_scale, self._tok_zp, self._c_item, self._c_scale, self._c_zp, self._c_deq):
            g.min_capacity = max(64, self._reserved_tokens)

    @property
    def cached_item(self) -> Optional[torch.Tensor]:
        return self._c_item.view()

    @property
    def cached_scale(self) -> Optional[torch.Tensor]:
        return self._c_scale.view()

    @property
    def cached_zp(self) -> Optional[torch.Tensor]:
        return self._c_zp.view()

    # ---------------- quantize ----------------
    def _quantize(self, x: torch.Tensor):
        if not isinstance(x, torch.Tensor) or not x.is_cuda:
            raise VarqError('VAR_Q requires GPU tensors; there is no CPU path in this package')
        m = self.quant_method
        self._staged = None
        if m == 'G_GROUP':
            q, s, z = ops.quant_pack_rows(x, self.group_size, self.quant_bits, asym=not self.symmetric, eps=self.eps)
            return q, s, z
        # The methods that append (VAR_Q/quant.py:196-201) write the step's codes where cache()
        # would copy them: behind the valid prefix of the cache buffer.  `quantized_item` is then
        # a window of that buffer, and cache() only moves the end of the prefix.
        buf = None
        if m not in ('G_HEAD_DIM', 'G_TENSOR') and x.dim() == 4 and self._c_item.dim == self.dim_cat:
            c = x.shape[3]
            last = (c + 32 // self.quant_bits - 1) // (32 // self.quant_bits) if self.pack_to_int32 else c
            buf = self._c_item.reserve(list(x.shape[:3]) + [last], torch.int32 if self.pack_to_int32 else torch.int8,
                                       x.device)
        if buf is None:
            return ops.quant_pack(x, self.dim_map[m], self.quant_bits, asym=not self.symmetric, eps=self.eps,
                                  pack=self.pack_to_int32)
        # likewise the scale of a per-(head, channel) method goes straight into the row of the
        # step tables that cache() would copy it to (`scale` is then a view of that row)
        s_out = z_out = None
        k = len(self._seg_ends)
        if m == 'G_SCALE_HEAD_DIM' and self.pack_to_int32 and k < MAX_TABLE_STEPS:
            H = x.shape[1 if self.qkv_format == 'BHLc' else 2]
            self._table_rows(H, x.shape[3], x.device)
            s_out = self._tab_scale[k]
            z_out = None if self.symmetric else self._tab_zp[k]
        q, s, z = ops.quant_pack(x, self.dim_map[m], self.quant_bits, asym=not self.symmetric, eps=self.eps,
                                 pack=self.pack_to_int32, out=buf, out_token_dim=self.dim_cat,
                                 out_token=self._c_item.len, scale_out=s_out, zp_out=z_out)
        self._staged = (buf, self._c_item.len, q)
        return q, s, z

    def _table_rows(self, H: int, c: int, device):
        if self._tab_scale is None or self._tab_scale.shape[1:] != (H, c):
            self._tab_scale = torch.empty((MAX_TABLE_STEPS, H, c), dtype=torch.float32, device=device)
            self._tab_zp = None if self.symmetric else torch.empty_like(self._tab_scale)

    def quant(self, item: torch.Tensor):
        m = self.quant_method
        if m in ('G_HEAD_DIM', 'G_TENSOR') and self.cached_item is not None and self.cached_scale is not None:
            item = torch.cat([self.dequant_all(), item], dim=self.dim_cat)
        elif m not in _REF_METHODS + _EXT_METHODS:
            raise ValueError(f"[VAR-Q]: Invalid quantization method: {m}")
        if self.pack_to_int32:
            assert self.quant_bits in (2, 4, 8), "bit-pack only implements 2/4/8 bits"
        if item.numel() == 0:
            # (the reference fails in its amax over an empty dim, VAR_Q/quant.py:113)
            raise RuntimeError(f'[VAR-Q]: nothing to quantize: item of shape {tuple(item.shape)}')
        q, s, z = self._quantize(item)
        if self.pack_to_int32:
            c, vals = item.shape[-1], 32 // self.quant_bits
            meta = {'orig_c': int(c), 'vals_per_word': int(vals), 'pad_len': int((-c) % vals), 'bits': int(self.quant_bits)}
            if self._pack_meta is not None:
                assert meta['bits'] == self._pack_meta['bits']
                assert meta['vals_per_word'] == self._pack_meta['vals_per_word']
                assert meta['orig_c'] == self._pack_meta['orig_c']
                assert meta['pad_len'] == self._pack_meta['pad_len']
            self._pack_meta = meta
        self.quantized_item, self.scale, self.zp = q, s, z

    def _fast_prepare(self, x: torch.Tensor):
        """First half of the one-call step (see `_step_fast`): room in the cache buffer and the
        table row for a step of the shipped rule, nothing launched, no state changed.  None
        when the quantizer or the item is of another kind."""
        bits = self.quant_bits
        if isinstance(x, torch.Tensor) and x.numel() == 0:
            return None                       # (quant() says why an empty step is refused)
        if self.quant_method != 'G_SCALE_HEAD_DIM' or not self.pack_to_int32 or bits not in (2, 4, 8):
            return None
        if not isinstance(x, torch.Tensor) or x.dim() != 4 or not x.is_cuda or not x.is_contiguous() \
                or x.dtype not in ops._DT or self._c_item.dim != self.dim_cat:
            return None
        k = len(self._seg_ends)
        s0, s1, s2, c = x.shape
        vals = 32 // bits
        if k >= MAX_TABLE_STEPS or c % vals or s0 * s1 * s2 == 0:
            return None
        bhl = self._qkv_format == 'BHLc'
        H, n = (s1, s2) if bhl else (s2, s1)
        buf = self._c_item.reserve([s0, s1, s2, c // vals], torch.int32, x.device)
        if buf is None:
            return None
        meta = {'orig_c': int(c), 'vals_per_word': int(vals), 'pad_len': 0, 'bits': int(bits)}
        if self._pack_meta is not None and self._pack_meta != meta:
            return None                       # (quant() raises the reference's assertion for this)
        self._table_rows(H, c, x.device)
        plan = self._fast_plans.get((s0, s1, s2, c))
        if plan is None:
            sh = i64arr([s0, s1, s2, c])
            mask = 0b0101 if bhl else 0b0011                      # reduce batch and tokens
            ws_bytes = max(int(_lib.load().varq_quant_workspace_bytes(sh, mask)), 8)
            plan = self._fast_plans[(s0, s1, s2, c)] = (sh, mask, ws_bytes)
        start, cap, per_tok = self._c_item.len, buf.shape[self.dim_cat], (1 if bhl else H)
        out_map = (n * per_tok, (cap - n) * per_tok, start * per_tok)
        srow = self._tab_scale[k]
        zrow = None if self.symmetric else self._tab_zp[k]
        return (x, buf, srow, zrow, plan, out_map, meta, bhl, H, n, c, start)

    def _fast_commit(self, prep):
        """Second half: the state that quant() followed by cache() leaves, the kernels having
        written the codes and the table row in place."""
        x, buf, srow, zrow, plan, out_map, meta, bhl, H, n, c, start = prep
        sshape = (1, H, 1, c) if bhl else (1, 1, H, c)
        self.quantized_item = buf.narrow(self.dim_cat, start, n)
        self.scale = srow.view(sshape)
        self.zp = None if zrow is None else zrow.view(sshape)
        self._pack_meta = meta
        self._staged = None
        self._c_item.len = start + n
        eshape = (-1, -1, n, -1) if bhl else (-1, n, -1, -1)
        scale, zp = self.scale, self.zp
        self._c_scale.append_later(lambda: scale.expand(*eshape))
        if zp is not None:
            self._c_zp.append_later(lambda: zp.expand(*eshape))
        self._seg_ends.append((self._seg_ends[-1] if self._seg_ends else 0) + n)

    def _step_fast(self, x: torch.Tensor) -> bool:
        """quant(x) followed by cache() for the shipped rule (G_SCALE_HEAD_DIM, packed codes)
        with the host work of a generation step cut to one library call: same kernels, same
        state afterwards.  False (nothing done) when the quantizer or the item is of another
        kind; the caller then takes the two general calls."""
        prep = self._fast_prepare(x)
        if prep is None:
            return False
        _, buf, srow, zrow, (sh, mask, ws_bytes), out_map, *_ = prep
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
        with ops._on_device(x.device):
            check(_lib.load().varq_quant_pack(x.data_ptr(), ops._DT[x.dtype], sh, mask, self.quant_bits,
                                              int(not self.symmetric), self.eps, buf.data_ptr(), None, srow.data_ptr(),
                                              None if zrow is None else zrow.data_ptr(), i64arr(out_map),
                                              ws.data_ptr(), ws_bytes, ops._stream(x)), 'varq_quant_pack')
        self._fast_commit(prep)
        return True

    @staticmethod
    def _step_fast_pair(kq: 'VAR_Q', vq: 'VAR_Q', k: torch.Tensor, v: torch.Tensor) -> bool:
        """`_step_fast` for K and V of a step in the same three launches, when the two
        quantizers are configured alike and their caches stand at the same place."""
        if not (isinstance(k, torch.Tensor) and isinstance(v, torch.Tensor)):
            return False
        if kq is vq or kq.quant_bits != vq.quant_bits or kq.symmetric != vq.symmetric or kq.eps != vq.eps \
                or kq._qkv_format != vq._qkv_format or k.shape != v.shape or k.dtype != v.dtype or k.device != v.device:
            return False
        pk = kq._fast_prepare(k)
        if pk is None:
            return False
        pv = vq._fast_prepare(v)
        if pv is None or pk[5] != pv[5]:          # (same window of the two cache buffers)
            return False
        sh, mask, ws_bytes = pk[4]
        ws = torch.empty(2 * ws_bytes, dtype=torch.uint8, device=k.device)
        zk, zv = pk[3], pv[3]
        with ops._on_device(k.device):
            check(_lib.load().varq_quant_pack2(k.data_ptr(), v.data_ptr(), ops._DT[k.dtype], sh, mask, kq.quant_bits,
                                               int(not kq.symmetric), kq.eps,
                                               pk[1].data_ptr(), None, pk[2].data_ptr(), None if zk is None else zk.data_ptr(),
                                               pv[1].data_ptr(), None, pv[2].data_ptr(), None if zv is None else zv.data_ptr(),
                                               i64arr(pk[5]), ws.data_ptr(), 2 * ws_bytes, ops._stream(k)),
                  'varq_quant_pack2')
        kq._fast_commit(pk)
        vq._fast_commit(pv)
        return True

    # ---------------- cache ----------------
    def _expand_scale_like_L(self, q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
        d = 1 if self.qkv_format == 'BLHc' else 2
        if scale.size(d) == 1 and q.size(d) > 1:
            shape = [-1, -1, -1, -1]
            shape[d] = q.size(d)
            scale = scale.expand(*shape)
        return scale

    def cache(self):
        m = self.quant_method
        q_cur = self.quantized_item
        s_cur = self._expand_scale_like_L(q_cur, self.scale)
        z_cur = None if self.zp is None else self._expand_scale_like_L(q_cur, self.zp)
        if m in ('G_SCALE_HEAD_DIM', 'G_SCALE', 'G_TOKEN', 'G_TOKEN_HEAD', 'G_TENSOR', 'G_GROUP', 'G_HEAD'):
            if self._c_item.dim != self.dim_cat:
                # the layout was re-assigned: fine before the first step, an error once steps are
                # cached (their tokens lie along the other dim; dropping them silently would leave
                # the generation running on a truncated cache)
                if self._c_item.len > 0:
                    raise ValueError('VAR_Q: qkv_format was changed to %s with %d tokens cached in the other layout'
                                     % (self.qkv_format, self._c_item.len))
                self._reset_cache()
            st, self._staged = self._staged, None
            if st is not None and st[0] is self._c_item.buf and st[1] == self._c_item.len and st[2] is q_cur:
                self._c_item.len += q_cur.size(self.dim_cat)      # the codes are in place already
            else:
                self._c_item.append(q_cur)
            self._c_scale.append_later(s_cur)
            if z_cur is not None:
                self._c_zp.append_later(z_cur)
            self._note_step(q_cur, replace=False)
        elif m == 'G_HEAD_DIM':
            self._c_item.replace(q_cur)
            self._c_scale.replace(s_cur)
            if z_cur is not None:
                self._c_zp.replace(z_cur)
            self._note_step(q_cur, replace=True)
        else:
            raise ValueError(f"[VAR-Q]: Invalid quantization method: {m}")

    def _note_step(self, q_cur: torch.Tensor, replace: bool):
        """Book-keeping for `fused_attention` (packed codes only)."""
        if not self.pack_to_int32:
            return
        if self._tok_scale.dim != self.dim_cat:   # layout was re-assigned before the first step
            room = self._c_item.min_capacity
            self._tok_scale, self._tok_zp = _Growable(self.dim_cat, room), _Growable(self.dim_cat, room)
        bhl = self.qkv_format == 'BHLc'
        B, H, n = q_cur.shape[0], q_cur.shape[1 if bhl else 2], q_cur.shape[2 if bhl else 1]
        c = self._pack_meta['orig_c']
        full = (1, H, 1, c) if bhl else (1, 1, H, c)
        if self.quant_method in _TABLE_METHODS:
            if replace:
                self._seg_ends = []
            k = len(self._seg_ends)
            self._seg_ends.append((self._seg_ends[-1] if self._seg_ends else 0) + n)
            if k >= MAX_TABLE_STEPS:
                return                                   # fused_attention refuses; the drop-in path is unaffected
            if self._tab_scale is None:
                self._table_rows(H, c, q_cur.device)
            if self.scale.data_ptr() != self._tab_scale[k].data_ptr():   # (else quant() wrote the row itself)
                self._tab_scale[k].copy_(self.scale.expand(*full).reshape(H, c))
                if self.zp is not None:
                    self._tab_zp[k].copy_(self.zp.expand(*full).reshape(H, c))
        else:
            ng = self.scale.shape[3]
            shape = (B, H, n, ng) if bhl else (B, n, H, ng)
            self._tok_scale.append(self.scale.expand(*shape))
            if self.zp is not None:
                self._tok_zp.append(self.zp.expand(*shape))

    # ---------------- dequantize ----------------
    def _dequant(self, q: torch.Tensor, scale: torch.Tensor, zp: Optional[torch.Tensor],
                 out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        if self.pack_to_int32:
            assert self._pack_meta is not None, "pack meta is missing"
            c = self._pack_meta['orig_c']
        else:
            c = q.shape[-1]
        return _dequant_views(q, scale, zp, c, self.quant_bits, out_dtype)

    def dequant_current(self, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        return self._dequant(self.quantized_item, self.scale, self.zp, out_dtype)

    def dequant_all(self, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """The whole cache dequantized (VAR_Q/quant.py:216-224: fp32).  out_dtype bfloat16 / float16
        gives the fp32 product rounded once to that type -- bit for bit what `.to(out_dtype)` of the
        fp32 result is, without writing and re-reading the fp32 tensor."""
        if self.cached_item is None:
            return self.dequant_current(out_dtype)
        return self._dequant(self.cached_item, self.cached_scale, self.cached_zp, out_dtype)

    def use_var_q(self, item: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        """quant + cache + dequant_all (VAR_Q/quant.py:226-230).  Like the reference, the whole
        cache is dequantized into a fresh fp32 tensor at every step and nothing of it is kept.
        out_dtype (an addition): the type the caller would cast the result to anyway (the attention
        modules do, VAR/models/basic_var.py:158); see dequant_all.  Ignored with keep_dequantized.

        With `keep_dequantized=True` (constructor) the fp32 values are kept from step to step
        instead: under the appending methods the codes and scales of earlier steps never change,
        so only the new step is dequantized and put behind them -- the same values (the step's
        scale is what the expanded cached scale holds for its tokens), O(step) instead of
        O(cache) per call.  The result is then the valid prefix of that buffer (like
        `cached_item`, a view that is not contiguous when the buffer has room to spare).  The
        price is memory: 4 bytes per cached element (up to 8 while the buffer has doubled), i.e.
        two to four times an unquantized bf16 cache, resident until the quantizer is deleted --
        172 MB per tensor at [2,16,10521,128].  `dequant_all()` itself always recomputes everything."""
        self.quant(item)
        self.cache()
        if not self.keep_dequantized:
            return self.dequant_all(out_dtype or torch.float32)
        d, n = self._c_deq, self.quantized_item.size(self.dim_cat)
        if self.quant_method == 'G_HEAD_DIM' or self._c_item.buf is None or d.dim != self.dim_cat or d.len + n != self._c_item.len:
            # (the replacing method; or the kept values are not those of the cache's earlier steps:
            # quant() and cache() were also called on their own, or the layout was re-assigned)
            full = self.dequant_all()
            if self.quant_method != 'G_HEAD_DIM' and self._c_item.buf is not None:
                self._c_deq = _Growable(self.dim_cat, self._c_item.min_capacity)
                self._c_deq.append(full)
            return full
        d.append(self.dequant_current())
        return d.view()


def _dequant_views(q: torch.Tensor, scale: torch.Tensor, zp: Optional[torch.Tensor], c: int, bits: int,
                   out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Dequantize codes given as a (possibly strided) 4-D view of a cache buffer
    whose rows are dense, with a scale that is any broadcastable strided view."""
    assert q.dim() == 4 and scale.dim() == 4
    n0, n1, n2, wq = q.shape
    assert q.stride(3) == 1 and all(st % wq == 0 for st in q.stride()[:3]), 'rows of the code tensor must be dense'
    rowmap = [n0, n1, n2, q.stride(0) // wq, q.stride(1) // wq, q.stride(2) // wq, 0, -1]
    if zp is not None and (zp.shape != scale.shape or zp.stride() != scale.stride()):
        scale, zp = scale.contiguous(), zp.expand_as(scale).contiguous()
    s3 = scale.shape[3]
    assert c % s3 == 0
    group = c // s3
    strides = [0 if scale.shape[d] == 1 else scale.stride(d) for d in range(4)]
    for d in range(3):
        assert scale.shape[d] in (1, q.shape[d]), f'scale dim {d}: {scale.shape[d]} vs {q.shape[d]}'
    return ops.dequant_window(q, scale, zp, (n0, n1, n2, c), strides, group, bits, rowmap, out_dtype)


# methods whose scale does not depend on the token: one table per cached step
_TABLE_METHODS = ('G_SCALE_HEAD_DIM', 'G_HEAD_DIM', 'G_TENSOR', 'G_SCALE', 'G_HEAD')
# methods with one scale (per channel group) per token
_TOKEN_METHODS = ('G_TOKEN', 'G_TOKEN_HEAD', 'G_GROUP')
MAX_TABLE_STEPS = 16


def fused_attention(q: torch.Tensor, k_quant: VAR_Q, v_quant: VAR_Q, softmax_scale: float,
                    kv_limit: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """softmax(scale * q K^T) V over the packed caches of two quantizers, without the
    dequantized full-length K/V that `dequant_all` would produce (the reference computes
    exactly that and hands it to its attention backend: VAR_Q/quant.py:216-230,
    Infinity/infinity/models/basic.py:339-351).

    q [B,H,Lq,c] for quantizers in layout 'BHLc', [B,Lq,H,c] for 'BLHc' (the layout of the
    reference's flash-attention call and of VAR-VAR_Q-8.json).  The attention runs in q's dtype
    when that is fp16 and c = 64 -- the VAR path, whose attention call casts q, k and v to fp16
    (VAR/models/basic_var.py:157-158 under the fp16 autocast of scripts/inference_multi_VAR.py:123)
    -- and in bf16 otherwise (q is cast); dequantized K and V are rounded to that type, as the
    reference's downcast does.  Both quantizers in
    the same layout, packed, same bit-width, c in {64, 128}, after at least one `cache()`.  Methods whose scale is shared by the
    tokens of a step (G_SCALE_HEAD_DIM -- the shipped rule --, G_HEAD_DIM, G_TENSOR, G_SCALE,
    G_HEAD) go through one table per cached step, at most MAX_TABLE_STEPS steps; per-token
    methods (G_TOKEN, G_TOKEN_HEAD, G_GROUP) through per-token scales.  Everything the
    kernels read is kept current by `cache()`, so a call launches the attention and nothing
    else.  kv_limit: int32 [Lq], query i sees keys j < kv_limit[i].  Returns a tensor of the
    attention's dtype in the shape of q."""
    layout = k_quant.qkv_format
    if v_quant.qkv_format != layout:
        raise ValueError(f'fused_attention: K is cached in layout {layout}, V in {v_quant.qkv_format}')
    for qz, n in ((k_quant, 'k_quant'), (v_quant, 'v_quant')):
        if not qz.pack_to_int32 or qz.cached_item is None:
            raise ValueError(f'fused_attention: {n} needs a packed cache (pack_to_int32=True, after cache())')
    bits = k_quant.quant_bits
    if v_quant.quant_bits != bits:
        raise ValueError('fused_attention: K and V must use the same bit-width')
    kbuf, vbuf = k_quant._c_item.buf, v_quant._c_item.buf
    Lk = k_quant._c_item.len
    if v_quant._c_item.len != Lk or kbuf.shape != vbuf.shape:
        raise ValueError('fused_attention: the K and V caches differ in length or capacity')
    bhl = layout == 'BHLc'
    B, H, cap = kbuf.shape[0], kbuf.shape[1 if bhl else 2], kbuf.shape[2 if bhl else 1]
    c = k_quant._pack_meta['orig_c']
    if c not in (64, 128):
        raise ValueError(f'fused_attention: head dim {c} not supported (64 or 128)')
    q = (q if (q.dtype == torch.float16 and c == 64) else q.to(torch.bfloat16)).contiguous()
    assert q.dim() == 4 and q.shape[0] == B and q.shape[1 if bhl else 2] == H and q.shape[3] == c, \
        'q must be [B,H,Lq,c] (BHLc) or [B,Lq,H,c] (BLHc)'
    km, vm = k_quant.quant_method, v_quant.quant_method
    if km in _TABLE_METHODS and vm in _TABLE_METHODS:
        ends = k_quant._seg_ends
        if ends != v_quant._seg_ends:
            raise ValueError('fused_attention: K and V were cached in different steps')
        if len(ends) > MAX_TABLE_STEPS or not ends or ends[-1] != Lk:
            raise ValueError(f'fused_attention: at most {MAX_TABLE_STEPS} cached steps, the same for K and V')
        return ops.fused_attn_channel(q, kbuf, k_quant._tab_scale, k_quant._tab_zp, vbuf, v_quant._tab_scale,
                                      v_quant._tab_zp, bits, Lk, softmax_scale, kv_limit=kv_limit, out=out,
                                      seg_ends=ends, layout=layout)
    if km in _TOKEN_METHODS and vm in _TOKEN_METHODS:
        ks, kz, vs, vz = k_quant._tok_scale.buf, k_quant._tok_zp.buf, v_quant._tok_scale.buf, v_quant._tok_zp.buf
        if ks.shape[:3] != kbuf.shape[:3] or vs.shape[:3] != kbuf.shape[:3]:
            raise ValueError('fused_attention: scale buffers and code buffers differ in capacity')
        return ops.fused_attn(q, kbuf, ks, kz, vbuf, vs, vz, bits, bits, Lk, softmax_scale, kv_limit=kv_limit, out=out,
                              layout=layout)
    raise ValueError(f'fused_attention: methods {km} / {vm} cannot be combined')


def fused_step(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_quant: VAR_Q, v_quant: VAR_Q, softmax_scale: float,
               kv_limit: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One generation step on the packed caches: quantize and cache the step's K and V with
    their quantizers (`quant` + `cache`, VAR_Q/quant.py:232-235 without the dequantization),
    then `fused_attention` of q over everything cached.  For the shipped rule K and V are
    quantized by one library call (three launches for both); any other rule goes through the
    general methods."""
    if isinstance(k, torch.Tensor) and isinstance(v, torch.Tensor):
        k, v = k.contiguous(), v.contiguous()      # (views of a qkv projection; the quantizers need dense rows)
    if not VAR_Q._step_fast_pair(k_quant, v_quant, k, v):
        for quantizer, item in ((k_quant, k), (v_quant, v)):
            if not quantizer._step_fast(item):
                quantizer.quant(item)
                quantizer.cache()
    return fused_attention(q, k_quant, v_quant, softmax_scale, kv_limit=kv_limit, out=out)

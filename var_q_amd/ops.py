"""Tensor-level entry points over the C ABI of libvarq_hip.so.

torch is used here for device memory and the current stream only; all
arithmetic happens in the HIP kernels.  Every function requires GPU tensors and
raises otherwise -- there is no CPU path in the product.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import ctypes

import torch

from . import _lib
from ._lib import VarqError, check, i64arr

_DT = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def _gpu(t: torch.Tensor, name: str) -> torch.Tensor:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        dev = getattr(t, 'device', type(t))
        raise VarqError(f'{name} must be a GPU tensor (got {dev}); the VAR-Q HIP path has no CPU fallback')
    return t


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)


def _stream(t: torch.Tensor) -> int:
    """Handle of the current stream of the tensor's device."""
    if _raw_stream is not None:
        idx = t.device.index
        return _raw_stream(torch.cuda.current_device() if idx is None else idx)
    return torch.cuda.current_stream(t.device).cuda_stream


class _on_device:
    """`with torch.cuda.device(d)` that does nothing when d is current already (every call here
    is on the hot path of a generation step)."""
    __slots__ = ('idx', 'prev')

    def __init__(self, device: torch.device):
        self.idx, self.prev = device.index, -1

    def __enter__(self):
        cur = torch.cuda.current_device()
        if self.idx is not None and cur != self.idx:
            self.prev = cur
            torch.cuda.set_device(self.idx)

    def __exit__(self, *exc):
        if self.prev >= 0:
            torch.cuda.set_device(self.prev)


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _dt(t: torch.Tensor) -> int:
    if t.dtype not in _DT:
        raise VarqError(f'unsupported dtype {t.dtype}; expected float32, bfloat16 or float16')
    return _DT[t.dtype]


# ---------------------------------------------------------------------------
# row-local (group-wise along the last dim) quantize + pack
# ---------------------------------------------------------------------------
def _check_cache_buffers(c: int, group: int, bits: int, asym: bool, words: torch.Tensor, scale: torch.Tensor,
                         zp: Optional[torch.Tensor], rowmap: Sequence[int], what: str) -> None:
    """The kernels trust the row map: make sure the buffers it points into have the row
    lengths the call implies and enough rows for the map's last row (dims addressed
    through a slot table count from their first slot)."""
    W, ng = c * bits // 32, c // group
    if words.shape[-1] != W or scale.shape[-1] != ng:
        raise VarqError(f'{what}: words / scale rows of {words.shape[-1]} / {scale.shape[-1]} entries, expected {W} / {ng}')
    if asym and (zp is None or zp.shape != scale.shape or zp.dtype != torch.float32 or not zp.is_contiguous()):
        raise VarqError(f'{what}: asym needs a contiguous fp32 zp buffer of the shape of scale')
    n, os_, off, slot_dim = rowmap[0:3], rowmap[3:6], rowmap[6], rowmap[7]
    last = off + sum((n[d] - 1) * os_[d] for d in range(3) if d != slot_dim and n[d] > 0)
    rows = min(words.numel() // W, scale.numel() // ng)
    if min(n) > 0 and not 0 <= last < rows:
        raise VarqError(f'{what}: the row map reaches row {last} of buffers that hold {rows} rows')


def quant_pack_rows(x: torch.Tensor, group: int, bits: int, asym: bool = True, eps: float = 1e-12
                    ) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """One-pass quantize+pack with one (scale[, zp]) per `group` contiguous
    channels of each row.  x [..., c] -> (words [..., c*bits/32] int32,
    scale [..., c/group] fp32, zp like scale or None)."""
    _gpu(x, 'x')
    x = x.contiguous()
    *lead, c = x.shape
    n_rows = x.numel() // c if c else 0
    words = torch.empty((*lead, c * bits // 32), dtype=torch.int32, device=x.device)
    scale = torch.empty((*lead, c // group), dtype=torch.float32, device=x.device)
    zp = torch.empty_like(scale) if asym else None
    lib = _lib.load()
    with _on_device(x.device):
        check(lib.varq_quant_pack_rows(x.data_ptr(), _dt(x), n_rows, c, group, bits, int(asym), eps, None, None,
                                       words.data_ptr(), scale.data_ptr(), _ptr(zp), _stream(x)), 'varq_quant_pack_rows')
    return words, scale, zp


def quant_pack_rows_into(x: torch.Tensor, group: int, bits: int, asym: bool, eps: float,
                         words: torch.Tensor, scale: torch.Tensor, zp: Optional[torch.Tensor],
                         rowmap: Sequence[int], slot: Optional[torch.Tensor] = None) -> None:
    """Same kernel writing into pre-allocated cache buffers through a row map
    {n0,n1,n2,os0,os1,os2,off,slot_dim} (see include/varq.h)."""
    _gpu(x, 'x'); _gpu(words, 'words'); _gpu(scale, 'scale')
    assert x.is_contiguous() and words.is_contiguous() and scale.is_contiguous()
    assert words.dtype == torch.int32 and scale.dtype == torch.float32
    c = x.shape[-1]
    n_rows = x.numel() // c
    assert rowmap[0] * rowmap[1] * rowmap[2] == n_rows
    _check_cache_buffers(c, group, bits, asym, words, scale, zp, rowmap, 'quant_pack_rows_into')
    lib = _lib.load()
    with _on_device(x.device):
        check(lib.varq_quant_pack_rows(x.data_ptr(), _dt(x), n_rows, c, group, bits, int(asym), eps, i64arr(rowmap),
                                       _ptr(slot), words.data_ptr(), scale.data_ptr(), _ptr(zp), _stream(x)),
              'varq_quant_pack_rows')


def quant_pack_rows_pair_into(x0: torch.Tensor, x1: torch.Tensor, group: int, bits: int, asym: bool, eps: float,
                              out0: Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]],
                              out1: Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]],
                              rowmap: Sequence[int], slot: Optional[torch.Tensor] = None) -> None:
    """Two tensors of one shape and dtype (K and V of a cache step) in one launch; out0 / out1
    = (words, scale, zp) buffers of each, addressed through the shared row map."""
    _gpu(x0, 'x0'); _gpu(x1, 'x1')
    assert x0.shape == x1.shape and x0.dtype == x1.dtype and x0.is_contiguous() and x1.is_contiguous()
    for w, s, z in (out0, out1):
        _gpu(w, 'words'); _gpu(s, 'scale')
        assert w.is_contiguous() and s.is_contiguous() and w.dtype == torch.int32 and s.dtype == torch.float32
    c = x0.shape[-1]
    n_rows = x0.numel() // c
    assert rowmap[0] * rowmap[1] * rowmap[2] == n_rows
    for w, s_, z in (out0, out1):
        _check_cache_buffers(c, group, bits, asym, w, s_, z, rowmap, 'quant_pack_rows_pair_into')
    lib = _lib.load()
    with _on_device(x0.device):
        check(lib.varq_quant_pack_rows2(x0.data_ptr(), x1.data_ptr(), _dt(x0), n_rows, c, group, bits, int(asym), eps,
                                        i64arr(rowmap), _ptr(slot),
                                        out0[0].data_ptr(), out0[1].data_ptr(), _ptr(out0[2]),
                                        out1[0].data_ptr(), out1[1].data_ptr(), _ptr(out1[2]), _stream(x0)),
              'varq_quant_pack_rows2')


# ---------------------------------------------------------------------------
# general (cross-row groups) quantize + pack
# ---------------------------------------------------------------------------
def quant_pack(x: torch.Tensor, reduce_dims: Sequence[int], bits: int, asym: bool = False, eps: float = 1e-12,
               pack: bool = True, out: Optional[torch.Tensor] = None, out_token_dim: Optional[int] = None,
               out_token: int = 0, scale_out: Optional[torch.Tensor] = None,
               zp_out: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Quantize a 4-D tensor with one group per index of the non-reduced dims.
    Returns (packed int32 words or int8 codes, scale with keepdim shape, zp or None).
    out / out_token_dim / out_token: write the codes into tokens out_token.. of a larger
    contiguous buffer that has the shape of the result except for more room along
    out_token_dim (1 or 2); the returned codes are that window of `out`.  scale_out, zp_out:
    contiguous fp32 buffers of n_groups elements that receive the scale and zero-point."""
    _gpu(x, 'x')
    assert x.dim() == 4, 'expected a 4-D [B,L,H,c] / [B,H,L,c] tensor'
    x = x.contiguous()
    shape = list(x.shape)
    mask = 0
    for d in reduce_dims:
        mask |= 1 << (d % 4)
    sshape = [1 if (mask >> d) & 1 else shape[d] for d in range(4)]
    n_groups = sshape[0] * sshape[1] * sshape[2] * sshape[3]
    if scale_out is not None:
        _gpu(scale_out, 'scale_out')
        assert scale_out.dtype == torch.float32 and scale_out.is_contiguous() and scale_out.numel() == n_groups
        scale = scale_out.view(sshape)
    else:
        scale = torch.empty(sshape, dtype=torch.float32, device=x.device)
    zp = None
    if asym:
        if zp_out is not None:
            _gpu(zp_out, 'zp_out')
            assert zp_out.dtype == torch.float32 and zp_out.is_contiguous() and zp_out.numel() == n_groups
            zp = zp_out.view(sshape)
        else:
            zp = torch.empty(sshape, dtype=torch.float32, device=x.device)
    c = shape[3]
    last = (c + 32 // bits - 1) // (32 // bits) if pack else c
    out_map = None
    if out is not None:
        _gpu(out, 'out')
        d = out_token_dim
        assert d in (1, 2) and out.is_contiguous() and out.dtype == (torch.int32 if pack else torch.int8)
        want = shape[:3] + [last]
        assert all(out.shape[i] == want[i] for i in range(4) if i != d) and 0 <= out_token <= out.shape[d] - shape[d], \
            f'out {tuple(out.shape)} has no room for {want} at token {out_token} of dim {d}'
        inner = shape[d] * (shape[2] if d == 1 else 1)            # rows of one block along the token dim
        per_tok = shape[2] if d == 1 else 1
        out_map = i64arr([inner, (out.shape[d] - shape[d]) * per_tok, out_token * per_tok])
        q = out.narrow(d, out_token, shape[d])
        dst = out
    else:
        q = torch.empty((*shape[:3], last), dtype=torch.int32 if pack else torch.int8, device=x.device)
        dst = q
    lib = _lib.load()
    sh = i64arr(shape)
    ws_bytes = lib.varq_quant_workspace_bytes(sh, mask)
    ws = torch.empty(max(ws_bytes, 8), dtype=torch.uint8, device=x.device)
    with _on_device(x.device):
        check(lib.varq_quant_pack(x.data_ptr(), _dt(x), sh, mask, bits, int(asym), eps,
                                  dst.data_ptr() if pack else None, None if pack else dst.data_ptr(),
                                  scale.data_ptr(), _ptr(zp), out_map, ws.data_ptr(), ws.numel(), _stream(x)),
              'varq_quant_pack')
    return q, scale, zp


def quant_pack_pair(x0: torch.Tensor, x1: torch.Tensor, reduce_dims: Sequence[int], bits: int, asym: bool = False,
                    eps: float = 1e-12, pack: bool = True):
    """`quant_pack` of two tensors of one shape and dtype (K and V of a step) in the same
    launches.  Returns ((q0, scale0, zp0), (q1, scale1, zp1)), each as from `quant_pack`."""
    _gpu(x0, 'x0')
    _gpu(x1, 'x1')
    assert x0.dim() == 4 and x0.shape == x1.shape and x0.dtype == x1.dtype and x0.device == x1.device
    x0, x1 = x0.contiguous(), x1.contiguous()
    shape = list(x0.shape)
    mask = 0
    for d in reduce_dims:
        mask |= 1 << (d % 4)
    sshape = [1 if (mask >> d) & 1 else shape[d] for d in range(4)]
    c = shape[3]
    last = (c + 32 // bits - 1) // (32 // bits) if pack else c
    outs = []
    for _ in range(2):
        outs.append((torch.empty((*shape[:3], last), dtype=torch.int32 if pack else torch.int8, device=x0.device),
                     torch.empty(sshape, dtype=torch.float32, device=x0.device),
                     torch.empty(sshape, dtype=torch.float32, device=x0.device) if asym else None))
    lib = _lib.load()
    sh = i64arr(shape)
    ws_bytes = 2 * max(int(lib.varq_quant_workspace_bytes(sh, mask)), 8)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x0.device)
    (q0, s0, z0), (q1, s1, z1) = outs
    with _on_device(x0.device):
        check(lib.varq_quant_pack2(x0.data_ptr(), x1.data_ptr(), _dt(x0), sh, mask, bits, int(asym), eps,
                                   q0.data_ptr() if pack else None, None if pack else q0.data_ptr(), s0.data_ptr(), _ptr(z0),
                                   q1.data_ptr() if pack else None, None if pack else q1.data_ptr(), s1.data_ptr(), _ptr(z1),
                                   None, ws.data_ptr(), ws_bytes, _stream(x0)), 'varq_quant_pack2')
    return outs[0], outs[1]


# ---------------------------------------------------------------------------
# pack / unpack of int8 codes
# ---------------------------------------------------------------------------
def pack(codes: torch.Tensor, bits: int) -> torch.Tensor:
    _gpu(codes, 'q_int8')
    codes = codes.contiguous()
    *lead, c = codes.shape
    vals = 32 // bits
    rows = codes.numel() // c if c else 0
    words = torch.empty((*lead, (c + vals - 1) // vals), dtype=torch.int32, device=codes.device)
    lib = _lib.load()
    with _on_device(codes.device):
        check(lib.varq_pack(codes.data_ptr(), rows, c, bits, words.data_ptr(), _stream(codes)), 'varq_pack')
    return words


def unpack(words: torch.Tensor, c: int, bits: int) -> torch.Tensor:
    _gpu(words, 'packed')
    words = words.contiguous()
    *lead, w = words.shape
    rows = words.numel() // w if w else 0
    codes = torch.empty((*lead, c), dtype=torch.int8, device=words.device)
    lib = _lib.load()
    with _on_device(words.device):
        check(lib.varq_unpack(words.data_ptr(), rows, c, bits, codes.data_ptr(), _stream(words)), 'varq_unpack')
    return codes


# ---------------------------------------------------------------------------
# unpack + dequantize
# ---------------------------------------------------------------------------
def dequant(q: torch.Tensor, scale: torch.Tensor, zp: Optional[torch.Tensor], c: int, bits: int,
            out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """q: packed int32 words [n0,n1,n2,W] or int8 codes [n0,n1,n2,c].  scale
    (and zp) broadcast against [n0,n1,n2,c] in the first three dims and hold
    1, c/g or c entries in the last (per-row, group-wise, per-channel); any
    strides, including stride-0 expands, are used as they are."""
    _gpu(q, 'q'); _gpu(scale, 'scale')
    assert q.dim() == 4 and scale.dim() == 4
    q = q.contiguous()
    n0, n1, n2 = q.shape[:3]
    packed = q.dtype == torch.int32
    assert packed or q.dtype == torch.int8
    if zp is not None and (zp.shape != scale.shape or zp.stride() != scale.stride()):
        zp = zp.expand_as(scale).contiguous()
        scale = scale.contiguous()
    s3 = scale.shape[3]
    assert c % s3 == 0, f'scale last dim {s3} does not divide c={c}'
    group = c // s3
    strides = []
    for d in range(4):
        if scale.shape[d] == 1:
            strides.append(0)
        else:
            assert d == 3 or scale.shape[d] == q.shape[d], f'scale dim {d} = {scale.shape[d]} vs {q.shape[d]}'
            strides.append(scale.stride(d))
    out = torch.empty((n0, n1, n2, c), dtype=out_dtype, device=q.device)
    lib = _lib.load()
    # collapse the leading dims when the scale does not depend on them: fuller blocks
    shape = [n0, n1, n2, c]
    if strides[0] == 0 and strides[1] == 0 and strides[2] == 0:
        shape = [1, 1, n0 * n1 * n2, c]
    elif strides[0] == 0 and strides[1] == 0:
        pass
    shape, strides, _ = _rows_as_channels(packed, shape, strides, group, bits, None)
    with _on_device(q.device):
        check(lib.varq_dequant(q.data_ptr() if packed else None, None if packed else q.data_ptr(),
                               scale.data_ptr(), _ptr(zp), i64arr(shape), i64arr(strides), group, bits, None,
                               out.data_ptr(), _DT[out_dtype], _stream(q)), 'varq_dequant')
    return out


def dequant_window(words: torch.Tensor, scale: torch.Tensor, zp: Optional[torch.Tensor], shape4: Sequence[int],
                   scale_strides4: Sequence[int], group: int, bits: int, in_rowmap: Sequence[int],
                   out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Dequantize a [n0,n1,n2,c] window of a larger packed cache; the window's
    rows are located through in_rowmap, scales through explicit strides."""
    _gpu(words, 'words'); _gpu(scale, 'scale')
    packed = words.dtype == torch.int32
    assert packed or words.dtype == torch.int8
    out = torch.empty(tuple(shape4), dtype=out_dtype, device=words.device)
    shape4, scale_strides4, in_rowmap = _rows_as_channels(packed, shape4, scale_strides4, group, bits, in_rowmap)
    lib = _lib.load()
    with _on_device(words.device):
        check(lib.varq_dequant(words.data_ptr() if packed else None, None if packed else words.data_ptr(),
                               scale.data_ptr(), _ptr(zp), i64arr(shape4),
                               i64arr(scale_strides4), group, bits, None if in_rowmap is None else i64arr(in_rowmap),
                               out.data_ptr(), _DT[out_dtype], _stream(words)), 'varq_dequant')
    return out


def _rows_as_channels(packed: bool, shape4, strides4, group: int, bits: int, rowmap):
    """One scale per (i2, channel) whatever i0 and i1 (the per-(head, channel) table of a
    [B,L,H,c] tensor: VAR_Q/quant.py:84-88 in layout BLHc), the n2 rows of an (i0, i1) pair next
    to each other in the window: the same bytes read as [1, n0, n1, n2*c] with one scale per
    channel of the long rows, which is the form the kernel has its table path for (a lane keeps
    one vector of eight scales for all its pieces instead of loading eight per piece).  The
    long rows must be a power-of-two number of octets, at most 256, and every row whole words."""
    n0, n1, n2, c = [int(v) for v in shape4]
    c8l = n2 * c // 8
    if not packed or group != 1 or n2 <= 1 or c % 8 or (c * bits) % 32 or list(strides4) != [0, 0, c, 1] \
            or c8l > 256 or c8l & (c8l - 1):
        return shape4, strides4, rowmap
    if rowmap is None:
        return [1, n0, n1, n2 * c], [0, 0, 0, 1], None
    rn0, rn1, rn2, os0, os1, os2, off, slot_dim = [int(v) for v in rowmap]
    if (rn0, rn1, rn2) != (n0, n1, n2) or os2 != 1 or slot_dim >= 0 or os0 % n2 or os1 % n2 or off % n2:
        return shape4, strides4, rowmap
    return [1, n0, n1, n2 * c], [0, 0, 0, 1], [1, n0, n1, 0, os0 // n2, os1 // n2, off // n2, -1]


# ---------------------------------------------------------------------------
# producer side: normalise + rotate + quantize straight into the cache
# ---------------------------------------------------------------------------
def qkv_prepare_append(qkv: torch.Tensor, q_out: torch.Tensor, group: int, bits: int, asym: bool, eps: float,
                       k_words: torch.Tensor, k_scale: torch.Tensor, k_zp: Optional[torch.Tensor],
                       v_words: torch.Tensor, v_scale: torch.Tensor, v_zp: Optional[torch.Tensor],
                       rowmap: Sequence[int], slot: Optional[torch.Tensor] = None,
                       q_scale_mul: Optional[torch.Tensor] = None, l2norm: bool = False, norm_eps: float = 1e-12,
                       rope: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, token_start: int = 0) -> None:
    """qkv [B,L,3,H,c] (output of the qkv projection) -> q_out [B,H,L,c] bf16 (normalised,
    scaled per head, rotated) and k, v quantized into the cache buffers through a row map
    over (B, L, H) (see include/varq.h)."""
    _gpu(qkv, 'qkv'); _gpu(q_out, 'q_out')
    assert qkv.dim() == 5 and qkv.shape[2] == 3 and qkv.is_contiguous()
    B, L, _, H, c = qkv.shape
    assert q_out.shape == (B, H, L, c) and q_out.dtype == torch.bfloat16 and q_out.is_contiguous()
    assert list(rowmap[:3]) == [B, L, H]
    for w, s_, z in ((k_words, k_scale, k_zp), (v_words, v_scale, v_zp)):
        _gpu(w, 'words'); _gpu(s_, 'scale')
        assert w.is_contiguous() and s_.is_contiguous() and w.dtype == torch.int32 and s_.dtype == torch.float32
        _check_cache_buffers(c, group, bits, asym, w, s_, z, rowmap, 'qkv_prepare_append')
    cos = sin = None
    if rope is not None:
        cos, sin = rope
        _gpu(cos, 'rope cos'); _gpu(sin, 'rope sin')
        assert cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
        assert cos.shape == sin.shape and cos.shape[1] == c // 2 and cos.shape[0] >= token_start + L
    if q_scale_mul is not None:
        _gpu(q_scale_mul, 'q_scale_mul')
        assert q_scale_mul.dtype == torch.float32 and q_scale_mul.numel() == H and q_scale_mul.is_contiguous()
    lib = _lib.load()
    with _on_device(qkv.device):
        check(lib.varq_qkv_prepare_append(qkv.data_ptr(), _dt(qkv), B, L, H, c, _ptr(q_scale_mul), int(l2norm), norm_eps,
                                          _ptr(cos), _ptr(sin), token_start, q_out.data_ptr(), group, bits, int(asym), eps,
                                          i64arr(rowmap), _ptr(slot), k_words.data_ptr(), k_scale.data_ptr(), _ptr(k_zp),
                                          v_words.data_ptr(), v_scale.data_ptr(), _ptr(v_zp), _stream(qkv)),
              'varq_qkv_prepare_append')


# ---------------------------------------------------------------------------
# fused dequant flash-attention
# ---------------------------------------------------------------------------
_LAYOUTS = {'BHLc': 0, 'BLHc': 1}
# dtypes of q / out (the library's dtype codes): bf16 everywhere, fp16 for head dim 64 (the VAR path)
_ATTN_DT = {torch.bfloat16: 1, torch.float16: 2}


def _attn_dims(q, k_words, layout):
    """(B, Hq, Lq, D, Hkv, Lstride, W) of the attention operands in either layout."""
    assert layout in _LAYOUTS, f'layout must be one of {sorted(_LAYOUTS)}'
    if layout == 'BHLc':
        B, Hq, Lq, D = q.shape
        Bk, Hkv, Lstride, W = k_words.shape
    else:
        B, Lq, Hq, D = q.shape
        Bk, Lstride, Hkv, W = k_words.shape
    assert Bk == B, 'batch sizes of q and the cache differ'
    return B, Hq, Lq, D, Hkv, Lstride, W


def _attn_out(q, out, layout, out_layout, dims):
    """(layout code of the call, output tensor): out looks like q unless out_layout says
    tokens first for a heads-first call."""
    B, Hq, Lq, D = dims
    if out_layout is None or out_layout == layout:
        code, shape = _LAYOUTS[layout], q.shape
    else:
        assert layout == 'BHLc' and out_layout == 'BLHc', 'out_layout: only tokens-first out of a heads-first call'
        code, shape = 2, (B, Lq, Hq, D)
    if out is None:
        out = torch.empty(shape, dtype=q.dtype, device=q.device)
    assert out.dtype == q.dtype and tuple(out.shape) == tuple(shape) and out.is_contiguous(), \
        'out must be contiguous, of the dtype of q and of the shape its layout implies'
    return code, out


def _attn_workspace(lib, B, Hkv, Lq, Lk, D, nseg, splits, device):
    """Device memory for the partial results of a launch that shares keys out (None if the
    library would not); allocated on the current stream, so its reuse after the call is ordered."""
    n = int(lib.varq_fused_attn_workspace_bytes(B, Hkv, Lq, Lk, D, nseg, int(splits)))
    if n == 0:
        return None, 0
    return torch.empty(n, dtype=torch.uint8, device=device), n


def fused_attn(q: torch.Tensor, k_words: torch.Tensor, k_scale: torch.Tensor, k_zp: Optional[torch.Tensor],
               v_words: torch.Tensor, v_scale: torch.Tensor, v_zp: Optional[torch.Tensor],
               k_bits: int, v_bits: int, Lk: int, softmax_scale: float,
               kv_limit: Optional[torch.Tensor] = None, head_map: Optional[torch.Tensor] = None,
               out: Optional[torch.Tensor] = None, splits: int = 0, layout: str = 'BHLc',
               exact_codes: bool = False, out_layout: Optional[str] = None) -> torch.Tensor:
    """q [B,Hq,Lq,D] bf16 (or fp16 at D=64, the VAR path); k/v_words [B,Hkv,Lstride,D*bits/32] int32;
    k/v_scale (zp) [B,Hkv,Lstride,D/group] fp32; attends keys 0..Lk-1.
    Returns out [B,Hq,Lq,D] of q's dtype (rows of heads not in head_map are untouched).
    K and V enter the matrix products dequantized and rounded to q's dtype, as the reference's
    attention sees them.  exact_codes=True asks for the form that never rounds K and V (exact
    code images in the products, scales applied in fp32): closer to the unrounded mathematics,
    farther from the reference, a few percent faster; it exists for 4- and 2-bit codes with one
    group per key at D=128 in bf16 and is ignored elsewhere.
    layout 'BLHc': every tensor has tokens before heads instead ([B,Lq,Hq,D], [B,Lstride,Hkv,...]),
    the layout of the reference's flash-attention call.
    out_layout 'BLHc' with layout 'BHLc': out is [B,Lq,Hq,D] while q and the cache stay heads
    first -- what an attention module hands to its output projection, without a transposing copy.
    splits: over how many workgroups the keys of a query block are shared out (0: the
    library decides from the shape, 1: never, 2..8: exactly)."""
    for t, n in ((q, 'q'), (k_words, 'k_words'), (v_words, 'v_words'), (k_scale, 'k_scale'), (v_scale, 'v_scale')):
        _gpu(t, n)
        assert t.is_contiguous(), f'{n} must be contiguous'
    assert q.dtype in _ATTN_DT and q.dim() == 4, 'q must be bf16 or fp16'
    B, Hq, Lq, D, Hkv, Lstride, Wk = _attn_dims(q, k_words, layout)
    assert v_words.shape[:3] == k_words.shape[:3]
    assert Wk * 32 == D * k_bits and v_words.shape[3] * 32 == D * v_bits
    assert k_scale.shape[:3] == k_words.shape[:3] and v_scale.shape[:3] == k_words.shape[:3]
    k_group, v_group = D // k_scale.shape[3], D // v_scale.shape[3]
    for z, sc, n in ((k_zp, k_scale, 'k_zp'), (v_zp, v_scale, 'v_zp')):
        if z is not None:
            _gpu(z, n)
            assert z.shape == sc.shape and z.dtype == torch.float32 and z.is_contiguous(), f'{n} must look like its scale'
    assert k_scale.dtype == torch.float32 and v_scale.dtype == torch.float32 and k_words.dtype == torch.int32 \
        and v_words.dtype == torch.int32
    assert 0 <= Lk <= Lstride, f'Lk={Lk} outside the cache of {Lstride} tokens'
    code, out = _attn_out(q, out, layout, out_layout, (B, Hq, Lq, D))
    if kv_limit is not None:
        _gpu(kv_limit, 'kv_limit')
        assert kv_limit.dtype == torch.int32 and kv_limit.numel() == Lq and kv_limit.is_contiguous()
    if head_map is not None:
        _gpu(head_map, 'head_map')
        assert head_map.dtype == torch.int32 and head_map.numel() == Hkv
    else:
        assert Hkv == Hq
    lib = _lib.load()
    with _on_device(q.device):
        ws, ws_bytes = _attn_workspace(lib, B, Hkv, Lq, Lk, D, 1, splits, q.device)
        check(lib.varq_fused_attn(q.data_ptr(), out.data_ptr(),
                                  k_words.data_ptr(), k_scale.data_ptr(), _ptr(k_zp), k_bits, k_group,
                                  v_words.data_ptr(), v_scale.data_ptr(), _ptr(v_zp), v_bits, v_group,
                                  B, Hq, Hkv, _ptr(head_map), Lq, Lk, Lstride, D,
                                  _ptr(kv_limit), float(softmax_scale), code, _ATTN_DT[q.dtype],
                                  int(bool(exact_codes)), _ptr(ws), ws_bytes,
                                  int(splits), _stream(q)), 'varq_fused_attn')
    return out


def fused_attn_channel(q: torch.Tensor, k_words: torch.Tensor, k_chan_scale: torch.Tensor,
                       k_chan_zp: Optional[torch.Tensor],
                       v_words: torch.Tensor, v_chan_scale: torch.Tensor, v_chan_zp: Optional[torch.Tensor],
                       bits: int, Lk: int, softmax_scale: float,
                       kv_limit: Optional[torch.Tensor] = None, head_map: Optional[torch.Tensor] = None,
                       out: Optional[torch.Tensor] = None, seg_ends: Optional[Sequence[int]] = None,
                       splits: int = 0, layout: str = 'BHLc', out_layout: Optional[str] = None) -> torch.Tensor:
    """Attention over a cache quantized per (head, channel): the scale layout of the
    reference's G_SCALE_HEAD_DIM / G_HEAD_DIM methods (VAR_Q/quant.py:84-88), scalar scales
    (G_TENSOR, G_SCALE) expanded to the table, and the affine per-head-per-dim variant.
    q [B,Hq,Lq,D] bf16 (or fp16 at D=64); k/v_words [B,Hkv,Lstride,D*bits/32] int32; k_chan_scale,
    v_chan_scale, v_chan_zp fp32 with at least nseg*Hkv*D elements (any shape that flattens to
    [>= nseg, Hkv, D]).  seg_ends (at most 16 increasing key counts, the last one = Lk) says
    where the tables change along the keys: a cache filled step by step by the reference's
    append methods has one table per step (VAR_Q/quant.py:196-201).
    With a single table the zero-point of K may be None even for an affine K: it shifts all
    logits of a query alike.  splits, layout and out_layout as in fused_attn."""
    for t, n in ((q, 'q'), (k_words, 'k_words'), (v_words, 'v_words'), (k_chan_scale, 'k_chan_scale'),
                 (v_chan_scale, 'v_chan_scale')):
        _gpu(t, n)
        assert t.is_contiguous(), f'{n} must be contiguous'
    assert q.dtype in _ATTN_DT and q.dim() == 4, 'q must be bf16 or fp16'
    B, Hq, Lq, D, Hkv, Lstride, W = _attn_dims(q, k_words, layout)
    assert v_words.shape == k_words.shape and W * 32 == D * bits
    nseg = 1 if seg_ends is None else len(seg_ends)
    ends = None
    if seg_ends is not None:
        assert 1 <= nseg <= 16 and int(seg_ends[-1]) == Lk, 'seg_ends: 1..16 entries, the last one equal to Lk'
        ends = (ctypes.c_int32 * nseg)(*[int(e) for e in seg_ends])
    for t, n in ((k_chan_scale, 'k_chan_scale'), (k_chan_zp, 'k_chan_zp'), (v_chan_scale, 'v_chan_scale'),
                 (v_chan_zp, 'v_chan_zp')):
        if t is not None:
            _gpu(t, n)
            assert t.dtype == torch.float32 and t.numel() >= nseg * Hkv * D and t.is_contiguous(), \
                f'{n} must be fp32 [nseg, Hkv, D] (more tables than segments are allowed)'
    assert k_words.dtype == torch.int32 and v_words.dtype == torch.int32
    assert 0 <= Lk <= Lstride, f'Lk={Lk} outside the cache of {Lstride} tokens'
    code, out = _attn_out(q, out, layout, out_layout, (B, Hq, Lq, D))
    if kv_limit is not None:
        _gpu(kv_limit, 'kv_limit')
        assert kv_limit.dtype == torch.int32 and kv_limit.numel() == Lq and kv_limit.is_contiguous()
    if head_map is not None:
        _gpu(head_map, 'head_map')
        assert head_map.dtype == torch.int32 and head_map.numel() == Hkv
    else:
        assert Hkv == Hq
    lib = _lib.load()
    with _on_device(q.device):
        ws, ws_bytes = _attn_workspace(lib, B, Hkv, Lq, Lk, D, nseg, splits, q.device)
        check(lib.varq_fused_attn_channel(q.data_ptr(), out.data_ptr(),
                                          k_words.data_ptr(), k_chan_scale.data_ptr(), _ptr(k_chan_zp),
                                          v_words.data_ptr(), v_chan_scale.data_ptr(), _ptr(v_chan_zp),
                                          nseg, ends, bits, B, Hq, Hkv, _ptr(head_map), Lq, Lk, Lstride, D,
                                          _ptr(kv_limit), float(softmax_scale), code, _ATTN_DT[q.dtype],
                                          _ptr(ws), ws_bytes, int(splits), _stream(q)), 'varq_fused_attn_channel')
    return out

"""The kernel for few queries over a long cache (at most 64 queries per (batch, head), at least
1024 keys, one scale group per key at head dim 128), which `fused_attn` takes when the sharing of
the keys is left to it: against the oracle path unpack -> dequant -> bf16 SDPA (strict bar, as
in test_gpu_attention.py), and against the general kernel on the same inputs (`splits=1` keeps a
launch on it): the two dequantize to the same bf16 operands and differ by summation order only."""
import math

import pytest
import torch

import varq_oracle as O
from gpu_util import note
from test_gpu_attention import _compare, _exact_fp64, _quantize
from var_q_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _case(dev, B, H, Lq, Lk, bits, seed, dist='normal', limit=False, layout='BHLc', Lstride=None, heads=None):
    D, g = 128, 128
    gen = torch.Generator().manual_seed(seed)
    Hkv = H if heads is None else len(heads)
    k = O.synth_kv((B, Hkv, Lk, D), seed + 1, dist).bfloat16()
    v = O.synth_kv((B, Hkv, Lk, D), seed + 2, dist).bfloat16()
    q = torch.randn(B, H, Lq, D, generator=gen).bfloat16()
    kw, ks, kz, kd = _quantize(k, g, bits)
    vw, vs, vz, vd = _quantize(v, g, bits)
    scale = 1.0 / math.sqrt(D)
    lim = bias = None
    if limit:
        lim = torch.randint(0, Lk + 1, (Lq,), generator=gen).int()
        lim[0] = Lk
        bias = torch.zeros(Lq, Lk)
        bias[torch.arange(Lk)[None, :] >= lim[:, None].long()] = float('-inf')
    args = [kw, ks, kz, vw, vs, vz]
    if Lstride:       # spare token rows behind the cached ones, filled with junk
        args = [torch.cat([t, torch.full((B, Hkv, Lstride - Lk, t.shape[3]), 0x7f if t.dtype == torch.int32 else 1e30, dtype=t.dtype)], 2)
                for t in args]
    qd = q
    if layout == 'BLHc':
        args, qd = [t.transpose(1, 2).contiguous() for t in args], q.transpose(1, 2).contiguous()
    args = [t.to(dev) for t in args]
    hm = None if heads is None else torch.tensor(heads, dtype=torch.int32, device=dev)
    kw_ = dict(kv_limit=None if lim is None else lim.to(dev), layout=layout, head_map=hm)
    note('few queries', (B, H, Lq, Lk), bits, dist, 'limit' if limit else '', layout, Lstride, heads)
    out0 = torch.zeros_like(qd).to(dev)
    out = ops.fused_attn(qd.to(dev), *args, bits, bits, Lk, scale, out=out0, **kw_)
    general = ops.fused_attn(qd.to(dev), *args, bits, bits, Lk, scale, splits=1, out=torch.zeros_like(out0), **kw_)
    torch.cuda.synchronize()
    if layout == 'BLHc':
        out, general = out.transpose(1, 2), general.transpose(1, 2)
    hsel = list(range(H)) if heads is None else heads
    qs = q[:, hsel]
    if lim is not None:
        seen = lim > 0
        assert float(out[:, :, ~seen].abs().max() if bool((~seen).any()) else 0.0) == 0.0, 'a query without keys must get zeros'
        out, general, qs, bias = out[:, :, seen], general[:, :, seen], qs[:, :, seen], bias[seen]
    out, general = out[:, hsel], general[:, hsel]
    ref = O.attention_ref(qs, kd, vd, scale, bias)
    _compare(out, ref, _exact_fp64(qs, kd, vd, scale, bias, dev), f'few queries {Lq}x{Lk} int{bits}')
    span = max(1.0, float(ref.abs().max()))
    assert float((out.float() - general.float()).abs().max().cpu()) <= span * 2 ** -6, 'the two kernels differ by more than two bf16 steps'
    if heads is not None:
        rest = [h for h in range(H) if h not in heads]
        assert float(out0[:, rest].abs().max()) == 0.0, 'heads outside the map were written'


@pytest.mark.parametrize('bits', [4, 2, 8])
@pytest.mark.parametrize('Lq,Lk', [(16, 10521), (64, 4121), (1, 1024), (33, 2521), (32, 1055)])
def test_against_oracle_and_general_kernel(dev, bits, Lq, Lk):
    assert _lib.load().varq_fused_attn_key_shares(2, 3, Lq, Lk, 128, 128, 128) >= 1
    _case(dev, 2, 3, Lq, Lk, bits, seed=bits * 1000 + Lq)


@pytest.mark.parametrize('bits', [4, 8])
def test_heavy_tails_key_limits_layouts_and_windows(dev, bits):
    _case(dev, 1, 2, 16, 6425, bits, seed=11 + bits, dist='student4')
    _case(dev, 2, 2, 40, 2000, bits, seed=12 + bits, limit=True)
    _case(dev, 2, 3, 20, 1500, bits, seed=13 + bits, layout='BLHc')
    _case(dev, 1, 2, 9, 1300, bits, seed=14 + bits, Lstride=1400, limit=True)
    _case(dev, 2, 5, 12, 1100, bits, seed=15 + bits, heads=[4, 1, 2])


def test_many_pairs_one_share_each(dev):
    """Enough (batch, head) pairs to fill the device without sharing keys out: one workgroup per
    pair, no workspace, output written directly."""
    assert _lib.load().varq_fused_attn_key_shares(8, 128, 16, 1024, 128, 128, 128) == 1
    _case(dev, 8, 128, 16, 1024, 4, seed=99)


def test_config4_shape_properties(dev):
    """The benchmark's shape (B=2, H=16, 10 521 keys, INT4 group 128, 16 queries) through what
    holds at any size: a constant V gives that constant, key order does not matter, rows behind
    the cached ones are not read."""
    B, H, Lq, Lk, D, bits, g = 2, 16, 16, 10521, 128, 4, 128
    gen = torch.Generator(device=dev).manual_seed(44)
    k = torch.randn(B, H, Lk, D, device=dev, generator=gen).bfloat16()
    v = torch.randn(B, H, Lk, D, device=dev, generator=gen).bfloat16()
    q = torch.randn(B, H, Lq, D, device=dev, generator=gen).bfloat16()
    kq, vq = ops.quant_pack_rows(k, g, bits, True), ops.quant_pack_rows(v, g, bits, True)
    scale = 1 / math.sqrt(D)
    assert _lib.load().varq_fused_attn_key_shares(B, H, Lq, Lk, D, g, g) > 8
    note('few queries, config-4 shape: constant V')
    vw = torch.full_like(vq[0], int.from_bytes(bytes([5 * 17] * 4), 'little', signed=True))
    vs = torch.rand(B, H, Lk, 1, device=dev, generator=gen) + 0.5
    out = ops.fused_attn(q, *kq, vw, vs, 5 - 1.25 / vs, bits, bits, Lk, scale)
    assert float((out.float() - 1.25).abs().max()) <= 2 ** -7
    note('few queries, config-4 shape: permuted keys, rows behind the end')
    base = ops.fused_attn(q, *kq, *vq, bits, bits, Lk, scale)
    perm = torch.randperm(Lk, device=dev, generator=gen)
    other = ops.fused_attn(q, *[t[:, :, perm].contiguous() for t in kq], *[t[:, :, perm].contiguous() for t in vq], bits, bits, Lk, scale)
    span = max(1.0, float(base.float().abs().max()))
    assert float((other.float() - base.float()).abs().max()) <= max(2e-2 * span / 4, span * 2 ** -7)
    longer = [torch.cat([t, torch.full_like(t[:, :, :300], 0x7f if t.dtype == torch.int32 else 1e30)], dim=2).contiguous()
              for t in (*kq, *vq)]
    assert torch.equal(ops.fused_attn(q, *longer, bits, bits, Lk, scale), base)
    torch.cuda.synchronize()


@pytest.mark.parametrize('seed', range(12))
def test_seeded_random_shapes(dev, seed):
    """Seeded random cases inside the kernel's range (1..64 queries, 1024..5000 keys, any batch and
    head count, either layout, with and without key limits, spare rows, head subsets)."""
    g = torch.Generator().manual_seed(9000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    B, H, Lq, Lk, bits = r(1, 3), r(1, 5), r(1, 64), r(1024, 5000), (4, 2, 8)[seed % 3]
    heads = None
    if H >= 3 and seed % 4 == 1:
        heads = sorted(set(r(0, H - 1) for _ in range(2)))
    _case(dev, B, H, Lq, Lk, bits, seed=700 + seed, dist=('normal', 'student4')[seed % 2], limit=seed % 3 == 0,
          layout=('BHLc', 'BLHc')[(seed // 2) % 2] if heads is None else 'BHLc', Lstride=Lk + r(1, 200) if seed % 5 == 2 else None, heads=heads)


@pytest.mark.parametrize('bits', [4, 8])
def test_zero_points_outside_the_byte_form(dev, bits):
    """4-bit codes are dequantized through bytes while the zero-points are integers of small
    size and through the general form from the first block on where a K zero-point is not (and
    per block for V): fractional and large zero-points set in here and there along the keys,
    against the oracle's dequantization with the same parameters."""
    B, H, Lq, Lk, D, g = 1, 2, 24, 3000, 128, 128
    gen = torch.Generator().manual_seed(321 + bits)
    k, v = O.synth_kv((B, H, Lk, D), 5, 'normal').bfloat16(), O.synth_kv((B, H, Lk, D), 6, 'normal').bfloat16()
    q = torch.randn(B, H, Lq, D, generator=gen).bfloat16()
    kq, ks, kz = O.quant_groupwise(k, g, bits, True)
    vq, vs, vz = O.quant_groupwise(v, g, bits, True)
    kz, vz = kz.clone(), vz.clone()
    kz[:, 0, 1700:] += 0.5          # head 0: every wavefront reaches a fractional K zero-point on its way
    kz[:, 1, 2999] = 300.0          # head 1: only the last key's, far outside a byte
    vz[:, 0, 40:45] -= 0.25         # V: a few keys of one block ...
    vz[:, 1, 1000:2000] = -200.0    # ... and a long run of blocks
    kd, vd = O.dequant_groupwise(kq, ks, kz, g), O.dequant_groupwise(vq, vs, vz, g)
    scale = 1.0 / math.sqrt(D)
    note('few queries, zero-points outside the byte form', bits)
    put = lambda t: t.to(dev)
    args = [put(O.pack_last_dim(kq, bits)[0]), put(ks), put(kz), put(O.pack_last_dim(vq, bits)[0]), put(vs), put(vz)]
    assert _lib.load().varq_fused_attn_key_shares(B, H, Lq, Lk, D, g, g) > 1
    out = ops.fused_attn(put(q), *args, bits, bits, Lk, scale)
    general = ops.fused_attn(put(q), *args, bits, bits, Lk, scale, splits=1)
    torch.cuda.synchronize()
    _compare(out, O.attention_ref(q, kd, vd, scale, None), _exact_fp64(q, kd, vd, scale, None, dev), f'few queries, odd zero-points, int{bits}')
    span = max(1.0, float(general.float().abs().max()))
    assert float((out.float() - general.float()).abs().max()) <= span * 2 ** -6


def _range_profile(name, Lk):
    t = torch.arange(Lk, dtype=torch.float32) / (Lk - 1)
    if name == 'up':
        return 4 * t - 2
    if name == 'down':
        return 2 - 4 * t
    if name == 'step':                       # one jump in the middle of a 32-key block
        return torch.where(torch.arange(Lk) < 1113, -2.0, 2.0)
    if name == 'saw':                        # up in five teeth, each higher than the last
        return (5 * t).frac() * 1.5 - 2 + 2.5 * t
    if name == 'late':                       # flat, then the last key alone far above the rest
        c = torch.full((Lk,), -1.0)
        c[-1] = 2.0
        return c
    raise ValueError(name)


@pytest.mark.parametrize('prof', ['up', 'down', 'step', 'saw', 'late'])
@pytest.mark.parametrize('bits,limit', [(4, False), (8, True)])
def test_softmax_range(dev, prof, bits, limit):
    """Logits that rise, fall, jump or zig-zag by up to ~200 octaves along the keys, with queries of
    both signs and several gains side by side: the softmax reference of the kernel moves in some
    lanes and not in others, once or many times (the yardstick is that of
    test_gpu_attention_softmax_range.py)."""
    from test_gpu_attention_softmax_range import _check
    B, H, Lq, Lk, D, g = 1, 2, 50, 1500, 128, 128
    gen = torch.Generator().manual_seed(77 + bits)
    w = torch.where(torch.rand(D, generator=gen) < 0.5, -1.0, 1.0)
    c = _range_profile(prof, Lk)
    k = (c[:, None] * w[None, :] + 0.2 * torch.randn(H, Lk, D, generator=gen)).unsqueeze(0).bfloat16()
    v = torch.randn(B, H, Lk, D, generator=gen).bfloat16()
    gain = torch.tensor([1.0, -1.0, 0.3, -0.3, 0.05, 0.0, 0.7])[torch.arange(Lq) % 7]
    q = (3.0 * gain[:, None] * w[None, :] + 0.1 * torch.randn(H, Lq, D, generator=gen)).unsqueeze(0).bfloat16()
    lim = bias = None
    if limit:
        lim = torch.randint(1, Lk + 1, (Lq,), generator=gen).int()
        bias = torch.zeros(Lq, Lk)
        bias[torch.arange(Lk)[None, :] >= lim[:, None].long()] = float('-inf')
    kw, ks, kz, kd = _quantize(k, g, bits)
    vw, vs, vz, vd = _quantize(v, g, bits)
    scale = 1.0 / math.sqrt(D)
    note('few queries, softmax range', prof, bits, limit)
    put = lambda t: None if t is None else t.to(dev)
    assert _lib.load().varq_fused_attn_key_shares(B, H, Lq, Lk, D, g, g) > 1
    out = ops.fused_attn(put(q), put(kw), put(ks), put(kz), put(vw), put(vs), put(vz), bits, bits, Lk, scale, kv_limit=put(lim))
    torch.cuda.synchronize()
    _check(out, O.attention_ref(q, kd, vd, scale, bias), O.attention_exact(q.float(), kd, vd, scale, bias),
           f'few queries, softmax range {prof} int{bits}' + (' limit' if limit else ''))


def test_workspace_missing_or_short(dev):
    """The key shares are cut down to what the caller's workspace holds: no workspace at all (one
    workgroup per (batch, head) walks the whole cache) and one that is too small for the shares
    the library would like, through the C ABI, against the call with the full workspace."""
    from var_q_amd._lib import check
    B, H, Lq, Lk, D, bits, g = 1, 3, 20, 4100, 128, 4, 128
    gen = torch.Generator(device=dev).manual_seed(606)
    k = torch.randn(B, H, Lk, D, device=dev, generator=gen).bfloat16()
    v = torch.randn(B, H, Lk, D, device=dev, generator=gen).bfloat16()
    q = torch.randn(B, H, Lq, D, device=dev, generator=gen).bfloat16()
    (kw, ks, kz), (vw, vs, vz) = ops.quant_pack_rows(k, g, bits, True), ops.quant_pack_rows(v, g, bits, True)
    scale = 1 / math.sqrt(D)
    lib = _lib.load()
    full = int(lib.varq_fused_attn_workspace_bytes(B, H, Lq, Lk, D, 1, 0))
    shares = int(lib.varq_fused_attn_key_shares(B, H, Lq, Lk, D, g, g))
    assert shares > 4 and full > 0
    want = ops.fused_attn(q, kw, ks, kz, vw, vs, vz, bits, bits, Lk, scale)
    span = max(1.0, float(want.float().abs().max()))
    for nbytes in (0, full // 3):
        note('few queries, workspace of', nbytes, 'bytes where', full, 'are asked for')
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
        out = torch.zeros_like(q)
        check(lib.varq_fused_attn(q.data_ptr(), out.data_ptr(), kw.data_ptr(), ks.data_ptr(), kz.data_ptr(), bits, g,
                                  vw.data_ptr(), vs.data_ptr(), vz.data_ptr(), bits, g, B, H, H, None, Lq, Lk, Lk, D, None,
                                  float(scale), 0, 1, 0, ws.data_ptr() if nbytes else None, nbytes, 0,
                                  torch.cuda.current_stream().cuda_stream), 'varq_fused_attn')
        torch.cuda.synchronize()
        assert float((out.float() - want.float()).abs().max()) <= span * 2 ** -6

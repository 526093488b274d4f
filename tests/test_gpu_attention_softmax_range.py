"""The online softmax over a wide range of logits.  The kernels keep a softmax reference per
query that moves only when a logit gets far above it (the exact-code kernels test the packed
weights for one that reached 2, the dequantizing kernels test the block's weight sum against
2^16) and then redo the block; ordinary test data never moves it after the first block.  Here the
logits of a query rise, fall, jump or zig-zag by up to ~200 octaves along the keys, with queries
of different sign and gain side by side in one wavefront, so that the reference moves in some
lanes and not in others, once or many times, in the middle of a tile, under a key limit and with
the keys shared between workgroups.

The yardstick.  At +-100 octaves the softmax is so sharp that rounding the dequantized K to bf16
(what the reference's attention and the oracle do) moves a logit by up to 100 * 2^-9 = 0.2 octaves
and the oracle's output by 0.1-0.2 from the fp64 value of the unrounded operands.  The
dequantizing kernels (the default form) round the same way and are held to the oracle as in
test_gpu_attention.py; the exact-code kernels (`exact_codes=True`) do not round and land within
1e-2 of the fp64 value instead.  This file tests the softmax bookkeeping, not parity: a result
passes when it is within the tolerance of either, cosine >= 0.9995 and max-abs <= 2e-2 x range
against the fp64 value, or test_gpu_attention.py's comparison with the oracle."""
import math

import pytest
import torch

import varq_oracle as O
from gpu_util import note
from test_gpu_attention import _compare
from var_q_amd import ops

pytestmark = pytest.mark.gpu

LQ, LK = 70, 300


def _check(out, ref, exact, what, exact_codes=False):
    o, e = out.double().cpu(), exact.double()
    span = max(1.0, float(e.abs().max()))
    err = float((o - e).abs().max())
    cos = float(torch.nn.functional.cosine_similarity(o.flatten(), e.flatten(), dim=0))
    assert not bool(torch.isnan(o).any()), what
    if err <= 2e-2 * span and cos >= 0.9995:
        print(f'[attn] {what}: range {span:.3g}  kernel-fp64 {err:.4g}  cosine {cos:.6f}', flush=True)
        return
    _compare(out, ref, exact, what, exact_codes=exact_codes)


def _profile(name):
    t = torch.arange(LK, dtype=torch.float32) / (LK - 1)
    if name == 'up':
        return 4 * t - 2
    if name == 'down':
        return 2 - 4 * t
    if name == 'step':                       # one jump in the middle of a 32-key block
        return torch.where(torch.arange(LK) < 113, -2.0, 2.0)
    if name == 'saw':                        # up in five teeth, each higher than the last
        return (5 * t).frac() * 1.5 - 2 + 2.5 * t
    if name == 'late':                       # flat, then the last key alone far above the rest
        c = torch.full((LK,), -1.0)
        c[-1] = 2.0
        return c
    raise ValueError(name)


def _data(D, prof, seed):
    g = torch.Generator().manual_seed(seed)
    w = torch.where(torch.rand(D, generator=g) < 0.5, -1.0, 1.0)
    c = _profile(prof)
    k = (c[:, None] * w[None, :] + 0.2 * torch.randn(2, LK, D, generator=g)).unsqueeze(0).bfloat16()
    v = torch.randn(1, 2, LK, D, generator=g).bfloat16()
    # gains of both signs and three sizes, interleaved so that every wavefront holds all of them:
    # logit = gain * 3 * sqrt(D) * c  (natural units), up to +-98 octaves at D=128
    gain = torch.tensor([1.0, -1.0, 0.3, -0.3, 0.05, 0.0, 0.7])[torch.arange(LQ) % 7]
    q = (3.0 * gain[:, None] * w[None, :] + 0.1 * torch.randn(2, LQ, D, generator=g)).unsqueeze(0).bfloat16()
    return q, k, v


def _limit(kind, seed):
    if kind == 'all':
        return None, None
    g = torch.Generator().manual_seed(seed)
    lim = torch.randint(1, LK + 1, (LQ,), generator=g).int()
    bias = torch.zeros(LQ, LK)
    bias[torch.arange(LK)[None, :] >= lim[:, None].long()] = float('-inf')
    return lim, bias


@pytest.mark.parametrize('prof', ['up', 'down', 'step', 'saw', 'late'])
@pytest.mark.parametrize('D,bits,gk,gv,exact_codes',
                         [(128, 4, 128, 128, True), (128, 2, 128, 128, True), (128, 4, 128, 128, False), (128, 2, 128, 128, False),
                          (128, 8, 128, 128, False), (128, 4, 64, 64, False), (128, 2, 32, 32, False), (64, 4, 64, 64, False),
                          (64, 8, 32, 32, False)])
@pytest.mark.parametrize('splits,limit', [(0, 'all'), (3, 'limit')])
def test_token_scales(dev, prof, D, bits, gk, gv, exact_codes, splits, limit):
    q, k, v = _data(D, prof, 17 * D + bits)
    lim, bias = _limit(limit, 5 + bits)
    kq, ks, kz = O.quant_groupwise(k, gk, bits, True)
    vq, vs, vz = O.quant_groupwise(v, gv, bits, True)
    kd, vd = O.dequant_groupwise(kq, ks, kz, gk), O.dequant_groupwise(vq, vs, vz, gv)
    scale = 1.0 / math.sqrt(D)
    note('softmax range, token scales', prof, D, bits, gk, gv, splits, limit)
    put = lambda t: None if t is None else t.to(dev)
    out = ops.fused_attn(put(q), put(O.pack_last_dim(kq, bits)[0]), put(ks), put(kz), put(O.pack_last_dim(vq, bits)[0]), put(vs),
                         put(vz), bits, bits, LK, scale, kv_limit=put(lim), splits=splits, exact_codes=exact_codes)
    torch.cuda.synchronize()
    _check(out, O.attention_ref(q, kd, vd, scale, bias), O.attention_exact(q.float(), kd, vd, scale, bias),
           f'softmax range {prof} D={D} int{bits} g{gk}/{gv} splits={splits} {limit}' + (' exact codes' if exact_codes else ''),
           exact_codes)


@pytest.mark.parametrize('prof', ['up', 'down', 'step', 'saw', 'late'])
@pytest.mark.parametrize('D,bits,cuts', [(64, 8, [LK]), (128, 4, [LK]), (64, 4, [40, 113, LK]), (128, 8, [150, LK])])
@pytest.mark.parametrize('splits,limit', [(0, 'all'), (2, 'limit')])
def test_channel_tables(dev, prof, D, bits, cuts, splits, limit):
    q, k, v = _data(D, prof, 31 * D + bits)
    lim, bias = _limit(limit, 9 + bits)
    per = []
    for x in (k, v):
        ws, ds, ss, zs, a = [], [], [], [], 0
        for e in cuts:
            cq, s, z = O.quant_reduce(x[:, :, a:e], (0, 2), bits, True)
            ws.append(O.pack_last_dim(cq, bits)[0])
            ds.append(O.dequant_asym(cq, s, z))
            ss.append(s.reshape(2, D))
            zs.append(z.reshape(2, D))
            a = e
        per.append((torch.cat(ws, 2).contiguous(), torch.stack(ss).contiguous(), torch.stack(zs).contiguous(), torch.cat(ds, 2)))
    (kw, ks, kz, kd), (vw, vs, vz, vd) = per
    scale = 1.0 / math.sqrt(D)
    note('softmax range, channel tables', prof, D, bits, cuts, splits, limit)
    put = lambda t: None if t is None else t.to(dev)
    out = ops.fused_attn_channel(put(q), put(kw), put(ks), put(kz), put(vw), put(vs), put(vz), bits, LK, scale, kv_limit=put(lim),
                                 seg_ends=cuts, splits=splits)
    torch.cuda.synchronize()
    _check(out, O.attention_ref(q, kd, vd, scale, bias), O.attention_exact(q.float(), kd, vd, scale, bias),
           f'softmax range, tables, {prof} D={D} int{bits} cuts={cuts} splits={splits} {limit}')

"""Attention with the keys of a query block shared out over several workgroups (partial
results in fp32, combined by a second kernel), forced to every share count the library
takes, against the same oracle and tolerances as the one-workgroup path."""
import math

import pytest
import torch

import varq_oracle as O
from gpu_util import note
from test_gpu_attention import _run as run_token
from test_gpu_attention_channel import VAR_STEPS, _run as run_channel, _stepwise
from var_q_amd import ops, schedules

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('splits', [1, 2, 3, 5, 8])
@pytest.mark.parametrize('D,gk,gv,bits', [(128, 128, 128, 4), (128, 64, 64, 8), (64, 64, 64, 2), (64, 32, 64, 4)])
def test_token_scales(dev, splits, D, gk, gv, bits):
    run_token(dev, 2, 3, 200, 1100, D, bits, gk, gv, seed=900 + splits + D, what='split token', splits=splits)


@pytest.mark.parametrize('Lq,Lk,splits', [(1, 1, 2), (4, 5, 8), (33, 64, 3), (129, 127, 2), (7, 300, 8), (300, 129, 4)])
def test_more_shares_than_tiles(dev, Lq, Lk, splits):
    """Shares without a tile leave an empty partial result; the combination skips them."""
    run_token(dev, 1, 2, Lq, Lk, 128, 4, 128, 128, seed=Lq * 1000 + Lk, what='split ragged', splits=splits)
    run_channel(dev, 1, 2, Lq, Lk, 128, 8, True, seed=Lq * 1000 + Lk + 1, what='split channel ragged', splits=splits)


@pytest.mark.parametrize('splits', [2, 4])
def test_block_causal_mask(dev, splits):
    """Queries of several scales in one block: the workgroups' tile counts differ, and so do
    their shares."""
    pn = O.VAR_PATCH_NUMS
    L = 680
    run_token(dev, 1, 2, L, L, 64, 4, 64, 64, seed=77, kv_limit=schedules.kv_limit(pn), bias=O.block_causal_bias(pn),
              what='split block-causal', splits=splits)
    run_channel(dev, 1, 2, L, L, 64, 8, False, seed=78, kv_limit=schedules.kv_limit(pn), bias=O.block_causal_bias(pn),
                what='split channel block-causal', splits=splits)


@pytest.mark.parametrize('splits', [2, 3, 8])
@pytest.mark.parametrize('bits,asym', [(8, False), (4, True)])
def test_stepwise_tables(dev, splits, bits, asym):
    """A share may begin in the middle of the cache: it starts with the tables of its first
    segment and crosses the later boundaries like the one-workgroup path."""
    _stepwise(dev, 2, 3, 64, VAR_STEPS, bits, asym, 256, seed=141 + splits, what='split stepwise', splits=splits)
    _stepwise(dev, 1, 2, 128, [1, 4, 16, 36, 64, 144, 256, 400], bits, asym, 400, seed=150 + splits,
              what='split stepwise D128', splits=splits)


def test_stepwise_masked(dev):
    _stepwise(dev, 1, 2, 64, VAR_STEPS, 4, True, 680, seed=44, masked=True, what='split stepwise masked', splits=3)


def test_head_subset_and_spare_rows(dev):
    """Three of five heads through a head map, cache buffers longer than the keys: the partial
    results are indexed by packed head, the combination writes the mapped heads only."""
    B, Hq, D, Lk, Lstride, bits = 2, 5, 128, 500, 640, 4
    heads = [4, 1, 2]
    gen = torch.Generator().manual_seed(12)
    k = torch.randn(B, len(heads), Lk, D, generator=gen).bfloat16()
    v = torch.randn(B, len(heads), Lk, D, generator=gen).bfloat16()
    q = torch.randn(B, Hq, 40, D, generator=gen).bfloat16()
    bufs = []
    for x in (k, v):
        w, s, z = ops.quant_pack_rows(x.to(dev), 128, bits, True)
        full = [torch.zeros(B, len(heads), Lstride, t.shape[3], dtype=t.dtype, device=dev) for t in (w, s, z)]
        for dst, src in zip(full, (w, s, z)):
            dst[:, :, :Lk] = src
        bufs.append(full)
    hm = torch.tensor(heads, dtype=torch.int32, device=dev)
    outs = []
    for splits in (1, 4):
        out = torch.full((B, Hq, 40, D), 7.0, dtype=torch.bfloat16, device=dev)
        note('fused_attn head subset', 'splits', splits)
        ops.fused_attn(q.to(dev), *bufs[0], *bufs[1], bits, bits, Lk, 0.1, head_map=hm, out=out, splits=splits)
        outs.append(out)
    torch.cuda.synchronize()
    a, b = outs[0].double(), outs[1].double()
    assert float((a - b).abs().max()) <= 2e-2 * max(1.0, float(a.abs().max())) / 4
    untouched = [h for h in range(Hq) if h not in heads]
    assert bool((outs[1][:, untouched] == 7.0).all()), 'rows of heads outside the map were written'


def test_library_choice_matches_one_workgroup(dev):
    """Left to the library, a step of 400 queries at batch 2 is shared out (the workspace
    query says so) and agrees with the unshared result to rounding."""
    B, H, Lq, Lk, D, bits = 2, 16, 400, 921, 128, 4
    gen = torch.Generator(device=dev).manual_seed(5)
    k = torch.randn(B, H, Lk, D, device=dev, generator=gen).bfloat16()
    v = torch.randn(B, H, Lk, D, device=dev, generator=gen).bfloat16()
    q = torch.randn(B, H, Lq, D, device=dev, generator=gen).bfloat16()
    kq, vq = ops.quant_pack_rows(k, 128, bits, True), ops.quant_pack_rows(v, 128, bits, True)
    from var_q_amd import _lib
    assert _lib.load().varq_fused_attn_workspace_bytes(B, H, Lq, Lk, D, 1, 0) > 0
    note('fused_attn library-chosen shares')
    auto = ops.fused_attn(q, *kq, *vq, bits, bits, Lk, 1 / math.sqrt(D))
    one = ops.fused_attn(q, *kq, *vq, bits, bits, Lk, 1 / math.sqrt(D), splits=1)
    torch.cuda.synchronize()
    assert float((auto.double() - one.double()).abs().max()) <= 2e-2 * max(1.0, float(one.abs().max())) / 4


@pytest.mark.parametrize('Lq', [1, 20, 64, 65, 128])
@pytest.mark.parametrize('D,gk,gv,bits', [(64, 64, 64, 4), (64, 32, 32, 8), (64, 32, 64, 2)])
def test_many_heads_few_queries_token_scales(dev, Lq, D, gk, gv, bits):
    """More (batch, head) pairs than compute units with at most 128 queries each -- the first
    steps of a schedule at a large batch -- run as workgroups of two or four wavefronts, two
    to a compute unit.  Against the oracle, and bit for bit against the same data attended in two halves
    (each half has too few pairs for that path)."""
    B, H, Lk = 33, 8, 150
    run_token(dev, B, H, Lq, Lk, D, bits, gk, gv, seed=700 + Lq + bits, what='small workgroups', splits=1)
    gen = torch.Generator(device=dev).manual_seed(Lq + bits)
    k = torch.randn(B, H, Lk, D, device=dev, generator=gen).bfloat16()
    v = torch.randn(B, H, Lk, D, device=dev, generator=gen).bfloat16()
    q = torch.randn(B, H, Lq, D, device=dev, generator=gen).bfloat16()
    kq = [ops.quant_pack_rows(k, gk, bits, True)[i] for i in range(3)]
    vq = [ops.quant_pack_rows(v, gv, bits, True)[i] for i in range(3)]
    note('small workgroups vs halves', (Lq, D, gk, gv, bits))
    whole = ops.fused_attn(q, *kq, *vq, bits, bits, Lk, 0.125, splits=1)
    halves = [ops.fused_attn(q[a:b].contiguous(), *[t[a:b].contiguous() for t in kq], *[t[a:b].contiguous() for t in vq],
                             bits, bits, Lk, 0.125, splits=1) for a, b in ((0, 16), (16, 33))]
    torch.cuda.synchronize()
    assert torch.equal(whole, torch.cat(halves, 0))


@pytest.mark.parametrize('fmt_blhc', [False, True])
def test_many_heads_few_queries_stepwise_tables(dev, fmt_blhc):
    """The same for a cache filled step by step with per-(head, channel) tables (the VAR
    rule at a large batch), in both layouts."""
    B, H, D, bits = 40, 8, 64, 8
    steps = [1, 4, 9, 16, 25, 36]
    _stepwise(dev, B, H, D, steps, bits, False, 36, seed=801, what='small workgroups stepwise')
    _stepwise(dev, B, H, D, steps, 4, True, 20, seed=802, what='small workgroups stepwise asym', splits=1)
    _stepwise(dev, B, H, D, steps + [49], 8, False, 100, seed=803, what='small workgroups stepwise, four wavefronts',
              splits=1)
    L, nseg = sum(steps), len(steps)
    ends = [sum(steps[:i + 1]) for i in range(nseg)]
    gen = torch.Generator(device=dev).manual_seed(9)
    kw = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, L, D * bits // 32), device=dev, generator=gen, dtype=torch.int64).int()
    vw = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, L, D * bits // 32), device=dev, generator=gen, dtype=torch.int64).int()
    ks = (torch.rand(nseg, H, D, device=dev, generator=gen) * 0.02 + 0.01).contiguous()
    vs = (torch.rand(nseg, H, D, device=dev, generator=gen) * 0.02 + 0.01).contiguous()
    q = torch.randn(B, H, 36, D, device=dev, generator=gen).bfloat16()
    tr = (lambda t: t.transpose(1, 2).contiguous()) if fmt_blhc else (lambda t: t)
    lay = 'BLHc' if fmt_blhc else 'BHLc'
    note('small workgroups stepwise vs halves', lay)
    whole = ops.fused_attn_channel(tr(q), tr(kw), ks, None, tr(vw), vs, None, bits, L, 0.1, seg_ends=ends, splits=1, layout=lay)
    halves = [ops.fused_attn_channel(tr(q[a:b]), tr(kw[a:b]), ks, None, tr(vw[a:b]), vs, None, bits, L, 0.1, seg_ends=ends,
                                     splits=1, layout=lay) for a, b in ((0, 20), (20, 40))]
    torch.cuda.synchronize()
    assert torch.equal(whole, torch.cat(halves, 0))

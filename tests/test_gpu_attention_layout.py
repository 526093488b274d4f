"""The attention kernels on operands laid out tokens-before-heads ([B,L,H,...], the layout of
the reference's flash-attention call: VAR/models/basic_var.py:127-131) give bit for bit what
they give on the same values laid out heads-before-tokens, which the other attention tests
check against the oracle."""
import math

import pytest
import torch

import varq_oracle as O
from gpu_util import note
from var_q_amd import ops, schedules

pytestmark = pytest.mark.gpu


def _blhc(t):
    return None if t is None else t.transpose(1, 2).contiguous()


@pytest.mark.parametrize('D,group,bits,asym', [(128, 128, 4, True), (128, 64, 8, True), (64, 32, 2, True), (64, 64, 8, False)])
@pytest.mark.parametrize('splits', [1, 3])
def test_token_scales(dev, D, group, bits, asym, splits):
    B, Hq, Lq, Lk, Lstride = 2, 5, 150, 700, 768
    heads = [3, 0, 4]
    gen = torch.Generator(device=dev).manual_seed(D + bits)
    k = torch.randn(B, len(heads), Lstride, D, device=dev, generator=gen).bfloat16()
    v = torch.randn(B, len(heads), Lstride, D, device=dev, generator=gen).bfloat16()
    q = torch.randn(B, Hq, Lq, D, device=dev, generator=gen).bfloat16()
    kq, vq = ops.quant_pack_rows(k, group, bits, asym), ops.quant_pack_rows(v, group, bits, asym)
    hm = torch.tensor(heads, dtype=torch.int32, device=dev)
    lim = torch.randint(1, Lk + 1, (Lq,), generator=torch.Generator().manual_seed(3)).int().to(dev)
    for limit in (None, lim):
        note('fused_attn layouts', (D, group, bits, asym), 'splits', splits, 'limit', limit is not None)
        a = torch.full((B, Hq, Lq, D), 7.0, dtype=torch.bfloat16, device=dev)
        ops.fused_attn(q, *kq, *vq, bits, bits, Lk, 1 / math.sqrt(D), kv_limit=limit, head_map=hm, out=a, splits=splits)
        b = torch.full((B, Lq, Hq, D), 7.0, dtype=torch.bfloat16, device=dev)
        ops.fused_attn(_blhc(q), *[_blhc(t) for t in kq], *[_blhc(t) for t in vq], bits, bits, Lk, 1 / math.sqrt(D),
                       kv_limit=limit, head_map=hm, out=b, splits=splits, layout='BLHc')
        torch.cuda.synchronize()
        assert torch.equal(b.transpose(1, 2), a)
        assert bool((a[:, [1, 2]] == 7.0).all()) and not bool((a[:, heads] == 7.0).all())


@pytest.mark.parametrize('D', [64, 128])
@pytest.mark.parametrize('splits', [1, 2])
def test_stepwise_tables(dev, D, splits):
    B, H, bits = 2, 3, 8
    steps = [n * n for n in O.VAR_PATCH_NUMS]
    L, nseg = sum(steps), len(steps)
    ends = [sum(steps[:i + 1]) for i in range(nseg)]
    gen = torch.Generator(device=dev).manual_seed(D)
    kw = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, L, D * bits // 32), device=dev, generator=gen, dtype=torch.int64).int()
    vw = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, L, D * bits // 32), device=dev, generator=gen, dtype=torch.int64).int()
    tab = lambda lo: (torch.rand(nseg, H, D, device=dev, generator=gen) * 0.02 + lo).contiguous()
    ks, vs, kz, vz = tab(0.01), tab(0.01), tab(-3.0) * 100, tab(-3.0) * 100
    q = torch.randn(B, H, 256, D, device=dev, generator=gen).bfloat16()
    lim = schedules.kv_limit(O.VAR_PATCH_NUMS)[L - 256:].contiguous().to(dev)
    note('fused_attn_channel layouts', D, 'splits', splits)
    a = ops.fused_attn_channel(q, kw, ks, kz, vw, vs, vz, bits, L, 0.1, kv_limit=lim, seg_ends=ends, splits=splits)
    b = ops.fused_attn_channel(_blhc(q), _blhc(kw), ks, kz, _blhc(vw), vs, vz, bits, L, 0.1, kv_limit=lim, seg_ends=ends,
                               splits=splits, layout='BLHc')
    torch.cuda.synchronize()
    assert not bool(torch.isnan(a.float()).any())
    assert torch.equal(b.transpose(1, 2), a)


@pytest.mark.parametrize('D,group,bits,Lq,Lk,splits', [(128, 128, 4, 150, 700, 1), (128, 128, 4, 150, 700, 3), (128, 64, 8, 16, 2100, 0),
                                                       (128, 128, 4, 64, 2100, 0), (64, 32, 2, 300, 500, 1), (64, 64, 8, 256, 680, 2)])
def test_tokens_first_output_of_a_heads_first_call(dev, D, group, bits, Lq, Lk, splits):
    """out_layout='BLHc' with q and the cache heads first: the same bits as the heads-first
    output, transposed; rows of heads outside the head map stay untouched.  Covers the general
    kernel with and without shared keys, the few-queries kernel (16 and 64 queries over 2100
    keys) and the kernel that combines the shares."""
    B, Hq = 2, 5
    heads = [3, 0, 4]
    gen = torch.Generator(device=dev).manual_seed(D + bits + Lq)
    k = torch.randn(B, len(heads), Lk, D, device=dev, generator=gen).bfloat16()
    v = torch.randn(B, len(heads), Lk, D, device=dev, generator=gen).bfloat16()
    q = torch.randn(B, Hq, Lq, D, device=dev, generator=gen).bfloat16()
    kq, vq = ops.quant_pack_rows(k, group, bits, True), ops.quant_pack_rows(v, group, bits, True)
    hm = torch.tensor(heads, dtype=torch.int32, device=dev)
    note('fused_attn tokens-first out', D, group, bits, Lq, Lk, splits)
    a = torch.full((B, Hq, Lq, D), 7.0, dtype=torch.bfloat16, device=dev)
    ops.fused_attn(q, *kq, *vq, bits, bits, Lk, 1 / math.sqrt(D), head_map=hm, out=a, splits=splits)
    b = torch.full((B, Lq, Hq, D), 7.0, dtype=torch.bfloat16, device=dev)
    ops.fused_attn(q, *kq, *vq, bits, bits, Lk, 1 / math.sqrt(D), head_map=hm, out=b, splits=splits, out_layout='BLHc')
    c = ops.fused_attn(q[:, heads].contiguous(), *kq, *vq, bits, bits, Lk, 1 / math.sqrt(D), splits=splits, out_layout='BLHc')
    torch.cuda.synchronize()
    assert torch.equal(b.transpose(1, 2), a)
    assert c.shape == (B, Lq, len(heads), D) and torch.equal(c.transpose(1, 2), a[:, heads])
    assert bool((b[:, :, [1, 2]] == 7.0).all()) and not bool((b[:, :, heads] == 7.0).all())


def test_tokens_first_output_with_tables(dev):
    B, H, D, bits, L = 2, 3, 64, 8, 700
    gen = torch.Generator(device=dev).manual_seed(5)
    kw = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, L, D * bits // 32), device=dev, generator=gen, dtype=torch.int64).int()
    vw = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, L, D * bits // 32), device=dev, generator=gen, dtype=torch.int64).int()
    ks, vs = (torch.rand(1, H, D, device=dev, generator=gen) * 0.02 + 0.01 for _ in range(2))
    q = torch.randn(B, H, 200, D, device=dev, generator=gen).bfloat16()
    note('fused_attn_channel tokens-first out')
    a = ops.fused_attn_channel(q, kw, ks, None, vw, vs, None, bits, L, 0.1)
    b = ops.fused_attn_channel(q, kw, ks, None, vw, vs, None, bits, L, 0.1, out_layout='BLHc')
    torch.cuda.synchronize()
    assert b.shape == (B, 200, H, D) and torch.equal(b.transpose(1, 2), a)

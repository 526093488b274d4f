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

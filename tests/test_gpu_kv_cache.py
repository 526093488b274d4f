"""Incremental generation over a scale schedule with the pre-allocated packed
cache: append a step, attend with that step's queries (BASELINE config 5 in
miniature, mixed per-head bit-widths)."""
import math

import pytest
import torch

import varq_oracle as O
from gpu_util import note
from var_q_amd import PackedKVCache

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('mixed', [False, True])
def test_incremental_schedule(dev, mixed):
    B, H, D, g = 2, 6, 128, 64
    pn = (1, 2, 4, 6, 8)
    L = sum(p * p for p in pn)
    gen = torch.Generator().manual_seed(5000)
    bits = [int(b) for b in torch.tensor([2, 4, 8])[torch.randint(0, 3, (H,), generator=gen)]] if mixed else 4
    if mixed:
        bits[0], bits[1], bits[2] = 2, 4, 8
    cache = PackedKVCache(B, H, L, D, bits, g, dev)
    ks, vs = [], []
    scale = 1.0 / math.sqrt(D)
    for p in pn:
        n = p * p
        k = O.synth_kv((B, H, n, D), 100 + p).bfloat16()
        v = O.synth_kv((B, H, n, D), 200 + p).bfloat16()
        q = torch.randn(B, H, n, D, generator=gen).bfloat16()
        ks.append(k); vs.append(v)
        note('kv cache step', p, 'bits', bits)
        cache.append(k.to(dev), v.to(dev))
        out = cache.attend(q.to(dev), scale)
        torch.cuda.synchronize()
        kcat, vcat = torch.cat(ks, 2), torch.cat(vs, 2)
        per_head = bits if mixed else [4] * H
        kd, vd = torch.empty_like(kcat, dtype=torch.float32), torch.empty_like(vcat, dtype=torch.float32)
        for h in range(H):
            for src, dst in ((kcat, kd), (vcat, vd)):
                qq, s, z = O.quant_groupwise(src[:, h], g, per_head[h], True)
                dst[:, h] = O.dequant_groupwise(qq, s, z, g)
        # cache contents are bit-exact, attention within tolerance
        assert torch.equal(cache.dequant('k').cpu(), kd) and torch.equal(cache.dequant('v').cpu(), vd)
        ref = O.attention_ref(q, kd, vd, scale).double()
        got = out.double().cpu()
        span = max(1.0, float(ref.abs().max()))
        assert float((got - ref).abs().max()) <= 2e-2 * span
        assert float(torch.nn.functional.cosine_similarity(got.flatten(), ref.flatten(), dim=0)) >= 0.9995
    assert cache.len == L


def test_overflow_is_refused(dev):
    cache = PackedKVCache(1, 2, 4, 64, 4, 64, dev)
    x = torch.randn(1, 2, 3, 64, device=dev).bfloat16()
    cache.append(x, x)
    with pytest.raises(AssertionError):
        cache.append(x, x)

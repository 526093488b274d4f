"""Incremental generation over a scale schedule with the pre-allocated packed
cache: append a step, attend with that step's queries (benchmark configuration 5 in
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


def test_classes_on_side_streams_equal_one_stream(dev):
    """attend() of a mixed-width cache launches its bit-width classes on one stream each;
    the result is the one-stream result bit for bit, also when the caller's stream goes
    straight on to overwrite the inputs."""
    B, H, D, L = 2, 6, 128, 700
    gen = torch.Generator().manual_seed(77)
    cache = PackedKVCache(B, H, L, D, [2, 4, 8, 8, 4, 2], 64, dev)
    k, v = (torch.randn(B, H, L, D, generator=gen).bfloat16().to(dev) for _ in range(2))
    q = torch.randn(B, H, 300, D, generator=gen).bfloat16().to(dev)
    cache.append(k, v)
    cache.splits = 1     # (on one stream the library would share the keys out; same arithmetic wanted here)
    assert cache.concurrent_min_flops > 0     # (the default keeps a call of this size on one stream ...)
    cache.concurrent_min_flops = 0            # (... so the streams are forced here)
    outs = {}
    for mode in (False, True, True):
        cache.concurrent_classes = mode
        note('kv cache attend, side streams', mode)
        qq = q.clone()
        o = cache.attend(qq, 0.09)
        qq.zero_()                       # ordered after all classes on the caller's stream
        outs.setdefault(mode, []).append(o)
    torch.cuda.synchronize()
    assert torch.equal(outs[False][0], outs[True][0]) and torch.equal(outs[True][0], outs[True][1])


def test_overflow_is_refused(dev):
    cache = PackedKVCache(1, 2, 4, 64, 4, 64, dev)
    x = torch.randn(1, 2, 3, 64, device=dev).bfloat16()
    cache.append(x, x)
    with pytest.raises(AssertionError):
        cache.append(x, x)


def test_descriptor_save_load_round_trip(dev, tmp_path):
    """The hand-over format: descriptor + named buffers; a cache written to a file and
    read back (into a larger capacity) holds the same codes and attends identically."""
    import json
    g = torch.Generator().manual_seed(77)
    B, H, D = 2, 6, 64
    bits = [8, 4, 2, 4, 8, 2]
    cache = PackedKVCache(B, H, 40, D, bits, 32, dev)
    for n in (1, 4, 9, 16):
        note('kv_cache save/load append', n)
        cache.append(torch.randn(B, H, n, D, generator=g).to(dev), torch.randn(B, H, n, D, generator=g).to(dev))
    d = cache.descriptor()
    json.dumps(d)                                     # serialisable
    assert d['len'] == 30 and d['per_head_bits'] == bits and [c['bits'] for c in d['classes']] == [2, 4, 8]
    for c in d['classes']:
        assert c['meta'] == {'orig_c': D, 'vals_per_word': 32 // c['bits'], 'pad_len': 0, 'bits': c['bits']}
        assert c['words']['shape'] == [B, len(c['heads']), 40, D * c['bits'] // 32]
        assert tuple(cache.tensors()['b%d.k_words' % c['bits']].shape) == tuple(c['words']['shape'])
    path = str(tmp_path / 'cache.safetensors')
    cache.save(path)
    back = PackedKVCache.load(path, dev, Lmax=64)
    assert back.len == 30 and back.Lmax == 64 and back.per_head_bits == bits
    assert torch.equal(back.dequant('k'), cache.dequant('k')) and torch.equal(back.dequant('v'), cache.dequant('v'))
    q = torch.randn(B, H, 16, D, generator=g).to(dev).bfloat16()
    assert torch.equal(back.attend(q, 0.125), cache.attend(q, 0.125))
    # and it keeps growing where the saved one stopped
    k, v = torch.randn(B, H, 5, D, generator=g).to(dev), torch.randn(B, H, 5, D, generator=g).to(dev)
    back.append(k, v)
    cache.append(k, v)
    assert torch.equal(back.dequant('k'), cache.dequant('k'))

"""The benchmark configurations end to end, at their own shapes and data distributions.

  * configuration 1: INT8 symmetric per-head quantization through the drop-in class
    (method G_HEAD), pack, unpack, dequantize, and the final-scale 256 queries over all
    680 keys -- both as the reference composes it (dequant_all -> attention) and through
    fused_attention;
  * configuration 2 at the full batch of 64 (K group 32, V group 64, INT4) and
    configuration 3 at the full batch of 32 (one table per (head, channel), INT2 affine
    and INT8 symmetric): codes bit-exact against the oracle at full size, the attention
    against the oracle on the first and last batch entries, and size-independent
    properties on the whole launch;
  * configuration 5: the whole 13-scale Infinity schedule through the pre-allocated
    mixed-width cache (one head per bit-width class, group 64), every scale's output
    against the oracle, with the library's own choice of key sharing and the classes
    on side streams.
Tolerances as in test_gpu_attention.py."""
import math

import pytest
import torch

import varq_oracle as O
from gpu_util import note
from test_gpu_attention import _compare
from var_q_amd import PackedKVCache, VAR_Q, ops, schedules
from var_q_amd.quant import fused_attention

pytestmark = pytest.mark.gpu


def _exact(q, kd, vd, scale, dev):
    return O.attention_exact(q.float().to(dev), kd.to(dev), vd.to(dev), scale).cpu()


def test_config1_per_head_int8_end_to_end(dev):
    """VAR-d16 K/V [2,16,680,64] fp32, 2 % of the channels x15, INT8 symmetric per head."""
    B, H, L, D, Lq = 2, 16, 680, 64, 256
    k, v = O.synth_kv((B, H, L, D), 1001), O.synth_kv((B, H, L, D), 2001)
    q = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(3001))
    scale = 1.0 / math.sqrt(D)
    kq, vq = VAR_Q(8, 'BHLc', 'G_HEAD'), VAR_Q(8, 'BHLc', 'G_HEAD')
    note('config 1: quantize, pack, cache')
    deq = {}
    for name, qz, x in (('k', kq, k), ('v', vq, v)):
        qz.quant(x.to(dev))
        qz.cache()
        s = O.scale_sym(x, (0, 2, 3), 8)
        codes = O.codes_sym(x, s, 8)
        words, meta = O.pack_last_dim(codes, 8)
        assert torch.equal(qz.scale.cpu(), s) and qz.scale.shape == (1, H, 1, 1)
        assert torch.equal(qz.cached_item.cpu(), words) and qz.cached_item.shape == (B, H, L, D // 4)
        assert qz._pack_meta == meta
        assert torch.equal(O.unpack_last_dim(words, meta), codes)
        deq[name] = O.dequant_sym(codes, s)
        note('config 1: unpack + dequantize', name)
        assert torch.equal(qz.dequant_all().cpu(), deq[name])      # fp32, bit for bit
    # the final scale's queries see every key: the block-causal limit of the last 256 tokens
    lim = schedules.kv_limit(O.VAR_PATCH_NUMS, L - Lq)
    assert int(lim.min()) == L
    bias = O.block_causal_bias(O.VAR_PATCH_NUMS, L - Lq)
    ref = O.attention_ref(q, deq['k'], deq['v'], scale, bias)
    exact = O.attention_exact(q, deq['k'], deq['v'], scale, bias)
    note('config 1: dequant_all -> attention, as the reference composes it')
    kd, vd = kq.dequant_all(), vq.dequant_all()
    plain = torch.nn.functional.scaled_dot_product_attention(q.to(dev).bfloat16(), kd.bfloat16(), vd.bfloat16(), scale=scale)
    _compare(plain, ref, exact, 'c1 drop-in')
    # ... and in fp32, the precision configuration 1 names: the oracle's fp32 attention on the CPU
    plain32 = torch.nn.functional.scaled_dot_product_attention(q.to(dev), kd, vd, scale=scale)
    ref32 = O.attention_ref(q, deq['k'], deq['v'], scale, bias, dtype=torch.float32)
    assert float((plain32.cpu() - ref32).abs().max()) <= 1e-4 * max(1.0, float(ref32.abs().max()))
    note('config 1: fused_attention over the two quantizers')
    out = fused_attention(q.to(dev), kq, vq, scale, kv_limit=lim.to(dev))
    torch.cuda.synchronize()
    _compare(out, O.attention_ref(q.bfloat16(), deq['k'], deq['v'], scale, bias),
             O.attention_exact(q.bfloat16().float(), deq['k'], deq['v'], scale, bias), 'c1 fused')


def _properties(run, vconst, Lk, dev, what):
    """What holds at any size.  run(kv_limit=None, perm=None, pad=0, v=None) -> output."""
    note(what, 'full size: limit == length')
    base = run()
    lq = base.shape[2]
    assert not bool(torch.isnan(base.float()).any())
    assert torch.equal(run(kv_limit=torch.full((lq,), Lk, dtype=torch.int32, device=dev)), base)
    note(what, 'full size: permuted keys')
    g = torch.Generator(device=dev).manual_seed(7)
    other = run(perm=torch.randperm(Lk, device=dev, generator=g))
    span = max(1.0, float(base.float().abs().max()))
    # (a quarter of the bar, or one bf16 step of the largest output where that is more)
    assert float((other.float() - base.float()).abs().max()) <= max(2e-2 * span / 4, span * 2 ** -7)
    assert float(torch.nn.functional.cosine_similarity(other.flatten().double(), base.flatten().double(), dim=0)) >= 0.99999
    note(what, 'full size: rows beyond the length')
    assert torch.equal(run(pad=70), base)
    note(what, 'full size: constant V')
    out = run(v=vconst)
    assert float((out.float() - 1.25).abs().max()) <= 2 ** -7, 'softmax weights do not sum to one'
    return base


def test_config2_full_batch(dev):
    """VAR-d16 batch shape: bf16 K/V [64,16,680,64], INT4 affine, K group 32, V group 64."""
    B, H, L, D, Lq, bits, gk, gv = 64, 16, 680, 64, 256, 4, 32, 64
    k, v = O.synth_kv((B, H, L, D), 1002).bfloat16(), O.synth_kv((B, H, L, D), 2002).bfloat16()
    q = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(3002)).bfloat16()
    scale = 1.0 / math.sqrt(D)
    note('config 2 full size: quantize + pack')
    kk, vv = ops.quant_pack_rows(k.to(dev), gk, bits, True), ops.quant_pack_rows(v.to(dev), gv, bits, True)
    deq = []
    for got, x, g in ((kk, k, gk), (vv, v, gv)):
        codes, s, z = O.quant_groupwise(x, g, bits, True)
        assert torch.equal(got[0].cpu(), O.pack_last_dim(codes, bits)[0])
        assert torch.equal(got[1].cpu(), s) and torch.equal(got[2].cpu(), z)
        assert got[0].shape == (B, H, L, D * bits // 32) and got[1].shape == (B, H, L, D // g)
        deq.append(O.dequant_groupwise(codes, s, z, g))
    qd = q.to(dev)

    def run(kv_limit=None, perm=None, pad=0, v=None):
        kt, vt = list(kk), list(vv if v is None else v)
        if perm is not None:
            kt, vt = [t[:, :, perm].contiguous() for t in kt], [t[:, :, perm].contiguous() for t in vt]
        if pad:
            junk = lambda t: torch.full_like(t[:, :, :pad], 0x7f if t.dtype == torch.int32 else 1e30)
            kt, vt = [torch.cat([t, junk(t)], 2).contiguous() for t in kt], [torch.cat([t, junk(t)], 2).contiguous() for t in vt]
        return ops.fused_attn(qd, *kt, *vt, bits, bits, L, scale, kv_limit=kv_limit)

    code = 5
    vs = torch.rand(B, H, L, D // gv, device=dev) + 0.5
    vconst = (torch.full_like(vv[0], int.from_bytes(bytes([code * 17] * 4), 'little', signed=True)), vs, code - 1.25 / vs)
    base = _properties(run, vconst, L, dev, 'config 2')
    torch.cuda.synchronize()
    for b in (0, B - 1):     # the oracle's attention on the first and last batch entries
        sl = slice(b, b + 1)
        _compare(base[sl], O.attention_ref(q[sl], deq[0][sl], deq[1][sl], scale),
                 _exact(q[sl], deq[0][sl], deq[1][sl], scale, dev), f'c2 full batch, entry {b}')


@pytest.mark.parametrize('bits,asym', [(2, True), (8, False)])
def test_config3_full_batch(dev, bits, asym):
    """VAR-d30 shape: bf16 K/V [32,30,680,64]; INT2 affine per head and channel, and the INT8
    symmetric per-channel variant (the reference's G_SCALE_HEAD_DIM / G_HEAD_DIM scale layout)."""
    B, H, L, D, Lq = 32, 30, 680, 64, 256
    k, v = O.synth_kv((B, H, L, D), 1003).bfloat16(), O.synth_kv((B, H, L, D), 2003).bfloat16()
    q = torch.randn(B, H, Lq, D, generator=torch.Generator().manual_seed(3003)).bfloat16()
    scale = 1.0 / math.sqrt(D)
    note('config 3 full size: quantize + pack', bits, asym)
    kk, vv = ops.quant_pack(k.to(dev), (0, 2), bits, asym), ops.quant_pack(v.to(dev), (0, 2), bits, asym)
    deq = []
    for got, x in ((kk, k), (vv, v)):
        codes, s, z = O.quant_reduce(x, (0, 2), bits, asym)
        assert torch.equal(got[0].cpu(), O.pack_last_dim(codes, bits)[0]) and torch.equal(got[1].cpu(), s)
        assert (z is None and got[2] is None) or torch.equal(got[2].cpu(), z)
        assert got[0].shape == (B, H, L, D * bits // 32) and got[1].shape == (1, H, 1, D)
        deq.append(O.dequant_asym(codes, s, z) if asym else O.dequant_sym(codes, s))
    tab = lambda t: None if t is None else t.reshape(H, D).contiguous()
    qd = q.to(dev)

    def run(kv_limit=None, perm=None, pad=0, v=None):
        kw, vw = kk[0], vv[0]
        vsc, vzp = tab(vv[1]), tab(vv[2])
        if v is not None:
            vw, vsc, vzp = v
        if perm is not None:
            kw, vw = kw[:, :, perm].contiguous(), vw[:, :, perm].contiguous()
        if pad:
            kw, vw = [torch.cat([t, torch.full_like(t[:, :, :pad], 0x7f)], 2).contiguous() for t in (kw, vw)]
        return ops.fused_attn_channel(qd, kw, tab(kk[1]), tab(kk[2]), vw, vsc, vzp, bits, L, scale, kv_limit=kv_limit)

    # a V cache that dequantizes to 1.25 everywhere: code 1 in every field, per-channel scales
    # between 0.5 and 1.5, zero-point 1 - 1.25 / scale
    field = {2: 0x55, 8: 0x01}[bits]
    vs = torch.rand(H, D, device=dev) + 0.5
    vconst = (torch.full_like(vv[0], int.from_bytes(bytes([field] * 4), 'little', signed=True)), vs, 1 - 1.25 / vs)
    base = _properties(run, vconst, L, dev, 'config 3')
    torch.cuda.synchronize()
    for b in (0, B - 1):
        sl = slice(b, b + 1)
        _compare(base[sl], O.attention_ref(q[sl], deq[0][sl], deq[1][sl], scale),
                 _exact(q[sl], deq[0][sl], deq[1][sl], scale, dev), f'c3 full batch int{bits}, entry {b}', oracle_bar=1e-2)


def test_config5_full_schedule_mixed_bits(dev):
    """The 13 scales of the Infinity schedule (10 521 tokens), one head per bit-width class
    (2, 4 and 8 bits), group 64, Student-t data with an outlier channel x20: append each
    scale's tokens, attend with that scale's queries over everything cached so far."""
    B, D, g = 1, 128, 64
    bits = [2, 4, 8]
    H = len(bits)
    pn = schedules.INFINITY_PATCH_NUMS
    L = schedules.total_tokens(pn)
    cache = PackedKVCache(B, H, L, D, bits, g, dev)
    assert cache.concurrent_classes and cache.splits == 0     # the defaults: side streams, library-chosen sharing
    scale = 1.0 / math.sqrt(D)
    gen = torch.Generator().manual_seed(5005)
    kd = torch.empty(B, H, L, D)
    vd = torch.empty(B, H, L, D)
    pos = 0
    for i, p in enumerate(pn):
        n = p * p
        k = O.synth_kv((B, H, n, D), 5100 + i, 'student4', 0.01, 20.0, outlier_seed=5001).bfloat16()
        v = O.synth_kv((B, H, n, D), 5200 + i, 'student4', 0.01, 20.0, outlier_seed=5002).bfloat16()
        q = torch.randn(B, H, n, D, generator=gen).bfloat16()
        note('config 5 scale', p, 'tokens', n, 'prefix', pos + n)
        cache.append(k.to(dev), v.to(dev))
        out = cache.attend(q.to(dev), scale)
        torch.cuda.synchronize()
        for h in range(H):          # groups are per token: a step's dequantized rows never change afterwards
            for src, dst in ((k, kd), (v, vd)):
                codes, s, z = O.quant_groupwise(src[:, h], g, bits[h], True)
                dst[:, h, pos:pos + n] = O.dequant_groupwise(codes, s, z, g)
        pos += n
        if p in (1, 8, 64):          # the cache holds exactly the oracle's values (checked where it is cheap and at the end)
            assert torch.equal(cache.dequant('k').cpu(), kd[:, :, :pos]) and torch.equal(cache.dequant('v').cpu(), vd[:, :, :pos])
        ref = O.attention_ref(q, kd[:, :, :pos], vd[:, :, :pos], scale)
        _compare(out, ref, _exact(q, kd[:, :, :pos], vd[:, :, :pos], scale, dev), f'c5 scale {p}')
    assert cache.len == L == 10521


def test_config5_full_size_seeded_bits(dev):
    """Configuration 5 at the size it is named at: B=8 (4 images x CFG pair), H=16, the seeded
    per-head bit-widths of bench.py, the 13 scales on heavy-tailed data (Student-t, nu=4, one
    channel x20, generated on the device).  Checked: for one (batch, head) per bit-width class the
    cache contents bit for bit against the oracle and that head's attention at scales 1, 8, 32
    and 64 against the oracle's bf16 attention (bench.c5_check, which bench.py's own leg runs);
    and on the last scale's launch -- all 128 (batch, head) pairs, the three classes side by
    side, the library's choice of key sharing -- what holds at any size (`_properties`)."""
    import bench
    B, H, D, g = bench.C5_B, bench.C5_H, bench.C5_D, bench.C5_GROUP
    bits = bench.c5_head_bits(torch)
    assert sorted(set(bits)) == [2, 4, 8] and len(bits) == H
    pn = schedules.INFINITY_PATCH_NUMS
    ns = schedules.tokens_per_scale(pn)
    L = sum(ns)
    gen = torch.Generator(device=dev).manual_seed(5505)

    def student(n):
        x = torch.randn(B, H, n, D, device=dev, generator=gen)
        chi = torch.randn(4, B, H, n, D, device=dev, generator=gen).square_().mean(0)
        x = x / chi.sqrt_()
        x[..., 77] *= 20.0
        return x.bfloat16()
    steps = [(torch.randn(B, H, n, D, device=dev, generator=gen).bfloat16(), student(n), student(n)) for n in ns]
    cache = PackedKVCache(B, H, L, D, bits, g, dev)
    scale = 1.0 / math.sqrt(D)
    outs = []
    for i, (q, k, v) in enumerate(steps):
        note('config 5 full size: scale', pn[i], 'tokens', ns[i])
        cache.append(k, v)
        outs.append(cache.attend(q, scale))
    torch.cuda.synchronize()
    assert cache.len == L
    note('config 5 full size: against the oracle')
    res = bench.c5_check(torch, O, dev, cache, steps, outs, bits)
    print('[c5 full size]', res, flush=True)
    assert res['cache_bit_exact'], res
    assert res['attn_maxabs_over_range_max'] <= 2e-2 and res['attn_cosine_min'] >= 0.9995, res
    assert len(res['pairs']) == 3

    # the last scale's queries over the whole cache, class by class into one output
    q = steps[-1][0]

    def run(kv_limit=None, perm=None, pad=0, v=None):
        out = torch.zeros_like(q)
        for ci, c in enumerate(cache.classes):
            kt = [c.k_words, c.k_scale, c.k_zp]
            vt = [c.v_words, c.v_scale, c.v_zp] if v is None else list(v[ci])
            if perm is not None:
                kt, vt = [t[:, :, perm].contiguous() for t in kt], [t[:, :, perm].contiguous() for t in vt]
            if pad:
                junk = lambda t: torch.full_like(t[:, :, :pad], 0x7f if t.dtype == torch.int32 else 1e30)
                kt, vt = [torch.cat([t, junk(t)], 2).contiguous() for t in kt], [torch.cat([t, junk(t)], 2).contiguous() for t in vt]
            ops.fused_attn(q, *kt, *vt, c.bits, c.bits, L, scale, kv_limit=kv_limit, head_map=c.head_map, out=out,
                           splits=1)       # (as attend() launches classes that run side by side)
        return out

    # V caches that dequantize to 1.25 everywhere: every field holds code 1 (2 and 8 bits) or 5 (4 bits)
    vconst = []
    for c in cache.classes:
        byte, code = {2: (0x55, 1), 4: (0x55, 5), 8: (0x01, 1)}[c.bits]
        vs = torch.rand(c.v_scale.shape, device=dev, generator=gen) + 0.5
        vconst.append((torch.full_like(c.v_words, int.from_bytes(bytes([byte] * 4), 'little', signed=True)), vs, code - 1.25 / vs))
    base = _properties(run, vconst, L, dev, 'config 5')
    assert torch.equal(base, outs[-1]), 'the classes launched one by one and PackedKVCache.attend differ'

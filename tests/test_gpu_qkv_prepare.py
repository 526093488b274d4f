"""Producer-side fusion (normalise + scale + rotate + quantize into the cache in one
kernel) against the CPU oracle: the prepared q (bf16), the packed words, scales and
zero-points of k and v are bit-exact, because the oracle fixes the one thing the
reference's tensor expressions leave open, the summation order of the norm."""
import pytest
import torch

import varq_oracle as O
from gpu_util import note
from var_q_amd import PackedKVCache, hooks, ops

pytestmark = pytest.mark.gpu


def _run(dev, B, L, H, c, dtype, bits, group, asym, l2norm, with_mul, with_rope, start=0, Lmax=None, off=0):
    g = torch.Generator().manual_seed(B * 131 + L * 17 + c + bits)
    qkv = (torch.randn(B, L, 3, H, c, generator=g) * 1.7).to(dtype)
    qkv[..., 3] *= 9
    mul = (torch.rand(H, generator=g) * 5 + 0.5) if with_mul else None
    rope = None
    if with_rope:
        hw = [(3, 4), (5, 5), (8, 8)]
        rope = hooks.rope2d_tables(c, hw)
        assert rope[0].shape[0] >= start + L
    qo, ko, vo = O.prepare_qkv(qkv, mul, l2norm, 1e-12, rope, start)
    Lmax = Lmax or (L + off)
    W, ns = c * bits // 32, c // group
    mk = lambda last, dt: torch.full((B, H, Lmax, last), 7, dtype=dt, device=dev)
    kw, vw = mk(W, torch.int32), mk(W, torch.int32)
    ks, kz, vs, vz = (mk(ns, torch.float32) for _ in range(4))
    q_out = torch.empty(B, H, L, c, dtype=torch.bfloat16, device=dev)
    rowmap = [B, L, H, H * Lmax, 1, Lmax, off, -1]
    ops.qkv_prepare_append(qkv.to(dev), q_out, group, bits, asym, 1e-12, kw, ks, kz if asym else None,
                           vw, vs, vz if asym else None, rowmap, None,
                           None if mul is None else mul.to(dev), l2norm, 1e-12,
                           None if rope is None else (rope[0].to(dev), rope[1].to(dev)), start)
    torch.cuda.synchronize()
    assert torch.equal(q_out.cpu().view(torch.int16), qo.view(torch.int16)), 'prepared q differs'
    for name, x, w, s, z in (('k', ko, kw, ks, kz), ('v', vo, vw, vs, vz)):
        cq, cs, cz = O.quant_groupwise(x, group, bits, asym)
        want, _ = O.pack_last_dim(cq, bits)
        sl = slice(off, off + L)
        assert torch.equal(s[:, :, sl].cpu(), cs), f'{name} scale differs'
        if asym:
            assert torch.equal(z[:, :, sl].cpu(), cz), f'{name} zero-point differs'
        assert torch.equal(w[:, :, sl].cpu(), want), f'{name} packed words differ'
        if off:
            assert bool((w[:, :, :off] == 7).all()) and bool((s[:, :, :off] == 7).all()), 'rows outside the step touched'


@pytest.mark.parametrize('c,group', [(64, 64), (64, 32), (128, 128), (128, 64), (128, 16), (32, 32)])
@pytest.mark.parametrize('bits,asym', [(4, True), (8, False), (2, True)])
def test_infinity_style_norm_scale_rope(dev, c, group, bits, asym):
    for dtype in (torch.bfloat16, torch.float32):
        note('qkv_prepare infinity', c, group, bits, asym, dtype)
        _run(dev, 2, 9, 3, c, dtype, bits, group, asym, True, True, True, start=5, Lmax=20, off=4)


@pytest.mark.parametrize('l2norm,with_mul,with_rope', [(False, False, False), (True, False, False), (True, True, False),
                                                       (False, False, True)])
def test_var_style_and_partial_pipelines(dev, l2norm, with_mul, with_rope):
    note('qkv_prepare var', l2norm, with_mul, with_rope)
    _run(dev, 3, 16, 5, 64, torch.float16, 4, 64, True, l2norm, with_mul, with_rope)
    _run(dev, 1, 1, 1, 128, torch.bfloat16, 8, 128, False, l2norm, with_mul, with_rope)


def test_zero_rows_and_tiny_norms(dev):
    """An all-zero token (norm clamps to eps) and denormal-sized rows."""
    B, L, H, c = 1, 4, 2, 64
    qkv = torch.randn(B, L, 3, H, c, generator=torch.Generator().manual_seed(9))
    qkv[0, 1] = 0.0
    qkv[0, 2] *= 1e-30
    q_ref, k_ref, _ = O.prepare_qkv(qkv, None, True)
    kw = torch.zeros(B, H, L, c // 8, dtype=torch.int32, device=dev)
    vw = torch.zeros_like(kw)
    ks, kz, vs, vz = (torch.zeros(B, H, L, 1, device=dev) for _ in range(4))
    q_out = torch.empty(B, H, L, c, dtype=torch.bfloat16, device=dev)
    note('qkv_prepare zero rows')
    ops.qkv_prepare_append(qkv.to(dev), q_out, 64, 4, True, 1e-12, kw, ks, kz, vw, vs, vz, [B, L, H, H * L, 1, L, 0, -1],
                           l2norm=True)
    assert torch.equal(q_out.cpu().view(torch.int16), q_ref.view(torch.int16))
    cq, cs, cz = O.quant_groupwise(k_ref, 64, 4, True)
    assert torch.equal(ks.cpu(), cs) and torch.equal(kz.cpu(), cz) and torch.equal(kw.cpu(), O.pack_last_dim(cq, 4)[0])


def test_cache_append_from_qkv_mixed_bits(dev):
    """Through the cache class, heads of different widths: equals preparing on the CPU
    and appending k, v the ordinary way."""
    B, H, D = 2, 6, 128
    bits = [4, 8, 2, 4, 8, 2]
    hw = [(1, 1), (2, 2), (4, 4)]
    rope = hooks.rope2d_tables(D, hw)
    rope_d = (rope[0].to(dev), rope[1].to(dev))
    mul = torch.rand(H, generator=torch.Generator().manual_seed(2)) * 3 + 1
    a = PackedKVCache(B, H, 21, D, bits, 64, dev)
    b = PackedKVCache(B, H, 21, D, bits, 64, dev)
    g = torch.Generator().manual_seed(3)
    for h_, w_ in hw:
        n = h_ * w_
        qkv = torch.randn(B, n, 3, H, D, generator=g).bfloat16()
        start = a.len
        note('qkv_prepare cache', n)
        q_gpu = a.append_from_qkv(qkv.to(dev), mul.to(dev), True, 1e-12, rope_d)
        q_ref, k_ref, v_ref = O.prepare_qkv(qkv, mul, True, 1e-12, rope, start)
        b.append(k_ref.to(dev), v_ref.to(dev))
        assert torch.equal(q_gpu.cpu().view(torch.int16), q_ref.view(torch.int16))
    assert a.len == b.len == 21
    assert torch.equal(a.dequant('k'), b.dequant('k')) and torch.equal(a.dequant('v'), b.dequant('v'))


@pytest.mark.parametrize('bits', [8, 4])
def test_zero_points_around_the_rounding_shortcuts_limit(dev, bits):
    """v is quantized as it comes (no norm, no rotation): rows of integers offset by about 2^21
    and 2^22 quantization steps put the zero-point on either side of the limit up to which the
    kernel rounds by adding 1.5 * 2^23; beyond it the division path must take over."""
    B, L, H, c = 1, 26, 1, 64
    qkv = torch.zeros(B, L, 3, H, c)
    bases = (2 ** 21 - 300, 2 ** 21 - 128, 2 ** 21 - 1, 2 ** 21, 2 ** 21 + 200, 2 ** 22 - 400, 2 ** 22 - 256,
             2 ** 22 - 130, 2 ** 22 - 128, 2 ** 22 - 1, 2 ** 22, 2 ** 22 + 300, 2 ** 23 - 256)
    k = torch.arange(c, dtype=torch.float32) * 255 // (c - 1)
    for i, base in enumerate(bases):
        qkv[0, 2 * i, 2, 0] = k + float(base)
        qkv[0, 2 * i + 1, 2, 0] = -(k + float(base))
    qkv[:, :, :2] = torch.randn(B, L, 2, H, c, generator=torch.Generator().manual_seed(4))
    _, _, v_ref = O.prepare_qkv(qkv, None, False)
    W = c * bits // 32
    kw, vw = (torch.zeros(B, H, L, W, dtype=torch.int32, device=dev) for _ in range(2))
    ks, kz, vs, vz = (torch.zeros(B, H, L, 1, device=dev) for _ in range(4))
    q_out = torch.empty(B, H, L, c, dtype=torch.bfloat16, device=dev)
    note('qkv_prepare zero-point limit', bits)
    ops.qkv_prepare_append(qkv.to(dev), q_out, c, bits, True, 1e-12, kw, ks, kz, vw, vs, vz, [B, L, H, H * L, 1, L, 0, -1])
    cq, cs, cz = O.quant_groupwise(v_ref, c, bits, True)
    assert torch.equal(vs.cpu(), cs) and torch.equal(vz.cpu(), cz)
    assert torch.equal(vw.cpu(), O.pack_last_dim(cq, bits)[0])


def test_half_a_million_tokens_of_one_head(dev):
    """One head of 524 328 tokens at c = 128 (32 771 tiles of 16 tokens, not a multiple of the eight
    that the workgroup order deals out together): the whole launch equals two launches over its
    halves (bit for bit, every output), and its last tokens equal the oracle's."""
    B, L, H, c, bits, group = 1, 32768 * 16 + 40, 1, 128, 4, 128
    g = torch.Generator(device=dev).manual_seed(77)
    qkv = torch.randn(B, L, 3, H, c, device=dev, generator=g).bfloat16()
    mul = torch.tensor([1.75], device=dev)

    def run(x, outs, off):
        n = x.shape[1]
        rowmap = [B, n, H, H * L, 1, L, off, -1]
        q_out = torch.empty(B, H, n, c, dtype=torch.bfloat16, device=dev)
        ops.qkv_prepare_append(x, q_out, group, bits, True, 1e-12, *outs, rowmap, None, mul, True, 1e-12, None, 0)
        return q_out

    def buffers():
        mk = lambda last, dt: torch.full((B, H, L, last), 7, dtype=dt, device=dev)
        W = c * bits // 32
        return (mk(W, torch.int32), mk(1, torch.float32), mk(1, torch.float32),
                mk(W, torch.int32), mk(1, torch.float32), mk(1, torch.float32))

    note('qkv_prepare 524328 tokens, one launch')
    whole = buffers()
    q_whole = run(qkv, whole, 0)
    note('qkv_prepare 524328 tokens, two launches')
    halves = buffers()
    Lh = L // 2 + 3
    q_a = run(qkv[:, :Lh].contiguous(), halves, 0)
    q_b = run(qkv[:, Lh:].contiguous(), halves, Lh)
    torch.cuda.synchronize()
    assert torch.equal(q_whole, torch.cat([q_a, q_b], dim=2))
    for a, b in zip(whole, halves):
        assert torch.equal(a, b)
    tail = 48
    q_ref, k_ref, v_ref = O.prepare_qkv(qkv[:, -tail:].cpu(), mul.cpu(), True, 1e-12, None, 0)
    assert torch.equal(q_whole[:, :, -tail:].cpu().view(torch.int16), q_ref.view(torch.int16))
    for x, (w, s, z) in ((k_ref, whole[:3]), (v_ref, whole[3:])):
        cq, cs, cz = O.quant_groupwise(x, group, bits, True)
        assert torch.equal(s[:, :, -tail:].cpu(), cs) and torch.equal(z[:, :, -tail:].cpu(), cz)
        assert torch.equal(w[:, :, -tail:].cpu(), O.pack_last_dim(cq, bits)[0])


def test_slot_table_over_heads_leaves_other_heads_alone(dev):
    """One call per bit-width class of a mixed cache: the heads of the class get q, k and v, the
    others nothing (their q included), so that the calls of all classes write every head once."""
    B, L, H, c, bits, group, Lmax = 2, 21, 5, 128, 4, 64, 32
    heads = [3, 0, 4]
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(B, L, 3, H, c, generator=g).bfloat16()
    rope = hooks.rope2d_tables(c, [(3, 3), (4, 4)])
    q_ref, k_ref, v_ref = O.prepare_qkv(qkv, None, True, 1e-12, rope, 0)
    slot = torch.full((H,), -1, dtype=torch.int32)
    for i, h in enumerate(heads):
        slot[h] = i
    hc, W, ns = len(heads), c * bits // 32, c // group
    mk = lambda last, dt: torch.full((B, hc, Lmax, last), 7, dtype=dt, device=dev)
    kw, vw = mk(W, torch.int32), mk(W, torch.int32)
    ks, kz, vs, vz = (mk(ns, torch.float32) for _ in range(4))
    q_out = torch.full((B, H, L, c), 7.0, dtype=torch.bfloat16, device=dev)
    note('qkv_prepare slot table over heads')
    ops.qkv_prepare_append(qkv.to(dev), q_out, group, bits, True, 1e-12, kw, ks, kz, vw, vs, vz,
                           [B, L, H, hc * Lmax, 1, Lmax, 3, 2], slot.to(dev), None, True, 1e-12,
                           (rope[0].to(dev), rope[1].to(dev)), 0)
    torch.cuda.synchronize()
    others = [h for h in range(H) if h not in heads]
    assert bool((q_out[:, others] == 7.0).all()), 'q of a head outside the class was written'
    assert torch.equal(q_out[:, heads].cpu().view(torch.int16), q_ref[:, heads].view(torch.int16))
    for x, w, s, z in ((k_ref, kw, ks, kz), (v_ref, vw, vs, vz)):
        cq, cs, cz = O.quant_groupwise(x[:, heads], group, bits, True)
        assert torch.equal(w[:, :, 3:3 + L].cpu(), O.pack_last_dim(cq, bits)[0])
        assert torch.equal(s[:, :, 3:3 + L].cpu(), cs) and torch.equal(z[:, :, 3:3 + L].cpu(), cz)
        assert bool((w[:, :, :3] == 7).all()) and bool((w[:, :, 3 + L:] == 7).all())


def test_seeded_random_shapes(dev):
    """Thirty seeded random calls: one to 300 tokens (up to 19 tiles of 16 tokens at c = 128, so
    tile counts on either side of the eight that one round of the workgroup order deals out),
    one to three batch entries, one to seven heads, every head dim, width and input type, each
    stage of the pipeline on or off."""
    import random
    rnd = random.Random(777)
    for case in range(30):
        c = rnd.choice([32, 64, 128])
        bits = rnd.choice([2, 4, 8])
        group = rnd.choice([g for g in (8, 16, 32, 64, 128) if g <= c and (bits != 2 or g >= 16)])
        asym = rnd.random() < 0.7
        dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
        B, L, H = rnd.randint(1, 3), rnd.randint(1, 300), rnd.randint(1, 7)
        l2norm, with_mul, with_rope = rnd.random() < 0.7, rnd.random() < 0.5, rnd.random() < 0.6
        start, off = rnd.randint(0, 30), rnd.randint(0, 3)
        g = torch.Generator().manual_seed(5000 + case)
        qkv = (torch.randn(B, L, 3, H, c, generator=g) * rnd.choice([0.05, 1.0, 20.0])).to(dtype)
        mul = (torch.rand(H, generator=g) * 5 + 0.5) if with_mul else None
        rope = hooks.rope2d_tables(c, [(19, 19)]) if with_rope else None      # 361 rows >= start + L
        qo, ko, vo = O.prepare_qkv(qkv, mul, l2norm, 1e-12, rope, start)
        Lmax, W, ns = L + off + rnd.randint(0, 2), c * bits // 32, c // group
        mk = lambda last, dt: torch.full((B, H, Lmax, last), 7, dtype=dt, device=dev)
        kw, vw = mk(W, torch.int32), mk(W, torch.int32)
        ks, kz, vs, vz = (mk(ns, torch.float32) for _ in range(4))
        q_out = torch.empty(B, H, L, c, dtype=torch.bfloat16, device=dev)
        note('qkv_prepare random', case, (B, L, H, c), bits, group, asym, dtype, l2norm, with_mul, with_rope, start, off)
        ops.qkv_prepare_append(qkv.to(dev), q_out, group, bits, asym, 1e-12, kw, ks, kz if asym else None,
                               vw, vs, vz if asym else None, [B, L, H, H * Lmax, 1, Lmax, off, -1], None,
                               None if mul is None else mul.to(dev), l2norm, 1e-12,
                               None if rope is None else (rope[0].to(dev), rope[1].to(dev)), start)
        torch.cuda.synchronize()
        assert torch.equal(q_out.cpu().view(torch.int16), qo.view(torch.int16)), f'case {case}: prepared q differs'
        sl = slice(off, off + L)
        for name, x, w, s, z in (('k', ko, kw, ks, kz), ('v', vo, vw, vs, vz)):
            cq, cs, cz = O.quant_groupwise(x, group, bits, asym)
            assert torch.equal(s[:, :, sl].cpu(), cs), f'case {case}: {name} scale differs'
            assert not asym or torch.equal(z[:, :, sl].cpu(), cz), f'case {case}: {name} zero-point differs'
            assert torch.equal(w[:, :, sl].cpu(), O.pack_last_dim(cq, bits)[0]), f'case {case}: {name} packed words differ'
            assert bool((w[:, :, :off] == 7).all()) and bool((w[:, :, off + L:] == 7).all()), f'case {case}: rows outside the step written'

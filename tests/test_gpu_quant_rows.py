"""Parity of the one-pass row-local quantize+pack kernel (through the C ABI)
with the CPU oracle: packed words, scales and zero-points bit-exact."""
import pytest
import torch

import varq_oracle as O
from gpu_util import adversarial_rows, note
from var_q_amd import ops

pytestmark = pytest.mark.gpu


def _check(x_cpu, group, bits, asym, dev):
    q, s, z = O.quant_groupwise(x_cpu, group, bits, asym)
    want_w, _ = O.pack_last_dim(q, bits)
    w, gs, gz = ops.quant_pack_rows(x_cpu.to(dev), group, bits, asym)
    torch.cuda.synchronize()
    assert torch.equal(gs.cpu(), s), 'scale mismatch'
    if asym:
        assert torch.equal(gz.cpu(), z), 'zero-point mismatch'
    else:
        assert gz is None
    bad = (w.cpu() != want_w)
    assert not bool(bad.any()), f'{int(bad.sum())} packed words differ'


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('asym', [False, True])
def test_random_shapes(dev, dtype, bits, asym):
    g = torch.Generator().manual_seed(bits * 7 + int(asym))
    for shape, group in [((3, 5, 7, 64), 64), ((3, 5, 7, 64), 32), ((2, 4, 33, 128), 128), ((2, 4, 33, 128), 64),
                         ((1, 2, 9, 128), 16), ((300, 64), 8), ((5, 512), 512), ((7, 256), 256)]:
        note('quant_rows', dtype, bits, asym, shape, group)
        x = (torch.randn(*shape, generator=g) * 3).to(dtype)
        x[..., 5] *= 15
        _check(x, group, bits, asym, dev)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('asym', [False, True])
@pytest.mark.parametrize('c,group', [(64, 64), (128, 128), (128, 32)])
def test_adversarial_rows(dev, dtype, bits, asym, c, group):
    note('quant_rows adversarial', dtype, bits, asym, c, group)
    _check(adversarial_rows(c, dtype), group, bits, asym, dev)


@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('asym', [False, True])
@pytest.mark.parametrize('c,group', [(128, 128), (64, 32), (16, 16)])
def test_scale_with_all_ones_significand(dev, bits, asym, c, group):
    """Scales of the form (2 - 2^-23) * 2^e are the one case where correcting x * (1/s)
    by a single residual step does not reproduce the IEEE quotient (x just above
    s/2 yields 0.5 instead of 0.50000006 and rounds to 0 instead of 1): the
    kernel must route such groups through its exact fallback."""
    import numpy as np
    levels = float((1 << bits) - 1) if asym else float((1 << (bits - 1)) - 1)
    rows = []
    for e in range(-6, 4):
        s_star = np.float32((2 - 2.0 ** -23) * 2.0 ** e)
        a = np.float32(np.float64(s_star) * levels)
        cands = [a]
        for _ in range(16):
            cands.append(np.nextafter(cands[-1], np.float32(np.inf)))
        lo = a
        for _ in range(16):
            lo = np.nextafter(lo, np.float32(-np.inf))
            cands.append(lo)
        hit = [v for v in cands if np.float32(v) / np.float32(levels) == s_star]
        assert hit, 'no range value gives the wanted scale'
        top = float(hit[0])
        half = np.float32(np.float64(s_star) * 0.5)
        x = np.zeros(c, dtype=np.float32)
        vals = [np.nextafter(half, np.float32(np.inf)), half, np.nextafter(half, np.float32(0)),
                np.float32(np.float64(s_star) * 1.5), np.nextafter(np.float32(np.float64(s_star) * 2.5), np.float32(np.inf))]
        vals = [v for v in vals if float(v) < top]
        for gi in range(c // group):
            base = gi * group
            x[base] = top                       # fixes the scale of the group (min stays 0 for asym)
            for j, v in enumerate(vals):
                x[base + 1 + j] = v
                if not asym and base + 8 + j < base + group:
                    x[base + 8 + j] = -v
        rows.append(torch.from_numpy(x))
    x = torch.stack(rows)
    q, sc, _ = O.quant_groupwise(x, group, bits, asym)
    assert bool(((sc.view(torch.int32) & 0x7fffff) == 0x7fffff).all()), 'test construction: scale significand not all ones'
    note('quant_rows all-ones scale', bits, asym, c, group)
    _check(x, group, bits, asym, dev)


def test_empty_and_single_row(dev):
    note('quant_rows empty')
    w, s, z = ops.quant_pack_rows(torch.empty(0, 64, dtype=torch.bfloat16, device=dev), 64, 4, True)
    assert w.shape == (0, 8) and s.shape == (0, 1)
    _check(torch.randn(1, 64).bfloat16(), 64, 4, True, dev)


def test_infinity2b_full_shape_int4_g128(dev):
    """benchmark configuration 4 at full size: [2,16,10521,128] bf16, INT4 asym g=128."""
    note('quant_rows c4 full')
    x = O.synth_kv((2, 16, 10521, 128), seed=1004, dist='student4', outlier_frac=0.01, outlier_mul=20.0,
                   dtype=torch.bfloat16)
    _check(x, 128, 4, True, dev)


def test_var_d16_batch_shape_int4(dev):
    """benchmark configuration 2 shapes (B reduced to 8 to keep the CPU oracle quick):
    K group 32, V group 64."""
    note('quant_rows c2')
    k = O.synth_kv((8, 16, 680, 64), seed=1002, dtype=torch.bfloat16)
    _check(k, 32, 4, True, dev)
    _check(k, 64, 4, True, dev)


def test_row_map_appends_into_cache(dev):
    """Two steps written at token offsets of a [B,H,Lmax,...] cache equal the
    concatenation of the steps quantized on their own (VAR_Q/quant.py:196-201)."""
    B, H, D, Lmax, g, bits = 2, 3, 64, 40, 32, 4
    gen = torch.Generator().manual_seed(3)
    words = torch.zeros(B, H, Lmax, D * bits // 32, dtype=torch.int32, device=dev)
    scale = torch.zeros(B, H, Lmax, D // g, device=dev)
    zp = torch.zeros_like(scale)
    off, parts = 0, []
    for n in (1, 4, 9):
        note('row map step', n)
        x = torch.randn(B, H, n, D, generator=gen).bfloat16()
        parts.append(x)
        ops.quant_pack_rows_into(x.to(dev), g, bits, True, 1e-12, words, scale, zp,
                                 [B, H, n, H * Lmax, Lmax, 1, off, -1])
        off += n
    cat = torch.cat(parts, dim=2)
    q, s, z = O.quant_groupwise(cat, g, bits, True)
    assert torch.equal(words[:, :, :off].cpu(), O.pack_last_dim(q, bits)[0])
    assert torch.equal(scale[:, :, :off].cpu(), s) and torch.equal(zp[:, :, :off].cpu(), z)
    assert int(words[:, :, off:].abs().sum()) == 0           # nothing written past the end


@pytest.mark.parametrize('bits,sym', [(8, True), (4, False), (2, False)])
def test_error_statistics_match_the_oracle(dev, bits, sym, tmp_path):
    """Range and L2-normalised error figures (var_q_amd/stats.py) against the same
    quantities computed from the oracle's codes on the CPU."""
    from var_q_amd.stats import CsvReport, quant_error_stats
    g = torch.Generator().manual_seed(bits)
    x = O.synth_kv((2, 3, 50, 128), 11, 'student4', 0.01, 20.0, torch.bfloat16, outlier_seed=12)
    note('quant stats', bits, sym)
    st = quant_error_stats(x.to(dev), 64, bits, sym, tag='k')
    q, s, z = O.quant_groupwise(x, 64, bits, not sym)
    deq = O.dequant_groupwise(q, s, z, 64)
    want = (torch.linalg.vector_norm((x.float() - deq).double()) / torch.linalg.vector_norm(x.double())).item()
    assert st['l2_norm_error'] == pytest.approx(want, rel=1e-6)
    assert st['max_abs_error'] == pytest.approx((x.float() - deq).abs().max().item(), rel=1e-6)
    assert st['scale_max'] == s.max().item() and st['scale_min'] == s.min().item()
    assert st['x_min'] == x.float().min().item() and st['x_max'] == x.float().max().item()
    assert st['n_groups'] == s.numel() and st['max_abs_error_in_steps'] <= 0.5 + 1e-3 or not sym
    rep = CsvReport(str(tmp_path / 'r.csv'))
    rep.add(st)
    assert float(rep.rows()[0]['l2_norm_error']) == pytest.approx(want, rel=1e-6)


@pytest.mark.parametrize('bits,group,asym,dtype', [(4, 128, True, torch.bfloat16), (8, 64, False, torch.float32),
                                                    (2, 32, True, torch.float16), (4, 16, True, torch.bfloat16)])
def test_pair_launch_equals_two_launches(dev, bits, group, asym, dtype):
    """varq_quant_pack_rows2: K and V of one step in one launch, written through a shared row
    map (a window of a larger cache, heads picked by a slot table); same bytes as two calls."""
    B, H, n, D, Lmax, start = 2, 5, 37, 128, 64, 11
    heads = [3, 0, 4]
    g = torch.Generator().manual_seed(bits * 7 + group)
    k = (torch.randn(B, H, n, D, generator=g) * 3).to(dtype).to(dev)
    v = (torch.randn(B, H, n, D, generator=g) * 3).to(dtype).to(dev)
    slot = torch.full((H,), -1, dtype=torch.int32)
    for i, h in enumerate(heads):
        slot[h] = i
    slot = slot.to(dev)
    hc, W, ng = len(heads), D * bits // 32, D // group
    rowmap = [B, H, n, hc * Lmax, Lmax, 1, start, 1]

    def bufs():
        return (torch.full((B, hc, Lmax, W), 7, dtype=torch.int32, device=dev),
                torch.full((B, hc, Lmax, ng), 7.0, device=dev), torch.full((B, hc, Lmax, ng), 7.0, device=dev) if asym else None)
    a_k, a_v, b_k, b_v = bufs(), bufs(), bufs(), bufs()
    note('quant_pack_rows2', bits, group, asym, dtype)
    ops.quant_pack_rows_into(k, group, bits, asym, 1e-12, *a_k, rowmap, slot)
    ops.quant_pack_rows_into(v, group, bits, asym, 1e-12, *a_v, rowmap, slot)
    ops.quant_pack_rows_pair_into(k, v, group, bits, asym, 1e-12, b_k, b_v, rowmap, slot)
    torch.cuda.synchronize()
    for x, y in zip(a_k + a_v, b_k + b_v):
        if x is not None:
            assert torch.equal(x, y)
    assert not torch.equal(a_k[0], a_v[0])        # the two tensors did differ


def _offset_rows(c):
    """fp32 rows of integers base .. base+255 (scale 1 for 8-bit affine codes), with bases that put
    the zero-point on either side of 2^21 and 2^22: the kernel's rounding shortcut needs the
    clamped quotient, up to 128 beyond the zero-point, inside +-2^22."""
    rows = []
    for base in (2 ** 21 - 300, 2 ** 21 - 128, 2 ** 21 - 1, 2 ** 21, 2 ** 21 + 200, 2 ** 22 - 400, 2 ** 22 - 256,
                 2 ** 22 - 130, 2 ** 22 - 128, 2 ** 22 - 1, 2 ** 22, 2 ** 22 + 300, 2 ** 23 - 256):
        for sign in (1.0, -1.0):
            k = torch.arange(c, dtype=torch.float32) * 255 // (c - 1)
            rows.append(sign * (k + float(base)) if sign > 0 else -(k + float(base)))
    return torch.stack(rows)


@pytest.mark.parametrize('bits', [8, 4, 2])
@pytest.mark.parametrize('c,group', [(128, 128), (64, 64), (64, 32)])
def test_zero_points_around_the_rounding_shortcuts_limit(dev, bits, c, group):
    note('quant_rows zero-point limit', bits, c, group)
    _check(_offset_rows(c), group, bits, True, dev)


@pytest.mark.parametrize('bits,group,asym,dtype', [(4, 128, True, torch.bfloat16), (8, 64, False, torch.float32),
                                                    (2, 32, True, torch.float16), (4, 16, True, torch.bfloat16),
                                                    (8, 8, True, torch.bfloat16)])
@pytest.mark.parametrize('n', [1, 3, 5, 37, 300])
def test_token_major_input_into_a_head_major_cache(dev, bits, group, asym, dtype, n):
    """K and V as the Infinity block holds them, [B, L, H, c], written into a [B, heads, Lmax]
    cache through a row map over (B, L, H) with a slot table over the heads
    (VAR_Q/quant.py:196-201 behind the transpose of Infinity/infinity/models/basic.py:330).
    With at least as many tokens as heads the kernel walks the tokens of one head, otherwise the
    heads of one token; either way the cache must hold what the head-major order of the same
    values gives, which in turn equals the oracle."""
    B, H, D, Lmax, start = 2, 5, 128, 320, 11
    heads = [3, 0, 4]
    g = torch.Generator().manual_seed(bits * 7 + group + n)
    k = (torch.randn(B, n, H, D, generator=g) * 3).to(dtype)
    v = (torch.randn(B, n, H, D, generator=g) * 3).to(dtype)
    slot = torch.full((H,), -1, dtype=torch.int32)
    for i, h in enumerate(heads):
        slot[h] = i
    slot = slot.to(dev)
    hc, W, ng = len(heads), D * bits // 32, D // group
    map_blhc = [B, n, H, hc * Lmax, 1, Lmax, start, 2]
    map_bhlc = [B, H, n, hc * Lmax, Lmax, 1, start, 1]

    def bufs():
        return (torch.full((B, hc, Lmax, W), 7, dtype=torch.int32, device=dev),
                torch.full((B, hc, Lmax, ng), 7.0, device=dev), torch.full((B, hc, Lmax, ng), 7.0, device=dev) if asym else None)
    a_k, a_v, b_k, b_v, c_k = bufs(), bufs(), bufs(), bufs(), bufs()
    note('quant_pack_rows token-major', bits, group, asym, dtype, n)
    ops.quant_pack_rows_pair_into(k.to(dev), v.to(dev), group, bits, asym, 1e-12, a_k, a_v, map_blhc, slot)
    ops.quant_pack_rows_into(k.to(dev), group, bits, asym, 1e-12, *c_k, map_blhc, slot)
    kt, vt = k.transpose(1, 2).contiguous(), v.transpose(1, 2).contiguous()
    ops.quant_pack_rows_pair_into(kt.to(dev), vt.to(dev), group, bits, asym, 1e-12, b_k, b_v, map_bhlc, slot)
    torch.cuda.synchronize()
    for x, y in zip(a_k + a_v + a_k, b_k + b_v + c_k):
        if x is not None:
            assert torch.equal(x, y)
    q, s, z = O.quant_groupwise(kt[:, heads], group, bits, asym)
    sl = slice(start, start + n)
    assert torch.equal(a_k[0][:, :, sl].cpu(), O.pack_last_dim(q, bits)[0])
    assert torch.equal(a_k[1][:, :, sl].cpu(), s) and (not asym or torch.equal(a_k[2][:, :, sl].cpu(), z))
    assert bool((a_k[0][:, :, :start] == 7).all()) and bool((a_k[0][:, :, start + n:] == 7).all())


def test_token_major_seeded_random_shapes(dev):
    """Forty seeded random shapes of a token-major step into a head-major cache (rows of 32 to
    256 channels, also 96: twelve octets per row, not a power of two; one to seventy tokens against one to nine heads;
    every width and dtype; with and without a slot table over the heads): the cache equals the
    oracle's codes, scales and zero-points at the step's rows and is untouched elsewhere."""
    import random
    rnd = random.Random(20240607)
    for case in range(40):
        c = rnd.choice([32, 64, 96, 128, 256])
        bits = rnd.choice([2, 4, 8])
        groups = [g for g in (8, 16, 32, 64, 128, 256) if c % g == 0 and (g // 8) & (g // 8 - 1) == 0 and (bits != 2 or g >= 16)]
        group = rnd.choice(groups)
        asym = rnd.random() < 0.6
        dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
        B, n, H = rnd.randint(1, 3), rnd.randint(1, 70), rnd.randint(1, 9)
        start = rnd.randint(0, 5)
        Lmax = start + n + rnd.randint(0, 4)
        with_slot = H > 1 and rnd.random() < 0.5
        heads = list(range(H))
        if with_slot:
            heads = rnd.sample(range(H), rnd.randint(1, H))     # (in any order: the slot table maps head -> place)
        g = torch.Generator().manual_seed(1000 + case)
        x = (torch.randn(B, n, H, c, generator=g) * rnd.choice([0.01, 1.0, 30.0])).to(dtype)
        slot = None
        if with_slot:
            slot = torch.full((H,), -1, dtype=torch.int32)
            for i, h in enumerate(heads):
                slot[h] = i
            slot = slot.to(dev)
        hc, W, ng = len(heads), c * bits // 32, c // group
        words = torch.full((B, hc, Lmax, W), 7, dtype=torch.int32, device=dev)
        scale = torch.full((B, hc, Lmax, ng), 7.0, device=dev)
        zp = torch.full((B, hc, Lmax, ng), 7.0, device=dev) if asym else None
        note('quant_pack_rows token-major random', case, (B, n, H, c), bits, group, asym, dtype, 'slot' if with_slot else 'all heads')
        ops.quant_pack_rows_into(x.to(dev), group, bits, asym, 1e-12, words, scale, zp,
                                 [B, n, H, hc * Lmax, 1, Lmax, start, 2 if with_slot else -1], slot)
        torch.cuda.synchronize()
        q, s, z = O.quant_groupwise(x.transpose(1, 2)[:, heads].contiguous(), group, bits, asym)
        sl = slice(start, start + n)
        assert torch.equal(words[:, :, sl].cpu(), O.pack_last_dim(q, bits)[0]), f'case {case}: packed words differ'
        assert torch.equal(scale[:, :, sl].cpu(), s), f'case {case}: scales differ'
        if asym:
            assert torch.equal(zp[:, :, sl].cpu(), z), f'case {case}: zero-points differ'
        assert bool((words[:, :, :start] == 7).all()) and bool((words[:, :, start + n:] == 7).all()), f'case {case}: rows outside the step written'
        assert bool((scale[:, :, :start] == 7).all()) and bool((scale[:, :, start + n:] == 7).all())

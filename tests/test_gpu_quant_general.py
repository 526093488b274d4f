"""Parity of the two-phase general quantizer (groups spanning rows: the six
grouping methods of VAR_Q/quant.py:75-95) with the CPU oracle, bit-exact."""
import pytest
import torch

import varq_oracle as O
from gpu_util import adversarial_rows, note
from var_q_amd import ops

pytestmark = pytest.mark.gpu

ALL_METHODS = list(O.METHODS)


def _check(x, dims, bits, asym, pack, dev):
    q, s, z = O.quant_reduce(x, dims, bits, asym)
    gq, gs, gz = ops.quant_pack(x.to(dev), dims, bits, asym=asym, pack=pack)
    torch.cuda.synchronize()
    assert gs.shape == s.shape and torch.equal(gs.cpu(), s), 'scale mismatch'
    if asym:
        assert torch.equal(gz.cpu(), z), 'zero-point mismatch'
    if pack:
        want, _ = O.pack_last_dim(q, bits)
        assert gq.dtype == torch.int32 and torch.equal(gq.cpu(), want), 'packed words mismatch'
    else:
        assert gq.dtype == torch.int8 and torch.equal(gq.cpu(), q), 'codes mismatch'


@pytest.mark.parametrize('fmt', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('method', ALL_METHODS)
@pytest.mark.parametrize('bits', [2, 4, 8])
def test_six_methods_symmetric(dev, fmt, method, bits):
    g = torch.Generator().manual_seed(bits)
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        for shape in [(2, 9, 3, 64), (4, 37, 5, 128), (1, 1, 2, 8)]:
            note('general', fmt, method, bits, dtype, shape)
            x = (torch.randn(*shape, generator=g) * 2).to(dtype)
            x[..., 3] *= 15
            _check(x, O.reduce_dims(method, fmt), bits, False, True, dev)


@pytest.mark.parametrize('method', ALL_METHODS)
@pytest.mark.parametrize('bits', [3, 5, 8])
def test_unpacked_codes_any_bits(dev, method, bits):
    note('general codes', method, bits)
    g = torch.Generator().manual_seed(bits)
    x = torch.randn(2, 6, 3, 16, generator=g)
    _check(x, O.reduce_dims(method, 'BHLc'), bits, False, False, dev)


@pytest.mark.parametrize('dims', [(0, 2), (0, 2, 3), (0, 1, 2, 3), (0, 3), (3,), (1, 2), (0,)])
@pytest.mark.parametrize('bits', [2, 4, 8])
def test_asymmetric_reduce_sets(dev, dims, bits):
    """Includes per-head-per-dim (0,2) and per-head (0,2,3) on BHLc."""
    note('general asym', dims, bits)
    g = torch.Generator().manual_seed(bits + len(dims))
    x = (torch.randn(3, 4, 21, 64, generator=g) * 2 + 0.7).bfloat16()
    _check(x, dims, bits, True, True, dev)


@pytest.mark.parametrize('c', [10, 24, 80, 1, 520])
def test_odd_channel_counts(dev, c):
    """Channel counts that leave a padded last word or miss the vector path."""
    g = torch.Generator().manual_seed(c)
    x = torch.randn(2, 5, 3, c, generator=g)
    for bits in (2, 4, 8):
        for method in ('G_SCALE_HEAD_DIM', 'G_TOKEN_HEAD', 'G_TENSOR'):
            note('general odd c', c, bits, method)
            _check(x, O.reduce_dims(method, 'BLHc'), bits, False, True, dev)
            _check(x.bfloat16(), O.reduce_dims(method, 'BLHc'), bits, True, True, dev)


def test_adversarial_values(dev):
    rows = adversarial_rows(64)                       # [32, 64]
    x = rows.view(2, 4, 4, 64)
    for method in ALL_METHODS:
        for bits in (2, 4, 8):
            for asym in (False, True):
                note('general adversarial', method, bits, asym)
                _check(x, O.reduce_dims(method, 'BHLc'), bits, asym, True, dev)


def test_var_d30_shapes(dev):
    """benchmark configuration 3 (batch reduced for the CPU oracle): INT2 asymmetric
    per-head-per-dim and INT8 symmetric per-channel on [B,30,680,64] bf16."""
    x = O.synth_kv((4, 30, 680, 64), seed=1003, dtype=torch.bfloat16)
    note('general c3 int2 asym per-head-per-dim')
    _check(x, (0, 2), 2, True, True, dev)
    note('general c3 int8 per-channel')
    _check(x, O.reduce_dims('G_SCALE_HEAD_DIM', 'BHLc'), 8, False, True, dev)


def test_var_d16_per_head_int8_fp32(dev):
    """benchmark configuration 1: fp32 [2,16,680,64], INT8 symmetric per-head."""
    note('general c1')
    x = O.synth_kv((2, 16, 680, 64), seed=1001)
    _check(x, (0, 2, 3), 8, False, True, dev)


def test_empty(dev):
    q, s, z = ops.quant_pack(torch.empty(2, 0, 3, 8, device=dev), (0, 1), 8)
    assert q.shape == (2, 0, 3, 2)


@pytest.mark.parametrize('mask', range(1, 16))
def test_every_reduce_set_on_tiled_shapes(dev, mask):
    """All 15 non-empty reduce sets over the four dims, on shapes that exercise the
    tiled path's cases: inner dim shorter and longer than a workgroup's row lanes,
    several chunks of partials per group, 3 and 64 column lanes."""
    dims = tuple(d for d in range(4) if (mask >> d) & 1)
    g = torch.Generator().manual_seed(100 + mask)
    for shape, dtype in [((3, 5, 70, 32), torch.bfloat16), ((2, 40, 7, 128), torch.float32),
                         ((5, 3, 33, 512), torch.bfloat16), ((2, 3, 100, 24), torch.float16),
                         ((64, 2, 300, 64), torch.bfloat16)]:
        x = (torch.randn(*shape, generator=g) * 3 + 0.25).to(dtype)
        x[..., 1] *= 9
        for bits, asym in ((8, False), (4, True)):
            note('general tiled', mask, shape, dtype, bits, asym)
            _check(x, dims, bits, asym, True, dev)


def test_all_ones_scale_significand_in_general_path(dev):
    """A group whose scale is (2 - 2^-23) * 2^e must take the exact division (see
    test_gpu_quant_rows.py::test_scale_with_all_ones_significand)."""
    import numpy as np
    s_star = np.float32((2 - 2.0 ** -23) * 0.25)
    top = None
    a = np.float32(np.float64(s_star) * 127.0)
    for cand in [a] + [np.nextafter(a, np.float32(np.inf))] * 0:
        if np.float32(cand) / np.float32(127.0) == s_star:
            top = float(cand)
    c = a
    for _ in range(16):
        if top is not None:
            break
        c = np.nextafter(c, np.float32(np.inf))
        if np.float32(c) / np.float32(127.0) == s_star:
            top = float(c)
    c = a
    for _ in range(16):
        if top is not None:
            break
        c = np.nextafter(c, np.float32(-np.inf))
        if np.float32(c) / np.float32(127.0) == s_star:
            top = float(c)
    assert top is not None
    half = np.float32(np.float64(s_star) * 0.5)
    x = torch.zeros(2, 3, 40, 64)
    x[0, 1, 5, :] = top                                            # per-channel groups of head 1: scale = s_star
    x[1, 1, 7, :] = float(np.nextafter(half, np.float32(np.inf)))  # rounds to 1 under IEEE division, 0 under the shortcut
    x[1, 1, 8, :] = float(half)
    x[0, 0, :, :] = torch.randn(40, 64, generator=torch.Generator().manual_seed(5))
    q, s, _ = O.quant_reduce(x, (0, 2), 8, False)
    assert bool(((s[0, 1, 0].view(torch.int32) & 0x7fffff) == 0x7fffff).all())
    assert int(q[1, 1, 7, 0]) == 1
    note('general all-ones scale')
    _check(x, (0, 2), 8, False, True, dev)


@pytest.mark.parametrize('token_dim', [1, 2])
@pytest.mark.parametrize('mask', [0b0101, 0b0011, 0b1111, 0b1000, 0b0111])
def test_codes_written_into_a_window_of_a_larger_buffer(dev, token_dim, mask):
    """The output map: a step lands at a token offset of a cache buffer with more room along
    the token dim, scale and zero-point in caller-provided buffers; the rest of the buffer is
    untouched and the window holds what the plain call returns.  Tiled shapes (c a multiple
    of 8) and the scalar kernels (c = 20)."""
    dims = tuple(d for d in range(4) if (mask >> d) & 1)
    g = torch.Generator().manual_seed(900 + mask + token_dim)
    for shape, bits, asym, pack in [((2, 5, 7, 64), 8, False, True), ((3, 4, 6, 128), 4, True, True),
                                    ((2, 3, 5, 20), 8, True, False), ((2, 9, 3, 32), 2, True, True)]:
        x = (torch.randn(*shape, generator=g) * 3).bfloat16().to(dev)
        want_q, want_s, want_z = ops.quant_pack(x, dims, bits, asym=asym, pack=pack)
        cap, at = shape[token_dim] + 11, 4
        big = list(want_q.shape)
        big[token_dim] = cap
        buf = torch.full(big, 0x5a if not pack else 0x5a5a5a5a, dtype=want_q.dtype, device=dev)
        s_out = torch.empty(want_s.numel(), dtype=torch.float32, device=dev)
        z_out = torch.empty(want_s.numel(), dtype=torch.float32, device=dev) if asym else None
        note('general out map', mask, shape, bits, asym, pack, token_dim)
        q, s, z = ops.quant_pack(x, dims, bits, asym=asym, pack=pack, out=buf, out_token_dim=token_dim, out_token=at,
                                 scale_out=s_out, zp_out=z_out)
        torch.cuda.synchronize()
        assert q.data_ptr() == buf.narrow(token_dim, at, shape[token_dim]).data_ptr()
        assert torch.equal(q, want_q) and torch.equal(s, want_s) and torch.equal(s_out.view(want_s.shape), want_s)
        if asym:
            assert torch.equal(z, want_z) and torch.equal(z_out.view(want_s.shape), want_z)
        fill = buf.new_full((), 0x5a if not pack else 0x5a5a5a5a)
        assert bool((buf.narrow(token_dim, 0, at) == fill).all())
        assert bool((buf.narrow(token_dim, at + shape[token_dim], cap - at - shape[token_dim]) == fill).all())


@pytest.mark.parametrize('mask', [0b0101, 0b0011, 0b1111, 0b1000, 0b0110, 0b0001])
def test_two_tensors_in_the_same_launches(dev, mask):
    """K and V of a step through `varq_quant_pack2`: the results of two separate calls, bit
    for bit, on tiled shapes (one launch set for both) and on a shape of the scalar kernels
    (c = 20: one after the other through the same workspace)."""
    dims = tuple(d for d in range(4) if (mask >> d) & 1)
    g = torch.Generator().manual_seed(1200 + mask)
    for shape, dtype, bits, asym, pack in [((2, 16, 300, 128), torch.bfloat16, 8, False, True),
                                           ((3, 40, 5, 64), torch.float32, 4, True, True),
                                           ((2, 3, 50, 20), torch.bfloat16, 8, True, False),
                                           ((64, 2, 33, 32), torch.float16, 2, True, True)]:
        x0 = (torch.randn(*shape, generator=g) * 2).to(dtype).to(dev)
        x1 = (torch.randn(*shape, generator=g) * 5 + 1).to(dtype).to(dev)
        note('general pair', mask, shape, dtype, bits, asym, pack)
        a, b = ops.quant_pack_pair(x0, x1, dims, bits, asym=asym, pack=pack)
        torch.cuda.synchronize()
        for got, x in ((a, x0), (b, x1)):
            want = ops.quant_pack(x, dims, bits, asym=asym, pack=pack)
            assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
            assert (got[2] is None) == (want[2] is None) and (got[2] is None or torch.equal(got[2], want[2]))


def test_empty_pair_and_empty_dequant(dev):
    """Tensors without rows reach the library as null pointers: nothing to do, no error."""
    note('general: empty pair, empty dequant')
    x = torch.empty(2, 3, 0, 64, dtype=torch.bfloat16, device=dev)
    (q0, s0, z0), (q1, s1, z1) = ops.quant_pack_pair(x, x, (0, 2), 4, asym=True)
    assert q0.shape == (2, 3, 0, 8) and q1.shape == (2, 3, 0, 8) and s0.shape == (1, 3, 1, 64)
    w = torch.empty(2, 3, 0, 8, dtype=torch.int32, device=dev)
    s = torch.empty(2, 3, 0, 1, device=dev)
    assert ops.dequant(w, s, s, 64, 4, torch.bfloat16).shape == (2, 3, 0, 64)
    torch.cuda.synchronize()

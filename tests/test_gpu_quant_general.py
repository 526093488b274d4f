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
    """BASELINE config 3 (batch reduced for the CPU oracle): INT2 asymmetric
    per-head-per-dim and INT8 symmetric per-channel on [B,30,680,64] bf16."""
    x = O.synth_kv((4, 30, 680, 64), seed=1003, dtype=torch.bfloat16)
    note('general c3 int2 asym per-head-per-dim')
    _check(x, (0, 2), 2, True, True, dev)
    note('general c3 int8 per-channel')
    _check(x, O.reduce_dims('G_SCALE_HEAD_DIM', 'BHLc'), 8, False, True, dev)


def test_var_d16_per_head_int8_fp32(dev):
    """BASELINE config 1: fp32 [2,16,680,64], INT8 symmetric per-head."""
    note('general c1')
    x = O.synth_kv((2, 16, 680, 64), seed=1001)
    _check(x, (0, 2, 3), 8, False, True, dev)


def test_empty(dev):
    q, s, z = ops.quant_pack(torch.empty(2, 0, 3, 8, device=dev), (0, 1), 8)
    assert q.shape == (2, 0, 3, 2)

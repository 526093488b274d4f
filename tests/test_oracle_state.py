"""Pins the oracle's cache state machine (VAR_Q/quant.py:140-230) through
invariants that follow from reading the reference: cached lengths, the
"append == concatenation of independently quantized steps" identity, the
replace semantics of G_HEAD_DIM, and the G_TENSOR duplication quirk."""
import pytest
import torch

import varq_oracle as O

STEPS = (1, 4, 9)


def _steps(fmt, seed=0, H=3, c=8, B=2):
    g = torch.Generator().manual_seed(seed)
    out = []
    for n in STEPS:
        x = torch.randn(B, n, H, c, generator=g)
        out.append(x if fmt == 'BLHc' else x.permute(0, 2, 1, 3).contiguous())
    return out


@pytest.mark.parametrize('fmt', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('method', ['G_SCALE_HEAD_DIM', 'G_SCALE', 'G_TOKEN', 'G_TOKEN_HEAD'])
@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('pack', [False, True])
def test_append_methods_equal_concat_of_independent_steps(fmt, method, bits, pack):
    q = O.OracleVARQ(bits, fmt, method, pack_to_int32=pack)
    d = q.dim_cat
    xs = _steps(fmt)
    outs = []
    for x in xs:
        y = q.use_var_q(x)
        s = O.scale_sym(x, q.dim_map[method], bits)
        outs.append(O.dequant_sym(O.codes_sym(x, s, bits), s))
        assert y.dtype == torch.float32
        assert torch.equal(y, torch.cat(outs, dim=d))
    total = sum(STEPS)
    assert q.cached_item.size(d) == total and q.cached_scale.size(d) == total
    if pack:
        assert q.cached_item.dtype == torch.int32 and q.cached_item.shape[-1] == -(-8 // (32 // bits))
        assert q._pack_meta == {'orig_c': 8, 'vals_per_word': 32 // bits, 'pad_len': (-8) % (32 // bits), 'bits': bits}
    else:
        assert q.cached_item.dtype == torch.int8


@pytest.mark.parametrize('fmt', ['BLHc', 'BHLc'])
def test_head_dim_requantizes_history_and_replaces(fmt):
    q = O.OracleVARQ(8, fmt, 'G_HEAD_DIM', pack_to_int32=False)
    d = q.dim_cat
    xs = _steps(fmt, seed=1)
    y0 = q.use_var_q(xs[0])
    y1 = q.use_var_q(xs[1])
    # second step quantizes cat(previous output, new item) as one tensor
    cat = torch.cat([y0, xs[1]], dim=d)
    s = O.scale_sym(cat, q.dim_map['G_HEAD_DIM'], 8)
    assert torch.equal(y1, O.dequant_sym(O.codes_sym(cat, s, 8), s))
    assert q.cached_item.size(d) == STEPS[0] + STEPS[1]
    # scale is kept as a stride-0 expand along L
    assert q.cached_scale.size(d) == STEPS[0] + STEPS[1] and q.cached_scale.stride(d) == 0


def test_g_tensor_duplicates_tokens_from_second_step():
    q = O.OracleVARQ(8, 'BLHc', 'G_TENSOR', pack_to_int32=False)
    xs = _steps('BLHc', seed=2)
    assert q.use_var_q(xs[0]).size(1) == 1
    assert q.use_var_q(xs[1]).size(1) == 1 + (1 + 4)          # old cache + re-quantized concatenation
    assert q.use_var_q(xs[2]).size(1) == 6 + (6 + 9)


def test_first_cached_scale_is_expand_view():
    q = O.OracleVARQ(8, 'BHLc', 'G_SCALE_HEAD_DIM', pack_to_int32=False)
    x = torch.randn(2, 3, 4, 8)
    q.quant(x); q.cache()
    assert q.cached_scale.shape == (1, 3, 4, 8) and q.cached_scale.stride(2) == 0
    assert q.scale.shape == (1, 3, 1, 8)


def test_constructor_contract():
    with pytest.raises(AssertionError):
        O.OracleVARQ(8, 'HBLc')
    with pytest.raises(AssertionError):
        O.OracleVARQ(8, 'BLHc', 'G_NOPE')
    with pytest.raises(AssertionError):
        O.OracleVARQ(1)
    with pytest.raises(AssertionError):
        O.OracleVARQ(9)
    q = O.OracleVARQ(4, 'BHLc')
    assert (q.bound_min, q.bound_max, q.dim_cat) == (-8, 7, 2)
    assert O.OracleVARQ(2).bound_min == -2 and O.OracleVARQ(8).bound_max == 127
    # bits that cannot be packed fail at pack time, not at construction
    q3 = O.OracleVARQ(3, 'BLHc', 'G_TOKEN', pack_to_int32=True)
    with pytest.raises(AssertionError):
        q3.quant(torch.randn(1, 2, 2, 8))

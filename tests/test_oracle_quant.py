"""Pins the oracle's quantizer arithmetic (VAR_Q/quant.py:112-124) by closed
forms and special cases, and its asymmetric / group-wise extensions by
invariants.  Nothing here retypes the oracle's formula with the same library
calls: the cross-checks use numpy scalar arithmetic or facts that hold for any
correct implementation."""
import numpy as np
import pytest
import torch

import varq_oracle as O


@pytest.mark.parametrize('bits', [2, 3, 4, 8])
def test_argmax_maps_to_qmax_and_codes_in_range(bits):
    g = torch.Generator().manual_seed(bits)
    x = torch.randn(2, 5, 3, 16, generator=g)
    qmin, qmax = O.qrange(bits)
    for dims in [(0, 1), (0, 3), (0, 1, 2, 3), (0, 2, 3)]:
        s = O.scale_sym(x, dims, bits)
        q = O.codes_sym(x, s, bits)
        assert q.dtype == torch.int8 and int(q.min()) >= qmin and int(q.max()) <= qmax
        # wherever |x| attains the group max, the code is +-qmax
        amax = x.abs().amax(dim=dims, keepdim=True)
        hit = x.abs() == amax
        assert torch.equal(q[hit].abs().to(torch.int64), torch.full((int(hit.sum()),), qmax))
        # unclamped error bound: |x - deq| <= scale/2 (+1 ulp)
        err = (x - O.dequant_sym(q, s)).abs()
        assert bool((err <= s * 0.5000001).all())


def test_scale_shapes_per_method():
    x = torch.randn(2, 6, 3, 8)   # BLHc: B=2, L=6, H=3, c=8
    want = {'G_TENSOR': (1, 1, 1, 1), 'G_SCALE': (1, 1, 1, 1), 'G_SCALE_HEAD_DIM': (1, 1, 3, 8),
            'G_HEAD_DIM': (1, 1, 3, 8), 'G_TOKEN': (1, 6, 1, 1), 'G_TOKEN_HEAD': (1, 6, 3, 1)}
    for m, shp in want.items():
        assert tuple(O.scale_sym(x, O.reduce_dims(m, 'BLHc'), 8).shape) == shp
    y = x.permute(0, 2, 1, 3).contiguous()  # BHLc
    want = {'G_TENSOR': (1, 1, 1, 1), 'G_SCALE': (1, 1, 1, 1), 'G_SCALE_HEAD_DIM': (1, 3, 1, 8),
            'G_HEAD_DIM': (1, 3, 1, 8), 'G_TOKEN': (1, 1, 6, 1), 'G_TOKEN_HEAD': (1, 3, 6, 1)}
    for m, shp in want.items():
        assert tuple(O.scale_sym(y, O.reduce_dims(m, 'BHLc'), 8).shape) == shp
    # the two layouts describe the same groups
    for m in O.METHODS:
        a = O.scale_sym(x, O.reduce_dims(m, 'BLHc'), 4)
        b = O.scale_sym(y, O.reduce_dims(m, 'BHLc'), 4)
        assert torch.equal(a.permute(0, 2, 1, 3), b)


def test_half_to_even_ties_and_true_division():
    # scale = 1 exactly (max_abs = qmax), values at exact .5 ties
    x = torch.tensor([[0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, 127.0]])
    s = O.scale_sym(x, (0, 1), 8)
    assert float(s) == 1.0
    assert O.codes_sym(x, s, 8).tolist() == [[0, 2, 2, 0, -2, -2, 4, 127]]
    # division by the scale is a true fp32 division, not a multiply by a rounded
    # reciprocal: find inputs where the two differ and check which one it is.
    rng = np.random.default_rng(0)
    sc = np.float32(0.3137)
    ks = np.arange(-120, 120, dtype=np.float32) + np.float32(0.5)
    near = (ks * sc).astype(np.float32)            # inputs whose quotient sits on a .5 tie, +-1 ulp
    xs = np.concatenate([near, np.nextafter(near, np.float32(np.inf)), np.nextafter(near, np.float32(-np.inf))])
    exact = np.rint(xs / sc)                       # numpy fp32 division, half-to-even
    recip = np.rint(xs * (np.float32(1) / sc))
    assert (exact != recip).any(), 'need a discriminating input'
    got = torch.round(torch.from_numpy(xs) / torch.tensor(sc)).numpy()
    assert np.array_equal(got, exact)
    q = O.codes_sym(torch.from_numpy(xs), torch.tensor(sc), 8).numpy()
    assert np.array_equal(q, np.clip(exact, -128, 127).astype(np.int8))
    # scale = amax / qmax is a true division as well
    big = torch.from_numpy(rng.standard_normal((4000, 4)).astype(np.float32))
    s = O.scale_sym(big, (1,), 8).numpy().ravel()
    assert np.array_equal(s, np.abs(big.numpy()).max(1) / np.float32(127.0))


def test_all_zero_group_and_two_bit():
    x = torch.zeros(2, 4, 2, 8)
    s = O.scale_sym(x, (0, 1), 4, eps=1e-12)
    assert bool((s == np.float32(1e-12)).all())
    assert int(O.codes_sym(x, s, 4).abs().max()) == 0
    # 2-bit symmetric: scale = max_abs, codes in {-1,0,1}
    y = torch.randn(3, 64, generator=torch.Generator().manual_seed(1))
    s2 = O.scale_sym(y, (1,), 2)
    assert torch.equal(s2.squeeze(1), y.abs().amax(1))
    q2 = O.codes_sym(y, s2, 2)
    assert set(q2.unique().tolist()) <= {-1, 0, 1}


def test_low_precision_inputs_are_widened_first():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 8, 4, 16, generator=g)
    for dt in (torch.bfloat16, torch.float16):
        xl = x.to(dt)
        s = O.scale_sym(xl, (0, 1), 8)
        assert s.dtype == torch.float32
        assert torch.equal(s, O.scale_sym(xl.float(), (0, 1), 8))
        assert torch.equal(O.codes_sym(xl, s, 8), O.codes_sym(xl.float(), s, 8))


@pytest.mark.parametrize('bits', [2, 4, 8])
def test_asym_invariants(bits):
    g = torch.Generator().manual_seed(10 + bits)
    x = torch.randn(4, 32, generator=g) * 3 + 1.0
    qmin, qmax = O.qrange(bits)
    s, z = O.asym_params(x, (1,), bits)
    q = O.codes_asym(x, s, z, bits)
    assert int(q.min()) >= qmin and int(q.max()) <= qmax
    mn, mx = x.amin(1, keepdim=True), x.amax(1, keepdim=True)
    assert bool((q[x == mn.expand_as(x)] == qmin).all())            # min -> qmin
    top = q[x == mx.expand_as(x)]
    assert bool(((top == qmax) | (top == qmax - 1)).all())           # max -> qmax or qmax-1
    assert bool((z == torch.round(z)).all())                         # integer valued
    err = (x - O.dequant_asym(q, s, z)).abs()
    assert bool((err <= s * 1.0000005).all())                        # one step at most (half + rounding of zp)
    assert np.allclose(s.numpy(), ((mx - mn) / (2 ** bits - 1)).numpy(), rtol=0, atol=0)


def test_asym_constant_group_and_offset_data():
    x = torch.full((2, 16), 3.0)
    s, z = O.asym_params(x, (1,), 4)
    assert bool((s == np.float32(1e-12)).all())
    q = O.codes_asym(x, s, z, 4)
    deq = O.dequant_asym(q, s, z)
    assert torch.allclose(deq, x, rtol=1e-6)
    # data far from zero: zero-point is large, codes still span the range
    y = torch.linspace(1000.0, 1001.5, 16).view(1, 16)
    s, z = O.asym_params(y, (1,), 4)
    q = O.codes_asym(y, s, z, 4)
    assert int(q.min()) == -8 and int(q.max()) in (6, 7)
    assert float((y - O.dequant_asym(q, s, z)).abs().max()) <= float(s) * 1.01


@pytest.mark.parametrize('asym', [False, True])
@pytest.mark.parametrize('group', [8, 32, 64])
def test_groupwise_equals_independent_rows(asym, group):
    """Group-wise along D == quantizing every g-channel slice on its own."""
    g = torch.Generator().manual_seed(group)
    x = torch.randn(2, 3, 5, 64, generator=g)
    q, s, z = O.quant_groupwise(x, group, 4, asym)
    for idx in [(0, 0, 0), (1, 2, 4), (0, 1, 3)]:
        for seg in range(64 // group):
            sl = x[idx][seg * group:(seg + 1) * group].view(1, group)
            qs, ss, zs = O.quant_reduce(sl, (1,), 4, asym)
            assert torch.equal(q[idx][seg * group:(seg + 1) * group], qs.view(-1))
            assert float(s[idx][seg]) == float(ss)
            if asym:
                assert float(z[idx][seg]) == float(zs)
    deq = O.dequant_groupwise(q, s, z, group)
    assert float((deq - x).abs().max()) <= float(s.max()) * (1.01 if asym else 0.51)


def test_numpy_scalar_restatement_small():
    """An element-by-element numpy float32 loop (different code path, different
    library) reproduces codes/scale/zp on a tiny tensor for both quantizers."""
    rng = np.random.default_rng(7)
    x = rng.standard_normal((3, 8)).astype(np.float32) * 4
    for bits in (2, 4, 8):
        qmin, qmax = O.qrange(bits)
        for asym in (False, True):
            q, s, z = O.quant_reduce(torch.from_numpy(x), (1,), bits, asym)
            for r in range(3):
                row = x[r]
                if asym:
                    mn, mx = row.min(), row.max()
                    sc = max(np.float32((mx - mn) / np.float32(2 ** bits - 1)), np.float32(1e-12))
                    zp = np.float32(qmin) - np.rint(np.float32(mn / sc))
                    codes = np.clip(np.rint(row / sc) + zp, qmin, qmax)
                    assert float(z[r]) == float(zp)
                else:
                    sc = max(np.float32(np.abs(row).max() / np.float32(qmax)), np.float32(1e-12))
                    codes = np.clip(np.rint(row / sc), qmin, qmax)
                assert float(s[r]) == float(sc)
                assert np.array_equal(q[r].numpy(), codes.astype(np.int8))

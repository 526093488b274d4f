"""Host-side checks of the self-attention hook modules (var_q_amd/hooks.py) on
CPU tensors, with the CPU oracle quantizer injected in place of the HIP one."""
import math

import pytest
import torch

import varq_oracle as O
from var_q_amd import hooks


@pytest.fixture(autouse=True)
def _inference_mode():
    with torch.no_grad():
        yield


def test_rope2d_tables_closed_form():
    hw = [(1, 1), (2, 2), (3, 5), (8, 8)]
    D = 32
    cos, sin = hooks.rope2d_tables(D, hw, normalized_by_hw=2)
    assert cos.shape == (sum(h * w for h, w in hw), D // 2) and sin.shape == cos.shape
    half = D // 2
    theta = [10000.0 ** (-(2 * j) / half) for j in range(half // 2)]
    uh, uw = hw[-1]
    start = 0
    for h, w in hw:
        for y in range(h):
            for x in range(w):
                yy, xx = round(y * uh / h), round(x * uw / w)
                t = start + y * w + x
                for j in range(half // 2):
                    assert cos[t, j].item() == pytest.approx(math.cos(yy * theta[j]), abs=1e-6)
                    assert sin[t, half // 2 + j].item() == pytest.approx(math.sin(xx * theta[j]), abs=1e-6)
        start += h * w
    # plain grid coordinates
    cos0, _ = hooks.rope2d_tables(D, hw, normalized_by_hw=0)
    assert cos0[1 + 4 + 1 * 5 + 2, 0].item() == pytest.approx(math.cos(1.0), abs=1e-6)   # scale (3,5), y=1
    with pytest.raises(ValueError):
        hooks.rope2d_tables(D, hw, normalized_by_hw=1)


@pytest.mark.parametrize('layout', ['BLHc', 'BHLc'])
def test_apply_rope2d_is_a_pairwise_rotation(layout):
    hw = [(2, 2), (4, 4)]
    D, H, B = 16, 3, 2
    cos, sin = hooks.rope2d_tables(D, hw)
    g = torch.Generator().manual_seed(0)
    L, start = 16, 4
    x = torch.randn(B, L, H, D, generator=g) if layout == 'BLHc' else torch.randn(B, H, L, D, generator=g)
    y = hooks.apply_rope2d(x, cos, sin, start, 1 if layout == 'BLHc' else 2)
    xc = torch.view_as_complex(x.reshape(*x.shape[:-1], -1, 2).contiguous())
    rot = torch.complex(cos[start:start + L], sin[start:start + L])
    rot = rot[None, :, None, :] if layout == 'BLHc' else rot[None, None, :, :]
    want = torch.view_as_real(xc * rot).reshape(x.shape)
    assert torch.allclose(y, want, atol=1e-6)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-5)      # rotations keep the norm


def test_fused_backend_needs_row_local_quantizer():
    with pytest.raises(AssertionError):
        hooks.VarSelfAttention(0, 64, 2, enable_quantization=True, fused=True, quant_method='G_SCALE_HEAD_DIM')


@pytest.mark.parametrize('layout', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('method', ['G_SCALE_HEAD_DIM', 'G_TOKEN_HEAD', 'G_HEAD_DIM'])
def test_var_module_with_oracle_quantizer_tracks_the_unquantized_cache(layout, method):
    """8-bit quantized caching must stay close to the plain concatenated cache, and the
    quantizer must have seen every step (cache length = tokens so far)."""
    torch.manual_seed(1)
    C, H = 64, 4
    kw = dict(embed_dim=C, num_heads=H, layout=layout, max_tokens=30)
    ref = hooks.VarSelfAttention(0, **kw)
    qz = hooks.VarSelfAttention(0, q_bits=8, quant_method=method, enable_quantization=True,
                                quantizer_factory=O.OracleVARQ, **kw)
    qz.load_state_dict(ref.state_dict())
    ref.kv_caching(True)
    qz.kv_caching(True)
    seen = 0
    for n in (1, 4, 9, 16):
        x = torch.randn(2, n, C)
        a, b = ref(x), qz(x)
        seen += n
        assert a.shape == b.shape == (2, n, C)
        assert qz.k_quant.cached_item.size(1 if layout == 'BLHc' else 2) == seen
        assert (a - b).abs().max().item() < 0.05 * a.abs().max().item() + 1e-3
    qz.kv_caching(False)
    assert qz.k_quant is None and not qz.caching


def test_infinity_module_rope_offsets_and_cache():
    torch.manual_seed(2)
    C, H = 128, 4          # head_dim 32
    hw = [(1, 1), (2, 2), (4, 4)]
    rope = hooks.rope2d_tables(C // H, hw)
    m = hooks.InfinitySelfAttention(C, H, layout='BHLc', q_bits=8, quant_method='G_SCALE_HEAD_DIM',
                                    enable_quantization=True, max_tokens=21, quantizer_factory=O.OracleVARQ)
    plain = hooks.InfinitySelfAttention(C, H, layout='BHLc', max_tokens=21)
    plain.load_state_dict(m.state_dict())
    m.kv_caching(True)
    plain.kv_caching(True)
    start = 0
    for h, w in hw:
        x = torch.randn(2, h * w, C)
        a = plain(x, rope=rope, token_start=start)
        b = m(x, rope=rope, token_start=start)
        start += h * w
        assert (a - b).abs().max().item() < 0.05 * a.abs().max().item() + 1e-3
    assert plain.cached_k.shape == (2, H, 21, C // H)
    # the cached keys are unit vectors: normalisation and rotation both preserve that
    assert torch.allclose(plain.cached_k.norm(dim=-1), torch.ones(2, H, 21), atol=1e-5)


def test_oracle_prepare_qkv_follows_the_reference_expressions():
    """The oracle of the fused producer fixes a summation order for the norm; against
    torch's own F.normalize / scale / rotation (the reference's expressions,
    Infinity basic.py:316-330 and :103-123) it may differ by rounding only."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(8)
    B, L, H, c = 2, 9, 3, 64
    qkv = torch.randn(B, L, 3, H, c, generator=g)
    mul = torch.rand(H, generator=g) * 4 + 1
    rope = hooks.rope2d_tables(c, [(2, 2), (3, 3)])
    q, k, v = O.prepare_qkv(qkv, mul, True, 1e-12, rope, 4)
    qr, kr, vr = (qkv[:, :, t].permute(0, 2, 1, 3) for t in range(3))
    qn = F.normalize(qr, dim=-1, eps=1e-12).mul(mul.view(1, H, 1, 1))
    kn = F.normalize(kr, dim=-1, eps=1e-12)
    qn, kn = hooks.apply_rope2d(qn, rope[0], rope[1], 4, 2), hooks.apply_rope2d(kn, rope[0], rope[1], 4, 2)
    assert torch.allclose(k, kn, atol=2e-7, rtol=1e-6)
    assert torch.allclose(q.float(), qn, atol=0, rtol=2 ** -7)          # bf16 result
    assert torch.equal(v, vr)
    # without normalisation and rotation the data passes through
    q2, k2, _ = O.prepare_qkv(qkv.bfloat16())
    assert torch.equal(k2, kr.bfloat16().float()) and torch.equal(q2, qr.bfloat16())

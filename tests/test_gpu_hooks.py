"""Self-attention hook modules on the GPU: the drop-in (unfused) backend against
the same module on the CPU with the oracle quantizer, and the fused backend
(packed cache + fused attention) A/B against the unfused one.

Tolerances: the fused and unfused backends quantize with the same kernels, so
their caches must dequantize to identical values; their outputs differ by the
attention arithmetic only (bf16 SDPA on dequantized K/V vs exact codes), for
which the bound is max-abs 2e-2 on unit-range attention outputs scaled by the
output range, cosine >= 0.9995."""
import pytest
import torch

import varq_oracle as O
from gpu_util import note
from var_q_amd import VAR_Q, hooks

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _inference_mode():
    with torch.no_grad():
        yield


def _cos(a, b):
    return float(torch.nn.functional.cosine_similarity(a.double().flatten(), b.double().flatten(), dim=0))


@pytest.mark.parametrize('layout', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('method,bits', [('G_SCALE_HEAD_DIM', 8), ('G_TOKEN_HEAD', 4), ('G_HEAD_DIM', 8)])
def test_var_dropin_matches_cpu_oracle_module(dev, layout, method, bits):
    torch.manual_seed(3)
    C, H = 256, 4
    kw = dict(embed_dim=C, num_heads=H, layout=layout, q_bits=bits, quant_method=method, enable_quantization=True,
              max_tokens=30)
    cpu = hooks.VarSelfAttention(0, quantizer_factory=O.OracleVARQ, **kw)
    gpu = hooks.VarSelfAttention(0, **kw).to(dev)
    gpu.load_state_dict(cpu.state_dict())
    cpu.kv_caching(True)
    gpu.kv_caching(True)
    for n in (1, 4, 9, 16):
        note('hooks var dropin', layout, method, bits, n)
        x = torch.randn(2, n, C)
        a, b = cpu(x), gpu(x.to(dev)).cpu()
        # the two differ by fp32 GEMM summation order, which can move a code by one step
        step = a.abs().max().item() / (2 ** (bits - 1))
        assert (a - b).abs().max().item() <= 2 * step + 1e-3, (n, (a - b).abs().max().item(), step)
        assert _cos(a, b) > (0.999 if bits == 8 else 0.99)


@pytest.mark.parametrize('layout', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('bits,sym', [(4, False), (8, True), (2, False)])
def test_var_fused_vs_unfused(dev, layout, bits, sym):
    torch.manual_seed(4)
    C, H = 512, 8        # head_dim 64 as in VAR
    pn = (1, 2, 3, 4, 5, 6, 8, 10, 13, 16)
    kw = dict(embed_dim=C, num_heads=H, layout=layout, q_bits=bits, quant_method='G_GROUP', group_size=64,
              symmetric=sym, enable_quantization=True, max_tokens=680)
    a_mod = hooks.VarSelfAttention(0, fused=False, **kw).to(dev).to(torch.bfloat16)
    b_mod = hooks.VarSelfAttention(0, fused=True, **kw).to(dev).to(torch.bfloat16)
    b_mod.load_state_dict(a_mod.state_dict())
    a_mod.kv_caching(True)
    b_mod.kv_caching(True)
    for p in pn:
        note('hooks var fused', layout, bits, sym, p)
        x = torch.randn(4, p * p, C, device=dev, dtype=torch.bfloat16)
        a, b = a_mod(x).float(), b_mod(x).float()
        rng = a.abs().max().item()
        assert (a - b).abs().max().item() <= 2e-2 * max(rng, 1.0), (p, (a - b).abs().max().item(), rng)
        assert _cos(a, b) >= 0.9995
    # both backends hold the same quantized cache
    ka = a_mod.k_quant.dequant_all()
    ka = ka if layout == 'BHLc' else ka.transpose(1, 2)
    assert torch.equal(ka.contiguous(), b_mod.packed_cache.dequant('k'))
    va = a_mod.v_quant.dequant_all()
    va = va if layout == 'BHLc' else va.transpose(1, 2)
    assert torch.equal(va.contiguous(), b_mod.packed_cache.dequant('v'))


def test_infinity_fused_vs_unfused_with_rope(dev):
    torch.manual_seed(5)
    C, H = 1024, 8       # head_dim 128 as in Infinity-2B
    hw = [(p, p) for p in (1, 2, 4, 6, 8, 12, 16, 20)]
    total = sum(h * w for h, w in hw)
    rope = hooks.rope2d_tables(C // H, hw)
    kw = dict(embed_dim=C, num_heads=H, layout='BHLc', q_bits=4, quant_method='G_GROUP', group_size=128,
              symmetric=False, enable_quantization=True, max_tokens=total)
    a_mod = hooks.InfinitySelfAttention(fused=False, **kw).to(dev).to(torch.bfloat16)
    b_mod = hooks.InfinitySelfAttention(fused=True, **kw).to(dev).to(torch.bfloat16)
    b_mod.load_state_dict(a_mod.state_dict())
    a_mod.kv_caching(True)
    b_mod.kv_caching(True)
    start = 0
    for h, w in hw:
        note('hooks infinity fused', h, w)
        x = torch.randn(2, h * w, C, device=dev, dtype=torch.bfloat16)
        a = a_mod(x, rope=rope, token_start=start).float()
        b = b_mod(x, rope=rope, token_start=start).float()
        start += h * w
        rng = a.abs().max().item()
        assert (a - b).abs().max().item() <= 2e-2 * max(rng, 1.0), ((h, w), (a - b).abs().max().item(), rng)
        assert _cos(a, b) >= 0.9995
    assert torch.equal(a_mod.k_quant.dequant_all(), b_mod.packed_cache.dequant('k'))


def test_unquantized_cache_path_matches_full_sequence_attention(dev):
    """Caching without quantization equals one full-sequence call under the
    block-causal mask of VAR/models/var.py:110-114."""
    torch.manual_seed(6)
    C, H = 128, 2
    pn = (1, 2, 3)
    m = hooks.VarSelfAttention(0, C, H, layout='BHLc', max_tokens=14).to(dev)
    xs = [torch.randn(1, p * p, C, device=dev) for p in pn]
    m.kv_caching(True)
    steps = torch.cat([m(x) for x in xs], dim=1)
    m.kv_caching(False)
    L = sum(p * p for p in pn)
    bias = O.block_causal_bias(pn).to(dev).view(1, 1, L, L)
    full = m(torch.cat(xs, dim=1), attn_bias=bias)
    assert torch.allclose(steps, full, atol=2e-5)


def test_infinity_fused_producer_vs_unfused(dev):
    """The one-kernel producer (normalise + scale + rotate + quantize into the cache) inside
    the module: same outputs as the unfused drop-in within the attention tolerance, and a
    cache that dequantizes to the unfused one within one quantization step (torch's own
    normalisation on the GPU rounds differently, so a code can move by one)."""
    torch.manual_seed(7)
    C, H = 1024, 8
    hw = [(p, p) for p in (1, 2, 4, 6, 8, 12)]
    total = sum(h * w for h, w in hw)
    rope = hooks.rope2d_tables(C // H, hw)
    kw = dict(embed_dim=C, num_heads=H, layout='BHLc', q_bits=4, quant_method='G_GROUP', group_size=128,
              symmetric=False, enable_quantization=True, max_tokens=total)
    a_mod = hooks.InfinitySelfAttention(fused=False, **kw).to(dev).to(torch.bfloat16)
    b_mod = hooks.InfinitySelfAttention(fused=True, fused_producer=True, **kw).to(dev).to(torch.bfloat16)
    b_mod.load_state_dict(a_mod.state_dict())
    a_mod.kv_caching(True)
    b_mod.kv_caching(True)
    start = 0
    for h, w in hw:
        note('hooks infinity fused producer', h, w)
        x = torch.randn(2, h * w, C, device=dev, dtype=torch.bfloat16)
        a = a_mod(x, rope=rope, token_start=start).float()
        b = b_mod(x, rope=rope, token_start=start).float()
        start += h * w
        rng = a.abs().max().item()
        assert (a - b).abs().max().item() <= 2e-2 * max(rng, 1.0), ((h, w), (a - b).abs().max().item(), rng)
        assert _cos(a, b) >= 0.9995
    ka, kb = a_mod.k_quant.dequant_all(), b_mod.packed_cache.dequant('k')
    step = a_mod.k_quant.cached_scale.max().item()
    assert (ka - kb).abs().max().item() <= 1.01 * step
    assert (ka != kb).float().mean().item() < 0.02


@pytest.mark.parametrize('layout', ['BLHc', 'BHLc'])
def test_var_fused_producer_vs_unfused(dev, layout):
    torch.manual_seed(8)
    C, H = 512, 8
    kw = dict(embed_dim=C, num_heads=H, layout=layout, q_bits=8, quant_method='G_GROUP', group_size=64,
              symmetric=True, enable_quantization=True, max_tokens=100)
    a_mod = hooks.VarSelfAttention(0, fused=False, **kw).to(dev).to(torch.bfloat16)
    b_mod = hooks.VarSelfAttention(0, fused=True, fused_producer=True, **kw).to(dev).to(torch.bfloat16)
    b_mod.load_state_dict(a_mod.state_dict())
    a_mod.kv_caching(True)
    b_mod.kv_caching(True)
    for p in (1, 2, 3, 4, 5, 6):
        note('hooks var fused producer', layout, p)
        x = torch.randn(4, p * p, C, device=dev, dtype=torch.bfloat16)
        a, b = a_mod(x).float(), b_mod(x).float()
        rng = a.abs().max().item()
        assert (a - b).abs().max().item() <= 2e-2 * max(rng, 1.0)
        assert _cos(a, b) >= 0.9995


@pytest.mark.parametrize('method,bits,sym', [('G_SCALE_HEAD_DIM', 8, True), ('G_HEAD_DIM', 8, True), ('G_TENSOR', 8, True),
                                             ('G_SCALE', 8, True), ('G_TOKEN', 8, True), ('G_TOKEN_HEAD', 4, True),
                                             ('G_SCALE_HEAD_DIM', 4, False), ('G_HEAD', 8, True)])
@pytest.mark.parametrize('layout', ['BHLc', 'BLHc'])
def test_quantizer_backend_vs_dropin(dev, method, bits, sym, layout):
    """fused='quantizer': the reference's own rules (quantizer + per-step cache as in the
    drop-in) with the attention reading the packed caches, A/B against the drop-in that
    dequantizes the whole cache and calls SDPA.  Both hold the same caches; the outputs
    differ by the attention arithmetic only.  BLHc is the layout of VAR-VAR_Q-8.json and of
    the reference's flash-attention call, BHLc that of its SDPA call."""
    torch.manual_seed(6)
    C, H = 512, 8
    pn = (1, 2, 3, 4, 5, 6, 8, 10, 13, 16)
    kw = dict(embed_dim=C, num_heads=H, layout=layout, q_bits=bits, quant_method=method, symmetric=sym,
              enable_quantization=True, max_tokens=680)
    a_mod = hooks.VarSelfAttention(0, fused=False, **kw).to(dev).to(torch.bfloat16)
    b_mod = hooks.VarSelfAttention(0, fused='quantizer', **kw).to(dev).to(torch.bfloat16)
    b_mod.load_state_dict(a_mod.state_dict())
    a_mod.kv_caching(True)
    b_mod.kv_caching(True)
    for p in pn:
        note('hooks quantizer backend', method, bits, sym, layout, p)
        x = torch.randn(2, p * p, C, device=dev, dtype=torch.bfloat16)
        a, b = a_mod(x).float(), b_mod(x).float()
        rng = a.abs().max().item()
        assert (a - b).abs().max().item() <= 2e-2 * max(rng, 1.0), (p, (a - b).abs().max().item(), rng)
        assert _cos(a, b) >= 0.9995
    assert torch.equal(a_mod.k_quant.dequant_all(), b_mod.k_quant.dequant_all())
    assert torch.equal(a_mod.v_quant.dequant_all(), b_mod.v_quant.dequant_all())


def test_quantizer_backend_infinity_shipped_rule(dev):
    """The Infinity hook with the shipped rule (G_SCALE_HEAD_DIM, 8 bits, BHLc,
    Infinity-VAR_Q-8.json) over the first scales of its schedule, head dim 128."""
    torch.manual_seed(7)
    C, H = 512, 4
    pn = (1, 2, 4, 6, 8, 12, 16)
    kw = dict(embed_dim=C, num_heads=H, layout='BHLc', q_bits=8, quant_method='G_SCALE_HEAD_DIM',
              enable_quantization=True, max_tokens=sum(p * p for p in pn))
    a_mod = hooks.InfinitySelfAttention(fused=False, **kw).to(dev).to(torch.bfloat16)
    b_mod = hooks.InfinitySelfAttention(fused='quantizer', **kw).to(dev).to(torch.bfloat16)
    b_mod.load_state_dict(a_mod.state_dict())
    a_mod.kv_caching(True)
    b_mod.kv_caching(True)
    rope = hooks.rope2d_tables(C // H, [(p, p) for p in pn])
    start = 0
    for p in pn:
        note('hooks quantizer backend infinity', p)
        x = torch.randn(2, p * p, C, device=dev, dtype=torch.bfloat16)
        a, b = a_mod(x, rope=rope, token_start=start).float(), b_mod(x, rope=rope, token_start=start).float()
        start += p * p
        rng = a.abs().max().item()
        assert (a - b).abs().max().item() <= 2e-2 * max(rng, 1.0), (p, (a - b).abs().max().item(), rng)
        assert _cos(a, b) >= 0.9995


@pytest.mark.parametrize('backend', ['quantizer', True])
@pytest.mark.parametrize('layout', ['BLHc', 'BHLc'])
def test_var_module_in_fp16_the_dtype_of_its_autocast(dev, backend, layout):
    """The VAR hook in fp16, the dtype the reference's VAR inference runs attention in
    (scripts/inference_multi_VAR.py:123; q, k, v cast at VAR/models/basic_var.py:157-158): the fused
    backends attend in fp16 as well (head dim 64) and agree with the drop-in + fp16 SDPA."""
    torch.manual_seed(8)
    C, H = 512, 8
    pn = (1, 2, 3, 4, 5, 6, 8, 10, 13, 16)
    kw = dict(embed_dim=C, num_heads=H, layout=layout, enable_quantization=True, max_tokens=680)
    if backend is True:
        kw.update(q_bits=4, quant_method='G_GROUP', group_size=64, symmetric=False)
    else:
        kw.update(q_bits=8, quant_method='G_SCALE_HEAD_DIM')
    a_mod = hooks.VarSelfAttention(0, fused=False, **kw).to(dev).half()
    b_mod = hooks.VarSelfAttention(0, fused=backend, **kw).to(dev).half()
    b_mod.load_state_dict(a_mod.state_dict())
    assert b_mod._attn_dtype(torch.float16) == torch.float16 and b_mod._attn_dtype(torch.float32) == torch.bfloat16
    a_mod.kv_caching(True)
    b_mod.kv_caching(True)
    for p in pn:
        note('hooks fp16', backend, layout, p)
        x = torch.randn(2, p * p, C, device=dev, dtype=torch.float16)
        a, b = a_mod(x), b_mod(x)
        assert b.dtype == torch.float16
        a, b = a.float(), b.float()
        rng = a.abs().max().item()
        assert (a - b).abs().max().item() <= 2e-2 * max(rng, 1.0), (p, (a - b).abs().max().item(), rng)
        assert _cos(a, b) >= 0.9995


class _PlainProtocol:
    """The package's quantizer behind the reference's call signature only (no out_dtype): the
    drop-in module then casts the fp32 result itself, as the reference's modules do."""

    def __init__(self, **kw):
        self.q = VAR_Q(**kw)

    def use_var_q(self, item):
        return self.q.use_var_q(item)

    def __getattr__(self, name):
        return getattr(self.q, name)


@pytest.mark.parametrize('layout,method', [('BLHc', 'G_SCALE_HEAD_DIM'), ('BHLc', 'G_SCALE_HEAD_DIM'), ('BLHc', 'G_TOKEN_HEAD')])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_dropin_module_dequantizes_into_the_attention_dtype(dev, layout, method, dtype):
    """fused=False with this package's quantizer: K and V come back in the module's compute
    dtype directly; the module's output is bit for bit the one it gives when the quantizer
    returns fp32 and the module casts."""
    torch.manual_seed(9)
    C, H = 256, 4
    kw = dict(embed_dim=C, num_heads=H, layout=layout, q_bits=8, quant_method=method, enable_quantization=True, max_tokens=40)
    a_mod = hooks.VarSelfAttention(0, fused=False, **kw).to(dev).to(dtype)
    b_mod = hooks.VarSelfAttention(0, fused=False, quantizer_factory=_PlainProtocol, **kw).to(dev).to(dtype)
    b_mod.load_state_dict(a_mod.state_dict())
    a_mod.kv_caching(True)
    b_mod.kv_caching(True)
    for n in (1, 4, 9, 16):
        note('hooks dropin into attention dtype', layout, method, dtype, n)
        x = torch.randn(2, n, C, device=dev, dtype=dtype)
        assert torch.equal(a_mod(x), b_mod(x))
    assert isinstance(a_mod.k_quant, VAR_Q) and not isinstance(b_mod.k_quant, VAR_Q)


def test_parameter_only_tensors_are_kept_for_one_cached_schedule(dev):
    """Under no_grad and kv_caching(True) the qkv bias and the per-head multiplier are built once
    per schedule; the outputs are those of the module that rebuilds them every call, and a
    parameter changed between two schedules is seen by the next one."""
    torch.manual_seed(11)
    C, H = 256, 4
    kw = dict(embed_dim=C, num_heads=H, layout='BLHc', q_bits=4, quant_method='G_GROUP', group_size=64, symmetric=False,
              enable_quantization=True, max_tokens=40, fused=True, fused_producer=True)
    a_mod = hooks.VarSelfAttention(0, **kw).to(dev).to(torch.bfloat16)
    b_mod = hooks.VarSelfAttention(0, **kw).to(dev).to(torch.bfloat16)
    with torch.no_grad():
        a_mod.q_bias.normal_(); a_mod.v_bias.normal_()
    b_mod.load_state_dict(a_mod.state_dict())
    xs = [torch.randn(2, n, C, device=dev, dtype=torch.bfloat16) for n in (1, 4, 9, 16)]
    for round_ in range(2):
        a_mod.kv_caching(True)
        b_mod.kv_caching(True)
        for x in xs:
            note('hooks session tensors', round_, x.shape[1])
            with torch.no_grad():
                a = a_mod(x)
            with torch.enable_grad():             # nothing is kept while gradients are recorded
                b = b_mod(x)
            assert torch.equal(a, b.detach())
        assert len(a_mod._session) >= 2 and len(b_mod._session) == 0
        a_mod.kv_caching(False)
        b_mod.kv_caching(False)
        assert a_mod._session == {}
        with torch.no_grad():                     # a new multiplier and bias for the second schedule
            for m in (a_mod, b_mod):
                m.scale_mul_1H11.fill_(1.25)
                m.q_bias.mul_(0.5)

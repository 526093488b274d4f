"""The drop-in VAR_Q class on the GPU against the oracle's restatement of the
reference class, step by step: codes, scales, cache contents and the fp32
tensors handed to attention are identical."""
import pytest
import torch

import varq_oracle as O
from gpu_util import note
from var_q_amd import VAR_Q

pytestmark = pytest.mark.gpu

STEPS = (1, 4, 9, 16)


def _steps(fmt, dtype, seed, H=3, c=64, B=2):
    g = torch.Generator().manual_seed(seed)
    out = []
    for n in STEPS:
        x = (torch.randn(B, n, H, c, generator=g) * 2).to(dtype)
        out.append(x if fmt == 'BLHc' else x.permute(0, 2, 1, 3).contiguous())
    return out


@pytest.mark.parametrize('fmt', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('method', list(O.METHODS))
@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('pack', [True, False])
def test_state_machine_matches_oracle(dev, fmt, method, bits, pack):
    note('VAR_Q', fmt, method, bits, pack)
    ref = O.OracleVARQ(bits, fmt, method, pack_to_int32=pack)
    gpu = VAR_Q(bits, fmt, method, pack_to_int32=pack)
    for i, x in enumerate(_steps(fmt, torch.bfloat16 if bits == 4 else torch.float32, seed=bits)):
        want = ref.use_var_q(x)
        got = gpu.use_var_q(x.to(dev))
        assert got.dtype == torch.float32 and got.shape == want.shape, (i, got.shape, want.shape)
        assert torch.equal(got.cpu(), want), f'step {i}: dequantized K/V differ'
        assert torch.equal(gpu.scale.cpu(), ref.scale)
        assert torch.equal(gpu.quantized_item.cpu(), ref.quantized_item)
        assert torch.equal(gpu.cached_item.cpu(), ref.cached_item)
        assert torch.equal(gpu.cached_scale.cpu(), ref.cached_scale.contiguous())
        assert gpu._pack_meta == ref._pack_meta
        assert torch.equal(gpu.dequant_current().cpu(), ref.dequant_current())


def test_hook_usage_pattern(dev):
    """Two quantizers per layer, k then v each step, as in
    VAR/models/basic_var.py:109-110,146-147 (BLHc, 8-bit, the shipped rule)."""
    note('VAR_Q hook pattern')
    kq, vq = VAR_Q(8, 'BLHc', 'G_SCALE_HEAD_DIM', blk_idx=3), VAR_Q(8, 'BLHc', 'G_SCALE_HEAD_DIM', blk_idx=3)
    kr, vr = O.OracleVARQ(8, 'BLHc'), O.OracleVARQ(8, 'BLHc')
    g = torch.Generator().manual_seed(11)
    for pn in (1, 2, 3, 4):
        k = torch.randn(4, pn * pn, 16, 64, generator=g).half()
        v = torch.randn(4, pn * pn, 16, 64, generator=g).half()
        assert torch.equal(kq.use_var_q(k.to(dev)).cpu(), kr.use_var_q(k))
        assert torch.equal(vq.use_var_q(v.to(dev)).cpu(), vr.use_var_q(v))
    assert kq.cached_item.shape == (4, 30, 16, 16)


@pytest.mark.parametrize('bits', [2, 4, 8])
@pytest.mark.parametrize('group', [32, 64])
def test_groupwise_asymmetric_extension(dev, bits, group):
    note('VAR_Q G_GROUP', bits, group)
    gpu = VAR_Q(bits, 'BHLc', 'G_GROUP', symmetric=False, group_size=group)
    g = torch.Generator().manual_seed(bits)
    parts = []
    for n in (1, 4, 9):
        x = (torch.randn(2, 3, n, 64, generator=g) + 0.3).bfloat16()
        parts.append(x)
        got = gpu.use_var_q(x.to(dev))
        cat = torch.cat(parts, dim=2)
        q, s, z = O.quant_groupwise(cat, group, bits, True)
        assert torch.equal(got.cpu(), O.dequant_groupwise(q, s, z, group))
        assert torch.equal(gpu.cached_scale.cpu(), s) and torch.equal(gpu.cached_zp.cpu(), z)
        assert torch.equal(gpu.cached_item.cpu(), O.pack_last_dim(q, bits)[0])


def test_per_head_extension_single_call(dev):
    note('VAR_Q G_HEAD')
    x = O.synth_kv((2, 16, 100, 64), seed=5)
    gpu = VAR_Q(8, 'BHLc', 'G_HEAD')
    got = gpu.use_var_q(x.to(dev))
    s = O.scale_sym(x, (0, 2, 3), 8)
    assert torch.equal(got.cpu(), O.dequant_sym(O.codes_sym(x, s, 8), s))
    assert gpu.scale.shape == (1, 16, 1, 1)


@pytest.mark.parametrize('method', list(O.METHODS))
@pytest.mark.parametrize('bits', [4, 8])
@pytest.mark.parametrize('fmt', ['BHLc', 'BLHc'])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_fused_attention_over_quantizer_caches(dev, method, bits, fmt, dtype):
    """`fused_attention` over the packed caches of two drop-in quantizers, all six methods of
    the reference in both of its layouts (BLHc is what its flash-attention call and
    VAR-VAR_Q-8.json use, BHLc what Infinity-VAR_Q-8.json names), four steps, against the
    oracle class's dequant_all -> SDPA on the CPU (the path the reference runs:
    VAR_Q/quant.py:216-230 into the attention backend) in the dtype of q: bf16 (Infinity), or
    fp16, the dtype of the VAR path (VAR/models/basic_var.py:157-158 under the fp16 autocast of
    scripts/inference_multi_VAR.py:123), which the head-dim-64 kernels run in as well.
    Tolerance: cosine >= 0.9995, max-abs 2e-2 in units of the output range."""
    from var_q_amd.quant import fused_attention
    note('fused_attention', method, bits, fmt, dtype)
    ks, vs = _steps(fmt, dtype, seed=20 + bits), _steps(fmt, dtype, seed=30 + bits)
    rk, rv = O.OracleVARQ(bits, fmt, method, pack_to_int32=False), O.OracleVARQ(bits, fmt, method, pack_to_int32=False)
    gk, gv = VAR_Q(bits, fmt, method), VAR_Q(bits, fmt, method)
    g = torch.Generator().manual_seed(5)
    bhl = (lambda t: t) if fmt == 'BHLc' else (lambda t: t.transpose(1, 2))   # to the oracle attention's [B,H,L,c]
    for k, v in zip(ks, vs):
        kd, vd = rk.use_var_q(k), rv.use_var_q(v)
        for qz, item in ((gk, k), (gv, v)):
            qz.quant(item.to(dev))
            qz.cache()
        q = torch.randn(k.shape[0], k.shape[1], k.shape[2], k.shape[3], generator=g).to(dtype)
        got = fused_attention(q.to(dev), gk, gv, 0.125)
        assert got.dtype == dtype
        out = bhl(got.float().cpu())
        assert out.shape == bhl(q).shape
        ref = O.attention_ref(bhl(q), bhl(kd), bhl(vd), 0.125, dtype=dtype).float()
        span = max(1.0, float(ref.abs().max()))
        err = float((out - ref).abs().max())
        cos = float(torch.nn.functional.cosine_similarity(out.flatten().double(), ref.flatten().double(), dim=0))
        assert cos >= 0.9995 and err <= 2e-2 * span, (method, bits, k.shape[2], err, span, cos)


def test_fused_attention_refuses_what_it_cannot_serve(dev):
    from var_q_amd.quant import fused_attention
    x = torch.randn(1, 2, 4, 64, device=dev)
    q = torch.randn(1, 2, 4, 64, device=dev)
    a, b = VAR_Q(8, 'BHLc', 'G_SCALE_HEAD_DIM'), VAR_Q(8, 'BHLc', 'G_SCALE_HEAD_DIM')
    with pytest.raises(ValueError, match='packed cache'):
        fused_attention(q, a, b, 1.0)                       # nothing cached yet
    for qz in (a, b):
        qz.use_var_q(x)
    fused_attention(q, a, b, 1.0)
    with pytest.raises(ValueError, match='layout'):             # K and V cached in different layouts
        c = VAR_Q(8, 'BLHc', 'G_SCALE_HEAD_DIM')
        c.use_var_q(x.transpose(1, 2).contiguous())
        fused_attention(q, a, c, 1.0)
    with pytest.raises(ValueError, match='bit-width'):
        d = VAR_Q(4, 'BHLc', 'G_SCALE_HEAD_DIM')
        d.use_var_q(x)
        fused_attention(q, a, d, 1.0)
    with pytest.raises(ValueError, match='cannot be combined'):
        e = VAR_Q(8, 'BHLc', 'G_TOKEN')
        e.use_var_q(x)
        fused_attention(q, a, e, 1.0)
    with pytest.raises(ValueError, match='steps'):
        for _ in range(16):                                   # 17 cached steps
            for qz in (a, b):
                qz.use_var_q(x)
        fused_attention(q, a, b, 1.0)


@pytest.mark.parametrize('fmt', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('pack', [True, False])
def test_quant_writes_into_the_cache_buffer(dev, fmt, pack):
    """The appending methods quantize a step straight into the cache buffer: `quantized_item`
    is a window of it and cache() copies nothing.  A second quant() before cache() replaces
    the first; an item put there by the caller is appended by copy as before.  Contents as
    the oracle class's."""
    ref = O.OracleVARQ(8, fmt, 'G_SCALE_HEAD_DIM', pack_to_int32=False)
    gpu = VAR_Q(8, fmt, 'G_SCALE_HEAD_DIM', pack_to_int32=pack)
    items = _steps(fmt, torch.bfloat16, seed=77)
    note('staged quant', fmt, pack)
    gpu.quant((items[0] * 3).to(dev))          # dropped: the next quant() takes its place
    for i, x in enumerate(items):
        ref.use_var_q(x)
        gpu.quant(x.to(dev))
        buf = gpu._c_item.buf
        lo, hi = buf.data_ptr(), buf.data_ptr() + buf.numel() * buf.element_size()
        assert lo <= gpu.quantized_item.data_ptr() < hi, 'the step was not quantized into the cache buffer'
        if i == 2:                              # the caller swaps the item: copied in as before
            gpu.quantized_item = gpu.quantized_item.clone()
        gpu.cache()
    codes = gpu.cached_item
    if pack:
        from var_q_amd import ops
        codes = ops.unpack(codes.contiguous(), items[0].shape[-1], 8)
    assert torch.equal(codes.cpu(), ref.cached_item)
    assert torch.equal(gpu.cached_scale.cpu(), ref.cached_scale)
    assert torch.equal(gpu.dequant_all().cpu(), ref.dequant_all())


@pytest.mark.parametrize('fmt', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('bits,sym', [(8, True), (4, False)])
def test_fused_step_leaves_the_state_of_quant_and_cache(dev, fmt, bits, sym):
    """`fused_step` (one library call per tensor for the shipped rule) against the general
    sequence quant(), cache(), fused_attention(): same attention output bit for bit and the
    same quantizer state afterwards -- current item, scale, caches, tables, segment ends --
    at every step; other rules take the general methods inside fused_step."""
    from var_q_amd.quant import fused_attention, fused_step
    ks, vs = _steps(fmt, torch.bfloat16, seed=61), _steps(fmt, torch.bfloat16, seed=62)
    g = torch.Generator().manual_seed(63)
    for method in ('G_SCALE_HEAD_DIM', 'G_TOKEN'):
        a = [VAR_Q(bits, fmt, method, symmetric=sym) for _ in range(2)]
        b = [VAR_Q(bits, fmt, method, symmetric=sym) for _ in range(2)]
        for k, v in zip(ks, vs):
            q = torch.randn(*k.shape, generator=g).bfloat16().to(dev)
            k, v = k.to(dev), v.to(dev)
            note('fused_step', fmt, bits, sym, method, tuple(k.shape))
            for qz, item in ((a[0], k), (a[1], v)):
                qz.quant(item)
                qz.cache()
            want = fused_attention(q, a[0], a[1], 0.125)
            got = fused_step(q, k, v, b[0], b[1], 0.125)
            assert torch.equal(got, want)
            for x, y in zip(a, b):
                assert torch.equal(x.quantized_item, y.quantized_item) and torch.equal(x.scale, y.scale)
                assert x.scale.shape == y.scale.shape and x._pack_meta == y._pack_meta and x._seg_ends == y._seg_ends
                assert (x.zp is None) == (y.zp is None) and (x.zp is None or torch.equal(x.zp, y.zp))
                assert torch.equal(x.cached_item, y.cached_item) and torch.equal(x.cached_scale, y.cached_scale)
                assert x.cached_scale.shape == y.cached_scale.shape
                assert (x.cached_zp is None) == (y.cached_zp is None) and (x.cached_zp is None or torch.equal(x.cached_zp, y.cached_zp))
                assert torch.equal(x.dequant_all(), y.dequant_all())


def test_reserve_tokens_keeps_the_buffers_in_place(dev):
    """With the schedule's length reserved the cache buffers are allocated once; contents as
    without the reservation."""
    from var_q_amd.quant import fused_step
    items = _steps('BHLc', torch.bfloat16, seed=91)
    total = sum(x.shape[2] for x in items)
    a, b = VAR_Q(8, 'BHLc', 'G_SCALE_HEAD_DIM'), VAR_Q(8, 'BHLc', 'G_SCALE_HEAD_DIM')
    b.reserve_tokens(1000)
    ptrs = set()
    for x in items:
        note('reserve_tokens', tuple(x.shape))
        a.use_var_q(x.to(dev))
        b.use_var_q(x.to(dev))
        ptrs.add(b._c_item.buf.data_ptr())
        assert b._c_item.buf.shape[2] >= 1000
    assert len(ptrs) == 1 and a._c_item.buf.shape[2] < 1000
    assert torch.equal(a.cached_item, b.cached_item) and torch.equal(a.cached_scale, b.cached_scale)
    assert a.cached_item.shape[2] == total


def test_layout_change_with_cached_steps_is_refused(dev):
    """qkv_format may be re-assigned before the first step (Infinity's attention assigns it every
    forward, basic.py:309,314); with steps cached in the other layout the next step raises instead
    of continuing on a truncated cache."""
    note('VAR_Q layout change')
    q = VAR_Q(8, 'BLHc', 'G_SCALE_HEAD_DIM')
    q.qkv_format = 'BHLc'
    x = torch.randn(2, 3, 4, 64, device=dev)
    assert q.use_var_q(x).shape == x.shape
    q.qkv_format = 'BHLc'                                   # the same layout again: nothing happens
    assert q.use_var_q(x).shape == (2, 3, 8, 64)
    q.qkv_format = 'BLHc'
    with pytest.raises(ValueError, match='qkv_format was changed'):
        q.use_var_q(x)


@pytest.mark.parametrize('fmt', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('method', ['G_SCALE_HEAD_DIM', 'G_TOKEN', 'G_HEAD_DIM', 'G_TENSOR'])
@pytest.mark.parametrize('keep', [True, False])
def test_use_var_q_keeps_the_dequantized_prefix(dev, fmt, method, keep):
    """With keep_dequantized=True use_var_q dequantizes only the new step and keeps the earlier
    values; calls of quant() and cache() on their own in between (the fused path makes them) must
    not leave it with stale values, and a result handed out earlier must not change when later
    steps arrive.  Without the flag (the default) nothing is kept and every call returns a fresh
    tensor, like the reference."""
    note('VAR_Q incremental dequant', fmt, method, keep)
    ref, gpu = O.OracleVARQ(8, fmt, method), VAR_Q(8, fmt, method, keep_dequantized=keep)
    steps = _steps(fmt, torch.float32, seed=77) + _steps(fmt, torch.float32, seed=78)
    held = []
    for i, x in enumerate(steps):
        if i in (2, 5):                      # a step cached without asking for the dequantized cache
            ref.quant(x); ref.cache()
            gpu.quant(x.to(dev)); gpu.cache()
            continue
        want, got = ref.use_var_q(x), gpu.use_var_q(x.to(dev))
        assert got.shape == want.shape and torch.equal(got.cpu(), want), f'step {i}'
        assert torch.equal(gpu.dequant_all().cpu(), want), f'step {i}: dequant_all'
        held.append((got, want.clone()))
        if not keep:
            assert gpu._c_deq.buf is None, 'the default keeps no dequantized copy of the cache'
    for got, want in held:
        assert torch.equal(got.cpu(), want), 'an earlier result changed'


@pytest.mark.parametrize('fmt', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('method', ['G_SCALE_HEAD_DIM', 'G_TOKEN', 'G_HEAD_DIM', 'G_TENSOR', 'G_TOKEN_HEAD', 'G_SCALE'])
@pytest.mark.parametrize('bits,pack', [(8, True), (4, True), (8, False)])
def test_use_var_q_into_the_attention_dtype(dev, fmt, method, bits, pack):
    """use_var_q(x, out_dtype=...) and dequant_all(out_dtype) give the fp32 result of the
    reference's protocol rounded once to that type, i.e. what the attention module's own cast of
    the fp32 tensor gives (VAR/models/basic_var.py:158), at every step."""
    note('VAR_Q dequantized into the attention dtype', fmt, method, bits, pack)
    ref = O.OracleVARQ(bits, fmt, method, pack_to_int32=pack)
    for out_dtype in (torch.bfloat16, torch.float16):
        gpu = VAR_Q(bits, fmt, method, pack_to_int32=pack)
        ref = O.OracleVARQ(bits, fmt, method, pack_to_int32=pack)
        for i, x in enumerate(_steps(fmt, torch.float32, seed=31)):
            want = ref.use_var_q(x).to(out_dtype)
            got = gpu.use_var_q(x.to(dev), out_dtype=out_dtype)
            assert got.dtype == out_dtype and torch.equal(got.cpu(), want), f'step {i} {out_dtype}'
            assert torch.equal(gpu.dequant_all(out_dtype).cpu(), want)
            assert gpu.dequant_all().dtype == torch.float32


@pytest.mark.parametrize('fmt', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('method', ['G_SCALE_HEAD_DIM', 'G_TOKEN_HEAD', 'G_TOKEN'])
def test_empty_step_is_refused_and_changes_nothing(dev, fmt, method):
    """A step without tokens: the reference fails in its amax over an empty dim
    (VAR_Q/quant.py:113, a RuntimeError of torch); here the quantizer says so itself, before
    anything is launched or cached, and the next step continues where the last one ended."""
    from var_q_amd.quant import fused_step
    g = torch.Generator().manual_seed(11)
    shape = (lambda n: (2, 3, n, 64)) if fmt == 'BHLc' else (lambda n: (2, n, 3, 64))
    dim = 2 if fmt == 'BHLc' else 1
    steps = [torch.randn(*shape(n), generator=g).bfloat16().to(dev) for n in (4, 9)]
    empty = torch.empty(*shape(0), dtype=torch.bfloat16, device=dev)
    note('empty step', fmt, method)
    a, b = VAR_Q(8, fmt, method), VAR_Q(8, fmt, method)
    with pytest.raises(RuntimeError, match='nothing to quantize'):
        VAR_Q(8, fmt, method).use_var_q(empty)
    r0 = a.use_var_q(steps[0])
    b.use_var_q(steps[0])
    with pytest.raises(RuntimeError, match='nothing to quantize'):
        a.use_var_q(empty)
    with pytest.raises(RuntimeError, match='nothing to quantize'):
        fused_step(empty, empty, empty, a, VAR_Q(8, fmt, method), 0.1)
    assert a.cached_item.size(dim) == 4 and torch.equal(a.dequant_all(), r0)
    assert torch.equal(a.use_var_q(steps[1]), b.use_var_q(steps[1]))


@pytest.mark.parametrize('fmt', ['BLHc', 'BHLc'])
@pytest.mark.parametrize('bits,pack', [(8, True), (8, False), (5, False)])
def test_table_rows_off_a_16_byte_boundary(dev, fmt, bits, pack):
    """H * c not a multiple of four: the rows of the per-step scale table behind the first are
    not 16-byte aligned (H=3, c=30: row 1 starts at byte 360).  Such a shape takes the kernels
    that move one parameter at a time, which need no such alignment; every step must work and
    match the oracle."""
    note('VAR_Q odd table rows', fmt, bits, pack)
    ref, gpu = O.OracleVARQ(bits, fmt, 'G_SCALE_HEAD_DIM', pack_to_int32=pack), VAR_Q(bits, fmt, 'G_SCALE_HEAD_DIM', pack_to_int32=pack)
    for i, x in enumerate(_steps(fmt, torch.float32, seed=5, H=3, c=30)):
        want, got = ref.use_var_q(x), gpu.use_var_q(x.to(dev))
        assert torch.equal(got.cpu(), want), f'step {i}'
        assert torch.equal(gpu.scale.cpu(), ref.scale) and torch.equal(gpu.cached_item.cpu(), ref.cached_item)

"""Fused attention over a cache quantized per (head, channel) -- the scale layout of the
reference's G_SCALE_HEAD_DIM / G_HEAD_DIM methods (VAR_Q/quant.py:84-88), scalar scales
(G_TENSOR), and the affine per-head-per-dim variant of benchmark configuration 3 --
against the oracle path quantize -> dequant -> bf16 SDPA and an fp64 evaluation of the same
formula, on the data of the benchmark configurations (outlier channels x15) throughout.
The kernel dequantizes K and V with the tables of each key's segment when a tile is widened
-- (code - zp) * scale in fp32, rounded to bf16, the oracle's own operands -- so the bar here
is half the general one: max|out - oracle| <= 1e-2 in units of the output range (cosine >=
0.9995 as everywhere); what is left is the bf16 rounding of the weights and of the output
(one bf16 step of an output near the top of the range is 0.4e-2 to 0.8e-2 of it).  The distance of both from the fp64 value is printed beside it (up to ~2 % of
the range on this data, the same for kernel and oracle).  The codes handed to the kernel are
the oracle's own, so the comparison isolates the attention."""
import math

import pytest
import torch

import varq_oracle as O
from gpu_util import note
from test_gpu_attention import _compare, _exact_fp64
from var_q_amd import ops, schedules

pytestmark = pytest.mark.gpu

ORACLE_BAR = 1e-2   # kernel vs oracle, in units of the output range: half the general bar (one bf16 step of the output is up to 0.8e-2)


def _quantize_channel(x, bits, asym, dims=(0, 2)):
    """x [B,H,L,D] -> packed words, [H*D] tables, dequantized fp32 (reduce over batch and tokens)."""
    q, s, z = O.quant_reduce(x, dims, bits, asym)
    deq = O.dequant_asym(q, s, z) if asym else O.dequant_sym(q, s)
    H, D = x.shape[1], x.shape[3]
    table = lambda t: None if t is None else t.expand(1, H, 1, D).reshape(H, D).contiguous()
    return O.pack_last_dim(q, bits)[0], table(s), table(z), deq


def _run(dev, B, H, Lq, Lk, D, bits, asym, seed, kv_limit=None, bias=None, dist='normal', dims=(0, 2), what='', splits=0,
         drop_k_zp=False):
    g = torch.Generator().manual_seed(seed)
    k = O.synth_kv((B, H, Lk, D), seed + 1, dist).bfloat16()
    v = O.synth_kv((B, H, Lk, D), seed + 2, dist).bfloat16()
    q = torch.randn(B, H, Lq, D, generator=g).bfloat16()
    kw, ks, kz, kd = _quantize_channel(k, bits, asym, dims)
    vw, vs, vz, vd = _quantize_channel(v, bits, asym, dims)
    scale = 1.0 / math.sqrt(D)
    note('fused_attn_channel', what, (B, H, Lq, Lk, D), bits, asym, 'splits', splits)
    # one table: the zero-point of K shifts all logits of a query alike and may be left out; the
    # dequantized K is then offset per channel and rounds differently from the oracle's
    kz_arg = None if (kz is None or drop_k_zp) else kz.to(dev)
    out = ops.fused_attn_channel(q.to(dev), kw.to(dev), ks.to(dev), kz_arg, vw.to(dev), vs.to(dev),
                                 None if vz is None else vz.to(dev), bits, Lk, scale,
                                 kv_limit=None if kv_limit is None else kv_limit.to(dev), splits=splits)
    torch.cuda.synchronize()
    ref = O.attention_ref(q, kd, vd, scale, bias)
    # (with K's zero-point left out the operands are not the reference's roundings: that call is
    # held to the clause of the modes that round differently, see test_gpu_attention.py)
    _compare(out, ref, _exact_fp64(q, kd, vd, scale, bias, dev), what, oracle_bar=2e-2 if drop_k_zp else ORACLE_BAR,
             exact_codes=drop_k_zp)


@pytest.mark.parametrize('D', [64, 128])
@pytest.mark.parametrize('bits,asym', [(8, False), (4, False), (2, True), (4, True), (8, True)])
def test_small_all_visible(dev, D, bits, asym):
    _run(dev, 2, 3, 200, 333, D, bits, asym, seed=bits * 10 + D + asym, what='channel small')


@pytest.mark.parametrize('bits', [2, 4, 8])
def test_k_zero_point_left_out(dev, bits):
    _run(dev, 2, 3, 200, 333, 64, bits, True, seed=bits * 10 + 5, what='channel, no K zero-point', drop_k_zp=True)


@pytest.mark.parametrize('Lq,Lk', [(1, 1), (4, 5), (33, 64), (129, 127), (7, 300)])
def test_ragged_sizes(dev, Lq, Lk):
    _run(dev, 1, 2, Lq, Lk, 128, 8, False, seed=Lq * 1000 + Lk, what='channel ragged')


def test_scalar_scale_is_a_constant_table(dev):
    """G_TENSOR: one scale for the whole tensor (VAR_Q/quant.py:78-80)."""
    _run(dev, 2, 2, 64, 150, 64, 8, False, seed=5, dims=(0, 1, 2, 3), what='channel scalar')


def test_block_causal_mask(dev):
    pn = O.VAR_PATCH_NUMS
    L = 680
    _run(dev, 1, 2, L, L, 64, 8, False, seed=31, kv_limit=schedules.kv_limit(pn), bias=O.block_causal_bias(pn),
         what='channel block-causal')


def test_config3_var_d30(dev):
    """Benchmark configuration 3 with the batch cut to 2 for the CPU oracle: VAR-d30 shape,
    INT2 asymmetric per-head-per-dim and INT8 symmetric per-channel, the final-scale 256
    queries over 680 keys."""
    _run(dev, 2, 30, 256, 680, 64, 2, True, seed=3003, what='c3 int2 per-head-per-dim')
    _run(dev, 2, 30, 256, 680, 64, 8, False, seed=3004, what='c3 int8 per-channel')


def test_head_subset_and_device_quantizer(dev):
    """Codes and tables straight from the device quantizer (the reference's method
    G_SCALE_HEAD_DIM on a BHLc tensor), spare token rows in the buffers, three of five heads."""
    B, Hq, D, Lk, Lstride, bits = 2, 5, 128, 90, 128, 8
    heads = [4, 1, 2]
    gen = torch.Generator().manual_seed(11)
    k = torch.randn(B, len(heads), Lk, D, generator=gen).bfloat16()
    v = torch.randn(B, len(heads), Lk, D, generator=gen).bfloat16()
    q = torch.randn(B, Hq, 40, D, generator=gen).bfloat16()
    kq, ks, _ = O.quant_reduce(k, (0, 2), bits, False)
    vq, vs, _ = O.quant_reduce(v, (0, 2), bits, False)
    kw_d, ks_d, _ = ops.quant_pack(k.to(dev), (0, 2), bits, False)
    vw_d, vs_d, _ = ops.quant_pack(v.to(dev), (0, 2), bits, False)
    assert torch.equal(kw_d.cpu(), O.pack_last_dim(kq, bits)[0]) and torch.equal(ks_d.cpu(), ks)
    kbuf = torch.zeros(B, len(heads), Lstride, kw_d.shape[3], dtype=torch.int32, device=dev)
    vbuf = torch.zeros_like(kbuf)
    kbuf[:, :, :Lk] = kw_d
    vbuf[:, :, :Lk] = vw_d
    out = torch.full((B, Hq, 40, D), 7.0, dtype=torch.bfloat16, device=dev)
    note('fused_attn_channel', 'head subset', (B, Hq, 40, Lk, D))
    ops.fused_attn_channel(q.to(dev), kbuf, ks_d.reshape(len(heads), D).contiguous(), None, vbuf,
                           vs_d.reshape(len(heads), D).contiguous(), None, bits, Lk, 0.1,
                           head_map=torch.tensor(heads, dtype=torch.int32, device=dev), out=out)
    torch.cuda.synchronize()
    qs = q[:, heads]
    kd, vd = O.dequant_sym(kq, ks), O.dequant_sym(vq, vs)
    _compare(out[:, heads], O.attention_ref(qs, kd, vd, 0.1), O.attention_exact(qs.float(), kd, vd, 0.1), 'channel head subset')
    untouched = [h for h in range(Hq) if h not in heads]
    assert bool((out[:, untouched] == 7.0).all()), 'rows of heads outside the map were written'


def _stepwise(dev, B, H, D, steps, bits, asym, Lq, seed, masked=False, what='', outlier_mul=15.0, splits=0):
    """A cache filled step by step: every step is quantized on its own with one (scale, zp)
    per (head, channel), as the reference's append methods do (VAR_Q/quant.py:140-201 for the
    symmetric case, run here through the oracle's state machine)."""
    g = torch.Generator().manual_seed(seed)
    L = sum(steps)
    k = O.synth_kv((B, H, L, D), seed + 1, outlier_mul=outlier_mul).bfloat16()
    v = O.synth_kv((B, H, L, D), seed + 2, outlier_mul=outlier_mul).bfloat16()
    q = torch.randn(B, H, Lq, D, generator=g).bfloat16()
    packed, tables, deq = [], [], []
    for x in (k, v):
        codes, sc, zp, dq = [], [], [], []
        if not asym:
            oq = O.OracleVARQ(quant_bits=bits, qkv_format='BHLc', quant_method='G_SCALE_HEAD_DIM', pack_to_int32=False)
        pos = 0
        for n in steps:
            item = x[:, :, pos:pos + n]
            pos += n
            if asym:
                c, s, z = O.quant_reduce(item, (0, 2), bits, True)
                dq.append(O.dequant_asym(c, s, z))
                zp.append(z.reshape(H, D))
            else:
                full = oq.use_var_q(item)           # the reference's own sequence of calls
                c, s = oq.quantized_item, oq.scale
            codes.append(c)
            sc.append(s.reshape(H, D))
        packed.append(O.pack_last_dim(torch.cat(codes, dim=2), bits)[0])
        tables.append((torch.stack(sc).contiguous(), torch.stack(zp).contiguous() if asym else None))
        deq.append(torch.cat(dq, dim=2) if asym else full)
    ends = [sum(steps[:i + 1]) for i in range(len(steps))]
    scale = 1.0 / math.sqrt(D)
    lim = bias = None
    if masked:   # the queries are the last Lq tokens; each sees keys up to the end of its own step
        level_end = torch.tensor([e for e, n in zip(ends, steps) for _ in range(n)], dtype=torch.int32)
        lim = level_end[L - Lq:].contiguous()
        bias = torch.where(torch.arange(L)[None, :] < lim[:, None].long(), 0.0, float('-inf'))[None, None]
    note('fused_attn_channel', what, (B, H, Lq, L, D), bits, asym, steps, 'splits', splits)
    out = ops.fused_attn_channel(q.to(dev), packed[0].to(dev), tables[0][0].to(dev),
                                 None if not asym else tables[0][1].to(dev), packed[1].to(dev),
                                 tables[1][0].to(dev), None if not asym else tables[1][1].to(dev), bits, L, scale,
                                 kv_limit=None if lim is None else lim.to(dev), seg_ends=ends, splits=splits)
    torch.cuda.synchronize()
    ref = O.attention_ref(q, deq[0], deq[1], scale, bias)
    _compare(out, ref, _exact_fp64(q, deq[0], deq[1], scale, bias, dev), what, oracle_bar=ORACLE_BAR)


VAR_STEPS = [n * n for n in O.VAR_PATCH_NUMS]


def test_stepwise_cache_reference_default_rule(dev):
    """The shipped rule (G_SCALE_HEAD_DIM, 8 bits, VAR-VAR_Q-8.json) over the VAR schedule:
    ten steps, ten tables, the final 256 queries see everything."""
    _stepwise(dev, 2, 3, 64, VAR_STEPS, 8, False, 256, seed=41, what='stepwise sym8 VAR')


@pytest.mark.parametrize('bits,asym', [(4, False), (2, True), (8, True)])
def test_stepwise_cache_other_widths(dev, bits, asym):
    """Eight steps of the Infinity schedule at D=128, on the data of the benchmark
    configurations (outlier channels x15), 2-bit codes included."""
    _stepwise(dev, 1, 2, 128, [1, 4, 16, 36, 64, 144, 256, 400], bits, asym, 400, seed=50 + bits, what='stepwise D128')


def test_stepwise_cache_masked_queries(dev):
    """Queries of the last three steps in one call, each limited to the end of its own step:
    short tiles at segment ends and the block-causal limit act together."""
    _stepwise(dev, 1, 2, 64, VAR_STEPS, 8, False, 100 + 169 + 256, seed=43, masked=True, what='stepwise masked')
    _stepwise(dev, 1, 2, 64, VAR_STEPS, 4, True, 680, seed=44, masked=True, what='stepwise masked asym')


def test_stepwise_cache_single_step_equals_plain_call(dev):
    """One segment given explicitly is the same launch as no segments."""
    _stepwise(dev, 1, 2, 64, [300], 8, False, 77, seed=45, what='stepwise single')

#!/usr/bin/env python3
"""Benchmark of the VAR-Q hot path on one MI355X.

One step = one pass over benchmark configuration 4 (Infinity-2B shape): quantize+pack K
and V [2,16,10521,128] bf16 to INT4 group-128 asymmetric, then fused dequant
attention of the final scale's 4096 queries over all 10521 packed keys.  Inputs
are resident in HBM before the timed region.  Prints ONE JSON line.

Before the W warm-up steps the same step runs untimed until 150 ms of GPU work have
passed, whatever W is: the first ~50 ms after idle run at lower clocks.

After the timed region (and outside `value`): the quantize+pack kernel and the
unpack+dequant kernel of configuration 4 timed as back-to-back launches between one
event pair (kernel time without the dispatch gaps); the CPU baseline (1 thread and all
threads, per stage, median of 3) with the parity check of the timed GPU results against
it; a leg for few queries over the whole packed cache (where the KV-read fraction of HBM peak
is the bound); and legs for configurations 2, 3 and 5 and for the shipped JSON rules.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-hbm] [--no-c2] [--no-c3] [--no-c5] [--no-prepare] [--no-rule]
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, 'oracle')):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16, published

B, H, L, D = 2, 16, 10521, 128
LQ = 4096
BITS, GROUP = 4, 128
NBUF = 4   # distinct input sets cycled through, 4*2*86 MB > the 256 MB Infinity Cache


def algorithmic_bytes():
    n = B * H * L * D
    groups = B * H * L * (D // GROUP)
    quant_pack = n * 2 + n * BITS // 8 + groups * 8            # per tensor: bf16 in, packed out, scale+zp out
    kv_read = 2 * (n * BITS // 8 + groups * 8)                  # packed K and V with scales/zps, read once
    attn_flops = 4 * B * H * LQ * L * D
    return quant_pack, kv_read, attn_flops


def cpu_model():
    try:
        for line in open('/proc/cpuinfo'):
            if line.lower().startswith('model name'):
                return line.split(':', 1)[1].strip()
    except OSError:
        pass
    return 'unknown'


def _median(v):
    v = sorted(v)
    return v[len(v) // 2]


def cpu_baseline(torch, O, k0, v0, q0, threads, reps=3):
    """The CPU oracle timed on this host, per stage, median of `reps` runs, with all the
    threads the box gives this process and with one thread: full-size quantize+pack of K and
    V, unpack+dequant of both, bf16 attention of the 4096 queries (all of them with all
    threads; a 512-query sample scaled x8 with one thread, to bound the run time)."""
    scale = 1.0 / math.sqrt(D)
    res, keep = {}, None
    for label, nthreads, nq in (('all_threads', threads, LQ), ('one_thread', 1, 512)):
        torch.set_num_threads(nthreads)
        tq, td, ta = [], [], []
        for _ in range(reps):
            t0 = time.perf_counter()
            kq, ks, kz = O.quant_groupwise(k0, GROUP, BITS, True)
            kw, kmeta = O.pack_last_dim(kq, BITS)
            vq, vs, vz = O.quant_groupwise(v0, GROUP, BITS, True)
            vw, vmeta = O.pack_last_dim(vq, BITS)
            t1 = time.perf_counter()
            kd = O.dequant_groupwise(O.unpack_last_dim(kw, kmeta), ks, kz, GROUP)
            vd = O.dequant_groupwise(O.unpack_last_dim(vw, vmeta), vs, vz, GROUP)
            t2 = time.perf_counter()
            ref = O.attention_ref(q0[:, :, :nq], kd, vd, scale)
            t3 = time.perf_counter()
            tq.append((t1 - t0) / 2)
            td.append(t2 - t1)
            ta.append((t3 - t2) * (LQ / nq))
        res[label] = {'threads': nthreads, 'quant_pack_s_per_tensor': round(_median(tq), 4),
                      'unpack_dequant_s_both': round(_median(td), 4), 'attention_s_4096_queries': round(_median(ta), 4),
                      'attention_queries_timed': nq}
        if keep is None:
            keep = {'kw': kw, 'ks': ks, 'kz': kz, 'vw': vw, 'vs': vs, 'vz': vz, 'kd': kd, 'vd': vd, 'ref': ref}
    torch.set_num_threads(threads)
    return res, keep


C5_B, C5_H, C5_D, C5_GROUP = 8, 16, 128, 64
C5_CHECK_SCALES = (1, 8, 32, 64)      # patch numbers of the scales whose attention output is checked


def c5_head_bits(torch):
    """Config 5's per-head bit-widths: seed-assigned from {2, 4, 8}."""
    g = torch.Generator().manual_seed(5000)
    return [(2, 4, 8)[int(i)] for i in torch.randint(0, 3, (C5_H,), generator=g)]


def c5_check(torch, O, dev, cache, steps, outs, bits):
    """Config 5 at its named size against the oracle, for one (batch, head) per bit-width class:
    the cache contents (packed words, scales, zero-points of all 10 521 tokens) bit for bit, and
    that head's attention output at the scales of C5_CHECK_SCALES against unpack -> dequant ->
    bf16 SDPA, max-abs <= 2e-2 x range and cosine >= 0.9995.  `steps` are the (q, k, v) of every
    scale on the device, `outs` the attention outputs of the pass that filled `cache`."""
    from var_q_amd.schedules import INFINITY_PATCH_NUMS
    ns = [pn * pn for pn in INFINITY_PATCH_NUMS]
    scale = 1.0 / math.sqrt(C5_D)
    res = {'cache_bit_exact': True, 'attn_cosine_min': 1.0, 'attn_maxabs_over_range_max': 0.0, 'pairs': []}
    for ci, c in enumerate(cache.classes):
        h = c.heads[0]
        b = (0, C5_B // 2, C5_B - 1)[ci % 3]
        slot = int(c.slot[h])
        deq = {}
        for name, idx, words, sc, zp in (('k', 1, c.k_words, c.k_scale, c.k_zp), ('v', 2, c.v_words, c.v_scale, c.v_zp)):
            x = torch.cat([st[idx][b, h] for st in steps], 0).cpu()                     # [L, D] as appended
            codes, s_ref, z_ref = O.quant_groupwise(x, C5_GROUP, c.bits, True)
            ok = (torch.equal(words[b, slot, :cache.len].cpu(), O.pack_last_dim(codes, c.bits)[0])
                  and torch.equal(sc[b, slot, :cache.len].cpu(), s_ref) and torch.equal(zp[b, slot, :cache.len].cpu(), z_ref))
            res['cache_bit_exact'] = res['cache_bit_exact'] and bool(ok)
            deq[name] = O.dequant_groupwise(codes, s_ref, z_ref, C5_GROUP)
        pos = 0
        for i, pn in enumerate(INFINITY_PATCH_NUMS):
            pos += ns[i]
            if pn not in C5_CHECK_SCALES:
                continue
            q = steps[i][0][b, h].cpu()
            ref = O.attention_ref(q[None, None], deq['k'][None, None, :pos], deq['v'][None, None, :pos], scale)[0, 0].double()
            got = outs[i][b, h].double().cpu()
            span = max(1.0, float(ref.abs().max()))
            res['attn_maxabs_over_range_max'] = max(res['attn_maxabs_over_range_max'], float((got - ref).abs().max()) / span)
            res['attn_cosine_min'] = min(res['attn_cosine_min'],
                                         float(torch.nn.functional.cosine_similarity(got.flatten(), ref.flatten(), dim=0)))
        res['pairs'].append({'bits': c.bits, 'batch': b, 'head': h})
    res['attn_maxabs_over_range_max'] = round(res['attn_maxabs_over_range_max'], 5)
    res['attn_cosine_min'] = round(res['attn_cosine_min'], 6)
    res['ok'] = bool(res['cache_bit_exact'] and res['attn_maxabs_over_range_max'] <= 2e-2 and res['attn_cosine_min'] >= 0.9995)
    return res


def c5_latency(torch, dev, passes=10, warm=3, check=True):
    """Config 5: B=8 (4 images x CFG pair), H=16, D=128, the 13 Infinity scales; heads carry
    2/4/8-bit codes (seeded), group 64 asymmetric.  Per scale: quantize+pack the step's K and V
    in place into the pre-allocated cache, then fused attention of that scale's queries over
    the prefix.  Returns seconds per pass (all scales, one layer); `checked` is c5_check on the
    last timed pass."""
    from var_q_amd import PackedKVCache
    from var_q_amd.schedules import INFINITY_PATCH_NUMS
    B5, H5, D5 = C5_B, C5_H, C5_D
    ns = [pn * pn for pn in INFINITY_PATCH_NUMS]
    bits = c5_head_bits(torch)
    cache = PackedKVCache(B5, H5, sum(ns), D5, bits, C5_GROUP, dev)
    gd = torch.Generator(device=dev).manual_seed(5005)
    steps = [tuple(torch.randn(B5, H5, n, D5, device=dev, generator=gd).bfloat16() for _ in range(3)) for n in ns]
    outs = [torch.empty_like(s[0]) for s in steps]
    def one_pass():
        cache.reset()
        for (q, k, v), o in zip(steps, outs):
            cache.append(k, v)
            cache.attend(q, 1.0 / math.sqrt(D5), out=o)
    warm_passes(torch, one_pass, warm)
    t0 = time.perf_counter()
    for _ in range(passes):
        one_pass()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / passes
    flops = sum(4 * B5 * H5 * n * sum(ns[:i + 1]) * D5 for i, n in enumerate(ns))
    # the same pass recorded once into a HIP graph and replayed: the first eight scales are a few
    # microseconds of GPU work each behind ~140 us of host work per scale (three bit-width classes
    # on side streams), which a replay does not pay
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        one_pass()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        one_pass()
    warm_passes(torch, graph.replay, warm)
    t0 = time.perf_counter()
    for _ in range(passes):
        graph.replay()
    torch.cuda.synchronize()
    dt_graph = (time.perf_counter() - t0) / passes
    checked = None
    if check:
        import varq_oracle as O
        checked = c5_check(torch, O, dev, cache, steps, outs, bits)
        if not checked['ok']:
            print('bench.py: config 5 differs from the oracle: %r' % checked, file=sys.stderr)
            sys.exit(1)
    return {'workload': 'config 5: 13-scale Infinity schedule, B=8 H=16 D=128, per-head bits %s, group 64 asymmetric, '
                        'in-place append + fused attention per scale, one layer' % ''.join(str(b) for b in bits),
            'ms_per_layer_pass': round(dt * 1e3, 4), 'ms_per_image_per_layer': round(dt * 1e3 / 4, 4),
            'attn_TFLOPs_incl_append': round(flops / dt / 1e12, 2), 'passes': passes,
            'graph_replay_ms_per_layer_pass': round(dt_graph * 1e3, 4), 'graph_replay_TFLOPs': round(flops / dt_graph / 1e12, 2),
            'checked': checked}


PREWARM_MS = 50.0     # 0 (--fixed-prewarm): warm up by launch count only, so that separate runs launch alike


def warm_passes(torch, one_pass, warm):
    """At least `warm` passes and PREWARM_MS of them before a pass-level timing."""
    t0 = time.perf_counter()
    done = 0
    while done < warm or ((time.perf_counter() - t0) * 1e3 < PREWARM_MS and done < 1000):
        one_pass()
        torch.cuda.synchronize()
        done += 1


def timed_launches(torch, fn, reps=20, warm=5, rounds=5):
    """Seconds per call of fn: `reps` back-to-back launches between one event pair on the
    current stream, median of `rounds` such measurements, after at least `warm` launches and
    PREWARM_MS of them (the clocks of an idle GPU take tens of milliseconds to come up)."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    done = 0
    while True:
        for _ in range(max(warm, 5)):
            fn()
        done += max(warm, 5)
        e1.record()
        e1.synchronize()
        if e0.elapsed_time(e1) >= PREWARM_MS or done >= 5000:
            break
    ts = []
    for _ in range(rounds):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ts.append(e0.elapsed_time(e1) / reps * 1e-3)
    return _median(ts)


def c2_rates(torch, dev):
    """Config 2: VAR-d16 batch shape, K/V bf16 [64,16,680,64], INT4 asymmetric, K in groups of
    32 channels, V in groups of 64 (per token), 8 codes per word; the final-scale 256 queries
    over all 680 keys.  Two K and two V tensors are cycled (4 x 89 MB > the 256 MB Infinity
    Cache) so that the quantizer reads HBM."""
    import varq_oracle as O
    from var_q_amd import ops
    B2, H2, L2, D2, LQ2, bits = 64, 16, 680, 64, 256, 4
    n_el = B2 * H2 * L2 * D2
    ks_in = [O.synth_kv((B2, H2, L2, D2), 1002 + i, dtype=torch.bfloat16).to(dev) for i in range(2)]
    vs_in = [O.synth_kv((B2, H2, L2, D2), 2002 + i, dtype=torch.bfloat16).to(dev) for i in range(2)]
    q = torch.randn(B2, H2, LQ2, D2, device=dev, generator=torch.Generator(device=dev).manual_seed(3002)).bfloat16()
    out = {'workload': 'config 2: VAR-d16 K/V bf16 [64,16,680,64] -> INT4 asymmetric, K group 32, V group 64; '
                       'final-scale 256 queries over 680 keys'}
    rowmap = [1, 1, B2 * H2 * L2, 0, 0, 1, 0, -1]
    packed = {}
    for name, xs, g in (('k_g32', ks_in, 32), ('v_g64', vs_in, 64)):
        w, sc, zp = ops.quant_pack_rows(xs[0], g, bits, True)
        packed[name] = (w, sc, zp)
        i = [0]

        def qfn():
            i[0] ^= 1
            ops.quant_pack_rows_into(xs[i[0]], g, bits, True, 1e-12, w, sc, zp, rowmap)
        t_q = timed_launches(torch, qfn)
        ops.quant_pack_rows_into(xs[0], g, bits, True, 1e-12, w, sc, zp, rowmap)     # (leave set 0 in the buffers)
        groups = n_el // g
        qbytes = n_el * 2 + n_el * bits // 8 + groups * 8
        t_d = timed_launches(torch, lambda: ops.dequant(w, sc, zp, D2, bits, torch.bfloat16))
        dbytes = n_el * bits // 8 + groups * 8 + n_el * 2
        out[name] = {'quant_pack_us': round(t_q * 1e6, 1), 'quant_pack_GBps': round(qbytes / t_q / 1e9, 1),
                     'quant_pack_frac_hbm_peak': round(qbytes / t_q / 1e9 / HBM_PEAK_GBPS, 4),
                     'quant_pack_tokens_per_s': round(B2 * L2 / t_q, 1),
                     'unpack_dequant_us': round(t_d * 1e6, 1), 'unpack_dequant_GBps': round(dbytes / t_d / 1e9, 1),
                     'unpack_dequant_frac_hbm_peak': round(dbytes / t_d / 1e9 / HBM_PEAK_GBPS, 4)}
    o = torch.empty_like(q)
    (kw, ksc, kzp), (vw, vsc, vzp) = packed['k_g32'], packed['v_g64']
    t_a = timed_launches(torch, lambda: ops.fused_attn(q, kw, ksc, kzp, vw, vsc, vzp, bits, bits, L2, 1.0 / math.sqrt(D2), out=o))
    flops = 4 * B2 * H2 * LQ2 * L2 * D2
    kv = sum(n_el * bits // 8 + (n_el // g) * 8 for g in (32, 64))
    out['fused_attn'] = {'us': round(t_a * 1e6, 1), 'TFLOPs': round(flops / t_a / 1e12, 1),
                         'frac_mfma_peak': round(flops / t_a / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                         'kv_read_GBps': round(kv / t_a / 1e9, 1), 'query_tokens_per_s': round(B2 * LQ2 / t_a, 1)}
    return out


def c3_rates(torch, dev, reps=20, warm=5):
    """Config 3: VAR-d30 shape, K/V bf16 [32,30,680,64], quantized per (head, channel) over
    batch and tokens: (i) INT2 asymmetric, (ii) INT8 symmetric (the reference's
    G_SCALE_HEAD_DIM).  Times quantize+pack, unpack+dequant (bf16 out) and the fused
    attention of the final 256 queries, with CUDA events around `reps` launches each."""
    from var_q_amd import ops
    B3, H3, L3, D3, LQ3 = 32, 30, 680, 64, 256
    gd = torch.Generator(device=dev).manual_seed(3003)
    k, v = (torch.randn(B3, H3, L3, D3, device=dev, generator=gd).bfloat16() for _ in range(2))
    q = torch.randn(B3, H3, LQ3, D3, device=dev, generator=gd).bfloat16()

    timed = lambda fn: timed_launches(torch, fn, reps, warm)

    out = {'workload': 'config 3: VAR-d30 K/V bf16 [32,30,680,64], one (scale, zp) per (head, channel); '
                       'final-scale 256 queries'}
    n_el = B3 * H3 * L3 * D3
    for name, bits, asym in (('int2_asym', 2, True), ('int8_sym', 8, False)):
        kw, ks, kz = ops.quant_pack(k, (0, 2), bits, asym)
        vw, vs, vz = ops.quant_pack(v, (0, 2), bits, asym)
        t_q = timed(lambda: ops.quant_pack(k, (0, 2), bits, asym))
        t_d = timed(lambda: ops.dequant(kw, ks, kz, D3, bits, torch.bfloat16))
        tab = lambda t: None if t is None else t.reshape(H3, D3).contiguous()
        o = torch.empty_like(q)
        t_a = timed(lambda: ops.fused_attn_channel(q, kw, tab(ks), tab(kz), vw, tab(vs), tab(vz), bits, L3,
                                                   1.0 / math.sqrt(D3), out=o))
        packed = n_el * bits // 8
        out[name] = {'quant_pack_us': round(t_q * 1e6, 1), 'quant_pack_GBps': round((n_el * 2 + packed) / t_q / 1e9, 1),
                     'unpack_dequant_us': round(t_d * 1e6, 1), 'unpack_dequant_GBps': round((packed + n_el * 2) / t_d / 1e9, 1),
                     'fused_attn_us': round(t_a * 1e6, 1),
                     'fused_attn_TFLOPs': round(4 * B3 * H3 * LQ3 * L3 * D3 / t_a / 1e12, 1)}
    return out


def prepare_rates(torch, dev):
    """Producer side in one pass (qkv_prepare_kernel): the qkv projection output of the last
    Infinity scale, bf16 [B=2, L=4096, 3, H=16, c=128] -> q normalised, scaled per head and
    rotated (bf16) and k, v normalised / rotated and quantized to INT4 group 128 into their cache
    rows.  Four input sets are cycled (4 x 101 MB)."""
    from var_q_amd import hooks, ops
    Bp, Lp, Hp, cp, bits, g = 2, 4096, 16, 128, 4, 128
    gd = torch.Generator(device=dev).manual_seed(6006)
    xs = [torch.randn(Bp, Lp, 3, Hp, cp, device=dev, generator=gd).bfloat16() for _ in range(4)]
    cos, sin = hooks.rope2d_tables(cp, [(64, 64)])
    rope = (cos.to(dev), sin.to(dev))
    mul = torch.rand(Hp, device=dev, generator=gd) + 1
    Wp = cp * bits // 32
    mk = lambda last, dt: torch.empty((Bp, Hp, Lp, last), dtype=dt, device=dev)
    t = dict(q=mk(cp, torch.bfloat16), kw=mk(Wp, torch.int32), vw=mk(Wp, torch.int32), ks=mk(1, torch.float32),
             kz=mk(1, torch.float32), vs=mk(1, torch.float32), vz=mk(1, torch.float32))
    rowmap = [Bp, Lp, Hp, Hp * Lp, 1, Lp, 0, -1]
    i = [0]

    def fn():
        i[0] += 1
        ops.qkv_prepare_append(xs[i[0] % 4], t['q'], g, bits, True, 1e-12, t['kw'], t['ks'], t['kz'], t['vw'], t['vs'], t['vz'],
                               rowmap, None, mul, True, 1e-12, rope, 0)
    dt = timed_launches(torch, fn, reps=40, warm=10)
    rows = Bp * Lp * Hp
    nbytes = rows * (3 * cp * 2 + cp * 2 + 2 * cp * bits // 8 + 2 * (cp // g) * 8)    # qkv in, q out, packed k and v, scales and zps
    return {'workload': 'qkv [2,4096,3,16,128] bf16 -> q bf16 (l2-norm, per-head scale, 2-D rotary) + k, v INT4 g128 into the cache',
            'us': round(dt * 1e6, 1), 'GBps': round(nbytes / dt / 1e9, 1), 'frac_hbm_peak': round(nbytes / dt / 1e9 / HBM_PEAK_GBPS, 4),
            'tokens_per_s': round(Bp * Lp / dt, 1), 'algorithmic_MB': round(nbytes / 1e6, 2)}


def pack_unpack_rates(torch, dev, token_major=True):
    """The pack and unpack kernels on their own (the reference's pack_last_dim_to_int32 /
    unpack_last_dim_from_int32 on int8 codes): configuration-4 shape [2,16,10521,128], INT4, INT2
    and INT8, 40 back-to-back launches through the C ABI between one event pair; four sets of
    source and destination buffers are cycled.  Bytes: the int8 codes plus the packed words, each moved once."""
    from var_q_amd import _lib
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    rows, c = B * H * L, D
    gd = torch.Generator(device=dev).manual_seed(7007)
    out = {'workload': 'int8 codes [2,16,10521,128] <-> packed int32 words, standalone pack / unpack kernels'}
    for bits in (4, 2, 8):
        lo, hi = -(1 << (bits - 1)), (1 << (bits - 1))
        codes = [torch.randint(lo, hi, (rows, c), device=dev, generator=gd, dtype=torch.int8) for _ in range(4)]
        words = [torch.empty((rows, c * bits // 32), dtype=torch.int32, device=dev) for _ in range(4)]
        back = [torch.empty((rows, c), dtype=torch.int8, device=dev) for _ in range(4)]
        i = [0]

        def pack():
            i[0] += 1
            _lib.check(lib.varq_pack(codes[i[0] % 4].data_ptr(), rows, c, bits, words[i[0] % 4].data_ptr(), stream), 'varq_pack')

        def unpack():
            i[0] += 1
            _lib.check(lib.varq_unpack(words[i[0] % 4].data_ptr(), rows, c, bits, back[i[0] % 4].data_ptr(), stream), 'varq_unpack')
        for j in range(4):
            i[0] = j - 1
            pack()
        t_p = timed_launches(torch, pack, reps=40, warm=8)
        t_u = timed_launches(torch, unpack, reps=40, warm=8)
        i[0] = 0
        unpack()
        torch.cuda.synchronize()
        assert torch.equal(back[1], codes[1]), 'pack -> unpack does not return the codes'
        nbytes = rows * c + rows * c * bits // 8
        out['int%d' % bits] = {'pack_us': round(t_p * 1e6, 1), 'pack_GBps': round(nbytes / t_p / 1e9, 1),
                               'pack_frac_hbm_peak': round(nbytes / t_p / 1e9 / HBM_PEAK_GBPS, 4),
                               'unpack_us': round(t_u * 1e6, 1), 'unpack_GBps': round(nbytes / t_u / 1e9, 1),
                               'unpack_frac_hbm_peak': round(nbytes / t_u / 1e9 / HBM_PEAK_GBPS, 4), 'algorithmic_MB': round(nbytes / 1e6, 2)}
        del codes, words, back
    if token_major:
        out['quantize_token_major_input'] = token_major_quantize_rate(torch, dev)
    return out


def token_major_quantize_rate(torch, dev):
    """The quantize+pack kernel on K and V in the order the Infinity block holds them,
    [B, L, H, c] = [2, 10521, 16, 128] (bf16), written into the head-major cache [B, H, L, ...]
    through a row map over (B, L, H): INT4 group 128 asymmetric, K and V in one launch, four
    input sets cycled.  Bytes: both inputs once, packed words, scales and zero-points once."""
    from var_q_amd import ops
    gd = torch.Generator(device=dev).manual_seed(8008)
    W = D * BITS // 32
    xs = [(torch.randn(B, L, H, D, device=dev, generator=gd).bfloat16(), torch.randn(B, L, H, D, device=dev, generator=gd).bfloat16())
          for _ in range(4)]
    mk = lambda last, dt: torch.empty((B, H, L, last), dtype=dt, device=dev)
    outs = [[(mk(W, torch.int32), mk(D // GROUP, torch.float32), mk(D // GROUP, torch.float32)) for _ in range(2)] for _ in range(4)]
    rowmap = [B, L, H, H * L, 1, L, 0, -1]
    i = [0]

    def fn():
        i[0] += 1
        k, v = xs[i[0] % 4]
        o = outs[i[0] % 4]
        ops.quant_pack_rows_pair_into(k, v, GROUP, BITS, True, 1e-12, o[0], o[1], rowmap, None)
    dt = timed_launches(torch, fn, reps=40, warm=8)
    # the same values in head-major order must give the same cache
    k, v = xs[1]
    ref = ops.quant_pack_rows(k.transpose(1, 2).contiguous(), GROUP, BITS, True)
    i[0] = 0
    fn()
    torch.cuda.synchronize()
    same = all(torch.equal(a, b) for a, b in zip(ref, outs[1][0]))
    nbytes = 2 * (B * H * L * D * 2 + B * H * L * (W * 4 + 2 * (D // GROUP) * 4))
    return {'workload': 'K and V [2,10521,16,128] bf16 (token-major) -> INT4 g128 in the head-major cache, one launch',
            'us': round(dt * 1e6, 1), 'GBps': round(nbytes / dt / 1e9, 1), 'frac_hbm_peak': round(nbytes / dt / 1e9 / HBM_PEAK_GBPS, 4),
            'algorithmic_MB': round(nbytes / 1e6, 2), 'equals_head_major_input': bool(same)}


def shipped_rule_latency(torch, dev, passes=5, warm=2):
    """The rules of the shipped JSON files (G_SCALE_HEAD_DIM, 8 bits), one layer, per scale
    quantize + cache K and V with the drop-in quantizers, then attend:
    Infinity-VAR_Q-8.json (layout BHLc) over the 13 Infinity scales, B=2 (one image, CFG pair),
    H=16, D=128; VAR-VAR_Q-8.json (layout BLHc) over the 10 VAR scales, B=64, H=16, D=64.
    'dropin' dequantizes the whole cache to fp32 and calls torch's
    scaled_dot_product_attention in bf16 (what the reference does), 'fused' quantizes, caches and
    attends over the packed caches (`fused_step`)."""
    import torch.nn.functional as F
    from var_q_amd import VAR_Q
    from var_q_amd.quant import fused_step
    from var_q_amd.schedules import INFINITY_PATCH_NUMS, VAR_PATCH_NUMS

    def run(fmt, B, H, D, patch_nums, seed):
        gd = torch.Generator(device=dev).manual_seed(seed)
        shape = (lambda n: (B, H, n, D)) if fmt == 'BHLc' else (lambda n: (B, n, H, D))
        steps = [tuple(torch.randn(*shape(pn * pn), device=dev, generator=gd).bfloat16() for _ in range(3))
                 for pn in patch_nums]
        scale = 1.0 / math.sqrt(D)
        total = sum(pn * pn for pn in patch_nums)
        heads_first = (lambda t: t) if fmt == 'BHLc' else (lambda t: t.transpose(1, 2))

        def one_pass(fused):
            kq, vq = VAR_Q(8, fmt, 'G_SCALE_HEAD_DIM'), VAR_Q(8, fmt, 'G_SCALE_HEAD_DIM')
            for quantizer in (kq, vq):            # (both paths: the cache buffers never have to grow)
                quantizer.reserve_tokens(total)
            for q, k, v in steps:
                if fused:
                    fused_step(q, k, v, kq, vq, scale)
                else:
                    kk, vv = kq.use_var_q(k), vq.use_var_q(v)
                    F.scaled_dot_product_attention(heads_first(q), heads_first(kk.to(torch.bfloat16)),
                                                   heads_first(vv.to(torch.bfloat16)), scale=scale)

        res = {}
        for name, fused in (('dropin_dequant_sdpa_ms', False), ('fused_ms', True)):
            warm_passes(torch, lambda: one_pass(fused), warm)
            t0 = time.perf_counter()
            for _ in range(passes):
                one_pass(fused)
            torch.cuda.synchronize()
            res[name] = round((time.perf_counter() - t0) / passes * 1e3, 3)
        # the fused pass recorded once into a HIP graph and replayed: the library launches kernels
        # only, so what is left of the host's share of a pass goes away
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            one_pass(True)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            one_pass(True)
        warm_passes(torch, graph.replay, warm)
        t0 = time.perf_counter()
        for _ in range(2 * passes):
            graph.replay()
        torch.cuda.synchronize()
        res['fused_graph_replay_ms'] = round((time.perf_counter() - t0) / (2 * passes) * 1e3, 3)
        del graph
        return res

    out = {'workload': 'shipped rule G_SCALE_HEAD_DIM 8-bit BHLc, 13 Infinity scales, B=2 H=16 D=128, one layer: '
                       'quantize + cache + attention per scale'}
    out.update(run('BHLc', 2, 16, 128, INFINITY_PATCH_NUMS, 7007))
    out['var_d16'] = {'workload': 'shipped rule G_SCALE_HEAD_DIM 8-bit BLHc, 10 VAR scales, B=64 H=16 D=64, one layer'}
    out['var_d16'].update(run('BLHc', 64, 16, 64, VAR_PATCH_NUMS, 7008))
    return out


def hbm_regime_rates(torch, dev, kv_sets):
    """The regime in which the metric's "KV-read fraction of HBM peak" is a bound: a few queries
    over the whole packed cache of configuration 4 (INT4 group 128, B=2, H=16, 10 521 keys),
    Lq = 16 and 64, where the arithmetic intensity (4 * Lq flop per packed byte) is below or near
    the machine balance.  The four packed caches of the timed steps are cycled (4 x 48.5 MB of
    codes, scales and zero-points), so the reads come from HBM.  Reports the time, the packed-KV
    GB/s and its fraction of the 8 TB/s peak, and how the keys were shared out."""
    from var_q_amd import _lib, ops
    lib = _lib.load()
    _, kv_bytes, _ = algorithmic_bytes()
    out = {'workload': 'INT4 g128 packed cache of configuration 4 [B=2,H=16,Lk=10521,D=128]; Lq queries per (batch, head) '
                       'over all keys, 4 packed caches cycled', 'kv_MB': round(kv_bytes / 1e6, 2)}
    gd = torch.Generator(device=dev).manual_seed(8008)
    scale = 1.0 / math.sqrt(D)
    for lq in (16, 64):
        q = torch.randn(B, H, lq, D, device=dev, generator=gd).bfloat16()
        o = torch.empty_like(q)
        i = [0]

        def fn():
            t = kv_sets[i[0] % len(kv_sets)]
            i[0] += 1
            ops.fused_attn(q, t['kw'], t['ks'], t['kz'], t['vw'], t['vs'], t['vz'], BITS, BITS, L, scale, out=o)
        dt = timed_launches(torch, fn, reps=40, warm=8)
        flops = 4 * B * H * lq * L * D
        out['Lq%d' % lq] = {'us': round(dt * 1e6, 1), 'kv_read_GBps': round(kv_bytes / dt / 1e9, 1),
                            'kv_read_frac_hbm_peak': round(kv_bytes / dt / 1e9 / HBM_PEAK_GBPS, 4),
                            'TFLOPs': round(flops / dt / 1e12, 1),
                            'key_shares': int(lib.varq_fused_attn_key_shares(B, H, lq, L, D, GROUP, GROUP))}
    # the same 16 queries over a cache four times as long (synthetic, same format): how the rate
    # grows once the costs that do not depend on the cache length weigh less
    L4 = 4 * L
    long_sets = []
    for _ in range(4):
        k4, v4 = (torch.randn(B, H, L4, D, device=dev, generator=gd).bfloat16() for _ in range(2))
        (kw, ks, kz), (vw, vs, vz) = ops.quant_pack_rows(k4, GROUP, BITS, True), ops.quant_pack_rows(v4, GROUP, BITS, True)
        long_sets.append((kw, ks, kz, vw, vs, vz))
        del k4, v4
    q = torch.randn(B, H, 16, D, device=dev, generator=gd).bfloat16()
    o = torch.empty_like(q)
    j = [0]

    def fn4():
        t = long_sets[j[0] % 4]
        j[0] += 1
        ops.fused_attn(q, *t, BITS, BITS, L4, scale, out=o)
    dt = timed_launches(torch, fn4, reps=40, warm=8)
    out['Lq16_four_times_the_keys'] = {'keys': L4, 'kv_MB': round(4 * kv_bytes / 1e6, 2), 'us': round(dt * 1e6, 1),
                                       'kv_read_GBps': round(4 * kv_bytes / dt / 1e9, 1),
                                       'kv_read_frac_hbm_peak': round(4 * kv_bytes / dt / 1e9 / HBM_PEAK_GBPS, 4),
                                       'key_shares': int(lib.varq_fused_attn_key_shares(B, H, 16, L4, D, GROUP, GROUP))}
    del long_sets
    # and over an INT8 group-128 cache of configuration 4's shape (twice the bytes per key, the same number of codes)
    sets8 = []
    for _ in range(4):
        k8, v8 = (torch.randn(B, H, L, D, device=dev, generator=gd).bfloat16() for _ in range(2))
        sets8.append((*ops.quant_pack_rows(k8, GROUP, 8, True), *ops.quant_pack_rows(v8, GROUP, 8, True)))
        del k8, v8
    kv8 = 2 * (B * H * L * D + B * H * L * (D // GROUP) * 8)
    j[0] = 0

    def fn8():
        t = sets8[j[0] % 4]
        j[0] += 1
        ops.fused_attn(q, *t, 8, 8, L, scale, out=o)
    dt = timed_launches(torch, fn8, reps=40, warm=8)
    out['Lq16_int8_cache'] = {'kv_MB': round(kv8 / 1e6, 2), 'us': round(dt * 1e6, 1), 'kv_read_GBps': round(kv8 / dt / 1e9, 1),
                              'kv_read_frac_hbm_peak': round(kv8 / dt / 1e9 / HBM_PEAK_GBPS, 4),
                              'key_shares': int(lib.varq_fused_attn_key_shares(B, H, 16, L, D, GROUP, GROUP))}
    del sets8
    out['config5_early_scales'] = c5_early_scales(torch, dev)
    return out


def c5_early_scales(torch, dev):
    """Configuration 5's scales of at most 64 queries (patch numbers 1, 2, 4, 6, 8 at B=8, H=16, mixed widths, group 64):
    the attention call of each scale over its prefix of the packed cache, the three bit-width classes side by side.  These
    caches are short (1 to 121 keys, 0.03 to 3.6 MB of packed K/V), so the calls are bound by launch latency, not by HBM:
    the figures say how far."""
    from var_q_amd import PackedKVCache
    from var_q_amd.schedules import INFINITY_PATCH_NUMS
    bits = c5_head_bits(torch)
    ns = [pn * pn for pn in INFINITY_PATCH_NUMS if pn * pn <= 64]
    cache = PackedKVCache(C5_B, C5_H, sum(ns), C5_D, bits, C5_GROUP, dev)
    gd = torch.Generator(device=dev).manual_seed(5006)
    res = {}
    for n in ns:
        q, k, v = (torch.randn(C5_B, C5_H, n, C5_D, device=dev, generator=gd).bfloat16() for _ in range(3))
        cache.append(k, v)
        o = torch.empty_like(q)
        dt = timed_launches(torch, lambda: cache.attend(q, 1.0 / math.sqrt(C5_D), out=o), reps=20, warm=5)
        kv = sum(2 * C5_B * cache.len * (C5_D * b // 8 + (C5_D // C5_GROUP) * 8) for b in bits)
        res['Lq%d_Lk%d' % (n, cache.len)] = {'us': round(dt * 1e6, 1), 'kv_MB': round(kv / 1e6, 3), 'kv_read_GBps': round(kv / dt / 1e9, 1),
                                             'kv_read_frac_hbm_peak': round(kv / dt / 1e9 / HBM_PEAK_GBPS, 5)}
    return res


def attention_check(torch, dev, out, q, kd, vd, ref, scale):
    """The timed attention output against the oracle (cosine) and against an fp64 evaluation of
    the same formula on the oracle's dequantized operands (max-abs in units of the output
    range), as the parity tests do; the fp64 softmax runs through torch on the GPU, one head at
    a time (checker plumbing)."""
    got = out.double().cpu()
    refd = ref.double()
    exact = torch.empty_like(refd)
    for b in range(q.shape[0]):
        for h in range(q.shape[1]):
            s = (q[b, h].double().to(dev) @ kd[b, h].double().to(dev).T) * scale
            exact[b, h] = (torch.softmax(s, dim=-1) @ vd[b, h].double().to(dev)).cpu()
    span = max(1.0, float(exact.abs().max()))
    return {
        'attn_cosine_vs_oracle': round(float(torch.nn.functional.cosine_similarity(got.flatten(), refd.flatten(), dim=0)), 6),
        'attn_output_range': round(span, 3),
        'attn_maxabs_vs_fp64_over_range': round(float((got - exact).abs().max()) / span, 5),
        'oracle_maxabs_vs_fp64_over_range': round(float((refd - exact).abs().max()) / span, 5),
        'attn_maxabs_vs_oracle_over_range': round(float((got - refd).abs().max()) / span, 5),
        'queries_checked': int(q.shape[2]),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=20)
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg (profiling runs)')
    ap.add_argument('--no-c2', action='store_true', help='skip the config-2 rates leg (profiling runs)')
    ap.add_argument('--no-c5', action='store_true', help='skip the config-5 latency leg (profiling runs)')
    ap.add_argument('--no-c3', action='store_true', help='skip the config-3 rates leg (profiling runs)')
    ap.add_argument('--single-launches', action='store_true', help='quantize K and V in two launches instead of one')
    ap.add_argument('--no-rule', action='store_true', help='skip the shipped-rule latency leg (profiling runs)')
    ap.add_argument('--no-prepare', action='store_true', help='skip the producer-side (qkv_prepare) leg (profiling runs)')
    ap.add_argument('--no-hbm', action='store_true', help='skip the few-queries-over-a-long-cache leg (profiling runs)')
    ap.add_argument('--no-pack', action='store_true', help='skip the standalone pack / unpack leg (profiling runs)')
    ap.add_argument('--no-token-major', action='store_true',
                    help='skip the token-major quantize leg (profiling runs: its launches are the headline pack kernel on the same grid)')
    ap.add_argument('--calib', action='store_true',
                    help='also launch a plain 256 MiB device copy 4 times: known traffic to scale the rocprofv3 '
                         'FETCH_SIZE / WRITE_SIZE counters by')
    ap.add_argument('--fixed-prewarm', action='store_true',
                    help='warm the secondary legs up by launch count instead of by time, so that the launches of '
                         'separate profiling runs can be matched by their order')
    args = ap.parse_args()
    if args.fixed_prewarm:
        global PREWARM_MS
        PREWARM_MS = 0.0
    if args.gpus != 1:
        print('bench.py measures one GPU: this path has no collectives and is not sharded; '
              'run with --gpus 1 (got --gpus %d)' % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    import varq_oracle as O
    from var_q_amd import _lib, ops
    assert torch.cuda.is_available(), 'bench.py needs a GPU'
    _lib.load()   # raises if the HIP library is missing: no fallback
    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)

    quant_bytes, kv_bytes, attn_flops = algorithmic_bytes()
    scale = 1.0 / math.sqrt(D)

    # ---- synthetic inputs (seeds as for the parity tests) --------------------
    k0 = O.synth_kv((B, H, L, D), 1004, 'student4', 0.01, 20.0, torch.bfloat16, outlier_seed=4004)
    v0 = O.synth_kv((B, H, L, D), 2004, 'student4', 0.01, 20.0, torch.bfloat16, outlier_seed=4004)
    q0 = torch.randn(B, H, LQ, D, generator=torch.Generator().manual_seed(3004)).bfloat16()
    ks_in, vs_in = [k0.to(dev)], [v0.to(dev)]
    for i in range(1, NBUF):   # further sets: same distribution, different memory and values
        ks_in.append(torch.roll(ks_in[0], shifts=i * 977, dims=2).contiguous())
        vs_in.append(torch.roll(vs_in[0], shifts=i * 977, dims=2).contiguous())
    q = q0.to(dev)

    W = D * BITS // 32
    mk = lambda last, dt: torch.empty((B, H, L, last), dtype=dt, device=dev)
    outs = [dict(kw=mk(W, torch.int32), ks=mk(1, torch.float32), kz=mk(1, torch.float32),
                 vw=mk(W, torch.int32), vs=mk(1, torch.float32), vz=mk(1, torch.float32)) for _ in range(NBUF)]
    o = torch.empty_like(q)
    rowmap = [1, 1, B * H * L, 0, 0, 1, 0, -1]

    PAIR = not args.single_launches

    def quantize(i):
        s, t = i % NBUF, outs[i % NBUF]
        if PAIR:   # K and V of the step in one launch, as the cache append does
            ops.quant_pack_rows_pair_into(ks_in[s], vs_in[s], GROUP, BITS, True, 1e-12, (t['kw'], t['ks'], t['kz']),
                                          (t['vw'], t['vs'], t['vz']), rowmap)
        else:
            ops.quant_pack_rows_into(ks_in[s], GROUP, BITS, True, 1e-12, t['kw'], t['ks'], t['kz'], rowmap)
            ops.quant_pack_rows_into(vs_in[s], GROUP, BITS, True, 1e-12, t['vw'], t['vs'], t['vz'], rowmap)

    def step(i, ev=None):
        t = outs[i % NBUF]
        if ev: ev[0].record()
        quantize(i)
        if ev: ev[1].record()
        ops.fused_attn(q, t['kw'], t['ks'], t['kz'], t['vw'], t['vs'], t['vz'], BITS, BITS, L, scale, out=o)
        if ev: ev[2].record()

    if args.calib:
        ca = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        cb = torch.empty_like(ca)
        for _ in range(4):
            cb.copy_(ca)          # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del ca, cb

    # clocks: the same step, untimed, until 150 ms of GPU work have passed
    prewarm_steps, e0 = 0, torch.cuda.Event(enable_timing=True)
    e0.record()
    while True:
        for _ in range(20):
            step(prewarm_steps)
            prewarm_steps += 1
        e1 = torch.cuda.Event(enable_timing=True)
        e1.record()
        torch.cuda.synchronize()
        if e0.elapsed_time(e1) >= 150.0 or prewarm_steps >= 2000:
            break
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()

    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i, events[i])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps

    # events sit on the stream the kernels are launched on (torch's current stream)
    t_quant_step = sum(e[0].elapsed_time(e[1]) for e in events) / args.steps * 1e-3 / 2   # per tensor, dispatch gap included
    t_at = sum(e[1].elapsed_time(e[2]) for e in events) / args.steps * 1e-3

    # ---- the HBM-bound kernels of configuration 4 as back-to-back launches between one event pair:
    #      kernel time without the gap between a recorded event and the next dispatch
    cnt = [0]

    def quantize_next():
        quantize(cnt[0])
        cnt[0] += 1
    t_quant = timed_launches(torch, quantize_next, reps=40, warm=8) / 2          # per tensor
    deq_out = torch.empty((B, H, L, D), dtype=torch.bfloat16, device=dev)
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    shape4, strides4 = _lib.i64arr([B, H, L, D]), _lib.i64arr([H * L, L, 1, 1])

    def dequant_next():   # the C ABI directly: no allocation and no Python wrapper between the launches
        t = outs[cnt[0] % NBUF]
        cnt[0] += 1
        _lib.check(lib.varq_dequant(t['kw'].data_ptr(), None, t['ks'].data_ptr(), t['kz'].data_ptr(), shape4, strides4,
                                    GROUP, BITS, None, deq_out.data_ptr(), 1, stream), 'varq_dequant')
    for i in range(NBUF):
        quantize(i)
    t_deq = timed_launches(torch, dequant_next, reps=40, warm=8)
    # the attention in its two operand forms, back-to-back launches on the same packed cache:
    # reference rounding (the default: what the timed steps ran) and exact codes (the opt-in)
    t0_ = outs[0]
    o_exact = torch.empty_like(q)
    attn_args = (q, t0_['kw'], t0_['ks'], t0_['kz'], t0_['vw'], t0_['vs'], t0_['vz'], BITS, BITS, L, scale)
    t_at_ref = timed_launches(torch, lambda: ops.fused_attn(*attn_args, out=o), reps=20, warm=5)
    t_at_exact = timed_launches(torch, lambda: ops.fused_attn(*attn_args, out=o_exact, exact_codes=True), reps=20, warm=5)
    n = B * H * L * D
    deq_bytes = n * BITS // 8 + (n // GROUP) * 8 + n * 2           # packed codes + scale/zp in, bf16 out

    # ---- CPU baseline + parity of the timed results against it ------------------
    cpu = None
    checked = None
    if not args.no_cpu:
        threads = min(os.cpu_count() or 1, int(os.environ.get('OMP_NUM_THREADS', os.cpu_count() or 1)))
        step(0)
        torch.cuda.synchronize()
        stages, c = cpu_baseline(torch, O, k0, v0, q0, threads)
        t = outs[0]
        words_ok = bool(torch.equal(t['kw'].cpu(), c['kw']) and torch.equal(t['vw'].cpu(), c['vw'])
                        and torch.equal(t['ks'].cpu(), c['ks']) and torch.equal(t['kz'].cpu(), c['kz'])
                        and torch.equal(t['vs'].cpu(), c['vs']) and torch.equal(t['vz'].cpu(), c['vz']))
        cnt[0] = 0            # input set 0 again: the one the CPU leg dequantized
        dequant_next()
        torch.cuda.synchronize()
        deq_ok = bool(torch.equal(deq_out.cpu(), c['kd'].bfloat16()))
        checked = {'packed_words_scales_zps_bit_exact': words_ok, 'unpack_dequant_bf16_bit_exact': deq_ok}
        checked.update(attention_check(torch, dev, o, q0, c['kd'], c['vd'], c['ref'], scale))
        # the default form is held to the oracle alone: max-abs <= 2e-2 x range, cosine >= 0.9995
        bad = (not words_ok or not deq_ok or checked['attn_cosine_vs_oracle'] < 0.9995
               or checked['attn_maxabs_vs_oracle_over_range'] > 2e-2)
        # the opt-in exact-code form does not round K and V as the reference does: it is held to the
        # fp64 value of the same formula, and to the oracle within the oracle's own distance from it
        ops.fused_attn(*attn_args, out=o_exact, exact_codes=True)
        torch.cuda.synchronize()
        ex = attention_check(torch, dev, o_exact, q0, c['kd'], c['vd'], c['ref'], scale)
        checked['exact_codes_form'] = {k_: ex[k_] for k_ in ('attn_cosine_vs_oracle', 'attn_maxabs_vs_fp64_over_range',
                                                             'attn_maxabs_vs_oracle_over_range')}
        bad = bad or (ex['attn_cosine_vs_oracle'] < 0.9995 or ex['attn_maxabs_vs_fp64_over_range'] > 2e-2
                      or ex['attn_maxabs_vs_oracle_over_range'] > 2e-2 + ex['oracle_maxabs_vs_fp64_over_range'])
        if bad:
            print('bench.py: GPU results differ from the oracle: %r' % checked, file=sys.stderr)
            sys.exit(1)
        a = stages['all_threads']
        t_cpu_attn = a['unpack_dequant_s_both'] + a['attention_s_4096_queries']
        cpu = {
            'value': round(kv_bytes / t_cpu_attn / 1e9, 4), 'unit': 'GB/s', 'cores': threads, 'kind': 'port',
            'cpu_model': cpu_model(), 'os_cpu_count': os.cpu_count(),
            'sample': ('torch-CPU oracle on this host, median of 3 runs per stage: full-size INT4 g128 quantize+pack of K and '
                       'V, unpack+dequant of both, bf16 attention of all 4096 queries (one thread: 512 queries scaled x8); '
                       'value = packed-KV bytes / (unpack+dequant + attention) with all threads'),
            'pack_GBps': round(quant_bytes / a['quant_pack_s_per_tensor'] / 1e9, 3),
            'stages': stages,
        }

    attn_tflops = attn_flops / t_at / 1e12
    kv_gbps = kv_bytes / t_at / 1e9
    pack_gbps = quant_bytes / t_quant / 1e9
    traffic = None
    tf = os.path.join(ROOT, 'profiles', 'traffic.json')   # HBM bytes per launch from the rocprofv3 --pmc runs
    if os.path.exists(tf):
        try:
            traffic = json.load(open(tf))
        except Exception:
            traffic = None
    line = {
        'metric': 'fused dequant-attn KV-read GB/s (%HBM peak) + pack GB/s, Infinity-2B shape',
        'value': round(kv_gbps, 3), 'unit': 'GB/s',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(ms_per_step, 4),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'bf16', 'dtype_detail': 'K and V dequantized in fp32 and rounded to bf16 as tiles enter LDS (the operands the '
                                         "reference's attention sees), bf16 MFMA, fp32 softmax and accumulation", 'data': 'synthetic',
        'config': {'workload': 'config 4: Infinity-2B KV [B=2,H=16,L=10521,D=128] bf16 -> INT4 group-128 asymmetric '
                               'quantize+pack of K and V, then fused dequant attention of the final 4096 queries',
                   'B': B, 'H': H, 'L': L, 'D': D, 'Lq': LQ, 'bits': BITS, 'group': GROUP, 'input_sets_cycled': NBUF,
                   'prewarm_steps_untimed': prewarm_steps},
        'attn_kv_read_frac_hbm_peak': round(kv_gbps / HBM_PEAK_GBPS, 5),
        'attn_ms': round(t_at * 1e3, 4), 'attn_TFLOPs': round(attn_tflops, 2),
        'attn_forms': {'reference_rounding_ms': round(t_at_ref * 1e3, 4), 'exact_codes_ms': round(t_at_exact * 1e3, 4),
                       'default': 'reference_rounding',
                       'timing': '20 back-to-back launches between one HIP event pair, median of 5; attn_ms is the default form '
                                 'inside the timed steps'},
        'attn_query_tokens_per_s': round(B * LQ / t_at, 1),
        'pack_GBps': round(pack_gbps, 2), 'pack_frac_hbm_peak': round(pack_gbps / HBM_PEAK_GBPS, 4),
        'pack_us_per_tensor': round(t_quant * 1e6, 2), 'pack_tokens_per_s': round(B * L / t_quant, 1),
        'pack_us_per_tensor_in_step': round(t_quant_step * 1e6, 2),
        'unpack_dequant_GBps': round(deq_bytes / t_deq / 1e9, 2), 'unpack_dequant_frac_hbm_peak': round(deq_bytes / t_deq / 1e9 / HBM_PEAK_GBPS, 4),
        'unpack_dequant_us_per_tensor': round(t_deq * 1e6, 2),
        'roofline': {'kernel': 'fused_attn_kernel<128,4,128,128,token scales, reference rounding>', 'bound': 'mfma', 'achieved': round(attn_tflops, 2),
                     'peak': MFMA_BF16_PEAK_TFLOPS, 'unit': 'TFLOP/s', 'frac': round(attn_tflops / MFMA_BF16_PEAK_TFLOPS, 4),
                     'traffic': None if not traffic else traffic.get('fused_attn'),
                     'timing': 'HIP events around each of the timed steps\' launches'},
        'roofline_pack': {'kernel': 'quant_pack_rows32_kernel<bf16,4,asym,4 lanes per group,dense>', 'bound': 'hbm', 'achieved': round(pack_gbps, 2),
                          'peak': HBM_PEAK_GBPS, 'unit': 'GB/s', 'frac': round(pack_gbps / HBM_PEAK_GBPS, 4),
                          'traffic': None if not traffic else traffic.get('quant_pack_rows', 0) // (1 if PAIR else 2) or None,
                          'tensors_per_launch': 2 if PAIR else 1,
                          'timing': '40 back-to-back launches over the %d cycled input sets between one HIP event pair, median '
                                    'of 5 (inside the timed steps, one launch between its own events: '
                                    'pack_us_per_tensor_in_step)' % NBUF},
        'roofline_dequant': {'kernel': 'dequant_kernel<int4 words, group 128, bf16 out>', 'bound': 'hbm',
                             'achieved': round(deq_bytes / t_deq / 1e9, 2), 'peak': HBM_PEAK_GBPS, 'unit': 'GB/s',
                             'frac': round(deq_bytes / t_deq / 1e9 / HBM_PEAK_GBPS, 4),
                             'traffic': None if not traffic else traffic.get('dequant'),
                             'timing': '40 back-to-back launches through the C ABI between one HIP event pair, median of 5'},
        'cpu_baseline': cpu, 'checked_against_oracle': checked,
        'hbm_regime_rates': None if args.no_hbm else hbm_regime_rates(torch, dev, outs),
        'config2_rates': None if args.no_c2 else c2_rates(torch, dev),
        'config5_latency': None if args.no_c5 else c5_latency(torch, dev, check=not args.no_cpu),
        'config3_rates': None if args.no_c3 else c3_rates(torch, dev),
        'qkv_prepare_rates': None if args.no_prepare else prepare_rates(torch, dev),
        'pack_unpack_rates': None if args.no_pack else pack_unpack_rates(torch, dev, not args.no_token_major),
        'shipped_rule_latency': None if args.no_rule else shipped_rule_latency(torch, dev),
    }
    print(json.dumps(line), flush=True)


if __name__ == '__main__':
    main()

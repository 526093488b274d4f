#!/usr/bin/env python3
"""Benchmark of the VAR-Q hot path on one MI355X.

One step = one pass over benchmark configuration 4 (Infinity-2B shape): quantize+pack K
and V [2,16,10521,128] bf16 to INT4 group-128 asymmetric, then fused dequant
attention of the final scale's 4096 queries over all 10521 packed keys.  Inputs
are resident in HBM before the timed region.  Prints ONE JSON line.

After the timed region (and outside `value`) it also replays benchmark configuration 5,
one image batch of the Infinity schedule through the pre-allocated mixed-bit
cache (append + attend per scale), and reports its latency per image.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-c5] [--no-c3] [--no-rule]
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


def cpu_baseline(torch, O, k0, v0, q0, threads):
    """The CPU oracle timed on this host: full-size quantize+pack of K and V,
    unpack+dequant of both, and bf16 SDPA on a 512-query sample (scaled x8)."""
    torch.set_num_threads(threads)
    t0 = time.perf_counter()
    kq, ks, kz = O.quant_groupwise(k0, GROUP, BITS, True)
    kw, kmeta = O.pack_last_dim(kq, BITS)
    t1 = time.perf_counter()
    vq, vs, vz = O.quant_groupwise(v0, GROUP, BITS, True)
    vw, vmeta = O.pack_last_dim(vq, BITS)
    t2 = time.perf_counter()
    kd = O.dequant_groupwise(O.unpack_last_dim(kw, kmeta), ks, kz, GROUP)
    vd = O.dequant_groupwise(O.unpack_last_dim(vw, vmeta), vs, vz, GROUP)
    t3 = time.perf_counter()
    nq = 512
    ref = O.attention_ref(q0[:, :, :nq], kd, vd, 1.0 / math.sqrt(D))
    t4 = time.perf_counter()
    t_quant = (t2 - t0) / 2
    t_attn = (t3 - t2) + (t4 - t3) * (LQ / nq)
    return {'kw': kw, 'ks': ks, 'kz': kz, 'vw': vw, 'ref': ref, 'nq': nq,
            't_quant_pack_per_tensor_s': t_quant, 't_unpack_dequant_s': t3 - t2, 't_sdpa_sample_s': t4 - t3,
            't_attn_equiv_s': t_attn}


def c5_latency(torch, dev, passes=10, warm=3):
    """Config 5: B=8 (4 images x CFG pair), H=16, D=128, the 13 Infinity scales; heads carry
    2/4/8-bit codes (seeded), group 64 asymmetric.  Per scale: quantize+pack the step's K and V
    in place into the pre-allocated cache, then fused attention of that scale's queries over
    the prefix.  Returns seconds per pass (all scales, one layer)."""
    from var_q_amd import PackedKVCache
    from var_q_amd.schedules import INFINITY_PATCH_NUMS
    B5, H5, D5 = 8, 16, 128
    ns = [pn * pn for pn in INFINITY_PATCH_NUMS]
    g = torch.Generator().manual_seed(5000)
    bits = [(2, 4, 8)[int(i)] for i in torch.randint(0, 3, (H5,), generator=g)]
    cache = PackedKVCache(B5, H5, sum(ns), D5, bits, 64, dev)
    gd = torch.Generator(device=dev).manual_seed(5005)
    steps = [tuple(torch.randn(B5, H5, n, D5, device=dev, generator=gd).bfloat16() for _ in range(3)) for n in ns]
    outs = [torch.empty_like(s[0]) for s in steps]
    def one_pass():
        cache.reset()
        for (q, k, v), o in zip(steps, outs):
            cache.append(k, v)
            cache.attend(q, 1.0 / math.sqrt(D5), out=o)
    for _ in range(warm):
        one_pass()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(passes):
        one_pass()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / passes
    flops = sum(4 * B5 * H5 * n * sum(ns[:i + 1]) * D5 for i, n in enumerate(ns))
    return {'workload': 'config 5: 13-scale Infinity schedule, B=8 H=16 D=128, per-head bits %s, group 64 asymmetric, '
                        'in-place append + fused attention per scale, one layer' % ''.join(str(b) for b in bits),
            'ms_per_layer_pass': round(dt * 1e3, 4), 'ms_per_image_per_layer': round(dt * 1e3 / 4, 4),
            'attn_TFLOPs_incl_append': round(flops / dt / 1e12, 2), 'passes': passes}


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

    def timed(fn):
        for _ in range(warm):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps * 1e-3

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
            for _ in range(warm):
                one_pass(fused)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(passes):
                one_pass(fused)
            torch.cuda.synchronize()
            res[name] = round((time.perf_counter() - t0) / passes * 1e3, 3)
        return res

    out = {'workload': 'shipped rule G_SCALE_HEAD_DIM 8-bit BHLc, 13 Infinity scales, B=2 H=16 D=128, one layer: '
                       'quantize + cache + attention per scale'}
    out.update(run('BHLc', 2, 16, 128, INFINITY_PATCH_NUMS, 7007))
    out['var_d16'] = {'workload': 'shipped rule G_SCALE_HEAD_DIM 8-bit BLHc, 10 VAR scales, B=64 H=16 D=64, one layer'}
    out['var_d16'].update(run('BLHc', 64, 16, 64, VAR_PATCH_NUMS, 7008))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=20)
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg (profiling runs)')
    ap.add_argument('--no-c5', action='store_true', help='skip the config-5 latency leg (profiling runs)')
    ap.add_argument('--no-c3', action='store_true', help='skip the config-3 rates leg (profiling runs)')
    ap.add_argument('--single-launches', action='store_true', help='quantize K and V in two launches instead of one')
    ap.add_argument('--no-rule', action='store_true', help='skip the shipped-rule latency leg (profiling runs)')
    ap.add_argument('--calib', action='store_true',
                    help='also launch a plain 256 MiB device copy 4 times: known traffic to scale the rocprofv3 '
                         'FETCH_SIZE / WRITE_SIZE counters by')
    args = ap.parse_args()
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

    def step(i, ev=None):
        s, t = i % NBUF, outs[i % NBUF]
        if ev: ev[0].record()
        if PAIR:   # K and V of the step in one launch, as the cache append does
            ops.quant_pack_rows_pair_into(ks_in[s], vs_in[s], GROUP, BITS, True, 1e-12, (t['kw'], t['ks'], t['kz']),
                                          (t['vw'], t['vs'], t['vz']), rowmap)
        else:
            ops.quant_pack_rows_into(ks_in[s], GROUP, BITS, True, 1e-12, t['kw'], t['ks'], t['kz'], rowmap)
            ops.quant_pack_rows_into(vs_in[s], GROUP, BITS, True, 1e-12, t['vw'], t['vs'], t['vz'], rowmap)
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
    t_quant = sum(e[0].elapsed_time(e[1]) for e in events) / args.steps * 1e-3 / 2   # two launches (K, V) per step
    t_at = sum(e[1].elapsed_time(e[2]) for e in events) / args.steps * 1e-3

    # ---- CPU baseline + parity of the timed results against it ------------------
    cpu = None
    checked = None
    if not args.no_cpu:
        threads = min(os.cpu_count() or 1, int(os.environ.get('OMP_NUM_THREADS', os.cpu_count() or 1)))
        step(0)
        torch.cuda.synchronize()
        c = cpu_baseline(torch, O, k0, v0, q0, threads)
        t = outs[0]
        words_ok = bool(torch.equal(t['kw'].cpu(), c['kw']) and torch.equal(t['vw'].cpu(), c['vw'])
                        and torch.equal(t['ks'].cpu(), c['ks']) and torch.equal(t['kz'].cpu(), c['kz']))
        got, ref = o[:, :, :c['nq']].double().cpu(), c['ref'].double()
        cosine = float(torch.nn.functional.cosine_similarity(got.flatten(), ref.flatten(), dim=0))
        checked = {'packed_words_scales_zps_bit_exact': words_ok, 'attn_cosine_vs_oracle': round(cosine, 6)}
        if not words_ok or cosine < 0.9995:
            print('bench.py: GPU results differ from the oracle: %r' % checked, file=sys.stderr)
            sys.exit(1)
        cpu = {
            'value': round(kv_bytes / c['t_attn_equiv_s'] / 1e9, 4), 'unit': 'GB/s', 'cores': threads, 'kind': 'port',
            'sample': ('torch-CPU oracle on this host: full-size INT4 g128 quantize+pack of K and V '
                       '(%.3f s per tensor = %.2f GB/s), unpack+dequant of both (%.3f s), bf16 SDPA on 512 of the '
                       '4096 queries (%.3f s, scaled x8); value = packed-KV bytes / (dequant + scaled SDPA)'
                       % (c['t_quant_pack_per_tensor_s'], quant_bytes / c['t_quant_pack_per_tensor_s'] / 1e9,
                          c['t_unpack_dequant_s'], c['t_sdpa_sample_s'])),
            'pack_GBps': round(quant_bytes / c['t_quant_pack_per_tensor_s'] / 1e9, 3),
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
        'dtype': 'bf16', 'dtype_detail': 'bf16 MFMA operands holding exact int4 codes, fp32 scales and accumulation', 'data': 'synthetic',
        'config': {'workload': 'config 4: Infinity-2B KV [B=2,H=16,L=10521,D=128] bf16 -> INT4 group-128 asymmetric '
                               'quantize+pack of K and V, then fused dequant attention of the final 4096 queries',
                   'B': B, 'H': H, 'L': L, 'D': D, 'Lq': LQ, 'bits': BITS, 'group': GROUP, 'input_sets_cycled': NBUF},
        'attn_kv_read_frac_hbm_peak': round(kv_gbps / HBM_PEAK_GBPS, 5),
        'attn_ms': round(t_at * 1e3, 4), 'attn_TFLOPs': round(attn_tflops, 2),
        'attn_query_tokens_per_s': round(B * LQ / t_at, 1),
        'pack_GBps': round(pack_gbps, 2), 'pack_frac_hbm_peak': round(pack_gbps / HBM_PEAK_GBPS, 4),
        'pack_us_per_tensor': round(t_quant * 1e6, 2), 'pack_tokens_per_s': round(B * L / t_quant, 1),
        'roofline': {'kernel': 'fused_attn_kernel<128,4,128,128,token scales>', 'bound': 'mfma', 'achieved': round(attn_tflops, 2),
                     'peak': MFMA_BF16_PEAK_TFLOPS, 'unit': 'TFLOP/s', 'frac': round(attn_tflops / MFMA_BF16_PEAK_TFLOPS, 4),
                     'traffic': None if not traffic else traffic.get('fused_attn')},
        'roofline_pack': {'kernel': 'quant_pack_rows32_kernel<bf16,4,asym,4 lanes per group,dense>', 'bound': 'hbm', 'achieved': round(pack_gbps, 2),
                          'peak': HBM_PEAK_GBPS, 'unit': 'GB/s', 'frac': round(pack_gbps / HBM_PEAK_GBPS, 4),
                          'traffic': None if not traffic else traffic.get('quant_pack_rows', 0) // (1 if PAIR else 2) or None,
                          'tensors_per_launch': 2 if PAIR else 1},
        'cpu_baseline': cpu, 'checked_against_oracle': checked,
        'config5_latency': None if args.no_c5 else c5_latency(torch, dev),
        'config3_rates': None if args.no_c3 else c3_rates(torch, dev),
        'shipped_rule_latency': None if args.no_rule else shipped_rule_latency(torch, dev),
    }
    print(json.dumps(line), flush=True)


if __name__ == '__main__':
    main()

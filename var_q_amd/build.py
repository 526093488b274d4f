"""Builds libvarq_hip.so (the C-ABI library of include/varq.h) in-tree with hipcc.

Run as `python -m var_q_amd.build`.  hipcc cross-compiles for gfx950 without a
GPU.  The library has no torch or Python dependency.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
LIB = os.path.join(HERE, 'libvarq_hip.so')

# Bit-exactness of the quantizer rests on these: IEEE fp32 division, no FMA
# contraction across the oracle's separately rounded operations, denormals kept.
COMMON = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC',
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-fhip-fp32-correctly-rounded-divide-sqrt', '-fno-gpu-flush-denormals-to-zero',
    '-Wall', '-Wno-unused-function',
]
# per-file extras
FLAGS = {
    'capi.hip': ['-ffp-contract=off'],
    'quant_rows.hip': ['-ffp-contract=off'],
    'quant_general.hip': ['-ffp-contract=off'],
    'pack_unpack.hip': ['-ffp-contract=off'],
    'dequant.hip': ['-ffp-contract=off'],
    'qkv_prepare.hip': ['-ffp-contract=off'],
    'fused_attn.hip': [],
}


def _hipcc():
    exe = shutil.which('hipcc') or '/opt/rocm/bin/hipcc'
    if not os.path.exists(exe):
        raise RuntimeError('hipcc not found; the VAR-Q HIP library cannot be built')
    return exe


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = '\n'.join(l for l in p.stdout.splitlines() if 'not a recognized feature for this target' not in l)
    if p.returncode != 0:
        raise RuntimeError('command failed: %s\n%s' % (' '.join(cmd), out))
    return out


def build(verbose=True, jobs=6):
    hipcc = _hipcc()
    objdir = os.path.join(HERE, 'build')
    os.makedirs(objdir, exist_ok=True)
    srcs = sorted(f for f in os.listdir(CSRC) if f.endswith('.hip'))
    objs = [os.path.join(objdir, s[:-4] + '.o') for s in srcs]

    def compile_one(i):
        cmd = [hipcc] + COMMON + FLAGS.get(srcs[i], []) + ['-c', os.path.join(CSRC, srcs[i]), '-o', objs[i]]
        out = _run(cmd)
        if verbose:
            print('[varq build] %s%s' % (srcs[i], ('\n' + out) if out.strip() else ''), flush=True)

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(compile_one, range(len(srcs))))
    tmp = LIB + '.tmp'
    _run([hipcc, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', tmp] + objs)
    os.replace(tmp, LIB)
    if verbose:
        print('[varq build] linked', LIB, flush=True)
    return LIB


if __name__ == '__main__':
    build()
    sys.exit(0)

"""The C-ABI library loads and exports every symbol include/varq.h declares;
argument validation rejects bad calls on the host, before anything is launched
(so these run without a GPU)."""
import ctypes
import os
import re

import pytest

from var_q_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, 'include', 'varq.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(varq_[a-z_0-9]+)\s*\(', text)))


def test_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared()
    assert 'varq_quant_pack_rows' in names and 'varq_fused_attn' in names and len(names) >= 9
    for n in names:
        assert hasattr(lib, n), f'{n} is declared in varq.h but not exported'
    assert sorted(_lib.SYMBOLS) == names, 'ctypes table and header disagree'
    assert lib.varq_abi_version() == _lib.ABI_VERSION == 8


def test_invalid_arguments_are_rejected_on_the_host():
    lib = _lib.load()
    i64 = _lib.i64arr
    fake = ctypes.c_void_p(0x1000)     # never dereferenced: validation fails first
    rc = lib.varq_quant_pack_rows(fake, 1, 4, 64, 64, 3, 1, 1e-12, None, None, fake, fake, fake, None)
    assert rc == -1 and b'bits' in lib.varq_last_error()
    rc = lib.varq_quant_pack_rows(fake, 1, 4, 60, 60, 4, 1, 1e-12, None, None, fake, fake, fake, None)
    assert rc == -1
    rc = lib.varq_quant_pack_rows(fake, 1, 4, 64, 24, 4, 1, 1e-12, None, None, fake, fake, fake, None)
    assert rc == -1 and b'group' in lib.varq_last_error()
    rc = lib.varq_quant_pack_rows(fake, 1, 4, 64, 64, 4, 1, 1e-12, None, None, fake, fake, None, None)
    assert rc == -1 and b'zp' in lib.varq_last_error()
    rc = lib.varq_pack(fake, 4, 16, 5, fake, None)
    assert rc == -1
    rc = lib.varq_unpack(fake, 4, 16, 3, fake, None)
    assert rc == -1
    rc = lib.varq_quant_pack(fake, 0, i64([2, 2, 2, 8]), 3, 9, 0, 1e-12, fake, None, fake, None, None, fake, 1 << 20, None)
    assert rc == -1
    rc = lib.varq_quant_pack(fake, 0, i64([2, 2, 2, 8]), 3, 3, 0, 1e-12, fake, None, fake, None, None, fake, 1 << 20, None)
    assert rc == -1 and b'2/4/8' in lib.varq_last_error()
    rc = lib.varq_quant_pack(fake, 0, i64([2, 2, 2, 8]), 3, 4, 0, 1e-12, fake, None, fake, None, None, fake, 4, None)
    assert rc == -4
    rc = lib.varq_quant_pack(fake, 0, i64([2, 2, 2, 8]), 3, 4, 0, 1e-12, fake, None, fake, None, i64([3, 5, 0]), fake, 1 << 20, None)
    assert rc == -1 and b'output map' in lib.varq_last_error()   # 8 rows are not whole blocks of 3
    # 24 groups: room for scale reciprocal + flag per group plus per-chunk partial min/max (a multiple of
    # the group count), never less than two words per group; odd channel counts use two words per group
    ws = lib.varq_quant_workspace_bytes(i64([2, 5, 3, 8]), 0b0011)
    assert ws >= 3 * 8 * 2 * 4 and ws % (3 * 8 * 4) == 0
    assert lib.varq_quant_workspace_bytes(i64([2, 5, 3, 7]), 0b0011) == 3 * 7 * 2 * 4
    # the entry point without a workspace turns down what its static scratch cannot hold, on the host
    assert lib.varq_quant_static_scratch_bytes() == 16 << 20
    rc = lib.varq_quant_pack_static(fake, 0, i64([8, 4096, 16, 128]), 0b0001, 8, 0, 1e-12, fake, None, fake, None, None, None)
    assert rc == -4 and b'static' in lib.varq_last_error()
    rc = lib.varq_fused_attn(fake, fake, fake, fake, fake, 4, 128, fake, fake, fake, 4, 128,
                             1, 2, 2, None, 16, 16, 16, 96, None, 1.0, 0, 1, 0, None, 0, 0, None)
    assert rc == -1 and b'D must be' in lib.varq_last_error()
    rc = lib.varq_fused_attn(fake, fake, fake, fake, fake, 4, 128, fake, fake, fake, 8, 128,
                             1, 2, 2, None, 16, 16, 16, 128, None, 1.0, 0, 1, 0, None, 0, 0, None)
    assert rc == -2
    # the type of q / out and the operand form: fp32 queries, an unknown form, fp16 at head dim 128
    dt = lambda io, form, D=128: lib.varq_fused_attn(fake, fake, fake, fake, fake, 4, D, fake, fake, fake, 4, D,
                                                     1, 2, 2, None, 16, 16, 16, D, None, 1.0, 0, io, form, None, 0, 0, None)
    assert dt(0, 0) == -1 and b'io_dtype' in lib.varq_last_error()
    assert dt(1, 2) == -1 and b'operand_form' in lib.varq_last_error()
    assert dt(2, 0) == -2 and b'fp16' in lib.varq_last_error()
    # keys shared out over workgroups: the split count and its workspace are checked first
    tok = lambda splits, ws=None, nbytes=0: lib.varq_fused_attn(
        fake, fake, fake, fake, fake, 4, 128, fake, fake, fake, 4, 128, 1, 2, 2, None, 16, 640, 640, 128, None, 1.0, 0, 1, 0,
        ws, nbytes, splits, None)
    assert tok(9) == -1 and b'splits' in lib.varq_last_error()
    assert tok(2) == -1 and b'workspace' in lib.varq_last_error()
    assert tok(2, fake, 64) == -1 and b'workspace' in lib.varq_last_error()
    need = lib.varq_fused_attn_workspace_bytes(1, 2, 16, 640, 128, 1, 2)
    assert need == 2 * (1 * 2 * 16) * (128 + 2) * 4
    assert tok(2, ctypes.c_void_p(0x1004), need) == -1 and b'aligned' in lib.varq_last_error()
    # left to the library: a grid that fills the device in whole rounds is not split, a step
    # of a few hundred queries over a long cache is
    assert lib.varq_fused_attn_workspace_bytes(2, 16, 4096, 10521, 128, 1, 0) == 0
    assert lib.varq_fused_attn_workspace_bytes(2, 16, 400, 921, 128, 8, 0) > 0
    assert lib.varq_fused_attn_workspace_bytes(2, 16, 400, 921, 128, 8, 1) == 0
    # the kernel for few queries over a long cache (D = 128, one group per key, at most 64 queries,
    # at least 1024 keys, a (batch, head) slice within 4 GB): its share counts on 256 compute units
    # (what the library assumes without a device), its workspace, and who is not taken
    ks = lib.varq_fused_attn_key_shares
    assert ks(2, 16, 16, 10521, 128, 128, 128) == 16 and ks(2, 16, 64, 10521, 128, 128, 128) == 8
    assert ks(8, 128, 16, 1024, 128, 128, 128) == 1            # enough (batch, head) pairs already
    assert ks(1, 1, 16, 100000, 128, 128, 128) == 64           # capped
    assert ks(1, 2, 16, 1056, 128, 128, 128) == 4              # at least eight 32-key blocks per share
    assert lib.varq_fused_attn_workspace_bytes(2, 16, 16, 10521, 128, 1, 0) == 16 * (2 * 16 * 16) * (128 + 2) * 4
    for args in ((2, 16, 65, 10521, 128, 128, 128), (2, 16, 16, 1000, 128, 128, 128), (2, 16, 16, 10521, 64, 64, 64),
                 (2, 16, 16, 10521, 128, 64, 128), (1, 64, 16, 1 << 20, 128, 128, 128)):
        shares = ks(*args)
        assert 1 <= shares <= 8, args                           # the general kernel's sharing, or none
    # per-channel attention: segment table checks
    i32 = lambda v: (ctypes.c_int32 * len(v))(*v)
    chan = lambda nseg, ends, Lk=16, D=128: lib.varq_fused_attn_channel(
        fake, fake, fake, fake, None, fake, fake, None, nseg, ends, 8, 1, 2, 2, None, 16, Lk, 16, D, None, 1.0, 0, 1, None, 0, 0, None)
    assert chan(0, None) == -1 and b'nseg' in lib.varq_last_error()
    assert chan(17, None) == -1 and b'nseg' in lib.varq_last_error()
    assert chan(2, None) == -1 and b'segment ends missing' in lib.varq_last_error()
    assert chan(3, i32([8, 4, 16])) == -1 and b'increase' in lib.varq_last_error()
    assert chan(2, i32([40, 16])) == -1 and b'beyond' in lib.varq_last_error()
    assert chan(1, None, D=96) == -1 and b'D must be' in lib.varq_last_error()
    rc = lib.varq_fused_attn_channel(fake, fake, fake, ctypes.c_void_p(0x1004), None, fake, fake, None, 1, None,
                                     8, 1, 2, 2, None, 16, 16, 16, 128, None, 1.0, 0, 1, None, 0, 0, None)
    assert rc == -1 and b'aligned' in lib.varq_last_error()
    rc = lib.varq_fused_attn_channel(fake, fake, fake, fake, None, fake, fake, None, 1, None,
                                     8, 1, 2, 2, None, 16, 16, 16, 128, None, 1.0, 0, 2, None, 0, 0, None)
    assert rc == -2 and b'fp16' in lib.varq_last_error()
    # empty inputs are a no-op success
    assert chan(1, None, Lk=0) == -1          # queries but no keys
    assert lib.varq_pack(None, 0, 16, 4, None, None) == 0
    assert lib.varq_quant_pack_rows(fake, 1, 0, 64, 64, 4, 1, 1e-12, None, None, fake, fake, fake, None) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, '_lib', None)
    monkeypatch.setattr(_lib, 'LIB_PATH', str(tmp_path / 'nope.so'))
    with pytest.raises(_lib.VarqError, match='no fallback'):
        _lib.load()

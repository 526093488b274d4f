"""ctypes binding of libvarq_hip.so (include/varq.h).  No fallback: if the
library is missing or a call fails, an exception is raised."""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, 'libvarq_hip.so')

ABI_VERSION = 8

SYMBOLS = {
    'varq_abi_version': (c_int, []),
    'varq_last_error': (c_char_p, []),
    'varq_quant_pack_rows': (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_int, c_int, c_float,
                                     POINTER(c_int64), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    'varq_quant_pack_rows2': (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int, c_int, c_float,
                                      POINTER(c_int64), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_void_p]),
    'varq_quant_workspace_bytes': (c_size_t, [POINTER(c_int64), c_int]),
    'varq_quant_pack': (c_int, [c_void_p, c_int, POINTER(c_int64), c_int, c_int, c_int, c_float,
                                c_void_p, c_void_p, c_void_p, c_void_p, POINTER(c_int64), c_void_p, c_size_t, c_void_p]),
    'varq_quant_pack2': (c_int, [c_void_p, c_void_p, c_int, POINTER(c_int64), c_int, c_int, c_int, c_float,
                                 c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 POINTER(c_int64), c_void_p, c_size_t, c_void_p]),
    'varq_quant_static_scratch_bytes': (c_size_t, []),
    'varq_quant_pack_static': (c_int, [c_void_p, c_int, POINTER(c_int64), c_int, c_int, c_int, c_float,
                                       c_void_p, c_void_p, c_void_p, c_void_p, POINTER(c_int64), c_void_p]),
    'varq_pack': (c_int, [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p]),
    'varq_unpack': (c_int, [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p]),
    'varq_dequant': (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, POINTER(c_int64), POINTER(c_int64),
                             c_int, c_int, POINTER(c_int64), c_void_p, c_int, c_void_p]),
    'varq_fused_attn': (c_int, [c_void_p, c_void_p,
                                c_void_p, c_void_p, c_void_p, c_int, c_int,
                                c_void_p, c_void_p, c_void_p, c_int, c_int,
                                c_int, c_int, c_int, c_void_p,
                                c_int, c_int, c_int, c_int,
                                c_void_p, c_float, c_int, c_int, c_int, c_void_p, c_size_t, c_int, c_void_p]),
    'varq_fused_attn_workspace_bytes': (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    'varq_fused_attn_key_shares': (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    'varq_fused_attn_channel': (c_int, [c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_void_p,
                                        c_int, POINTER(c_int32),
                                        c_int, c_int, c_int, c_int, c_void_p,
                                        c_int, c_int, c_int, c_int,
                                        c_void_p, c_float, c_int, c_int, c_void_p, c_size_t, c_int, c_void_p]),
    'varq_qkv_prepare_append': (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int,
                                        c_void_p, c_int, c_float,
                                        c_void_p, c_void_p, c_int,
                                        c_void_p, c_int, c_int, c_int, c_float,
                                        POINTER(c_int64), c_void_p,
                                        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
}

_lib = None


class VarqError(RuntimeError):
    pass


def load():
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise VarqError(
            f'{LIB_PATH} is missing: build it with `python -m var_q_amd.build` '
            '(hipcc, gfx950).  There is no fallback path.')
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    got = lib.varq_abi_version()
    if got != ABI_VERSION:
        raise VarqError(f'libvarq_hip.so ABI {got} != expected {ABI_VERSION}; rebuild')
    _lib = lib
    return lib


def check(rc, what):
    if rc != 0:
        msg = load().varq_last_error().decode('utf-8', 'replace')
        raise VarqError(f'{what} failed (status {rc}): {msg}')


def i64arr(vals):
    return (c_int64 * len(vals))(*[int(v) for v in vals])

"""Drop-in for the reference module VAR_Q/pack_unpack.py.

Same four function names, signatures, return values and assertion behaviour
(VAR_Q/pack_unpack.py:107-134, 136-162, 177-196, 198-211).  All four run the
HIP pack/unpack kernels; the `_triton` names are kept so that imports written
against the reference (VAR_Q/quant.py:4) keep working, with no Triton behind
them.  GPU tensors only: the reference's `_python` pair also takes CPU tensors
(VAR_Q/pack_unpack.py:177-211); here a CPU tensor raises VarqError -- this library has no
CPU path on purpose (the CPU restatement of the layout is test infrastructure).
"""
from typing import Dict, Tuple

import torch

from . import ops
from ._lib import VarqError


def _need_gpu(t: torch.Tensor, what: str):
    if not t.is_cuda:
        raise VarqError(f'{what}: CPU tensor; the HIP pack/unpack kernels take GPU tensors only and there is no '
                        'CPU fallback (the reference\'s _python functions accept CPU tensors, this drop-in does not)')


def _meta(c: int, bits: int) -> Dict[str, int]:
    vals = 32 // bits
    return {'orig_c': int(c), 'vals_per_word': int(vals), 'pad_len': int((-c) % vals), 'bits': int(bits)}


def pack_last_dim_to_int32_hip(q_int8: torch.Tensor, bits: int) -> Tuple[torch.Tensor, Dict[str, int]]:
    """int8 codes [..., C] -> (int32 words [..., ceil(C/(32/bits))], meta)."""
    assert q_int8.is_cuda, "HIP version requires a GPU tensor"     # (the reference's _triton assert, pack_unpack.py:109)
    assert q_int8.dtype == torch.int8
    assert bits in (2, 4, 8), "bit-pack only implements 2/4/8 bits"
    return ops.pack(q_int8, bits), _meta(q_int8.shape[-1], bits)


def unpack_last_dim_from_int32_hip(packed: torch.Tensor, meta: Dict[str, int]) -> torch.Tensor:
    """int32 words + meta -> sign-extended int8 codes [..., orig_c]."""
    assert packed.is_cuda, "HIP version requires a GPU tensor"
    assert packed.dtype == torch.int32
    bits, orig_c = int(meta['bits']), int(meta['orig_c'])
    assert bits in (2, 4, 8), "bit-pack only implements 2/4/8 bits"
    return ops.unpack(packed, orig_c, bits)


# names of the reference module
pack_last_dim_to_int32_triton = pack_last_dim_to_int32_hip
unpack_last_dim_from_int32_triton = unpack_last_dim_from_int32_hip


def pack_last_dim_to_int32_python(q_int8: torch.Tensor, bits: int) -> Tuple[torch.Tensor, Dict[str, int]]:
    """The reference's CPU-capable twin (VAR_Q/pack_unpack.py:177-196): same result through the
    HIP kernel for a GPU tensor; a CPU tensor raises VarqError (no CPU path here)."""
    _need_gpu(q_int8, 'pack_last_dim_to_int32_python')
    return pack_last_dim_to_int32_hip(q_int8, bits)


def unpack_last_dim_from_int32_python(packed: torch.Tensor, meta: Dict[str, int]) -> torch.Tensor:
    """The reference's CPU-capable twin (VAR_Q/pack_unpack.py:198-211); CPU tensors raise VarqError."""
    _need_gpu(packed, 'unpack_last_dim_from_int32_python')
    return unpack_last_dim_from_int32_hip(packed, meta)

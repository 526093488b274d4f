"""Drop-in for the reference module VAR_Q/config_loader.py:10-128: JSON
quant-rule files -> section dictionaries.  Same class, methods and error
behaviour.  The `quantization` section additionally accepts the keys of the
asymmetric / group-wise / mixed-bit modes (`symmetric`, `group_size`,
`per_head_bits`); files written for the reference load unchanged.
"""
import json
import os
from typing import Any, Dict, Tuple

import torch


class VARQConfig:
    """Configuration manager for VAR-Q rules (VAR and Infinity)."""

    def __init__(self, config_path: str = None):
        if config_path is None:
            config_path = os.path.join(os.path.dirname(__file__), 'config.json')
        with open(config_path, 'r') as f:
            self.config = json.load(f)

    def _section(self, name: str) -> Dict[str, Any]:
        return self.config[name].copy()

    def get_model_config(self) -> Dict[str, Any]:
        return self._section('model')

    def get_quantization_config(self) -> Dict[str, Any]:
        return self._section('quantization')

    def get_inference_config(self) -> Dict[str, Any]:
        return self._section('inference')

    def get_checkpoint_config(self) -> Dict[str, Any]:
        return self._section('checkpoints')

    def get_checkpoint_paths(self, model_depth: int = None) -> Tuple[str, str]:
        ck = self.get_checkpoint_config()
        vae_ckpt = ck['vae_ckpt']
        if 'model_path' in ck:
            model_ckpt = ck['model_path']
        elif 'var_ckpt_template' in ck and model_depth is not None:
            model_ckpt = ck['var_ckpt_template'].format(model_depth)
        else:
            raise ValueError("Either 'model_path' or 'var_ckpt_template' with model_depth must be provided")
        return vae_ckpt, model_ckpt

    def get_device(self) -> str:
        device = self.config['inference']['device']
        if device == 'cuda' and not torch.cuda.is_available():
            return 'cpu'
        return device

    def get_batch_processing_config(self) -> Dict[str, Any]:
        return self.config.get('batch_processing', {}).copy()

    def is_infinity_model(self) -> bool:
        return 'infinity' in self.get_model_config().get('model_type', '').lower()

    def is_var_model(self) -> bool:
        return not self.is_infinity_model()

    def update_config(self, updates: Dict[str, Any]):
        def merge(dst, src):
            for key, val in src.items():
                dst[key] = merge(dst.get(key, {}), val) if isinstance(val, dict) else val
            return dst
        self.config = merge(self.config, updates)

    def save_config(self, save_path: str = None):
        if save_path is None:
            save_path = os.path.join(os.path.dirname(__file__), 'config.json')
        with open(save_path, 'w') as f:
            json.dump(self.config, f, indent=2)

    # -- extended `quantization` keys (a superset of the reference's JSON rule files) ---
    #   symmetric      bool, default true    max-abs (reference) or min-max affine codes
    #   group_size     int                   channels per group for quant_method "G_GROUP"
    #   per_head_bits  list of H ints in {2,4,8}: mixed precision, packed cache only
    def validate_quantization(self) -> Dict[str, Any]:
        """The `quantization` section, checked; raises ValueError naming the bad key."""
        qc = self.get_quantization_config()
        bits = qc.get('q_bits', 8)
        if not (isinstance(bits, int) and 1 < bits <= 8):
            raise ValueError('quantization.q_bits must be an int in (1, 8], got %r' % (bits,))
        if qc.get('qkv_format', 'BLHc') not in ('BLHc', 'BHLc'):
            raise ValueError('quantization.qkv_format must be "BLHc" or "BHLc", got %r' % (qc.get('qkv_format'),))
        if 'symmetric' in qc and not isinstance(qc['symmetric'], bool):
            raise ValueError('quantization.symmetric must be true or false')
        if qc.get('quant_method') == 'G_GROUP' and not (isinstance(qc.get('group_size'), int) and qc['group_size'] > 0):
            raise ValueError('quantization.quant_method "G_GROUP" needs a positive integer group_size')
        if 'per_head_bits' in qc:
            phb = qc['per_head_bits']
            if not (isinstance(phb, list) and phb and all(b in (2, 4, 8) for b in phb)):
                raise ValueError('quantization.per_head_bits must be a non-empty list over {2, 4, 8}')
            if qc.get('quant_method') != 'G_GROUP':
                raise ValueError('quantization.per_head_bits needs quant_method "G_GROUP" (packed cache)')
        return qc

    def quantizer_kwargs(self) -> Dict[str, Any]:
        """Constructor arguments for quant.VAR_Q from the `quantization` section
        (the four keys the reference threads into its attention blocks,
        VAR/models/__init__.py:108-111, plus the extended keys)."""
        qc = self.validate_quantization()
        kw = {'quant_bits': qc.get('q_bits', 8), 'qkv_format': qc.get('qkv_format', 'BLHc'),
              'quant_method': qc.get('quant_method', 'G_SCALE_HEAD_DIM')}
        for src, dst in (('symmetric', 'symmetric'), ('group_size', 'group_size')):
            if src in qc:
                kw[dst] = qc[src]
        return kw

    def packed_cache_kwargs(self, B: int, H: int, Lmax: int, D: int) -> Dict[str, Any]:
        """Constructor arguments for kv_cache.PackedKVCache (needs the row-local
        group-wise quantizer, i.e. quant_method "G_GROUP")."""
        qc = self.validate_quantization()
        if qc.get('quant_method') != 'G_GROUP':
            raise ValueError('the packed cache needs quantization.quant_method "G_GROUP"')
        bits = qc.get('per_head_bits', qc.get('q_bits', 8))
        if isinstance(bits, list) and len(bits) != H:
            raise ValueError('quantization.per_head_bits has %d entries for %d heads' % (len(bits), H))
        return {'B': B, 'H': H, 'Lmax': Lmax, 'D': D, 'bits': bits, 'group_size': qc['group_size'],
                'symmetric': qc.get('symmetric', True)}


def load_varq_config(config_path: str = None) -> VARQConfig:
    return VARQConfig(config_path)

"""Dtype tree casts of the reference's mesh_transformer/util.py:87-92 (the psum wrappers of
util.py:100-147 are the identity on one shard and have no counterpart here)."""
import torch


def _map(tree, fn):
    if isinstance(tree, dict):
        return {k: _map(v, fn) for k, v in tree.items()}
    if isinstance(tree, (list, tuple)):
        return type(tree)(_map(v, fn) for v in tree)
    return fn(tree)


def to_f32(t):
    """util.py:87-88: bfloat16 leaves -> float32, everything else untouched."""
    return _map(t, lambda x: x.to(torch.float32) if isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 else x)


def to_bf16(t):
    """util.py:91-92: float32 leaves -> bfloat16 (round to nearest even)."""
    return _map(t, lambda x: x.to(torch.bfloat16) if isinstance(x, torch.Tensor) and x.dtype == torch.float32 else x)

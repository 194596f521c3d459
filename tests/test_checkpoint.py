"""Sharded-checkpoint reader (the reference's mesh_transformer/checkpoint.py format) on the CPU."""
import os

import numpy as np
import pytest
import torch

from oracle import ckpt_oracle as CK
from oracle import gptj_oracle as O

CFG = dict(layers=2, d_model=64, n_heads=8, n_vocab=128, norm="layernorm", pe="rotary", pe_rotary_dims=4,
           seq=32, cores_per_replica=1)


def trained_like(cfg, seed):
    """Seeded tree whose LayerNorm parameters and biases are not at their initial values."""
    t = O.seeded_params(cfg, seed)
    g = torch.Generator().manual_seed(seed)
    for mod, leaves in t.items():
        if mod.endswith("replicated_layer_norm"):
            leaves["scale"] = 1 + 0.1 * torch.randn(leaves["scale"].shape, generator=g)
            leaves["offset"] = 0.1 * torch.randn(leaves["offset"].shape, generator=g)
    return t


def test_shard_tree_means_the_same_function():
    """The 8-way parameters, run as the reference runs them (loop over shards, sums where it psums), give the
    logits of the unsharded model: pins the sharding conventions the reader has to undo."""
    t = trained_like(CFG, 3)
    toks = O.seeded_prompt(1, 1, 20, hi=128)[0]
    ref = O.Model(CFG, t, torch.float64).forward(toks)
    for mp in (2, 8):
        got = CK.sharded_forward(CK.shard_tree(t, mp, CFG), CFG, toks, mp)
        assert float((got - ref).abs().max()) < 1e-9, mp


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_read_ckpt_folds_8_shards_into_1(tmp_path, dtype):
    from mesh_transformer import checkpoint as ckpt
    from mesh_transformer.util import to_bf16
    t = trained_like(CFG, 4)
    if dtype == torch.bfloat16:
        t = to_bf16(t)                           # dividing a bias by 8 and multiplying back is exact in bf16 too
    stacked = {"params": CK.shard_tree(t, 8, CFG), "step": np.full(8, 383500, np.uint32)}
    d = str(tmp_path) + os.sep
    for s in range(8):
        ckpt.write_ckpt(stacked, d, s)
    assert sorted(os.listdir(d)) == [f"shard_{s}" for s in range(8)]
    assert sorted(os.listdir(d + "shard_0")) == sorted(f"{i}.npz" for i in range(16))
    skeleton = {"params": O.seeded_params(CFG, 0, dtype), "step": np.array(0)}
    state = ckpt.read_ckpt(skeleton, d, 8, shards_out=1)
    assert int(state["step"]) == 383500
    for mod, leaves in t.items():
        for k, v in leaves.items():
            got = state["params"][mod][k]
            assert got.dtype == dtype and got.shape == v.shape, (mod, k)
            assert torch.equal(got, v), (mod, k)
    # leaf by leaf (checkpoint.py:178-227): the same tree
    low = ckpt.read_ckpt_lowmem(skeleton, d, 8, shards_out=1)
    assert int(low["step"]) == 383500
    for mod, leaves in t.items():
        for k, v in leaves.items():
            assert low["params"][mod][k].dtype == dtype and torch.equal(low["params"][mod][k], v), (mod, k)
    # same shard count in and out: the stacked tree comes back as it is
    same = ckpt.read_ckpt(stacked, d, 8)
    for mod, leaves in stacked["params"].items():
        for k, v in leaves.items():
            assert torch.equal(same["params"][mod][k], v)


def test_read_ckpt_refuses_what_it_cannot_load(tmp_path):
    from mesh_transformer import checkpoint as ckpt
    t = O.seeded_params(CFG, 5)
    d = str(tmp_path) + os.sep
    full = {"opt_state": {"mu": {"x": torch.zeros(2, 3)}}, "params": CK.shard_tree(t, 2, CFG), "step": np.zeros(2, np.uint32)}
    for s in range(2):
        ckpt.write_ckpt(full, d, s)
    with pytest.raises(ValueError, match="slim"):
        ckpt.read_ckpt({"params": t, "step": np.array(0)}, d, 2, shards_out=1)
    with pytest.raises(ValueError):          # the optimizer leaves come first in tree order: a shape mismatch or too many
        ckpt.read_ckpt_lowmem({"params": t, "step": np.array(0)}, d, 2, shards_out=1)
    with pytest.raises(FileNotFoundError):
        ckpt.read_ckpt({"params": t, "step": np.array(0)}, d, 4, shards_out=1)
    bad = dict(CFG, d_model=32)
    with pytest.raises(ValueError):
        slim = {"params": CK.shard_tree(t, 2, CFG), "step": np.zeros(2, np.uint32)}
        d2 = str(tmp_path / "slim") + os.sep
        for s in range(2):
            ckpt.write_ckpt(slim, d2, s)
        ckpt.read_ckpt({"params": O.seeded_params(bad, 0), "step": np.array(0)}, d2, 2, shards_out=1)


def test_flatten_order_is_sorted_keys():
    from mesh_transformer import checkpoint as ckpt
    tree = {"step": 1, "params": {"b": {"w": 2, "b": 3}, "a/~/x": {"scale": 4, "offset": 5}}}
    leaves, paths = ckpt.tree_flatten(tree)
    assert paths == [("params", "a/~/x", "offset"), ("params", "a/~/x", "scale"), ("params", "b", "b"),
                     ("params", "b", "w"), ("step",)]
    assert leaves == [5, 4, 3, 2, 1]
    assert ckpt.tree_unflatten(paths, leaves) == tree
    assert [len(c) for c in ckpt.split(list(range(35)), 16)] == [3, 3, 3] + [2] * 13

"""Reader (and writer) for the reference's sharded checkpoint format, mesh_transformer/checkpoint.py.

Layout on disk (checkpoint.py:57-79): `<dir>shard_<s>/<p>.npz` for every tensor-parallel shard s and piece
p in 0..15; a piece holds, as arr_0, arr_1, ..., a contiguous run of the leaves of the flattened state in
jax.tree_flatten order (dict keys sorted at every level), each leaf being shard s's slice without the leading
shard axis.  bfloat16 leaves are stored with numpy's 2-byte void dtype `V2` (checkpoint.py:19-25).

`read_ckpt(state, dir, shards_in, shards_out)` mirrors checkpoint.py:135-175 for the inference state
{"params": ..., "step": ...}: with shards_out == 1 it folds an N-shard checkpoint into the unsharded tree this
build runs (reshard rules of checkpoint.py:96-132).  Everything happens on the host with numpy/torch; hand the
result to CausalTransformer.from_params / assign it to network.state.
"""
import os

import numpy as np
import torch

pieces = 16  # how many files each shard is split across (checkpoint.py:16)

_V2 = np.dtype("V2")


def _to_numpy(leaf):
    """A leaf as the array np.savez should store: bfloat16 becomes 2-byte void."""
    if isinstance(leaf, torch.Tensor):
        t = leaf.detach().cpu().contiguous()
        if t.dtype == torch.bfloat16:
            return t.view(torch.int16).numpy().view(_V2)
        return t.numpy()
    return np.asarray(leaf)


def _from_numpy(a):
    """Stored array -> torch tensor (V2 -> bfloat16, checkpoint.py:21-22)."""
    a = np.ascontiguousarray(a)
    if a.dtype == _V2:
        return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    return torch.from_numpy(a.copy())


def tree_flatten(tree):
    """Leaves in jax.tree_flatten order (sorted dict keys, depth first) and the list of their key paths."""
    leaves, paths = [], []

    def walk(node, path):
        if isinstance(node, dict):
            for k in sorted(node):
                walk(node[k], path + (k,))
        else:
            leaves.append(node)
            paths.append(path)

    walk(tree, ())
    return leaves, paths


def tree_unflatten(paths, leaves):
    out = {}
    for path, leaf in zip(paths, leaves):
        node = out
        for k in path[:-1]:
            node = node.setdefault(k, {})
        node[path[-1]] = leaf
    return out


def split(a, n):
    """checkpoint.py:52-54: n nearly equal contiguous runs."""
    k, m = divmod(len(a), n)
    return [a[i * k + min(i, m):(i + 1) * k + min(i + 1, m)] for i in range(n)]


def write_ckpt(pytree, dir, shard):
    """checkpoint.py:57-79: write shard `shard` of a state whose leaves carry a leading shard axis."""
    leaves, _ = tree_flatten(pytree)
    mine = [_to_numpy(l)[shard] if np.ndim(_to_numpy(l)) else _to_numpy(l) for l in leaves]
    d = os.path.join(dir, f"shard_{shard}")
    os.makedirs(d, exist_ok=True)
    for idx, chunk in enumerate(split(mine, pieces)):
        with open(os.path.join(d, f"{idx}.npz"), "wb") as f:
            np.savez(f, *chunk)


def read_shard(ckpt_dir):
    """checkpoint.py:82-93: all leaves of one shard, in order."""
    out = []
    for idx in range(pieces):
        with np.load(os.path.join(ckpt_dir, f"{idx}.npz"), allow_pickle=False) as z:
            for name in z.files:          # arr_0, arr_1, ... in insertion order
                out.append(z[name])
    return out


def _as_float(x):
    return x.view(np.int16).astype(np.int32) if x.dtype == _V2 else x


def reshard(x, old_shape):
    """checkpoint.py:96-132: fold the stacked shards x [shards_in, ...] of one leaf into old_shape [1, ...].

    1-D (step counters): keep the first.  2-D: shards 1.. all equal and all 0 or all 1 -> a replicated LayerNorm
    parameter, only shard 0 of which is ever trained (layers.py:23-26): keep shard 0; all equal otherwise -> a
    bias added on every shard before the sum over shards (fc_out and embedding bias): scale by the number of
    shards folded; else a column-split bias: concatenate.  3-D: a weight split over its last axis (q, k, v,
    fc_in, logits: transpose then reshape) or over its first (out, fc_out, embedding: reshape)."""
    if x.ndim == 1:
        return x[0:1]
    if x.ndim == 2:
        xv = _as_float(x)
        if (xv[1:] == xv[-1]).all():
            f = _from_numpy(x)
            if (f[1:].float() == 0).all() or (f[1:].float() == 1).all():
                return x[0:1]
            scaled = f[0:1].float() * (x.shape[0] / old_shape[0])
            return _to_numpy(scaled.to(f.dtype))
        return x.reshape(old_shape)
    if x.ndim == 3:
        if x.shape[0] * x.shape[2] == old_shape[2]:
            return np.transpose(x, (1, 0, 2)).reshape(old_shape)
        if x.shape[0] * x.shape[1] == old_shape[1]:
            return x.reshape(old_shape)
        raise ValueError(f"unimplemented reshard {x.shape} -> {old_shape}")
    raise ValueError(f"unimplemented reshard of a {x.ndim}-d leaf")


def _fit(x, o, path, shards_in, shards_out):
    """One leaf: stacked shards x [shards_in, ...] -> the shape of the state's leaf o (resharded if asked)."""
    shape = tuple(o.shape) if hasattr(o, "shape") else ()
    if shards_out != shards_in:
        if shards_out != 1:
            raise ValueError("this build runs unsharded: shards_out must be 1 (or equal to shards_in)")
        want = shape if len(shape) == x.ndim else (1,) + shape
        x = reshard(x, want)
    if len(shape) != x.ndim and int(np.prod(shape, dtype=np.int64)) == x.size:
        x = x.reshape(shape)          # the step counter is a scalar here, [shards] in the reference
    if tuple(x.shape) != shape:
        raise ValueError(f"Incompatible checkpoints {x.shape} vs {shape} at {'/'.join(path)}")
    return _from_numpy(x)


def read_ckpt_lowmem(pytree, dir, shards_in, shards_out=None, load_opt=True, device=None):
    """checkpoint.py:178-227: the same result as read_ckpt, read leaf by leaf - piece file by piece file, the same
    array of every shard, stacked, resharded and put on `device` (the reference spreads the leaves over its devices
    with jax.device_put; here there is one) - so that the host never holds more than one leaf of every shard at a
    time (0.8 GB for the 6B embedding instead of the 12 GB tree).  device=None keeps the leaves on the host."""
    if shards_out is None:
        shards_out = shards_in
    skel = {k: v for k, v in pytree.items() if k != "opt_state"}
    old, paths = tree_flatten(skel)
    out = []
    for idx in range(pieces):
        files = [np.load(os.path.join(dir, f"shard_{s}", f"{idx}.npz"), allow_pickle=False) for s in range(shards_in)]
        try:
            names = files[0].files
            if any(f.files != names for f in files):
                raise ValueError("shards hold different numbers of arrays")
            for name in names:
                if len(out) >= len(old):
                    raise ValueError(f"checkpoint has more leaves than the state's {len(old)}: only slim checkpoints "
                                     "(parameters and step, no optimizer state) can be loaded")
                leaf = _fit(np.stack([f[name] for f in files]), old[len(out)], paths[len(out)], shards_in, shards_out)
                out.append(leaf.to(device) if device is not None and leaf.ndim > 0 else leaf)
        finally:
            for f in files:
                f.close()
    if len(out) != len(old):
        raise ValueError(f"checkpoint has {len(out)} leaves, the state has {len(old)}")
    state = tree_unflatten(paths, out)
    if "opt_state" in pytree:
        state["opt_state"] = pytree["opt_state"]
    return state


def read_ckpt(pytree, dir, shards_in, shards_out=None, load_opt=True):
    """checkpoint.py:135-175.  `pytree` gives the structure and the target shapes (e.g. network.state);
    returns a new state with torch tensors on the host.  Only the inference state is supported: a checkpoint
    that also holds optimizer state has more leaves than `pytree` and is refused."""
    if shards_out is None:
        shards_out = shards_in
    skel = {k: v for k, v in pytree.items() if k != "opt_state"}
    old, paths = tree_flatten(skel)
    shards = [read_shard(os.path.join(dir, f"shard_{i}")) for i in range(shards_in)]
    n = len(shards[0])
    if any(len(s) != n for s in shards):
        raise ValueError("shards hold different numbers of arrays")
    if n != len(old):
        raise ValueError(f"checkpoint has {n} leaves, the state has {len(old)}: only slim checkpoints "
                         "(parameters and step, no optimizer state) can be loaded")
    out = []
    for o, path, *parts in zip(old, paths, *shards):
        out.append(_fit(np.stack(parts), o, path, shards_in, shards_out))
    state = tree_unflatten(paths, out)
    if "opt_state" in pytree:
        state["opt_state"] = pytree["opt_state"]
    return state

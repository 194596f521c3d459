"""CPU oracle for the sharded-checkpoint row: what an N-way tensor-parallel parameter tree of the reference MEANS.

TEST INFRASTRUCTURE ONLY (imported by tests/ alone).  Two things, both derived from the reference's layer
definitions rather than from its resharding code:

  shard_tree(tree, mp)        the per-shard parameters [mp, ...] that the reference's modules would hold for the
                              same function (layers.py:166-185, 230-258, 546-559; replicated LayerNorm parameters
                              layers.py:17-36; biases that are added on every shard before a sum over shards)
  sharded_forward(...)        the forward pass as the reference computes it under xmap over the 'shard' axis
                              (f_psum / g_psum of util.py:100-147, all_gather of layers.py:23-26, 565-567), written
                              as an explicit loop over shards in float64

Pinning: sharded_forward(shard_tree(T)) must equal the unsharded oracle forward of T (tests/test_checkpoint.py),
which fixes shard_tree by the mathematics of the sharded layers; the product's reader is then checked against it.
The exact bytes of a checkpoint written by the reference's jax code (np.savez of jax arrays) are not available
here: the on-disk container is restated from checkpoint.py:27-93 and that part is parity unpinned.
"""
import math

import numpy as np
import torch

from . import gptj_oracle as O


def shard_tree(tree, mp: int, cfg):
    """Unsharded tree (leading axis 1) -> the mp-way stacked tree."""
    d, V = cfg["d_model"], cfg["n_vocab"]
    out = {}

    def cols(w):      # [1, in, out] -> [mp, in, out/mp]: shard s owns a contiguous block of output columns
        i, o = w.shape[1], w.shape[2]
        return w[0].reshape(i, mp, o // mp).permute(1, 0, 2).contiguous()

    def rows(w):      # [1, in, out] -> [mp, in/mp, out]: shard s owns a contiguous block of input rows
        i, o = w.shape[1], w.shape[2]
        return w[0].reshape(mp, i // mp, o).contiguous()

    def replicated_ln(v, init):   # only shard 0's copy is used (all_gather(...)[0]) and hence trained
        return torch.cat([v, torch.full((mp - 1,) + tuple(v.shape[1:]), init, dtype=v.dtype)], 0)

    def summed_bias(b):           # added on every shard, then summed over shards
        return (b / mp).repeat(mp, 1)

    for mod, leaves in tree.items():
        o = {}
        if mod.endswith("replicated_layer_norm"):
            o["scale"] = replicated_ln(leaves["scale"], 1.0)
            o["offset"] = replicated_ln(leaves["offset"], 0.0)
        elif mod == O.EMBED:
            o["w"] = rows(leaves["w"])                      # vocabulary split (layers.py:172-176)
            o["b"] = summed_bias(leaves["b"])
        elif mod == O.PROJ:
            o["w"] = cols(leaves["w"])                      # vocabulary split (layers.py:553-559)
            o["b"] = leaves["b"][0].reshape(mp, -1)
        else:
            name = mod.rsplit("/", 1)[-1]
            if name in ("linear", "linear_1", "linear_2"):  # q, v, k: heads split (layers.py:249-251)
                o["w"] = cols(leaves["w"])
            elif name == "linear_3":                        # o (layers.py:253)
                o["w"] = rows(leaves["w"])
            elif name == "linear_4":                        # fc_in (layers.py:256)
                o["w"] = cols(leaves["w"])
                o["b"] = leaves["b"][0].reshape(mp, -1)
            elif name == "linear_5":                        # fc_out (layers.py:258)
                o["w"] = rows(leaves["w"])
                o["b"] = summed_bias(leaves["b"])
            else:
                raise KeyError(mod)
        out[mod] = o
    return out


def sharded_forward(st, cfg, tokens, mp: int):
    """Logits [T, V] of the full forward, computed shard by shard from the stacked tree `st`."""
    dt = torch.float64
    g = lambda mod, leaf, s: st[mod][leaf][s].to(dt)
    d, H, V = cfg["d_model"], cfg["n_heads"], cfg["n_vocab"]
    dh, r = d // H, O.rotary_dims(cfg)
    Hs, Vs = H // mp, V // mp
    tok = torch.as_tensor(np.asarray(tokens).astype(np.int64))
    T = tok.shape[0]
    # EmbeddingShard (layers.py:187-202): one_hot over the shard's vocabulary slice, then g_psum
    x = torch.zeros(T, d, dtype=dt)
    for s in range(mp):
        local = tok - s * Vs
        hot = torch.zeros(T, Vs, dtype=dt)
        ok = (local >= 0) & (local < Vs)
        hot[torch.arange(T)[ok], local[ok]] = 1.0
        x = x + hot @ g(O.EMBED, "w", s) + g(O.EMBED, "b", s)
    causal = O.MASK * (1.0 - torch.tril(torch.ones(T, T, dtype=dt)))
    for i in range(cfg["layers"]):
        k_ = lambda m: O.layer_key(i, m)
        h = O.replicated_layer_norm(x, g(k_("replicated_layer_norm"), "scale", 0), g(k_("replicated_layer_norm"), "offset", 0))
        delta = torch.zeros_like(x)
        for s in range(mp):                                  # TransformerLayerShard.__call__ on shard s
            q = (h @ g(k_("linear"), "w", s)).reshape(T, Hs, dh)
            v = (h @ g(k_("linear_1"), "w", s)).reshape(T, Hs, dh)
            k = (h @ g(k_("linear_2"), "w", s)).reshape(T, Hs, dh)
            sincos = O.fixed_pos_embedding(T, r)
            q = torch.cat([O.apply_rotary_pos_emb(q[:, :, :r], sincos), q[:, :, r:]], -1)
            k = torch.cat([O.apply_rotary_pos_emb(k[:, :, :r], sincos), k[:, :, r:]], -1)
            sc = torch.einsum("thd,Thd->htT", q, k) / math.sqrt(dh) + causal
            a = torch.einsum("htT,Thd->thd", torch.softmax(sc, -1), v).reshape(T, Hs * dh)
            attn = a @ g(k_("linear_3"), "w", s)
            ff = O.gelu_tanh(h @ g(k_("linear_4"), "w", s) + g(k_("linear_4"), "b", s)) @ g(k_("linear_5"), "w", s) \
                + g(k_("linear_5"), "b", s)
            delta = delta + attn + ff                        # g_psum
        x = x + delta
    h = O.replicated_layer_norm(x, g(O.PROJ_LN, "scale", 0), g(O.PROJ_LN, "offset", 0))
    # ProjectionShard.__call__ (layers.py:561-567): all_gather over shards, transpose, flatten
    return torch.cat([h @ g(O.PROJ, "w", s) + g(O.PROJ, "b", s) for s in range(mp)], -1)

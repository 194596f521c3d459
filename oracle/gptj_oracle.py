"""CPU oracle for the GPT-J generate path of mesh-transformer-jax.

TEST INFRASTRUCTURE ONLY.  This module is the checker for the HIP path: it may
be imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of
bench.py, and by nothing that ships.  It is a from-scratch restatement (torch on
the CPU, float64 for ground truth, float32 for the timed baseline) of the
reference's arithmetic with the reference's literal conventions: the K/V window
is rebuilt by concatenate+slice every step, K is cached un-rotated and the whole
window is re-rotated at window indices every step, masks are additive -1e10.

Every function names the reference lines it follows (paths are relative to the
reference checkout).

Pinning status (what, other than this file's own formulas, fixes each result):
  * replicated_layer_norm  - torch.nn.functional.layer_norm, invariants
  * embedding_shard        - one-hot matmul identity
  * rotary                 - 2x2 rotations per pair, shift invariance, the
                             independent interleaved implementation in
                             transformers.models.gptj
  * self_attn / masks      - brute-force loops, F.scaled_dot_product_attention,
                             left-pad invariance
  * ff / gelu              - torch gelu(approximate="tanh")
  * whole layer / model    - transformers.GPTJForCausalLM from a local config
                             through the reference's own weight-name map
  * decode_once / window   - teacher forcing against the full forward,
                             brute-force sliding window
  * loss (evaluation)      - torch.nn.functional.cross_entropy and argmax on the
                             full-forward logits; masked keys cannot influence a row
  * nucleaus_filter        - reference demo vector (sampling.py:49) worked by
                             hand, brute force over prefixes, invariants
  * inverse_cdf_draw       - own contract (the reference's Gumbel draw is
                             replaced by design); brute force + chi-square
  * jax.random.categorical token stream, haiku TruncatedNormal values:
    parity unpinned (need the absent jax/haiku; both are replaced by design).
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional, Tuple

import numpy as np
import torch

MASK = -1e10  # additive mask constant, layers.py:307,334,360


# ----------------------------------------------------------------------------
# parameter tree helpers (names: to_hf_weights.py:160-173,183-223)
# ----------------------------------------------------------------------------
ROOT = "causal_transformer_shard/~/"


def layer_key(i: int, leaf: str) -> str:
    return f"{ROOT}layer_{i}/~/{leaf}"


EMBED = ROOT + "embedding_shard/~/linear"
PROJ_LN = ROOT + "projection_shard/~/replicated_layer_norm"
PROJ = ROOT + "projection_shard/~/linear"


def d_head(cfg) -> int:
    return cfg["d_model"] // cfg["n_heads"]


def rotary_dims(cfg) -> int:
    # layers.py:244 - defaults to the full head dim
    return cfg.get("pe_rotary_dims", d_head(cfg))


def param_shapes(cfg) -> Dict[str, Dict[str, Tuple[int, ...]]]:
    """Haiku tree of CausalTransformerShard at cores_per_replica == 1.

    Shapes follow hk.Linear ([in, out] weights) as used at layers.py:185,249-258,559;
    the leading axis of size 1 is the xmap "shard" axis (transformer_shard.py:218-222).
    """
    d, V, F = cfg["d_model"], cfg["n_vocab"], 4 * cfg["d_model"]
    t: Dict[str, Dict[str, Tuple[int, ...]]] = {EMBED: {"w": (1, V, d), "b": (1, d)}}
    for i in range(cfg["layers"]):
        t[layer_key(i, "replicated_layer_norm")] = {"scale": (1, d), "offset": (1, d)}
        t[layer_key(i, "linear")] = {"w": (1, d, d)}      # q
        t[layer_key(i, "linear_1")] = {"w": (1, d, d)}    # v
        t[layer_key(i, "linear_2")] = {"w": (1, d, d)}    # k
        t[layer_key(i, "linear_3")] = {"w": (1, d, d)}    # o
        t[layer_key(i, "linear_4")] = {"w": (1, d, F), "b": (1, F)}
        t[layer_key(i, "linear_5")] = {"w": (1, F, d), "b": (1, d)}
    t[PROJ_LN] = {"scale": (1, d), "offset": (1, d)}
    t[PROJ] = {"w": (1, d, V), "b": (1, V)}
    return t


def count_params(cfg) -> int:
    return sum(int(np.prod(s)) for m in param_shapes(cfg).values() for s in m.values())


def seeded_params(cfg, seed: int, weight_dtype=torch.float32, std: float = 0.02):
    """Synthetic tree: every weight and bias ~ N(0, std) from numpy Philox(seed), drawn in
    sorted key order as float32; LayerNorm scale = 1, offset = 0.  weight_dtype=bfloat16
    rounds each leaf once (round-to-nearest-even), which is what util.py:91-92 does."""
    rng = np.random.Generator(np.random.Philox(seed))
    shapes = param_shapes(cfg)
    out = {}
    for mod in sorted(shapes):
        out[mod] = {}
        for leaf in sorted(shapes[mod]):
            shp = shapes[mod][leaf]
            if leaf == "scale":
                a = np.ones(shp, np.float32)
            elif leaf == "offset":
                a = np.zeros(shp, np.float32)
            else:
                a = rng.standard_normal(shp, dtype=np.float32) * np.float32(std)
            out[mod][leaf] = torch.from_numpy(a).to(weight_dtype)
    return out


def hashed_params(cfg, seed: int, weight_dtype=torch.bfloat16, std: float = 0.02, device="cpu"):
    """Synthetic tree for sizes where drawing normals on the host is too slow and a device generator would not be
    reproducible elsewhere: element i of leaf number j (sorted key order) is a 16-bit integer hash of (seed, j, i),
    centred and scaled to standard deviation `std` (uniform, not normal).  Integer arithmetic, one exact
    subtraction and one float32 multiplication: the same bits on any device.  LayerNorm scale = 1, offset = 0."""
    shapes = param_shapes(cfg)
    scale = np.float32(std * np.sqrt(12.0) / 65536.0)
    out, j = {}, 0
    for mod in sorted(shapes):
        out[mod] = {}
        for leaf in sorted(shapes[mod]):
            shp = shapes[mod][leaf]
            j += 1
            if leaf == "scale":
                a = torch.ones(shp, dtype=torch.float32, device=device)
            elif leaf == "offset":
                a = torch.zeros(shp, dtype=torch.float32, device=device)
            else:
                n = int(np.prod(shp))
                h = torch.arange(n, dtype=torch.int64, device=device)
                h = (h * 2654435761 + (seed * 1000003 + j) * 40503) & 0xFFFFFFFF
                h ^= h >> 15
                h = (h * 2246822519) & 0xFFFFFFFF
                h ^= h >> 13
                h = (h * 3266489917) & 0xFFFFFFFF
                h ^= h >> 16
                a = (((h & 0xFFFF).to(torch.float32) - 32767.5) * float(scale)).reshape(shp)
                del h
            out[mod][leaf] = a.to(weight_dtype)
    return out


def add_outliers(tree, cfg, gains=(0.5, 2.0, 0.5, 2.0)):
    """Turns a synthetic tree into one shaped like a trained model, in place and with the SAME bits on any device: every
    new value is a small integer pattern that bfloat16 holds exactly, every rescaling a power of two.  Four residual
    channels carry +-50 .. +-500 from the embedding bias on and grow by a quarter of that through every fc_out bias;
    LayerNorm scales run from 0.5 to 30 in steps of 0.5 (1 on the outlier channels) with offsets in [-0.5, 0.5]; the
    rows of q, v, k and fc_in are divided by 1, 2 or 4 where the scale is below 2, 8 or 32 (and multiplied by `gains`,
    powers of two, as whole matrices), the embedding matrix by 32; one k matrix holds +-4 next to its small entries."""
    d, n = cfg["d_model"], cfg["layers"]
    dev = tree[EMBED]["w"].device
    c = torch.arange(d, device=dev)
    ch = torch.tensor([7, 300, 511, 900], device=dev)
    big = torch.tensor([300.0, -500.0, 50.0, -120.0], device=dev)
    dt = tree[EMBED]["w"].dtype

    def put(leaf, value):                                 # value float32 -> the leaf's dtype, one rounding
        leaf.copy_(value.to(dt))

    put(tree[EMBED]["w"], tree[EMBED]["w"].float() * 32.0)
    b = tree[EMBED]["b"].float()
    b[0, ch] = big
    put(tree[EMBED]["b"], b)
    for i in range(n):
        sc = 0.5 + ((c * 37 + i * 11) % 60).float() * 0.5
        sc[ch] = 1.0
        off = (((c * 53 + i * 7) % 17).float() - 8.0) / 16.0
        ln = tree[layer_key(i, "replicated_layer_norm")]
        put(ln["scale"], sc[None])
        put(ln["offset"], off[None])
        b2 = tree[layer_key(i, "linear_5")]["b"].float()
        b2[0, ch] += big * 0.25
        put(tree[layer_key(i, "linear_5")]["b"], b2)
        row = torch.where(sc < 2.0, 1.0, torch.where(sc < 8.0, 0.5, 0.25))       # per input channel
        for name, gain in zip(("linear", "linear_1", "linear_2", "linear_4"), gains):
            w = tree[layer_key(i, name)]["w"]
            put(w, w.float() * (row * gain)[None, :, None])
    w = tree[layer_key(min(1, n - 1), "linear_2")]["w"]
    w[0, 5, 17], w[0, 700, 333] = 4.0, -4.0
    put(tree[PROJ_LN]["scale"], (0.5 + ((c * 29) % 6).float() * 0.5)[None])
    put(tree[PROJ_LN]["offset"], ((((c * 31) % 9).float() - 4.0) / 16.0)[None])
    return tree


def seeded_prompt(seed: int, batch: int, n: int, hi: int = 50257) -> np.ndarray:
    rng = np.random.Generator(np.random.Philox(seed + 1000003))
    return rng.integers(0, hi, size=(batch, n), dtype=np.int64).astype(np.uint32)


def left_pad(tokens: np.ndarray, L: int) -> np.ndarray:
    """device_sample.py:92-96 - zero-pad on the left to length L."""
    B, P = tokens.shape
    out = np.zeros((B, L), np.uint32)
    out[:, L - P:] = tokens
    return out


# ----------------------------------------------------------------------------
# layers
# ----------------------------------------------------------------------------
def replicated_layer_norm(x, scale, offset):
    """layers.py:17-36 - biased variance, eps inside rsqrt, scale folded into inv."""
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    inv = scale * torch.rsqrt(var + 1e-5)
    return inv * (x - mean) + offset


def embedding_shard(tokens, w, b):
    """layers.py:187-202 - one_hot(tok) @ W + b; a one-hot row selects exactly one row."""
    return w[tokens.long()] + b


def fixed_pos_embedding(n_pos: int, dim: int):
    """layers.py:128-134 - float64 numpy tables [n_pos, dim/2]."""
    inv_freq = 1.0 / (10000 ** (np.arange(0, dim, 2) / dim))
    ang = np.einsum("i,j->ij", np.arange(n_pos), inv_freq)
    return np.sin(ang), np.cos(ang)


def rotate_every_two(x):
    """layers.py:137-143 - (x0,x1,x2,x3,..) -> (-x1,x0,-x3,x2,..)."""
    x1 = x[..., ::2]
    x2 = x[..., 1::2]
    return torch.stack((-x2, x1), dim=-1).reshape(x.shape)


def apply_rotary_pos_emb(x, sincos):
    """layers.py:146-148 - x is [t, H, r]; uses the LAST t rows of the tables."""
    sin, cos = sincos
    t = x.shape[0]
    sin = torch.as_tensor(sin, dtype=x.dtype).repeat_interleave(2, dim=-1)[-t:, None, :]
    cos = torch.as_tensor(cos, dtype=x.dtype).repeat_interleave(2, dim=-1)[-t:, None, :]
    return x * cos + rotate_every_two(x) * sin


def gelu_tanh(x):
    """jax.nn.gelu default (approximate=True), layers.py:289."""
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


class Layer:
    """TransformerLayerShard, layers.py:229-366, at cores_per_replica == 1."""

    def __init__(self, cfg, params, i: int, dtype):
        g = lambda mod, leaf: params[layer_key(i, mod)][leaf][0].to(dtype)
        self.H, self.dh, self.r = cfg["n_heads"], d_head(cfg), rotary_dims(cfg)
        self.rot = cfg["pe"] == "rotary"
        self.ln_s, self.ln_o = g("replicated_layer_norm", "scale"), g("replicated_layer_norm", "offset")
        self.wq, self.wv, self.wk, self.wo = g("linear", "w"), g("linear_1", "w"), g("linear_2", "w"), g("linear_3", "w")
        self.w1, self.b1 = g("linear_4", "w"), g("linear_4", "b")
        self.w2, self.b2 = g("linear_5", "w"), g("linear_5", "b")

    def norm(self, x):
        return replicated_layer_norm(x, self.ln_s, self.ln_o)

    def qvk_proj(self, x):
        """layers.py:292-297."""
        shp = x.shape[:-1] + (self.H, self.dh)
        return (x @ self.wq).reshape(shp), (x @ self.wv).reshape(shp), (x @ self.wk).reshape(shp)

    def self_attn(self, q, v, k, attn_bias):
        """layers.py:260-285."""
        if self.rot:
            r = self.r
            sincos = fixed_pos_embedding(k.shape[0], r)
            q = torch.cat([apply_rotary_pos_emb(q[:, :, :r], sincos), q[:, :, r:]], -1)
            k = torch.cat([apply_rotary_pos_emb(k[:, :, :r], sincos), k[:, :, r:]], -1)
        s = torch.einsum("thd,Thd->htT", q, k)
        s = s / math.sqrt(self.dh)
        s = s + attn_bias
        w = torch.softmax(s, -1)
        a = torch.einsum("htT,Thd->thd", w, v).reshape(-1, self.H * self.dh)
        return a @ self.wo

    def ff(self, x):
        """layers.py:287-290."""
        return gelu_tanh(x @ self.w1 + self.b1) @ self.w2 + self.b2

    def __call__(self, x, attn_bias=0.0):
        """layers.py:299-313 - returns the residual DELTA."""
        x = self.norm(x)
        q, v, k = self.qvk_proj(x)
        T = x.shape[0]
        bias = MASK * (1.0 - torch.tril(torch.ones(T, T, dtype=x.dtype))) + attn_bias
        return self.self_attn(q, v, k, bias) + self.ff(x)

    def get_init_decode_state(self, x, given_length: int, attn_bias=0.0):
        """layers.py:347-366 - causal + left-pad mask; state keeps un-rotated k, v."""
        x = self.norm(x)
        q, v, k = self.qvk_proj(x)
        T = x.shape[0]
        bias = MASK * (1.0 - torch.tril(torch.ones(T, T, dtype=x.dtype)))
        bias = bias - 1e10 * (torch.arange(T) < (T - given_length)).to(x.dtype)
        bias = bias + attn_bias
        out = self.self_attn(q, v, k, bias) + self.ff(x)
        return out, {"k": k, "v": v, "tokens_decoded": int(given_length)}

    def decode_once(self, state, x, attn_bias=0.0):
        """layers.py:316-344 - slide the window by one, mask the still-empty slots."""
        x = self.norm(x)
        assert x.shape[0] == 1
        q, v, k = self.qvk_proj(x)
        v = torch.cat((state["v"], v), 0)[1:]
        k = torch.cat((state["k"], k), 0)[1:]
        tokens_decoded = state["tokens_decoded"] + 1
        length = v.shape[0]
        bias = MASK * (torch.arange(length) < (length - tokens_decoded)).to(x.dtype) + attn_bias
        out = self.self_attn(q, v, k, bias) + self.ff(x)
        return out, {"tokens_decoded": tokens_decoded, "k": k, "v": v}


class Model:
    """CausalTransformerShard, transformer_shard.py:21-115 (generate path only)."""

    def __init__(self, cfg, params, dtype=torch.float64):
        assert cfg.get("cores_per_replica", 1) == 1
        assert cfg.get("norm", "layernorm") == "layernorm" and cfg.get("pe", "rotary") in ("rotary",)
        self.cfg, self.dtype = cfg, dtype
        self.we, self.be = params[EMBED]["w"][0].to(dtype), params[EMBED]["b"][0].to(dtype)
        self.layers = [Layer(cfg, params, i, dtype) for i in range(cfg["layers"])]
        self.pln_s, self.pln_o = params[PROJ_LN]["scale"][0].to(dtype), params[PROJ_LN]["offset"][0].to(dtype)
        self.wp, self.bp = params[PROJ]["w"][0].to(dtype), params[PROJ]["b"][0].to(dtype)

    def embed(self, tokens):
        return embedding_shard(torch.as_tensor(np.asarray(tokens).astype(np.int64)), self.we, self.be)

    def proj(self, x):
        """ProjectionShard.__call__, layers.py:561-567."""
        return replicated_layer_norm(x, self.pln_s, self.pln_o) @ self.wp + self.bp

    def forward(self, tokens, taps: Optional[list] = None):
        """Full forward with logits at every position (embed -> layers -> proj), the
        composition used by transformer_shard.py:47-62 without the loss."""
        x = self.embed(tokens)
        for l in self.layers:
            x = x + l(x, 0.0)
            if taps is not None:
                taps.append(x.clone())
        return self.proj(x)

    def loss(self, ctx, tgt, ctx_length=None):
        """CausalTransformerShard.eval/loss (transformer_shard.py:47-72) under the evaluation mask
        (arange > ctx_length) * -1e10 on the keys (:130), then ProjectionShard.loss (layers.py:569-593) with
        z_loss = 0: loss = log(sum exp(l - max)) - (l[target] - max), correct = (l[target] - max == 0)."""
        T = len(ctx)
        L = T if ctx_length is None else int(ctx_length)
        mask = (torch.arange(T) > L).to(self.dtype) * -1e10
        x = self.embed(ctx)
        for l in self.layers:
            x = x + l(x, mask)
        logits = self.proj(x)
        logits = logits - logits.max(-1, keepdim=True).values
        pred = logits[torch.arange(T), torch.as_tensor(np.asarray(tgt).astype(np.int64))]
        all_loss = torch.log(torch.exp(logits).sum(-1)) - pred
        return {"loss": all_loss.mean(), "last_loss": all_loss[-1], "all_loss": all_loss, "correct": pred == 0.0}

    def generate_initial(self, context, length: int, taps: Optional[list] = None):
        """transformer_shard.py:74-95 - prefill on context[:-1]; context[-1] seeds decode."""
        last = np.asarray(context[-1:]).astype(np.uint32)
        x = self.embed(context[:-1])
        states = []
        for l in self.layers:
            res, st = l.get_init_decode_state(x, length - 1, 0.0)
            x = x + res
            states.append(st)
            if taps is not None:
                taps.append(x.clone())
        return last, states

    def generate_once(self, new_tok, states, taps: Optional[list] = None):
        """transformer_shard.py:97-115."""
        x = self.embed(new_tok)
        new_states = []
        for l, s in zip(self.layers, states):
            res, st = l.decode_once(s, x, 0.0)
            x = x + res
            new_states.append(st)
            if taps is not None:
                taps.append(x.clone())
        return self.proj(x), new_states

    def generate(self, ctx, ctx_length, gen_length: int, sampler: Callable, sampler_options: dict,
                 uniforms=None, return_logits=False, final_states: Optional[list] = None):
        """transformer_shard.py:190-216,326-339 - per sequence: prefill, then gen_length steps of
        generate_once + sampler.  sampler(u, logits[1,V] float32, **opts) -> uint32 token; `u` is the
        step's host-supplied uniform (stands in for the reference's PRNG key).  final_states, a list, receives
        the decode state each sequence ends with (the carry of transformer_shard.py:196-212)."""
        ctx = np.asarray(ctx)
        B = ctx.shape[0]
        toks = np.zeros((B, gen_length, 1), np.uint32)
        logits_out = np.zeros((B, gen_length, 1, self.cfg["n_vocab"]), np.float32) if return_logits else None
        for b in range(B):
            opts = {k: (None if v is None else np.asarray(v)[b]) for k, v in sampler_options.items()}
            nxt, states = self.generate_initial(ctx[b], int(ctx_length[b]))
            for t in range(gen_length):
                logits, states = self.generate_once(nxt, states)
                lg32 = logits.to(torch.float32).numpy()
                u = None if uniforms is None else float(uniforms[b][t])
                tok = sampler(u, lg32, **opts)
                nxt = np.asarray([tok], np.uint32)
                toks[b, t, 0] = tok
                if return_logits:
                    logits_out[b, t] = lg32
            if final_states is not None:      # the scan's last carry of this sequence: per-layer {k, v, tokens_decoded}
                final_states.append(states)
        return (toks, None, logits_out) if return_logits else (toks, None)


# ----------------------------------------------------------------------------
# sampling (sampling.py:6-44)
# ----------------------------------------------------------------------------
def descending_order(logits_row: np.ndarray) -> np.ndarray:
    """sampling.py:12 - argsort ascending (stable) then reversed: among equal logits the
    HIGHER token id comes first."""
    return np.argsort(logits_row, kind="stable")[::-1]


def nucleaus_filter(logits: np.ndarray, top_p=0.9, top_k=None, acc=np.float64) -> np.ndarray:
    """sampling.py:10-38 on float32 logits [1, V] (raw, un-tempered).

    The softmax and its running sum are evaluated in `acc` precision; the contract
    shared with the HIP kernel is acc=float64 (a keep/remove decision then differs from
    the exact real-number result only if a cumulative mass lies within ~1e-15 of top_p;
    the kernel sums the float64 weights exactly as integers of 2^-62, which moves a sum
    by less than 1.4e-14, so the two agree unless a running sum is that close to its threshold).
    top_p == 1.0 exactly is such a case by construction (the total mass is 1 up to rounding, so
    tail tokens may be removed depending on summation order); "keep everything" is top_p > 1.
    Returns the filtered float32 logits in token order."""
    logits = np.array(logits, np.float32, copy=True)
    assert logits.ndim == 2
    out = logits.copy()
    for i in range(logits.shape[0]):
        row = logits[i]
        order = descending_order(row)
        srt = row[order].astype(acc)
        e = np.exp(srt - srt[0])
        cum = np.cumsum(e / e.sum(dtype=acc), dtype=acc)
        if top_k is not None:
            # sampling.py:15-26 - the subtracted value is 1e10 * token_id for ranks >= top_k
            rank_ge_k = np.arange(row.shape[0]) >= int(top_k)
            val = np.where(rank_ge_k, order, 0).astype(np.float32)
            pen = np.zeros_like(row)
            pen[order] = val
            out[i] = out[i] - np.float32(1e10) * pen
        rm_sorted = cum > acc(top_p)
        rm_sorted = np.concatenate(([False], rm_sorted[:-1]))   # sampling.py:29-30
        rm = np.zeros(row.shape[0], bool)
        rm[order] = rm_sorted
        out[i] = out[i] - np.float32(1e10) * rm.astype(np.float32)
    return out


def keep_mask(logits: np.ndarray, top_p=0.9, top_k=None) -> np.ndarray:
    """True where nucleaus_filter leaves a token reachable (penalty 0)."""
    f = nucleaus_filter(logits, top_p, top_k)
    return f == np.asarray(logits, np.float32)


def inverse_cdf_draw(logits: np.ndarray, filtered: np.ndarray, temp, u: float) -> int:
    """Replacement for jax.random.categorical(key, filtered / temp) (sampling.py:6-7):
    walk the tokens in descending order of the RAW logits, weights exp(filtered/temp - max)
    in float64, and return the first token whose running weight exceeds u * total."""
    row, frow = np.asarray(logits, np.float32)[0], np.asarray(filtered, np.float32)[0]
    order = descending_order(row)
    t = frow[order].astype(np.float64) / np.float64(temp)
    e = np.exp(t - t.max())
    cum = np.cumsum(e, dtype=np.float64)
    j = int(np.searchsorted(cum, np.float64(u) * cum[-1], side="right"))
    if j >= row.shape[0]:
        j = int(np.nonzero(e > 0)[0][-1])
    return int(order[j])


def nucleaus_sample(u, logits, top_p=0.9, temp=1.0, top_k=None) -> int:
    """sampling.py:41-44 with the draw replaced: filter on raw logits, temperature after."""
    f = nucleaus_filter(logits, top_p, top_k)
    return inverse_cdf_draw(logits, f, temp, u)


def softmax_sample(u, logits, temp=1.0) -> int:
    """sampling.py:6-7 with the draw replaced: categorical over softmax(logits / temp), nothing filtered."""
    return inverse_cdf_draw(logits, np.asarray(logits, np.float32), temp, u)


def greedy_sample(u, logits, **_) -> int:
    """argmax through the sampler contract (transformer_shard.py:203); lowest id on ties."""
    return int(np.argmax(np.asarray(logits)[0]))

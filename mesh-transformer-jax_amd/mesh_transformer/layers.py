"""Module-level surface of the reference's mesh_transformer/layers.py for the GPT-J path
(ReplicatedLayerNorm, EmbeddingShard, TransformerLayerShard, ProjectionShard, rotary helpers), as thin
wrappers over the HIP kernels so that every seam of the model can be compared on its own.

The reference modules are haiku modules: their constructors take (config, name, ...) and the parameters come from
the enclosing hk.transform.  The constructors here have the reference's positional arguments; the parameter tree
(haiku names, leading shard axis of 1) comes from the enclosing `with layers.transform(tree):` block - the stand-in
for hk.transform(...).apply(params, ...) - or from the keyword-only `params=` argument.
Inputs and outputs are float32 CUDA tensors shaped like the reference's per-sequence arrays
([tokens, d_model]); attn_bias must be 0 (only pe == "rotary" is on this path).
The kernels are reached through the torch.ops.mtj operators (mesh_transformer.ops) and the engine.
"""
import contextlib

import numpy as np
import torch

from . import ops  # noqa: F401  (registers torch.ops.mtj.*)
from .engine import ROOT, Engine, _f32, rotary_tables

_AMBIENT = []


@contextlib.contextmanager
def transform(params):
    """Parameter scope of the modules constructed inside it (what hk.transform(...).apply(params, ...) provides)."""
    _AMBIENT.append(params)
    try:
        yield params
    finally:
        _AMBIENT.pop()


def _tree(params):
    if params is not None:
        return params
    if _AMBIENT:
        return _AMBIENT[-1]
    raise RuntimeError("no parameters in scope: construct the module inside `with layers.transform(tree):` or pass params=")


def fixed_pos_embedding(x, seq_dim=0):
    """layers.py:128-134: float64 sin/cos tables [n_pos, dim/2] for the last axis of x."""
    dim = x.shape[-1]
    inv_freq = 1.0 / (10000 ** (np.arange(0, dim, 2) / dim))
    ang = np.einsum("i,j->ij", np.arange(x.shape[seq_dim]), inv_freq)
    return np.sin(ang), np.cos(ang)


def _dev(x):
    if not torch.cuda.is_available():
        raise RuntimeError("mesh_transformer.layers runs on an MI355X; no GPU is visible")
    return x.device if isinstance(x, torch.Tensor) and x.is_cuda else torch.device("cuda:0")


def _f32_in(x, dev):
    return torch.as_tensor(x).to(dev, torch.float32).contiguous()


class ReplicatedLayerNorm:
    """layers.py:12-36: ReplicatedLayerNorm(offset=True).  Its parameters {"scale", "offset"} ([1, d] each) are the
    module `name` of the tree in scope (default: the projection's LayerNorm), or `params=` directly."""

    def __init__(self, offset=True, *, params=None, name=ROOT + "projection_shard/~/replicated_layer_norm"):
        self.offset = offset
        self.params = params if params is not None else _tree(None)[name]

    def __call__(self, inputs):
        dev = _dev(inputs)
        x = _f32_in(inputs, dev)
        scale = _f32(torch.as_tensor(self.params["scale"]).to(dev).reshape(-1))
        off = _f32(torch.as_tensor(self.params["offset"]).to(dev).reshape(-1)) if self.offset else torch.zeros_like(scale)
        with torch.cuda.device(dev):
            return torch.ops.mtj.layernorm(x, scale, off, 0)


class EmbeddingShard:
    """layers.py:165-202 with pe == "rotary" (no positional table)."""

    def __init__(self, config, name=None, *, params=None):
        assert config["n_vocab"] % config.get("cores_per_replica", 1) == 0     # layers.py:172
        self.config = config
        p = _tree(params)[ROOT + "embedding_shard/~/linear"]
        self.w, self.b = p["w"], p["b"]

    def __call__(self, x, dtype=None):
        dev = _dev(self.w)
        w = torch.as_tensor(self.w).to(dev)[0].contiguous()
        b = _f32(torch.as_tensor(self.b).to(dev)[0])
        tok = torch.as_tensor(np.asarray(x).astype(np.int32) if not isinstance(x, torch.Tensor) else x.to(torch.int32)).to(dev)
        with torch.cuda.device(dev):
            return torch.ops.mtj.embed(tok.reshape(-1).contiguous(), w, b)


def _mask_geometry(attn_bias, t, T):
    """What the kernels can apply of an additive attention bias [.., t, T]: the causal mask, plus `pad` masked leading
    keys (the -1e10 terms that __call__, get_init_decode_state and decode_once build, layers.py:299-366).
    Returns pad; anything else is not on this path."""
    b = np.asarray(attn_bias.cpu() if isinstance(attn_bias, torch.Tensor) else attn_bias, dtype=np.float64)
    if b.ndim == 0 or b.size == 1:
        if float(b.reshape(-1)[0]) != 0.0:
            raise NotImplementedError("a constant attention bias is not on the GPT-J path")
        if t != 1:
            raise NotImplementedError("attention without a causal mask (attn_bias = 0 on more than one query) has no kernel")
        return 0
    if b.shape[-1] != T or (b.ndim >= 2 and b.shape[-2] != t):
        raise ValueError(f"attn_bias must broadcast to [heads, {t}, {T}]")
    b = b.reshape(-1, t, T) if b.ndim >= 2 else np.broadcast_to(b, (1, t, T))
    masked = b[0] < -1e9
    if np.any(b != b[:1]) or np.any((b[0] != 0.0) & ~masked):
        raise NotImplementedError("only masks of 0 / -1e10 shared by all heads are on the GPT-J path")
    last = masked[-1]
    pad = int(np.argmin(last)) if not last.all() else T
    want = np.arange(T)[None, :] < pad
    if t == T and T > 1:
        want = want | (np.arange(T)[None, :] > np.arange(T)[:, None])
    elif t != 1:
        raise NotImplementedError("self_attn runs a whole window (t == T) or one new token (t == 1)")
    if not np.array_equal(masked, np.broadcast_to(want, (t, T))):
        raise NotImplementedError("attention bias is not causal + left padding")
    return pad


class TransformerLayerShard:
    """layers.py:229-366.  Returns the residual DELTA, like the reference; the caller adds x.

    Decode state: {"k", "v": [1, H, Tcap, dh] device tensors (float32 for a float32 model, float16 for a bfloat16 one;
    k stored rotated,
    slot = position % Tcap), "tokens_decoded": int}.  decode_once updates k and v IN PLACE (the reference
    returns new arrays); the returned dict aliases the same tensors."""

    def __init__(self, config, name=None, init_scale=1.0, *, params=None, device="cuda:0"):
        heads, dim = config["n_heads"], config["d_model"]
        assert dim % heads == 0                                    # layers.py:238
        assert heads % config.get("cores_per_replica", 1) == 0     # layers.py:239
        self.config = config
        self.index = int(name.split("_")[-1]) if name else 0      # transformer_shard.py:37: name=f"layer_{i}"
        self.eng = Engine(config, _tree(params), device, layer_ids=[self.index], embed=False, proj=False)
        self.dim, self.heads, self.dim_per_head = dim, heads, dim // heads
        self.pe_rotary_dims = config.get("pe_rotary_dims", self.dim_per_head)

    # ---- the pieces of the layer (layers.py:260-297) on their own
    def _h(self, x):
        """float32 rows -> the GEMM operand type of this model (float16 saturates, as the kernels' own conversions do)"""
        w = self.eng.w
        x = _f32_in(x, self.eng.device).reshape(-1, w.d)
        return x if w.act_torch_dtype == torch.float32 else x.clamp(-65504.0, 65504.0).to(w.act_torch_dtype)

    def _scratch(self, T):
        """Buffers of the piecewise entry points: a session of its own, so that the window of a live decode state (which
        belongs to the engine's sessions) is never touched."""
        from .engine import Session
        ses = getattr(self, "_scratch_ses", None)
        if ses is None or ses.Tcap != T:
            self._scratch_ses = ses = None
            ses = self._scratch_ses = Session(self.eng, 1, T, T, T + 1)
        return ses

    def qvk_proj(self, x):
        """layers.py:292-297: q, v, k = x @ Wq, x @ Wv, x @ Wk (no bias) as [..., heads, d_head]; x is the LayerNorm output."""
        eng, w = self.eng, self.eng.w
        lead = tuple(np.shape(x)[:-1])
        with torch.cuda.device(eng.device):
            h = self._h(x)
            out = torch.ops.mtj.gemm(h, w.w_in_mm[self.index][:3 * w.d], None, w.alpha_in[self.index], 0)  # rows q|v|k
        d = w.d
        return tuple(out[:, j * d:(j + 1) * d].reshape(lead + (self.heads, self.dim_per_head)) for j in range(3))

    def self_attn(self, q, v, k, attn_bias):
        """layers.py:260-285: rotary embedding of q and k at the window indices (q on the last rows), scores / sqrt(d_head)
        + attn_bias, softmax, weighted values, output projection.  q [t, H, dh], v and k [T, H, dh] float32 and NOT yet
        rotated; attn_bias must be what the layer drivers build: the causal mask (t == T) or none (t == 1), plus masked
        leading keys.  Query rows that are themselves padding come back as the projection of zeros."""
        eng, w, i = self.eng, self.eng.w, self.index
        dev, H, dh, d = eng.device, self.heads, self.dim_per_head, w.d
        q, v, k = (_f32_in(a, dev) for a in (q, v, k))
        t, T = q.shape[0], k.shape[0]
        pad = _mask_geometry(attn_bias, t, T)
        A = w.act_dtype
        with torch.cuda.device(dev):
            ses = self._scratch(T)
            kv_pos0 = torch.tensor([-pad], dtype=torch.int32, device=dev)
            if t == T and T > 1:
                torch.ops.mtj.rope_append_(q.reshape(T, d), v.reshape(T, d), k.reshape(T, d), kv_pos0, ses.sin, ses.cos,
                                           ses.q_pf, ses.kc[i], ses.vc[i], ses.vt, H, self.pe_rotary_dims, T, ses.ldvt)
                att = torch.ops.mtj.attn_prefill(ses.q_pf, ses.kc[i], ses.vt.view(1, H, dh, ses.ldvt), kv_pos0, T, None)
            else:
                q_pos = torch.tensor([T - 1 - pad], dtype=torch.int32, device=dev)
                torch.ops.mtj.rope_append_(None, v.reshape(T, d), k.reshape(T, d), kv_pos0, ses.sin, ses.cos, None,
                                           ses.kc[i], ses.vc[i], None, H, self.pe_rotary_dims, T, 0)
                torch.ops.mtj.rope_append_(q.reshape(1, d), None, None, q_pos, ses.sin, ses.cos, ses.q, None, None, None,
                                           H, self.pe_rotary_dims, 1, 0)
                att = torch.ops.mtj.attn_decode(ses.q, ses.kc[i], ses.vc[i], q_pos, A)
            # out projection: the out | fc_out matrix on [attention | 0]
            act = ses.act_pf[:t]
            act.zero_()
            act[:, :d].copy_(att)
            out = torch.zeros(t, d, dtype=torch.float32, device=dev)
            torch.ops.mtj.gemm_resid_(out, act, w.w_out_mm[i], None, w.alpha_out[i])
        return out

    def ff(self, x):
        """layers.py:287-290: gelu(x @ W1 + b1) @ W2 + b2 (tanh gelu); x is the LayerNorm output, [T, d]."""
        eng, w, i = self.eng, self.eng.w, self.index
        dev, d = eng.device, w.d
        with torch.cuda.device(dev):
            h = self._h(x)
            T = h.shape[0]
            ses = self._scratch(T)
            act = ses.act_pf[:T]
            pos0 = torch.zeros(1, dtype=torch.int32, device=dev)
            # the fused q|v|k|fc_in launch: its fc_in columns are gelu(x @ W1 + b1); q, k, v land in the scratch window
            torch.ops.mtj.inproj_(h, w.w_in_mm[i], w.b1[i], w.alpha_in[i], pos0, ses.sin, ses.cos, ses.q_pf, ses.kc[i],
                                  ses.vc[i], None, act, self.heads, self.pe_rotary_dims, T, 0)
            act[:, :d].zero_()
            out = torch.zeros(T, d, dtype=torch.float32, device=dev)
            torch.ops.mtj.gemm_resid_(out, act, w.w_out_mm[i], w.b2[i], w.alpha_out[i])
        return out

    # ---- whole-layer entry points
    def _prefill(self, x, given_length):
        eng, w = self.eng, self.eng.w
        x = _f32_in(x, eng.device)
        T = x.shape[0]
        with torch.cuda.device(eng.device):
            ses = eng.session(1, max(T, 1), T, T + 1)
            pad = T - int(given_length)
            pos0 = torch.tensor([-pad], dtype=torch.int32, device=eng.device)
            delta = torch.zeros(T, w.d, dtype=torch.float32, device=eng.device)
            # the layer kernels add into a residual stream: run them on a copy and subtract
            xs = x.clone()
            eng.layer_prefill(ses, self.index, xs, ses.h_pf[:T], ses.act_pf[:T], T, pos0)
            delta = xs - x
        return delta, ses, pad

    def __call__(self, x, attn_bias=0):
        assert np.all(np.asarray(attn_bias) == 0), "attn_bias (T5 relative positions) is not on the GPT-J path"
        delta, _, _ = self._prefill(x, x.shape[0])
        return delta

    def get_init_decode_state(self, x, given_length, attn_bias=0):
        assert np.all(np.asarray(attn_bias) == 0)
        delta, ses, pad = self._prefill(x, given_length)
        T = x.shape[0]
        # window of T slots; the given_length real tokens sit at positions 0 .. given_length-1
        state = {"k": ses.kc[self.index], "v": ses.vc[self.index], "tokens_decoded": int(given_length), "_ses": ses}
        return delta, state

    def decode_once(self, decode_state, x, attn_bias=0):
        assert np.all(np.asarray(attn_bias) == 0)
        eng, w = self.eng, self.eng.w
        x = _f32_in(x, eng.device)
        assert x.shape[0] == 1                                     # layers.py:320
        ses = decode_state["_ses"]
        n = int(decode_state["tokens_decoded"])
        with torch.cuda.device(eng.device):
            if ses.max_pos <= n + 1:
                ses.max_pos = 2 * (n + 1)
                ses.sin, ses.cos = rotary_tables(ses.max_pos, eng.r, eng.device)
            ses.pos.fill_(n)                                        # position of the new token
            ses.x.copy_(x)
            eng.layer_decode(ses, self.index)
            delta = ses.x - x
        return delta, {"k": ses.kc[self.index], "v": ses.vc[self.index], "tokens_decoded": n + 1, "_ses": ses}


class ProjectionShard:
    """layers.py:545-567: final LayerNorm + logits projection (the all_gather is the identity at one shard)."""

    def __init__(self, config, name=None, *, params=None, device="cuda:0"):
        assert config["n_vocab"] % config.get("cores_per_replica", 1) == 0     # layers.py:552
        self.eng = Engine(config, _tree(params), device, layer_ids=[], embed=False, proj=True)

    def __call__(self, x):
        eng, w = self.eng, self.eng.w
        x = _f32_in(x, eng.device).reshape(-1, w.d)
        with torch.cuda.device(eng.device):
            h = torch.ops.mtj.layernorm(x, w.pln_s, w.pln_o, w.act_dtype)
            return torch.ops.mtj.gemm(h, w.w_p_mm, w.b_p, w.alpha_p, 0)

    def loss(self, x, targets, z_loss=1):
        """layers.py:569-593: per-row cross entropy of `targets` under the projected logits and `correct` (the target
        holds the row maximum); with z_loss the mean over rows of 1e-4 * z_loss * log(sum exp(logits - max))^2 is added to
        every row.  x float32 [T, d] (before the final LayerNorm), targets [T].  The [T, V] logits are never stored."""
        eng, w = self.eng, self.eng.w
        x = _f32_in(x, eng.device).reshape(-1, w.d)
        tg = torch.as_tensor(np.asarray(targets).astype(np.int32) if not isinstance(targets, torch.Tensor) else targets)
        tg = tg.to(eng.device, torch.int32).reshape(-1).contiguous()
        with torch.cuda.device(eng.device):
            h = torch.ops.mtj.layernorm(x, w.pln_s, w.pln_o, w.act_dtype)
            loss, correct = torch.ops.mtj.gemm_xent(h, w.w_p_mm, w.b_p, w.alpha_p, tg)
            if z_loss:
                # a target outside the vocabulary selects nothing: the loss of such a row is its log-sum-exp
                lse, _ = torch.ops.mtj.gemm_xent(h, w.w_p_mm, w.b_p, w.alpha_p, torch.full_like(tg, -1))
                loss = loss + (1e-4 * float(z_loss)) * lse.square().mean()
        return loss, correct

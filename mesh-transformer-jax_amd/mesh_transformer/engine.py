"""Single-GPU execution engine behind CausalTransformer.generate.

Owns the packed weights, the K/V window, the activation buffers and the HIP-graph of one decode
step.  All arithmetic happens in the HIP kernels reached through _abi; torch is used for device
memory, streams and graph capture only.

Data layout in HBM (T = weight dtype, float32 or bfloat16):
  W_in  [3d+F, d]  T   rows q|v|k|fc_in, K-contiguous   (layers.py:249-251,256)
  W_out [d, d+F]   T   columns out|fc_out               (layers.py:253-254,257-258)
  W_p   [V, d]     T   logits projection                (layers.py:559)
  K, V  [B, H, Tcap, dh] T per layer; K is stored rotated; slot = position % Tcap
  x     [M, d] float32 residual stream; act [M, d+F] = attention output | gelu(fc_in)
"""
import ctypes as C

import numpy as np
import torch

from . import _abi
from ._abi import BF16, EPI_INPROJ, EPI_RESID, EPI_STORE, F32, InProj, NextEmbed, check, ptr

ROOT = "causal_transformer_shard/~/"


def _leaf(tree, mod, name):
    t = tree[ROOT + mod][name]
    if t.dim() < 1 or t.shape[0] != 1:
        raise ValueError(f"{mod}/{name}: expected a leading shard axis of size 1 (cores_per_replica == 1), got {tuple(t.shape)}")
    return t[0]


def _f32(t):
    return t.to(torch.float32).contiguous()


class PackedWeights:
    """Kernel-side view of the haiku tree (names: to_hf_weights.py:160-173)."""

    def __init__(self, config, tree, device, layer_ids=None, embed=True, proj=True):
        L = _abi.lib()
        tree = {m: {k: torch.as_tensor(v).to(device) for k, v in leaves.items()} for m, leaves in tree.items()
                if m.startswith(ROOT)}
        self.d = d = config["d_model"]
        self.F = F = 4 * d
        self.V = V = config["n_vocab"]
        self.layer_ids = list(range(config["layers"])) if layer_ids is None else list(layer_ids)
        self.torch_dtype = next(v for m in tree.values() for k, v in m.items() if k == "w").dtype
        self.dtype = _abi.dtype_code(self.torch_dtype)
        s = _abi.stream_handle()

        def pack(dst, src, k_total, n_off, k_off):
            src = src.contiguous()
            if src.dtype != self.torch_dtype:
                raise ValueError("all weight matrices must share one dtype")
            K, N = src.shape
            check(L.mtj_pack_weight(ptr(src), N, K, N, ptr(dst), k_total, n_off, k_off, self.dtype, s))

        self.we = self.be = self.w_p = self.b_p = self.pln_s = self.pln_o = None
        if embed:
            we = _leaf(tree, "embedding_shard/~/linear", "w")
            if tuple(we.shape) != (V, d):
                raise ValueError(f"embedding weight has shape {tuple(we.shape)}, config says {(V, d)}")
            self.we = we.contiguous()
            self.be = _f32(_leaf(tree, "embedding_shard/~/linear", "b"))
        self.w_in, self.b1, self.w_out, self.b2, self.ln_s, self.ln_o = {}, {}, {}, {}, {}, {}
        for i in self.layer_ids:
            g = lambda mod, name: _leaf(tree, f"layer_{i}/~/{mod}", name)
            if tuple(g("linear_4", "w").shape) != (d, F) or tuple(g("linear", "w").shape) != (d, d):
                raise ValueError(f"layer_{i}: weight shapes do not match d_model={d}")
            w_in = torch.empty(3 * d + F, d, dtype=self.torch_dtype, device=device)
            pack(w_in, g("linear", "w"), d, 0, 0)          # q
            pack(w_in, g("linear_1", "w"), d, d, 0)        # v
            pack(w_in, g("linear_2", "w"), d, 2 * d, 0)    # k
            pack(w_in, g("linear_4", "w"), d, 3 * d, 0)    # fc_in
            w_out = torch.empty(d, d + F, dtype=self.torch_dtype, device=device)
            pack(w_out, g("linear_3", "w"), d + F, 0, 0)   # out
            pack(w_out, g("linear_5", "w"), d + F, 0, d)   # fc_out
            self.w_in[i], self.w_out[i] = w_in, w_out
            self.b1[i], self.b2[i] = _f32(g("linear_4", "b")), _f32(g("linear_5", "b"))
            self.ln_s[i] = _f32(g("replicated_layer_norm", "scale"))
            self.ln_o[i] = _f32(g("replicated_layer_norm", "offset"))
        if proj:
            self.w_p = torch.empty(V, d, dtype=self.torch_dtype, device=device)
            pack(self.w_p, _leaf(tree, "projection_shard/~/linear", "w"), d, 0, 0)
            self.b_p = _f32(_leaf(tree, "projection_shard/~/linear", "b"))
            self.pln_s = _f32(_leaf(tree, "projection_shard/~/replicated_layer_norm", "scale"))
            self.pln_o = _f32(_leaf(tree, "projection_shard/~/replicated_layer_norm", "offset"))


def rotary_tables(n_pos, r, device):
    """fixed_pos_embedding (layers.py:128-134): float64 on the host, rounded once to float32."""
    inv_freq = 1.0 / (10000 ** (np.arange(0, r, 2) / r))
    ang = np.einsum("i,j->ij", np.arange(n_pos), inv_freq)
    sin = torch.from_numpy(np.sin(ang).astype(np.float32)).to(device)
    cos = torch.from_numpy(np.cos(ang).astype(np.float32)).to(device)
    return sin, cos


class Session:
    """Buffers of one (batch, window) geometry: K/V window, activations, sampler scratch."""

    def __init__(self, eng, B, Tcap, Tp_max, max_pos):
        L = _abi.lib()
        cfg, w, dev = eng.config, eng.w, eng.device
        self.B, self.Tcap, self.Tp_max, self.max_pos = B, Tcap, Tp_max, max_pos
        d, F, H, dh, V = w.d, w.F, eng.H, eng.dh, w.V
        T = w.torch_dtype
        self.kc = {i: torch.zeros(B, H, Tcap, dh, dtype=T, device=dev) for i in w.layer_ids}
        self.vc = {i: torch.zeros(B, H, Tcap, dh, dtype=T, device=dev) for i in w.layer_ids}
        self.sin, self.cos = rotary_tables(max_pos, eng.r, dev)
        # prefill buffers
        M = max(B * Tp_max, 1)
        # row length of the transposed-V scratch: a multiple of 64 elements, but never a multiple of 2 KiB in
        # bytes - rows a power-of-two apart all land in the same memory channel
        self.ldvt = max((Tp_max + 63) // 64 * 64, 64)
        if (self.ldvt * (2 if T == torch.bfloat16 else 4)) % 2048 == 0:
            self.ldvt += 64
        self.x_pf = torch.empty(M, d, dtype=torch.float32, device=dev)
        self.h_pf = torch.empty(M, d, dtype=T, device=dev)
        self.act_pf = torch.empty(M, d + F, dtype=T, device=dev)
        self.q_pf = torch.empty(M * d, dtype=T, device=dev)
        self.vt = torch.zeros(B * H * dh * self.ldvt, dtype=T, device=dev)
        # decode buffers
        self.gemv_path = (B == 1)
        act_t = torch.float32 if self.gemv_path else T
        self.x = torch.empty(B, d, dtype=torch.float32, device=dev)
        self.h = torch.empty(B, d, dtype=T, device=dev)
        self.act = torch.zeros(B, d + F, dtype=act_t, device=dev)
        self.q = torch.empty(B, H, dh, dtype=torch.float32, device=dev)
        self.logits = torch.empty(B, V, dtype=torch.float32, device=dev)
        nb = 0 if self.gemv_path else L.mtj_gemm_splitk_work_bytes(B, d, d + F, w.dtype)
        nb = max(nb, L.mtj_gemm_splitk_work_bytes(M, d, d + F, w.dtype))     # the out projection of a short prefill
        self.gemm_work = torch.empty(max(nb, 256), dtype=torch.uint8, device=dev)
        self.attn_work = torch.zeros(max(L.mtj_attn_decode_work_bytes(B, H, dh, Tcap), 256), dtype=torch.uint8, device=dev)
        self.sample_work = None
        self.tok = torch.zeros(B, dtype=torch.int32, device=dev)
        self.pos = torch.zeros(B, dtype=torch.int32, device=dev)
        self.pos_start = torch.zeros(B, dtype=torch.int32, device=dev)
        self.pos0 = torch.zeros(B, dtype=torch.int32, device=dev)
        self.graphs = {}


class Engine:
    def __init__(self, config, tree, device="cuda:0", layer_ids=None, embed=True, proj=True):
        if config.get("cores_per_replica", 1) != 1:
            raise ValueError("this build runs the whole model on one GPU: cores_per_replica must be 1")
        if config.get("norm", "layernorm") != "layernorm":
            raise NotImplementedError("only norm == 'layernorm' is on the GPT-J path")
        if config.get("pe", "rotary") != "rotary":
            raise NotImplementedError("only pe == 'rotary' is on the GPT-J path")
        self.config = config
        self.device = torch.device(device)
        self.H = config["n_heads"]
        d = config["d_model"]
        assert d % self.H == 0                                   # layers.py:238
        self.dh = d // self.H
        self.r = config.get("pe_rotary_dims", self.dh)           # layers.py:244
        if self.dh not in (64, 256):
            raise NotImplementedError(f"d_head {self.dh}: attention kernels exist for 64 and 256")
        if self.r % 2 or self.r > self.dh:
            raise ValueError("pe_rotary_dims must be even and <= d_head")
        with torch.cuda.device(self.device):
            self.w = PackedWeights(config, tree, self.device, layer_ids, embed, proj)
        self.sessions = {}

    # ------------------------------------------------------------------ kernels
    def _inproj(self, ses, layer, Tp, pos0, q, q_dtype, act, act_dtype, vt):
        ip = InProj()
        ip.n_heads, ip.d_head, ip.rotary_dims = self.H, self.dh, self.r
        ip.Tp, ip.Tcap, ip.max_pos = Tp, ses.Tcap, ses.max_pos
        ip.pos0, ip.sin_tab, ip.cos_tab = ptr(pos0), ptr(ses.sin), ptr(ses.cos)
        ip.q, ip.q_dtype = ptr(q), q_dtype
        ip.k_cache, ip.v_cache = ptr(ses.kc[layer]), ptr(ses.vc[layer])
        ip.v_t, ip.ldvt = (ptr(vt), ses.ldvt) if vt is not None else (None, 0)
        ip.act, ip.ld_act, ip.act_dtype = ptr(act), act.shape[1], act_dtype
        return ip

    def prefill(self, ses, tokens_rect, Tp, key_limit=None):
        """generate_initial (transformer_shard.py:74-95) on a [B, Tp] right-aligned rectangle; the
        dead logits projection of :95 is not computed."""
        L, w, s = _abi.lib(), self.w, _abi.stream_handle()
        B, d, F = ses.B, w.d, w.F
        M = B * Tp
        x, h, act = ses.x_pf[:M], ses.h_pf[:M], ses.act_pf[:M]
        check(L.mtj_embed(ptr(tokens_rect), M, ptr(w.we), ptr(w.be), w.V, d, w.dtype, ptr(x), s))
        for i in w.layer_ids:
            self.layer_prefill(ses, i, x, h, act, Tp, ses.pos0, key_limit)
        return x

    def project(self, ses, x, out):
        """ProjectionShard.__call__ (layers.py:561-567) on every row of x: out [M, V] float32."""
        L, w, s = _abi.lib(), self.w, _abi.stream_handle()
        M, d, V = x.shape[0], w.d, w.V
        h = ses.h_pf[:M]
        check(L.mtj_layernorm(ptr(x), ptr(w.pln_s), ptr(w.pln_o), M, d, ptr(h), w.dtype, s))
        check(L.mtj_gemm(ptr(h), d, ptr(w.w_p), ptr(w.b_p), M, V, d, w.dtype, EPI_STORE, ptr(out), V, F32, None, s))

    def layer_prefill(self, ses, i, x, h, act, Tp, pos0, key_limit=None):
        L, w, s = _abi.lib(), self.w, _abi.stream_handle()
        M, d, F = x.shape[0], w.d, w.F
        check(L.mtj_layernorm(ptr(x), ptr(w.ln_s[i]), ptr(w.ln_o[i]), M, d, ptr(h), w.dtype, s))
        ip = self._inproj(ses, i, Tp, pos0, ses.q_pf, w.dtype, act, w.dtype, ses.vt)
        check(L.mtj_gemm(ptr(h), d, ptr(w.w_in[i]), ptr(w.b1[i]), M, 3 * d + F, d, w.dtype, EPI_INPROJ,
                         None, 0, 0, C.byref(ip), s))
        check(L.mtj_attn_prefill(ptr(ses.q_pf), ptr(ses.kc[i]), ptr(ses.vt), ptr(pos0), ses.B, self.H, Tp, ses.Tcap,
                                 self.dh, ses.ldvt, ptr(act), d + F, w.dtype, ptr(key_limit), s))
        check(L.mtj_gemm_splitk(ptr(act), d + F, ptr(w.w_out[i]), ptr(w.b2[i]), M, d, d + F, w.dtype, EPI_RESID,
                                ptr(x), d, F32, ptr(ses.gemm_work), ses.gemm_work.numel(), s))

    def embed_tok(self, ses):
        """x = EmbeddingShard(tok) for the decode step that follows."""
        w = self.w
        check(_abi.lib().mtj_embed(ptr(ses.tok), ses.B, ptr(w.we), ptr(w.be), w.V, w.d, w.dtype, ptr(ses.x),
                                   _abi.stream_handle()))

    def _next(self, ses, fuse):
        if not fuse:
            return None
        w = self.w
        ne = NextEmbed()
        ne.w, ne.bias, ne.x_next, ne.d, ne.dtype = ptr(w.we), ptr(w.be), ptr(ses.x), w.d, w.dtype
        return C.byref(ne)

    def decode_model(self, ses):
        """generate_once (transformer_shard.py:97-115) from the embedded token in ses.x to the logits; the K/V
        window is updated in place."""
        L, w, s = _abi.lib(), self.w, _abi.stream_handle()
        B, d, F, V = ses.B, w.d, w.F, w.V
        if not ses.gemv_path and w.w_p is not None:
            # batched decode: the reduce of every out projection also applies the LayerNorm that follows it (the
            # next layer's, at the end the projection's), so only the first layer launches a LayerNorm of its own
            ids = w.layer_ids
            check(L.mtj_layernorm(ptr(ses.x), ptr(w.ln_s[ids[0]]), ptr(w.ln_o[ids[0]]), B, d, ptr(ses.h), w.dtype, s))
            for j, i in enumerate(ids):
                nxt = (w.ln_s[ids[j + 1]], w.ln_o[ids[j + 1]]) if j + 1 < len(ids) else (w.pln_s, w.pln_o)
                self.layer_decode(ses, i, normed=True, next_ln=nxt)
            check(L.mtj_gemm(ptr(ses.h), d, ptr(w.w_p), ptr(w.b_p), B, V, d, w.dtype, EPI_STORE, ptr(ses.logits), V,
                             F32, None, s))
            return
        for i in w.layer_ids:
            self.layer_decode(ses, i)
        if ses.gemv_path:
            check(L.mtj_gemv(ptr(ses.x), ptr(w.pln_s), ptr(w.pln_o), ptr(w.w_p), ptr(w.b_p), V, d, w.dtype, EPI_STORE,
                             ptr(ses.logits), F32, None, s))
        else:
            check(L.mtj_layernorm(ptr(ses.x), ptr(w.pln_s), ptr(w.pln_o), B, d, ptr(ses.h), w.dtype, s))
            check(L.mtj_gemm(ptr(ses.h), d, ptr(w.w_p), ptr(w.b_p), B, V, d, w.dtype, EPI_STORE, ptr(ses.logits), V,
                             F32, None, s))

    def layer_decode(self, ses, i, normed=False, next_ln=None):
        """decode_once of layer i plus the residual add.  normed: ses.h already holds LayerNorm_i(ses.x); next_ln:
        (scale, offset) of the LayerNorm that follows the residual add, applied into ses.h by the same launch."""
        L, w, s = _abi.lib(), self.w, _abi.stream_handle()
        B, d, F = ses.B, w.d, w.F
        if ses.gemv_path:
            ip = self._inproj(ses, i, 1, ses.pos, ses.q, F32, ses.act, F32, None)
            check(L.mtj_gemv(ptr(ses.x), ptr(w.ln_s[i]), ptr(w.ln_o[i]), ptr(w.w_in[i]), ptr(w.b1[i]), 3 * d + F, d,
                             w.dtype, EPI_INPROJ, None, 0, C.byref(ip), s))
            check(L.mtj_attn_decode(ptr(ses.q), ptr(ses.kc[i]), ptr(ses.vc[i]), ptr(ses.pos), B, self.H, ses.Tcap,
                                    self.dh, ptr(ses.act), d + F, F32, w.dtype, ptr(ses.attn_work), s))
            check(L.mtj_gemv(ptr(ses.act), None, None, ptr(w.w_out[i]), ptr(w.b2[i]), d, d + F, w.dtype, EPI_RESID,
                             ptr(ses.x), F32, None, s))
        else:
            if not normed:
                check(L.mtj_layernorm(ptr(ses.x), ptr(w.ln_s[i]), ptr(w.ln_o[i]), B, d, ptr(ses.h), w.dtype, s))
            ip = self._inproj(ses, i, 1, ses.pos, ses.q, F32, ses.act, w.dtype, None)
            check(L.mtj_gemm(ptr(ses.h), d, ptr(w.w_in[i]), ptr(w.b1[i]), B, 3 * d + F, d, w.dtype, EPI_INPROJ,
                             None, 0, 0, C.byref(ip), s))
            check(L.mtj_attn_decode(ptr(ses.q), ptr(ses.kc[i]), ptr(ses.vc[i]), ptr(ses.pos), B, self.H, ses.Tcap,
                                    self.dh, ptr(ses.act), d + F, w.dtype, w.dtype, ptr(ses.attn_work), s))
            if next_ln is not None:
                check(L.mtj_gemm_splitk_ln(ptr(ses.act), d + F, ptr(w.w_out[i]), ptr(w.b2[i]), B, d, d + F, w.dtype,
                                           ptr(ses.x), d, ptr(ses.gemm_work), ses.gemm_work.numel(), ptr(next_ln[0]),
                                           ptr(next_ln[1]), ptr(ses.h), d, w.dtype, s))
            else:
                check(L.mtj_gemm_splitk(ptr(ses.act), d + F, ptr(w.w_out[i]), ptr(w.b2[i]), B, d, d + F, w.dtype,
                                        EPI_RESID, ptr(ses.x), d, F32, ptr(ses.gemm_work), ses.gemm_work.numel(), s))

    def sample_greedy(self, ses, out_tokens, embed_next=True):
        check(_abi.lib().mtj_sample_greedy(ptr(ses.logits), ses.B, self.w.V, ptr(ses.tok), ptr(out_tokens),
                                           out_tokens.shape[1], ptr(ses.pos), ptr(ses.pos_start),
                                           self._next(ses, embed_next), _abi.stream_handle()))

    def sample_nucleus(self, ses, out_tokens, top_p, temp, top_k, uniforms, keep_mask=None, filtered=None,
                       embed_next=True):
        L = _abi.lib()
        if ses.sample_work is None:
            ses.sample_work = torch.empty(L.mtj_sample_work_bytes(ses.B, self.w.V), dtype=torch.uint8, device=self.device)
        check(L.mtj_sample_nucleus(ptr(ses.logits), ses.B, self.w.V, ptr(top_p), ptr(temp), ptr(top_k), ptr(uniforms),
                                   uniforms.shape[1], ptr(ses.tok), ptr(out_tokens), out_tokens.shape[1], ptr(ses.pos),
                                   ptr(ses.pos_start), ptr(keep_mask), ptr(filtered), ptr(ses.sample_work),
                                   self._next(ses, embed_next), _abi.stream_handle()))

    # ------------------------------------------------------------------ sessions
    def session(self, B, Tcap, Tp_max, max_pos):
        key = (B, Tcap)
        ses = self.sessions.get(key)
        if ses is None or ses.Tp_max < Tp_max or ses.max_pos < max_pos:
            self.sessions.pop(key, None)
            ses = None
            torch.cuda.empty_cache()
            ses = Session(self, B, Tcap, max(Tp_max, 1), max_pos)
            self.sessions[key] = ses
        return ses

"""Single-GPU execution engine behind CausalTransformer.generate.

Owns the packed weights, the K/V window, the activation buffers and the HIP-graph of one decode
step.  All arithmetic happens in the HIP kernels reached through _abi; torch is used for device
memory, streams and graph capture only.

Data layout in HBM (T = weight dtype, float32 or bfloat16; A = float32 for a float32 model, float16 for a
bfloat16 one: the 16-bit storage type of activations, K/V and the matrix-core operands):
  W_in  [3d+F, d]  T   rows q|v|k|fc_in, K-contiguous   (layers.py:249-251,256)
  W_out [d, d+F]   T   columns out|fc_out               (layers.py:253-254,257-258)
  W_p   [V, d]     T   logits projection                (layers.py:559)
  the same three in A (times a power of two) for the matrix-core GEMMs of a bfloat16 model
  K, V  [B, H, Tcap, dh] A per layer; K is stored rotated; slot = position % Tcap
  x     [M, d] float32 residual stream; act [M, d+F] = attention output | gelu(fc_in)
"""
import ctypes as C

import math

import numpy as np
import torch

from . import _abi
from ._abi import BF16, EPI_INPROJ, EPI_RESID, EPI_STORE, F16, F32, AttnMerge, InProj, NextEmbed, check, ptr

ROOT = "causal_transformer_shard/~/"


def _leaf(tree, mod, name):
    t = tree[ROOT + mod][name]
    if t.dim() < 1 or t.shape[0] != 1:
        raise ValueError(f"{mod}/{name}: expected a leading shard axis of size 1 (cores_per_replica == 1), got {tuple(t.shape)}")
    return t[0]


def _f32(t):
    return t.to(torch.float32).contiguous()


def splitk_work_bound(M_max, N, K, dtype):
    """Bytes of split-K workspace that cover every row count 1 .. M_max of an [M, K] x [K, N] product.  The number of
    K ranges falls as M grows, so the need is not monotonic in M; it is constant in the number of ranges between
    multiples of 128 rows (and below 64 rows), so those row counts are the candidates."""
    L = _abi.lib()
    cand = set(range(1, min(M_max, 64) + 1)) | set(range(128, M_max + 1, 128)) | {M_max}
    return max(L.mtj_gemm_splitk_work_bytes(m, N, K, dtype) for m in cand)


class PackedWeights:
    """Kernel-side view of the haiku tree (names: to_hf_weights.py:160-173).

    A bfloat16 tree is packed twice: in bfloat16 for the batch-1 matrix-vector kernels (float32 activations), and in
    float16 for the matrix cores, whose operands must share one 16-bit type: float16 holds every bfloat16 weight
    exactly once the matrix is scaled by a power of two that keeps its largest entry finite, and rounds the
    activation operand to 11 significant bits instead of 8 (the reference multiplies float32 activations,
    jnp.dot(f32, bf16)).  mm_dtype / alpha_* describe those copies; for a float32 tree they are the same tensors."""

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
        if self.dtype not in (F32, BF16):
            raise ValueError("weights must be float32 or bfloat16")
        half = self.dtype == BF16
        self.mm_dtype = F16 if half else F32                      # operands of the matrix-core GEMMs
        self.mm_torch_dtype = torch.float16 if half else torch.float32
        self.act_dtype, self.act_torch_dtype = self.mm_dtype, self.mm_torch_dtype   # activations, q, K/V storage
        s = _abi.stream_handle()

        def pow2_scale(parts):
            """largest power of two that keeps every scaled weight of the matrix below 2^15"""
            amax = max(float(p.abs().max()) for p in parts)
            if not math.isfinite(amax) or amax == 0.0:
                return 1.0
            return 2.0 ** min(math.floor(math.log2(32768.0 / amax)), 24)

        def pack_mm(dst, src, k_total, n_off, k_off, scale):
            src = src.contiguous()
            K, N = src.shape
            check(L.mtj_pack_weight_cvt(ptr(src), N, K, N, ptr(dst), k_total, n_off, k_off, self.dtype, self.mm_dtype,
                                        scale, s))

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
        self.w_in_mm, self.w_out_mm, self.alpha_in, self.alpha_out = {}, {}, {}, {}
        self.w_p_mm, self.alpha_p = None, 1.0
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
            if half:
                parts_in = [g("linear", "w"), g("linear_1", "w"), g("linear_2", "w"), g("linear_4", "w")]
                sc = pow2_scale(parts_in)
                w_in_mm = torch.empty(3 * d + F, d, dtype=self.mm_torch_dtype, device=device)
                for part, off in zip(parts_in, (0, d, 2 * d, 3 * d)):
                    pack_mm(w_in_mm, part, d, off, 0, sc)
                self.w_in_mm[i], self.alpha_in[i] = w_in_mm, 1.0 / sc
                parts_out = [g("linear_3", "w"), g("linear_5", "w")]
                sc = pow2_scale(parts_out)
                w_out_mm = torch.empty(d, d + F, dtype=self.mm_torch_dtype, device=device)
                pack_mm(w_out_mm, parts_out[0], d + F, 0, 0, sc)
                pack_mm(w_out_mm, parts_out[1], d + F, 0, d, sc)
                self.w_out_mm[i], self.alpha_out[i] = w_out_mm, 1.0 / sc
            else:
                self.w_in_mm[i], self.w_out_mm[i], self.alpha_in[i], self.alpha_out[i] = w_in, w_out, 1.0, 1.0
            self.b1[i], self.b2[i] = _f32(g("linear_4", "b")), _f32(g("linear_5", "b"))
            self.ln_s[i] = _f32(g("replicated_layer_norm", "scale"))
            self.ln_o[i] = _f32(g("replicated_layer_norm", "offset"))
        if proj:
            self.w_p = torch.empty(V, d, dtype=self.torch_dtype, device=device)
            wp = _leaf(tree, "projection_shard/~/linear", "w")
            pack(self.w_p, wp, d, 0, 0)
            if half:
                sc = pow2_scale([wp])
                self.w_p_mm = torch.empty(V, d, dtype=self.mm_torch_dtype, device=device)
                pack_mm(self.w_p_mm, wp, d, 0, 0, sc)
                self.alpha_p = 1.0 / sc
            else:
                self.w_p_mm = self.w_p
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
        T = w.act_torch_dtype
        self.kc = {i: torch.zeros(B, H, Tcap, dh, dtype=T, device=dev) for i in w.layer_ids}
        self.vc = {i: torch.zeros(B, H, Tcap, dh, dtype=T, device=dev) for i in w.layer_ids}
        self.sin, self.cos = rotary_tables(max_pos, eng.r, dev)
        # prefill buffers
        M = max(B * Tp_max, 1)
        # row length of the transposed-V scratch: a multiple of 64 elements, but never a multiple of 2 KiB in
        # bytes - rows a power-of-two apart all land in the same memory channel
        self.ldvt = max((Tp_max + 63) // 64 * 64, 64)
        if (self.ldvt * (4 if T == torch.float32 else 2)) % 2048 == 0:
            self.ldvt += 64
        self.x_pf = torch.empty(M, d, dtype=torch.float32, device=dev)
        self.h_pf = torch.empty(M, d, dtype=T, device=dev)
        # rows of the prefill activations are 128 bytes longer than d + F: with a row pitch that is a multiple of 4 KiB
        # (40960 bytes at the 6B shape) the 256 rows of an operand tile can compete for the same L2 channels (the
        # output GEMM alone, M = 16384: 1013 -> 1107 TFLOP/s with the longer rows; inside a layer the gain is ~1 %)
        self.act_pf = torch.empty(M, d + F + 64, dtype=T, device=dev)[:, :d + F]
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
        # split-K workspace of the out projection: batched decode (B rows) and every prefill this session can see
        # (1 .. B * Tp_max rows; a shorter prompt is cut into MORE K ranges, so the longest one is not the bound)
        nb = 0 if self.gemv_path else L.mtj_gemm_splitk_work_bytes(B, d, d + F, w.mm_dtype)
        nb = max(nb, splitk_work_bound(M, d, d + F, w.mm_dtype))
        self.gemm_work = torch.empty(max(nb, 256), dtype=torch.uint8, device=dev)
        self.attn_work = torch.zeros(max(L.mtj_attn_decode_work_bytes(B, H, dh, Tcap), 256), dtype=torch.uint8, device=dev)
        # batch 1: the out projection computes the attention itself when the shape allows it (its counter block is
        # zeroed here, once, and then only the kernel touches it)
        self.fused_attn = bool(self.gemv_path and cfg.get("fused_decode_attention", True) and
                               L.mtj_gemv_attn_supported(d, d + F, w.dtype, H, dh, w.act_dtype, Tcap))
        self.oa_work = torch.zeros(L.mtj_gemv_attn_work_bytes(H, dh), dtype=torch.uint8, device=dev) if self.fused_attn else None
        self.sample_work = None
        # best-so-far word and arrival counter of the logits launch that is its own greedy sampler (batch 1)
        self.fused_greedy = bool(self.gemv_path and cfg.get("fused_greedy_sampler", True))
        self.greedy_work = torch.zeros(256, dtype=torch.uint8, device=dev) if self.fused_greedy else None
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
        ip.q, ip.q_dtype, ip.kv_dtype = ptr(q), q_dtype, self.w.act_dtype
        ip.k_cache, ip.v_cache = ptr(ses.kc[layer]), ptr(ses.vc[layer])
        ip.v_t, ip.ldvt = (ptr(vt), ses.ldvt) if vt is not None else (None, 0)
        ip.act, ip.ld_act, ip.act_dtype = ptr(act), act.stride(0), act_dtype
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
        check(L.mtj_layernorm(ptr(x), ptr(w.pln_s), ptr(w.pln_o), M, d, ptr(h), w.act_dtype, s))
        check(L.mtj_gemm(ptr(h), d, ptr(w.w_p_mm), ptr(w.b_p), M, V, d, w.mm_dtype, EPI_STORE, ptr(out), V, F32, None,
                         w.alpha_p, s))

    def project_loss(self, ses, x, target, loss, correct):
        """ProjectionShard.loss (layers.py:569-593) on every row of x against target [M] int32: loss [M] float32 and
        correct [M] uint8.  The logits live only in the accumulators of the projection GEMM, whose epilogue keeps
        (max, sum of exp, target logit) per row and column tile."""
        L, w, s = _abi.lib(), self.w, _abi.stream_handle()
        M, d, V = x.shape[0], w.d, w.V
        h = ses.h_pf[:M]
        need = L.mtj_gemm_xent_work_bytes(M, V, w.mm_dtype)
        if getattr(ses, "xent_work", None) is None or ses.xent_work.numel() * 4 < need:
            ses.xent_work = torch.empty((need + 3) // 4, dtype=torch.float32, device=x.device)
        check(L.mtj_layernorm(ptr(x), ptr(w.pln_s), ptr(w.pln_o), M, d, ptr(h), w.act_dtype, s))
        check(L.mtj_gemm_xent(ptr(h), d, ptr(w.w_p_mm), ptr(w.b_p), M, V, d, w.mm_dtype, w.alpha_p, ptr(target),
                              ptr(loss), ptr(correct), ptr(ses.xent_work), ses.xent_work.numel() * 4, s))

    def layer_prefill(self, ses, i, x, h, act, Tp, pos0, key_limit=None):
        L, w, s = _abi.lib(), self.w, _abi.stream_handle()
        M, d, F = x.shape[0], w.d, w.F
        A = w.act_dtype
        check(L.mtj_layernorm(ptr(x), ptr(w.ln_s[i]), ptr(w.ln_o[i]), M, d, ptr(h), A, s))
        ip = self._inproj(ses, i, Tp, pos0, ses.q_pf, A, act, A, ses.vt)
        check(L.mtj_gemm(ptr(h), d, ptr(w.w_in_mm[i]), ptr(w.b1[i]), M, 3 * d + F, d, w.mm_dtype, EPI_INPROJ,
                         None, 0, 0, C.byref(ip), w.alpha_in[i], s))
        check(L.mtj_attn_prefill(ptr(ses.q_pf), ptr(ses.kc[i]), ptr(ses.vt), ptr(pos0), ses.B, self.H, Tp, ses.Tcap,
                                 self.dh, ses.ldvt, ptr(act), act.stride(0), A, ptr(key_limit), s))
        check(L.mtj_gemm_splitk(ptr(act), act.stride(0), ptr(w.w_out_mm[i]), ptr(w.b2[i]), M, d, d + F, w.mm_dtype, EPI_RESID,
                                ptr(x), d, F32, ptr(ses.gemm_work), ses.gemm_work.numel(), w.alpha_out[i], s))

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

    def decode_model(self, ses, logits=None, greedy_out=None, embed_next=True):
        """generate_once (transformer_shard.py:97-115) from the embedded token in ses.x to the logits (ses.logits, or
        the [B, V] float32 tensor given); the K/V window is updated in place.  With greedy_out (the [B, G] token
        buffer) the batch-1 logits launch also is the greedy sampler - sample_greedy's effects are then already in
        place and the call returns True; otherwise (batched decode) it returns False and the caller samples."""
        L, w, s = _abi.lib(), self.w, _abi.stream_handle()
        B, d, F, V = ses.B, w.d, w.F, w.V
        logits = ses.logits if logits is None else logits
        if not ses.gemv_path and w.w_p is not None:
            # batched decode: the reduce of every out projection also applies the LayerNorm that follows it (the
            # next layer's, at the end the projection's), so only the first layer launches a LayerNorm of its own
            ids = w.layer_ids
            check(L.mtj_layernorm(ptr(ses.x), ptr(w.ln_s[ids[0]]), ptr(w.ln_o[ids[0]]), B, d, ptr(ses.h), w.act_dtype, s))
            for j, i in enumerate(ids):
                nxt = (w.ln_s[ids[j + 1]], w.ln_o[ids[j + 1]]) if j + 1 < len(ids) else (w.pln_s, w.pln_o)
                self.layer_decode(ses, i, normed=True, next_ln=nxt)
            check(L.mtj_gemm(ptr(ses.h), d, ptr(w.w_p_mm), ptr(w.b_p), B, V, d, w.mm_dtype, EPI_STORE, ptr(logits), V,
                             F32, None, w.alpha_p, s))
            return False
        for i in w.layer_ids:
            self.layer_decode(ses, i)
        if ses.fused_greedy and greedy_out is not None:
            check(L.mtj_gemv_greedy(ptr(ses.x), ptr(w.pln_s), ptr(w.pln_o), ptr(w.w_p), ptr(w.b_p), V, d, w.dtype,
                                    ptr(logits), ptr(ses.tok), ptr(greedy_out), greedy_out.shape[1], ptr(ses.pos),
                                    ptr(ses.pos_start), self._next(ses, embed_next), ptr(ses.greedy_work), s))
            return True
        if ses.gemv_path:
            check(L.mtj_gemv(ptr(ses.x), ptr(w.pln_s), ptr(w.pln_o), ptr(w.w_p), ptr(w.b_p), V, d, w.dtype, EPI_STORE,
                             ptr(logits), F32, None, None, s))
        else:
            check(L.mtj_layernorm(ptr(ses.x), ptr(w.pln_s), ptr(w.pln_o), B, d, ptr(ses.h), w.act_dtype, s))
            check(L.mtj_gemm(ptr(ses.h), d, ptr(w.w_p_mm), ptr(w.b_p), B, V, d, w.mm_dtype, EPI_STORE, ptr(logits), V,
                             F32, None, w.alpha_p, s))

    def layer_decode(self, ses, i, normed=False, next_ln=None):
        """decode_once of layer i plus the residual add.  normed: ses.h already holds LayerNorm_i(ses.x); next_ln:
        (scale, offset) of the LayerNorm that follows the residual add, applied into ses.h by the same launch."""
        L, w, s = _abi.lib(), self.w, _abi.stream_handle()
        B, d, F = ses.B, w.d, w.F
        if ses.gemv_path:
            ip = self._inproj(ses, i, 1, ses.pos, ses.q, F32, ses.act, F32, None)
            check(L.mtj_gemv(ptr(ses.x), ptr(w.ln_s[i]), ptr(w.ln_o[i]), ptr(w.w_in[i]), ptr(w.b1[i]), 3 * d + F, d,
                             w.dtype, EPI_INPROJ, None, 0, C.byref(ip), None, s))
            if ses.fused_attn:
                check(L.mtj_gemv_attn(ptr(ses.act), ptr(w.w_out[i]), ptr(w.b2[i]), d, d + F, w.dtype, ptr(ses.x), ptr(ses.q),
                                      ptr(ses.kc[i]), ptr(ses.vc[i]), ptr(ses.pos), self.H, ses.Tcap, self.dh, w.act_dtype,
                                      ptr(ses.oa_work), s))
                return
            # the per-range attention partials are merged by the out projection while it stages its input
            am = AttnMerge()
            check(L.mtj_attn_decode_partials(ptr(ses.q), ptr(ses.kc[i]), ptr(ses.vc[i]), ptr(ses.pos), B, self.H, ses.Tcap,
                                             self.dh, w.act_dtype, ptr(ses.attn_work), C.byref(am), s))
            check(L.mtj_gemv(ptr(ses.act), None, None, ptr(w.w_out[i]), ptr(w.b2[i]), d, d + F, w.dtype, EPI_RESID,
                             ptr(ses.x), F32, None, C.byref(am), s))
        else:
            A = w.act_dtype
            if not normed:
                check(L.mtj_layernorm(ptr(ses.x), ptr(w.ln_s[i]), ptr(w.ln_o[i]), B, d, ptr(ses.h), A, s))
            ip = self._inproj(ses, i, 1, ses.pos, ses.q, F32, ses.act, A, None)
            check(L.mtj_gemm(ptr(ses.h), d, ptr(w.w_in_mm[i]), ptr(w.b1[i]), B, 3 * d + F, d, w.mm_dtype, EPI_INPROJ,
                             None, 0, 0, C.byref(ip), w.alpha_in[i], s))
            check(L.mtj_attn_decode(ptr(ses.q), ptr(ses.kc[i]), ptr(ses.vc[i]), ptr(ses.pos), B, self.H, ses.Tcap,
                                    self.dh, ptr(ses.act), d + F, A, A, ptr(ses.attn_work), s))
            if next_ln is not None:
                check(L.mtj_gemm_splitk_ln(ptr(ses.act), d + F, ptr(w.w_out_mm[i]), ptr(w.b2[i]), B, d, d + F, w.mm_dtype,
                                           ptr(ses.x), d, ptr(ses.gemm_work), ses.gemm_work.numel(), ptr(next_ln[0]),
                                           ptr(next_ln[1]), ptr(ses.h), d, A, w.alpha_out[i], s))
            else:
                check(L.mtj_gemm_splitk(ptr(ses.act), d + F, ptr(w.w_out_mm[i]), ptr(w.b2[i]), B, d, d + F, w.mm_dtype,
                                        EPI_RESID, ptr(ses.x), d, F32, ptr(ses.gemm_work), ses.gemm_work.numel(),
                                        w.alpha_out[i], s))

    def sample_greedy(self, ses, out_tokens, embed_next=True, logits=None):
        check(_abi.lib().mtj_sample_greedy(ptr(ses.logits if logits is None else logits), ses.B, self.w.V, ptr(ses.tok), ptr(out_tokens),
                                           out_tokens.shape[1], ptr(ses.pos), ptr(ses.pos_start),
                                           self._next(ses, embed_next), _abi.stream_handle()))

    def sample_nucleus(self, ses, out_tokens, top_p, temp, top_k, uniforms, keep_mask=None, filtered=None,
                       embed_next=True, logits=None):
        L = _abi.lib()
        if ses.sample_work is None:
            ses.sample_work = torch.empty(L.mtj_sample_work_bytes(ses.B, self.w.V), dtype=torch.uint8, device=self.device)
        check(L.mtj_sample_nucleus(ptr(ses.logits if logits is None else logits), ses.B, self.w.V, ptr(top_p), ptr(temp), ptr(top_k), ptr(uniforms),
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

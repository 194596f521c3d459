"""PyTorch custom ops over the C ABI: every kernel entry point of include/mtj_abi.h as a dispatcher-visible operator
in the `mtj` namespace (torch.ops.mtj.*), implemented for the CUDA/HIP dispatch key only - there is no CPU or
composite implementation, so calling one with host tensors fails in the dispatcher.

The operators are a thin layer: they check tensor types, pull raw device pointers and the current HIP stream out of
the tensors and call the same `extern "C"` functions that `mesh_transformer.engine` calls directly through ctypes
(the engine keeps the direct calls: a decode step is 114 launches and replayed from a HIP graph, where a dispatcher
hop per launch would buy nothing).  Operators that write into caller-owned memory are declared as mutating
(`Tensor(a!)`) and return nothing; the others allocate their output with torch.

    torch.ops.mtj.layernorm(x, scale, offset, out_dtype)          ReplicatedLayerNorm          layers.py:17-36
    torch.ops.mtj.embed(tok, W, b)                                 EmbeddingShard               layers.py:187-202
    torch.ops.mtj.pack_weight(w) / pack_weight_f16(w, scale)       [in,out] -> packed [out,in]
    torch.ops.mtj.gemm(A, W, bias, alpha, out_dtype)               hk.Linear on many rows       layers.py:249-258,559
    torch.ops.mtj.gemm_resid_(x, A, W, bias, alpha)                ... + residual add           layers.py:313
    torch.ops.mtj.gemv(x, W, bias, ln_scale, ln_offset)            hk.Linear on one row (+ LN)  layers.py:316-344
    torch.ops.mtj.inproj_(...)                                     fused q|v|k|fc_in projection layers.py:261-297,325-326
    torch.ops.mtj.rope_append_(...)                                rotary + K/V window append   layers.py:261-273,325-326
    torch.ops.mtj.attn_prefill(q, k_cache, v_t, pos0, Tp, key_limit)   self_attn + masks        layers.py:260-285,347-366
    torch.ops.mtj.attn_decode(q, k_cache, v_cache, pos, out_dtype) one-token attention          layers.py:316-344
    torch.ops.mtj.xent(logits, target)                             ProjectionShard.loss         layers.py:569-593
    torch.ops.mtj.gemm_xent(A, W, bias, alpha, target)             ... on logits never stored   layers.py:559,569-593
    torch.ops.mtj.sample_greedy(logits) / sample_nucleus(...)      config["sampler"]            sampling.py:6-44
"""
import ctypes as C

import torch

from . import _abi
from ._abi import EPI_INPROJ, EPI_RESID, EPI_STORE, F16, F32, InProj, check, ptr

_lib = torch.library.Library("mtj", "DEF")
_DT = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
_TORCH = {0: torch.float32, 1: torch.bfloat16, 2: torch.float16}


def _code(t):
    try:
        return _DT[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {t.dtype}") from None


def _s():
    return torch.cuda.current_stream().cuda_stream


def _define(schema, fn):
    _lib.define(schema)
    _lib.impl(schema.split("(")[0], fn, "CUDA")


# ---------------------------------------------------------------- elementwise / row kernels
def _layernorm(x, scale, offset, out_dtype):
    x = x.contiguous()
    out = torch.empty_like(x, dtype=_TORCH[out_dtype])
    rows = x.reshape(-1, x.shape[-1])
    check(_abi.lib().mtj_layernorm(ptr(rows), ptr(scale), ptr(offset), rows.shape[0], rows.shape[1], ptr(out), out_dtype, _s()))
    return out


def _embed(tok, W, b):
    tok = tok.reshape(-1).to(torch.int32).contiguous()
    out = torch.empty(tok.shape[0], W.shape[1], dtype=torch.float32, device=W.device)
    check(_abi.lib().mtj_embed(ptr(tok), tok.shape[0], ptr(W), ptr(b), W.shape[0], W.shape[1], _code(W), ptr(out), _s()))
    return out


def _xent(logits, target):
    M, V = logits.shape
    loss = torch.empty(M, dtype=torch.float32, device=logits.device)
    correct = torch.empty(M, dtype=torch.uint8, device=logits.device)
    check(_abi.lib().mtj_xent(ptr(logits), logits.stride(0), ptr(target), M, V, ptr(loss), ptr(correct), _s()))
    return loss, correct.bool()


# ---------------------------------------------------------------- weights
def _pack_weight(w):
    K, N = w.shape
    dst = torch.empty(N, K, dtype=w.dtype, device=w.device)
    check(_abi.lib().mtj_pack_weight(ptr(w), w.stride(0), K, N, ptr(dst), K, 0, 0, _code(w), _s()))
    return dst


def _pack_weight_f16(w, scale):
    K, N = w.shape
    dst = torch.empty(N, K, dtype=torch.float16, device=w.device)
    check(_abi.lib().mtj_pack_weight_cvt(ptr(w), w.stride(0), K, N, ptr(dst), K, 0, 0, _code(w), F16, scale, _s()))
    return dst


# ---------------------------------------------------------------- GEMM / GEMV
def _gemm(A, W, bias, alpha, out_dtype):
    M, K = A.shape
    N = W.shape[0]
    out = torch.empty(M, N, dtype=_TORCH[out_dtype], device=A.device)
    check(_abi.lib().mtj_gemm(ptr(A), A.stride(0), ptr(W), ptr(bias), M, N, K, _code(W), EPI_STORE, ptr(out), N, out_dtype,
                              None, alpha, _s()))
    return out


def _gemm_xent(A, W, bias, alpha, target):
    M, K = A.shape
    N = W.shape[0]
    L = _abi.lib()
    nb = L.mtj_gemm_xent_work_bytes(M, N, _code(W))
    work = torch.empty(nb, dtype=torch.uint8, device=A.device)
    loss = torch.empty(M, dtype=torch.float32, device=A.device)
    correct = torch.empty(M, dtype=torch.uint8, device=A.device)
    target = target.reshape(-1).to(torch.int32).contiguous()
    check(L.mtj_gemm_xent(ptr(A), A.stride(0), ptr(W), ptr(bias), M, N, K, _code(W), alpha, ptr(target), ptr(loss),
                          ptr(correct), ptr(work), nb, _s()))
    return loss, correct.bool()


def _gemm_resid_(x, A, W, bias, alpha):
    M, K = A.shape
    N = W.shape[0]
    L = _abi.lib()
    nb = L.mtj_gemm_splitk_work_bytes(M, N, K, _code(W))
    work = torch.empty(max(nb, 16), dtype=torch.uint8, device=A.device)
    check(L.mtj_gemm_splitk(ptr(A), A.stride(0), ptr(W), ptr(bias), M, N, K, _code(W), EPI_RESID, ptr(x), x.stride(0), F32,
                            ptr(work), work.numel(), alpha, _s()))


def _gemv(x, W, bias, ln_scale, ln_offset):
    N, K = W.shape
    out = torch.empty(N, dtype=torch.float32, device=x.device)
    check(_abi.lib().mtj_gemv(ptr(x), ptr(ln_scale), ptr(ln_offset), ptr(W), ptr(bias), N, K, _code(W), EPI_STORE, ptr(out),
                              F32, None, None, _s()))
    return out


def _inproj_(h, W, b1, alpha, pos0, sin_tab, cos_tab, q, k_cache, v_cache, v_t, act, n_heads, rotary_dims, Tp, ldvt):
    """Fused q|v|k|fc_in projection of `h` ([M, d] rows in the GEMM dtype, or one float32 row for the GEMV) with RoPE,
    the K/V window append (slot = position % Tcap), the optional transposed V copy and gelu(fc_in + b1) into
    act[:, d:].  h float32 with one row selects the matrix-vector kernel (LayerNorm must then be applied by the caller)."""
    M, d = h.shape
    ip = InProj()
    ip.n_heads, ip.d_head, ip.rotary_dims = n_heads, d // n_heads, rotary_dims
    ip.Tp, ip.Tcap, ip.max_pos = Tp, k_cache.shape[2], sin_tab.shape[0]
    ip.pos0, ip.sin_tab, ip.cos_tab = ptr(pos0), ptr(sin_tab), ptr(cos_tab)
    ip.q, ip.q_dtype, ip.kv_dtype = ptr(q), _code(q), _code(k_cache)
    ip.k_cache, ip.v_cache = ptr(k_cache), ptr(v_cache)
    ip.v_t, ip.ldvt = (ptr(v_t), ldvt) if v_t is not None else (None, 0)
    ip.act, ip.ld_act, ip.act_dtype = ptr(act), act.stride(0), _code(act)
    L = _abi.lib()
    N = W.shape[0]
    if M == 1 and h.dtype == torch.float32 and W.dtype != torch.float16:
        check(L.mtj_gemv(ptr(h), None, None, ptr(W), ptr(b1), N, d, _code(W), EPI_INPROJ, None, 0, C.byref(ip), None, _s()))
    else:
        check(L.mtj_gemm(ptr(h), h.stride(0), ptr(W), ptr(b1), M, N, d, _code(W), EPI_INPROJ, None, 0, 0, C.byref(ip), alpha,
                         _s()))


def _rope_append_(q_in, v_in, k_in, pos0, sin_tab, cos_tab, q, k_cache, v_cache, v_t, n_heads, rotary_dims, Tp, ldvt):
    """Rotary embedding + window append of projected rows (float32 [M, d] each, any may be None): what inproj_ does
    after its GEMM.  Row m is token m % Tp of sequence m // Tp at position pos0[b] + t."""
    src = next(t for t in (q_in, v_in, k_in) if t is not None)
    M, d = src.shape
    ip = InProj()
    ip.n_heads, ip.d_head, ip.rotary_dims = n_heads, d // n_heads, rotary_dims
    ref = k_cache if k_cache is not None else v_cache
    ip.Tp, ip.Tcap, ip.max_pos = Tp, (ref.shape[2] if ref is not None else Tp), sin_tab.shape[0]
    ip.pos0, ip.sin_tab, ip.cos_tab = ptr(pos0), ptr(sin_tab), ptr(cos_tab)
    ip.q, ip.q_dtype = (ptr(q), _code(q)) if q is not None else (None, 0)
    ip.kv_dtype = _code(ref) if ref is not None else 0
    ip.k_cache, ip.v_cache = ptr(k_cache), ptr(v_cache)
    ip.v_t, ip.ldvt = (ptr(v_t), ldvt) if v_t is not None else (None, 0)
    srcs = [None if t is None else t.contiguous() for t in (q_in, v_in, k_in)]     # alive until the call is enqueued
    check(_abi.lib().mtj_rope_append(ptr(srcs[0]), ptr(srcs[1]), ptr(srcs[2]), M, C.byref(ip), _s()))


# ---------------------------------------------------------------- attention
def _attn_prefill(q, k_cache, v_t, pos0, Tp, key_limit):
    B, H, Tcap, dh = k_cache.shape
    ldvt = v_t.shape[-1]
    out = torch.empty(B * Tp, H * dh, dtype=q.dtype, device=q.device)
    check(_abi.lib().mtj_attn_prefill(ptr(q), ptr(k_cache), ptr(v_t), ptr(pos0), B, H, Tp, Tcap, dh, ldvt, ptr(out), H * dh,
                                      _code(q), ptr(key_limit), _s()))
    return out


def _attn_decode(q, k_cache, v_cache, pos, out_dtype):
    B, H, Tcap, dh = k_cache.shape
    L = _abi.lib()
    work = torch.empty(max(L.mtj_attn_decode_work_bytes(B, H, dh, Tcap), 16), dtype=torch.uint8, device=q.device)
    out = torch.empty(B, H * dh, dtype=_TORCH[out_dtype], device=q.device)
    check(L.mtj_attn_decode(ptr(q), ptr(k_cache), ptr(v_cache), ptr(pos), B, H, Tcap, dh, ptr(out), H * dh, out_dtype,
                            _code(k_cache), ptr(work), _s()))
    return out


# ---------------------------------------------------------------- samplers
def _sample_greedy(logits):
    R, V = logits.shape
    tok = torch.zeros(R, dtype=torch.int32, device=logits.device)
    pos = torch.zeros(R, dtype=torch.int32, device=logits.device)
    pos_start = torch.zeros_like(pos)              # alive until the call has been enqueued
    check(_abi.lib().mtj_sample_greedy(ptr(logits), R, V, ptr(tok), None, 0, ptr(pos), ptr(pos_start), None, _s()))
    return tok


def _sample_nucleus(logits, top_p, temp, top_k, uniforms):
    """logits float32 [R, V]; top_p, temp, uniforms float64 [R]; top_k int32 [R] or None.
    Returns (token int32 [R], filtered logits float32 [R, V], keep mask bool [R, V])."""
    R, V = logits.shape
    dev = logits.device
    L = _abi.lib()
    tok = torch.zeros(R, dtype=torch.int32, device=dev)
    pos = torch.zeros(R, dtype=torch.int32, device=dev)
    pos_start = torch.zeros_like(pos)
    filtered = torch.empty(R, V, dtype=torch.float32, device=dev)
    mask = torch.empty(R, V, dtype=torch.uint8, device=dev)
    work = torch.empty(L.mtj_sample_work_bytes(R, V), dtype=torch.uint8, device=dev)
    u = uniforms.reshape(R, 1).contiguous()
    check(L.mtj_sample_nucleus(ptr(logits), R, V, ptr(top_p), ptr(temp), ptr(top_k), ptr(u), 1, ptr(tok), None, 0, ptr(pos),
                               ptr(pos_start), ptr(mask), ptr(filtered), ptr(work), None, _s()))
    return tok, filtered, mask.bool()


_define("layernorm(Tensor x, Tensor scale, Tensor offset, int out_dtype) -> Tensor", _layernorm)
_define("embed(Tensor tok, Tensor W, Tensor b) -> Tensor", _embed)
_define("xent(Tensor logits, Tensor target) -> (Tensor, Tensor)", _xent)
_define("pack_weight(Tensor w) -> Tensor", _pack_weight)
_define("pack_weight_f16(Tensor w, float scale) -> Tensor", _pack_weight_f16)
_define("gemm(Tensor A, Tensor W, Tensor? bias, float alpha, int out_dtype) -> Tensor", _gemm)
_define("gemm_xent(Tensor A, Tensor W, Tensor? bias, float alpha, Tensor target) -> (Tensor, Tensor)", _gemm_xent)
_define("gemm_resid_(Tensor(a!) x, Tensor A, Tensor W, Tensor? bias, float alpha) -> ()", _gemm_resid_)
_define("gemv(Tensor x, Tensor W, Tensor? bias, Tensor? ln_scale, Tensor? ln_offset) -> Tensor", _gemv)
_define("inproj_(Tensor h, Tensor W, Tensor b1, float alpha, Tensor pos0, Tensor sin_tab, Tensor cos_tab, Tensor(a!) q, "
        "Tensor(b!) k_cache, Tensor(c!) v_cache, Tensor(d!)? v_t, Tensor(e!) act, int n_heads, int rotary_dims, int Tp, "
        "int ldvt) -> ()", _inproj_)
_define("rope_append_(Tensor? q_in, Tensor? v_in, Tensor? k_in, Tensor pos0, Tensor sin_tab, Tensor cos_tab, Tensor(a!)? q, "
        "Tensor(b!)? k_cache, Tensor(c!)? v_cache, Tensor(d!)? v_t, int n_heads, int rotary_dims, int Tp, int ldvt) -> ()",
        _rope_append_)
_define("attn_prefill(Tensor q, Tensor k_cache, Tensor v_t, Tensor pos0, int Tp, Tensor? key_limit) -> Tensor", _attn_prefill)
_define("attn_decode(Tensor q, Tensor k_cache, Tensor v_cache, Tensor pos, int out_dtype) -> Tensor", _attn_decode)
_define("sample_greedy(Tensor logits) -> Tensor", _sample_greedy)
_define("sample_nucleus(Tensor logits, Tensor top_p, Tensor temp, Tensor? top_k, Tensor uniforms) -> (Tensor, Tensor, Tensor)",
        _sample_nucleus)

OPS = ("layernorm", "embed", "xent", "pack_weight", "pack_weight_f16", "gemm", "gemm_xent", "gemm_resid_", "gemv", "inproj_",
       "rope_append_", "attn_prefill", "attn_decode", "sample_greedy", "sample_nucleus")

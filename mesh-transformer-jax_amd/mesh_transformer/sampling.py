"""Samplers with the reference's contract (mesh_transformer/sampling.py):
    sampler(key, logits[rows, V], sampler_input, **options) -> (uint32 token[rows], info)

The arithmetic runs in the HIP sampling kernel.  The reference draws with
jax.random.categorical(key, ...) (Gumbel-max on a threefry key); here the draw is an inverse-CDF
walk driven by a uniform in [0, 1).  `key` is therefore interpreted as: None -> a fresh random
uniform; a float or float array -> the uniform(s) themselves; an int -> seed of a Philox stream.
"""
import numpy as np
import torch

from . import _abi
from ._abi import check, ptr


def _uniforms(key, rows):
    if key is None:
        return np.random.Generator(np.random.Philox()).random(rows)
    a = np.asarray(key)
    if a.dtype.kind == "f":
        return np.broadcast_to(a.astype(np.float64).reshape(-1), (rows,)).copy()
    return np.random.Generator(np.random.Philox(int(a.reshape(-1)[0]))).random(rows)


def _run(logits, top_p, temp, top_k, u, want_filtered, want_mask):
    L = _abi.lib()
    if not torch.cuda.is_available():
        raise RuntimeError("the sampling kernels need an MI355X; no GPU is visible")
    is_np = not isinstance(logits, torch.Tensor)
    lg = torch.as_tensor(np.asarray(logits, np.float32) if is_np else logits)
    dev = lg.device if lg.is_cuda else torch.device("cuda:0")
    lg = lg.to(dev, torch.float32).contiguous()
    if lg.dim() != 2:
        raise ValueError("logits must be [rows, n_vocab]")       # the reference indexes [:, ::-1]
    R, V = lg.shape
    with torch.cuda.device(dev):
        f64 = lambda v: torch.from_numpy(np.ascontiguousarray(np.broadcast_to(np.asarray(v, np.float64), (R,)))).to(dev)
        tp, tm = f64(top_p), f64(temp)
        tk = None if top_k is None else torch.from_numpy(
            np.ascontiguousarray(np.broadcast_to(np.asarray(top_k, np.int32), (R,)))).to(dev)
        uu = f64(u).reshape(R, 1).contiguous()
        tok = torch.zeros(R, dtype=torch.int32, device=dev)
        pos = torch.zeros(R, dtype=torch.int32, device=dev)
        pos_start = torch.zeros(R, dtype=torch.int32, device=dev)
        filtered = torch.empty(R, V, dtype=torch.float32, device=dev) if want_filtered else None
        mask = torch.empty(R, V, dtype=torch.uint8, device=dev) if want_mask else None
        work = torch.empty(L.mtj_sample_work_bytes(R, V), dtype=torch.uint8, device=dev)
        check(L.mtj_sample_nucleus(ptr(lg), R, V, ptr(tp), ptr(tm), ptr(tk), ptr(uu), 1, ptr(tok), None, 0, ptr(pos),
                                   ptr(pos_start), ptr(mask), ptr(filtered), ptr(work), None, _abi.stream_handle()))
        torch.cuda.current_stream().synchronize()
    conv = (lambda t: None if t is None else t.cpu().numpy()) if is_np else (lambda t: t)
    return conv(tok), conv(filtered), conv(mask)


def nucleaus_filter(logits, top_p=0.9, top_k=None):
    """sampling.py:10-38: subtract 1e10 from every token outside the top-p nucleus (and, with top_k,
    1e10 * token_id from every token of rank >= top_k), computed on the raw logits."""
    return _run(logits, top_p, 1.0, top_k, 0.0, True, False)[1]


def nucleaus_keep_mask(logits, top_p=0.9, top_k=None):
    """True where nucleaus_filter leaves the logit untouched."""
    m = _run(logits, top_p, 1.0, top_k, 0.0, False, True)[2]
    return m.astype(bool) if isinstance(m, np.ndarray) else m.bool()


def softmax_sample(key, logits, _, temp=1):
    """sampling.py:6-7: categorical draw from softmax(logits / temp)."""
    rows = np.shape(logits)[0]
    tok = _run(logits, 2.0, temp, None, _uniforms(key, rows), False, False)[0]   # top_p >= 1 removes nothing
    return (tok.astype(np.uint32) if isinstance(tok, np.ndarray) else tok), None


def nucleaus_sample(key, logits, _, top_p=0.9, temp=1, top_k=None):
    """sampling.py:41-44: filter on the raw logits, then temperature, then the draw."""
    rows = np.shape(logits)[0]
    tok = _run(logits, top_p, temp, top_k, _uniforms(key, rows), False, False)[0]
    return (tok.astype(np.uint32) if isinstance(tok, np.ndarray) else tok), None


def greedy_sample(key, logits, _, **unused):
    """argmax through the sampler contract (lowest id among maxima, like jnp.argmax)."""
    L = _abi.lib()
    is_np = not isinstance(logits, torch.Tensor)
    lg = torch.as_tensor(np.asarray(logits, np.float32) if is_np else logits)
    dev = lg.device if lg.is_cuda else torch.device("cuda:0")
    lg = lg.to(dev, torch.float32).contiguous()
    R, V = lg.shape
    with torch.cuda.device(dev):
        tok = torch.zeros(R, dtype=torch.int32, device=dev)
        pos = torch.zeros(R, dtype=torch.int32, device=dev)
        pos_start = torch.zeros_like(pos)
        check(L.mtj_sample_greedy(ptr(lg), R, V, ptr(tok), None, 0, ptr(pos), ptr(pos_start), None, _abi.stream_handle()))
        torch.cuda.current_stream().synchronize()
    return (tok.cpu().numpy().astype(np.uint32) if is_np else tok), None


def builtin_kind(sampler):
    """Which fused device sampler a config["sampler"] callable maps to (None: call it on the host)."""
    if sampler is nucleaus_sample:
        return "nucleus"
    if sampler is softmax_sample:
        return "softmax"
    if sampler is greedy_sample:
        return "greedy"
    return None

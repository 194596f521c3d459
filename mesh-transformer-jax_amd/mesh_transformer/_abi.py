"""ctypes binding of include/mtj_abi.h.

The shared library is built in-tree by `make -C mesh-transformer-jax_amd/csrc` (see
__graft_entry__.build()).  There is no fallback: if the library is missing every call
raises, so a GPU run can never silently take another path.
"""
import ctypes as C
import os

F32, BF16, F16 = 0, 1, 2
EPI_STORE, EPI_RESID, EPI_INPROJ = 0, 1, 2
ABI_VERSION = 4

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmtj_hip.so")

_p, _i64, _i32 = C.c_void_p, C.c_int64, C.c_int


class InProj(C.Structure):
    """mtj_inproj"""
    _fields_ = [
        ("n_heads", C.c_int32), ("d_head", C.c_int32), ("rotary_dims", C.c_int32),
        ("Tp", C.c_int32), ("Tcap", C.c_int32), ("max_pos", C.c_int32),
        ("pos0", _p), ("sin_tab", _p), ("cos_tab", _p),
        ("q", _p), ("q_dtype", C.c_int32), ("kv_dtype", C.c_int32),
        ("k_cache", _p), ("v_cache", _p), ("v_t", _p), ("ldvt", _i64),
        ("act", _p), ("ld_act", _i64), ("act_dtype", C.c_int32),
    ]


class AttnMerge(C.Structure):
    """mtj_attn_merge"""
    _fields_ = [("partials", _p), ("n_heads", C.c_int32), ("d_head", C.c_int32), ("splits", C.c_int32)]


class NextEmbed(C.Structure):
    """mtj_next_embed"""
    _fields_ = [("w", _p), ("bias", _p), ("x_next", _p), ("d", _i64), ("dtype", C.c_int32)]


# name -> (restype, argtypes); one entry per declaration in mtj_abi.h
SIGNATURES = {
    "mtj_version": (_i32, []),
    "mtj_last_error": (C.c_char_p, []),
    "mtj_pack_weight": (_i32, [_p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _i32, _p]),
    "mtj_pack_weight_cvt": (_i32, [_p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _i32, _i32, C.c_float, _p]),
    "mtj_embed": (_i32, [_p, _i64, _p, _p, _i64, _i64, _i32, _p, _p]),
    "mtj_layernorm": (_i32, [_p, _p, _p, _i64, _i64, _p, _i32, _p]),
    "mtj_rope_append": (_i32, [_p, _p, _p, _i64, C.POINTER(InProj), _p]),
    "mtj_xent": (_i32, [_p, _i64, _p, _i64, _i64, _p, _p, _p]),
    "mtj_gemm": (_i32, [_p, _i64, _p, _p, _i64, _i64, _i64, _i32, _i32, _p, _i64, _i32, C.POINTER(InProj), C.c_float, _p]),
    "mtj_gemm_splitk_work_bytes": (_i64, [_i64, _i64, _i64, _i32]),
    "mtj_gemm_splitk": (_i32, [_p, _i64, _p, _p, _i64, _i64, _i64, _i32, _i32, _p, _i64, _i32, _p, _i64, C.c_float, _p]),
    "mtj_gemm_splitk_ln": (_i32, [_p, _i64, _p, _p, _i64, _i64, _i64, _i32, _p, _i64, _p, _i64, _p, _p, _p, _i64, _i32,
                                 C.c_float, _p]),
    "mtj_gemm_xent_work_bytes": (_i64, [_i64, _i64, _i32]),
    "mtj_gemm_xent": (_i32, [_p, _i64, _p, _p, _i64, _i64, _i64, _i32, C.c_float, _p, _p, _p, _p, _i64, _p]),
    "mtj_gemv": (_i32, [_p, _p, _p, _p, _p, _i64, _i64, _i32, _i32, _p, _i32, C.POINTER(InProj), C.POINTER(AttnMerge), _p]),
    "mtj_gemv_attn_supported": (_i32, [_i64, _i64, _i32, _i64, _i64, _i32, _i64]),
    "mtj_gemv_attn_work_bytes": (_i64, [_i64, _i64]),
    "mtj_gemv_attn": (_i32, [_p, _p, _p, _i64, _i64, _i32, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i32, _p, _p]),
    "mtj_attn_prefill": (_i32, [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _p, _i64, _i32, _p, _p]),
    "mtj_attn_decode_splits": (_i32, [_i64, _i64, _i64]),
    "mtj_attn_decode_work_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "mtj_attn_decode_partials": (_i32, [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i32, _p, C.POINTER(AttnMerge), _p]),
    "mtj_attn_decode": (_i32, [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _i64, _i32, _i32, _p, _p]),
    "mtj_attn_decode_static_max_bytes": (_i64, []),
    "mtj_attn_decode_static": (_i32, [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _i64, _i32, _i32, _p]),
    "mtj_sample_greedy": (_i32, [_p, _i64, _i64, _p, _p, _i64, _p, _p, C.POINTER(NextEmbed), _p]),
    "mtj_gemv_greedy": (_i32, [_p, _p, _p, _p, _p, _i64, _i64, _i32, _p, _p, _p, _i64, _p, _p, C.POINTER(NextEmbed), _p, _p]),
    "mtj_sample_work_bytes": (_i64, [_i64, _i64]),
    "mtj_sample_nucleus": (_i32, [_p, _i64, _i64, _p, _p, _p, _p, _i64, _p, _p, _i64, _p, _p, _p, _p, _p,
                                 C.POINTER(NextEmbed), _p]),
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP kernels first "
                "(python -c 'import __graft_entry__ as g; g.build()' or make -C mesh-transformer-jax_amd/csrc)")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)          # AttributeError if the library does not export it
            fn.restype, fn.argtypes = res, args
        v = l.mtj_version()
        if v != ABI_VERSION:
            raise RuntimeError(f"libmtj_hip.so has ABI version {v}, binding expects {ABI_VERSION}")
        _lib = l
    return _lib


class MtjError(RuntimeError):
    pass


def check(code: int) -> None:
    """Error contract of the C ABI: negative code + message -> Python exception
    (shape problems as ValueError, like the reference's asserts; the rest as RuntimeError)."""
    if code == 0:
        return
    msg = lib().mtj_last_error().decode(errors="replace")
    if code in (-1, -2, -3, -5):
        raise ValueError(f"mtj error {code}: {msg}")
    raise MtjError(f"mtj error {code}: {msg}")


def ptr(t):
    """Device pointer of a torch tensor (None -> NULL).  Host tensors are refused: the kernels
    dereference whatever they are given."""
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("expected a CUDA/HIP tensor, got a host tensor")
    return t.data_ptr()


def dtype_code(torch_dtype) -> int:
    import torch
    if torch_dtype == torch.float32:
        return F32
    if torch_dtype == torch.bfloat16:
        return BF16
    if torch_dtype == torch.float16:
        return F16
    raise ValueError(f"unsupported dtype {torch_dtype}: float32, bfloat16 or float16")


def stream_handle():
    import torch
    return torch.cuda.current_stream().cuda_stream

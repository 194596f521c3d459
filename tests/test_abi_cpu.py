"""CPU-side checks of the boundary: the shared library loads without a GPU and exports exactly the symbols that
include/mtj_abi.h declares; the Python binding covers every one of them; argument validation that needs no
device works.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mtj_abi.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mtj_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for s in ("mtj_version", "mtj_last_error", "mtj_pack_weight", "mtj_embed", "mtj_layernorm", "mtj_gemm", "mtj_gemv",
              "mtj_attn_prefill", "mtj_attn_decode", "mtj_attn_decode_work_bytes", "mtj_sample_greedy",
              "mtj_sample_nucleus", "mtj_sample_work_bytes", "mtj_gemv_greedy"):
        assert s in syms


def test_library_exports_every_declared_symbol_and_binding_covers_them():
    from mesh_transformer import _abi
    lib = _abi.lib()                      # raises if the library is missing: there is no fallback path
    syms = declared_symbols()
    for s in syms:
        assert hasattr(lib, s), f"{s} is declared in mtj_abi.h but not exported by libmtj_hip.so"
    assert sorted(_abi.SIGNATURES) == syms
    assert lib.mtj_version() == _abi.ABI_VERSION


def test_struct_layouts_match_the_header():
    from mesh_transformer import _abi
    # field order of mtj_inproj / mtj_next_embed as written in the header
    text = open(HEADER).read()
    body = text[text.index("typedef struct {"):text.index("} mtj_inproj;")]
    names = re.findall(r"\b([a-zA-Z_0-9]+)\s*(?:,|;)", re.sub(r"/\*.*?\*/", "", body, flags=re.S))
    assert names == [f[0] for f in _abi.InProj._fields_]
    assert ctypes.sizeof(_abi.InProj) % 8 == 0
    body = text[text.index("typedef struct {", text.index("mtj_inproj;")):text.index("} mtj_attn_merge;")]
    names = re.findall(r"\b([a-zA-Z_0-9]+)\s*(?:,|;)", re.sub(r"/\*.*?\*/", "", body, flags=re.S))
    assert names == [f[0] for f in _abi.AttnMerge._fields_]
    body = text[text.index("typedef struct {", text.index("mtj_attn_merge;")):text.index("} mtj_next_embed;")]
    names = re.findall(r"\b([a-zA-Z_0-9]+)\s*(?:,|;)", re.sub(r"/\*.*?\*/", "", body, flags=re.S))
    assert names == [f[0] for f in _abi.NextEmbed._fields_]


def test_argument_validation_needs_no_device():
    from mesh_transformer import _abi
    lib = _abi.lib()
    # shape errors are reported before anything touches the GPU
    assert lib.mtj_layernorm(None, None, None, 1, 8, None, 0, None) == -1
    assert b"null pointer" in lib.mtj_last_error()
    with pytest.raises(ValueError):
        _abi.check(lib.mtj_gemv(None, None, None, None, None, 8, 8, 0, 0, None, 0, None, None, None))
    # one sequence of 16 heads: 8 key ranges per head (128 workgroups); 32 sequences fill the chip with one range each
    assert lib.mtj_attn_decode_splits(1, 16, 2047) == 8 and lib.mtj_attn_decode_splits(32, 16, 2047) == 1
    assert lib.mtj_attn_decode_splits(1, 16, 20) == 2          # never fewer than 16 slots per range at a full window
    assert lib.mtj_attn_decode_work_bytes(1, 16, 256, 2047) == 16 * 8 * 260 * 4
    assert lib.mtj_sample_work_bytes(32, 50400) == 256         # kept in the ABI; the sampler sorts nothing


def test_host_tensors_are_refused():
    import torch
    from mesh_transformer import _abi
    with pytest.raises(ValueError):
        _abi.ptr(torch.zeros(4))
    assert _abi.ptr(None) is None


def test_product_fails_loudly_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    from mesh_transformer.transformer_shard import CausalTransformer
    cfg = dict(layers=1, d_model=64, n_heads=1, n_vocab=64, pe="rotary", cores_per_replica=1)
    with pytest.raises(RuntimeError):
        CausalTransformer(cfg)
    from mesh_transformer import sampling
    with pytest.raises(RuntimeError):
        sampling.nucleaus_filter(np.zeros((1, 8), np.float32))


def test_util_casts():
    import torch
    from mesh_transformer.util import to_bf16, to_f32
    t = {"a": {"w": torch.ones(2, 2), "i": torch.ones(2, dtype=torch.int32)}}
    b = to_bf16(t)
    assert b["a"]["w"].dtype == torch.bfloat16 and b["a"]["i"].dtype == torch.int32
    assert to_f32(b)["a"]["w"].dtype == torch.float32


def test_session_workspace_covers_every_prompt_length():
    """The out projection of a prefill is cut into MORE K ranges the FEWER rows it has, so the workspace of a session
    sized for its longest prompt must also hold the partials of every shorter one (host-side sizes only)."""
    from mesh_transformer import _abi
    from mesh_transformer.engine import splitk_work_bound
    lib = _abi.lib()
    for dtype in (_abi.F32, _abi.F16, _abi.BF16):
        for M_max, N, K in ((8 * 599, 4096, 20480), (700, 512, 2560), (2047, 4096, 20480), (100, 4096, 20480)):
            bound = splitk_work_bound(M_max, N, K, dtype)
            need = max(lib.mtj_gemm_splitk_work_bytes(m, N, K, dtype) for m in range(1, M_max + 1))
            assert bound == need, (dtype, M_max, N, K)
    # the case that used to fail: a session first sized for 8 x 599 rows, later used with 8 x 99
    assert lib.mtj_gemm_splitk_work_bytes(8 * 99, 4096, 20480, _abi.F16) > lib.mtj_gemm_splitk_work_bytes(8 * 599, 4096, 20480, _abi.F16)


def test_torch_ops_are_registered_for_the_gpu_only():
    """Every kernel entry point is a dispatcher-visible operator torch.ops.mtj.*; there is no CPU implementation, so
    host tensors are refused by the dispatcher instead of taking another path."""
    import torch
    from mesh_transformer import ops
    for name in ops.OPS:
        assert hasattr(torch.ops.mtj, name), name
    assert "Tensor(a!)" in str(torch.ops.mtj.gemm_resid_.default._schema)
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.mtj.layernorm(torch.zeros(2, 8), torch.ones(8), torch.zeros(8), 0)

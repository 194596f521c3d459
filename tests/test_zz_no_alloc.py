"""mtj_attn_decode_static: the decode-attention entry point that allocates nothing (its partial results live in a
device array built into the library) against mtj_attn_decode with a caller-provided workspace, through the C ABI.

Both run the same kernels in the same order, so the outputs must be bit-identical; the float64 reference of the
window attention (decode_once, layers.py:316-344) is checked too.  Calls in a row, later ones with smaller
inputs, so that stale partials of an earlier call would show."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _run(L, a, B, H, Tcap, dh, positions, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, dh, generator=g).to(DEV)
    kc = torch.randn(B, H, Tcap, dh, generator=g).to(dtype).to(DEV)
    vc = torch.randn(B, H, Tcap, dh, generator=g).to(dtype).to(DEV)
    pos = torch.tensor(positions, dtype=torch.int32, device=DEV)
    work = torch.zeros(L.mtj_attn_decode_work_bytes(B, H, dh, Tcap), dtype=torch.uint8, device=DEV)
    ld = H * dh
    ref_out = torch.zeros(B, ld, device=DEV)
    out = torch.full((B, ld), float("nan"), device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    dt = a.dtype_code(dtype)
    a.check(L.mtj_attn_decode(a.ptr(q), a.ptr(kc), a.ptr(vc), a.ptr(pos), B, H, Tcap, dh, a.ptr(ref_out), ld, 0, dt,
                              a.ptr(work), s))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    a.check(L.mtj_attn_decode_static(a.ptr(q), a.ptr(kc), a.ptr(vc), a.ptr(pos), B, H, Tcap, dh, a.ptr(out), ld, 0, dt, s))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(out, ref_out), float((out - ref_out).abs().max())
    for b, p in enumerate(positions):
        n = min(p + 1, Tcap)
        sc = torch.einsum("hd,hTd->hT", q[b].double(), kc[b, :, :n].double()) / math.sqrt(dh)
        ref = torch.einsum("hT,hTd->hd", torch.softmax(sc, -1), vc[b, :, :n].double()).reshape(-1)
        err = float((out[b].double() - ref).norm() / ref.norm())
        assert err < 3e-6, (b, p, err)


def test_static_scratch_matches_workspace_variant_twice():
    from mesh_transformer import _abi as a
    L = a.lib()
    assert L.mtj_attn_decode_static_max_bytes() >= L.mtj_attn_decode_work_bytes(32, 16, 256, 2047)
    # first call: batch 3, a 700-slot window, ragged fill (one sequence wrapped around); second: smaller in every way
    _run(L, a, 3, 16, 700, 256, [699, 130, 2000], torch.bfloat16, 0)
    _run(L, a, 1, 4, 130, 64, [57], torch.float32, 1)
    _run(L, a, 2, 16, 700, 256, [5, 698], torch.bfloat16, 2)


def test_static_scratch_rejects_oversize():
    from mesh_transformer import _abi as a
    L = a.lib()
    B, H, dh, Tcap = 300, 16, 256, 4096
    assert L.mtj_attn_decode_work_bytes(B, H, dh, Tcap) > L.mtj_attn_decode_static_max_bytes()
    t = torch.zeros(16, device=DEV)              # never dereferenced: the size check comes first
    p = torch.zeros(B, dtype=torch.int32, device=DEV)
    rc = L.mtj_attn_decode_static(a.ptr(t), a.ptr(t), a.ptr(t), a.ptr(p), B, H, Tcap, dh, a.ptr(t), H * dh, 0, 1,
                                  torch.cuda.current_stream().cuda_stream)
    assert rc == -5
    assert b"built-in" in L.mtj_last_error()
    with pytest.raises(ValueError):
        a.check(rc)


def test_static_scratch_under_graph_capture():
    """The entry point is meant for captured code: after the set-up call and one eager call, a captured call must
    replay to the bits of the eager workspace variant - several replays, with the inputs rewritten (by ordinary
    eager work) between them."""
    from mesh_transformer import _abi as a
    L = a.lib()
    assert L.mtj_attn_decode_static_max_bytes() > 0             # resolves the array's address on this device
    B, H, Tcap, dh = 2, 16, 300, 256
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, H, dh, generator=g).to(DEV)
    kc = torch.randn(B, H, Tcap, dh, generator=g).to(torch.float16).to(DEV)
    vc = torch.randn(B, H, Tcap, dh, generator=g).to(torch.float16).to(DEV)
    pos = torch.tensor([10, 250], dtype=torch.int32, device=DEV)
    work = torch.zeros(L.mtj_attn_decode_work_bytes(B, H, dh, Tcap), dtype=torch.uint8, device=DEV)
    ld = H * dh
    out, ref = torch.zeros(B, ld, device=DEV), torch.zeros(B, ld, device=DEV)
    dt = a.dtype_code(torch.float16)

    def static_call():
        a.check(L.mtj_attn_decode_static(a.ptr(q), a.ptr(kc), a.ptr(vc), a.ptr(pos), B, H, Tcap, dh, a.ptr(out), ld, 0, dt,
                                         torch.cuda.current_stream().cuda_stream))

    static_call()                                               # eager once: kernel attributes
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_call()
    for rep, positions in enumerate(([10, 250], [299, 0], [150, 700])):
        pos.copy_(torch.tensor(positions, dtype=torch.int32))
        q.copy_(torch.randn(B, H, dh, generator=g))
        out.fill_(float("nan"))
        graph.replay()
        a.check(L.mtj_attn_decode(a.ptr(q), a.ptr(kc), a.ptr(vc), a.ptr(pos), B, H, Tcap, dh, a.ptr(ref), ld, 0, dt,
                                  a.ptr(work), torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert torch.equal(out, ref), (rep, float((out - ref).abs().max()))

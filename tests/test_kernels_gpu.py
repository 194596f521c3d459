"""Kernel-level parity through the C ABI (ctypes) on a real MI355X.

References are float64 evaluations of the same mathematics on the same (already rounded) inputs -
torch on the host or device for plain linear algebra, the CPU oracle for everything that carries a
convention of the reference (rotary interleaving, masks, window, sampler order)."""
import ctypes as C
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import gptj_oracle as O

DEV = "cuda:0"


@pytest.fixture(scope="module")
def L():
    from mesh_transformer import _abi
    return _abi.lib()


def abi():
    from mesh_transformer import _abi
    return _abi


def S():
    return torch.cuda.current_stream().cuda_stream


def rel_err(got, ref):
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).norm() / ref.norm().clamp_min(1e-30))


def max_err(got, ref):
    return float((got.double().cpu() - ref.double().cpu()).abs().max())


TD = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
# float32 path: the 1e-4 relative budget of the whole layer leaves ~1e-5 per kernel; 16-bit outputs carry their
# own rounding (2^-9 relative for bfloat16, 2^-12 for float16)
TOL = {"f32": 2e-6, "bf16": 6e-3, "f16": 8e-4}
DTS = ["f32", "bf16", "f16"]


# ------------------------------------------------------------------ pack / embed / layernorm
@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_pack_weight_transposes_with_offsets(L, dt):
    a = abi()
    g = torch.Generator().manual_seed(0)
    K, N1, N2 = 96, 70, 40
    w1 = torch.randn(K, N1, generator=g).to(TD[dt]).to(DEV)
    w2 = torch.randn(K // 2, N2, generator=g).to(TD[dt]).to(DEV)
    dst = torch.zeros(N1 + N2, K, dtype=TD[dt], device=DEV)
    a.check(L.mtj_pack_weight(a.ptr(w1), N1, K, N1, a.ptr(dst), K, 0, 0, a.dtype_code(TD[dt]), S()))
    a.check(L.mtj_pack_weight(a.ptr(w2), N2, K // 2, N2, a.ptr(dst), K, N1, K // 2, a.dtype_code(TD[dt]), S()))
    torch.cuda.synchronize()
    ref = torch.zeros_like(dst)
    ref[:N1] = w1.T
    ref[N1:, K // 2:] = w2.T
    assert torch.equal(dst, ref)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_embed_is_row_gather_plus_bias(L, dt):
    a = abi()
    g = torch.Generator().manual_seed(1)
    V, d = 1000, 512
    W = (torch.randn(V, d, generator=g) * 0.02).to(TD[dt]).to(DEV)
    b = (torch.randn(d, generator=g) * 0.02).to(DEV)
    tok = torch.tensor([0, 999, 5, 5, 123], dtype=torch.int32, device=DEV)
    out = torch.empty(5, d, device=DEV)
    a.check(L.mtj_embed(a.ptr(tok), 5, a.ptr(W), a.ptr(b), V, d, a.dtype_code(TD[dt]), a.ptr(out), S()))
    torch.cuda.synchronize()
    assert torch.equal(out, W[tok.long()].float() + b)      # one non-zero term per dot: exact


@pytest.mark.parametrize("d", [512, 4096, 1024 + 4])
@pytest.mark.parametrize("out_dt", ["f32", "bf16"])
def test_layernorm(L, d, out_dt):
    a = abi()
    g = torch.Generator().manual_seed(2)
    M = 37
    x = (torch.randn(M, d, generator=g) * 3 + 1.5).to(DEV)
    sc = (1 + 0.1 * torch.randn(d, generator=g)).to(DEV)
    of = (0.1 * torch.randn(d, generator=g)).to(DEV)
    out = torch.empty(M, d, dtype=TD[out_dt], device=DEV)
    a.check(L.mtj_layernorm(a.ptr(x), a.ptr(sc), a.ptr(of), M, d, a.ptr(out), a.dtype_code(TD[out_dt]), S()))
    torch.cuda.synchronize()
    ref = O.replicated_layer_norm(x.double().cpu(), sc.double().cpu(), of.double().cpu())
    assert rel_err(out, ref) < (2e-6 if out_dt == "f32" else 3e-3)
    # a constant row gives exactly `offset`
    xc = torch.full((1, d), 2.75, device=DEV)
    o2 = torch.empty(1, d, device=DEV)
    a.check(L.mtj_layernorm(a.ptr(xc), a.ptr(sc), a.ptr(of), 1, d, a.ptr(o2), 0, S()))
    torch.cuda.synchronize()
    assert torch.equal(o2[0], of)


def test_layernorm_rejects_bad_shapes(L):
    a = abi()
    x = torch.zeros(2, 6, device=DEV)
    with pytest.raises(ValueError):
        a.check(L.mtj_layernorm(a.ptr(x), a.ptr(x), a.ptr(x), 2, 6, a.ptr(x), 0, S()))


# ------------------------------------------------------------------ GEMM
def _packed(w_haiku):
    """haiku [K, N] -> packed [N, K] through the library."""
    a = abi()
    K, N = w_haiku.shape
    dst = torch.empty(N, K, dtype=w_haiku.dtype, device=DEV)
    a.check(abi().lib().mtj_pack_weight(a.ptr(w_haiku), N, K, N, a.ptr(dst), K, 0, 0, a.dtype_code(w_haiku.dtype), S()))
    return dst


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (32, 256, 128), (33, 300, 192), (128, 128, 512), (200, 1000, 256),
                                   (64, 520, 2560), (257, 96, 64)])
def test_gemm_store_and_resid(L, dt, M, N, K):
    a = abi()
    g = torch.Generator().manual_seed(M * 7 + N)
    A = torch.randn(M, K, generator=g).to(TD[dt]).to(DEV)
    Wh = (torch.randn(K, N, generator=g) * 0.05).to(TD[dt]).to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    W = _packed(Wh)
    ref = A.double() @ Wh.double() + bias.double()
    out = torch.empty(M, N, device=DEV)
    a.check(L.mtj_gemm(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, N, K, a.dtype_code(TD[dt]), a.EPI_STORE, a.ptr(out), N, 0,
                       None, 1.0, S()))
    torch.cuda.synchronize()
    assert rel_err(out, ref) < 5e-6, (dt, M, N, K)      # inputs are already rounded: only fp32 accumulation differs
    # RESID: x += A W + b, with a padded leading dimension
    x0 = torch.randn(M, N + 8, generator=g).to(DEV)
    x = x0.clone()
    a.check(L.mtj_gemm(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, N, K, a.dtype_code(TD[dt]), a.EPI_RESID, a.ptr(x), N + 8, 0,
                       None, 1.0, S()))
    torch.cuda.synchronize()
    assert rel_err(x[:, :N], x0[:, :N].double() + ref) < 5e-6
    assert torch.equal(x[:, N:], x0[:, N:])
    # 16-bit outputs
    for odt in ("bf16", "f16"):
        ob = torch.empty(M, N, dtype=TD[odt], device=DEV)
        a.check(L.mtj_gemm(a.ptr(A), K, a.ptr(W), None, M, N, K, a.dtype_code(TD[dt]), a.EPI_STORE, a.ptr(ob), N,
                           a.dtype_code(TD[odt]), None, 1.0, S()))
        torch.cuda.synchronize()
        assert rel_err(ob, A.double() @ Wh.double()) < TOL[odt] / 2


def test_pack_cvt_holds_bf16_weights_exactly_in_float16_and_alpha_undoes_the_scale(L):
    """The matrix-core path of a bfloat16 model: weights go to float16 times a power of two (exact for every weight
    whose scaled magnitude is a normal float16), the GEMM multiplies the accumulator by the inverse."""
    a = abi()
    g = torch.Generator().manual_seed(11)
    M, N, K = 96, 384, 256
    Wh = (torch.randn(K, N, generator=g) * 0.02).to(torch.bfloat16)
    Wh[0, 0], Wh[1, 1], Wh[2, 2] = 0.11, -3e-6, 2e-9                 # the largest weight and two tiny ones
    Wh = Wh.to(DEV)
    scale = 2.0 ** 17                                                # 0.11 * 2^17 < 2^15
    W16 = torch.empty(N, K, dtype=torch.float16, device=DEV)
    a.check(L.mtj_pack_weight_cvt(a.ptr(Wh), N, K, N, a.ptr(W16), K, 0, 0, a.BF16, a.F16, scale, S()))
    torch.cuda.synchronize()
    back = W16.double().T / scale
    exact = Wh.double()
    assert torch.equal(back[exact.abs() * scale >= 2.0 ** -14], exact[exact.abs() * scale >= 2.0 ** -14])
    assert float((back - exact).abs().max()) <= 2.0 ** -25 / scale + 1e-300      # subnormal tail: half a step of 2^-24
    A = torch.randn(M, K, generator=g).to(torch.float16).to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    out = torch.empty(M, N, device=DEV)
    a.check(L.mtj_gemm(a.ptr(A), K, a.ptr(W16), a.ptr(bias), M, N, K, a.F16, a.EPI_STORE, a.ptr(out), N, 0, None,
                       1.0 / scale, S()))
    torch.cuda.synchronize()
    assert rel_err(out, A.double() @ exact + bias.double()) < 5e-6
    # saturation instead of infinity
    big = torch.full((64, 64), 3.0e38, dtype=torch.bfloat16, device=DEV)
    o16 = torch.empty(64, 64, dtype=torch.float16, device=DEV)
    a.check(L.mtj_pack_weight_cvt(a.ptr(big), 64, 64, 64, a.ptr(o16), 64, 0, 0, a.BF16, a.F16, 1.0, S()))
    torch.cuda.synchronize()
    assert float(o16.float().max()) == 65504.0


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("M,N,K", [(32, 4096, 20480), (5, 512, 2560), (64, 260, 1024), (8, 50400, 4096), (3, 64, 64),
                                   (511, 4096, 20480), (200, 512, 2560), (700, 1024, 4096), (130, 4096, 20480), (300, 2048, 8192)])
def test_gemm_splitk_matches_reference_and_is_deterministic(L, dt, M, N, K):
    """Skinny products: K ranges run as separate workgroups and are added in a fixed order."""
    a = abi()
    g = torch.Generator().manual_seed(M * 11 + N)
    A = torch.randn(M, K, generator=g).to(TD[dt]).to(DEV)
    Wh = (torch.randn(K, N, generator=g) * 0.05).to(TD[dt]).to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    W = _packed(Wh)
    ref = A.double() @ Wh.double() + bias.double()
    code = a.dtype_code(TD[dt])
    nb = L.mtj_gemm_splitk_work_bytes(M, N, K, code)
    if (M, N, K) == (32, 4096, 20480):
        assert nb == 8 * M * N * 4                       # the out/fc_out projection of batched decode is cut 8 ways
    work = torch.empty(max(nb, 16), dtype=torch.uint8, device=DEV)
    outs = []
    for _ in range(2):
        out = torch.empty(M, N, device=DEV)
        a.check(L.mtj_gemm_splitk(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, N, K, code, a.EPI_STORE, a.ptr(out), N, 0,
                                  a.ptr(work), work.numel(), 1.0, S()))
        torch.cuda.synchronize()
        outs.append(out)
    assert rel_err(outs[0], ref) < 5e-6
    assert torch.equal(outs[0], outs[1])
    x0 = torch.randn(M, N, generator=g).to(DEV)
    x = x0.clone()
    a.check(L.mtj_gemm_splitk(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, N, K, code, a.EPI_RESID, a.ptr(x), N, 0,
                              a.ptr(work), work.numel(), 1.0, S()))
    torch.cuda.synchronize()
    assert rel_err(x, x0.double() + ref) < 5e-6
    if nb:
        with pytest.raises(ValueError):                  # a work buffer that is too small is refused
            a.check(L.mtj_gemm_splitk(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, N, K, code, a.EPI_STORE, a.ptr(out), N, 0,
                                      a.ptr(work), nb - 4, 1.0, S()))


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("M,N,K", [(32, 4096, 20480), (5, 512, 2560), (3, 64, 64), (8, 1024, 4096)])
def test_gemm_splitk_with_the_following_layernorm(L, dt, M, N, K):
    """The residual reduce that also normalises the rows it completes: x as from mtj_gemm_splitk (bit for bit), h as
    ReplicatedLayerNorm of that x."""
    a = abi()
    g = torch.Generator().manual_seed(M * 7 + N + K)
    A = torch.randn(M, K, generator=g).to(TD[dt]).to(DEV)
    Wh = (torch.randn(K, N, generator=g) * 0.05).to(TD[dt]).to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    sc = (1 + 0.1 * torch.randn(N, generator=g)).to(DEV)
    of = (0.1 * torch.randn(N, generator=g)).to(DEV)
    W = _packed(Wh)
    code = a.dtype_code(TD[dt])
    nb = L.mtj_gemm_splitk_work_bytes(M, N, K, code)
    work = torch.empty(max(nb, 16), dtype=torch.uint8, device=DEV)
    x0 = torch.randn(M, N, generator=g).to(DEV)
    x_ref = x0.clone()
    a.check(L.mtj_gemm_splitk(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, N, K, code, a.EPI_RESID, a.ptr(x_ref), N, 0,
                              a.ptr(work), work.numel(), 1.0, S()))
    for h_dt in DTS:
        x = x0.clone()
        h = torch.zeros(M, N, dtype=TD[h_dt], device=DEV)
        a.check(L.mtj_gemm_splitk_ln(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, N, K, code, a.ptr(x), N, a.ptr(work),
                                     work.numel(), a.ptr(sc), a.ptr(of), a.ptr(h), N, a.dtype_code(TD[h_dt]), 1.0, S()))
        torch.cuda.synchronize()
        assert torch.equal(x, x_ref)
        ref = O.replicated_layer_norm(x.double().cpu(), sc.double().cpu(), of.double().cpu()).to(DEV)
        assert rel_err(h, ref) < {"f32": 6e-6, "bf16": 4e-3, "f16": 5e-4}[h_dt]


def test_gemm_rejects_bad_arguments(L):
    a = abi()
    A = torch.zeros(4, 48, device=DEV)
    with pytest.raises(ValueError):   # K not a multiple of the k-tile
        a.check(L.mtj_gemm(a.ptr(A), 48, a.ptr(A), None, 4, 4, 48, 0, a.EPI_STORE, a.ptr(A), 4, 0, None, 1.0, S()))
    with pytest.raises(ValueError):   # INPROJ without geometry
        a.check(L.mtj_gemm(a.ptr(A), 32, a.ptr(A), None, 4, 4, 32, 0, a.EPI_INPROJ, None, 0, 0, None, 1.0, S()))


# ------------------------------------------------------------------ GEMV
@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("N,K", [(512, 256), (28672, 4096), (4096, 20480), (50400, 4096), (514, 2560), (6, 520),
                                 # whole-tile rows with 0 or 1, exactly 1, 3, and 4-or-5 tiles per wavefront
                                 (8, 4096), (4096, 4096), (12288, 4096), (9000, 8192)])
def test_gemv_store_resid_and_layernorm(L, dt, N, K):
    a = abi()
    g = torch.Generator().manual_seed(N + K)
    x = torch.randn(K, generator=g).to(DEV)
    Wh = (torch.randn(K, N, generator=g) * 0.02).to(TD[dt]).to(DEV)
    W = _packed(Wh)
    bias = torch.randn(N, generator=g).to(DEV)
    ref = x.double() @ Wh.double() + bias.double()
    out = torch.empty(N, device=DEV)
    a.check(L.mtj_gemv(a.ptr(x), None, None, a.ptr(W), a.ptr(bias), N, K, a.dtype_code(TD[dt]), a.EPI_STORE, a.ptr(out), 0,
                       None, None, S()))
    torch.cuda.synchronize()
    assert rel_err(out, ref) < 5e-6
    y0 = torch.randn(N, generator=g).to(DEV)
    y = y0.clone()
    a.check(L.mtj_gemv(a.ptr(x), None, None, a.ptr(W), a.ptr(bias), N, K, a.dtype_code(TD[dt]), a.EPI_RESID, a.ptr(y), 0,
                       None, None, S()))
    torch.cuda.synchronize()
    assert rel_err(y, y0.double() + ref) < 5e-6
    if K <= 16384:
        sc = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV)
        of = (0.1 * torch.randn(K, generator=g)).to(DEV)
        xr = (x * 2 + 0.7)
        a.check(L.mtj_gemv(a.ptr(xr), a.ptr(sc), a.ptr(of), a.ptr(W), a.ptr(bias), N, K, a.dtype_code(TD[dt]), a.EPI_STORE,
                           a.ptr(out), 0, None, None, S()))
        torch.cuda.synchronize()
        h = O.replicated_layer_norm(xr.double().cpu()[None], sc.double().cpu(), of.double().cpu())[0].to(DEV)
        assert rel_err(out, h @ Wh.double() + bias.double()) < 6e-6


# ------------------------------------------------------------------ fused input projection (GEMM and GEMV)
def _layer_params(cfg, seed, dt):
    p = O.seeded_params(cfg, seed, TD[dt])
    return p


def _inproj_reference(cfg, p, x64, positions):
    """q (rotated), k (rotated), v, gelu(fc_in) of layer 0 for rows at the given absolute positions (float64)."""
    l = O.Layer(cfg, p, 0, torch.float64)
    h = l.norm(x64)
    q, v, k = l.qvk_proj(h)
    r = l.r
    sin, cos = O.fixed_pos_embedding(int(max(positions)) + 1, r)
    sin, cos = sin[positions], cos[positions]

    def rot(t):
        tr = t[:, :, :r]
        s = torch.as_tensor(sin).repeat_interleave(2, -1)[:, None, :]
        c = torch.as_tensor(cos).repeat_interleave(2, -1)[:, None, :]
        return torch.cat([tr * c + O.rotate_every_two(tr) * s, t[:, :, r:]], -1)

    return rot(q), rot(k), v, O.gelu_tanh(h @ l.w1 + l.b1), h


def _run_inproj_prefill(cfg, p, dt, B, Tp, Tcap, pads, seed):
    """LayerNorm + fused q|v|k|fc_in GEMM of layer 0 through the engine's buffers; compares q, the K/V window, V^T and
    gelu(fc_in) of every real row with the float64 oracle.  A bfloat16 model runs its matrix-core path in float16."""
    from mesh_transformer.engine import Engine
    a = abi()
    d = cfg["d_model"]
    eng = Engine(cfg, {k: {n: v.to(DEV) for n, v in m.items()} for k, m in p.items()}, DEV, layer_ids=[0], embed=False, proj=False)
    ses = eng.session(B, Tcap, Tp, Tp + 8)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B * Tp, d, generator=g).to(DEV)
    pos0 = torch.tensor([-pd for pd in pads], dtype=torch.int32, device=DEV)
    w = eng.w
    L = a.lib()
    h = ses.h_pf[:B * Tp]
    act = ses.act_pf[:B * Tp]
    a.check(L.mtj_layernorm(a.ptr(x), a.ptr(w.ln_s[0]), a.ptr(w.ln_o[0]), B * Tp, d, a.ptr(h), w.act_dtype, S()))
    ip = eng._inproj(ses, 0, Tp, pos0, ses.q_pf, w.act_dtype, act, w.act_dtype, ses.vt)
    a.check(L.mtj_gemm(a.ptr(h), d, a.ptr(w.w_in_mm[0]), a.ptr(w.b1[0]), B * Tp, 3 * d + 4 * d, d, w.mm_dtype, a.EPI_INPROJ,
                       None, 0, 0, C.byref(ip), w.alpha_in[0], S()))
    torch.cuda.synchronize()
    H, dh = eng.H, eng.dh
    tol = 6e-6 if dt == "f32" else 1.2e-3        # float16 operand and float16 storage: 2^-12 relative each
    for b in range(B):
        pd = pads[b]
        rows = x[b * Tp + pd:(b + 1) * Tp].double().cpu()
        positions = np.arange(Tp - pd)
        q_ref, k_ref, v_ref, g_ref, _ = _inproj_reference(cfg, p, rows, positions)
        q = ses.q_pf[:B * H * Tp * dh].reshape(B, H, Tp, dh)[b, :, pd:].permute(1, 0, 2)
        assert rel_err(q, q_ref) < tol
        kk = ses.kc[0][b, :, :Tp - pd].permute(1, 0, 2)
        vv = ses.vc[0][b, :, :Tp - pd].permute(1, 0, 2)
        assert rel_err(kk, k_ref) < tol and rel_err(vv, v_ref) < tol
        vt = ses.vt.reshape(B, H, dh, ses.ldvt)[b, :, :, :Tp - pd].permute(2, 0, 1)
        assert torch.equal(vt.contiguous(), vv.contiguous())
        assert rel_err(act[b * Tp + pd:(b + 1) * Tp, d:], g_ref) < tol
        # nothing was written for padding rows: the slots after the real tokens are still zero
        assert float(ses.kc[0][b, :, Tp - pd:].abs().max()) == 0.0


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("shape", ["tiny", "head256"])
def test_inproj_gemm_prefill_with_left_padding(dt, shape):
    cfg = dict(layers=1, d_model=512, n_heads=8, n_vocab=64, pe="rotary", pe_rotary_dims=32, cores_per_replica=1) \
        if shape == "tiny" else \
        dict(layers=1, d_model=512, n_heads=2, n_vocab=64, pe="rotary", pe_rotary_dims=64, cores_per_replica=1)
    _run_inproj_prefill(cfg, _layer_params(cfg, 3, dt), dt, B=2, Tp=40, Tcap=50, pads=[0, 7], seed=4)


def test_inproj_gemm_on_the_256x256_direct_to_lds_kernel():
    """M = 1024 rows x N = 14336 columns is 4 x 56 = 224 tiles of 256 x 256: mtj_gemm dispatches gemm_dma_kernel (at
    least 200 such tiles), whose 8-wavefront epilogue (RoPE, K/V ring, V^T, GELU) the small shapes never reach."""
    cfg = dict(layers=1, d_model=2048, n_heads=8, n_vocab=64, pe="rotary", pe_rotary_dims=64, cores_per_replica=1)
    _run_inproj_prefill(cfg, _layer_params(cfg, 9, "bf16"), "bf16", B=2, Tp=512, Tcap=600, pads=[0, 37], seed=10)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_gemm_resid_and_store_on_the_256x256_direct_to_lds_kernel(L, dt):
    """M = N = 4096 is 256 tiles of 256 x 256, so mtj_gemm itself (no K split) runs gemm_dma_kernel with the RESID and
    STORE epilogues; K = 4096 * 5 is the out|fc_out depth of the 6B model.  Reference: float64 product on the GPU."""
    a = abi()
    g = torch.Generator().manual_seed(21)
    M, N, K = 4096, 4096, 20480
    A = torch.randn(M, K, generator=g).to(TD[dt]).to(DEV)
    Wh = (torch.randn(K, N, generator=g) * 0.02).to(TD[dt]).to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    W = _packed(Wh)
    ref = A.double() @ Wh.double() + bias.double()
    x0 = torch.randn(M, N, generator=g).to(DEV)
    x = x0.clone()
    code = a.dtype_code(TD[dt])
    a.check(L.mtj_gemm(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, N, K, code, a.EPI_RESID, a.ptr(x), N, 0, None, 1.0, S()))
    out = torch.empty(M - 100, N, device=DEV)                 # a ragged last row tile
    a.check(L.mtj_gemm(a.ptr(A), K, a.ptr(W), a.ptr(bias), M - 100, N, K, code, a.EPI_STORE, a.ptr(out), N, 0, None, 0.5, S()))
    torch.cuda.synchronize()
    assert rel_err(x, x0.double() + ref) < 5e-6
    assert rel_err(out, 0.5 * (ref[:M - 100] - bias.double()) + bias.double()) < 5e-6


@pytest.mark.parametrize("K", [64, 128, 192, 320])
@pytest.mark.parametrize("N,ldo", [(4096, 4096), (4090, 4091)])
def test_direct_to_lds_kernel_with_few_k_tiles_and_ragged_columns(L, K, N, ldo):
    """One, two, three and five k-tiles of 64 (the main loop of gemm_dma_kernel handles k-tiles in pairs, requests
    operands two k-tiles ahead and must not read a tile that was never requested), and a column count / output pitch
    that is not a multiple of four, which sends the epilogue down its element-wise stores (16 x 16 = 256 tiles of
    256 x 256 either way, so mtj_gemm dispatches that kernel).  Reference: float64 product on the GPU."""
    a = abi()
    g = torch.Generator().manual_seed(K + N)
    M = 4000                                                   # a ragged last row tile as well
    A = torch.randn(M, K, generator=g).to(torch.float16).to(DEV)
    Wh = (torch.randn(K, N, generator=g) * 0.05).to(torch.float16).to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    W = _packed(Wh)
    ref = A.double() @ Wh.double() + bias.double()
    x0 = torch.randn(M, ldo, generator=g).to(DEV)
    x = x0.clone()
    code = a.dtype_code(torch.float16)
    a.check(L.mtj_gemm(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, N, K, code, a.EPI_RESID, a.ptr(x), ldo, 0, None, 1.0, S()))
    out = torch.full((M, ldo), 7.0, dtype=torch.float16, device=DEV)
    a.check(L.mtj_gemm(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, N, K, code, a.EPI_STORE, a.ptr(out), ldo, a.dtype_code(torch.float16),
                       None, 1.0, S()))
    torch.cuda.synchronize()
    assert rel_err(x[:, :N], x0[:, :N].double() + ref) < 5e-6
    assert torch.equal(x[:, N:], x0[:, N:])                    # nothing written beyond column N
    assert rel_err(out[:, :N], ref) < 1e-3                     # float16 output
    assert bool((out[:, N:] == 7.0).all())


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_inproj_gemv_decode_appends_to_ring(dt):
    from mesh_transformer.engine import Engine
    a = abi()
    cfg = dict(layers=1, d_model=512, n_heads=8, n_vocab=64, pe="rotary", pe_rotary_dims=32, cores_per_replica=1)
    p = _layer_params(cfg, 5, dt)
    eng = Engine(cfg, {k: {n: v.to(DEV) for n, v in m.items()} for k, m in p.items()}, DEV, layer_ids=[0], embed=False, proj=False)
    Tcap = 6
    ses = eng.session(1, Tcap, 1, 64)
    L, w = a.lib(), eng.w
    g = torch.Generator().manual_seed(6)
    for pos in (0, 5, 6, 13):            # 6 and 13 wrap around the 6-slot window
        x = torch.randn(1, 512, generator=g).to(DEV)
        ses.pos.fill_(pos)
        ip = eng._inproj(ses, 0, 1, ses.pos, ses.q, 0, ses.act, 0, None)
        a.check(L.mtj_gemv(a.ptr(x), a.ptr(w.ln_s[0]), a.ptr(w.ln_o[0]), a.ptr(w.w_in[0]), a.ptr(w.b1[0]), 3 * 512 + 2048, 512,
                           w.dtype, a.EPI_INPROJ, None, 0, C.byref(ip), None, S()))
        torch.cuda.synchronize()
        q_ref, k_ref, v_ref, g_ref, _ = _inproj_reference(cfg, p, x.double().cpu(), np.array([pos]))
        tol = TOL[dt] * 3 if dt == "f32" else 5e-4       # the K/V window of a bfloat16 model is float16
        assert rel_err(ses.q.reshape(1, eng.H, eng.dh), q_ref) < 3e-6
        assert rel_err(ses.kc[0][0, :, pos % Tcap][None], k_ref) < tol
        assert rel_err(ses.vc[0][0, :, pos % Tcap][None], v_ref) < tol
        assert rel_err(ses.act[:, 512:], g_ref) < 3e-6


# ------------------------------------------------------------------ attention
def _attn_reference(q, k, v, n_pad):
    """q, k, v: [T, H, dh] float64, already rotated; causal + left-pad mask; returns [T - n_pad, H*dh]."""
    T, H, dh = q.shape
    s = torch.einsum("thd,Thd->htT", q, k) / math.sqrt(dh)
    bias = O.MASK * (1.0 - torch.tril(torch.ones(T, T, dtype=torch.float64)))
    bias = bias - 1e10 * (torch.arange(T) < n_pad).double()
    w = torch.softmax(s + bias, -1)
    return torch.einsum("htT,Thd->thd", w, v).reshape(T, H * dh)[n_pad:]


ATT_TOL = {"f32": 3e-6, "bf16": 8e-3, "f16": 1e-3}      # probabilities and the output are rounded to the storage type


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("dh,H", [(64, 3), (256, 2)])
@pytest.mark.parametrize("Tp", [1, 33, 128, 200])
def test_attn_prefill(L, dt, dh, H, Tp):
    a = abi()
    g = torch.Generator().manual_seed(Tp + dh)
    B, Tcap = 2, Tp + 3
    pads = [0, min(5, Tp - 1)]
    ldvt = (Tp + 63) // 64 * 64
    q = torch.randn(B, H, Tp, dh, generator=g).to(TD[dt]).to(DEV)
    kc = torch.zeros(B, H, Tcap, dh, dtype=TD[dt], device=DEV)
    vt = torch.full((B, H, dh, ldvt), float("nan"), dtype=TD[dt], device=DEV)   # unwritten keys must never be read
    kk = torch.randn(B, H, Tp, dh, generator=g).to(TD[dt]).to(DEV)
    vv = torch.randn(B, H, Tp, dh, generator=g).to(TD[dt]).to(DEV)
    for b in range(B):
        n = Tp - pads[b]
        kc[b, :, :n] = kk[b, :, pads[b]:]
        vt[b, :, :, :n] = vv[b, :, pads[b]:].permute(0, 2, 1)
    pos0 = torch.tensor([-pd for pd in pads], dtype=torch.int32, device=DEV)
    ld_out = H * dh + 16
    out = torch.full((B * Tp, ld_out), 7.0, dtype=TD[dt], device=DEV)
    a.check(L.mtj_attn_prefill(a.ptr(q), a.ptr(kc), a.ptr(vt), a.ptr(pos0), B, H, Tp, Tcap, dh, ldvt, a.ptr(out), ld_out,
                               a.dtype_code(TD[dt]), None, S()))
    torch.cuda.synchronize()
    for b in range(B):
        pd = pads[b]
        ref = _attn_reference(q[b].permute(1, 0, 2).double().cpu(), kk[b].permute(1, 0, 2).double().cpu(),
                              vv[b].permute(1, 0, 2).double().cpu(), pd)
        got = out[b * Tp + pd:(b + 1) * Tp, :H * dh]
        assert rel_err(got, ref) < ATT_TOL[dt], (dt, dh, Tp, b)
        assert float(out[b * Tp:b * Tp + pd, :H * dh].float().abs().max() if pd else 0.0) == 0.0   # padding rows: zeros
    assert torch.all(out[:, H * dh:] == 7.0)
    # evaluation mask (transformer_shard.py:130): keys beyond key_limit[b] are hidden from every query
    if Tp >= 33:
        lim = [Tp // 2, Tp - 1]
        kl = torch.tensor(lim, dtype=torch.int32, device=DEV)
        zero = torch.zeros(B, dtype=torch.int32, device=DEV)
        kc2 = kk.clone()
        vt2 = torch.zeros(B, H, dh, ldvt, dtype=TD[dt], device=DEV)
        vt2[:, :, :, :Tp] = vv.permute(0, 1, 3, 2)
        kcf = torch.zeros(B, H, Tcap, dh, dtype=TD[dt], device=DEV)
        kcf[:, :, :Tp] = kc2
        a.check(L.mtj_attn_prefill(a.ptr(q), a.ptr(kcf), a.ptr(vt2), a.ptr(zero), B, H, Tp, Tcap, dh, ldvt, a.ptr(out),
                                   ld_out, a.dtype_code(TD[dt]), a.ptr(kl), S()))
        torch.cuda.synchronize()
        for b in range(B):
            qq, kq, vq = (t[b].permute(1, 0, 2).double().cpu() for t in (q, kk, vv))
            sc = torch.einsum("thd,Thd->htT", qq, kq) / math.sqrt(dh)
            bias = O.MASK * (1.0 - torch.tril(torch.ones(Tp, Tp, dtype=torch.float64)))
            bias = bias + (torch.arange(Tp) > lim[b]).double() * -1e10
            ref = torch.einsum("htT,Thd->thd", torch.softmax(sc + bias, -1), vq).reshape(Tp, H * dh)
            assert rel_err(out[b * Tp:(b + 1) * Tp, :H * dh], ref) < ATT_TOL[dt], (dt, dh, Tp, b)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_attn_prefill_full_context_d256(L, dt):
    """2048 queries per sequence at d_head 256 with ragged left padding: 16 query blocks per head, dispatched longest
    first, every key tile count from 1 to 64 - the shape of the 6B prefill, against the float64 reference."""
    a = abi()
    g = torch.Generator().manual_seed(77)
    B, H, Tp, dh = 2, 2, 2048, 256
    Tcap, pads = Tp, [0, 301]
    ldvt = Tp + 64
    q = torch.randn(B, H, Tp, dh, generator=g).to(TD[dt]).to(DEV)
    kk = torch.randn(B, H, Tp, dh, generator=g).to(TD[dt]).to(DEV)
    vv = torch.randn(B, H, Tp, dh, generator=g).to(TD[dt]).to(DEV)
    kc = torch.zeros(B, H, Tcap, dh, dtype=TD[dt], device=DEV)
    vt = torch.full((B, H, dh, ldvt), float("nan"), dtype=TD[dt], device=DEV)
    for b in range(B):
        n = Tp - pads[b]
        kc[b, :, :n] = kk[b, :, pads[b]:]
        vt[b, :, :, :n] = vv[b, :, pads[b]:].permute(0, 2, 1)
    pos0 = torch.tensor([-pd for pd in pads], dtype=torch.int32, device=DEV)
    out = torch.zeros(B * Tp, H * dh, dtype=TD[dt], device=DEV)
    a.check(L.mtj_attn_prefill(a.ptr(q), a.ptr(kc), a.ptr(vt), a.ptr(pos0), B, H, Tp, Tcap, dh, ldvt, a.ptr(out), H * dh,
                               a.dtype_code(TD[dt]), None, S()))
    torch.cuda.synchronize()
    for b in range(B):
        pd = pads[b]
        ref = _attn_reference(q[b].permute(1, 0, 2).double().cpu(), kk[b].permute(1, 0, 2).double().cpu(),
                              vv[b].permute(1, 0, 2).double().cpu(), pd)
        got = out[b * Tp + pd:(b + 1) * Tp].double().cpu()
        assert rel_err(got, ref) < ATT_TOL[dt], (dt, b)
        # no row is far off either (a wrong tile or a stale buffer would show as a few bad rows)
        row_err = (got - ref).norm(dim=1) / ref.norm(dim=1)
        assert float(row_err.max()) < 4 * ATT_TOL[dt], (dt, b, int(row_err.argmax()))


def _attn_all_heads_f32(q, kk, vv, pads, key_limit=None):
    """Every (sequence, head) at once in float32 on the GPU: a plain torch evaluation of the same masked softmax, for
    shapes where the float64 host reference is only affordable on a few heads."""
    B, H, Tp, dh = q.shape
    sc = torch.einsum("bhtd,bhTd->bhtT", q.float(), kk.float()) / math.sqrt(dh)
    idx = torch.arange(Tp, device=q.device)
    hide = idx[None, :] > idx[:, None]                                  # causal
    hide = hide[None] | (idx[None, None, :] < torch.tensor(pads, device=q.device)[:, None, None])
    if key_limit is not None:
        hide = hide | (idx[None, None, :] > torch.tensor(key_limit, device=q.device)[:, None, None])
    sc = sc.masked_fill(hide[:, None], float("-inf"))
    out = torch.einsum("bhtT,bhTd->bthd", torch.softmax(sc, -1), vv.float())
    return out.reshape(B, Tp, H * dh)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("B,H,Tp,with_limit", [(64, 16, 200, False), (32, 16, 257, True), (128, 8, 33, False),
                                               (8, 16, 2048, False), (11, 16, 1500, True), (35, 10, 700, False)])
def test_attn_prefill_256_query_workgroups(L, dt, B, H, Tp, with_limit):
    """Shapes with at least 1024 blocks of 256 queries run the kernel in which one wavefront owns 64 queries (d_head
    256) and a workgroup two query blocks: ragged left padding per sequence, a query count that is no multiple of
    anything, a partial last key tile (unwritten V^T columns are NaN), the evaluation key limit, the full 2048-token
    context, an odd number of query blocks (the middle one has no partner), a number of (sequence, head) pairs that is
    no multiple of 8.  Against the float64 reference on four (sequence, head) pairs and a float32 torch evaluation on
    all of them."""
    a = abi()
    g = torch.Generator().manual_seed(B * 1000 + Tp)
    dh = 256
    assert B * H * ((Tp + 255) // 256) >= 1024
    Tcap = Tp + 7
    pads = [int(x) for x in torch.randint(0, max(min(Tp - 1, Tp // 3), 1), (B,), generator=g)]
    pads[0] = 0
    lim = [int(x) for x in torch.randint(Tp // 3, Tp, (B,), generator=g)] if with_limit else None
    if with_limit:
        pads = [0] * B                                              # the evaluation path has no padding
    ldvt = (Tp + 63) // 64 * 64
    q = torch.randn(B, H, Tp, dh, generator=g).to(TD[dt]).to(DEV)
    kk = torch.randn(B, H, Tp, dh, generator=g).to(TD[dt]).to(DEV)
    vv = torch.randn(B, H, Tp, dh, generator=g).to(TD[dt]).to(DEV)
    kc = torch.zeros(B, H, Tcap, dh, dtype=TD[dt], device=DEV)
    vt = torch.full((B, H, dh, ldvt), float("nan"), dtype=TD[dt], device=DEV)   # unwritten keys must never be read
    for b in range(B):
        n = Tp - pads[b]
        kc[b, :, :n] = kk[b, :, pads[b]:]
        vt[b, :, :, :n] = vv[b, :, pads[b]:].permute(0, 2, 1)
    pos0 = torch.tensor([-pd for pd in pads], dtype=torch.int32, device=DEV)
    kl = torch.tensor(lim, dtype=torch.int32, device=DEV) if with_limit else None
    ld_out = H * dh + 8
    out = torch.full((B * Tp, ld_out), 7.0, dtype=TD[dt], device=DEV)
    a.check(L.mtj_attn_prefill(a.ptr(q), a.ptr(kc), a.ptr(vt), a.ptr(pos0), B, H, Tp, Tcap, dh, ldvt, a.ptr(out), ld_out,
                               a.dtype_code(TD[dt]), a.ptr(kl), S()))
    torch.cuda.synchronize()
    assert torch.all(out[:, H * dh:] == 7.0)
    got = out[:, :H * dh].reshape(B, Tp, H * dh).float()
    assert bool(torch.isfinite(got).all())
    ref32 = _attn_all_heads_f32(q, kk, vv, pads, lim)
    for b in range(B):
        pd = pads[b]
        if pd:
            assert float(got[b, :pd].abs().max()) == 0.0            # padding rows: zeros
        e = float((got[b, pd:] - ref32[b, pd:]).norm() / ref32[b, pd:].norm())
        assert e < ATT_TOL[dt], (dt, b, e)
        row = (got[b, pd:] - ref32[b, pd:]).norm(dim=1) / ref32[b, pd:].norm(dim=1)
        assert float(row.max()) < 6 * ATT_TOL[dt], (dt, b, int(row.argmax()) + pd)
    for b, h in ((0, 0), (1, H - 1), (B - 1, H // 2), (B // 2, 3)):
        qq, kq, vq = (t[b, h].double().cpu() for t in (q, kk, vv))
        sc = qq @ kq.T / math.sqrt(dh)
        idx = torch.arange(Tp)
        hide = (idx[None, :] > idx[:, None]) | (idx[None, :] < pads[b])
        if with_limit:
            hide = hide | (idx[None, :] > lim[b])
        ref = torch.softmax(sc.masked_fill(hide, float("-inf")), -1) @ vq
        assert rel_err(got[b, pads[b]:, h * dh:(h + 1) * dh], ref[pads[b]:]) < ATT_TOL[dt], (dt, b, h)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("dh,H", [(64, 8), (256, 16)])
@pytest.mark.parametrize("Tcap,positions", [(7, [0, 6, 9]), (300, [0, 150, 299]), (2047, [511, 2046, 5000]), (2047, [700]),
                                            # many sequences, ragged positions, some beyond the window
                                            (1000, [(i * 131) % 1300 for i in range(24)])])
def test_attn_decode_window(L, dt, dh, H, Tcap, positions):
    a = abi()
    g = torch.Generator().manual_seed(Tcap + dh)
    B = len(positions)
    q = torch.randn(B, H, dh, generator=g).to(DEV)
    kc = torch.randn(B, H, Tcap, dh, generator=g).to(TD[dt]).to(DEV)
    vc = torch.randn(B, H, Tcap, dh, generator=g).to(TD[dt]).to(DEV)
    pos = torch.tensor(positions, dtype=torch.int32, device=DEV)
    work = torch.zeros(L.mtj_attn_decode_work_bytes(B, H, dh, Tcap), dtype=torch.uint8, device=DEV)
    out = torch.zeros(B, H * dh + 8, device=DEV)
    a.check(L.mtj_attn_decode(a.ptr(q), a.ptr(kc), a.ptr(vc), a.ptr(pos), B, H, Tcap, dh, a.ptr(out), H * dh + 8, 0,
                              a.dtype_code(TD[dt]), a.ptr(work), S()))
    torch.cuda.synchronize()
    for b, p in enumerate(positions):
        n = min(p + 1, Tcap)
        s = torch.einsum("hd,hTd->hT", q[b].double(), kc[b, :, :n].double()) / math.sqrt(dh)
        ref = torch.einsum("hT,hTd->hd", torch.softmax(s, -1), vc[b, :, :n].double()).reshape(-1)
        assert rel_err(out[b, :H * dh], ref) < 3e-6, (dt, dh, Tcap, p)


@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("dh,H,F", [(64, 8, 2048), (256, 16, 16384)])
@pytest.mark.parametrize("Tcap,p", [(2047, 650), (2047, 2046), (130, 3), (9, 40)])
def test_attn_decode_partials_merged_by_the_out_projection_gemv(L, dt, dh, H, F, Tcap, p):
    """Batch 1: the per-range partials of the one-token attention are merged by mtj_gemv while it stages its input;
    x += [attention | gelu] @ W_out + b must equal the float64 evaluation of layers.py:275-285, 290, 313."""
    a = abi()
    g = torch.Generator().manual_seed(Tcap + dh + p)
    d = H * dh
    q = torch.randn(1, H, dh, generator=g).to(DEV)
    kc = torch.randn(1, H, Tcap, dh, generator=g).to(TD[dt]).to(DEV)
    vc = torch.randn(1, H, Tcap, dh, generator=g).to(TD[dt]).to(DEV)
    pos = torch.tensor([p], dtype=torch.int32, device=DEV)
    work = torch.zeros(L.mtj_attn_decode_work_bytes(1, H, dh, Tcap), dtype=torch.uint8, device=DEV)
    am = a.AttnMerge()
    a.check(L.mtj_attn_decode_partials(a.ptr(q), a.ptr(kc), a.ptr(vc), a.ptr(pos), 1, H, Tcap, dh, a.dtype_code(TD[dt]),
                                       a.ptr(work), C.byref(am), S()))
    assert am.splits == L.mtj_attn_decode_splits(1, H, Tcap) and am.n_heads == H and am.d_head == dh
    wdt = "f32" if dt == "f32" else "bf16"
    act = torch.randn(1, d + F, generator=g).to(DEV)
    act[:, :d] = float("nan")                                   # the attention columns must come from the partials
    Wh = (torch.randn(d + F, d, generator=g) * 0.02).to(TD[wdt]).to(DEV)
    W = _packed(Wh)
    bias = torch.randn(d, generator=g).to(DEV)
    x0 = torch.randn(d, generator=g).to(DEV)
    x = x0.clone()
    a.check(L.mtj_gemv(a.ptr(act), None, None, a.ptr(W), a.ptr(bias), d, d + F, a.dtype_code(TD[wdt]), a.EPI_RESID, a.ptr(x),
                       0, None, C.byref(am), S()))
    torch.cuda.synchronize()
    n = min(p + 1, Tcap)
    sc = torch.einsum("hd,hTd->hT", q[0].double(), kc[0, :, :n].double()) / math.sqrt(dh)
    att = torch.einsum("hT,hTd->hd", torch.softmax(sc, -1), vc[0, :, :n].double()).reshape(-1)
    inp = torch.cat([att, act[0, d:].double()])
    ref = x0.double() + inp @ Wh.double() + bias.double()
    assert rel_err(x, ref) < 5e-6, (dt, dh, Tcap, p)


@pytest.mark.parametrize("dt,dh,H,F", [("f16", 256, 16, 16384), ("f32", 64, 32, 8192), ("f16", 64, 64, 4096)])
def test_out_projection_with_the_attention_inside(L, dt, dh, H, F):
    """mtj_gemv_attn: x += [attention(q, window) | gelu] @ W_out + b in ONE launch (the attention partials are produced
    by the first workgroups and merged behind an arrival counter), against the float64 evaluation of
    layers.py:275-285, 290, 313 - several window fills, launches back to back on one counter block."""
    a = abi()
    wdt = "f32" if dt == "f32" else "bf16"
    d = H * dh
    Tcap = 2047
    assert L.mtj_gemv_attn_supported(d, d + F, a.dtype_code(TD[wdt]), H, dh, a.dtype_code(TD[dt]), Tcap) == 1
    g = torch.Generator().manual_seed(dh + H)
    kc = torch.randn(1, H, Tcap, dh, generator=g).to(TD[dt]).to(DEV)
    vc = torch.randn(1, H, Tcap, dh, generator=g).to(TD[dt]).to(DEV)
    Wh = (torch.randn(d + F, d, generator=g) * 0.02).to(TD[wdt]).to(DEV)
    W = _packed(Wh)
    bias = torch.randn(d, generator=g).to(DEV)
    work = torch.zeros(L.mtj_gemv_attn_work_bytes(H, dh), dtype=torch.uint8, device=DEV)
    for p in (650, 0, 5, 2046, 7000, 63):
        q = torch.randn(1, H, dh, generator=g).to(DEV)
        act = torch.randn(1, d + F, generator=g).to(DEV)
        act[:, :d] = float("nan")                              # the attention columns must not be read from x
        x0 = torch.randn(d, generator=g).to(DEV)
        x = x0.clone()
        pos = torch.tensor([p], dtype=torch.int32, device=DEV)
        a.check(L.mtj_gemv_attn(a.ptr(act), a.ptr(W), a.ptr(bias), d, d + F, a.dtype_code(TD[wdt]), a.ptr(x), a.ptr(q),
                                a.ptr(kc), a.ptr(vc), a.ptr(pos), H, Tcap, dh, a.dtype_code(TD[dt]), a.ptr(work), S()))
        torch.cuda.synchronize()
        n = min(p + 1, Tcap)
        sc = torch.einsum("hd,hTd->hT", q[0].double(), kc[0, :, :n].double()) / math.sqrt(dh)
        att = torch.einsum("hT,hTd->hd", torch.softmax(sc, -1), vc[0, :, :n].double()).reshape(-1)
        ref = x0.double() + torch.cat([att, act[0, d:].double()]) @ Wh.double() + bias.double()
        assert rel_err(x, ref) < 5e-6, (dt, dh, p)
    words = work[:16].view(torch.int32).cpu()
    assert int(words[2]) == 0                                  # no launch gave up waiting
    assert int(words[0]) % 6 == 0 and int(words[0]) > 0        # six launches, every workgroup arrived each time


def test_out_projection_with_attention_refuses_other_shapes(L):
    a = abi()
    assert L.mtj_gemv_attn_supported(512, 2560, a.BF16, 8, 64, a.F16, 200) == 0     # K is not a whole number of tiles
    assert L.mtj_gemv_attn_supported(4096, 4096, a.BF16, 16, 256, a.F16, 200) == 0  # nothing but attention columns
    t = torch.zeros(4096, device=DEV)
    rc = L.mtj_gemv_attn(a.ptr(t), a.ptr(t), None, 512, 2560, a.BF16, a.ptr(t[2048:]), a.ptr(t), a.ptr(t), a.ptr(t),
                         a.ptr(t.view(torch.int32)), 8, 200, 64, a.F16, a.ptr(t), S())
    assert rc == -5 and b"mtj_gemv_attn_supported" in L.mtj_last_error()


# ------------------------------------------------------------------ the same kernels as torch.ops.mtj operators
def test_torch_ops_reach_the_same_kernels():
    from mesh_transformer import ops  # noqa: F401
    g = torch.Generator().manual_seed(5)
    M, K, N = 70, 256, 192
    x = torch.randn(M, K, generator=g).to(DEV)
    sc, of = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV), (0.1 * torch.randn(K, generator=g)).to(DEV)
    h = torch.ops.mtj.layernorm(x, sc, of, 0)
    ref = O.replicated_layer_norm(x.double().cpu(), sc.double().cpu(), of.double().cpu())
    assert rel_err(h, ref) < 3e-6
    h16 = torch.ops.mtj.layernorm(x, sc, of, 2)
    assert h16.dtype == torch.float16 and rel_err(h16, ref) < 5e-4
    Wh = (torch.randn(K, N, generator=g) * 0.05).to(torch.bfloat16).to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    W16 = torch.ops.mtj.pack_weight_f16(Wh, 64.0)
    y = torch.ops.mtj.gemm(h16, W16, bias, 1.0 / 64.0, 0)
    assert rel_err(y, h16.double() @ Wh.double() + bias.double()) < 5e-6
    x2 = torch.randn(M, N, generator=g).to(DEV)
    x2_0 = x2.clone()
    torch.ops.mtj.gemm_resid_(x2, h16, W16, bias, 1.0 / 64.0)
    assert rel_err(x2, x2_0.double() + h16.double() @ Wh.double() + bias.double()) < 5e-6
    Wp = torch.ops.mtj.pack_weight(Wh)
    assert torch.equal(Wp, Wh.T.contiguous())
    v = torch.ops.mtj.gemv(x[0].contiguous(), Wp, bias, sc, of)
    assert rel_err(v, ref[0].to(DEV) @ Wh.double() + bias.double()) < 6e-6
    # one-token attention, embedding, cross entropy, samplers
    B, H, Tcap, dh = 2, 4, 50, 64
    q = torch.randn(B, H, dh, generator=g).to(DEV)
    kc = torch.randn(B, H, Tcap, dh, generator=g).to(torch.float16).to(DEV)
    vc = torch.randn(B, H, Tcap, dh, generator=g).to(torch.float16).to(DEV)
    pos = torch.tensor([10, 70], dtype=torch.int32, device=DEV)
    o = torch.ops.mtj.attn_decode(q, kc, vc, pos, 0)
    for b, p in enumerate([10, 70]):
        n = min(p + 1, Tcap)
        s_ = torch.einsum("hd,hTd->hT", q[b].double(), kc[b, :, :n].double()) / math.sqrt(dh)
        assert rel_err(o[b], torch.einsum("hT,hTd->hd", torch.softmax(s_, -1), vc[b, :, :n].double()).reshape(-1)) < 3e-6
    We = torch.randn(100, 32, generator=g).to(DEV)
    tok = torch.tensor([3, 99], dtype=torch.int32, device=DEV)
    assert torch.equal(torch.ops.mtj.embed(tok, We, bias[:32].contiguous()), We[tok.long()] + bias[:32])
    lg = torch.randn(5, 300, generator=g).to(DEV)
    tgt = torch.tensor([1, 299, 7, 0, 150], dtype=torch.int32, device=DEV)
    loss, correct = torch.ops.mtj.xent(lg, tgt)
    assert rel_err(loss, torch.nn.functional.cross_entropy(lg.double(), tgt.long(), reduction="none")) < 1e-6
    assert torch.equal(torch.ops.mtj.sample_greedy(lg).long(), lg.argmax(-1))
    f64 = lambda v: torch.full((5,), v, dtype=torch.float64, device=DEV)
    t, filt, keep = torch.ops.mtj.sample_nucleus(lg, f64(0.5), f64(1.0), None, f64(0.3))
    want = O.nucleaus_filter(lg.cpu().numpy(), 0.5)
    assert np.array_equal(filt.cpu().numpy(), want) and np.array_equal(keep.cpu().numpy(), want == lg.cpu().numpy())


# ------------------------------------------------------------------ samplers: bit-exact against the oracle
def _sample(L, logits, top_p, temp, top_k, u):
    a = abi()
    R, V = logits.shape
    lg = torch.from_numpy(logits).to(DEV)
    f64 = lambda v: torch.tensor(np.broadcast_to(np.asarray(v, np.float64), (R,)).copy(), dtype=torch.float64, device=DEV)
    tk = None if top_k is None else torch.tensor(np.broadcast_to(np.asarray(top_k, np.int32), (R,)).copy(), dtype=torch.int32, device=DEV)
    uu = f64(u).reshape(R, 1).contiguous()
    tok = torch.zeros(R, dtype=torch.int32, device=DEV)
    pos = torch.zeros(R, dtype=torch.int32, device=DEV)
    pos_start = torch.zeros(R, dtype=torch.int32, device=DEV)
    mask = torch.zeros(R, V, dtype=torch.uint8, device=DEV)
    filt = torch.zeros(R, V, dtype=torch.float32, device=DEV)
    work = torch.empty(L.mtj_sample_work_bytes(R, V), dtype=torch.uint8, device=DEV)
    tp, tm = f64(top_p), f64(temp)
    a.check(L.mtj_sample_nucleus(a.ptr(lg), R, V, a.ptr(tp), a.ptr(tm), a.ptr(tk), a.ptr(uu), 1, a.ptr(tok), None, 0,
                                 a.ptr(pos), a.ptr(pos_start), a.ptr(mask), a.ptr(filt), a.ptr(work), None, S()))
    torch.cuda.synchronize()
    assert torch.all(pos == 1)
    return tok.cpu().numpy(), mask.cpu().numpy().astype(bool), filt.cpu().numpy()


def test_nucleus_reference_demo_vector(L):
    demo = np.array([[-2, -1, 0, 0.8, 0, 0.1, 0.3, 0.4, 0.5, 0.6, 0.7, -3]], np.float32)   # sampling.py:49
    tok, mask, filt = _sample(L, demo, 0.9, 1.0, None, 0.5)
    assert set(np.nonzero(~mask[0])[0].tolist()) == {0, 1, 11}
    assert np.array_equal(filt, O.nucleaus_filter(demo, 0.9))


@pytest.mark.parametrize("V", [12, 1000, 50400])
@pytest.mark.parametrize("spread", [0.3, 1.3, 6.0])
def test_nucleus_bit_exact_vs_oracle(L, V, spread):
    rng = np.random.default_rng(V + int(spread * 10))
    R = 6
    logits = (rng.standard_normal((R, V)) * spread).astype(np.float32)
    logits[1, : V // 2] = logits[1, V // 2: 2 * (V // 2)]        # a row full of ties
    logits[2, 3] = -0.0
    logits[2, 4] = 0.0
    # top_p == 1.0 exactly is left out on purpose: the total mass is 1 up to rounding, so whether the running
    # sum "exceeds" it depends on the order of a float64 summation, which a parallel scan does not share with
    # a sequential cumsum; 2.0 is the well-posed "keep everything"
    top_p = np.array([0.9, 0.5, 0.999, 0.05, 2.0, 0.7])
    temp = np.array([0.8, 1.0, 1.5, 0.3, 0.8, 2.0])
    u = rng.random(R)
    for top_k in (None, np.array([40, 1, 5, V, 3, 100], np.int32)):
        tok, mask, filt = _sample(L, logits, top_p, temp, top_k, u)
        for r in range(R):
            k = None if top_k is None else int(top_k[r])
            f_ref = O.nucleaus_filter(logits[r:r + 1], float(top_p[r]), k)
            assert np.array_equal(filt[r:r + 1], f_ref), (V, spread, r, k)
            assert np.array_equal(mask[r], f_ref[0] == logits[r])
            assert tok[r] == O.inverse_cdf_draw(logits[r:r + 1], f_ref, float(temp[r]), float(u[r])), (V, spread, r, k)


def _check_rows(L, logits, top_p, temp, top_k, u):
    tok, mask, filt = _sample(L, logits, top_p, temp, top_k, u)
    for r in range(logits.shape[0]):
        k = None if top_k is None else int(np.broadcast_to(top_k, (logits.shape[0],))[r])
        tp, tm, ur = (float(np.broadcast_to(v, (logits.shape[0],))[r]) for v in (top_p, temp, u))
        f_ref = O.nucleaus_filter(logits[r:r + 1], tp, k)
        assert np.array_equal(filt[r:r + 1], f_ref), r
        assert np.array_equal(mask[r], f_ref[0] == logits[r]), r
        assert tok[r] == O.inverse_cdf_draw(logits[r:r + 1], f_ref, tm, ur), r


@pytest.mark.parametrize("V", [50400, 65536, 700])
def test_nucleus_crowded_and_degenerate_rows(L, V):
    """Rows that defeat the bucketing of the selection: every logit equal, hundreds of copies of the value at which
    the running mass crosses, -inf entries, one far outlier, a row whose whole weight sits on one token."""
    rng = np.random.default_rng(V)
    R = 7
    logits = (rng.standard_normal((R, V)) * 2.0).astype(np.float32)
    logits[0] = 0.25                                        # one bucket, one value: ids decide
    logits[1, rng.permutation(V)[: V // 3]] = logits[1].max()   # the mass crosses inside a run of equal maxima
    logits[2, ::5] = -np.inf
    logits[3, 17] = 3.0e5                                   # everything else has no weight
    logits[4] = np.round(logits[4] * 4) / 4                 # 40-odd distinct values
    logits[5, : V // 2] = -1.0e4
    logits[6] = np.linspace(-3, 3, V, dtype=np.float32)[rng.permutation(V)]
    top_p = np.array([0.9001, 0.5003, 0.9, 0.9, 0.8002, 0.95, 0.3001])
    temp = np.array([1.0, 0.7, 1.3, 0.8, 1.0, 2.5, 0.05])
    for u in (rng.random(R), np.zeros(R), np.full(R, 0.999999)):
        _check_rows(L, logits, top_p, temp, None, u)
    _check_rows(L, logits, top_p, temp, np.array([V // 2, 3, 1, 2, 100, V - 1, 64], np.int32), rng.random(R))


def test_nucleus_unusual_parameters(L):
    """Parameters outside the usual case, where a filtered token keeps a weight or the order of filtered / temp
    turns around: top_k 0 (every rank penalised by 1e10 * id), temperatures of 1e8 and 1e10 (1e10 / temp is no longer
    out of reach), u = 1 (no running weight exceeds the total: the last token with a weight), top_p 0 and below."""
    rng = np.random.default_rng(11)
    V, R = 3000, 6
    logits = (rng.standard_normal((R, V)) * 1.5).astype(np.float32)
    top_p = np.array([0.9, 0.6, 0.9, 0.0, -1.0, 0.7])
    temp = np.array([1.0, 1e8, 1e10, 0.9, 1.1, 0.6])
    u = np.array([0.3, 0.77, 0.52, 0.5, 0.5, 1.0])
    _check_rows(L, logits, top_p, temp, None, u)
    _check_rows(L, logits, top_p, temp, np.array([0, 10, 5, V, V + 7, 1], np.int32), u)
    _check_rows(L, logits[:, :1].copy(), top_p, temp, None, u)          # a vocabulary of one


def test_nucleus_against_the_committed_fixture(L):
    """tests/golden/nucleus_cases.npz: keep-masks and tokens bit for bit."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "nucleus_cases.npz"))
    V = g["logits"].shape[1]
    keep = np.unpackbits(g["keep"], axis=-1)[:, :V].astype(bool)
    for r in range(g["logits"].shape[0]):
        k = None if g["top_k"][r] == 0 else np.array([g["top_k"][r]], np.int32)
        tok, mask, _ = _sample(L, g["logits"][r:r + 1], g["top_p"][r], g["temp"][r], k, g["u"][r])
        assert np.array_equal(mask[0], keep[r]), r
        assert tok[0] == g["token"][r], r
    _, mask, _ = _sample(L, g["demo"], 0.9, 1.0, None, 0.5)
    assert np.array_equal(mask[0], g["demo_keep"])


@pytest.mark.parametrize("M,V,ld", [(1, 12, 12), (37, 50400, 50400), (5, 1000, 1024)])
def test_xent_rows(L, M, V, ld):
    a = abi()
    g = torch.Generator().manual_seed(M + V)
    lg = (torch.randn(M, ld, generator=g) * 3).to(DEV)
    tgt = torch.randint(0, V, (M,), generator=g).to(torch.int32)
    tgt[0] = int(lg[0, :V].argmax())                       # a correct one
    if M > 2:
        tgt[2] = V + 5                                     # outside the vocabulary: selects nothing
    tgt = tgt.to(DEV)
    loss = torch.empty(M, device=DEV)
    correct = torch.empty(M, dtype=torch.uint8, device=DEV)
    a.check(L.mtj_xent(a.ptr(lg), ld, a.ptr(tgt), M, V, a.ptr(loss), a.ptr(correct), S()))
    torch.cuda.synchronize()
    l64 = lg[:, :V].double()
    lse = torch.logsumexp(l64, -1)
    inside = tgt.long() < V
    ref = lse - torch.where(inside, l64.gather(1, tgt.long().clamp(max=V - 1)[:, None])[:, 0], l64.max(-1).values)
    assert rel_err(loss, ref) < 2e-6
    want = (l64.argmax(-1) == tgt.long()) | ~inside         # pred = 0 also when nothing is selected
    assert torch.equal(correct.bool(), want)


@pytest.mark.parametrize("dt,M,V,K", [("f32", 37, 50400, 256), ("bf16", 37, 50400, 512), ("f16", 64, 1000, 256),
                                      ("f32", 200, 1000, 256), ("bf16", 300, 5000, 128), ("f16", 1, 132, 64),
                                      ("bf16", 2048, 50400, 1024), ("f16", 2000, 50400, 512)])
def test_logits_and_cross_entropy_in_one_gemm(L, dt, M, V, K):
    """mtj_gemm_xent against mtj_gemm (STORE) + mtj_xent on the same operands and against float64; the last two shapes
    are 8 x 197 tiles of 256 x 256 (the direct-to-LDS kernel, ragged in both directions), the others the 32-, 64- and
    128-row tiles.  Targets include the row's best column, a column in the ragged last tile and one outside the vocabulary."""
    a = abi()
    g = torch.Generator().manual_seed(M + V + K)
    A = torch.randn(M, K, generator=g).to(TD[dt]).to(DEV)
    Wh = (torch.randn(K, V, generator=g) * 0.2).to(TD[dt]).to(DEV)
    bias = torch.randn(V, generator=g).to(DEV)
    W = _packed(Wh)
    code, alpha = a.dtype_code(TD[dt]), 0.5
    logits = torch.empty(M, V, device=DEV)
    a.check(L.mtj_gemm(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, V, K, code, a.EPI_STORE, a.ptr(logits), V, 0, None, alpha, S()))
    tgt = torch.randint(0, V, (M,), generator=g).to(torch.int32).to(DEV)
    best = logits.argmax(-1).to(torch.int32)
    tgt[::3] = best[::3]
    if M > 4:
        tgt[1] = V - 1
        tgt[4] = V + 5
    loss0, loss1 = torch.empty(M, device=DEV), torch.full((M,), -1.0, device=DEV)
    ok0, ok1 = torch.empty(M, dtype=torch.uint8, device=DEV), torch.full((M,), 7, dtype=torch.uint8, device=DEV)
    a.check(L.mtj_xent(a.ptr(logits), V, a.ptr(tgt), M, V, a.ptr(loss0), a.ptr(ok0), S()))
    nb = L.mtj_gemm_xent_work_bytes(M, V, code)
    assert 0 < nb <= (2 * ((V + 127) // 128) + 1) * M * 4
    work = torch.full((nb // 4,), float("nan"), device=DEV)              # nothing is expected to be there
    a.check(L.mtj_gemm_xent(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, V, K, code, alpha, a.ptr(tgt), a.ptr(loss1), a.ptr(ok1),
                            a.ptr(work), nb, S()))
    torch.cuda.synchronize()
    assert torch.equal(ok1, ok0)
    assert (loss1 - loss0).abs().max().item() < 2e-5 * max(1.0, loss0.abs().max().item())
    l64 = alpha * (A.double() @ Wh.double()) + bias.double()
    inside = tgt.long() < V
    ref = torch.logsumexp(l64, -1) - torch.where(inside, l64.gather(1, tgt.long().clamp(max=V - 1)[:, None])[:, 0],
                                                 l64.max(-1).values)
    assert (loss1.double() - ref).abs().max().item() < 2e-5 * max(1.0, ref.abs().max().item())
    with pytest.raises(ValueError):
        a.check(L.mtj_gemm_xent(a.ptr(A), K, a.ptr(W), a.ptr(bias), M, V, K, code, alpha, a.ptr(tgt), a.ptr(loss1),
                                a.ptr(ok1), a.ptr(work), nb - 4, S()))


@pytest.mark.parametrize("dt,N,K,ln", [("bf16", 50400, 4096, True), ("f32", 1000, 512, False), ("f16", 50400, 1024, True),
                                       ("bf16", 70, 64, False), ("bf16", 4100, 4096, True)])
def test_logits_launch_that_is_its_own_greedy_sampler(L, dt, N, K, ln):
    """mtj_gemv_greedy against mtj_gemv (STORE) followed by mtj_sample_greedy on the same operands: logits, token,
    token buffer, position and next-step embedding bit for bit, over several launches in a row on one work buffer
    (every launch leaves it zeroed), with tied maxima (lowest index wins), a maximum in the last row, -0.0 against
    +0.0 and a NaN among the logits."""
    a = abi()
    g = torch.Generator().manual_seed(N + K)
    code = a.dtype_code(TD[dt])
    W = (torch.randn(N, K, generator=g) * 0.05).to(TD[dt]).to(DEV)
    sc, of = (torch.rand(K, generator=g) + 0.5).to(DEV), (torch.randn(K, generator=g) * 0.1).to(DEV)
    We = (torch.randn(N, 96, generator=g) * 0.02).to(torch.bfloat16).to(DEV)
    be = torch.randn(96, generator=g).to(DEV)
    work = torch.zeros(256, dtype=torch.uint8, device=DEV)
    steps = 6
    out0 = torch.full((1, steps), -1, dtype=torch.int32, device=DEV)
    out1 = out0.clone()
    pos0 = torch.tensor([9], dtype=torch.int32, device=DEV)
    pos1 = pos0.clone()
    pos_start = torch.tensor([9], dtype=torch.int32, device=DEV)
    for t in range(steps):
        x = torch.randn(K, generator=g).to(DEV)
        bias = torch.randn(N, generator=g).to(DEV)
        if t == 1:                                   # two equal maxima far apart, made through the bias of zeroed rows
            W2 = W.clone(); W2[7] = 0; W2[N - 3] = 0
            bias[7] = 50.0; bias[N - 3] = 50.0
        elif t == 2:                                 # the maximum is the very last row
            W2 = W.clone(); W2[N - 1] = 0
            bias[N - 1] = 60.0
        elif t == 3:                                 # all rows zero: +0.0 everywhere but one -0.0; index 0 wins
            W2 = torch.zeros_like(W)
            bias.zero_(); bias[0] = -0.0
        elif t == 4:                                 # a NaN never wins
            W2 = W.clone(); W2[5] = 0
            bias[5] = float("nan")
        else:
            W2 = W
        lnp = (a.ptr(sc), a.ptr(of)) if ln else (None, None)
        lg0, lg1 = torch.empty(1, N, device=DEV), torch.empty(1, N, device=DEV)
        tok0, tok1 = (torch.zeros(1, dtype=torch.int32, device=DEV) for _ in range(2))
        xn0, xn1 = torch.zeros(1, 96, device=DEV), torch.zeros(1, 96, device=DEV)
        ne = a.NextEmbed()
        ne.w, ne.bias, ne.x_next, ne.d, ne.dtype = a.ptr(We), a.ptr(be), a.ptr(xn0), 96, 1
        a.check(L.mtj_gemv(a.ptr(x), lnp[0], lnp[1], a.ptr(W2), a.ptr(bias), N, K, code, a.EPI_STORE, a.ptr(lg0), 0, None, None, S()))
        a.check(L.mtj_sample_greedy(a.ptr(lg0), 1, N, a.ptr(tok0), a.ptr(out0), steps, a.ptr(pos0), a.ptr(pos_start),
                                    C.byref(ne), S()))
        ne.x_next = a.ptr(xn1)
        a.check(L.mtj_gemv_greedy(a.ptr(x), lnp[0], lnp[1], a.ptr(W2), a.ptr(bias), N, K, code, a.ptr(lg1), a.ptr(tok1),
                                  a.ptr(out1), steps, a.ptr(pos1), a.ptr(pos_start), C.byref(ne), a.ptr(work), S()))
        torch.cuda.synchronize()
        assert torch.equal(lg0.view(torch.int32), lg1.view(torch.int32)), t
        assert tok0.item() == tok1.item(), (t, tok0.item(), tok1.item())
        assert torch.equal(xn0, xn1) and torch.equal(pos0, pos1), t
        assert int(work.view(torch.int64).abs().sum()) == 0, t            # ready for the next launch
        if t == 1:
            assert tok1.item() == 7
        if t == 2:
            assert tok1.item() == N - 1
        if t == 3:
            assert tok1.item() == 0
    assert torch.equal(out0, out1) and (out1 >= 0).all()
    with pytest.raises(ValueError):
        a.check(L.mtj_gemv_greedy(a.ptr(x), None, None, a.ptr(W), a.ptr(bias), N, K, code, a.ptr(lg1), a.ptr(tok1), None, 0,
                                  a.ptr(pos1), a.ptr(pos_start), None, None, S()))


def test_greedy_lowest_index_on_ties(L):
    a = abi()
    V = 50400
    lg = torch.zeros(3, V, device=DEV)
    lg[0, 777] = 2.0
    lg[0, 40000] = 2.0
    lg[1, V - 1] = 1.0
    tok = torch.zeros(3, dtype=torch.int32, device=DEV)
    pos = torch.tensor([4, 5, 6], dtype=torch.int32, device=DEV)
    pos_start = torch.tensor([4, 4, 4], dtype=torch.int32, device=DEV)
    out = torch.full((3, 4), -1, dtype=torch.int32, device=DEV)
    W = (torch.randn(V, 96) * 0.02).to(torch.bfloat16).to(DEV)
    bias = torch.randn(96).to(DEV)
    xn = torch.zeros(3, 96, device=DEV)
    ne = a.NextEmbed()
    ne.w, ne.bias, ne.x_next, ne.d, ne.dtype = a.ptr(W), a.ptr(bias), a.ptr(xn), 96, 1
    a.check(L.mtj_sample_greedy(a.ptr(lg), 3, V, a.ptr(tok), a.ptr(out), 4, a.ptr(pos), a.ptr(pos_start), C.byref(ne), S()))
    torch.cuda.synchronize()
    assert tok.tolist() == [777, V - 1, 0]
    assert out.tolist() == [[777, -1, -1, -1], [-1, V - 1, -1, -1], [-1, -1, 0, -1]]
    assert pos.tolist() == [5, 6, 7]
    assert torch.equal(xn, W[tok.long()].float() + bias)      # the chosen token's embedding, for the next step

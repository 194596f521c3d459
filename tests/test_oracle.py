"""Pins for the CPU oracle: every check here is against something other than the oracle's own
formula (a library routine, a brute-force loop, an invariant, the reference's demo vector, or the
independent GPT-J implementation in `transformers` built from a local config object)."""
import itertools
import math

import os
import sys

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import gptj_oracle as O

TINY = dict(layers=2, d_model=64, n_heads=4, n_vocab=96, norm="layernorm", pe="rotary", pe_rotary_dims=8,
            seq=32, cores_per_replica=1)
SIXB = dict(layers=28, d_model=4096, n_heads=16, n_vocab=50400, norm="layernorm", pe="rotary",
            pe_rotary_dims=64, seq=2048, cores_per_replica=1)


def rnd(*shape, seed=0):
    return torch.from_numpy(np.random.default_rng(seed).standard_normal(shape))


def test_param_count_matches_published():
    # README.md:77 prints 6,053,381,344 with the replicated leaves counted 8 times
    unique = O.count_params(SIXB)
    assert unique == 6_050_886_880
    d = 4096
    replicated = 28 * (2 * d + d) + d + 2 * d      # LN scale/offset + fc_out bias per layer; embed bias; final LN
    assert unique + 7 * replicated == 6_053_381_344


def test_layer_norm_is_library_layer_norm():
    x, s, o = rnd(5, 64), rnd(64, seed=1), rnd(64, seed=2)
    got = O.replicated_layer_norm(x, s, o)
    ref = F.layer_norm(x, (64,), s, o, eps=1e-5)
    assert torch.allclose(got, ref, rtol=1e-12, atol=1e-12)
    const = torch.full((1, 64), 3.25, dtype=torch.float64)
    assert torch.equal(O.replicated_layer_norm(const, s, o), o.expand(1, 64))
    y = O.replicated_layer_norm(x, torch.ones(64, dtype=torch.float64), torch.zeros(64, dtype=torch.float64))
    assert torch.allclose(y.mean(-1), torch.zeros(5, dtype=torch.float64), atol=1e-12)
    assert torch.allclose((y ** 2).mean(-1), torch.ones(5, dtype=torch.float64), atol=1e-4)


def test_embedding_is_onehot_matmul():
    w, b = rnd(96, 64), rnd(64, seed=3)
    tok = torch.tensor([0, 5, 95, 5])
    onehot = F.one_hot(tok, 96).to(torch.float64)
    assert torch.equal(O.embedding_shard(tok, w, b), onehot @ w + b)


def test_rotary_closed_form_and_invariants():
    T, H, r = 7, 3, 8
    x = rnd(T, H, r, seed=4)
    sincos = O.fixed_pos_embedding(T, r)
    y = O.apply_rotary_pos_emb(x, sincos)
    # brute force: a 2x2 rotation per adjacent pair, angle pos * 10000^(-2i/r)
    for t, h, i in itertools.product(range(T), range(H), range(r // 2)):
        th = t * 10000.0 ** (-2 * i / r)
        a, b = x[t, h, 2 * i].item(), x[t, h, 2 * i + 1].item()
        assert abs(y[t, h, 2 * i].item() - (a * math.cos(th) - b * math.sin(th))) < 1e-12
        assert abs(y[t, h, 2 * i + 1].item() - (b * math.cos(th) + a * math.sin(th))) < 1e-12
    assert torch.allclose(y[0], x[0])                                            # position 0 is the identity
    assert torch.allclose(y.reshape(T, H, -1, 2).norm(dim=-1), x.reshape(T, H, -1, 2).norm(dim=-1))
    # q uses the LAST q.shape[0] rows of the table (layers.py:147)
    q1 = O.apply_rotary_pos_emb(x[-1:], sincos)
    assert torch.allclose(q1[0], y[-1])
    # shift invariance of rotated dot products
    big = O.fixed_pos_embedding(T + 5, r)
    k = rnd(T, H, r, seed=5)
    s0 = torch.einsum("thd,Thd->htT", y, O.apply_rotary_pos_emb(k, sincos))
    s5 = torch.einsum("thd,Thd->htT", O.apply_rotary_pos_emb(x, big), O.apply_rotary_pos_emb(k, big))
    assert torch.allclose(s0, s5, atol=1e-12)


def test_rotary_matches_transformers_gptj():
    m = pytest.importorskip("transformers.models.gptj.modeling_gptj")
    T, H, r = 9, 2, 16
    x = rnd(T, H, r, seed=6).float()
    tab = m.create_sinusoidal_positions(T, r)
    sin, cos = tab[:, : r // 2][None], tab[:, r // 2:][None]
    ref = m.apply_rotary_pos_emb(x[None], sin, cos)[0]
    got = O.apply_rotary_pos_emb(x, O.fixed_pos_embedding(T, r))
    assert torch.allclose(got, ref, atol=1e-5)


def test_gelu_is_tanh_approximation():
    x = torch.linspace(-6, 6, 1001, dtype=torch.float64)
    assert torch.allclose(O.gelu_tanh(x), F.gelu(x, approximate="tanh"), atol=1e-14)


def _tiny_model(dtype=torch.float64, cfg=TINY, seed=0):
    p = O.seeded_params(cfg, seed)
    # exercise LN scale/offset too
    g = np.random.default_rng(7)
    for mod in p:
        if "scale" in p[mod]:
            p[mod]["scale"] = torch.from_numpy(1 + 0.1 * g.standard_normal(p[mod]["scale"].shape)).float()
            p[mod]["offset"] = torch.from_numpy(0.1 * g.standard_normal(p[mod]["offset"].shape)).float()
    return O.Model(cfg, p, dtype), p


def test_self_attn_brute_force_and_sdpa():
    model, _ = _tiny_model()
    l = model.layers[0]
    T = 6
    q, v, k = rnd(T, l.H, l.dh, seed=8), rnd(T, l.H, l.dh, seed=9), rnd(T, l.H, l.dh, seed=10)
    bias = O.MASK * (1.0 - torch.tril(torch.ones(T, T, dtype=torch.float64)))
    got = l.self_attn(q, v, k, bias)
    sc = O.fixed_pos_embedding(T, l.r)
    qr = torch.cat([O.apply_rotary_pos_emb(q[:, :, :l.r], sc), q[:, :, l.r:]], -1)
    kr = torch.cat([O.apply_rotary_pos_emb(k[:, :, :l.r], sc), k[:, :, l.r:]], -1)
    # brute force
    out = torch.zeros(T, l.H, l.dh, dtype=torch.float64)
    for h in range(l.H):
        for t in range(T):
            s = torch.tensor([(qr[t, h] @ kr[j, h]).item() / math.sqrt(l.dh) for j in range(t + 1)], dtype=torch.float64)
            w = torch.exp(s - s.max())
            w = w / w.sum()
            out[t, h] = sum(w[j] * v[j, h] for j in range(t + 1))
    assert torch.allclose(got, out.reshape(T, -1) @ l.wo, atol=1e-11)
    # library routine
    sd = F.scaled_dot_product_attention(qr.permute(1, 0, 2)[None], kr.permute(1, 0, 2)[None], v.permute(1, 0, 2)[None],
                                        is_causal=True)[0].permute(1, 0, 2).reshape(T, -1)
    assert torch.allclose(got, sd @ l.wo, atol=1e-10)


def test_left_pad_invariance():
    model, _ = _tiny_model()
    toks = np.array([5, 17, 3, 90, 41, 8, 77], np.uint32)
    outs = []
    for pad, fill in ((0, 0), (3, 0), (9, 13)):
        ctx = np.concatenate([np.full(pad, fill, np.uint32), toks])
        taps = []
        model.generate_initial(ctx, len(toks), taps)
        outs.append(taps[-1][pad:])
    assert torch.allclose(outs[0], outs[1], atol=1e-10) and torch.allclose(outs[0], outs[2], atol=1e-10)


def _hf_from_tree(cfg, p):
    """Build transformers' GPT-J from a LOCAL config and load the tree through the name map
    in to_hf_weights.py:160-173 (all Linear weights transposed; wte.weight = W_e + b_e, :386-397)."""
    tr = pytest.importorskip("transformers")
    hc = tr.GPTJConfig(vocab_size=cfg["n_vocab"], n_positions=512, n_embd=cfg["d_model"], n_layer=cfg["layers"],
                       n_head=cfg["n_heads"], rotary_dim=cfg["pe_rotary_dims"], activation_function="gelu_new",
                       layer_norm_epsilon=1e-5, resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0,
                       tie_word_embeddings=False)
    hf = tr.GPTJForCausalLM(hc).double().eval()
    sd = {}
    f = lambda t: t[0].double()
    sd["transformer.wte.weight"] = f(p[O.EMBED]["w"]) + f(p[O.EMBED]["b"])
    names = {"linear": "attn.q_proj", "linear_1": "attn.v_proj", "linear_2": "attn.k_proj", "linear_3": "attn.out_proj",
             "linear_4": "mlp.fc_in", "linear_5": "mlp.fc_out"}
    for i in range(cfg["layers"]):
        for hk_name, hf_name in names.items():
            m = p[O.layer_key(i, hk_name)]
            sd[f"transformer.h.{i}.{hf_name}.weight"] = f(m["w"]).T.contiguous()
            if "b" in m:
                sd[f"transformer.h.{i}.{hf_name}.bias"] = f(m["b"])
        ln = p[O.layer_key(i, "replicated_layer_norm")]
        sd[f"transformer.h.{i}.ln_1.weight"], sd[f"transformer.h.{i}.ln_1.bias"] = f(ln["scale"]), f(ln["offset"])
    sd["transformer.ln_f.weight"], sd["transformer.ln_f.bias"] = f(p[O.PROJ_LN]["scale"]), f(p[O.PROJ_LN]["offset"])
    sd["lm_head.weight"], sd["lm_head.bias"] = f(p[O.PROJ]["w"]).T.contiguous(), f(p[O.PROJ]["b"])
    missing, unexpected = hf.load_state_dict(sd, strict=False)
    assert not unexpected and all("embed_positions" in k or "masked_bias" in k or k.endswith("attn.bias") for k in missing), (missing, unexpected)
    return hf


def test_forward_matches_transformers_gptj():
    model, p = _tiny_model()
    hf = _hf_from_tree(TINY, p)
    toks = O.seeded_prompt(0, 1, 21, hi=TINY["n_vocab"])[0]
    got = model.forward(toks)
    with torch.no_grad():
        ref = hf(torch.from_numpy(toks.astype(np.int64))[None]).logits[0]
    assert torch.allclose(got, ref, atol=1e-9), (got - ref).abs().max()


def test_decode_is_teacher_forcing_of_forward():
    """With P + G <= L only padding is evicted: step-t logits equal the last-position logits of
    a full forward over prompt + generated[:t]."""
    model, _ = _tiny_model()
    prompt = O.seeded_prompt(1, 1, 6, hi=TINY["n_vocab"])
    G, L = 5, 16
    toks, _, logits = model.generate(O.left_pad(prompt, L), [6], G, O.greedy_sample, {}, return_logits=True)
    seq = list(prompt[0])
    for t in range(G):
        full = model.forward(np.array(seq, np.uint32))[-1].float().numpy()
        assert np.allclose(logits[0, t, 0], full, atol=1e-5)
        assert toks[0, t, 0] == int(np.argmax(full))
        seq.append(int(toks[0, t, 0]))


def test_sliding_window_evicts_oldest_real_tokens():
    """L == P (no padding): every decode step drops the oldest real token; the logits equal a
    forward pass whose layer-wise attention sees only the last T keys.  Checked on a 1-layer model,
    where windowed attention is the same as a forward over the last T tokens."""
    cfg = dict(TINY, layers=1)
    model, _ = _tiny_model(cfg=cfg)
    prompt = O.seeded_prompt(2, 1, 9, hi=cfg["n_vocab"])
    G = 4
    toks, _, logits = model.generate(prompt, [9], G, O.greedy_sample, {}, return_logits=True)
    seq = list(prompt[0])
    T = 8
    for t in range(G):
        # one layer: K/V of a token do not depend on other tokens, RoPE depends on offsets only
        full = model.forward(np.array(seq[-T:], np.uint32))[-1].float().numpy()
        assert np.allclose(logits[0, t, 0], full, atol=1e-5)
        seq.append(int(toks[0, t, 0]))


# ------------------------------------------------------------------ sampling
DEMO = np.array([[-2, -1, 0, 0.8, 0, 0.1, 0.3, 0.4, 0.5, 0.6, 0.7, -3]], np.float32)   # sampling.py:49


def test_nucleus_demo_vector_known_answer():
    f = O.nucleaus_filter(DEMO, top_p=0.9)
    removed = set(np.nonzero(f[0] != DEMO[0])[0].tolist())
    assert removed == {0, 1, 11}
    assert np.all(f[0][[0, 1, 11]] < -9e9)
    order = O.descending_order(DEMO[0]).tolist()
    assert order == [3, 10, 9, 8, 7, 6, 5, 4, 2, 1, 0, 11]      # ties (ids 2 and 4): higher id first
    # f32 accumulation gives the same answer on this vector
    assert np.array_equal(O.nucleaus_filter(DEMO, 0.9, acc=np.float32), f)


def test_nucleus_brute_force_prefix():
    rng = np.random.default_rng(11)
    for trial in range(200):
        V = int(rng.integers(2, 9))
        l = rng.standard_normal((1, V)).astype(np.float32)
        if trial % 3 == 0:
            l[0, rng.integers(0, V)] = l[0, rng.integers(0, V)]          # force ties
        top_p = float(rng.uniform(0.05, 1.0))
        keep = O.keep_mask(l, top_p)[0]
        p = np.exp(l[0].astype(np.float64) - l[0].max())
        p /= p.sum()
        # order: descending value, ties by higher id
        order = sorted(range(V), key=lambda i: (-l[0, i], -i))
        # shortest prefix whose mass exceeds top_p (crossing token included); everything if none does
        n, mass = V, 0.0
        for j, i in enumerate(order):
            mass += p[i]
            if mass > top_p:
                n = j + 1
                break
        assert set(np.nonzero(keep)[0].tolist()) == set(order[:n]), (l, top_p)
        assert keep[order[0]]                      # a maximal token always survives


def test_top_k_quirk_token_zero_is_never_removed():
    l = np.array([[0.1, 3.0, 2.0, 1.0, 0.5]], np.float32)
    f = O.nucleaus_filter(l, top_p=1.0, top_k=2)
    assert f[0, 0] == l[0, 0]                      # rank 4 >= k but 1e10 * token_id == 0
    assert f[0, 1] == l[0, 1] and f[0, 2] == l[0, 2]
    assert f[0, 3] == np.float32(1.0) - np.float32(1e10) * np.float32(3) and f[0, 4] < -3e10


def test_filter_runs_before_temperature():
    # a row where filtering the tempered logits would give a different keep-set
    l = np.array([[2.0, 1.0, 0.0, -1.0]], np.float32)
    raw = O.keep_mask(l, 0.9)[0]
    tempered = O.keep_mask(l / np.float32(0.3), 0.9)[0]
    assert raw.sum() != tempered.sum()
    hits = {O.nucleaus_sample(u, l, top_p=0.9, temp=0.3) for u in np.linspace(0, 0.999999, 4001)}
    assert hits == set(np.nonzero(raw)[0].tolist())


def test_inverse_cdf_draw_brute_force_and_chi_square():
    rng = np.random.default_rng(12)
    l = rng.standard_normal((1, 7)).astype(np.float32) * 2
    f = O.nucleaus_filter(l, 0.8)
    temp = 0.7
    order = sorted(range(7), key=lambda i: (-l[0, i], -i))
    w = np.array([math.exp(float(f[0, i]) / temp - float(f[0].max()) / temp) for i in order])
    for u in rng.random(300):
        acc, want = 0.0, None
        for j, i in enumerate(order):
            acc += w[j]
            if acc > u * w.sum():
                want = i
                break
        assert O.inverse_cdf_draw(l, f, temp, u) == want
    n = 40000
    counts = np.bincount([O.inverse_cdf_draw(l, f, temp, u) for u in rng.random(n)], minlength=7)
    p = np.zeros(7)
    p[order] = w / w.sum()
    nz = p > 0
    assert counts[~nz].sum() == 0
    chi2 = ((counts[nz] - n * p[nz]) ** 2 / (n * p[nz])).sum()
    assert chi2 < 30, chi2       # dof <= 6; P(chi2 > 30) ~ 4e-5


def test_softmax_sample_follows_the_library_softmax():
    """softmax_sample (sampling.py:6-7): the empirical distribution of the draw is torch.softmax(logits / temp)."""
    rng = np.random.default_rng(5)
    l = rng.standard_normal((1, 6)).astype(np.float32) * 1.5
    temp, n = 1.3, 40000
    p = torch.softmax(torch.from_numpy(l[0]).double() / temp, -1).numpy()
    counts = np.bincount([O.softmax_sample(u, l, temp=temp) for u in rng.random(n)], minlength=6)
    chi2 = ((counts - n * p) ** 2 / (n * p)).sum()
    assert chi2 < 28, chi2       # dof 5; P(chi2 > 28) ~ 4e-5


def test_greedy_lowest_index_on_ties():
    assert O.greedy_sample(None, np.array([[1.0, 3.0, 3.0, 2.0]], np.float32)) == 1


def test_loss_is_cross_entropy_and_the_evaluation_mask_hides_keys():
    cfg = dict(layers=2, d_model=64, n_heads=4, n_vocab=96, norm="layernorm", pe="rotary", pe_rotary_dims=8,
               cores_per_replica=1)
    params = O.seeded_params(cfg, 11)
    m = O.Model(cfg, params, torch.float64)
    rng = np.random.default_rng(0)
    ctx, tgt = rng.integers(0, 96, 24), rng.integers(0, 96, 24)
    out = m.loss(ctx, tgt)
    logits = m.forward(ctx)
    ce = F.cross_entropy(logits, torch.as_tensor(tgt), reduction="none")
    assert torch.allclose(out["all_loss"], ce, atol=1e-12)
    assert torch.equal(out["correct"], logits.argmax(-1) == torch.as_tensor(tgt))
    assert abs(float(out["loss"]) - float(ce.mean())) < 1e-12 and float(out["last_loss"]) == float(out["all_loss"][-1])
    # ctx_length = 15: rows 0..15 are what they were; keys 16.. are hidden, so tokens 16..22 cannot reach row 23
    cut = m.loss(ctx, tgt, 15)
    assert torch.allclose(cut["all_loss"][:16], out["all_loss"][:16], atol=1e-12)
    assert not torch.allclose(cut["all_loss"][16:], out["all_loss"][16:], atol=1e-6)
    ctx2 = ctx.copy()
    ctx2[16:23] = rng.integers(0, 96, 7)
    cut2 = m.loss(ctx2, tgt, 15)
    assert abs(float(cut2["all_loss"][23]) - float(cut["all_loss"][23])) < 1e-12
    assert abs(float(m.loss(ctx2, tgt)["all_loss"][23]) - float(out["all_loss"][23])) > 1e-9


# ---------------------------------------------------------------------------- committed fixtures
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_golden_fixtures_match_the_oracle():
    """tests/golden/*.npz (written by tests/golden/make_golden.py) are what the oracle computes today."""
    sys.path.insert(0, GOLDEN)
    import make_golden as G
    for name, fn in (("config1_greedy.npz", G.config1), ("nucleus_cases.npz", G.nucleus)):
        want = np.load(os.path.join(GOLDEN, name))
        got = fn()
        assert sorted(want.files) == sorted(got)
        for k in want.files:
            if want[k].dtype.kind == "f":
                np.testing.assert_allclose(got[k], want[k], rtol=1e-9, atol=1e-12, err_msg=f"{name}:{k}")
            else:
                assert np.array_equal(got[k], want[k]), f"{name}:{k}"
    demo = np.load(os.path.join(GOLDEN, "nucleus_cases.npz"))
    assert set(np.nonzero(~demo["demo_keep"])[0].tolist()) == {0, 1, 11}      # hand-worked, sampling.py:49

"""Model-level parity on a real MI355X: CausalTransformer.generate and the layer wrappers against the CPU
oracle (float64 arithmetic on the same - possibly bf16-rounded - weights), on seeded inputs."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import gptj_oracle as O

DEV = "cuda:0"

# BASELINE config 1: tiny fp32 stack
CFG1 = dict(layers=2, d_model=512, n_heads=8, n_vocab=50400, norm="layernorm", pe="rotary", pe_rotary_dims=32,
            seq=168, cores_per_replica=1)
# reduced full-head-shape stack for the bf16 path (d_head 256, rotary 64 like the 6B model)
CFG_BF = dict(layers=4, d_model=1024, n_heads=4, n_vocab=50400, norm="layernorm", pe="rotary", pe_rotary_dims=64,
              seq=128, cores_per_replica=1)


def rel(got, ref):
    got = torch.as_tensor(np.asarray(got.cpu() if isinstance(got, torch.Tensor) else got)).double()
    ref = torch.as_tensor(np.asarray(ref)).double()
    return float((got - ref).norm() / ref.norm())


def net_for(cfg, params, sampler):
    from mesh_transformer.transformer_shard import CausalTransformer
    c = dict(cfg, sampler=sampler)
    return CausalTransformer(c, params)


def test_config1_layers_fp32_within_1e4_relative():
    """Per-layer bound of the float32 path: prefill (left-padded) and one decode step of every layer."""
    from mesh_transformer import layers
    from mesh_transformer.layers import TransformerLayerShard, EmbeddingShard, ProjectionShard, ReplicatedLayerNorm
    params = O.seeded_params(CFG1, 0)
    scope = layers.transform(params)          # the modules take their parameters from the enclosing scope, like haiku's
    scope.__enter__()
    model = O.Model(CFG1, params, torch.float64)
    prompt = O.seeded_prompt(0, 1, 128)
    ctx = O.left_pad(prompt, 168)[0]
    T, given = 167, 127
    x_ref = model.embed(ctx[:-1])
    emb = EmbeddingShard(CFG1)(ctx[:-1])
    assert rel(emb, x_ref) < 1e-6
    x_new_ref = model.embed(ctx[-1:])
    for i, lref in enumerate(model.layers):
        layer = TransformerLayerShard(CFG1, f"layer_{i}", 2.0 / CFG1["layers"])     # transformer_shard.py:35-37
        d_ref, st_ref = lref.get_init_decode_state(x_ref, given, 0.0)
        d_got, st = layer.get_init_decode_state(x_ref.float(), given, 0)
        pad = T - given
        e = rel(d_got[pad:], d_ref[pad:])
        print(f"layer {i} prefill delta rel err {e:.3e}")
        assert e < 1e-4
        # unpadded forward through __call__
        d2_ref = lref(x_ref[pad:], 0.0)
        assert rel(layer(x_ref[pad:].float(), 0), d2_ref) < 1e-4
        # one decode step on top of the prefilled state
        d_got, st = layer.get_init_decode_state(x_ref.float(), given, 0)
        dd_ref, _ = lref.decode_once(st_ref, x_new_ref, 0.0)
        dd_got, st2 = layer.decode_once(st, x_new_ref.float(), 0)
        e = rel(dd_got, dd_ref)
        print(f"layer {i} decode delta rel err {e:.3e}")
        assert e < 1e-4 and st2["tokens_decoded"] == given + 1
        x_ref = x_ref + d_ref
        x_new_ref = x_new_ref + dd_ref
    lg = ProjectionShard(CFG1)(x_new_ref.float())
    assert rel(lg, model.proj(x_new_ref)) < 1e-4
    ln = ReplicatedLayerNorm()(x_new_ref.float())
    assert rel(ln, O.replicated_layer_norm(x_new_ref, model.pln_s, model.pln_o)) < 1e-5
    ln = ReplicatedLayerNorm(params=params[O.PROJ_LN])(x_new_ref.float())
    assert rel(ln, O.replicated_layer_norm(x_new_ref, model.pln_s, model.pln_o)) < 1e-5
    scope.__exit__(None, None, None)
    with pytest.raises(RuntimeError):
        EmbeddingShard(CFG1)                  # no parameters in scope


def test_config1_generate_fp32_greedy_stream():
    """BASELINE config 1: 128-token prompt (left-padded so that P + G <= L), 32 greedy steps."""
    from mesh_transformer import sampling
    params = O.seeded_params(CFG1, 0)
    prompt = O.seeded_prompt(0, 1, 128)
    ctx = O.left_pad(prompt, 168)
    net = net_for(CFG1, params, sampling.greedy_sample)
    _, out = net.generate(ctx, [128], 32, {}, return_logits=True)
    ref_t, _, ref_l = O.Model(CFG1, params, torch.float64).generate(ctx, [128], 32, O.greedy_sample, {}, return_logits=True)
    err = np.abs(out[2] - ref_l).max()
    print("config1: max |dlogit|", err, "rel", rel(out[2], ref_l))
    assert out[0].shape == (1, 32, 1) and out[0].dtype == np.uint32 and out[1] is None
    assert np.array_equal(out[0], ref_t)
    assert rel(out[2], ref_l) < 1e-4
    # the graph-replayed path (no logits returned) must give the same stream
    _, out2 = net.generate(ctx, [128], 32, {})
    assert np.array_equal(out2[0], ref_t)
    # and so must a second call on the warm session
    _, out3 = net.generate(ctx, [128], 32, {})
    assert np.array_equal(out3[0], ref_t)


def test_bf16_logits_and_greedy_stream():
    """bf16 weights: |dlogit| <= 2e-2 and identical greedy tokens over the first 32 steps (north-star tolerance)."""
    from mesh_transformer import sampling
    params = O.seeded_params(CFG_BF, 1, torch.bfloat16)
    prompt = O.seeded_prompt(1, 1, 64)
    ctx = O.left_pad(prompt, 128)
    net = net_for(CFG_BF, params, sampling.greedy_sample)
    _, out = net.generate(ctx, [64], 32, {}, return_logits=True)
    ref_t, _, ref_l = O.Model(CFG_BF, params, torch.float64).generate(ctx, [64], 32, O.greedy_sample, {}, return_logits=True)
    err = np.abs(out[2] - ref_l).max(axis=-1)[0, :, 0]
    srt = np.sort(ref_l[0, :, 0, :], axis=-1)
    margin = srt[:, -1] - srt[:, -2]
    print("bf16: max |dlogit| per step", np.round(err, 4).tolist())
    print("bf16: oracle top-1/top-2 margin per step", np.round(margin, 4).tolist())
    assert err.max() < 2e-2
    same = out[0][0, :, 0] == ref_t[0, :, 0]
    first_diff = int(np.argmin(same)) if not same.all() else -1
    assert same.all(), f"streams diverge at step {first_diff} (margin there {margin[first_diff]:.4g}, |dlogit| {err[first_diff]:.4g})"
    _, out2 = net.generate(ctx, [64], 32, {})
    assert np.array_equal(out2[0], out[0])


def test_batched_ragged_nucleus_bit_exact_given_logits():
    """B = 3 (MFMA decode path), different prompt lengths, top-p / temperature per row.  The sampled token and the
    keep-mask must equal the oracle's on the SAME logits and uniforms; the whole stream must also equal the
    oracle's own float64 run."""
    from mesh_transformer import sampling
    cfg = dict(CFG1, n_vocab=2048)
    params = O.seeded_params(cfg, 2)
    lens = [9, 30, 17]
    L, G = 48, 12
    ctx = np.zeros((3, L), np.uint32)
    for b, n in enumerate(lens):
        ctx[b, L - n:] = O.seeded_prompt(10 + b, 1, n, hi=2048)[0]
    opts = {"top_p": np.array([0.9, 0.6, 0.95]), "temp": np.array([0.8, 1.0, 1.3])}
    u = np.random.Generator(np.random.Philox(3)).random((3, G))
    net = net_for(cfg, params, sampling.nucleaus_sample)
    _, out = net.generate(ctx, lens, G, opts, return_logits=True, uniforms=u, return_keep_mask=True)
    toks, logits, masks = out[0], out[2], out[3]
    for b in range(3):
        for t in range(G):
            lg = logits[b, t]
            f = O.nucleaus_filter(lg, opts["top_p"][b])
            assert np.array_equal(masks[b, t], f[0] == lg[0])
            assert toks[b, t, 0] == O.inverse_cdf_draw(lg, f, opts["temp"][b], u[b, t]), (b, t)
    ref = O.Model(cfg, params, torch.float64).generate(ctx, lens, G, O.nucleaus_sample, opts, uniforms=u)
    assert np.array_equal(toks, ref[0])
    # graph-replayed run gives the same stream
    _, out2 = net.generate(ctx, lens, G, opts, uniforms=u)
    assert np.array_equal(out2[0], toks)


def test_forward_logits_every_position():
    """CausalTransformer.forward (embed -> layers -> projection at every position) against the oracle's full
    forward: fp32 within 1e-4 relative; left padding leaves the real rows unchanged and zeroes the padded ones;
    bf16 within the 2e-2 logit tolerance."""
    from mesh_transformer import sampling
    params = O.seeded_params(CFG1, 0)
    toks = O.seeded_prompt(5, 2, 70)
    net = net_for(CFG1, params, sampling.greedy_sample)
    got = net.forward(toks)
    assert got.shape == (2, 70, CFG1["n_vocab"]) and got.dtype == torch.float32
    m = O.Model(CFG1, params, torch.float64)
    for b in range(2):
        assert rel(got[b], m.forward(toks[b])) < 1e-4
    # ragged: sequence 1 keeps only its last 33 tokens, left-padded
    ctx = toks.copy()
    ctx[1, :37] = 0
    got2 = net.forward(ctx, [70, 33])
    assert rel(got2[0], m.forward(toks[0])) < 1e-4
    assert rel(got2[1, 37:], m.forward(toks[1, 37:])) < 1e-4
    assert float(got2[1, :37].abs().max()) == 0.0
    # bf16 weights, d_head 256
    pb = O.seeded_params(CFG_BF, 1, torch.bfloat16)
    tb = O.seeded_prompt(6, 1, 96)
    gb = net_for(CFG_BF, pb, sampling.greedy_sample).forward(tb)
    refb = O.Model(CFG_BF, pb, torch.float64).forward(tb[0])
    assert float((gb[0].double().cpu() - refb).abs().max()) < 2e-2
    with pytest.raises(ValueError):
        net.forward(toks, [70, 71])


def test_config1_against_the_committed_fixture():
    """BASELINE config 1 against tests/golden/config1_greedy.npz: tokens identical, top-8 logits of every step
    within 1e-4 relative, logit checksums."""
    import os
    from mesh_transformer import sampling
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config1_greedy.npz"))
    net = net_for(CFG1, O.seeded_params(CFG1, 0), sampling.greedy_sample)
    ctx = O.left_pad(g["prompt"], 168)
    _, out = net.generate(ctx, [128], 32, {}, return_logits=True)
    assert np.array_equal(out[0][0, :, 0], g["tokens"])
    lg = out[2][0, :, 0, :].astype(np.float64)
    got_top = np.take_along_axis(lg, g["top8_ids"].astype(np.int64), -1)
    assert np.abs(got_top - g["top8_logits"]).max() <= 1e-4 * np.abs(g["top8_logits"]).max()
    np.testing.assert_allclose(lg.sum(-1), g["logits_sum"], rtol=0, atol=1e-4 * np.sqrt(g["logits_sqsum"]).max())
    np.testing.assert_allclose((lg ** 2).sum(-1), g["logits_sqsum"], rtol=2e-4)


def test_eval_losses_match_the_oracle():
    """CausalTransformer.eval: per-token cross entropy, `correct`, and the evaluation mask of ragged batches."""
    from mesh_transformer import sampling
    params = O.seeded_params(CFG1, 9)
    net = net_for(CFG1, params, sampling.greedy_sample)
    rng = np.random.default_rng(1)
    obs = rng.integers(0, 50257, (3, 40)).astype(np.uint32)
    tgt = np.roll(obs, -1, axis=1)
    lens = np.array([40, 17, 1])
    out = net.eval({"obs": obs, "target": tgt, "ctx_length": lens})
    m = O.Model(CFG1, params, torch.float64)
    for b in range(3):
        ref = m.loss(obs[b], tgt[b], lens[b])
        assert rel(out["all_loss"][b], ref["all_loss"]) < 1e-4, b
        assert abs(out["loss"][b] - float(ref["loss"])) < 1e-4 * float(ref["loss"])
        assert abs(out["last_loss"][b] - float(ref["last_loss"])) < 1e-3
        assert np.array_equal(out["correct"][b], ref["correct"].numpy())
    full = net.eval({"obs": obs[:1], "target": tgt[:1]})
    assert rel(full["all_loss"][0], m.loss(obs[0], tgt[0])["all_loss"]) < 1e-4
    with pytest.raises(ValueError):
        net.eval({"obs": obs, "target": tgt[:, :5]})


def test_batching_loop_on_the_gpu():
    """device_serve.py:138-194 around the real network: two requests in a batch of four; with top_p -> 0 the nucleus
    is the top token alone, so the completions equal the oracle's greedy streams."""
    from mesh_transformer import sampling, serving
    cfg = dict(CFG1, n_vocab=2048, seq=40)
    params = O.seeded_params(cfg, 12)
    net = net_for(cfg, params, sampling.nucleaus_sample)
    loop = serving.BatchingLoop(net, seq=40, total_batch=4, gen_length=6)
    prompts = [O.seeded_prompt(20, 1, 9, hi=2048)[0], O.seeded_prompt(21, 1, 23, hi=2048)[0]]
    qs = [loop.submit(p.tolist(), 1e-9, 1.0) for p in prompts]
    assert loop.step() == 2
    m = O.Model(cfg, params, torch.float64)
    for p, q in zip(prompts, qs):
        ref = m.generate(O.left_pad(p[None], 40), [len(p)], 6, O.greedy_sample, {})
        assert np.array_equal(q.get_nowait(), ref[0][0, :, 0])


def test_infer_on_the_gpu_against_the_oracle():
    """The single-prompt caller of resharding_example.py:55-75 / device_sample.py:86-103 (pad to seq, generate with
    top_p / temp / top_k, index output[1][0][0, :, 0]) through the real network.  With top_p -> 0 the nucleus is the
    top token alone (top_k = 5 on top of it changes nothing: the reference's top-k spares token 0, sampling.py:15-26,
    but top_p removes it), so with the uniforms drawn inside generate the completion is the oracle's nucleus run on
    ANY uniforms; a prompt longer than seq keeps its last seq tokens."""
    from mesh_transformer import sampling, serving
    cfg = dict(CFG1, n_vocab=2048, seq=48)
    params = O.seeded_params(cfg, 13)
    net = net_for(cfg, params, sampling.nucleaus_sample)
    m = O.Model(cfg, params, torch.float64)
    for n in (17, 60):
        prompt = O.seeded_prompt(40 + n, 1, n, hi=2048)[0]
        got = serving.infer(net, prompt.tolist(), gen_len=7, top_p=1e-9, temp=0.7, top_k=5)
        kept = prompt[-48:]
        ctx = O.left_pad(kept[None], 48)
        opts = {"top_p": np.array([1e-9]), "temp": np.array([0.7]), "top_k": np.array([5])}
        ref = m.generate(ctx, [len(kept)], 7, O.nucleaus_sample, opts, uniforms=np.full((1, 7), 0.37))
        ref2 = m.generate(ctx, [len(kept)], 7, O.nucleaus_sample, opts, uniforms=np.full((1, 7), 0.93))
        assert np.array_equal(ref[0], ref2[0])                       # the draw has one reachable token
        assert got.dtype == np.uint32 and np.array_equal(got, ref[0][0, :, 0]), n
    text = serving.infer(net, [5, 6, 7], gen_len=3, top_p=1e-9, decode=lambda a: " ".join(str(int(t)) for t in a))
    assert len(text.split()) == 3


def test_generate_from_an_8_shard_checkpoint(tmp_path):
    """resharding_example.py:40-60: network.state = read_ckpt(network.state, dir, 8, shards_out=1), then generate."""
    import os
    from oracle import ckpt_oracle as CK
    from mesh_transformer import checkpoint, sampling
    params = O.seeded_params(CFG1, 7)
    d = str(tmp_path) + os.sep
    stacked = {"params": CK.shard_tree(params, 8, CFG1), "step": np.full(8, 5, np.uint32)}
    for s in range(8):
        checkpoint.write_ckpt(stacked, d, s)
    net = net_for(CFG1, None, sampling.greedy_sample)            # random init, then the checkpoint replaces it
    net.state = checkpoint.read_ckpt(net.state, d, 8, shards_out=1)
    prompt = O.seeded_prompt(8, 1, 24)
    ctx = O.left_pad(prompt, 48)
    _, out = net.generate(ctx, [24], 8, {})
    ref = O.Model(CFG1, params, torch.float64).generate(ctx, [24], 8, O.greedy_sample, {})
    assert np.array_equal(out[0], ref[0])


def test_parameter_updates_reach_the_packed_weights():
    """The packed copies follow the tree: calls on unchanged parameters reuse them, an in-place update of a leaf
    (no new tensor object, same memory) rebuilds them, and invalidate() forces a rebuild."""
    from mesh_transformer import sampling
    params = O.seeded_params(CFG1, 4)
    ctx = O.left_pad(O.seeded_prompt(4, 1, 40), 64)
    net = net_for(CFG1, params, sampling.greedy_sample)
    _, out = net.generate(ctx, [40], 4, {}, return_logits=True)
    eng = net.engine()
    _, again = net.generate(ctx, [40], 4, {}, return_logits=True)
    assert net.engine() is eng and np.array_equal(again[2], out[2])
    leaf = net.state["params"]["causal_transformer_shard/~/projection_shard/~/linear"]["b"]
    bump = torch.zeros_like(leaf)
    bump.view(-1)[123] = 50.0                      # makes token 123 the best one at every step
    leaf.add_(bump)
    _, new = net.generate(ctx, [40], 4, {}, return_logits=True)
    assert net.engine() is not eng
    assert (new[0][0, :, 0] == 123).all()
    np.testing.assert_allclose(new[2][0, :1, 0, 123], out[2][0, :1, 0, 123] + 50.0, rtol=0, atol=1e-4)
    eng2 = net.engine()
    net.invalidate()
    assert net.engine() is not eng2


def test_sliding_window_evicts_oldest_tokens():
    """ctx not padded (L == P): every decode step drops the oldest real token (layers.py:325-326)."""
    from mesh_transformer import sampling
    cfg = dict(CFG1, n_vocab=1024)
    params = O.seeded_params(cfg, 4)
    prompt = O.seeded_prompt(4, 1, 20, hi=1024)
    net = net_for(cfg, params, sampling.greedy_sample)
    _, out = net.generate(prompt, [20], 10, {}, return_logits=True)
    ref_t, _, ref_l = O.Model(cfg, params, torch.float64).generate(prompt, [20], 10, O.greedy_sample, {}, return_logits=True)
    assert rel(out[2], ref_l) < 1e-4
    assert np.array_equal(out[0], ref_t)


def test_host_callable_sampler_contract():
    """Any callable with the reference's sampler signature works (slow path through the host)."""
    calls = []

    def my_sampler(key, logits, sampler_input, bonus=0):
        calls.append((logits.shape, int(bonus)))
        return np.array([int(np.argmax(logits[0])) if bonus == 0 else 7], np.uint32), None

    cfg = dict(CFG1, n_vocab=1024)
    params = O.seeded_params(cfg, 5)
    prompt = O.left_pad(O.seeded_prompt(5, 2, 6, hi=1024), 16)
    net = net_for(cfg, params, my_sampler)
    _, out = net.generate(prompt, [6, 6], 4, {"bonus": np.array([0, 1])})
    ref_t, _ = O.Model(cfg, params, torch.float64).generate(prompt[:1], [6], 4, O.greedy_sample, {})
    assert np.array_equal(out[0][0], ref_t[0])
    assert out[0][1, :, 0].tolist() == [7, 7, 7, 7]
    assert calls[0] == ((1, 1024), 0) and len(calls) == 8


def test_generate_argument_checks():
    from mesh_transformer import sampling
    cfg = dict(CFG1, n_vocab=1024)
    net = net_for(cfg, O.seeded_params(cfg, 6), sampling.greedy_sample)
    with pytest.raises(ValueError):
        net.generate(np.zeros((1, 8), np.uint32), [9], 2, {})          # ctx_length > ctx
    with pytest.raises(ValueError):
        net.generate(np.zeros((2, 8), np.uint32), [3], 2, {})          # one length per row
    with pytest.raises(ValueError):
        from mesh_transformer.transformer_shard import CausalTransformer
        CausalTransformer(dict(cfg, cores_per_replica=8))


def test_fused_decode_attention_give_up_is_raised_once_and_recovered_from():
    """The batch-1 out projection that computes the attention itself waits for its partials for a bounded time and
    flags a give-up in word 2 of its counter block.  The flag is forced from the host here (every kernel still exits
    normally: a launch that finds the flag up does not wait): generate must raise once, clear the flag, move the
    session to the separate attention launches, and the next call must match the oracle again."""
    from mesh_transformer import sampling
    cfg = dict(layers=2, d_model=2048, n_heads=32, n_vocab=2048, norm="layernorm", pe="rotary", pe_rotary_dims=32,
               seq=64, cores_per_replica=1)            # float32, K = 5 whole tiles: the fused kernel applies
    params = O.seeded_params(cfg, 21)
    ctx = O.left_pad(O.seeded_prompt(21, 1, 20, hi=2048), 64)
    net = net_for(cfg, params, sampling.greedy_sample)
    ref = O.Model(cfg, params, torch.float64).generate(ctx, [20], 12, O.greedy_sample, {})
    _, out = net.generate(ctx, [20], 12, {})
    ses = net.engine().sessions[(1, 63)]
    assert ses.fused_attn and np.array_equal(out[0], ref[0])
    flag = ses.oa_work[8:12].view(torch.int32)
    assert int(flag[0]) == 0
    flag.fill_(1)
    with pytest.raises(RuntimeError, match="gave up"):
        net.generate(ctx, [20], 12, {})
    assert int(flag[0]) == 0 and not ses.fused_attn and not ses.graphs
    _, again = net.generate(ctx, [20], 12, {})
    assert net.engine().sessions[(1, 63)] is ses and np.array_equal(again[0], ref[0])


@pytest.mark.parametrize("which", ["fp32", "bf16"])
def test_layer_pieces_qvk_proj_self_attn_ff_and_projection_loss(which):
    """The module-level seams of layers.py:260-297 and 569-593 one by one against the float64 oracle: qvk_proj,
    self_attn on a whole left-padded window (causal + pad bias, as get_init_decode_state builds it) and on one new
    token (pad bias only, as decode_once builds it), ff, and ProjectionShard.loss with and without z_loss - the loss
    reference is the library cross entropy plus the z term written out on the oracle's logits."""
    from mesh_transformer import layers
    from mesh_transformer.layers import TransformerLayerShard, ProjectionShard
    cfg, dt, tol = (CFG1, torch.float32, 1e-4) if which == "fp32" else (CFG_BF, torch.bfloat16, 4e-3)
    params = O.seeded_params(cfg, 31, dt)
    model = O.Model(cfg, params, torch.float64)
    lref = model.layers[1]
    g = torch.Generator().manual_seed(31)
    T, pad = 45, 7
    x = torch.randn(T, cfg["d_model"], generator=g, dtype=torch.float64)
    xn = lref.norm(x)
    with layers.transform(params):
        layer = TransformerLayerShard(cfg, "layer_1", 2.0 / cfg["layers"])
        proj = ProjectionShard(cfg)
    q, v, k = layer.qvk_proj(xn.float())
    qr, vr, kr = lref.qvk_proj(xn)
    H, dh = cfg["n_heads"], cfg["d_model"] // cfg["n_heads"]
    assert tuple(q.shape) == (T, H, dh)
    for got, ref in ((q, qr), (v, vr), (k, kr)):
        assert rel(got, ref) < tol
    # whole window: causal mask + masked leading keys
    bias = O.MASK * (1.0 - torch.tril(torch.ones(T, T, dtype=torch.float64)))
    bias = bias - 1e10 * (torch.arange(T) < pad).double()
    a_ref = lref.self_attn(qr, vr, kr, bias)
    a_got = layer.self_attn(qr.float(), vr.float(), kr.float(), bias.numpy())
    assert rel(a_got[pad:], a_ref[pad:]) < tol
    # one new token against the window (decode_once): q is the last row, rotated at the last window index
    bias1 = -1e10 * (torch.arange(T) < pad).double()
    d_ref = lref.self_attn(qr[-1:], vr, kr, bias1)
    d_got = layer.self_attn(qr[-1:].float(), vr.float(), kr.float(), bias1.numpy())
    assert rel(d_got, d_ref) < tol
    assert rel(d_got, a_ref[-1:]) < tol                       # the same thing, computed by the other kernel
    with pytest.raises(NotImplementedError):
        layer.self_attn(qr.float(), vr.float(), kr.float(), 0)                # several queries without a causal mask
    with pytest.raises(NotImplementedError):
        layer.self_attn(qr.float(), vr.float(), kr.float(), (bias * 1e-12).numpy())   # not a 0 / -1e10 mask
    assert rel(layer.ff(xn.float()), lref.ff(xn)) < tol
    # ProjectionShard.loss
    tgt = torch.randint(0, cfg["n_vocab"], (T,), generator=g)
    logits = model.proj(x)
    tgt[3] = int(logits[3].argmax())                          # one row whose target holds the maximum
    ce = torch.nn.functional.cross_entropy(logits, tgt, reduction="none")
    lse = torch.logsumexp(logits - logits.max(-1, keepdim=True).values, -1)
    for z in (0.0, 1.0, 2.5):
        loss, correct = proj.loss(x.float(), tgt.numpy(), z)
        ref = ce + (1e-4 * lse ** 2 * z).mean()
        assert float((loss.double().cpu() - ref).abs().max()) < (1e-4 if which == "fp32" else 2e-2) * float(ref.abs().max())
        assert bool(correct[3]) and np.array_equal(correct.cpu().numpy(), (logits.argmax(-1) == tgt).numpy())


def test_softmax_sample_is_a_device_sampler():
    """config["sampler"] = softmax_sample (sampling.py:6-7) runs on the fused device sampler (nothing filtered) and
    follows the oracle's stream on the same uniforms; per-row temperatures."""
    from mesh_transformer import sampling
    assert sampling.builtin_kind(sampling.softmax_sample) == "softmax"
    cfg = dict(CFG1, n_vocab=2048)
    params = O.seeded_params(cfg, 14)
    ctx = O.left_pad(O.seeded_prompt(14, 2, 21, hi=2048), 40)
    G = 10
    u = np.random.Generator(np.random.Philox(14)).random((2, G))
    opts = {"temp": np.array([0.7, 1.4])}
    net = net_for(cfg, params, sampling.softmax_sample)
    _, out = net.generate(ctx, [21, 21], G, opts, uniforms=u)
    ref = O.Model(cfg, params, torch.float64).generate(ctx, [21, 21], G, O.softmax_sample, opts, uniforms=u)
    assert np.array_equal(out[0], ref[0])
    assert len({int(t) for t in out[0].reshape(-1)}) > 4       # a draw, not an argmax


@pytest.mark.parametrize("case", ["padded", "sliding"])
def test_generate_returns_the_scan_carry(case):
    """The first return value of generate (transformer_shard.py:196-216): last token, per-layer decode state in the
    reference's layout ([B, T, H, dh], window order, K not rotated, tokens_decoded), key."""
    from mesh_transformer import sampling
    cfg = dict(CFG1, n_vocab=1024)
    params = O.seeded_params(cfg, 15)
    if case == "padded":
        lens, L, G = [9, 14], 32, 6
    else:
        lens, L, G = [12, 12], 12, 5                            # the window slides: the oldest tokens are evicted
    ctx = np.zeros((2, L), np.uint32)
    for b, n in enumerate(lens):
        ctx[b, L - n:] = O.seeded_prompt(50 + b, 1, n, hi=1024)[0]
    net = net_for(cfg, params, sampling.greedy_sample)
    final, out = net.generate(ctx, lens, G, {})
    ref_states = []
    ref = O.Model(cfg, params, torch.float64).generate(ctx, lens, G, O.greedy_sample, {}, final_states=ref_states)
    assert np.array_equal(out[0], ref[0])
    last, states, key = final
    assert key is None and last.shape == (2, 1) and np.array_equal(last, ref[0][:, -1])
    assert len(states) == cfg["layers"]
    T = L - 1
    for i, st in enumerate(states):
        assert st["k"].shape == (2, T, cfg["n_heads"], 64) and st["tokens_decoded"].dtype == np.uint32
        for b, n in enumerate(lens):
            r = ref_states[b][i]
            assert int(st["tokens_decoded"][b]) == r["tokens_decoded"] == n - 1 + G
            real = min(n - 1 + G, T)
            assert rel(st["k"][b, T - real:], r["k"][T - real:]) < 1e-5
            assert rel(st["v"][b, T - real:], r["v"][T - real:]) < 1e-5
            assert not st["k"][b, :T - real].any()
    net.generate(ctx, lens, G, {})
    with pytest.raises(RuntimeError):
        states[0]                                               # the window has been reused by the later call


def test_logits_from_the_graph_path_equal_the_eager_ones():
    """return_logits keeps the recorded steps (the logits of a step go to a slot of a staging buffer); the eager
    path (steps_per_graph = 0) must give the same bits, replay after replay."""
    from mesh_transformer import sampling
    cfg = dict(CFG1, n_vocab=4096)
    params = O.seeded_params(cfg, 16)
    ctx = O.left_pad(O.seeded_prompt(16, 2, 19, hi=4096), 64)
    u = np.random.Generator(np.random.Philox(16)).random((2, 27))
    opts = {"top_p": np.array([0.9, 0.8]), "temp": np.array([0.8, 1.1])}
    eager = net_for(dict(cfg, steps_per_graph=0), params, sampling.nucleaus_sample)
    _, ref = eager.generate(ctx, [19, 19], 27, opts, return_logits=True, uniforms=u)
    net = net_for(cfg, params, sampling.nucleaus_sample)
    for _ in range(2):
        _, out = net.generate(ctx, [19, 19], 27, opts, return_logits=True, uniforms=u)
        assert np.array_equal(out[0], ref[0]) and np.array_equal(out[2], ref[2])
    assert any(k[3] for k in net.engine().sessions[(2, 63)].graphs)


# ------------------------------------------------------------------ float16 range: outlier channels, large LayerNorm scales
def outlier_params(cfg, seed, saturate=False):
    """A bf16 tree shaped like a trained model rather than like an initialiser: four residual channels carry +-50 ..
    +-500 from the embedding bias on and grow by the fc_out bias in every layer (past 1000 at the end), LayerNorm scales
    run from 0.5 to 30 with offsets ~N(0, 0.5), the input matrices are rescaled so that LayerNorm outputs reach ~40,
    q and k ~25, attention scores a standard deviation of 1-11, fc_in ~50, the embedding matrix has entries up to ~5
    and one k matrix holds +-4 next to N(0, 0.02) entries (its float16 copy gets a small power-of-two scale).
    saturate: one fc_in bias of 1e5, so that one gelu output lies beyond the float16 range."""
    p = O.seeded_params(cfg, seed, torch.float32)
    rng = np.random.Generator(np.random.Philox(seed + 1000))
    d = cfg["d_model"]
    ch = np.array([7, 300, 511, 900])
    big = np.array([300.0, -500.0, 50.0, -120.0], np.float32)
    p[O.EMBED]["w"][0] *= 50.0
    p[O.EMBED]["b"][0, ch] = torch.from_numpy(big)
    for i in range(cfg["layers"]):
        ln = p[O.layer_key(i, "replicated_layer_norm")]
        sc = rng.uniform(0.5, 30.0, d).astype(np.float32)
        sc[ch] = 1.0
        ln["scale"][0] = torch.from_numpy(sc)
        ln["offset"][0] = torch.from_numpy(rng.standard_normal(d).astype(np.float32) * 0.5)
        p[O.layer_key(i, "linear_5")]["b"][0, ch] += torch.from_numpy(big * 0.3)
        for name, gain in (("linear", 2.0), ("linear_1", 8.0), ("linear_2", 2.0), ("linear_4", 10.0)):
            p[O.layer_key(i, name)]["w"][0] *= gain / torch.from_numpy(np.sqrt(sc))[:, None]
    w = p[O.layer_key(1, "linear_2")]["w"]
    w[0, 5, 17], w[0, 700, 333] = 4.0, -4.0
    p[O.PROJ_LN]["scale"][0] = torch.from_numpy(rng.uniform(0.5, 3.0, d).astype(np.float32))
    p[O.PROJ_LN]["offset"][0] = torch.from_numpy(rng.standard_normal(d).astype(np.float32) * 0.2)
    if saturate:
        p[O.layer_key(0, "linear_4")]["b"][0, 5] = 1.0e5
    return {m: {k: v.to(torch.bfloat16) for k, v in l.items()} for m, l in p.items()}


def test_outlier_channels_and_large_layernorm_scales_stay_within_the_bf16_bound():
    """The matrix-core paths round their operands to float16 (5 exponent bits).  With the outlier tree above every
    path must still be within 2e-2 of the float64 oracle on the logits: batch-1 generate (float32 activations at
    decode, float16 in its prefill), batch-2 generate (float16 everywhere), the every-position forward, and eval."""
    from mesh_transformer import sampling
    params = outlier_params(CFG_BF, 77)
    m = O.Model(CFG_BF, params, torch.float64)
    net = net_for(CFG_BF, params, sampling.greedy_sample)
    prompt = O.seeded_prompt(77, 2, 64)
    ctx = O.left_pad(prompt, 128)
    ctx[1, :64 + 23] = 0                                        # row 1 keeps 41 tokens
    lens = [64, 41]
    G = 12
    for rows in ([0], [0, 1]):
        c, n = ctx[rows], [lens[r] for r in rows]
        _, out = net.generate(c, n, G, {}, return_logits=True)
        ref_t, _, ref_l = m.generate(c, n, G, O.greedy_sample, {}, return_logits=True)
        # teacher forcing is not needed while the streams agree; compare up to the first difference (if any)
        same = (out[0] == ref_t).all(axis=(0, 2))
        upto = G if same.all() else int(np.argmin(same)) + 1
        err = float(np.abs(out[2][:, :upto] - ref_l[:, :upto]).max())
        print(f"outliers, batch {len(rows)}: max |dlogit| {err:.2e} over {upto} steps; logits std {ref_l.std():.2f} max {np.abs(ref_l).max():.1f}")
        assert err < 2e-2 and upto >= 8
    toks = O.seeded_prompt(78, 1, 96)
    got = net.forward(toks)[0].double().cpu()
    ref = m.forward(toks[0])
    err = float((got - ref).abs().max())
    print(f"outliers, forward: max |dlogit| {err:.2e}; residual stream reaches {float(m.embed(toks[0]).abs().max()):.0f} at the input")
    assert err < 2e-2
    tgt = np.roll(toks, -1, axis=1)
    ev = net.eval({"obs": toks, "target": tgt})
    rl = m.loss(toks[0], tgt[0])
    assert float(np.abs(ev["all_loss"][0] - rl["all_loss"].numpy()).max()) < 2e-2


def test_operands_beyond_the_float16_range_saturate_and_stay_finite():
    """One gelu output of 1e5 (an fc_in bias of 1e5): on the matrix-core paths that operand is 65504 - conversions to
    float16 saturate instead of overflowing to infinity - so the caller sees finite logits, equal (within the usual
    2e-2) to the reference evaluated with that operand clamped to +-65504, and not to the unclamped reference.  The
    batch-1 decode step keeps float32 activations and does not clamp."""
    from mesh_transformer import sampling
    params = outlier_params(CFG_BF, 79, saturate=True)
    net = net_for(CFG_BF, params, sampling.greedy_sample)
    toks = O.seeded_prompt(79, 1, 48)
    got = net.forward(toks)[0].double().cpu()
    assert bool(torch.isfinite(got).all())
    m = O.Model(CFG_BF, params, torch.float64)
    free = m.forward(toks[0])
    l0 = m.layers[0]
    l0.ff = lambda x: torch.clamp(O.gelu_tanh(x @ l0.w1 + l0.b1), -65504.0, 65504.0) @ l0.w2 + l0.b2
    clamped = m.forward(toks[0])
    e_c, e_f = float((got - clamped).abs().max()), float((got - free).abs().max())
    print(f"saturating operand: max |dlogit| vs clamped reference {e_c:.2e}, vs unclamped {e_f:.2e}")
    assert e_c < 2e-2 < e_f
    _, out = net.generate(O.left_pad(toks, 64), [48], 4, {}, return_logits=True)
    assert np.isfinite(out[2]).all()

"""The batch-1 decode step as one persistent launch (config key "decode_single_launch") against the
launch-per-matrix path and the CPU oracle, on seeded inputs."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import gptj_oracle as O

CFG_F32 = dict(layers=2, d_model=512, n_heads=8, n_vocab=50400, norm="layernorm", pe="rotary", pe_rotary_dims=32,
               seq=168, cores_per_replica=1)
CFG_BF = dict(layers=4, d_model=1024, n_heads=4, n_vocab=50400, norm="layernorm", pe="rotary", pe_rotary_dims=64,
              seq=128, cores_per_replica=1)


def make(cfg, params, single):
    from mesh_transformer import sampling
    from mesh_transformer.transformer_shard import CausalTransformer
    return CausalTransformer(dict(cfg, sampler=sampling.greedy_sample, decode_single_launch=single), params)


@pytest.mark.parametrize("graphs", [0, 8])
def test_single_launch_fp32_matches_the_oracle_and_the_other_path(graphs):
    """float32, d_head 64: logits within 1e-4 relative of the float64 oracle, tokens equal, over 40 steps that
    start with a short prompt (attention ranges with one key, then growing)."""
    params = O.seeded_params(CFG_F32, 3)
    prompt = O.seeded_prompt(3, 1, 5)
    ctx = O.left_pad(prompt, 168)
    G = 40
    print("fp32 single launch, graphs", graphs, flush=True)
    cfg = dict(CFG_F32, steps_per_graph=graphs)
    _, one = make(cfg, params, True).generate(ctx, [5], G, {}, return_logits=True)
    _, many = make(cfg, params, False).generate(ctx, [5], G, {}, return_logits=True)
    ref_t, _, ref_l = O.Model(CFG_F32, params, torch.float64).generate(ctx, [5], G, O.greedy_sample, {}, return_logits=True)
    scale = np.abs(ref_l).max()
    assert np.abs(one[2] - ref_l).max() / scale < 1e-4
    assert np.abs(one[2] - many[2]).max() / scale < 1e-4
    assert (one[0] == ref_t).all() and (one[0] == many[0]).all()


def test_single_launch_bf16_logits_and_greedy_stream():
    """bf16, d_head 256: 64-token prompt, 32 steps; logits within 2e-2 of the oracle on the same bf16-rounded weights
    and the same greedy tokens as the oracle and as the launch-per-matrix path."""
    params = O.seeded_params(CFG_BF, 1, torch.bfloat16)
    prompt = O.seeded_prompt(1, 1, 64)
    ctx = O.left_pad(prompt, 128)
    G = 32
    print("bf16 single launch", flush=True)
    _, one = make(CFG_BF, params, True).generate(ctx, [64], G, {}, return_logits=True)
    _, many = make(CFG_BF, params, False).generate(ctx, [64], G, {}, return_logits=True)
    ref_t, _, ref_l = O.Model(CFG_BF, params, torch.float64).generate(ctx, [64], G, O.greedy_sample, {}, return_logits=True)
    err = np.abs(one[2] - ref_l).max()
    print("bf16 single launch: max |dlogit|", err, "vs other path", np.abs(one[2] - many[2]).max())
    assert err < 2e-2
    assert np.array_equal(one[0], ref_t) and np.array_equal(one[0], many[0])

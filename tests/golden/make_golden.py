"""Writes the fixtures of this directory from the CPU oracle (oracle/gptj_oracle.py, float64).

The reference ships no golden vectors and cannot be imported here (jax and haiku are absent), so these are
outputs of the oracle - itself pinned by tests/test_oracle.py - frozen so that a drift of the oracle, of the
seeded inputs or of the HIP path shows up as a diff against committed data.  Run from the repository root:

    python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import gptj_oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

# BASELINE config 1: tiny fp32 stack, seed 0, 128-token prompt, 32 greedy steps (ctx padded to 168 >= 128 + 32)
CFG1 = dict(layers=2, d_model=512, n_heads=8, n_vocab=50400, norm="layernorm", pe="rotary", pe_rotary_dims=32,
            seq=168, cores_per_replica=1)


def config1():
    params = O.seeded_params(CFG1, 0)
    prompt = O.seeded_prompt(0, 1, 128)
    ctx = O.left_pad(prompt, 168)
    m = O.Model(CFG1, params, torch.float64)
    toks, _, logits = m.generate(ctx, [128], 32, O.greedy_sample, {}, return_logits=True)
    lg = logits[0, :, 0, :]                                    # [32, V]
    top = np.argsort(-lg, axis=-1, kind="stable")[:, :8]
    taps = []
    m.generate_initial(ctx[0], 128, taps)
    return dict(prompt=prompt.astype(np.uint32), tokens=toks[0, :, 0].astype(np.uint32),
                top8_ids=top.astype(np.int32), top8_logits=np.take_along_axis(lg, top, -1).astype(np.float64),
                logits_sum=lg.sum(-1).astype(np.float64), logits_sqsum=(lg ** 2).sum(-1).astype(np.float64),
                prefill_layer_norms=np.array([float(t[-128:].norm()) for t in taps]))


def nucleus():
    rng = np.random.default_rng(2024)
    V = 1000
    logits = (rng.standard_normal((5, V)) * 2.0).astype(np.float32)
    logits[1, :500] = logits[1, 500:]                          # ties
    logits[2, 3], logits[2, 4] = -0.0, 0.0
    top_p = np.array([0.9, 0.5, 0.999, 0.05, 0.7])
    temp = np.array([0.8, 1.0, 1.5, 0.3, 2.0])
    top_k = np.array([0, 1, 5, 0, 100], np.int32)              # 0 = no top-k
    u = rng.random(5)
    keep = np.zeros((5, V), bool)
    tok = np.zeros(5, np.int32)
    for r in range(5):
        k = None if top_k[r] == 0 else int(top_k[r])
        f = O.nucleaus_filter(logits[r:r + 1], float(top_p[r]), k)
        keep[r] = f[0] == logits[r]
        tok[r] = O.inverse_cdf_draw(logits[r:r + 1], f, float(temp[r]), float(u[r]))
    demo = np.array([[-2, -1, 0, 0.8, 0, 0.1, 0.3, 0.4, 0.5, 0.6, 0.7, -3]], np.float32)   # sampling.py:49
    demo_keep = O.nucleaus_filter(demo, 0.9)[0] == demo[0]
    return dict(logits=logits, top_p=top_p, temp=temp, top_k=top_k, u=u, keep=np.packbits(keep, axis=-1), token=tok,
                demo=demo, demo_keep=demo_keep)


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "config1_greedy.npz"), **config1())
    np.savez_compressed(os.path.join(HERE, "nucleus_cases.npz"), **nucleus())
    with open(os.path.join(HERE, "README.json"), "w") as f:
        json.dump({"config1_greedy.npz": "BASELINE config 1 through the float64 oracle: seeded prompt, 32 greedy tokens, "
                   "top-8 logits per step, logit checksums, residual norms after each prefill layer",
                   "nucleus_cases.npz": "nucleaus_filter keep-masks (bit-packed) and inverse-CDF tokens of the oracle on "
                   "seeded logits with ties, signed zeros and the top-k quirk; the reference's demo vector (sampling.py:49)",
                   "generator": "tests/golden/make_golden.py", "cfg1": CFG1}, f, indent=1)
    print("written")

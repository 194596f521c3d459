#!/usr/bin/env python3
"""Benchmark of the GPT-J-6B generate path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

A "step" is one batch-1 greedy decode step of GPT-J-6B (bf16 weights, random init) after a 512-token
prompt left-padded to 2048 (BASELINE config 3).  W untimed steps, then exactly K steps between two
device synchronisations.  Prints ONE JSON line; `value` is generated tokens per second.

Also reported on the same line:
  roofline      the dominant kernel (the fused LayerNorm + q|v|k|fc_in GEMV, 28 launches per step):
                algorithmic bytes of one launch / its average duration (HIP events), against 8 TB/s
  step_hbm      whole-step algorithmic bytes / measured step time
  prefill       the 511-token prefill of the same run, and one full-shape layer at [8 x 2048] tokens
                (BASELINE config 2), as TFLOP/s against the 2.5 PFLOP/s 16-bit MFMA peak
  decode_b32    BASELINE config 4 in full: batch 32, 1024-token prompts padded to 2048, 1024 steps of nucleus sampling
                (top_p 0.9, temperature 0.8, host Philox(3) uniforms) that fill the K/V window to 2047 keys; ms/step and
                algorithmic HBM fraction over the whole run and over its last 64 steps
  forward_16x2048  BASELINE config 5: full-context forward of 16 x 2048 tokens with the 50400-wide logits at
                every position, TFLOP/s against the MFMA peak
  cpu_baseline  the CPU oracle (torch float32 on the host cores) on a bounded sample of the workload
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "mesh-transformer-jax_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK = 8.0e12          # B/s
# HBM bytes of one launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by what
# the same counter reads for a plain 234,881,024-byte copy (profiles/gemv_inproj_hbm_traffic_pmc.md)
DOMINANT_KERNEL_TRAFFIC = 235603296
MFMA_BF16_PEAK = 2.5e15    # flop/s dense

CFG_6B = dict(layers=28, d_model=4096, n_heads=16, n_vocab=50400, norm="layernorm", pe="rotary", pe_rotary_dims=64,
              seq=2048, cores_per_replica=1, early_cast=True)


def synthetic_tree(cfg, seed, device, dtype, std=0.02):
    """Random-init tree: every weight and bias ~ N(0, 0.02), LayerNorm scale 1 / offset 0."""
    import torch
    from mesh_transformer.engine import ROOT as R
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    d, V, F = cfg["d_model"], cfg["n_vocab"], 4 * cfg["d_model"]
    rn = lambda *s: (torch.randn(*s, generator=g, device=device, dtype=torch.float32) * std).to(dtype)
    ln = lambda: {"scale": torch.ones(1, d, dtype=dtype, device=device), "offset": torch.zeros(1, d, dtype=dtype, device=device)}
    t = {R + "embedding_shard/~/linear": {"w": rn(1, V, d), "b": rn(1, d)}}
    for i in range(cfg["layers"]):
        p = f"{R}layer_{i}/~/"
        t[p + "replicated_layer_norm"] = ln()
        for name in ("linear", "linear_1", "linear_2", "linear_3"):
            t[p + name] = {"w": rn(1, d, d)}
        t[p + "linear_4"] = {"w": rn(1, d, F), "b": rn(1, F)}
        t[p + "linear_5"] = {"w": rn(1, F, d), "b": rn(1, d)}
    t[R + "projection_shard/~/replicated_layer_norm"] = ln()
    t[R + "projection_shard/~/linear"] = {"w": rn(1, d, V), "b": rn(1, V)}
    return t


def decode_bytes_per_step(cfg, ctx_mean, B=1):
    """Algorithmic HBM bytes of one decode step: every weight once, K/V window read + one slot written,
    embedding rows, logits."""
    d, V, n, F = cfg["d_model"], cfg["n_vocab"], cfg["layers"], 4 * cfg["d_model"]
    layer = (4 * d * d + 2 * d * F) * 2 + (F + d + 2 * d) * 2          # bf16 matrices + biases/LN as stored
    weights = n * layer + (d * V + V + 2 * d) * 2
    kv = B * n * 2 * d * 2 * (ctx_mean + 1)
    return weights + kv + B * d * 2 + B * V * 4


def gemv_inproj_bytes(cfg):
    d, F = cfg["d_model"], 4 * cfg["d_model"]
    return (3 * d + F) * d * 2 + d * 4 + 2 * d * 4 + F * 4 + (3 * d + F) * 4   # W_in + x + LN params + b1 + outputs


def time_dominant_kernel(net, ses, reps=20):
    """Average duration of the fused LayerNorm + q|v|k|fc_in GEMV, measured with HIP events on the stream it is
    launched on: 28 back-to-back launches (one per layer, 6.6 GB of distinct weights, so nothing is re-read
    from cache) per repetition."""
    import ctypes as C
    import torch
    from mesh_transformer import _abi
    from mesh_transformer._abi import EPI_INPROJ, F32, check, ptr
    eng = net.engine()
    L, w = _abi.lib(), eng.w
    d, F = w.d, w.F
    s = _abi.stream_handle()
    ses.pos.fill_(600)
    ses.x.normal_()

    def sweep():
        for i in w.layer_ids:
            ip = eng._inproj(ses, i, 1, ses.pos, ses.q, F32, ses.act, F32, None)
            check(L.mtj_gemv(ptr(ses.x), ptr(w.ln_s[i]), ptr(w.ln_o[i]), ptr(w.w_in[i]), ptr(w.b1[i]), 3 * d + F, d,
                             w.dtype, EPI_INPROJ, None, 0, C.byref(ip), None, s))

    sweep()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        sweep()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e-3 / (reps * len(w.layer_ids))


def time_prefill_layer(net, B=8, T=2048, reps=5):
    """One full-shape layer forward on [B x T] tokens (BASELINE config 2): LayerNorm, fused input GEMM,
    flash attention, output GEMM.  Returns seconds per layer forward."""
    import torch
    eng = net.engine()
    ses = eng.session(B, T, T, T + 8)
    M = B * T
    x = torch.randn(M, eng.w.d, device=eng.device)
    pos0 = torch.zeros(B, dtype=torch.int32, device=eng.device)
    run = lambda: eng.layer_prefill(ses, 0, x, ses.h_pf[:M], ses.act_pf[:M], T, pos0)
    run()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        run()
    b.record()
    torch.cuda.synchronize()
    eng.sessions.pop((B, T), None)
    return a.elapsed_time(b) * 1e-3 / reps


def time_decode_b32(net, cfg, B=32, P=1024, L=2048, G=1024, tail=64):
    """BASELINE config 4 at its real length: batch 32 nucleus decode after 1024-token prompts, 1024 generated tokens,
    so the K/V window grows from 1024 to 2047 keys per sequence (15 -> 30 GB of K/V read per step).  Reported over the
    whole run and over its last `tail` steps."""
    import numpy as np
    from oracle import gptj_oracle as O
    u = np.random.Generator(np.random.Philox(3)).random((B, G))
    ctx = O.left_pad(O.seeded_prompt(3, B, P), L)
    opts = {"top_p": np.full(B, 0.9), "temp": np.full(B, 0.8)}
    tm = {"warmup": G - tail}
    from mesh_transformer import sampling
    nucleus = sampling.nucleaus_sample                                # whatever sampler the net was configured with
    net.generate(ctx, np.full(B, P), G, opts, uniforms=u, sampler=nucleus)   # untimed: allocates, records the graphs
    net.generate(ctx, np.full(B, P), G, opts, uniforms=u, sampler=nucleus, timing=tm)
    net.engine().sessions.pop((B, L - 1), None)

    def leg(seconds, first, n):
        ms = seconds * 1e3 / n
        ctx_mean = (P - 1) + first + (n - 1) / 2.0
        nbytes = decode_bytes_per_step(cfg, ctx_mean, B)
        return {"ms_per_step": ms, "tok_s": B * 1e3 / ms, "steps": n, "ctx_mean": ctx_mean,
                "step_hbm": {"bytes": nbytes, "achieved": nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s",
                             "frac": nbytes / (ms * 1e-3) / HBM_PEAK}}

    res = leg(tm["warmup_s"] + tm["decode_s"], 0, G)
    res.update(batch=B, prompt=P, sampler="nucleus top_p 0.9 temp 0.8, host Philox(3) uniforms",
               prefill_ms=tm["prefill_s"] * 1e3, prefill_tok_s=tm["prefill_tokens"] / tm["prefill_s"],
               last_steps=leg(tm["decode_s"], G - tail, tail))
    return res


def time_forward_16x2048(net, cfg, B=16, L=2048):
    """BASELINE config 5: every-position logits of B x L uniform-random tokens (seed 4)."""
    import numpy as np
    import torch
    rng = np.random.Generator(np.random.Philox(4))
    ctx = rng.integers(0, 50257, (B, L)).astype(np.uint32)
    net.forward(ctx)                                                   # untimed: allocates
    tm = {}
    out = net.forward(ctx, timing=tm)
    del out
    net.engine().sessions.pop((B, L), None)
    torch.cuda.empty_cache()
    d, F, n, V = cfg["d_model"], 4 * cfg["d_model"], cfg["layers"], cfg["n_vocab"]
    fl = B * L * 2 * (n * (4 * d * d + 2 * d * F) + d * V) + B * n * 4 * d * L * (L + 1) / 2
    t = tm["forward_s"]
    return {"ms": t * 1e3, "tok_s": B * L / t, "tflops": fl / t / 1e12, "frac_mfma": fl / t / MFMA_BF16_PEAK,
            "flops": "dense 2*params per token + causal attention 4*d*(t+1) per query"}


def cpu_model_name():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(net, cfg, n_layers=4, steps=8, prompt=512, L=2048):
    """The CPU oracle (torch float32, all host threads) on a bounded sample: the first `n_layers` layers of the
    same weights at full shape plus embedding and logits projection; 512-token prompt left-padded to 2048,
    prefill, then `steps` greedy decode steps.  Per-step time is extrapolated linearly to 28 layers."""
    import numpy as np
    import torch
    from oracle import gptj_oracle as O
    tree = net.state["params"]
    sub = dict(cfg, layers=n_layers)
    keep = {}
    for mod, leaves in tree.items():
        if "/layer_" in mod and int(mod.split("/layer_")[1].split("/")[0]) >= n_layers:
            continue
        keep[mod] = {k: v.cpu() for k, v in leaves.items()}
    model = O.Model(sub, keep, torch.float32)
    ctx = O.left_pad(O.seeded_prompt(2, 1, prompt), L)[0]
    t0 = time.perf_counter()
    nxt, states = model.generate_initial(ctx, prompt)
    t1 = time.perf_counter()
    per = []
    for _ in range(steps):
        a = time.perf_counter()
        logits, states = model.generate_once(nxt, states)
        nxt = np.asarray([O.greedy_sample(None, logits.numpy())], np.uint32)
        per.append(time.perf_counter() - a)
    # cost of embedding + logits projection alone
    x = torch.randn(1, cfg["d_model"])
    a = time.perf_counter()
    for _ in range(steps):
        model.proj(x)
    t_proj = (time.perf_counter() - a) / steps
    t_step = float(np.median(per))
    t_full = (t_step - t_proj) * cfg["layers"] / n_layers + t_proj
    return {
        "value": 1.0 / t_full, "unit": "tok/s", "cores": torch.get_num_threads(), "cpu": cpu_model_name(), "kind": "port",
        "sample": f"CPU oracle (torch float32), {n_layers} of {cfg['layers']} layers at full shape + logits, "
                  f"{prompt}-token prompt padded to {L}, {steps} decode steps (median {t_step * 1e3:.1f} ms/step for "
                  f"{n_layers} layers, prefill {t1 - t0:.1f} s); per-step time extrapolated linearly to {cfg['layers']} layers",
    }


def pmc_probe(dev):
    """Work for a hardware-counter pass: a device-to-device copy of exactly the size of W_in (the calibration
    for FETCH_SIZE / WRITE_SIZE), then the dominant GEMV 8 times over two layers' distinct weights."""
    import ctypes as C
    import torch
    from mesh_transformer import _abi, sampling
    from mesh_transformer._abi import EPI_INPROJ, F32, check, ptr
    from mesh_transformer.transformer_shard import CausalTransformer
    cfg = dict(CFG_6B, layers=2, sampler=sampling.greedy_sample)
    net = CausalTransformer(cfg, synthetic_tree(cfg, 2, dev, torch.bfloat16))
    eng = net.engine()
    ses = eng.session(1, 2047, 1, 1024)
    L, w = _abi.lib(), eng.w
    src = torch.empty(234881024, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    dst.copy_(src)
    torch.cuda.synchronize()
    ses.pos.fill_(600)
    ses.x.normal_()
    s = _abi.stream_handle()
    for rep in range(4):
        for i in w.layer_ids:
            ip = eng._inproj(ses, i, 1, ses.pos, ses.q, F32, ses.act, F32, None)
            check(L.mtj_gemv(ptr(ses.x), ptr(w.ln_s[i]), ptr(w.ln_o[i]), ptr(w.w_in[i]), ptr(w.b1[i]), 3 * w.d + w.F, w.d,
                             w.dtype, EPI_INPROJ, None, 0, C.byref(ip), None, s))
    torch.cuda.synchronize()
    print("pmc probe done")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=17)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip the prefill-layer measurement")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="counter probe for rocprofv3 --pmc: one plain 234,881,024-byte device copy, then 8 launches "
                         "of the dominant kernel on a 2-layer model of the 6B shape; prints no JSON")
    ap.add_argument("--decode-b32-probe", nargs=2, type=int, metavar=("PROMPT", "STEPS"),
                    help="profiling probe: BASELINE config 4 (batch 32, nucleus sampling) with PROMPT-token prompts padded to "
                         "2048 and STEPS decode steps, twice (the second run replays the recorded graphs); prints ms/step, "
                         "no bench line")
    ap.add_argument("--prefill-probe", action="store_true",
                    help="profiling probe: 6 forwards of one full-shape layer on 8 x 2048 tokens (BASELINE config 2) "
                         "on a 1-layer model of the 6B shape; prints the time per forward, no bench line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the whole model on ONE GPU (no collectives, no sharding); "
              f"--gpus {args.gpus} is not supported, run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from mesh_transformer import _abi, sampling
    from mesh_transformer.transformer_shard import CausalTransformer
    from oracle import gptj_oracle as O   # prompt generator + cpu_baseline leg only

    _abi.lib()
    dev = torch.device("cuda:0")
    if args.pmc_probe:
        pmc_probe(dev)
        return
    if args.decode_b32_probe:
        P, G = args.decode_b32_probe
        cfg = dict(CFG_6B, sampler=sampling.nucleaus_sample)
        net = CausalTransformer(cfg, synthetic_tree(cfg, 2, dev, torch.bfloat16))
        B, L = 32, 2048
        u = np.random.Generator(np.random.Philox(3)).random((B, G))
        ctx = O.left_pad(O.seeded_prompt(3, B, P), L)
        opts = {"top_p": np.full(B, 0.9), "temp": np.full(B, 0.8)}
        net.generate(ctx, np.full(B, P), G, opts, uniforms=u)
        tm = {"warmup": 1}
        net.generate(ctx, np.full(B, P), G, opts, uniforms=u, timing=tm)
        print(json.dumps({"decode_b32_ms_per_step": tm["decode_s"] * 1e3 / tm["decode_steps"], "prompt": P, "steps": G,
                          "keys": [P, P + G - 1]}))
        return
    if args.prefill_probe:
        c1 = dict(CFG_6B, layers=1, sampler=sampling.greedy_sample)
        n1 = CausalTransformer(c1, synthetic_tree(c1, 1, dev, torch.bfloat16))
        t = time_prefill_layer(n1)
        fl = 8 * 2048 * (2 * 201326592 + 4 * 4096 * 2049 / 2)
        print(json.dumps({"layer_8x2048_ms": t * 1e3, "tflops": fl / t / 1e12, "frac_mfma": fl / t / 2.5e15}))
        return
    cfg = dict(CFG_6B, sampler=sampling.greedy_sample)
    K, W = args.steps, args.warmup
    net = CausalTransformer(cfg, synthetic_tree(cfg, 2, dev, torch.bfloat16))
    P, L = 512, 2048
    ctx = O.left_pad(O.seeded_prompt(2, 1, P), L)

    net.generate(ctx, [P], W + K, {})                   # untimed: packs weights, allocates, records the graphs
    timing = {"warmup": W}
    _, out = net.generate(ctx, [P], W + K, {}, timing=timing)
    ms_per_step = timing["decode_s"] * 1e3 / timing["decode_steps"]
    tok_s = timing["decode_steps"] / timing["decode_s"]

    ctx_mean = (P - 1) + W + (K - 1) / 2.0
    step_bytes = decode_bytes_per_step(cfg, ctx_mean)
    step_bw = step_bytes / (ms_per_step * 1e-3)

    ses = net.engine().sessions[(1, L - 1)]
    t_k = time_dominant_kernel(net, ses)
    k_bytes = gemv_inproj_bytes(cfg)
    roofline = {"bound": "hbm", "kernel": "gemv_kernel (LayerNorm + q|v|k|fc_in, N=28672, K=4096, bf16)",
                "achieved": k_bytes / t_k / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                "frac": k_bytes / t_k / HBM_PEAK, "traffic": DOMINANT_KERNEL_TRAFFIC, "bytes_per_launch": k_bytes,
                "avg_launch_us": t_k * 1e6}

    d, F, n = cfg["d_model"], 4 * cfg["d_model"], cfg["layers"]
    pf_tokens = timing["prefill_tokens"]
    pf_flops = pf_tokens * 2 * n * (4 * d * d + 2 * d * F) + n * 4 * d * pf_tokens * (pf_tokens + 1) / 2
    prefill = {"tokens": pf_tokens, "ms": timing["prefill_s"] * 1e3, "tok_s": pf_tokens / timing["prefill_s"],
               "tflops": pf_flops / timing["prefill_s"] / 1e12, "frac_mfma": pf_flops / timing["prefill_s"] / MFMA_BF16_PEAK}
    if not args.no_extras:
        Bl, Tl = 8, 2048
        t_layer = time_prefill_layer(net, Bl, Tl)
        Ml = Bl * Tl
        fl = Ml * 2 * (4 * d * d + 2 * d * F) + Bl * 4 * d * Tl * (Tl + 1) / 2
        prefill["layer_8x2048"] = {"ms": t_layer * 1e3, "tflops": fl / t_layer / 1e12, "frac_mfma": fl / t_layer / MFMA_BF16_PEAK,
                                   "tok_s_28_layers": Ml / (t_layer * n)}

    res = {
        "metric": "GPT-J-6B bf16 decode tok/s (bs1, % HBM peak); prefill tok/s (% MFMA peak)",
        "value": tok_s, "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE config 3: GPT-J-6B bf16 random-init N(0,0.02), batch 1, 512-token prompt "
                               "left-padded to 2048, greedy decode; one step = one generated token",
                   "global_batch": 1, "prompt": P, "ctx": L, "steps_per_graph": int(cfg.get("steps_per_graph", 8))},
        "roofline": roofline,
        "step_hbm": {"bytes": step_bytes, "achieved": step_bw / 1e9, "unit": "GB/s", "frac": step_bw / HBM_PEAK},
        "prefill": prefill,
        "precision": "bf16 weights; batch-1 decode multiplies them with float32 activations, the matrix-core paths "
                     "(prefill, batched decode) with float16 activations and float16 copies of the same weight values",
    }
    if not args.no_extras:
        res["decode_b32"] = time_decode_b32(net, cfg)
        res["forward_16x2048"] = time_forward_16x2048(net, cfg)
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline(net, cfg)
    print(json.dumps(res))


if __name__ == "__main__":
    main()

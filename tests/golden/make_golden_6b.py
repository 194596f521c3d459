"""Writes the full-shape (GPT-J-6B) fixtures of the CPU oracle - float32 arithmetic on the bf16-rounded hashed synthetic
tree (oracle.gptj_oracle.hashed_params), i.e. the reference's jnp.dot(f32, bf16) numerics:

  gptj6b_decode.npz    512-token prompt left-padded to 576, 32 greedy steps: tokens, top-32 / every 50th logit per step
  gptj6b_forward.npz   every-position logits of a 128-token forward (top-32 / every 50th logit per position)
  gptj6b_batch2.npz    two prompts (100 and 128 tokens, padded to 144), 8 greedy steps each
  gptj6b_outlier_forward.npz   the 128-token forward on the same tree after oracle.gptj_oracle.add_outliers (residual
                       channels of +-50 .. +-500 that grow with depth, LayerNorm scales up to 30, an entry of 4 in a k matrix)

Greedy runs look for a prompt whose every greedy choice is decided by a clear margin (a near-tie would make the stream,
and all logits after it, depend on rounding): the prefill is shared and only the last prompt token is varied.  The
top-1/top-2 margin of every step is stored, so a test knows up to which step a free-running stream is decided.
Needs ~45 GB of host memory and a quarter of an hour on 8 cores; run from the repository root:
    python tests/golden/make_golden_6b.py [decode] [forward] [batch2] [outlier]"""
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import gptj_oracle as O   # noqa: E402

CFG_6B = dict(layers=28, d_model=4096, n_heads=16, n_vocab=50400, norm="layernorm", pe="rotary", pe_rotary_dims=64,
              seq=2048, cores_per_replica=1)
SEED, TOPK, STRIDE, MIN_MARGIN = 6, 32, 50, 0.03
OUT = os.path.join(ROOT, "tests", "golden")
T0 = time.time()


def log(*a):
    print(f"[{time.time() - T0:7.1f}s]", *a, flush=True)


def summary(lg):
    """lg [R, V] float32 -> the stored subset: top-32 ids/values and every 50th logit of each row, and checksums"""
    lg = np.asarray(lg, np.float32)
    order = np.argsort(-lg, axis=-1, kind="stable")[:, :TOPK]
    return dict(top_ids=order.astype(np.int32), top_logits=np.take_along_axis(lg, order, -1),
                strided_logits=lg[:, ::STRIDE].copy(), stride=STRIDE,
                logit_sum=lg.astype(np.float64).sum(-1), logit_abs_sum=np.abs(lg.astype(np.float64)).sum(-1))


def greedy_with_margin(model, ctx, length, G, candidates):
    """Prefill ctx[:-1] once, then try last tokens until all G greedy choices have a margin >= MIN_MARGIN.
    Returns (clear_steps, last_token, run) of the best candidate; run(last, False) completes it whatever the margins:
    (tokens [G], logits [G, V], margins [G])."""
    _, states0 = model.generate_initial(ctx, length)

    def run(last, stop_at_tie):
        states = [dict(s) for s in states0]
        nxt = np.asarray([last], np.uint32)
        toks, rows, margins = [], [], []
        for t in range(G):
            logits, states = model.generate_once(nxt, states)
            lg = logits.to(torch.float32).numpy()[0]
            top2 = np.partition(lg, -2)[-2:]
            margin = float(top2[1] - top2[0])
            if stop_at_tie and margin < MIN_MARGIN:
                break
            tok = int(np.argmax(lg))
            toks.append(tok)
            rows.append(lg)
            margins.append(margin)
            nxt = np.asarray([tok], np.uint32)
        return np.asarray(toks, np.int64), rows, np.asarray(margins)

    best, best_len = None, -1
    for last in candidates:
        toks, _, _ = run(last, True)
        if len(toks) > best_len:
            best, best_len = int(last), len(toks)
        if best_len == G:
            break
    return best_len, best, run


def greedy_fixture(model, make_ctx, length, G, seeds, n_last=4):
    """Searches prompts (make_ctx(seed) -> ctx [L]) and last tokens for a greedy run of G steps in which every choice is
    decided by MIN_MARGIN; if there is none, the run with the longest clear prefix is used and the stored margins say
    how far a free-running stream is decided.  Returns (ctx, tokens, logits, margins)."""
    best = (-1, None, None, None)
    for seed in seeds:
        ctx = make_ctx(seed)
        cands = [int(c) for c in O.seeded_prompt(1000 + seed, 1, n_last)[0]]
        n, last, run = greedy_with_margin(model, ctx, length, G, cands)
        log(f"  prompt seed {seed}: last token {last} is clear for {n} of {G} steps")
        if n > best[0]:
            best = (n, ctx.copy(), last, run)
        if n == G:
            break
    n, ctx, last, run = best
    # run() closes over the prefill of the LAST prompt tried: redo the prefill when the best one is an earlier prompt
    if not np.array_equal(ctx, make_ctx(seed)):
        _, last2, run = greedy_with_margin(model, ctx, length, G, [last])
    ctx[-1] = last
    toks, rows, margins = run(last, False)
    return ctx, toks, np.stack(rows), margins


def make_decode(model):
    P, L, G = 512, 576, 32
    ctx, toks, lg, margins = greedy_fixture(model, lambda s: O.left_pad(O.seeded_prompt(s, 1, P), L)[0], P, G, range(7, 47))
    log("decode tokens", toks.tolist(), "margins", np.round(margins, 4).tolist())
    np.savez_compressed(os.path.join(OUT, "gptj6b_decode.npz"), seed=SEED, ctx=ctx[None].astype(np.uint32),
                        ctx_length=np.asarray([P]), tokens=toks, margins=margins, **summary(lg))


def make_forward(model):
    T = 128
    prompt = O.seeded_prompt(5, 1, T)[0]
    lg = model.forward(prompt).to(torch.float32).numpy()
    log("forward logits", lg.shape, "std", float(lg.std()))
    # evaluation quantities of ProjectionShard.loss (layers.py:569-593) for the next-token targets: the last target is
    # the argmax of the last row, every fourth other target is replaced by the row's argmax so that `correct` has
    # both outcomes
    target = np.concatenate([prompt[1:], lg[-1:].argmax(-1)]).astype(np.int64)
    target[::4] = lg[::4].argmax(-1)
    l64 = lg.astype(np.float64)
    mx = l64.max(-1)
    tl = l64[np.arange(T), target]
    all_loss = np.log(np.exp(l64 - mx[:, None]).sum(-1)) - (tl - mx)
    srt = np.sort(l64, -1)
    target_margin = np.where(tl == mx, srt[:, -1] - srt[:, -2], mx - tl)
    np.savez_compressed(os.path.join(OUT, "gptj6b_forward.npz"), seed=SEED, ctx=prompt[None].astype(np.uint32),
                        target=target[None].astype(np.uint32), all_loss=all_loss, correct=(tl == mx),
                        target_margin=target_margin, **summary(lg))


def make_outlier_forward(model):
    T = 128
    prompt = O.seeded_prompt(5, 1, T)[0]
    taps = []
    lg = model.forward(prompt, taps).to(torch.float32).numpy()
    log("outlier forward logits", lg.shape, "std", float(lg.std()), "absmax", float(np.abs(lg).max()),
        "residual absmax per layer", [round(float(t.abs().max())) for t in taps])
    np.savez_compressed(os.path.join(OUT, "gptj6b_outlier_forward.npz"), seed=SEED, ctx=prompt[None].astype(np.uint32),
                        resid_absmax=np.asarray([float(t.abs().max()) for t in taps]), **summary(lg))


def make_batch2(model):
    lens, L, G = [100, 128], 144, 8
    ctxs, toks, rows, margins = [], [], [], []
    for b, n in enumerate(lens):
        def make_ctx(seed, n=n):
            c = np.zeros(L, np.uint32)
            c[L - n:] = O.seeded_prompt(seed, 1, n)[0]
            return c
        ctx, tk, lg, mg = greedy_fixture(model, make_ctx, n, G, range(20 + 10 * b, 30 + 10 * b))
        ctxs.append(ctx)
        toks.append(tk)
        rows.append(lg)
        margins.append(mg)
        log("batch2 row", b, "tokens", tk.tolist(), "margins", np.round(mg, 4).tolist())
    s = [summary(r) for r in rows]
    np.savez_compressed(os.path.join(OUT, "gptj6b_batch2.npz"), seed=SEED, ctx=np.stack(ctxs), ctx_length=np.asarray(lens),
                        tokens=np.stack(toks), margins=np.stack(margins), stride=STRIDE,
                        **{k: np.stack([x[k] for x in s]) for k in s[0] if k != "stride"})


def main():
    what = sys.argv[1:] or ["decode", "forward", "batch2", "outlier"]
    if "outlier" in what:
        tree = O.add_outliers(O.hashed_params(CFG_6B, SEED, torch.bfloat16), CFG_6B)
        log("outlier tree built")
        model = O.Model(CFG_6B, tree, torch.float32)
        del tree
        with torch.no_grad():
            make_outlier_forward(model)
        del model
        if what == ["outlier"]:
            log("done")
            return
    tree = O.hashed_params(CFG_6B, SEED, torch.bfloat16)
    log("tree built")
    model = O.Model(CFG_6B, tree, torch.float32)
    del tree
    log("model in float32")
    with torch.no_grad():
        if "forward" in what:
            make_forward(model)
        if "batch2" in what:
            make_batch2(model)
        if "decode" in what:
            make_decode(model)
    log("done")


if __name__ == "__main__":
    torch.set_num_threads(os.cpu_count() or 8)
    main()

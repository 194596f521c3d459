"""Host side of the zero-shot evaluation (tasks/eval_harness.py, tasks/util.py, TPU_cluster.eval): request -> row
conversion, batching, sequence shrinking and the masked reduction, on hand-derived cases; then the whole adaptor on a
real MI355X against the float64 oracle."""
import numpy as np
import pytest
import torch

from mesh_transformer import eval_harness as E


class WordTokenizer:
    """'<|endoftext|>' -> 50256, every other blank-separated word w -> its number (words are decimal numbers)"""

    def encode(self, s):
        s = s.replace("<|endoftext|>", " 50256 ")
        return [int(w) for w in s.split()]


TOK = WordTokenizer()


def test_process_request_rows_and_mask():
    r = E.process_request(("11 12 13", " 14 15"), 8, TOK)
    # tokens: 50256 11 12 13 | 14 15 -> obs is all but the last, target all but the first, right-padded with 50256
    assert r["obs"].tolist() == [50256, 11, 12, 13, 14, 50256, 50256, 50256]
    assert r["target"].tolist() == [11, 12, 13, 14, 15, 50256, 50256, 50256]
    assert r["eval_mask"].tolist() == [False, False, False, True, True, False, False, False]   # targets 14 and 15
    assert r["ctx_length"] == 8
    # seq shorter than the request: only the last seq tokens survive (12 13 14 15), the mask moves with them
    r = E.process_request(("11 12 13", " 14 15"), 4, TOK)
    assert r["obs"].tolist() == [12, 13, 14, 50256]
    assert r["target"].tolist() == [13, 14, 15, 50256]
    assert r["eval_mask"].tolist() == [False, True, True, False]
    # a continuation of one token directly after the end-of-text token
    r = E.process_request(("", "7"), 4, TOK)
    assert r["obs"].tolist() == [50256, 50256, 50256, 50256] and r["target"].tolist() == [7, 50256, 50256, 50256]
    assert r["eval_mask"].tolist() == [True, False, False, False]


def test_shrink_seq_halves_while_the_mask_fits():
    def batch(length, last):
        m = np.zeros((2, length), bool)
        m[0, last] = True
        return {"obs": np.arange(2 * length).reshape(2, length), "target": np.ones((2, length), int), "eval_mask": m,
                "ctx_length": np.array([length, length])}
    b = E.shrink_seq(batch(16, 4))             # last masked index 4: 16 -> 8 (5 < 8), not 4 (5 >= 4)
    assert b["obs"].shape == (2, 8) and b["target"].shape == (2, 8) and b["eval_mask"].shape == (2, 8)
    assert b["obs"][1].tolist() == list(range(16, 24))
    assert E.shrink_seq(batch(16, 4), min_seq=16)["obs"].shape == (2, 16)
    assert E.shrink_seq(batch(16, 4), min_seq=8)["obs"].shape == (2, 8)
    assert E.shrink_seq(batch(16, 7))["obs"].shape == (2, 16)           # 8 >= 8: nothing may be cut
    assert E.shrink_seq(batch(16, 0))["obs"].shape == (2, 2)            # 16 -> 8 -> 4 -> 2, then 1 >= 1 stops
    assert b["ctx_length"].tolist() == [16, 16]                          # untouched, as in the reference


def test_sample_batch_fills_the_last_batch_with_empty_rows():
    rows = [E.process_request((f"{i}", " 5"), 6, TOK) for i in range(5)]
    got = list(E.sample_batch(iter(rows), 2, rows[0]))
    assert len(got) == 3
    assert all(b["obs"].shape == (2, 6) and b["eval_mask"].shape == (2, 6) for b in got)
    assert got[0]["obs"][1].tolist() == rows[1]["obs"].tolist()
    last = got[2]
    assert last["ctx_length"].tolist() == [6, 0]
    assert not last["eval_mask"][1].any() and not last["obs"][1].any() and not last["target"][1].any()
    assert list(E.sample_batch(iter([]), 2, rows[0])) == []


class FixedNet:
    def __init__(self, all_loss, correct):
        self.all_loss, self.correct = np.asarray(all_loss, float), np.asarray(correct, bool)
        self.seen = []

    def eval(self, sample):
        assert "eval_mask" not in sample
        self.seen.append(sample)
        return {"all_loss": self.all_loss, "correct": self.correct, "last_loss": self.all_loss[:, -1],
                "loss": self.all_loss.mean(-1)}


def test_masked_eval_reduction():
    net = FixedNet([[1, 2, 4, 8], [1, 2, 4, 8], [1, 2, 4, 8]], [[1, 1, 0, 1], [1, 1, 0, 1], [0, 0, 0, 0]])
    mask = np.array([[0, 1, 0, 1], [0, 1, 1, 0], [0, 0, 0, 0]], bool)
    out = E.masked_eval(net, {"obs": np.zeros((3, 4), int), "target": np.zeros((3, 4), int), "eval_mask": mask,
                              "ctx_length": np.array([4, 4, 0])})
    assert out["mask_loss"].tolist() == [10.0, 6.0, 0.0]
    assert out["each_correct"].tolist() == [True, False, False]       # row 1 misses position 2, row 2 has no mask
    assert out["total"] == 2 and out["correct"] == 1
    assert out["last_correct"] == 1                                   # only row 0 has its last position masked and right
    assert out["last_loss"] == 16.0                                   # last_loss of the rows with a mask


def test_adaptor_with_a_stub_network_keeps_request_order_and_length():
    class Echo:
        """loss of position i = target token / 100; correct where the target is even"""

        def eval(self, s):
            t = np.asarray(s["target"], float)
            return {"all_loss": t / 100, "correct": t % 2 == 0, "last_loss": t[:, -1] / 100, "loss": t.mean(-1) / 100}
    ad = E.EvalHarnessAdaptor(Echo(), seq=8, batch=2, shrink=True, tokenizer=TOK)
    reqs = [("1 3", " 2 4"), ("1", " 6 7"), ("9 9 9", " 8")]
    got = ad.loglikelihood(reqs)
    assert len(got) == 3
    assert got[0] == (pytest.approx(-0.06), True)
    assert got[1] == (pytest.approx(-0.13), False)
    assert got[2] == (pytest.approx(-0.08), True)
    assert ad.loglikelihood([]) == []
    with pytest.raises(Exception):
        ad.greedy_until(reqs)
    with pytest.raises(Exception):
        ad.loglikelihood_rolling(reqs)
    with pytest.raises(ValueError):
        E.EvalHarnessAdaptor(Echo(), 8, 2, False)


@pytest.mark.gpu
def test_loglikelihood_on_the_gpu_against_the_oracle():
    """Five requests in batches of two (one filler row), rows shrunk from 64 to 16 positions: every log-likelihood
    within 1e-4 relative of the float64 oracle's and the same greedy flags; request 4's continuation is built from
    the oracle's own best tokens, so at least one flag is set."""
    from oracle import gptj_oracle as O
    from mesh_transformer import sampling
    from mesh_transformer.transformer_shard import CausalTransformer
    cfg = dict(layers=2, d_model=512, n_heads=8, n_vocab=50400, norm="layernorm", pe="rotary", pe_rotary_dims=32,
               seq=64, cores_per_replica=1)
    params = O.seeded_params(cfg, 3)
    m = O.Model(cfg, params, torch.float64)
    rng = np.random.default_rng(5)
    words = lambda n: " ".join(str(int(t)) for t in rng.integers(0, 50000, n))
    reqs = [(words(5), " " + words(3)), (words(9), " " + words(1)), (words(2), " " + words(4)), (words(7), " " + words(2))]
    ctx = words(6)
    toks = [50256] + [int(w) for w in ctx.split()]
    best = []
    for _ in range(2):                              # the oracle's greedy continuation of ctx
        best.append(int(m.forward(np.asarray(toks + best, np.uint32))[-1].argmax()))
    reqs.append((ctx, " " + " ".join(map(str, best))))
    net = CausalTransformer(dict(cfg, sampler=sampling.greedy_sample), params)
    got = E.EvalHarnessAdaptor(net, seq=64, batch=2, shrink=True, min_seq=16, tokenizer=TOK).loglikelihood(reqs)
    assert len(got) == len(reqs)
    for (c, k), (ll, ok) in zip(reqs, got):
        t = np.asarray(TOK.encode("<|endoftext|>" + c) + TOK.encode(k), np.uint32)
        n_cont = len(TOK.encode(k))
        logp = torch.log_softmax(m.forward(t[:-1]).double(), -1)
        pos = np.arange(len(t) - 1 - n_cont, len(t) - 1)
        want = float(logp[pos, t[1:][pos].astype(np.int64)].sum())
        assert abs(ll - want) < 1e-4 * abs(want), (c, k, ll, want)
        assert ok == bool((logp[pos].argmax(-1).numpy() == t[1:][pos]).all())
    assert got[-1][1] is True

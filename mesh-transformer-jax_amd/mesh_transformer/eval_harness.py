"""Zero-shot evaluation through CausalTransformer.eval: the host side of tasks/eval_harness.py:14-88, tasks/util.py:12-63
and the per-example bookkeeping of TPU_cluster.eval (TPU_cluster.py:66-115), for one device.

A request is a (context, continuation) pair of strings.  It becomes one row {obs, target, eval_mask, ctx_length}: the
tokens of "<|endoftext|>" + context followed by those of the continuation, cut to the last `seq` + 1 tokens, obs = all but
the last, target = all but the first, both padded on the RIGHT with token 50256, and eval_mask marking the positions
whose target is a continuation token.  Rows are batched (short batches are filled with all-zero rows whose mask is
empty), optionally halved in length while no masked position is lost, evaluated, and reduced per row to
(-sum of the masked losses, every masked target is the model's best token).

Nothing here needs lm_eval: EvalHarnessAdaptor has the three methods that library calls on a model, and any object with
`encode(str) -> list[int]` serves as the tokenizer (GPT2TokenizerFast loaded from a local directory in practice).
ftfy's fix_text is applied to both strings when that package is importable, as the reference does."""
import itertools

import numpy as np

PAD_TOKEN = 50256          # "<|endoftext|>", also the reference's padding value (tasks/eval_harness.py:41-42)

try:                       # tasks/eval_harness.py:30-31
    from ftfy import fix_text as _fix_text

    def _normalise(s):
        return _fix_text(s, normalization="NFKC")
except ImportError:        # the strings are used as they come
    def _normalise(s):
        return s


def process_request(request, seq, tokenizer):
    """tasks/eval_harness.py:25-49 for one (context, continuation) pair."""
    ctx, cont = request
    ctx_tokens = list(tokenizer.encode("<|endoftext|>" + _normalise(ctx)))
    cont_tokens = list(tokenizer.encode(_normalise(cont)))
    tokens = np.asarray(ctx_tokens + cont_tokens, dtype=np.int64)[-seq:]
    n = len(tokens)
    pad = seq - (n - 1)
    where = np.arange(seq)
    return {
        "obs": np.pad(tokens[:-1], (0, pad), constant_values=PAD_TOKEN),
        "target": np.pad(tokens[1:], (0, pad), constant_values=PAD_TOKEN),
        "ctx_length": seq,
        # target position i holds token i + 1: the continuation starts at token n - len(cont)
        "eval_mask": (where > n - len(cont_tokens) - 2) & (where < n - 1),
    }


def shrink_seq(examples, min_seq=None):
    """tasks/util.py:12-33: halves the row length as long as every masked position stays inside (and, with min_seq,
    the length stays at least min_seq).  Works on the batch dictionary in place and returns it."""
    while True:
        length = examples["obs"].shape[-1]
        half = length // 2
        if min_seq is not None and half < min_seq:
            return examples
        last_masked = int(np.max(examples["eval_mask"] * np.arange(length))) + 1
        if last_masked >= half:
            return examples
        for k in ("obs", "target", "eval_mask"):
            examples[k] = examples[k][:, :half]


def sample_batch(examples, bs, like):
    """tasks/util.py:36-63: groups rows into batches of bs; the last batch is filled with all-zero rows shaped like
    `like`, whose ctx_length is 0 and whose mask selects nothing."""
    filler = {"obs": np.zeros_like(like["obs"]), "target": np.zeros_like(like["target"]),
              "eval_mask": np.zeros_like(like["eval_mask"]), "ctx_length": 0}
    it = iter(examples)
    while True:
        rows = list(itertools.islice(it, bs))
        if not rows:
            return
        rows += [filler] * (bs - len(rows))
        yield {k: np.array([r[k] for r in rows]) for k in ("obs", "target", "eval_mask", "ctx_length")}


def masked_eval(network, batch):
    """TPU_cluster.eval (TPU_cluster.py:66-115) for a single device: runs network.eval on the batch and reduces it with
    batch["eval_mask"].  A row counts as correct when it has masked positions and the target is the best token at
    every one of them."""
    out = network.eval({k: v for k, v in batch.items() if k != "eval_mask"})
    mask = np.asarray(batch["eval_mask"], dtype=bool)
    hit = np.logical_and(out["correct"], mask)
    n_valid, n_hit = mask.sum(-1), hit.sum(-1)
    valid = n_valid > 0
    each_correct = np.logical_and(valid, n_hit == n_valid)
    return {
        "total": int(valid.sum()),
        "correct": int(each_correct.sum()),
        "last_correct": int(hit[:, -1].sum()),
        "last_loss": float((valid * out["last_loss"]).sum()),
        "mask_loss": (out["all_loss"] * mask).sum(-1),
        "each_correct": each_correct,
    }


class EvalHarnessAdaptor:
    """tasks/eval_harness.py:52-88 with the same constructor arguments; `tpu_cluster` is anything with
    eval(batch) -> {"mask_loss", "each_correct"} - a CausalTransformer is wrapped with masked_eval."""

    def __init__(self, tpu_cluster, seq, batch, shrink, min_seq=None, tokenizer=None):
        if tokenizer is None:
            raise ValueError("pass tokenizer=: an object with encode(str) -> token ids (e.g. GPT2TokenizerFast loaded "
                             "from a local directory)")
        self.tpu = tpu_cluster
        self.seq = seq
        self.batch = batch
        self.shrink = shrink
        self.min_seq = min_seq
        self.tokenizer = tokenizer

    def greedy_until(self, requests):
        raise Exception("unimplemented")

    def loglikelihood_rolling(self, requests):
        raise Exception("unimplemented")

    def convert_requests(self, requests):
        return (process_request(r, self.seq, self.tokenizer) for r in requests)

    def _eval(self, b):
        out = self.tpu.eval(b)
        if "mask_loss" not in out:                  # a bare network: do the cluster's reduction here
            out = masked_eval(_Evaluated(out), b)
        return out

    def loglikelihood(self, requests):
        """[(log-likelihood of the continuation, it is the greedy continuation)] in request order."""
        requests = list(requests)
        if not requests:
            return []
        like = process_request(requests[0], self.seq, self.tokenizer)
        output = []
        for b in sample_batch(self.convert_requests(requests), self.batch, like):
            if self.shrink:
                b = shrink_seq(b, min_seq=self.min_seq)
            out = self._eval(b)
            output += [(float(-loss), bool(ok)) for loss, ok in zip(out["mask_loss"], out["each_correct"])]
        return output[:len(requests)]


class _Evaluated:
    """hands an already computed eval result to masked_eval"""

    def __init__(self, out):
        self.out = out

    def eval(self, _):
        return self.out

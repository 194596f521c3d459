"""Host-side glue of the reference's inference callers, without their web framework and tokenizer download:
the padding convention of device_sample.py:92-96 / device_serve.py:166-181 and the batching loop of
device_serve.py:138-194 (collect pending requests, fill the batch with dummy requests, one generate call with
per-request top_p / temp, route each completion back to its requester).

Text handling is pluggable: `encode(str) -> list[int]` and `decode(array) -> str` (e.g. the methods of a locally
available GPT-2 tokenizer).  Without them requests carry token ids and completions are uint32 arrays.
"""
import queue
import time

import numpy as np


def pad_context(tokens, seq):
    """device_sample.py:92-96, device_serve.py:172-179: left-pad the token ids with zeros to `seq`; a longer prompt
    keeps its last `seq` tokens.  Returns (uint32 [seq], length) with length clamped to seq (the reference passes
    the unclamped length on)."""
    tokens = np.asarray(tokens, np.int64).reshape(-1)
    pad_amount = max(seq - len(tokens), 0)
    padded = np.pad(tokens, ((pad_amount, 0),)).astype(np.uint32)[-seq:]
    return padded, min(len(tokens), seq)


def infer(network, tokens, gen_len=512, top_p=0.9, temp=1.0, top_k=None, seq=None, decode=None):
    """One completion for one prompt (resharding_example.py:55-75, device_sample.py:86-103)."""
    seq = seq or network.config["seq"]
    padded, length = pad_context(tokens, seq)
    opts = {"top_p": np.ones(1) * top_p, "temp": np.ones(1) * temp}
    if top_k is not None:
        opts["top_k"] = np.ones(1, np.uint32) * top_k
    output = network.generate(padded[None, :], np.ones(1, np.uint32) * length, gen_len, opts)
    completion = np.asarray(output[1][0][0, :, 0])
    return decode(completion) if decode else completion


class BatchingLoop:
    """device_serve.py:138-194.  `submit` is what the request handler does (:54-64); `step` is one turn of the
    consumer loop; `serve_forever` repeats it."""

    DUMMY = "whatever"     # the context of the requests that fill a partial batch (device_serve.py:160)

    def __init__(self, network, seq, total_batch, gen_length=256, encode=None, decode=None, poll_s=0.01):
        self.network, self.seq, self.total_batch, self.gen_length = network, seq, total_batch, gen_length
        self.encode, self.decode, self.poll_s = encode, decode, poll_s
        self.requests_queue = queue.Queue()

    def submit(self, context, top_p, temp):
        """Queue a request; the completion arrives on the returned queue."""
        response_queue = queue.Queue()
        self.requests_queue.put(({"context": context, "top_p": float(top_p), "temp": float(temp)}, response_queue))
        return response_queue

    def _tokens(self, ctx):
        if isinstance(ctx, str):
            return self.encode(ctx) if self.encode else [0]
        return ctx

    def step(self, block=True):
        """Serve up to total_batch pending requests with one generate call; returns how many were served."""
        all_ctx, all_top_p, all_temp, all_q = [], [], [], []
        while len(all_ctx) < self.total_batch:
            try:
                o, q = self.requests_queue.get(block=False)
                all_ctx.append(o["context"])
                all_top_p.append(o["top_p"])
                all_temp.append(o["temp"])
                all_q.append(q)
            except queue.Empty:
                if len(all_ctx) or not block:
                    break
                time.sleep(self.poll_s)
        if not all_ctx:
            return 0
        while len(all_ctx) < self.total_batch:          # fill the batch with dummy requests (:159-162)
            all_ctx.append(self.DUMMY)
            all_top_p.append(1)
            all_temp.append(1)
        all_tokenized, all_length = [], []
        for ctx in all_ctx:
            padded_tokens, length = np.zeros(self.seq, np.uint32), 1
            try:
                padded_tokens, length = pad_context(self._tokens(ctx), self.seq)
                length = max(length, 1)
            except Exception:                            # device_serve.py:180-181: a bad request must not stop the loop
                print("oops exception")
            all_tokenized.append(padded_tokens)
            all_length.append(length)
        output = self.network.generate(np.array(all_tokenized), np.array(all_length), self.gen_length,
                                       {"top_p": np.array(all_top_p, np.float64), "temp": np.array(all_temp, np.float64)})
        for o, q in zip(np.asarray(output[1][0])[:, :, 0], all_q):
            q.put(self.decode(o) if self.decode else o)
        return len(all_q)

    def serve_forever(self):
        while True:
            self.step()

"""Host-side glue of the reference's inference callers, without their web framework and tokenizer download:
the padding convention of device_sample.py:92-96 / device_serve.py:166-181 and the batching loop of
device_serve.py:138-194 (collect pending requests, fill the batch with dummy requests, one generate call with
per-request top_p / temp, route each completion back to its requester).

Text handling is pluggable: `encode(str) -> list[int]` and `decode(array) -> str` (e.g. the methods of a locally
available GPT-2 tokenizer).  Without them requests carry token ids and completions are uint32 arrays.
"""
import logging
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


class _Pending:
    """One queued request and the queue its completion goes to."""
    __slots__ = ("prompt", "top_p", "temp", "reply")

    def __init__(self, prompt, top_p, temp):
        self.prompt, self.top_p, self.temp = prompt, float(top_p), float(temp)
        self.reply = queue.Queue(maxsize=1)


class BatchingLoop:
    """The consumer side of the reference's serving script (device_serve.py:138-194) around one generate() call per
    turn: the batch has a fixed size (the compiled shape there, the recorded HIP graphs here), rows that no request
    claims run a one-token filler prompt with top_p = temp = 1, every request carries its own top_p / temp, and a
    request whose prompt cannot be turned into tokens is answered from an empty prompt instead of stopping the loop.
    `submit` is what a request handler calls (device_serve.py:54-64); `step` serves one batch; `serve_forever` repeats."""

    def __init__(self, network, seq, total_batch, gen_length=256, encode=None, decode=None, poll_s=0.01, filler=(0,)):
        self.network, self.seq, self.total_batch, self.gen_length = network, seq, total_batch, gen_length
        self.encode, self.decode, self.poll_s = encode, decode, poll_s
        self.filler = np.asarray(filler, np.int64)
        self.pending = queue.Queue()

    def submit(self, context, top_p, temp):
        """Queue a request (text, or token ids); its completion arrives on the returned queue."""
        req = _Pending(context, top_p, temp)
        self.pending.put(req)
        return req.reply

    def _take(self, block):
        """Up to total_batch requests, oldest first; waits for the first one when `block`, never for the rest."""
        batch = []
        while len(batch) < self.total_batch:
            try:
                batch.append(self.pending.get_nowait())
            except queue.Empty:
                if batch or not block:
                    break
                time.sleep(self.poll_s)
        return batch

    def _row(self, prompt):
        """(padded ids [seq], length) of one prompt; an unusable prompt becomes the empty one."""
        try:
            ids = self.encode(prompt) if isinstance(prompt, str) and self.encode else ([0] if isinstance(prompt, str) else prompt)
            row, n = pad_context(ids, self.seq)
        except Exception as e:                         # device_serve.py:180-181: the loop outlives a bad request
            logging.getLogger(__name__).warning("request dropped to an empty prompt: %r", e)
            row, n = np.zeros(self.seq, np.uint32), 0
        return row, max(n, 1)

    def step(self, block=True):
        """Serve the pending requests (at most total_batch) with one generate call; returns how many were served."""
        batch = self._take(block)
        if not batch:
            return 0
        B = self.total_batch
        ctx = np.zeros((B, self.seq), np.uint32)
        length = np.ones(B, np.int64)
        top_p, temp = np.ones(B), np.ones(B)           # rows without a request: top_p = temp = 1 (device_serve.py:159-162)
        for b in range(B):
            if b < len(batch):
                ctx[b], length[b] = self._row(batch[b].prompt)
                top_p[b], temp[b] = batch[b].top_p, batch[b].temp
            else:
                ctx[b], length[b] = self._row(self.filler)
        out = self.network.generate(ctx, length, self.gen_length, {"top_p": top_p, "temp": temp})
        tokens = np.asarray(out[1][0])[:, :, 0]
        for req, row in zip(batch, tokens):
            req.reply.put(self.decode(row) if self.decode else row)
        return len(batch)

    def serve_forever(self):
        while True:
            self.step()

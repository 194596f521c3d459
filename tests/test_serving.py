"""Host-side caller glue (padding convention, batching loop) against the reference's conventions, on the CPU with a
stand-in network that records what generate() was given."""
import numpy as np

from mesh_transformer import serving


class FakeNetwork:
    config = {"seq": 16}

    def __init__(self):
        self.calls = []

    def generate(self, ctx, ctx_length, gen_length, sampler_options, return_logits=False):
        self.calls.append((np.array(ctx), np.array(ctx_length), gen_length, {k: np.array(v) for k, v in sampler_options.items()}))
        B = ctx.shape[0]
        # completion of row b: its last prompt token, then b, b, ...
        toks = np.zeros((B, gen_length, 1), np.uint32)
        toks[:, 0, 0] = ctx[:, -1]
        toks[:, 1:, 0] = np.arange(B)[:, None]
        return None, (toks, None)


def test_pad_context_follows_the_callers():
    p, n = serving.pad_context([5, 6, 7], 8)
    assert p.dtype == np.uint32 and p.tolist() == [0, 0, 0, 0, 0, 5, 6, 7] and n == 3     # device_sample.py:92-96
    p, n = serving.pad_context(list(range(1, 13)), 8)
    assert p.tolist() == list(range(5, 13)) and n == 8                                     # keeps the last seq tokens
    p, n = serving.pad_context([], 4)
    assert p.tolist() == [0, 0, 0, 0] and n == 0


def test_infer_indexes_the_output_like_the_reference():
    net = FakeNetwork()
    out = serving.infer(net, [3, 4, 9], gen_len=5, top_p=0.8, temp=0.7, top_k=40)
    assert out.tolist() == [9, 0, 0, 0, 0]
    ctx, length, G, opts = net.calls[0]
    assert ctx.shape == (1, 16) and length.tolist() == [3] and G == 5
    assert opts["top_p"].tolist() == [0.8] and opts["temp"].tolist() == [0.7] and opts["top_k"].tolist() == [40]
    assert serving.infer(net, [1], gen_len=2, decode=lambda a: "|".join(map(str, a))) == "1|0"


def test_batching_loop_fills_routes_and_keeps_going():
    net = FakeNetwork()
    loop = serving.BatchingLoop(net, seq=8, total_batch=4, gen_length=3)
    assert loop.step(block=False) == 0 and not net.calls
    q1 = loop.submit([11, 12], 0.9, 0.8)
    q2 = loop.submit([21], 0.5, 1.2)
    assert loop.step() == 2
    ctx, length, G, opts = net.calls[0]
    assert ctx.shape == (4, 8) and G == 3
    assert ctx[0].tolist() == [0] * 6 + [11, 12] and ctx[1].tolist() == [0] * 7 + [21]
    assert length.tolist() == [2, 1, 1, 1]                       # dummy requests hold one token
    assert opts["top_p"].tolist() == [0.9, 0.5, 1, 1] and opts["temp"].tolist() == [0.8, 1.2, 1, 1]
    assert q1.get_nowait().tolist() == [12, 0, 0] and q2.get_nowait().tolist() == [21, 1, 1]
    # more requests than one batch holds: served over two turns, in order
    qs = [loop.submit([30 + i], 1, 1) for i in range(6)]
    assert loop.step() == 4 and loop.step() == 2
    assert [q.get_nowait()[0] for q in qs] == [30, 31, 32, 33, 34, 35]
    # text requests go through encode / decode; a request that cannot be encoded does not stop the loop
    def enc(s):
        if s == "bad":
            raise ValueError
        return [ord(c) for c in s]
    loop2 = serving.BatchingLoop(net, seq=8, total_batch=2, gen_length=2, encode=enc, decode=lambda a: chr(int(a[0])))
    qa, qb = loop2.submit("hi", 1, 1), loop2.submit("bad", 1, 1)
    assert loop2.step() == 2
    assert qa.get_nowait() == "i" and qb.get_nowait() == chr(0)

"""CausalTransformer with the call surface of the reference's mesh_transformer/transformer_shard.py
(constructor from a config dict, .state["params"] in the haiku tree layout, .generate(...)), running
on one MI355X through the HIP kernels.  Only the generate path exists here: train/eval/init_xmap,
the xmap/pjit sharding and the optimizer state are not part of this build.
"""
import random
import time

import numpy as np
import torch

from . import _abi, sampling
from .engine import ROOT, Engine


def _init_tree(config, device, seed=42):
    """Random-init parameter tree with haiku's shapes, names and initialisers
    (transformer_shard.py:175-188, layers.py:180-185,249-258,559): hk.Linear weights are
    TruncatedNormal(1/sqrt(fan_in)), out / fc_out use init_scale/sqrt(d_model) with
    init_scale = 2/layers (transformer_shard.py:35), biases 0, LayerNorm scale 1 / offset 0.
    "early_cast" in the config gives bfloat16 leaves (transformer_shard.py:185)."""
    d, V, n = config["d_model"], config["n_vocab"], config["layers"]
    F = 4 * d
    dt = torch.bfloat16 if "early_cast" in config else torch.float32
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)

    def tn(shape, std):
        t = torch.empty(shape, dtype=torch.float32, device=device)
        torch.nn.init.trunc_normal_(t, 0.0, std, -2 * std, 2 * std, generator=gen)
        return t.to(dt)

    zeros = lambda *s: torch.zeros(*s, dtype=dt, device=device)
    ones = lambda *s: torch.ones(*s, dtype=dt, device=device)
    tree = {ROOT + "embedding_shard/~/linear": {"w": tn((1, V, d), V ** -0.5), "b": zeros(1, d)}}
    o_std = (2.0 / n) / d ** 0.5
    for i in range(n):
        p = f"{ROOT}layer_{i}/~/"
        tree[p + "replicated_layer_norm"] = {"scale": ones(1, d), "offset": zeros(1, d)}
        tree[p + "linear"] = {"w": tn((1, d, d), d ** -0.5)}       # q
        tree[p + "linear_1"] = {"w": tn((1, d, d), d ** -0.5)}     # v
        tree[p + "linear_2"] = {"w": tn((1, d, d), d ** -0.5)}     # k
        tree[p + "linear_3"] = {"w": tn((1, d, d), o_std)}         # o
        tree[p + "linear_4"] = {"w": tn((1, d, F), d ** -0.5), "b": zeros(1, F)}
        tree[p + "linear_5"] = {"w": tn((1, F, d), o_std), "b": zeros(1, d)}
    tree[ROOT + "projection_shard/~/replicated_layer_norm"] = {"scale": ones(1, d), "offset": zeros(1, d)}
    tree[ROOT + "projection_shard/~/linear"] = {"w": tn((1, d, V), d ** -0.5), "b": zeros(1, V)}
    return tree


def _to_device_tree(tree, device):
    out = {}
    for mod, leaves in tree.items():
        out[mod] = {k: torch.as_tensor(v).to(device) for k, v in leaves.items()}
    return out


class DecodeStates:
    """The per-layer decode state that the reference's scan carries out of generate (transformer_shard.py:196-212,
    layers.py:340-344): a sequence over the layers of {"k", "v": [B, T, H, dh], "tokens_decoded": uint32 [B]} with the
    window in the reference's order (oldest slot first, the newest token last) and K NOT rotated.

    The engine keeps K rotated at absolute positions in a ring, so an entry is computed (copied out of the ring,
    rotated back) only when it is indexed; nothing is handed out that aliases the engine's memory.  Slots that still
    hold left padding are zero (the reference keeps the projections of its pad tokens there, which no real token can
    see).  Reading an entry after a later generate call on the same geometry raises: the window has moved on."""

    def __init__(self, eng, ses, tokens_decoded):
        self._eng, self._ses, self._epoch = eng, ses, ses.epoch
        self._n = np.asarray(tokens_decoded).astype(np.int64)     # tokens in the window = next position, per sequence

    def __len__(self):
        return len(self._eng.w.layer_ids)

    def __iter__(self):
        return (self[i] for i in range(len(self)))

    def __getitem__(self, layer):
        eng, ses = self._eng, self._ses
        if ses.epoch != self._epoch:
            raise RuntimeError("this decode state belongs to an earlier generate call; the K/V window has been reused")
        i = eng.w.layer_ids[layer]
        T, dev, r = ses.Tcap, eng.device, eng.r
        with torch.cuda.device(dev):
            n = torch.from_numpy(self._n).to(dev)                                   # [B]
            p = n[:, None] - T + torch.arange(T, device=dev)[None, :]               # position held by window slot j
            real = p >= 0
            slot = torch.where(real, p % T, torch.zeros_like(p))                    # [B, T]
            idx = slot[:, None, :, None].expand(-1, eng.H, -1, eng.dh)
            k = torch.gather(ses.kc[i], 2, idx).float()                             # [B, H, T, dh], rotated
            v = torch.gather(ses.vc[i], 2, idx).float()
            pp = p.clamp(0, ses.max_pos - 1)
            sn, cs = ses.sin[pp][:, None], ses.cos[pp][:, None]                     # [B, 1, T, r/2]
            ke, ko = k[..., 0:r:2].clone(), k[..., 1:r:2].clone()
            k[..., 0:r:2] = ke * cs + ko * sn                                       # the rotation of layers.py:137-148, inverted
            k[..., 1:r:2] = ko * cs - ke * sn
            keep = real[:, None, :, None]
            k, v = (k * keep).permute(0, 2, 1, 3), (v * keep).permute(0, 2, 1, 3)
            return {"k": k.cpu().numpy(), "v": v.cpu().numpy(), "tokens_decoded": self._n.astype(np.uint32)}


class CausalTransformer:
    """Drop-in for transformer_shard.py:118-339 on the generate path.

    config keys read: layers, d_model, n_heads, n_vocab, norm, pe, pe_rotary_dims, cores_per_replica,
    sampler (callable, transformer_shard.py:191), early_cast.  Extra, optional: "device",
    "steps_per_graph" (decode steps recorded into one HIP graph, default 8; 0 disables graphs),
    "fused_decode_attention" (batch-1 decode computes the attention inside the out-projection launch, default True),
    "fused_greedy_sampler" (batch-1 greedy decode takes the argmax inside the logits launch, default True)."""

    def __init__(self, config, params=None):
        self.config = config
        if config.get("cores_per_replica", 1) != 1:       # transformer_shard.py:257 asserts mp == cores_per_replica
            raise ValueError("cores_per_replica must be 1: the model runs unsharded on one GPU")
        if not torch.cuda.is_available():
            raise RuntimeError("CausalTransformer needs an MI355X (HIP device); no GPU is visible")
        _abi.lib()  # fail now, loudly, if the HIP library is not built
        self.device = torch.device(config.get("device", "cuda:0"))
        tree = _init_tree(config, self.device) if params is None else _to_device_tree(params, self.device)
        self.state = {"params": tree, "step": np.array(0)}
        self.gen_length = None
        self.return_logits = False
        self._engine = None
        self._engine_key = None
        n = sum(int(v.numel()) for m in tree.values() for v in m.values())
        print(f"Total parameters: {n}")                  # transformer_shard.py:279-280

    def from_params(self, tree):
        """Replace the parameter tree (haiku names, leading shard axis of 1)."""
        self.state = {"params": _to_device_tree(tree, self.device), "step": np.array(0)}
        return self

    def invalidate(self):
        """Forget the packed weights: the next call packs the current parameter tree again.  Needed only after the
        leaves' memory was written behind torch's back (a raw pointer, another library); assignments to .state and
        in-place tensor updates are noticed without it."""
        self._engine = None
        self._engine_key = None

    def engine(self):
        tree = self.state["params"]
        # a leaf is identified by its memory and by torch's version counter, which every in-place update bumps
        key = tuple((v.data_ptr(), v._version) for m in sorted(tree) for _, v in sorted(tree[m].items()))
        if self._engine is None or key != self._engine_key:
            self._engine = None
            self._engine = Engine(self.config, tree, self.device)
            self._engine_key = key
        return self._engine

    # ------------------------------------------------------------------ generate
    def generate(self, ctx, ctx_length, gen_length, sampler_options, return_logits=False, uniforms=None,
                 sampler=None, return_keep_mask=False, timing=None):
        """transformer_shard.py:326-339.

        ctx uint32 [B, L] left-padded (device_sample.py:92-96), ctx_length [B], sampler_options a dict of
        [B] arrays (top_p, temp, optional top_k).  Returns (final_state, (tokens [B, G, 1] uint32, None
        [, logits [B, G, 1, V] float32])) so that callers' `out[1][0][:, :, 0]` works unchanged.  final_state is the
        scan's last carry (last token [B, 1], a sequence of per-layer {"k", "v", "tokens_decoded"}, None for the key);
        the per-layer entries are built when they are read (see DecodeStates).

        Beyond the reference: `uniforms` float64 [B, G] in [0, 1) drive the inverse-CDF draw (default:
        drawn from an unseeded Philox stream, like the reference's unseeded key at :327);
        `sampler` overrides config["sampler"]; `timing`, a dict with key "warmup" (decode steps left out of
        the timed region), is filled with device-synchronised wall times: prefill_s, warmup_s, decode_s,
        decode_steps."""
        eng = self.engine()
        self.gen_length, self.return_logits = gen_length, return_logits
        ctx = np.ascontiguousarray(np.asarray(ctx)).astype(np.int64)
        if ctx.ndim != 2:
            raise ValueError("ctx must be [batch, length]")
        B, Lc = ctx.shape
        P = np.asarray(ctx_length).astype(np.int64).reshape(-1)
        if P.shape[0] != B:
            raise ValueError("ctx_length must have one entry per sequence")
        if Lc < 2 or P.min() < 1 or P.max() > Lc:
            raise ValueError("need ctx length >= 2 and 1 <= ctx_length <= ctx length")
        G = int(gen_length)
        if G < 1:
            raise ValueError("gen_length must be positive")
        Tcap = Lc - 1                                    # K/V window = prefill length (layers.py:325-326)
        Tp = int(P.max()) - 1                            # real prompt tokens that go through prefill
        max_pos = int(P.max()) + G + 1
        sampler = sampler if sampler is not None else self.config.get("sampler", sampling.nucleaus_sample)
        kind = sampling.builtin_kind(sampler)

        dev = self.device
        with torch.cuda.device(dev):
            ses = eng.session(B, Tcap, Tp, max_pos)
            if ses.max_pos < max_pos:                   # the kernels would rotate later positions with the last table row
                raise RuntimeError("rotary tables are shorter than prompt + generated tokens")
            self._ensure_io(ses, G, eng.w.V)
            # --- inputs
            ses.pos0.copy_(torch.from_numpy((-(Tp - (P - 1))).astype(np.int32)))
            ses.pos.copy_(torch.from_numpy((P - 1).astype(np.int32)))
            ses.pos_start.copy_(ses.pos)
            ses.tok.copy_(torch.from_numpy(ctx[:, -1].astype(np.int32)))
            ses.out_tokens.zero_()
            opts = dict(sampler_options or {})
            if kind in ("nucleus", "softmax"):
                # softmax_sample (sampling.py:6-7) is the nucleus kernel with nothing filtered: top_p above 1, no top_k
                tp = np.broadcast_to(np.asarray(opts.get("top_p", 0.9) if kind == "nucleus" else 2.0, np.float64), (B,))
                tm = np.broadcast_to(np.asarray(opts.get("temp", 1.0), np.float64), (B,))
                ses.top_p.copy_(torch.from_numpy(np.array(tp)))
                ses.temp.copy_(torch.from_numpy(np.array(tm)))
                tk = opts.get("top_k", None) if kind == "nucleus" else None
                ses.use_top_k = tk is not None
                if ses.use_top_k:
                    ses.top_k.copy_(torch.from_numpy(np.array(np.broadcast_to(np.asarray(tk, np.int32), (B,)))))
                if uniforms is None:
                    rng = np.random.Generator(np.random.Philox(random.randint(0, 2 ** 60)))
                    uniforms = rng.random((B, G))
                u = np.asarray(uniforms, np.float64)
                if u.shape != (B, G):
                    raise ValueError(f"uniforms must have shape {(B, G)}")
                ses.uniforms[:, :G].copy_(torch.from_numpy(np.ascontiguousarray(u)))
            # --- prefill
            rect = None
            if Tp > 0:
                rect = torch.from_numpy(np.ascontiguousarray(ctx[:, Lc - 1 - Tp:Lc - 1]).astype(np.int32)).to(dev)
            logits_out = torch.empty(B, G, eng.w.V, dtype=torch.float32, device=dev) if return_logits else None
            masks = torch.empty(G, B, eng.w.V, dtype=torch.uint8, device=dev) if return_keep_mask else None   # [step, row, V]

            def clock():
                torch.cuda.synchronize(dev)
                return time.perf_counter()

            t0 = clock() if timing is not None else 0.0
            if Tp > 0:
                eng.prefill(ses, rect, Tp)
            t1 = clock() if timing is not None else 0.0
            # --- decode: the samplers also embed the token they choose, so only the first step needs this
            eng.embed_tok(ses)
            if kind is None:
                self._decode_host_sampler(eng, ses, G, sampler, opts, logits_out)
            elif timing is None:
                self._decode(eng, ses, 0, G, kind, logits_out, masks)
            else:
                W = min(int(timing.get("warmup", 0)), G - 1)
                self._decode(eng, ses, 0, W, kind, logits_out, masks)
                t2 = clock()
                self._decode(eng, ses, W, G, kind, logits_out, masks)
                t3 = clock()
                timing.update(prefill_s=t1 - t0, prefill_tokens=B * Tp, warmup_s=t2 - t1, decode_s=t3 - t2,
                              decode_steps=G - W)
            torch.cuda.synchronize(dev)
            if ses.fused_attn and int(ses.oa_work[8:12].view(torch.int32)[0]) != 0:
                # a fused launch gave up its (time-bounded) wait: this call's tokens are void.  Clear the flag and
                # keep this session on the separate attention launches from now on; the next call works.
                ses.oa_work[8:12].zero_()
                ses.fused_attn = False
                ses.graphs = {}
                torch.cuda.synchronize(dev)
                raise RuntimeError("a fused out-projection launch gave up waiting for its attention partials (not all "
                                   "of its workgroups were resident on the GPU within 5 ms); this call's output is "
                                   "discarded and the session now uses separate attention launches - call generate again")
            toks = ses.out_tokens[:, :G].cpu().numpy().astype(np.uint32)[:, :, None]
            ses.epoch = getattr(ses, "epoch", 0) + 1
            # the scan's final carry (transformer_shard.py:196-212): (last token, per-layer decode state, key)
            final_state = (toks[:, -1], DecodeStates(eng, ses, P - 1 + G), None)
            out = (toks, None)
            if return_logits:
                out = out + (logits_out.cpu().numpy()[:, :, None, :],)
            if return_keep_mask:
                out = out + (masks.permute(1, 0, 2).cpu().numpy().astype(bool),)
            return final_state, out

    # ------------------------------------------------------------------ full forward
    def forward(self, ctx, ctx_length=None, timing=None):
        """Logits at every position: embed -> layers -> ProjectionShard, the composition of
        transformer_shard.py:47-62 without the loss (the full-context prefill with the 50400-wide projection).

        ctx [B, L] token ids, left-padded when ctx_length [B] is given.  Returns a float32 torch tensor
        [B, Tp, V] on the GPU with Tp = max(ctx_length) (= L without padding); row t of sequence b belongs to
        ctx[b, L - Tp + t], rows of padding are zero.  `timing`, a dict, receives forward_s and tokens."""
        eng = self.engine()
        ctx = np.ascontiguousarray(np.asarray(ctx)).astype(np.int64)
        if ctx.ndim != 2:
            raise ValueError("ctx must be [batch, length]")
        B, Lc = ctx.shape
        P = np.full(B, Lc, np.int64) if ctx_length is None else np.asarray(ctx_length).astype(np.int64).reshape(-1)
        if P.shape[0] != B or P.min() < 1 or P.max() > Lc:
            raise ValueError("ctx_length needs one entry per sequence, each in [1, ctx length]")
        Tp = int(P.max())
        dev = self.device
        with torch.cuda.device(dev):
            ses = eng.session(B, Tp, Tp, Tp + 1)
            ses.pos0.copy_(torch.from_numpy((-(Tp - P)).astype(np.int32)))
            rect = torch.from_numpy(np.ascontiguousarray(ctx[:, Lc - Tp:]).astype(np.int32)).to(dev)
            logits = torch.empty(B * Tp, eng.w.V, dtype=torch.float32, device=dev)
            torch.cuda.synchronize(dev)
            t0 = time.perf_counter()
            x = eng.prefill(ses, rect, Tp)
            eng.project(ses, x, logits)
            torch.cuda.synchronize(dev)
            if timing is not None:
                timing.update(forward_s=time.perf_counter() - t0, tokens=int(P.sum()))
            logits = logits.view(B, Tp, eng.w.V)
            if int(P.min()) < Tp:
                pad = torch.arange(Tp, device=dev)[None, :] < torch.from_numpy(Tp - P).to(dev)[:, None]
                logits[pad] = 0.0
            return logits

    # ------------------------------------------------------------------ evaluation
    def eval(self, sample):
        """transformer_shard.py:308-324 with CausalTransformerShard.loss/eval (:47-72, 123-132) and
        ProjectionShard.loss (layers.py:569-593): per-token cross entropy of sample["target"] [B, T] under the model
        run on sample["obs"] [B, T]; keys beyond sample["ctx_length"] [B] (default T) are masked for every query.
        Returns numpy arrays {"loss" [B] (mean over all T positions, as the reference), "last_loss" [B],
        "all_loss" [B, T], "correct" [B, T] (the target holds the maximum logit)}."""
        eng = self.engine()
        obs = np.ascontiguousarray(np.asarray(sample["obs"])).astype(np.int64)
        tgt = np.ascontiguousarray(np.asarray(sample["target"])).astype(np.int64)
        if obs.ndim != 2 or tgt.shape != obs.shape:
            raise ValueError("obs and target must both be [batch, length]")
        B, T = obs.shape
        cl = np.asarray(sample["ctx_length"]).astype(np.int64).reshape(-1) if "ctx_length" in sample else np.full(B, T)
        if cl.shape[0] != B:
            raise ValueError("ctx_length must have one entry per sequence")
        dev, L, V = self.device, _abi.lib(), eng.w.V
        with torch.cuda.device(dev):
            ses = eng.session(B, T, T, T + 1)
            ses.pos0.zero_()
            rect = torch.from_numpy(obs.astype(np.int32)).to(dev)
            limit = torch.from_numpy(np.minimum(cl, 2 ** 31 - 1).astype(np.int32)).to(dev)
            target = torch.from_numpy(tgt.astype(np.int32)).to(dev).reshape(-1)
            x = eng.prefill(ses, rect, T, key_limit=limit)
            loss = torch.empty(B * T, dtype=torch.float32, device=dev)
            correct = torch.empty(B * T, dtype=torch.uint8, device=dev)
            eng.project_loss(ses, x, target, loss, correct)       # the [B*T, V] logits are never stored
            torch.cuda.synchronize(dev)
            all_loss = loss.view(B, T).cpu().numpy()
            return {"loss": all_loss.mean(-1), "last_loss": all_loss[:, -1].copy(), "all_loss": all_loss,
                    "correct": correct.view(B, T).cpu().numpy().astype(bool)}

    def _ensure_io(self, ses, G, V):
        if getattr(ses, "G_max", 0) < G:
            dev = self.device
            ses.G_max = max(G, 64)
            ses.out_tokens = torch.zeros(ses.B, ses.G_max, dtype=torch.int32, device=dev)
            ses.uniforms = torch.zeros(ses.B, ses.G_max, dtype=torch.float64, device=dev)
            ses.top_p = torch.zeros(ses.B, dtype=torch.float64, device=dev)
            ses.temp = torch.ones(ses.B, dtype=torch.float64, device=dev)
            ses.top_k = torch.zeros(ses.B, dtype=torch.int32, device=dev)
            ses.use_top_k = False
            ses.graphs = {}

    def _step(self, eng, ses, kind, keep_mask=None, logits=None):
        if kind == "greedy":
            if not eng.decode_model(ses, logits, greedy_out=ses.out_tokens):
                eng.sample_greedy(ses, ses.out_tokens, logits=logits)
        else:
            eng.decode_model(ses, logits)
            eng.sample_nucleus(ses, ses.out_tokens, ses.top_p, ses.temp, ses.top_k if ses.use_top_k else None,
                               ses.uniforms, keep_mask=keep_mask, logits=logits)

    def _decode(self, eng, ses, t, G, kind, logits_out, masks):
        """Decode steps t .. G-1.  With logits_out the recorded steps write their logits into per-step slots of a
        staging buffer (the same compiled program with one more output, like transformer_shard.py:205-208)."""
        spg = int(self.config.get("steps_per_graph", 8))
        eager = spg <= 0 or masks is not None
        while t < G:
            if eager or t == 0:
                # the first step always runs eagerly: it also performs the kernels' one-time setup
                self._step(eng, ses, kind, None if masks is None else masks[t])
                if logits_out is not None:
                    logits_out[:, t].copy_(ses.logits)
                t += 1
                continue
            n = spg if G - t >= spg else 1
            self._graph(eng, ses, kind, n, logits_out is not None).replay()
            if logits_out is not None:
                logits_out[:, t:t + n].copy_(ses.logits_stage[:n].transpose(0, 1))
            t += n

    def _graph(self, eng, ses, kind, n, with_logits=False):
        key = (kind, n, ses.use_top_k, with_logits)
        g = ses.graphs.get(key)
        if g is None:
            if kind != "greedy" and ses.sample_work is None:
                ses.sample_work = torch.empty(_abi.lib().mtj_sample_work_bytes(ses.B, eng.w.V), dtype=torch.uint8,
                                              device=self.device)
            if with_logits and (getattr(ses, "logits_stage", None) is None or ses.logits_stage.shape[0] < n):
                for k in [k for k in ses.graphs if k[3]]:          # recorded against the buffer that is replaced
                    del ses.graphs[k]
                ses.logits_stage = torch.empty(max(n, int(self.config.get("steps_per_graph", 8))), ses.B, eng.w.V,
                                               dtype=torch.float32, device=self.device)
            torch.cuda.synchronize(self.device)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for j in range(n):
                    self._step(eng, ses, kind, logits=ses.logits_stage[j] if with_logits else None)
            ses.graphs[key] = g
        return g

    def _decode_host_sampler(self, eng, ses, G, sampler, opts, logits_out):
        """Any callable honouring the reference contract (transformer_shard.py:203):
        sampler(key, logits[1, V], sampler_input, **options_of_this_sequence) -> (token[1], info)."""
        B = ses.B
        for t in range(G):
            if t:
                eng.embed_tok(ses)
            eng.decode_model(ses)
            lg = ses.logits.cpu().numpy()
            if logits_out is not None:
                logits_out[:, t].copy_(ses.logits)
            nxt = np.zeros(B, np.int32)
            for b in range(B):
                ob = {k: (None if v is None else np.asarray(v).reshape(-1)[b] if np.ndim(v) else v) for k, v in opts.items()}
                tok, _ = sampler(None, lg[b:b + 1], np.uint32(0), **ob)
                nxt[b] = int(np.asarray(tok).reshape(-1)[0])
            nt = torch.from_numpy(nxt).to(self.device)
            ses.tok.copy_(nt)
            ses.out_tokens[:, t].copy_(nt)
            ses.pos.add_(1)

"""Each part alone against the plain implementation, at sizes of its own, and the generality of
the arrangement: a toy mixer with state of its own, a toy position encoding and a toy
architecture are defined HERE, registered, built from a config.json and stepped, without a
change to the framework's files."""
import json
import math

import numpy as np
import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make_rt(dtype, tuned=True, max_tokens=256):
    from flambeau_amd.engine import Runtime
    return Runtime(DEV, dtype, max_tokens, tuned)


def rnd(*shape, scale=1.0, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def delta_of(rt, result):
    """What a mixer or feed-forward returned, as the delta tensor."""
    from flambeau_amd.parts import Product
    return result.compute(rt) if isinstance(result, Product) else result


def tol(dtype):
    return 2e-5 if dtype == torch.float32 else 2e-2


def put(rt, t, role="matrix"):
    return rt.to_device(t, role)


def step_for(rt, seqs, page_size, n_pages, shuffle_seed=0):
    """A StepState for requests ``seqs`` = (start position, tokens): pages handed out in a
    shuffled order, everything a mixer reads on the device."""
    from flambeau_amd.parts import HostBatch, StepState
    from flambeau_amd.kernels import tuned
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(shuffle_seed)).tolist()
    q_starts, q_lens, starts, pos, tok_seq = [], [], [], [], []
    width = max(-(-(st + q) // page_size) for st, q in seqs) + 1
    table = np.full((len(seqs), width), -1, dtype=np.int32)
    at = 0
    for s, (st, q) in enumerate(seqs):
        nb = -(-(st + q) // page_size)
        table[s, :nb] = [perm.pop() for _ in range(nb)]
        q_starts.append(at); q_lens.append(q); starts.append(st)
        pos += range(st, st + q); tok_seq += [s] * q
        at += q
    batch = HostBatch(q_starts, q_lens, starts, list(range(len(seqs))), at, 0)
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)
    extra = {k: i32(v) for k, v in tuned.attention_metadata(batch).items()}
    extra["attn_tiles"] = extra["attn_tiles"].reshape(-1, 4)
    extra["attn_rows"] = extra["attn_rows"].reshape(-1, 4)
    return StepState(n_tokens=at, n_seqs=len(seqs), tokens=i32([0] * at), positions=i32(pos), tok_seq=i32(tok_seq),
                     seq_slots=i32(range(len(seqs))), seq_q_start=i32(q_starts), seq_q_len=i32(q_lens),
                     seq_ctx_len=i32([st + q for st, q in seqs]), block_tables=[i32(table)], logit_rows=i32([]),
                     host=batch, extra=extra)


# ---------------------------------------------------------------- norm, feed-forward, embedding, head
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(dtype):
    from flambeau_amd.parts import NORMS, PartSpec
    rt = make_rt(dtype)
    H, eps = 200, 3e-4
    norm = NORMS.create(PartSpec("rmsnorm", dict(hidden_size=H, eps=eps)))
    assert norm.tensors()["weight"].shape == (H,) and norm.tensors()["weight"].role == "vector32"
    w = 1 + rnd(H, scale=0.2, seed=1)
    norm.bind({"weight": put(rt, w, "vector32")}, rt)
    x, d = rnd(9, H, seed=2), rnd(9, H, scale=0.5, seed=3)
    xd = x.to(DEV)
    out = torch.empty(9, H, dtype=dtype, device=DEV)
    norm.forward(xd, out, delta=d.to(DEV), store_sum=True)
    want = pm.rmsnorm((x + d).numpy(), w.numpy(), eps)
    assert np.abs(out.double().cpu().numpy() - want).max() < tol(dtype) * np.abs(want).max()
    assert torch.equal(xd.cpu(), x + d)


@pytest.mark.parametrize("tuned", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [3, 130])
def test_swiglu_part(dtype, tuned, n):
    from flambeau_amd.parts import FEED_FORWARDS, PartSpec
    rt = make_rt(dtype, tuned)
    H, I = 72, 152
    ffn = FEED_FORWARDS.create(PartSpec("swiglu", dict(hidden_size=H, intermediate_size=I)))
    assert {k: v.shape for k, v in ffn.tensors().items()} == {"gate.weight": (I, H), "up.weight": (I, H), "down.weight": (H, I)}
    w = {k: rnd(*v.shape, scale=0.2, seed=i).to(dtype) for i, (k, v) in enumerate(ffn.tensors().items())}
    ffn.bind({k: put(rt, v) for k, v in w.items()}, rt)
    x = rnd(n, H, seed=9).to(dtype)
    got = delta_of(rt, ffn.forward(x.to(DEV), None))
    assert got.dtype == torch.float32
    want = pm.swiglu_mlp(x.double().numpy(), *(w[k].double().numpy() for k in ("gate.weight", "up.weight", "down.weight")))
    assert np.abs(got.double().cpu().numpy() - want).max() < tol(dtype) * np.abs(want).max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tied", [False, True])
def test_embedding_and_head_parts(dtype, tied):
    from flambeau_amd.parts import OutputHead, TokenEmbedding
    rt = make_rt(dtype)
    V, H = 150, 40
    emb, head = TokenEmbedding(V, H), OutputHead(V, H, tied=tied)
    assert ("weight" in head.tensors()) == (not tied)
    E, W = rnd(V, H, seed=1).to(dtype), rnd(V, H, seed=2).to(dtype)
    emb.bind({"weight": put(rt, E, "table")}, rt)
    head.bind({} if tied else {"weight": put(rt, W)}, rt, embedding_table=emb.weight)
    toks = torch.tensor([3, 149, 0, 77], dtype=torch.int32, device=DEV)
    resid = torch.empty(4, H, dtype=torch.float32, device=DEV)
    emb.forward(toks, resid)
    assert torch.equal(resid.cpu(), E[toks.cpu().long()].float())
    x = rnd(5, H, seed=3).to(dtype)
    logits = head.forward(x.to(DEV), max_rows=8)
    want = pm.linear(x.double().numpy(), (E if tied else W).double().numpy())
    assert logits.dtype == torch.float32
    assert np.abs(logits.double().cpu().numpy() - want).max() < tol(dtype) * np.abs(want).max()


# ---------------------------------------------------------------- the attention mixer and the block
def _mixer_weights(mixer, dtype, seed=0, scale=0.25):
    return {k: rnd(*v.shape, scale=scale, seed=seed + i).to(dtype) for i, (k, v) in enumerate(mixer.tensors().items())}


@pytest.mark.parametrize("tuned", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,window,theta,ps", [(6, 2, 24, 0, 1e4, 8), (4, 4, 16, 13, 1e6, 16), (8, 1, 64, 40, 5e5, 4)])
def test_attention_mixer_part(dtype, tuned, nh, nkv, hd, window, theta, ps):
    """A whole prompt in one step, then the same prompt as a portion, a short portion and single
    tokens into a second cache: both must equal the plain mixer."""
    from flambeau_amd.cache.storage import CacheStorage
    from flambeau_amd.parts import MIXERS, PartSpec
    rt = make_rt(dtype, tuned)
    H, n = 56, 75
    spec = PartSpec("paged_gqa_attention", dict(hidden_size=H, n_heads=nh, n_kv_heads=nkv, head_dim=hd, window=window,
                                                position=PartSpec("rope_neox", dict(head_dim=hd, theta=theta))))
    mixer = MIXERS.create(spec)
    w = _mixer_weights(mixer, dtype)
    mixer.bind({k: put(rt, v) for k, v in w.items()}, rt)
    x = rnd(n, H, seed=7).to(dtype)
    wd = {"a." + k.replace(".weight", "_proj.weight"): v.double().numpy() for k, v in w.items()}
    want = pm.attention_mixer(x.double().numpy(), wd, "a.", np.arange(n), nh, nkv, hd, theta, window)
    for cuts in ([n], [40, 5, 1, 1, 20, 2, 6]):
        store = CacheStorage([mixer.cache_spec()], [None], rt.device, dtype, n_pages=32, page_size=ps, max_slots=2)
        got, at = [], 0
        for k in cuts:
            step = step_for(rt, [(at, k)], ps, 32, shuffle_seed=1)       # same seed: the same pages every step
            got.append(delta_of(rt, mixer.forward(x[at:at + k].to(DEV).contiguous(), step, store.entries[0])).double().cpu().numpy())
            at += k
        got = np.concatenate(got)
        assert np.abs(got - want).max() < tol(dtype) * np.abs(want).max(), cuts


@pytest.mark.parametrize("tuned", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_rotation_with_a_ladder_of_its_own(dtype, tuned):
    """A toy position encoding defined here: the built-in split-half rotation with other frequencies
    (every rung slowed down by a factor of its own) and a magnitude on cosines and sines.  It only
    overrides ``inverse_frequencies``; the table, the fused rotate-and-store kernels and the rotation
    kernel serve it as they serve the built-in ladder, in every cutting."""
    from flambeau_amd.cache.storage import CacheStorage
    from flambeau_amd.parts import MIXERS, POSITION_ENCODINGS, PartSpec
    from flambeau_amd.parts.rope import RotaryNeoX
    if "toy_slowed_ladder" not in POSITION_ENCODINGS.known():
        @POSITION_ENCODINGS.register("toy_slowed_ladder")
        class Slowed(RotaryNeoX):
            magnitude = 1.25

            def inverse_frequencies(self):
                half = self.rotated_dims // 2
                return [self.theta ** (-2.0 * i / self.rotated_dims) / (1.0 + 0.5 * i) for i in range(half)]
    rt = make_rt(dtype, tuned)
    H, n, nh, nkv, hd, theta, ps, window = 56, 75, 4, 2, 32, 1e4, 8, 50
    mixer = MIXERS.create(PartSpec("paged_gqa_attention", dict(hidden_size=H, n_heads=nh, n_kv_heads=nkv, head_dim=hd, window=window,
                                                            position=PartSpec("toy_slowed_ladder", dict(head_dim=hd, theta=theta)))))
    w = _mixer_weights(mixer, dtype)
    mixer.bind({k: put(rt, v) for k, v in w.items()}, rt)
    x = rnd(n, H, seed=7).to(dtype)
    W = {k: v.double().numpy() for k, v in w.items()}
    xs = x.double().numpy()

    def rotate(t):                                   # t [n, heads, hd]: the toy's formula, written out
        half = hd // 2
        freqs = np.array([theta ** (-2.0 * i / hd) / (1.0 + 0.5 * i) for i in range(half)])
        ang = np.arange(n)[:, None] * freqs[None, :]
        c, s_ = 1.25 * np.cos(ang)[:, None, :], 1.25 * np.sin(ang)[:, None, :]
        lo, hi = t[:, :, :half], t[:, :, half:]
        return np.concatenate([lo * c - hi * s_, lo * s_ + hi * c], axis=2)
    q = rotate(pm.linear(xs, W["q.weight"]).reshape(n, nh, hd))
    k = rotate(pm.linear(xs, W["k.weight"]).reshape(n, nkv, hd))
    v = pm.linear(xs, W["v.weight"]).reshape(n, nkv, hd)
    want = pm.linear(pm.attention(q, k, v, np.arange(n), pm.default_scale(hd), window).reshape(n, nh * hd), W["o.weight"])
    plain_ladder = pm.attention_mixer(xs, {"a." + k_.replace(".weight", "_proj.weight"): v_ for k_, v_ in W.items()}, "a.",
                                      np.arange(n), nh, nkv, hd, theta, window)
    assert np.abs(want - plain_ladder).max() > 0.05 * np.abs(want).max()          # the toy is not the built-in ladder
    for cuts in ([n], [40, 5, 1, 1, 20, 2, 6]):
        store = CacheStorage([mixer.cache_spec()], [None], rt.device, dtype, n_pages=32, page_size=ps, max_slots=2)
        got, at = [], 0
        for c in cuts:
            step = step_for(rt, [(at, c)], ps, 32, shuffle_seed=1)
            got.append(delta_of(rt, mixer.forward(x[at:at + c].to(DEV).contiguous(), step, store.entries[0])).double().cpu().numpy())
            at += c
        assert np.abs(np.concatenate(got) - want).max() < tol(dtype) * np.abs(want).max(), cuts


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prenorm_block_part(dtype):
    from flambeau_amd.cache.storage import CacheStorage
    from flambeau_amd.parts import BLOCKS, PartSpec, ResidualStream
    rt = make_rt(dtype)
    H, nh, nkv, hd, I, eps, n = 48, 3, 1, 16, 100, 1e-5, 37
    norm = PartSpec("rmsnorm", dict(hidden_size=H, eps=eps))
    mixer = PartSpec("paged_gqa_attention", dict(hidden_size=H, n_heads=nh, n_kv_heads=nkv, head_dim=hd,
                                                 position=PartSpec("rope_neox", dict(head_dim=hd, theta=1e4))))
    ffn = PartSpec("swiglu", dict(hidden_size=H, intermediate_size=I))
    block = BLOCKS.create(PartSpec("prenorm", dict(mixer=mixer, feed_forward=ffn, norm=norm)))
    names = block.tensors()
    assert set(names) == {"mixer_norm.weight", "mixer.q.weight", "mixer.k.weight", "mixer.v.weight", "mixer.o.weight",
                          "ffn_norm.weight", "ffn.gate.weight", "ffn.up.weight", "ffn.down.weight"}
    w = {}
    for i, (k, ts) in enumerate(names.items()):
        w[k] = (1 + rnd(*ts.shape, scale=0.1, seed=i)) if ts.role == "vector32" else rnd(*ts.shape, scale=0.2, seed=i).to(dtype)
    block.bind({k: put(rt, v, names[k].role) for k, v in w.items()}, rt)
    x = rnd(n, H, seed=50)
    store = CacheStorage([block.cache_spec()], [None], rt.device, dtype, n_pages=8, page_size=8, max_slots=1)
    stream = ResidualStream(x.to(DEV), rt)
    block.forward(stream, step_for(rt, [(0, n)], 8, 8), store.entries[0])
    got = stream.flush().double().cpu().numpy()
    W = {k: v.double().numpy() for k, v in w.items()}
    xs = x.double().numpy()
    a = pm.rmsnorm(xs, W["mixer_norm.weight"], eps)
    wd = {"a." + k[6:].replace(".weight", "_proj.weight"): v for k, v in W.items() if k.startswith("mixer.")}
    xs = xs + pm.attention_mixer(a, wd, "a.", np.arange(n), nh, nkv, hd, 1e4, 0)
    b = pm.rmsnorm(xs, W["ffn_norm.weight"], eps)
    want = xs + pm.swiglu_mlp(b, W["ffn.gate.weight"], W["ffn.up.weight"], W["ffn.down.weight"])
    assert np.abs(got - want).max() < tol(dtype) * np.abs(want).max()


# ---------------------------------------------------------------- toy parts, defined here
def _register_toys():
    """A mixer with per-request state (a decaying sum of its inputs), a position encoding that is
    not a rotation (it scales queries and keys by a function of the position), a feed-forward
    that routes every token to one of its experts, a norm that subtracts the mean, and an
    architecture that puts them beside the built-in parts, layer by layer."""
    from dataclasses import dataclass
    from flambeau_amd.config.base import KeyReader
    from flambeau_amd.kernels import ops
    from flambeau_amd.models.decoder import LayerSpec, ModelSpec, RunEntry
    from flambeau_amd.parts import (FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, CacheSpec, FeedForward, Mixer, Norm,
                                    PageGroup, PartSpec, PositionEncoding, StateSpec, TensorSpec)
    from flambeau_amd.registry import register_architecture

    if "toy_decay_sum" in MIXERS.known():
        return

    @MIXERS.register("toy_decay_sum")
    class DecaySum(Mixer):
        """s <- decay * s + x_t (per request, in order); delta_t = s W^T."""
        def __init__(self, hidden_size, decay):
            self.hidden_size, self.decay = hidden_size, decay

        def cache_spec(self):
            return StateSpec((self.hidden_size,), torch.float32)

        def tensors(self):
            return {"w.weight": TensorSpec((self.hidden_size, self.hidden_size))}

        def bind(self, weights, rt):
            self.rt, self.w = rt, rt.prepare_weight(weights["w.weight"])

        def forward(self, x, step, cache):
            n, H = x.shape
            sums = torch.empty(n, H, dtype=torch.float32, device=x.device)
            for q0, ql, slot in zip(step.host.q_starts, step.host.q_lens, step.host.slots):
                s = cache.state[slot]
                for i in range(q0, q0 + ql):
                    s = self.decay * s + x[i].float()
                    sums[i] = s
                cache.state[slot] = s
            delta = self.rt.buffer("delta", n, H, torch.float32)
            self.rt.gemm(sums.to(x.dtype), self.w, delta)
            return delta

    @dataclass(frozen=True)
    class LatentRows(CacheSpec):
        """A paged cache that is not keys and values: one float32 row of ``width`` per token, in a
        pool laid out ``[entries, pages, page_size, width]``; the newest ``window`` rows are needed."""
        width: int
        window: int

        def page_group(self):
            return PageGroup(0, self.width, self.window)

        def allocate_pool(self, n_entries, n_pages, page_size, dtype, device):
            return torch.full((n_entries, n_pages, page_size, self.width), float("nan"), dtype=torch.float32, device=device)

        def layer_view(self, pool, index):
            return pool[index]

        def bytes_per_token(self, element_size):
            return 4 * self.width

    @MIXERS.register("toy_window_mean")
    class WindowMean(Mixer):
        """z_t = x_t is kept in pages of its own kind; delta_t = mean(z over the last ``window`` tokens) W^T."""
        def __init__(self, hidden_size, window):
            self.hidden_size, self.window = hidden_size, window

        def cache_spec(self):
            return LatentRows(self.hidden_size, self.window)

        def tensors(self):
            return {"w.weight": TensorSpec((self.hidden_size, self.hidden_size))}

        def bind(self, weights, rt):
            self.rt, self.w = rt, rt.prepare_weight(weights["w.weight"])

        def forward(self, x, step, cache):
            n, H = x.shape
            pool, table = cache.kv, step.block_tables[cache.group]
            ps = pool.shape[1]
            pos, seq = step.positions.long(), step.tok_seq.long()
            pool[table[seq, pos // ps].long(), pos % ps] = x.float()          # this step's rows first, then every query reads the pages
            means = torch.empty(n, H, dtype=torch.float32, device=x.device)
            for s, (q0, ql, p0) in enumerate(zip(step.host.q_starts, step.host.q_lens, step.host.start_pos)):
                for i in range(ql):
                    p = p0 + i
                    t = torch.arange(max(0, p - self.window + 1), p + 1, device=x.device)
                    means[q0 + i] = pool[table[s, t // ps].long(), t % ps].mean(dim=0)
            delta = self.rt.buffer("delta", n, H, torch.float32)
            self.rt.gemm(means.to(x.dtype), self.w, delta)
            return delta

    @POSITION_ENCODINGS.register("toy_position_scale")
    class PositionScale(PositionEncoding):
        """q and k of position p are multiplied by 1 + rate * cos(p): no rotation, so the mixer
        calls ``apply`` and stores without rotating."""
        def __init__(self, rate):
            self.rate = rate

        def apply(self, qkv, positions, n_heads, n_kv_heads, head_dim):
            f = 1.0 + self.rate * torch.cos(positions.float())
            qkv[:, :(n_heads + n_kv_heads) * head_dim] *= f[:, None]

    @FEED_FORWARDS.register("toy_routed")
    class Routed(FeedForward):
        """Every token goes to the expert its router scores highest (logits and softmax in 32-bit);
        delta = p_expert * Down_e silu(Up_e x).  The tokens of an expert are gathered and run
        through the framework's matrix products."""
        def __init__(self, hidden_size, inner_size, n_experts):
            self.H, self.I, self.E = hidden_size, inner_size, n_experts

        def tensors(self):
            t = {"router.weight": TensorSpec((self.E, self.H))}
            for e in range(self.E):
                t[f"e{e}.up.weight"] = TensorSpec((self.I, self.H))
                t[f"e{e}.down.weight"] = TensorSpec((self.H, self.I))
            return t

        def bind(self, weights, rt):
            self.rt = rt
            self.router = weights["router.weight"].float()
            self.up = [rt.prepare_weight(weights[f"e{e}.up.weight"]) for e in range(self.E)]
            self.down = [rt.prepare_weight(weights[f"e{e}.down.weight"]) for e in range(self.E)]

        def forward(self, x, step):
            n = x.shape[0]
            p = torch.softmax(x.float() @ self.router.T, dim=-1)
            choice = p.argmax(dim=-1)
            delta = torch.zeros(n, self.H, dtype=torch.float32, device=x.device)
            for e in range(self.E):
                rows = (choice == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                h = torch.empty(rows.numel(), self.I, dtype=torch.float32, device=x.device)
                self.rt.gemm(x[rows].contiguous(), self.up[e], h)
                d = torch.empty(rows.numel(), self.H, dtype=torch.float32, device=x.device)
                self.rt.gemm((h * torch.sigmoid(h)).to(x.dtype), self.down[e], d)
                delta[rows] = d * p[rows, e][:, None]
            return delta

    @NORMS.register("toy_centered_norm")
    class CenteredNorm(Norm):
        """y = (x - mean) * rsqrt(var + eps) * w."""
        def __init__(self, hidden_size, eps):
            self.hidden_size, self.eps = hidden_size, eps

        def tensors(self):
            return {"weight": TensorSpec((self.hidden_size,), "vector32")}

        def bind(self, weights, rt):
            self.rt, self.weight = rt, weights["weight"]

        def forward(self, x, out, delta=None, store_sum=False, rows=None):
            s = x if delta is None else x + delta
            if store_sum and delta is not None:
                x.copy_(s)
            if rows is not None:
                s = s[rows.long()]
            c = s - s.mean(dim=-1, keepdim=True)
            out.copy_((c * torch.rsqrt((c * c).mean(dim=-1, keepdim=True) + self.eps) * self.weight).to(out.dtype))
            return out

    @dataclass(frozen=True)
    class ToyConfig:
        hidden_size: int
        vocab_size: int
        layer_kinds: tuple
        ffn_kinds: tuple
        decay: float
        rate: float
        max_position_embeddings: int

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            r = KeyReader(raw, where)
            return cls(r.integer("hidden_size"), r.integer("vocab_size"), tuple(raw["layer_kinds"]),
                       tuple(raw["ffn_kinds"]), r.number("decay"), r.number("rate"), r.integer("max_position_embeddings"))

    def toy_spec(cfg):
        H = cfg.hidden_size
        norm = PartSpec("rmsnorm", dict(hidden_size=H, eps=1e-5))
        centered = PartSpec("toy_centered_norm", dict(hidden_size=H, eps=1e-3))
        ffns = {"swiglu": PartSpec("swiglu", dict(hidden_size=H, intermediate_size=2 * H)),
                "routed": PartSpec("toy_routed", dict(hidden_size=H, inner_size=24, n_experts=3))}
        mixers = {
            "mean": PartSpec("toy_window_mean", dict(hidden_size=H, window=10)),
            "decay": PartSpec("toy_decay_sum", dict(hidden_size=H, decay=cfg.decay)),
            "attn": PartSpec("paged_gqa_attention", dict(hidden_size=H, n_heads=2, n_kv_heads=1, head_dim=16,
                                                         position=PartSpec("toy_position_scale", dict(rate=cfg.rate)))),
        }
        layers = []
        for l, kind in enumerate(cfg.layer_kinds):
            routed = cfg.ffn_kinds[l] == "routed"
            # a routed layer norms with the centered norm, the others with the built-in one
            block = PartSpec("prenorm", dict(mixer=mixers[kind], feed_forward=ffns[cfg.ffn_kinds[l]],
                                             norm=centered if routed else norm))
            local = ["w"] if kind in ("decay", "mean") else ["q", "k", "v", "o"]
            names = {f"mixer.{t}.weight": f"toy.{l}.mix.{t}" for t in local}
            names.update({"mixer_norm.weight": f"toy.{l}.n1", "ffn_norm.weight": f"toy.{l}.n2"})
            if routed:
                names["ffn.router.weight"] = f"toy.{l}.router"
                for e in range(3):
                    names.update({f"ffn.e{e}.up.weight": f"toy.{l}.e{e}.up", f"ffn.e{e}.down.weight": f"toy.{l}.e{e}.down"})
            else:
                names.update({"ffn.gate.weight": f"toy.{l}.gate", "ffn.up.weight": f"toy.{l}.up", "ffn.down.weight": f"toy.{l}.down"})
            layers.append(LayerSpec(block, names))
        # the order layers run in is data: layer 1 runs twice, its second run reads the first's cache
        order = [RunEntry(l) for l in range(len(layers))]
        if cfg.layer_kinds[1] == "attn":
            order.append(RunEntry(1, cache_of=1))
        return ModelSpec("ToyStateLM", H, cfg.vocab_size, cfg.max_position_embeddings, layers, order, norm,
                         {"embedding.weight": "toy.embed", "final_norm.weight": "toy.norm", "head.weight": "toy.head"})

    register_architecture("ToyStateLM", ToyConfig, toy_spec)


def _toy_plain(cfg, w, toks):
    """The toy architecture in numpy, whole sequence."""
    H, n = cfg["hidden_size"], len(toks)
    x = w["toy.embed"][toks]
    order = list(range(len(cfg["layer_kinds"])))
    if cfg["layer_kinds"][1] == "attn":
        order.append(1)
    kept = {}            # keys and values a layer's first run stored

    def centered(v, g):
        c = v - v.mean(axis=-1, keepdims=True)
        return c / np.sqrt((c * c).mean(axis=-1, keepdims=True) + 1e-3) * g

    for l in order:
        routed = cfg["ffn_kinds"][l] == "routed"
        a = centered(x, w[f"toy.{l}.n1"]) if routed else pm.rmsnorm(x, w[f"toy.{l}.n1"], 1e-5)
        if cfg["layer_kinds"][l] == "decay":
            s, sums = np.zeros(H), []
            for t in range(n):
                s = cfg["decay"] * s + a[t]
                sums.append(s)
            d = np.stack(sums) @ w[f"toy.{l}.mix.w"].T
        elif cfg["layer_kinds"][l] == "mean":
            d = np.stack([a[max(0, t - 9):t + 1].mean(axis=0) for t in range(n)]) @ w[f"toy.{l}.mix.w"].T
        else:
            f = (1.0 + cfg["rate"] * np.cos(np.arange(n)))[:, None, None]
            q = (a @ w[f"toy.{l}.mix.q"].T).reshape(n, 2, 16) * f
            if l in kept:                      # the second run reads the cache of the first
                k, v = kept[l]
            else:
                k = (a @ w[f"toy.{l}.mix.k"].T).reshape(n, 1, 16) * f
                v = (a @ w[f"toy.{l}.mix.v"].T).reshape(n, 1, 16)
                kept[l] = (k, v)
            d = pm.attention(q, k, v, np.arange(n), 0.25, 0).reshape(n, 32) @ w[f"toy.{l}.mix.o"].T
        x = x + d
        if routed:
            b = centered(x, w[f"toy.{l}.n2"])
            logits = b @ w[f"toy.{l}.router"].T
            p = np.exp(logits - logits.max(axis=-1, keepdims=True))
            p = p / p.sum(axis=-1, keepdims=True)
            d = np.zeros_like(x)
            for t in range(n):
                e = int(np.argmax(p[t]))
                h = w[f"toy.{l}.e{e}.up"] @ b[t]
                d[t] = p[t, e] * (w[f"toy.{l}.e{e}.down"] @ pm.silu(h))
            x = x + d
        else:
            b = pm.rmsnorm(x, w[f"toy.{l}.n2"], 1e-5)
            x = x + pm.swiglu_mlp(b, w[f"toy.{l}.gate"], w[f"toy.{l}.up"], w[f"toy.{l}.down"])
    return pm.rmsnorm(x, w["toy.norm"], 1e-5) @ w["toy.head"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_is_registered_built_and_stepped(tmp_path, dtype):
    """Parts that only this test knows (a mixer with a state per request, a mixer whose pages hold
    something else than keys and values, a routed feed-forward, another norm, another position
    encoding), an architecture made of them and of built-in parts, a layer that runs twice: registered,
    built from a config.json and stepped in every cutting, without a change to the framework's files.
    In bfloat16 the routed feed-forward stays out: an expert chosen by an argmax over rounded numbers
    may differ from the plain choice, which says nothing about the framework."""
    import replay_helpers as rh
    from flambeau_amd.engine import ModelRunner, load_model
    from flambeau_amd.weights import write_random_model
    _register_toys()
    routed = dtype == "float32"
    cfg = dict(architectures=["ToyStateLM"], hidden_size=32, vocab_size=90, layer_kinds=["decay", "attn", "mean", "decay"],
               ffn_kinds=["routed" if routed else "swiglu", "swiglu", "swiglu", "routed" if routed else "swiglu"],
               decay=0.8, rate=0.3, max_position_embeddings=128)
    d = write_random_model(cfg, tmp_path / "toy", seed=4, std=0.15, gain_std=0.05, store_dtype=torch.float32)
    model, _ = load_model(d, dtype=dtype, max_batch_tokens=128)
    assert [type(b.mixer).__name__ for b in model.blocks] == ["DecaySum", "PagedGQAAttention", "WindowMean", "DecaySum"]
    if routed:
        assert [type(b.ffn).__name__ for b in model.blocks] == ["Routed", "SwiGLU", "SwiGLU", "Routed"]
        assert [type(b.ffn_norm).__name__ for b in model.blocks] == ["CenteredNorm", "RMSNorm", "RMSNorm", "CenteredNorm"]
    runner = ModelRunner(model, n_pages=16, page_size=8, max_slots=3, max_logit_rows=128)
    # a mixer with state of its own never replays a padded graph; blocks with parts that call torch are not
    # recorded: they run again, between the recorded stretches, whenever a step of a known shape is replayed
    assert not runner.decode_graphs and runner.step_programs
    # two states; two page pools of different kinds (keys and values; latent rows), each with a table of its own
    assert len(runner.storage.states) == 2 and len(runner.storage.pools) == 2
    assert runner.storage.pools[0].shape[0] == 1                       # the repeated layer reads, it owns no cache
    assert runner.storage.pools[1].shape == (1, 16, 8, 32) and [g.window for g in runner.manager.groups] == [0, 10]
    w = {k: v for k, v in pm.read_safetensors(d / "model.safetensors").items()}
    if dtype == "bfloat16":
        w = {k: pm.round_bf16(v) if v.ndim == 2 else v for k, v in w.items()}
    reqs = rh.make_requests(90, [30, 17, 41, 9, 25], seed=2)
    ref = {rid: _toy_plain(cfg, w, toks) for rid, toks in reqs.items()}
    for mode, steps in [("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs, tail=8)),
                        ("portions", rh.trace_portions(reqs, sizes=(2, 7, 3, 11))),
                        ("mixed", rh.trace_mixed(reqs, seed=1, max_live=3, max_portion=9, decode_tail=4))]:
        got = rh.run_in_process(runner, steps)
        rh.compare(got, reqs, ref, dtype, f"toy {mode}")
    assert not runner.manager.live and runner.manager.free_pages() == [16, 16]
    assert runner.n_replayed > 20 and runner.n_recorded > 3
    # slots are zeroed when they are claimed again: a second pass over the same requests agrees
    rh.compare(rh.run_in_process(runner, rh.trace_mixed(reqs, seed=3, max_live=3)), reqs, ref, dtype, "toy again")


def test_a_part_that_cannot_be_captured_keeps_decode_steps_out_of_graphs(tmp_path):
    """All mixers are attention (a padded decode step could replay a device graph), but one layer's
    feed-forward is the toy that calls torch and looks at its routing on the host: such a model's
    decode steps are not captured (a capture refuses those calls); its other blocks are still
    recorded, and every cutting gives the plain numbers."""
    import replay_helpers as rh
    from flambeau_amd.engine import ModelRunner, load_model
    from flambeau_amd.weights import write_random_model
    _register_toys()
    cfg = dict(architectures=["ToyStateLM"], hidden_size=32, vocab_size=70, layer_kinds=["attn", "attn"],
               ffn_kinds=["swiglu", "routed"], decay=0.8, rate=0.3, max_position_embeddings=128)
    d = write_random_model(cfg, tmp_path / "toy2", seed=6, std=0.15, gain_std=0.05, store_dtype=torch.float32)
    model, _ = load_model(d, dtype="float32", max_batch_tokens=128)
    assert not model.capturable() and model.replayable()
    runner = ModelRunner(model, n_pages=14, page_size=8, max_slots=3, max_logit_rows=128)
    assert not runner.decode_graphs and runner.step_programs
    w = {k: v for k, v in pm.read_safetensors(d / "model.safetensors").items()}
    reqs = rh.make_requests(70, [21, 9, 33, 14], seed=8)
    ref = {rid: _toy_plain(cfg, w, toks) for rid, toks in reqs.items()}
    for mode, steps in [("tail", rh.trace_tail(reqs, tail=12)), ("mixed", rh.trace_mixed(reqs, seed=2, max_live=3, max_portion=9, decode_tail=6))]:
        rh.compare(rh.run_in_process(runner, steps), reqs, ref, "float32", f"toy {mode}")
    assert runner.n_replayed > 5
    # the built-in architecture's parts can all be captured
    from flambeau_amd.engine import random_model
    from tiny_configs import TINY
    assert random_model(TINY["A"]["config"], 1, dtype="bfloat16")[0].capturable()


def _register_parallel_toys():
    """Another arrangement of a layer, another embedding and another head, known to this test only."""
    from dataclasses import dataclass
    from flambeau_amd.config.base import KeyReader
    from flambeau_amd.models.decoder import LayerSpec, ModelSpec, RunEntry
    from flambeau_amd.parts import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, Block, OutputHead, PartSpec,
                                    TokenEmbedding)
    from flambeau_amd.registry import known_architectures, register_architecture
    if "ToyParallelLM" in known_architectures():
        return

    @BLOCKS.register("toy_parallel")
    class ParallelBlock(Block):
        """x += Mixer(Norm(x)) + FeedForward(Norm(x)): one norm, both parts read the same normed rows."""
        replayable = True

        def __init__(self, mixer, feed_forward, norm):
            self.norm, self.mixer, self.ffn = NORMS.create(norm), MIXERS.create(mixer), FEED_FORWARDS.create(feed_forward)
            self._parts = {"norm": self.norm, "mixer": self.mixer, "ffn": self.ffn}

        def cache_spec(self):
            return self.mixer.cache_spec()

        def mixers(self):
            return [self.mixer]

        def subparts(self):
            return list(self._parts.values())

        def tensors(self):
            return {f"{p}.{name}": spec for p, part in self._parts.items() for name, spec in part.tensors().items()}

        def bind(self, weights, rt):
            self.rt = rt
            for p, part in self._parts.items():
                part.bind({k[len(p) + 1:]: v for k, v in weights.items() if k.startswith(p + ".")}, rt)

        def forward(self, stream, step, cache):
            a = stream.normed(self.norm, name="toy_parallel_normed")
            stream.push(self.mixer.forward(a, step, cache))
            stream.push(self.ffn.forward(a, step))

    @EMBEDDINGS.register("toy_scaled_embedding")
    class ScaledEmbedding(TokenEmbedding):
        """h0 = scale * E[token]."""
        replayable = False

        def __init__(self, vocab_size, hidden_size, scale):
            super().__init__(vocab_size, hidden_size)
            self.scale = scale

        def forward(self, tokens, out):
            super().forward(tokens, out)
            return out.mul_(self.scale)

    @HEADS.register("toy_capped_head")
    class CappedHead(OutputHead):
        """logits = cap * tanh(x W^T / cap)."""
        replayable = False

        def __init__(self, vocab_size, hidden_size, cap, tied=False):
            super().__init__(vocab_size, hidden_size, tied)
            self.cap = cap

        def forward(self, x, max_rows):
            logits = super().forward(x, max_rows)
            return logits.copy_(self.cap * torch.tanh(logits / self.cap))

    @dataclass(frozen=True)
    class ParallelConfig:
        hidden_size: int
        vocab_size: int
        n_layers: int
        embedding_scale: float
        logit_cap: float
        window: int
        max_position_embeddings: int

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            r = KeyReader(raw, where)
            return cls(r.integer("hidden_size"), r.integer("vocab_size"), r.integer("n_layers"), r.number("embedding_scale"),
                       r.number("logit_cap"), r.integer("window"), r.integer("max_position_embeddings"))

    def spec(cfg):
        H = cfg.hidden_size
        norm = PartSpec("rmsnorm", dict(hidden_size=H, eps=1e-4))
        mixer = PartSpec("paged_gqa_attention", dict(hidden_size=H, n_heads=4, n_kv_heads=2, head_dim=16, window=cfg.window,
                                                     position=PartSpec("rope_neox", dict(head_dim=16, theta=500.0))))
        ffn = PartSpec("swiglu", dict(hidden_size=H, intermediate_size=56))
        layers = []
        for l in range(cfg.n_layers):
            names = {f"mixer.{t}.weight": f"p{l}.{t}_proj.weight" for t in "qkvo"}
            names.update({"norm.weight": f"p{l}.norm", "ffn.gate.weight": f"p{l}.gate", "ffn.up.weight": f"p{l}.up",
                          "ffn.down.weight": f"p{l}.down"})
            layers.append(LayerSpec(PartSpec("toy_parallel", dict(mixer=mixer, feed_forward=ffn, norm=norm)), names))
        sizes = dict(vocab_size=cfg.vocab_size, hidden_size=H)
        return ModelSpec("ToyParallelLM", H, cfg.vocab_size, cfg.max_position_embeddings, layers,
                         [RunEntry(l) for l in range(cfg.n_layers)], norm,
                         {"embedding.weight": "table", "final_norm.weight": "norm"}, tied_head=True,
                         embedding=PartSpec("toy_scaled_embedding", dict(sizes, scale=cfg.embedding_scale)),
                         head=PartSpec("toy_capped_head", dict(sizes, cap=cfg.logit_cap, tied=True)))

    register_architecture("ToyParallelLM", ParallelConfig, spec)


def _parallel_plain(cfg, w, toks):
    n, pos = len(toks), np.arange(len(toks))
    x = cfg["embedding_scale"] * w["table"][toks]
    for l in range(cfg["n_layers"]):
        a = pm.rmsnorm(x, w[f"p{l}.norm"], 1e-4)
        x = x + pm.attention_mixer(a, w, f"p{l}.", pos, 4, 2, 16, 500.0, cfg["window"]) \
              + pm.swiglu_mlp(a, w[f"p{l}.gate"], w[f"p{l}.up"], w[f"p{l}.down"])
    logits = pm.rmsnorm(x, w["norm"], 1e-4) @ w["table"].T
    return cfg["logit_cap"] * np.tanh(logits / cfg["logit_cap"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_another_arrangement_embedding_and_head_from_a_test_file(tmp_path, dtype):
    """A layer whose mixer and feed-forward read the same normed rows, an embedding with a scale, a tied
    head with a soft cap on its logits: registered here, named by the model's description
    (``ModelSpec.embedding``, ``.head``, a block kind), built from a config.json and stepped in every cutting."""
    import replay_helpers as rh
    from flambeau_amd.engine import ModelRunner, load_model
    from flambeau_amd.weights import write_random_model
    _register_parallel_toys()
    cfg = dict(architectures=["ToyParallelLM"], hidden_size=40, vocab_size=77, n_layers=3, embedding_scale=6.3, logit_cap=4.0,
               window=21, max_position_embeddings=128)
    d = write_random_model(cfg, tmp_path / "par", seed=9, std=0.15, gain_std=0.05, store_dtype=torch.float32)
    model, _ = load_model(d, dtype=dtype, max_batch_tokens=128)
    assert [type(b).__name__ for b in model.blocks] == ["ParallelBlock"] * 3
    assert type(model.embedding).__name__ == "ScaledEmbedding" and type(model.head).__name__ == "CappedHead"
    assert not model.replayable()          # embedding and head call torch: such a model's steps are run, never replayed
    runner = ModelRunner(model, n_pages=14, page_size=8, max_slots=3, max_logit_rows=128)
    assert not runner.step_programs and not runner.decode_graphs
    w = {k: v for k, v in pm.read_safetensors(d / "model.safetensors").items()}
    if dtype == "bfloat16":
        w = {k: pm.round_bf16(v) if v.ndim == 2 else v for k, v in w.items()}
    reqs = rh.make_requests(77, [33, 11, 40, 26], seed=12)
    ref = {rid: _parallel_plain(cfg, w, toks) for rid, toks in reqs.items()}
    assert max(np.abs(r).max() for r in ref.values()) > 2.0          # the cap bends the logits
    for mode, steps in [("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs, tail=10)),
                        ("portions", rh.trace_portions(reqs, sizes=(2, 9, 3, 14))),
                        ("mixed", rh.trace_mixed(reqs, seed=6, max_live=3, max_portion=9, decode_tail=5))]:
        rh.compare(rh.run_in_process(runner, steps), reqs, ref, dtype, f"parallel toy {mode}")
    assert not runner.manager.live and runner.manager.free_pages() == [14]


def test_unknown_part_names_the_known_ones():
    from flambeau_amd.parts import MIXERS, PartSpec
    with pytest.raises(KeyError, match="paged_gqa_attention"):
        MIXERS.create(PartSpec("no_such_mixer", {}))

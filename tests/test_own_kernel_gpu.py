"""A part that brings a kernel of its own: the test compiles a small HIP library (one launch function
and its trampoline), gives its argument list to the kernel interface, makes it known to the recorder of
step programs, and registers a feed-forward that launches it between two of the framework's matrix
products, all without a change to the framework's files.  The model built from it is replayable and
capturable like the built-in one: its steps are recorded and replayed natively, decode steps run
as device graphs, and every cutting gives the plain numbers."""
import ctypes
from dataclasses import dataclass
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu

HERE = Path(__file__).resolve().parent / "own_kernel"
_registered = False


def own_library():
    from flambeau_amd.csrc import build
    return build.build_own_library("toy_temper", [HERE / "toy_temper.hip"], HERE / "_build")


def _register():
    global _registered
    if _registered:
        return
    _registered = True
    from flambeau_amd.config.base import KeyReader
    from flambeau_amd.kernels import library, ops
    from flambeau_amd.models.decoder import LayerSpec, ModelSpec, RunEntry
    from flambeau_amd.parts import FEED_FORWARDS, FeedForward, PartSpec, Product, TensorSpec
    from flambeau_amd.registry import register_architecture

    own = ctypes.CDLL(str(own_library()))
    library.register_signatures({"toy_temper": [library.P, library.P, library.I, library.L, library.F, library.P]}, library=own)
    library.make_recordable("toy_temper", own.toy_temper_replay)

    @FEED_FORWARDS.register("toy_tempered")
    class Tempered(FeedForward):
        """delta = Down(h * sigmoid(alpha h)), h = Up x."""
        replayable = True

        def __init__(self, hidden_size, inner_size, alpha):
            self.H, self.I, self.alpha = hidden_size, inner_size, alpha

        def tensors(self):
            return {"up.weight": TensorSpec((self.I, self.H)), "down.weight": TensorSpec((self.H, self.I))}

        def bind(self, weights, rt):
            self.rt = rt
            self.up = rt.prepare_weight(weights["up.weight"])
            self.down = rt.prepare_weight(weights["down.weight"])

        def forward(self, x, step):
            rt, n = self.rt, x.shape[0]
            h = rt.buffer("toy_h", n, self.I, torch.float32)
            rt.gemm(x, self.up, h)
            act = rt.buffer("toy_act", n, self.I)
            library.call("toy_temper", h.data_ptr(), act.data_ptr(), int(act.dtype == torch.bfloat16), n * self.I,
                         float(self.alpha), ops.stream_handle())
            return Product(act, self.down)

    @dataclass(frozen=True)
    class TemperedConfig:
        hidden_size: int
        vocab_size: int
        n_layers: int
        inner_size: int
        alpha: float
        max_position_embeddings: int

        @classmethod
        def from_dict(cls, raw, where="config.json"):
            r = KeyReader(raw, where)
            return cls(r.integer("hidden_size"), r.integer("vocab_size"), r.integer("n_layers"), r.integer("inner_size"),
                       r.number("alpha"), r.integer("max_position_embeddings"))

    def spec(cfg):
        H = cfg.hidden_size
        norm = PartSpec("rmsnorm", dict(hidden_size=H, eps=1e-5))
        mixer = PartSpec("paged_gqa_attention", dict(hidden_size=H, n_heads=3, n_kv_heads=1, head_dim=16,
                                                     position=PartSpec("rope_neox", dict(head_dim=16, theta=100.0))))
        ffn = PartSpec("toy_tempered", dict(hidden_size=H, inner_size=cfg.inner_size, alpha=cfg.alpha))
        layers = []
        for l in range(cfg.n_layers):
            names = {f"mixer.{t}.weight": f"l{l}.{t}_proj.weight" for t in "qkvo"}
            names.update({"mixer_norm.weight": f"l{l}.n1", "ffn_norm.weight": f"l{l}.n2",
                          "ffn.up.weight": f"l{l}.up", "ffn.down.weight": f"l{l}.down"})
            layers.append(LayerSpec(PartSpec("prenorm", dict(mixer=mixer, feed_forward=ffn, norm=norm)), names))
        return ModelSpec("ToyTemperedLM", H, cfg.vocab_size, cfg.max_position_embeddings, layers,
                         [RunEntry(l) for l in range(cfg.n_layers)], norm,
                         {"embedding.weight": "embed", "final_norm.weight": "norm", "head.weight": "head"})

    register_architecture("ToyTemperedLM", TemperedConfig, spec)


def _plain(cfg, w, toks):
    n = len(toks)
    pos = np.arange(n)
    x = w["embed"][toks]
    for l in range(cfg["n_layers"]):
        a = pm.rmsnorm(x, w[f"l{l}.n1"], 1e-5)
        x = x + pm.attention_mixer(a, w, f"l{l}.", pos, 3, 1, 16, 100.0, 0)
        b = pm.rmsnorm(x, w[f"l{l}.n2"], 1e-5)
        h = b @ w[f"l{l}.up"].T
        x = x + (h / (1.0 + np.exp(-cfg["alpha"] * h))) @ w[f"l{l}.down"].T
    return pm.rmsnorm(x, w["norm"], 1e-5) @ w["head"].T


def test_the_kernel_alone():
    _register()
    from flambeau_amd.kernels import library, ops
    for n in (1, 255, 70001):
        h = torch.randn(n, device="cuda") * 3
        for dtype in (torch.float32, torch.bfloat16):
            out = torch.empty(n, device="cuda", dtype=dtype)
            library.call("toy_temper", h.data_ptr(), out.data_ptr(), int(dtype == torch.bfloat16), n, 0.7, ops.stream_handle())
            want = (h.double() * torch.sigmoid(0.7 * h.double())).float()
            if dtype == torch.bfloat16:
                assert ((out.float() - want).abs() <= want.abs() * 2 ** -8 + 1e-30).all()
            else:
                assert (out - want).abs().max() < 2e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_part_with_a_kernel_of_its_own_is_recorded_replayed_and_captured(tmp_path, dtype):
    import replay_helpers as rh
    from flambeau_amd.engine import ModelRunner, load_model
    from flambeau_amd.kernels import library
    from flambeau_amd.weights import write_random_model
    _register()
    assert library.recordable("toy_temper")
    cfg = dict(architectures=["ToyTemperedLM"], hidden_size=48, vocab_size=83, n_layers=3, inner_size=40, alpha=1.7,
               max_position_embeddings=256)
    d = write_random_model(cfg, tmp_path / "own", seed=11, std=0.12, gain_std=0.05, store_dtype=torch.float32)
    model, _ = load_model(d, dtype=dtype, max_batch_tokens=128)
    assert model.replayable() and model.capturable()
    runner = ModelRunner(model, n_pages=20, page_size=8, max_slots=4, max_logit_rows=128)
    assert runner.step_programs and runner.decode_graphs
    w = {k: v for k, v in pm.read_safetensors(d / "model.safetensors").items()}
    if dtype == "bfloat16":
        w = {k: pm.round_bf16(v) if v.ndim == 2 else v for k, v in w.items()}
    reqs = rh.make_requests(83, [37, 12, 51, 22, 30], seed=5)
    ref = {rid: _plain(cfg, w, toks) for rid, toks in reqs.items()}
    for mode, steps in [("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs, tail=16)),
                        ("portions", rh.trace_portions(reqs, sizes=(2, 7, 3, 11))),
                        ("mixed", rh.trace_mixed(reqs, seed=4, max_live=4, max_portion=9, decode_tail=8))]:
        rh.compare(rh.run_in_process(runner, steps), reqs, ref, dtype, f"own kernel {mode}")
    assert not runner.manager.live
    # the steps were replayed from recorded programs that hold the test's launch function by name,
    # and decode steps ran as device graphs
    assert runner.n_replayed > 20 and runner._graphs
    programs = [p for rec in runner._programs.values() for p in rec.stretches if isinstance(p, library.Program)]
    assert programs and all(p.names().count("toy_temper") == cfg["n_layers"] for p in programs)

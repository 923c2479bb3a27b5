"""A decoder described as data, and the model built from the description.

``ModelSpec`` lists the layers (each a block ``PartSpec`` plus the file names of its tensors)
and, separately, the order in which they run: a list of ``RunEntry`` that may name a layer
twice (shared weights) or let an entry read the cache an earlier entry wrote.  Caches belong
to run-order entries, not to layers.  ``DecoderModel`` turns the description into parts,
says which tensors it needs (``manifest``), takes them (``bind``) and runs a batch
(``forward``).  The reference's counterpart is the ``Arch`` trait and the layer loop of a
model crate (crates/forward/src/runtime/mod.rs:59-136, crates/models/qwen35-v2/src/model.rs:11-51).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..kernels import ops
from ..kernels.library import suspended
from ..parts import BLOCKS, EMBEDDINGS, HEADS, NORMS, PartSpec, ResidualStream


@dataclass
class LayerSpec:
    block: PartSpec
    names: dict                       # the block's local tensor name -> name in the weight files


@dataclass
class RunEntry:
    layer: int                        # index into ModelSpec.layers
    cache_of: int | None = None       # index of an earlier run-order entry whose cache is read


@dataclass
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_position: int
    layers: list
    run_order: list
    final_norm: PartSpec
    names: dict                       # "embedding.weight", "final_norm.weight", "head.weight" -> file names
    tied_head: bool = False
    eos_token_id: int | None = None
    bos_token_id: int | None = None
    embedding: PartSpec | None = None  # None: the plain table look-up ("token_embedding")
    head: PartSpec | None = None       # None: the plain matrix product ("linear_head"), tied or not
    eos_token_ids: tuple = ()         # every id that ends a sequence (eos_token_id is the first)
    ignored_tensors: tuple = ()       # name patterns (fnmatch) of tensors a file may hold and the model does not read


SMALL_STEP = 16      # up to this many rows the output head runs on every row of a step


class DecoderModel:
    def __init__(self, spec: ModelSpec, rt):
        self.spec = spec
        self.rt = rt
        sizes = dict(vocab_size=spec.vocab_size, hidden_size=spec.hidden_size)
        self.embedding = EMBEDDINGS.create(spec.embedding or PartSpec("token_embedding", sizes))
        self.blocks = [BLOCKS.create(ls.block) for ls in spec.layers]
        self.final_norm = NORMS.create(spec.final_norm)
        self.head = HEADS.create(spec.head or PartSpec("linear_head", dict(sizes, tied=spec.tied_head)))
        self._signature_mixers = None
        self._recorded_blocks = None        # per block: can its launches be recorded?
        for i, e in enumerate(spec.run_order):
            if not 0 <= e.layer < len(self.blocks):
                raise ValueError(f"run-order entry {i} names layer {e.layer}, the model has {len(self.blocks)}")

    # ------------------------------------------------------------ tensors
    def manifest(self) -> dict:
        """``{file tensor name: (owner, local name, TensorSpec)}`` of everything the model loads."""
        out = {}

        def put(file_name, owner, local, tspec):
            if file_name in out:
                raise ValueError(f"tensor '{file_name}' is asked for twice")
            out[file_name] = (owner, local, tspec)

        for local, ts in self.embedding.tensors().items():
            put(self.spec.names["embedding." + local], "embedding", local, ts)
        for li, (ls, block) in enumerate(zip(self.spec.layers, self.blocks)):
            for local, ts in block.tensors().items():
                if local not in ls.names:
                    raise KeyError(f"layer {li}: no file name given for the tensor '{local}'")
                put(ls.names[local], li, local, ts)
        for local, ts in self.final_norm.tensors().items():
            put(self.spec.names["final_norm." + local], "final_norm", local, ts)
        for local, ts in self.head.tensors().items():
            put(self.spec.names["head." + local], "head", local, ts)
        return out

    def bind(self, tensors: dict) -> None:
        """``tensors``: file name -> device tensor, as ``manifest`` asked for them."""
        per_owner: dict = {}
        for file_name, (owner, local, _) in self.manifest().items():
            per_owner.setdefault(owner, {})[local] = tensors[file_name]
        self.embedding.bind(per_owner.get("embedding", {}), self.rt)
        for li, block in enumerate(self.blocks):
            block.bind(per_owner.get(li, {}), self.rt)
        self.final_norm.bind(per_owner.get("final_norm", {}), self.rt)
        self.head.bind(per_owner.get("head", {}), self.rt, embedding_table=self.embedding.weight)

    # ------------------------------------------------------------ cache needs
    def cache_entries(self):
        """Per run-order entry: (cache spec or None, index of the entry it shares with or None)."""
        specs, shares = [], []
        for e in self.spec.run_order:
            specs.append(self.blocks[e.layer].cache_spec())
            shares.append(e.cache_of)
        return specs, shares

    def all_parts(self) -> list:
        """Every part of the model, the parts of parts included."""
        out, todo = [], [self.embedding, self.final_norm, self.head, *self.blocks]
        while todo:
            p = todo.pop()
            out.append(p)
            todo += list(getattr(p, "subparts", lambda: [])())
        return out

    def replayable(self) -> bool:
        """True if steps of this model can be recorded and replayed (``Part.replayable``): embedding,
        final norm and head must be; a block that is not runs as it is between the recorded stretches."""
        return all(self._part_replayable(p) for p in (self.embedding, self.final_norm, self.head))

    def capturable(self) -> bool:
        """True if a whole step of this model can go into a device graph: every part only enqueues
        launches of the kernel library (``Part.replayable``), the blocks included (a part that calls
        other libraries or waits for the device cannot be captured)."""
        return self.replayable() and all(self._part_replayable(b) for b in self.blocks)

    @staticmethod
    def _part_replayable(part) -> bool:
        todo = [part]
        while todo:
            p = todo.pop()
            if not getattr(p, "replayable", False):
                return False
            todo += list(getattr(p, "subparts", lambda: [])())
        return True

    def step_signature(self, batch) -> tuple:
        """What the mixers decide from the batch's numbers beyond its shape (``Mixer.step_signature``),
        one entry per group of like mixers.  Mixers of blocks that are never recorded decide anew in
        every step and have no say here."""
        if self._signature_mixers is None:
            seen = {}
            for b in self.blocks:
                if not self._part_replayable(b):
                    continue
                for m in getattr(b, "mixers", lambda: [])():
                    seen.setdefault(m.signature_group(), m)
            self._signature_mixers = list(seen.values())
        return tuple(m.step_signature(batch) for m in self._signature_mixers)

    def mixer_classes(self):
        return list(self.mixers_by_class())

    def mixers_by_class(self) -> dict:
        """The model's mixers, grouped by their class in the order of first appearance."""
        found = {}
        for b in self.blocks:
            for m in getattr(b, "mixers", lambda: [])():
                found.setdefault(type(m), []).append(m)
        return found

    # ------------------------------------------------------------ the forward pass of one batch
    def forward(self, step, caches, max_logit_rows: int):
        with ops.pinned_stream():             # one look-up of torch's current stream for all launches of the pass
            return self._forward(step, caches, max_logit_rows)

    def _forward(self, step, caches, max_logit_rows: int):
        """Logits ``[R, vocab]`` (float32) at ``step.logit_rows``; ``caches[i]`` belongs to
        run-order entry ``i``."""
        rt = self.rt
        step.scratch.clear()
        resid = rt.buffer("residual", step.n_tokens, self.spec.hidden_size, torch.float32)
        self.embedding.forward(step.tokens, resid)
        stream = ResidualStream(resid, rt)
        if self._recorded_blocks is None:
            self._recorded_blocks = [self._part_replayable(b) for b in self.blocks]
        for i, e in enumerate(self.spec.run_order):
            block = self.blocks[e.layer]
            if step.recorder is not None and not self._recorded_blocks[e.layer]:
                # A block that cannot be replayed ends the recorded stretch: when the step is replayed it
                # runs again with that step's metadata.  Whatever it allocates lies elsewhere then, so
                # all that passes between it and the recorded stretches is the residual stream itself:
                # pending sums are added before it starts and before it ends.
                stream.flush()

                def run_block(now, block=block, cache=caches[i], resid=resid, rt=rt):
                    own = ResidualStream(resid, rt)
                    block.forward(own, now, cache)
                    own.flush()
                step.recorder.cut(run_block)
                with suspended():
                    run_block(step)
            else:
                block.forward(stream, step, caches[i])
        if step.logit_rows.shape[0] == 0:
            stream.flush()
            return None
        every_row = step.host.every_row          # rows 0 .. n - 1 in order (a decode step, a whole prompt)
        if every_row or step.n_tokens <= SMALL_STEP:
            # a few rows cost what one row costs: all of them take the path of a decode step (the
            # same kernels whatever is wanted), and the wanted ones are picked afterwards
            x = stream.normed(self.final_norm, name="final", lazy=True)
            logits = self.head.forward(x, max(max_logit_rows, step.n_tokens))
            if every_row:
                return logits
            picked = rt.buffer("logits_picked", step.logit_rows.shape[0], logits.shape[1], torch.float32, max_rows=max_logit_rows)
            return ops.gather_rows(logits, step.logit_rows, picked)
        x = stream.normed(self.final_norm, rows=step.logit_rows, name="final")
        return self.head.forward(x, max_logit_rows)

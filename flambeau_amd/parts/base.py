"""What a model is built from: the interfaces of the parts and the records they exchange.

A decoder layer is an arrangement (``Block``) of a ``Mixer`` (attention here), a
``FeedForward``, ``Norm``s and, inside the mixer, a ``PositionEncoding``.  Each part
is created from a ``PartSpec`` (a registry key plus its sizes and constants), says
which tensors it needs, is given them, and is then run on a batch.  No part knows
which model it is in: everything it needs arrives through its parameters, the
``StepState`` and its ``LayerCache``.

The reference's counterpart is the composite-op vocabulary a model writes against
(crates/forward/src/ctx.rs:14-206) with per-kind weight bundles
(ctx.rs:316-496) and the per-layer cache shape (crates/forward/src/core/scratch.rs:137-165).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable

import torch


# ---------------------------------------------------------------- descriptions
@dataclass(frozen=True)
class PartSpec:
    """A part chosen by the configuration: registry key and parameters."""
    kind: str
    params: dict = field(default_factory=dict)

    def __hash__(self):
        return hash((self.kind, tuple(sorted((k, repr(v)) for k, v in self.params.items()))))


@dataclass(frozen=True)
class TensorSpec:
    """A tensor a part needs.  ``role``: ``matrix``/``table`` are stored in the compute
    dtype; ``vector32`` (norm gains, biases, decay rates) is always held in float32; ``int32`` integer
    tables.  ``init`` says what random weights give it: ``None`` = by role (matrices and tables
    N(0, std^2), vectors a gain 1 + N(0, gain_std^2)); ``"normal"``, ``"gain"``, ``"zeros"``,
    ``"ones"``; or a function ``(generator, shape, device) -> float32 tensor`` (a part whose vector is
    a bias or the logarithm of a decay says so here)."""
    shape: tuple
    role: str = "matrix"
    init: object = None


class CacheSpec:
    """What one run-order entry keeps per request, and how that is laid out on the device.  The cache
    storage and the manager know nothing of keys, values or states: they ask the spec.

    A spec is either *paged* (per-token rows that grow with the request: ``page_group()`` names the
    group of layers it shares pages and block tables with, ``allocate_pool`` makes the group's
    memory, ``layer_view`` hands one entry its part of it) or *per slot* (a record of fixed size per
    live request: ``allocate_state``).  Another kind of cache (latent rows, keys and values of
    different widths) is another subclass; nothing in ``cache/`` changes."""

    def page_group(self):
        """A hashable key with a ``window`` attribute (newest rows still needed, 0: all): entries with
        equal keys share one page pool, one free list and one block table per request.  ``None``:
        this cache is not paged."""
        return None

    def allocate_pool(self, n_entries: int, n_pages: int, page_size: int, dtype, device):
        """The memory of a group of ``n_entries`` paged caches; its first axis indexes the entries."""
        raise NotImplementedError

    def layer_view(self, pool, index: int):
        """What entry ``index`` of the group sees of the pool (given to its mixer as ``LayerCache.kv``)."""
        raise NotImplementedError

    def allocate_state(self, max_slots: int, device):
        """``[max_slots, ...]``: one record per slot, or ``None`` if this cache keeps none."""
        return None

    def bytes_per_token(self, element_size: int) -> int:
        """Bytes one token adds to one entry's cache (for reports)."""
        return 0


@dataclass(frozen=True)
class PageGroup:
    """Key of a group of paged caches.  ``window`` = newest rows still needed, 0 = all."""
    n_kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class PagedKVSpec(CacheSpec):
    """Per-token rows that grow with the request: keys and values in pages.
    ``window`` = number of newest keys still needed (0: all).  One (page, kv head) holds
    ``page_size`` rows of ``head_dim`` values back to back, keys row by row and values transposed."""
    n_kv_heads: int
    head_dim: int
    window: int = 0

    def page_group(self):
        return PageGroup(self.n_kv_heads, self.head_dim, self.window)

    def allocate_pool(self, n_entries, n_pages, page_size, dtype, device):
        return torch.zeros((n_entries, n_pages, 2, self.n_kv_heads, page_size, self.head_dim), dtype=dtype, device=device)

    def layer_view(self, pool, index):
        from ..kernels.ops import PagedLayerCache
        return PagedLayerCache(pool[index])

    def bytes_per_token(self, element_size):
        return 2 * self.n_kv_heads * self.head_dim * element_size


@dataclass(frozen=True)
class StateSpec(CacheSpec):
    """Per-request state of fixed size, one record per slot, zeroed when a slot is claimed."""
    shape: tuple
    dtype: torch.dtype = torch.float32

    def allocate_state(self, max_slots, device):
        return torch.zeros((max_slots, *self.shape), dtype=self.dtype, device=device)


@dataclass
class LayerCache:
    """What one run-order entry sees of the cache."""
    kv: Any = None                 # kernels.ops.PagedLayerCache or None
    group: int = -1                # index of the block table in StepState.block_tables
    state: torch.Tensor | None = None   # [max_slots, *StateSpec.shape]
    writes: bool = True            # False: the entry reads another layer's cache


@dataclass
class StepState:
    """One batch on the device.  Tokens of all requests lie one after another;
    ``tok_seq[i]`` is the index (within this step) of the request token ``i`` belongs to."""
    n_tokens: int
    n_seqs: int
    tokens: torch.Tensor           # int32 [n]
    positions: torch.Tensor        # int32 [n] absolute position of each token
    tok_seq: torch.Tensor          # int32 [n]
    seq_slots: torch.Tensor        # int32 [S] state slot of each request
    seq_q_start: torch.Tensor      # int32 [S] first row of the request in this batch
    seq_q_len: torch.Tensor        # int32 [S]
    seq_ctx_len: torch.Tensor      # int32 [S] tokens in the cache after this step
    block_tables: list             # per cache group: int32 [S, max_blocks], -1 = no page
    logit_rows: torch.Tensor       # int32 [R] rows whose logits are wanted
    host: "HostBatch"              # the same numbers on the host, for choosing kernels
    extra: dict = field(default_factory=dict)   # metadata parts asked for (step_metadata)
    scratch: dict = field(default_factory=dict)  # what parts compute once per forward pass and share between layers; emptied when a pass begins
    recorder: object = None        # set while the step is being recorded (engine/step.py): ``cut(fn)`` ends a recorded stretch


@dataclass
class HostBatch:
    """Host-side description of a batch, before upload."""
    q_starts: list
    q_lens: list
    start_pos: list                # position of each request's first token in this step
    slots: list
    n_tokens: int
    n_logit_rows: int
    ctx_bound: int | None = None   # set for a fixed-shape batch (graph replay): longest context it may ever hold
    every_row: bool = False        # the wanted rows are exactly rows 0 .. n_tokens - 1, in that order
    notes: dict = field(default_factory=dict)   # what parts found out about the batch while they laid out its metadata (``step_metadata``) and want to find again in ``step_signature`` or ``forward``

    @property
    def n_seqs(self): return len(self.q_lens)
    @property
    def all_single(self): return all(q == 1 for q in self.q_lens)
    @property
    def max_q_len(self): return max(self.q_lens) if self.q_lens else 0
    @property
    def max_ctx_len(self): return max((s + q for s, q in zip(self.start_pos, self.q_lens)), default=0)


# ---------------------------------------------------------------- interfaces
class Part:
    """Base of all parts.  Subclasses take their sizes and constants as keyword
    parameters, list their tensors, and receive them in ``bind``."""

    # True if everything the part does on the device goes through the kernel library's launch
    # functions, with arguments that are decided by the step's shape (rows per request, wanted rows,
    # table widths, buffers) and, for a mixer, by what its ``step_signature`` returns.  A model
    # of such parts can have its steps recorded and replayed from native code.  A part that calls
    # torch operations, or looks at a step's values on the host, is not.
    replayable = False

    def subparts(self) -> list:
        """The parts this part is made of (a block's mixer, norms and feed-forward; a mixer's
        position encoding)."""
        return []

    def tensors(self) -> dict:
        """``{local name: TensorSpec}``."""
        return {}

    def bind(self, weights: dict, rt) -> None:
        """Take the loaded tensors (already on the device, in the dtype their role asks for)."""
        self.rt = rt


class Product:
    """A part's output as a matrix product that is not yet computed: ``x @ weight.T`` (``weight``
    from ``rt.prepare_weight``).  A mixer or feed-forward may return it instead of the delta
    tensor; the residual stream that receives it computes it, fused with what follows where a
    kernel for that exists."""

    def __init__(self, x, weight):
        self.x = x
        self.weight = weight

    def compute(self, rt, out=None):
        """The product itself, float32 ``[n, weight.rows]``."""
        if out is None:
            out = rt.buffer("delta", self.x.shape[0], self.weight.rows, torch.float32)
        return rt.gemm(self.x, self.weight, out)


class Norm(Part):
    def forward(self, x, out, delta=None, store_sum=False, rows=None):
        """``out = norm(x (+ delta))``; ``x`` is the 32-bit residual stream; with
        ``store_sum`` the sum is written back to ``x``; ``rows`` selects rows."""
        raise NotImplementedError

    def after_product(self, rt, resid, product: Product):
        """Optional fusion: add ``product`` to ``resid`` and return the normed sum as an object
        that ``rt.gemm`` and ``rt.gemm_swiglu`` take in place of a tensor, or ``None`` if this
        norm or these sizes have no such kernel (the caller then computes the product, and
        ``forward`` norms)."""
        return None


class PositionEncoding(Part):
    def rotary_parameters(self):
        """``(rotated_dims, theta)`` if this encoding is the split-half rotation the fused
        rotate-and-store kernel implements, else ``None`` (then ``apply`` is called)."""
        return None

    def rotary_table(self, rt, step):
        """Optional: cosines and sines ``[n, rotated_dims / 2, 2]`` (float32) of the step's
        positions for the rotation of ``rotary_parameters``, or ``None`` (the kernels then compute
        the angles themselves)."""
        return None

    def apply(self, q, k, positions, n_heads, n_kv_heads, head_dim):
        """Encode positions into ``q`` and ``k`` in place (rows of the fused projection)."""
        raise NotImplementedError


class Mixer(Part):
    # True if running the same step twice leaves the cache as running it once does (keys and
    # values are written by position).  A mixer that advances a state of its own is not, and a
    # model with such a mixer never replays captured steps.
    graph_safe = False
    # True if ``forward`` hands its input ``x`` to ``rt.gemm`` / ``rt.gemm_swiglu`` only: ``x`` may
    # then be a normed input that exists in factors (see ``Norm.after_product``), not a tensor.
    lazy_input = False

    def cache_spec(self):
        """``PagedKVSpec``, ``StateSpec`` or ``None``."""
        return None

    @classmethod
    def step_metadata(cls, batch: HostBatch) -> dict:
        """Integer arrays (numpy int32) this kind of mixer wants on the device for the batch,
        uploaded with the rest of the step's metadata and found in ``StepState.extra``.  A class
        whose arrays depend on its mixers' sizes defines ``step_metadata_for(cls, batch, mixers)``
        (``mixers``: the model's mixers of this class) instead; the shapes of the arrays may depend
        on the batch's shape only."""
        return {}

    def step_signature(self, batch: HostBatch):
        """Whatever this mixer decides from the batch's numbers beyond its shape (how many ways it
        splits the keys of a long context, ...), as a hashable value: two batches of the same shape
        and the same signature must make the mixer launch the same kernels with the same arguments.
        The default is exact and rarely repeats: where every request starts."""
        return tuple(batch.start_pos)

    def signature_group(self):
        """Mixers with equal groups give equal signatures (one of them is asked per step)."""
        return id(self)

    def forward(self, x, step: StepState, cache: LayerCache):
        """``x``: normed activations [n, hidden] in the compute dtype.  Returns the
        32-bit delta [n, hidden] that is added to the residual stream, or a ``Product`` that
        computes it."""
        raise NotImplementedError


class FeedForward(Part):
    lazy_input = False      # as for Mixer

    def forward(self, x, step: StepState):
        """Returns the 32-bit delta [n, hidden], or a ``Product`` that computes it."""
        raise NotImplementedError


class Block(Part):
    """An arrangement of parts.  ``forward`` advances the residual stream by one layer."""

    def cache_spec(self):
        return None

    def forward(self, stream, step: StepState, cache: LayerCache) -> None:
        raise NotImplementedError


# ---------------------------------------------------------------- registries
class PartRegistry:
    """Registry key -> constructor, one registry per family of parts."""

    def __init__(self, family: str):
        self.family = family
        self._makers: dict[str, Callable] = {}

    def register(self, kind: str, maker: Callable | None = None):
        def deco(m):
            self._makers[kind] = m
            return m
        return deco(maker) if maker is not None else deco

    def create(self, spec: PartSpec, **more):
        try:
            maker = self._makers[spec.kind]
        except KeyError:
            known = ", ".join(sorted(self._makers)) or "(none)"
            raise KeyError(f"unknown {self.family} '{spec.kind}'; known: {known}") from None
        return maker(**spec.params, **more)

    def known(self):
        return sorted(self._makers)


EMBEDDINGS = PartRegistry("embedding")
HEADS = PartRegistry("output head")
MIXERS = PartRegistry("mixer")
FEED_FORWARDS = PartRegistry("feed-forward")
NORMS = PartRegistry("norm")
POSITION_ENCODINGS = PartRegistry("position encoding")
BLOCKS = PartRegistry("block")

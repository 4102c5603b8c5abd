"""Interfaces of the parts a layer is put together from, and their registries.

A part owns its sizes and constants (given to its constructor), says which
checkpoint tensors it needs (``weight_specs``), takes them (``bind``) and runs
(``forward``).  No part knows which model it is in: a model file only chooses
parts by name and hands them numbers from its configuration.

Kinds of parts and what each must provide:

* ``Norm``:      forward(x, branch, branch_scale, ctx, rows=None) -> normed [n or R, H]
                 (adds ``branch_scale * branch`` into the float residual ``x`` first)
* ``PositionEncoding``: rotary_params() -> (inv_freq, magnitude) or None, and
                 apply(q, k, ctx) for encodings that are not a plain rotation, and/or
                 score_bias() -> per-head slopes for encodings that bias the scores by distance
* ``Mixer``:     cache_needs() and forward(h, ctx, cache, writes_cache) -> branch [n, H] or [P, n, H]
* ``FeedForward``: forward(h, ctx) -> branch [n, H] or [P, n, H]
* ``Block``:     forward(stream, ctx, cache, writes_cache): the arrangement of the above
                 around the residual stream

Two optional protocols let neighbouring parts share a kernel without knowing each other: a norm may leave
its row factor to the product that follows (``forward_unscaled`` / ``takes_row_scale``), and a part may leave
its last product to the norm that follows (``DeferredBranch``: ``can_defer_last`` /
``takes_deferred_branch``).  A part that implements neither is handed plain tensors.

Branches may come back as float partial sums ``[P, n, H]`` of a split matrix
product; whoever adds them to the residual sums them.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Mapping, Optional, Sequence, Tuple

import torch

from ..cache.paged import CacheNeeds, CacheView, SequenceCache


# ---------------------------------------------------------------------------
# weights
# ---------------------------------------------------------------------------
@dataclass(frozen=True)
class WeightSpec:
    """A checkpoint tensor a part needs.  ``init`` names the rule by which the random-weights writer draws it
    (weights.register_init_rule; built in: 'matrix' and 'table' N(0, std), 'norm' 1 + N(0, norm_std)).
    ``storage`` is the dtype it is written in and kept in by the loader ('bfloat16', 'float32' or 'int32')."""
    name: str
    shape: Tuple[int, ...]
    init: str = "matrix"
    storage: str = "bfloat16"


# ---------------------------------------------------------------------------
# run-time objects handed to parts
# ---------------------------------------------------------------------------
class Workspace:
    """Named scratch buffers that live as long as the engine: a part asks for
    ``get(name, shape, dtype)`` and receives the same memory at every step (it
    grows when a larger shape is asked for), so steps allocate nothing and a
    captured step replays on fixed addresses."""

    def __init__(self, device):
        self.device = torch.device(device)
        self._buf: Dict[str, torch.Tensor] = {}
        self.generation = 0           # counts the times a buffer moved (captured graphs hold the old address)
        self.sealed = False           # set by the engine once it is built: what is asked for later is noted
        self.grown: List[str] = []    # names of buffers made or enlarged after that

    def get(self, name: str, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= int(s)
        nbytes = n * torch.empty((), dtype=dtype).element_size()
        buf = self._buf.get(name)
        if buf is None or buf.numel() < nbytes:
            if buf is not None:
                self.generation += 1
            buf = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=self.device)
            self._buf[name] = buf
            if self.sealed and name not in self.grown:
                self.grown.append(name)
        return buf[:nbytes].view(dtype).view(*shape)

    def bytes(self) -> int:
        return sum(b.numel() for b in self._buf.values())


@dataclass
class Runtime:
    """What an engine gives every part at bind time."""
    device: torch.device
    dtype: torch.dtype            # element type of activations, weights and cache: float32 or bfloat16
    workspace: Workspace
    max_seq_len: int              # longest sequence the engine holds
    tiled_weights: bool = True    # keep a second copy of linear weights in the decode product's layout
    page_size: int = 64           # tokens a cache page


class _NoTimer:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_TIMER = _NoTimer()


@dataclass
class StepContext:
    """One step's batch as every part sees it: packed tokens of several sequences."""
    n_tokens: int
    n_seqs: int
    token_ids: torch.Tensor       # int32 [n]
    positions: torch.Tensor       # int32 [n] absolute position of each token in its sequence
    tok_slot: torch.Tensor        # int32 [n] cache slot of each token
    cu_q: torch.Tensor            # int32 [B+1] start of each sequence's tokens in the packed batch
    seq_slot: torch.Tensor        # int32 [B]
    seq_len: torch.Tensor         # int32 [B] tokens each sequence holds after this step
    q_lens: List[int]             # host copies
    kv_lens: List[int]
    max_pos: int                  # largest position in the step
    single_token: bool            # every sequence brings exactly one token
    ws: Workspace
    cache: Optional[SequenceCache]
    logit_rows: Optional[torch.Tensor] = None     # int32 [R]: packed token rows whose logits are wanted
    extras: Dict[str, object] = field(default_factory=dict)   # what kernels derive from the batch once a step
    perf: Optional[object] = None                 # label-keyed timers (utils.perf.PerfTimers) when switched on

    def timed(self, label: str):
        """A context manager that times the GPU work inside it under ``prefill_<label>`` or ``decode_<label>``
        while the timers are switched on, and does nothing otherwise.  The reference's labels make the same
        distinction (src/model/minicpm4/minicpm4_layer.cuh:46-83, minicpm4_attn.cuh:107-202)."""
        if self.perf is None or not self.perf.enabled:
            return _NO_TIMER
        return self.perf.gpu(("decode_" if self.single_token else "prefill_") + label)


class DeferredBranch:
    """A branch whose last linear layer has not run yet: branch = ``linear``(``a``).  A part that is asked to
    (``forward(..., defer_last=True)``) may hand this back instead of a tensor; a norm that knows a kernel which
    runs that product together with the residual add takes it as it is (``Norm.takes_deferred_branch``), for
    everybody else ``evaluate()`` runs the product as the part would have and gives the tensor."""

    def __init__(self, linear, a: torch.Tensor, ctx: "StepContext", tag: str):
        self.linear, self.a, self.ctx, self.tag = linear, a, ctx, tag
        self._value: Optional[torch.Tensor] = None

    def evaluate(self) -> torch.Tensor:
        if self._value is None:
            self._value = self.linear.forward(self.a, self.ctx, self.tag, out_dtype=torch.float32, partials=True)
        return self._value


def branch_tensor(branch):
    """The branch as a tensor (or None), whatever form it was handed over in."""
    return branch.evaluate() if isinstance(branch, DeferredBranch) else branch


class ResidualStream:
    """The float residual ``x`` [n, H] and a branch not yet added to it.  ``pending`` reads as a tensor;
    ``take_pending()`` gives it in the form it was left in, which may be a DeferredBranch."""

    def __init__(self, x: torch.Tensor, pending=None, pending_scale: float = 1.0):
        self.x = x
        self._pending = pending
        self.pending_scale = pending_scale

    @property
    def pending(self) -> Optional[torch.Tensor]:
        self._pending = branch_tensor(self._pending)
        return self._pending

    @pending.setter
    def pending(self, value):
        self._pending = value

    def take_pending(self):
        return self._pending


# ---------------------------------------------------------------------------
# the part interfaces
# ---------------------------------------------------------------------------
class Part:
    def parts(self) -> List["Part"]:
        return []

    def weight_specs(self) -> List[WeightSpec]:
        return []

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        """Take the tensors named by weight_specs (already on the device) and prepare for forward."""

    # False for a part whose forward reads device data on the host, allocates, or launches different work from
    # step to step (a router that counts tokens per expert, a recurrence that loops in Python over lengths):
    # such a forward cannot be recorded once and replayed.  An engine whose model holds one runs every step
    # eagerly, whatever its hip_graph option says.
    graph_capturable = True

    def reserve_workspace(self, ws: "Workspace", rt: Runtime, max_step_tokens: int, max_slots: int):
        """Called once when the engine is built, after bind: ask ``ws`` for the scratch whose size grows with the
        context (``rt.max_seq_len``) rather than with the step, so that it is part of the engine's memory figure
        and no later step has to grow it.  Scratch that depends on the step's tokens only is sized by the
        engine's rehearsal passes and needs nothing here."""

    # helpers over the tree
    def all_parts(self) -> List["Part"]:
        out: List["Part"] = [self]
        for p in self.parts():
            out.extend(p.all_parts())
        return out

    def all_weight_specs(self) -> List[WeightSpec]:
        out = list(self.weight_specs())
        for p in self.parts():
            out.extend(p.all_weight_specs())
        return out

    def bind_all(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.bind(tensors, rt)
        for p in self.parts():
            p.bind_all(tensors, rt)


class Norm(Part):
    def forward(self, x: torch.Tensor, branch: Optional[torch.Tensor], branch_scale: float, ctx: StepContext,
                rows: Optional[torch.Tensor] = None, tag: str = "norm") -> torch.Tensor:
        raise NotImplementedError

    def forward_unscaled(self, x: torch.Tensor, branch: Optional[torch.Tensor], branch_scale: float,
                         ctx: StepContext, tag: str = "norm"):
        """For a norm whose result is (one number a row) * (something computed column by column), and a consumer
        that begins with a linear layer: add the branch as forward does and return (rows without the row
        factor, ops.RowScale that yields it), for the consumer's product to multiply its result by.  None if
        this norm, or this step, has no such form; the caller then uses forward.  Only called when the
        consumer's takes_row_scale() said yes."""
        return None

    # True if forward and forward_unscaled accept a DeferredBranch as ``branch``
    takes_deferred_branch = False


class PositionEncoding(Part):
    def rotary_params(self) -> Optional[Tuple[torch.Tensor, float]]:
        """(inv_freq float32 [head_dim/2], magnitude) if this encoding is a rotate-half rotation by
        position * inv_freq, which the fused kernel applies while it writes the cache; else None."""
        return None

    def apply(self, q: torch.Tensor, k: Optional[torch.Tensor], ctx: StepContext):
        """Encode positions into q [n, heads, hd] and k [n, kv_heads, hd] in place (used when
        rotary_params() is None and a subclass defines it)."""
        raise NotImplementedError

    def score_bias(self) -> Optional[torch.Tensor]:
        """float32 [heads] on the device, or None: an encoding that lowers the score of key j for the query at
        position p by slope[head] * (p - j) instead of (or beside) changing q and k.  The attention kernels
        take it as it is; nothing about positions is then stored in the cache."""
        return None

    def rewrites_vectors(self) -> bool:
        """Whether ``apply`` is this encoding's own (an encoding that only biases scores leaves it out)."""
        return type(self).apply is not PositionEncoding.apply


class Mixer(Part):
    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds()

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True
                ) -> torch.Tensor:
        raise NotImplementedError

    def takes_row_scale(self, n: int, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool) -> bool:
        """True if forward, for this step of n tokens, accepts ``row_scale=`` (Norm.forward_unscaled) beside h.
        A subclass that overrides forward of a mixer that says yes takes the argument too, or says no here."""
        return False

    # True (set in the class that defines ``forward``) if that forward accepts ``defer_last=True`` and may then
    # return a DeferredBranch
    can_defer_last = False


class FeedForward(Part):
    def forward(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError

    def takes_row_scale(self, n: int, ctx: StepContext) -> bool:
        """True if forward, for this step of n tokens, accepts ``row_scale=`` (Norm.forward_unscaled) beside h."""
        return False

    # True if forward accepts ``defer_last=True`` and may then return a DeferredBranch
    can_defer_last = False


def forward_declares(part: Part, flag: str) -> bool:
    """Whether the class that defines ``part.forward`` sets the class attribute ``flag`` itself.  Optional
    protocols that add a keyword to ``forward`` (``can_defer_last``) are declared beside the ``forward`` that
    implements them: a subclass that overrides ``forward`` and says nothing is not handed the keyword."""
    for cls in type(part).__mro__:
        if "forward" in cls.__dict__:
            return bool(cls.__dict__.get(flag, False))
    return False


class Block(Part):
    mixer: Mixer

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        raise NotImplementedError


# ---------------------------------------------------------------------------
# registries: kind name -> constructor
# ---------------------------------------------------------------------------
class Registry:
    def __init__(self, what: str):
        self.what = what
        self._items: Dict[str, Callable] = {}

    def register(self, name: str, ctor: Optional[Callable] = None):
        def deco(c):
            if name in self._items and self._items[name] is not c:
                raise ValueError(f"{self.what} '{name}' is already registered")
            self._items[name] = c
            return c
        return deco if ctor is None else deco(ctor)

    def unregister(self, name: str):
        self._items.pop(name, None)

    def get(self, name: str) -> Callable:
        try:
            return self._items[name]
        except KeyError:
            raise KeyError(f"unknown {self.what} '{name}' (registered: {sorted(self._items)})") from None

    def build(self, kind: str, /, **params):
        return self.get(kind)(**params)

    def names(self):
        return sorted(self._items)


NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
BLOCKS = Registry("block")


@dataclass(frozen=True)
class PartSpec:
    """A part chosen by name with its parameters: what a model file writes per layer."""
    kind: str
    params: Tuple[Tuple[str, object], ...] = ()

    @staticmethod
    def of(kind: str, **params) -> "PartSpec":
        return PartSpec(kind, tuple(sorted(params.items())))

    def build(self, registry: Registry, **extra):
        return registry.build(self.kind, **dict(self.params), **extra)

"""What every part has in common: a registry by (category, kind), the builder that turns a
description into parts, and the context a step hands to them.

A part is built from its ``PartSpec`` alone (sizes, constants, parameters, sub-parts); it does not know
which model it is in.  Interfaces, by category:

  norm          ``__call__(x, delta=None, update=False, rows=None, out_dtype=None)`` -> normed rows.  x is the
                float32 residual stream [n, width]; ``delta`` is a branch output still to be added (added in
                32-bit; with ``update`` the sum is written back to x); ``rows`` selects rows.
  position      ``tables(ctx)`` -> (cos, sin) float32 [n, rotary_dim/2] for the step's tokens, or None; fields
                ``rotary_dim`` and ``pairing`` ("half_split" | "interleaved").
  mixer         ``forward(h, ctx)`` -> branch output [n, hidden]; ``cache_needs(spec)`` (static) -> what it
                keeps per sequence (``KVNeed`` / ``StateNeed``); reads ``ctx.layer_cache``.
  feed_forward  ``forward(h, ctx)`` -> branch output [n, hidden].
                A mixer or feed-forward may set ``takes_sink = True`` and have ``forward(h, ctx, sink=None)``: h
                may then be ``Prenormed`` rows, and with a sink the part returns what the sink's norm makes of
                the residual stream after its output is added (parts/residual.py), usually by handing the sink
                to its last ``Linear``.
  block         ``entry_norm``: the norm applied to the residual stream before the block's first branch;
                ``forward(x, h, ctx, sink)`` -> normed rows: x is the residual stream (updated in place), h is
                ``entry_norm`` of x (a tensor or ``Prenormed`` rows), sink names the norm that reads x after the
                block and the rows it wants; what that norm gives is returned.
  embedding     ``forward(token_ids)`` -> float32 [n, hidden].
  head          ``forward(h)`` -> float32 logits [rows, vocab].
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..config.spec import PartSpec

CATEGORIES = ("norm", "position", "mixer", "feed_forward", "block", "embedding", "head")
_REGISTRY: dict[tuple[str, str], type] = {}


def register_part(category: str, kind: str):
    """Class decorator: make ``kind`` available under ``category``.  Registering a kind again replaces
    it (a test may swap a toy part in and out)."""
    if category not in CATEGORIES:
        raise ValueError(f"part category {category!r} is not one of {CATEGORIES}")

    def deco(cls):
        _REGISTRY[(category, kind)] = cls
        cls.category, cls.kind = category, kind
        return cls
    return deco


def part_class(category: str, kind: str) -> type:
    try:
        return _REGISTRY[(category, kind)]
    except KeyError:
        known = sorted(k for c, k in _REGISTRY if c == category)
        raise KeyError(f"no {category} part of kind {kind!r}; registered: {', '.join(known)}") from None


def cache_needs(spec: PartSpec) -> list:
    """What the part described by ``spec`` keeps per sequence (blocks pass their mixer's needs on)."""
    cls = part_class(spec.category, spec.kind)
    fn = getattr(cls, "cache_needs", None)
    return list(fn(spec)) if fn else []


class Builder:
    """Builds parts from descriptions; hands them their parameters and the run's precision."""

    def __init__(self, weights, dtype: torch.dtype, device):
        self.weights, self.dtype, self.device = weights, dtype, torch.device(device)

    def build(self, spec: PartSpec):
        return part_class(spec.category, spec.kind)(spec, self)

    def tensor(self, spec: PartSpec, name: str) -> torch.Tensor:
        return self.weights.get(spec.tensors[name])


@dataclass
class StepContext:
    """The tokens of one step, packed: sequence b brings ``seq_new[b]`` tokens, rows
    ``cu_new[b] .. cu_new[b+1]`` of every [n, ...] tensor, at positions ``seq_start[b] ..``."""
    n_tokens: int
    n_seqs: int
    max_new: int                 # the longest run of new tokens in the step
    max_total: int               # the longest sequence after the step
    dtype: torch.dtype           # element type of activations
    token_ids: torch.Tensor      # int32 [n]
    positions: torch.Tensor      # int32 [n]
    tok_slot: torch.Tensor       # int32 [n]   the cache slot of each token's sequence
    seq_slot: torch.Tensor       # int32 [B]
    seq_start: torch.Tensor      # int32 [B]   length before the step
    seq_new: torch.Tensor        # int32 [B]
    cu_new: torch.Tensor         # int32 [B + 1]
    is_decode: bool = False      # every sequence brings exactly one token
    decode_slices: int = 0       # if set: into how many slices decode attention cuts a key range (else chosen per call)
    layer_cache: object = None   # the LayerCache of the run-order entry that is running
    memo: dict = field(default_factory=dict)   # what parts make once per step (rotation tables)
    host: dict = field(default_factory=dict)   # the same facts as Python lists, for parts that plan on the host


def context_ints(n_tokens: int, n_seqs: int) -> int:
    """How many int32 a step's index arrays take together."""
    return 3 * n_tokens + 4 * n_seqs + 1


def make_context(slots, starts, new_tokens, dtype, device, max_total=None, into: torch.Tensor | None = None,
                 max_new: int | None = None, staging: torch.Tensor | None = None) -> StepContext:
    """A context from host lists: ``new_tokens[b]`` is the list of token ids of sequence b.  This is the one place
    where a step's arrays are laid out: a part that needs one more of them finds it here.

    ``into``: an int32 device buffer of ``context_ints(n, B)`` elements to lay the arrays in instead of a new
    one: a recorded step keeps its arrays at fixed addresses and gets new contents before every replay.
    ``max_new``, ``max_total``: bounds to size launches by instead of the step's own longest run and sequence (a
    recorded step is sized for the largest step it will be replayed for).
    ``staging`` (with ``into``): a pinned host buffer of the same size through which the arrays go to the device
    without the host waiting for the device; the caller must not write it again before that copy has run."""
    # laid out with numpy: a prompt of some thousand tokens as Python lists costs the host a millisecond before the
    # first kernel is launched
    counts = [len(t) for t in new_tokens]
    cu = [0]
    for c in counts:
        cu.append(cu[-1] + c)
    n, B = cu[-1], len(slots)
    packed = np.empty((context_ints(n, B),), dtype=np.int32)
    for b in range(B):
        lo, hi = cu[b], cu[b + 1]
        packed[lo:hi] = new_tokens[b]
        packed[n + lo:n + hi] = np.arange(starts[b], starts[b] + counts[b], dtype=np.int32)
        packed[2 * n + lo:2 * n + hi] = slots[b]
    o = 3 * n
    for arr in (slots, starts, counts, cu):
        packed[o:o + len(arr)] = arr
        o += len(arr)
    host = torch.from_numpy(packed)
    if into is None:
        flat = host.to(device)
    else:
        if into.shape != host.shape or into.dtype != torch.int32:
            raise ValueError(f"a step of {n} tokens in {B} sequences needs {host.numel()} int32, the buffer has {tuple(into.shape)}")
        flat = into
        if staging is None:
            flat.copy_(host)
        else:
            staging.copy_(host)
            flat.copy_(staging, non_blocking=True)
    o = 0
    parts = []
    for size in (n, n, n, B, B, B, B + 1):
        parts.append(flat[o:o + size])
        o += size
    return StepContext(
        n_tokens=n, n_seqs=B, max_new=max_new if max_new is not None else (max(counts) if counts else 0),
        max_total=max_total if max_total is not None else max((s + c for s, c in zip(starts, counts)), default=0),
        dtype=dtype, token_ids=parts[0], positions=parts[1], tok_slot=parts[2], seq_slot=parts[3], seq_start=parts[4],
        seq_new=parts[5], cu_new=parts[6], is_decode=all(c == 1 for c in counts),
        host={"slots": list(slots), "starts": list(starts), "counts": counts, "cu": cu},
    )

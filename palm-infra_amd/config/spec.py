"""What a model is made of, as data.

A configuration class of an architecture turns its ``config.json`` into a :class:`ModelSpec`: a tree
of :class:`PartSpec` (kind, sizes and constants, where each parameter comes from in the checkpoint)
and the order in which the layers run.  The loader, the random-weights writer, the cache planner and
the model builder all read this one description; none of them knows an architecture by name.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Iterator, Mapping

# What a parameter is used as decides how it is kept in memory:
#   matrix, table : bfloat16 in the bfloat16 mode (32-bit if the file stores it in 32-bit)
#   vector        : always float32 (norm weights, biases: the widening is exact)
#   integer       : int32
ROLES = ("matrix", "table", "vector", "integer")


@dataclass(frozen=True)
class Stored:
    """How a piece of a parameter lies in the checkpoint when it is not a whole tensor in the parameter's own layout:
    the stored tensor has shape ``shape``; of it the rows ``rows = (a, b)`` are taken (None: all); ``transposed``: what
    was taken is the transpose of the piece (a matrix that the checkpoint keeps as [in, out]).  So a checkpoint that
    stores q, k and v fused in one tensor, in any order, is three pieces with three row ranges of one name."""
    shape: tuple[int, ...]
    rows: tuple[int, int] | None = None
    transposed: bool = False

    def piece_shape(self) -> tuple[int, ...]:
        shape = tuple(self.shape)
        if self.rows is not None:
            a, b = self.rows
            if not shape or not 0 <= a < b <= shape[0]:
                raise ValueError(f"rows {a}:{b} do not lie in a stored tensor of shape {shape}")
            shape = (b - a,) + shape[1:]
        if self.transposed:
            if len(shape) != 2:
                raise ValueError(f"only a matrix can be stored transposed, not a tensor of shape {shape}")
            shape = (shape[1], shape[0])
        return shape


@dataclass(frozen=True)
class TensorRef:
    """One parameter of a part: one or more pieces, joined along their rows.  Piece i is the checkpoint tensor
    ``names[i]`` and has shape ``shapes[i]`` in the parameter; usually it is that tensor whole and as stored, else
    ``stored[i]`` says how it lies in the tensor (a range of its rows, transposed)."""
    names: tuple[str, ...]
    shapes: tuple[tuple[int, ...], ...]
    role: str = "matrix"
    # how the random-weights writer fills it: ("normal", mean, std)
    init: tuple = ("normal", 0.0, 0.02)
    stored: tuple = ()          # empty, or one ``Stored`` or None for each piece

    def __post_init__(self):
        if self.role not in ROLES:
            raise ValueError(f"TensorRef role {self.role!r} is not one of {ROLES}")
        if len(self.names) != len(self.shapes) or not self.names:
            raise ValueError("TensorRef needs one shape for each name")
        tail = self.shapes[0][1:]
        if any(s[1:] != tail for s in self.shapes):
            raise ValueError(f"tensors {self.names} cannot be joined along rows: shapes {self.shapes}")
        if self.stored:
            if len(self.stored) != len(self.names):
                raise ValueError("TensorRef needs one entry of `stored` (or None) for each name")
            for name, shape, how in zip(self.names, self.shapes, self.stored):
                if how is not None and tuple(how.piece_shape()) != tuple(shape):
                    raise ValueError(f"piece {name}: what is taken of the stored tensor has shape {how.piece_shape()}, "
                                     f"the parameter expects {tuple(shape)}")

    @property
    def shape(self) -> tuple[int, ...]:
        rows = sum(s[0] for s in self.shapes)
        return (rows,) + tuple(self.shapes[0][1:])

    @property
    def key(self) -> tuple:
        """What tells this parameter from every other one (two parameters may take different rows of one tensor)."""
        return (self.names, self.stored) if any(h is not None for h in self.stored) else self.names

    def pieces(self):
        """(name, shape in the parameter, Stored or None) for each piece, in the order of the rows."""
        stored = self.stored or (None,) * len(self.names)
        return list(zip(self.names, self.shapes, stored))

    def stored_shapes(self):
        """(name, shape as the checkpoint stores the tensor) for each piece."""
        return [(name, tuple(how.shape) if how is not None else tuple(shape)) for name, shape, how in self.pieces()]


def tensor(name: str, shape, role: str = "matrix", init=("normal", 0.0, 0.02), stored: Stored | None = None) -> TensorRef:
    return TensorRef((name,), (tuple(int(s) for s in shape),), role, tuple(init), (stored,) if stored is not None else ())


def joined(names, shapes, role: str = "matrix", init=("normal", 0.0, 0.02), stored=()) -> TensorRef:
    return TensorRef(tuple(names), tuple(tuple(int(x) for x in s) for s in shapes), role, tuple(init), tuple(stored))


@dataclass(frozen=True)
class PartSpec:
    """A part of a model: its category (norm, position, mixer, feed_forward, block, embedding,
    head), the kind registered under that category, its sizes and constants, the checkpoint tensors
    of its parameters, and the parts it is built from."""
    category: str
    kind: str
    params: Mapping[str, object] = field(default_factory=dict)
    tensors: Mapping[str, TensorRef] = field(default_factory=dict)
    parts: Mapping[str, "PartSpec"] = field(default_factory=dict)

    def walk(self) -> Iterator["PartSpec"]:
        yield self
        for child in self.parts.values():
            yield from child.walk()


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order: which layer runs, and whose cache it uses.  ``cache_of`` names an
    earlier entry of the order (by its index in the order); the call then reads that entry's cache
    and writes none of its own."""
    layer: int
    cache_of: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    # the longest sequence the model itself can take (a learned position table has a last row); None if only the
    # cache bounds it, as with rotation, whose angles are computed from the position
    max_positions: int | None
    embedding: PartSpec
    layers: tuple[PartSpec, ...]
    order: tuple[LayerCall, ...]
    final_norm: PartSpec
    head: PartSpec
    stop_token_ids: tuple[int, ...] = ()

    def __post_init__(self):
        for i, call in enumerate(self.order):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"run order entry {i} names layer {call.layer}; there are {len(self.layers)}")
            if call.cache_of is not None:
                if not 0 <= call.cache_of < i:
                    raise ValueError(f"run order entry {i} reads the cache of entry {call.cache_of}, "
                                     "which does not run before it")
                if self.order[call.cache_of].cache_of is not None:
                    raise ValueError(f"run order entry {i} reads the cache of entry {call.cache_of}, "
                                     "which holds none of its own")

    def parts(self) -> Iterator[PartSpec]:
        yield from self.embedding.walk()
        for layer in self.layers:
            yield from layer.walk()
        yield from self.final_norm.walk()
        yield from self.head.walk()

    def tensor_refs(self) -> list[TensorRef]:
        """Every parameter of the model once (a tied head names the embedding's tensor again)."""
        seen, out = set(), []
        for part in self.parts():
            for ref in part.tensors.values():
                if ref.key not in seen:
                    seen.add(ref.key)
                    out.append(ref)
        return out

    def expected_tensors(self) -> dict[str, tuple[tuple[int, ...], str]]:
        """Checkpoint tensor name -> (shape as stored, role)."""
        out = {}
        for ref in self.tensor_refs():
            for name, shape in ref.stored_shapes():
                if name in out and out[name][0] != shape:
                    raise ValueError(f"tensor {name} is used with two shapes: {out[name][0]} and {shape}")
                out[name] = (shape, ref.role)
        return out

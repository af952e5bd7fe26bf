"""Binding a checkpoint's tensors to a model's parameters by name.

The reference renames, re-types and merges tensors in its converter (models/qwen3.py:57-168): q, k
and v rows are joined into one matrix, gate and up likewise, norm weights are kept in 32-bit, and
``lm_head.weight`` stands for the head if the file has it, else the embedding.  Here the model's
description names the checkpoint tensors of every parameter (``TensorRef``: whole tensors joined along
their rows, or a range of a stored tensor's rows, or a stored tensor's transpose), and this loader
checks all of them before it copies anything.  Tensors that the model does not name are an error
unless the caller says ``strict=False``; they are then listed and left alone, as the reference leaves
them (models/qwen3.py:105-106).

Precision of what is kept: in the ``bfloat16`` mode matrices and tables are bfloat16 unless the file
stores them in 32-bit (those stay 32-bit; float16 is re-rounded to bfloat16), vectors are widened to
float32 (exact), integer tables are int32.  In the ``float32`` mode every float tensor is float32.
"""
from __future__ import annotations

import sys

import torch

from ..config.spec import ModelSpec, TensorRef
from ..kernels import ops
from .random_numbers import tensor_key
from .safetensors_io import ModelFiles

_FLOAT_NAMES = ("F32", "F16", "BF16", "F64")
_INT_NAMES = ("I64", "I32", "I16", "I8", "U8")


class WeightError(ValueError):
    """The checkpoint does not hold what the model needs.  ``missing``, ``unexpected`` and
    ``wrong_shape`` list everything that is wrong, not only the first fault."""

    def __init__(self, where, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_dtype = list(wrong_shape), list(wrong_dtype)
        lines = [f"weights in {where} do not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n}: expected {list(e)}, file has {list(g)}" for n, e, g in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  wrong dtypes ({len(self.wrong_dtype)}): " + "; ".join(
                f"{n}: {why}" for n, why in self.wrong_dtype))
        super().__init__("\n".join(lines))


def check_names(spec: ModelSpec, shapes: dict[str, tuple], dtypes: dict[str, str] | None = None, where="checkpoint",
                strict: bool = True) -> list[str]:
    """Compare the tensors a checkpoint holds (name -> shape) with the model's; raise one error that
    lists all missing and unexpected tensors and all wrong shapes.  With ``strict=False`` tensors that the
    model does not name are no error: their names are returned (the warning list) and nothing else is done
    with them."""
    expected = spec.expected_tensors()
    missing = [n for n in expected if n not in shapes]
    unexpected = [n for n in shapes if n not in expected]
    wrong = [(n, expected[n][0], tuple(shapes[n])) for n in expected
             if n in shapes and tuple(shapes[n]) != tuple(expected[n][0])]
    wrong_dtype = []
    if dtypes is not None:
        for n, (_, role) in expected.items():
            if n not in dtypes:
                continue
            if role == "integer" and dtypes[n] not in _INT_NAMES:
                wrong_dtype.append((n, f"an integer table is stored as {dtypes[n]}"))
            if role != "integer" and dtypes[n] not in _FLOAT_NAMES:
                wrong_dtype.append((n, f"a float tensor is stored as {dtypes[n]}"))
    if missing or wrong or wrong_dtype or (unexpected and strict):
        raise WeightError(where, missing, unexpected, wrong, wrong_dtype)
    return unexpected


def kept_dtype(ref: TensorRef, stored: list[str], mode: torch.dtype) -> torch.dtype:
    if ref.role == "integer":
        return torch.int32
    if mode == torch.float32 or ref.role == "vector":
        return torch.float32
    if any(s in ("F32", "F64") for s in stored):
        return torch.float32
    return torch.bfloat16


class Weights:
    """The parameters of a model on the device, looked up by the ``TensorRef`` that names them."""

    def __init__(self, tensors: dict[tuple[str, ...], torch.Tensor]):
        self._tensors = tensors

    def get(self, ref: TensorRef) -> torch.Tensor:
        return self._tensors[ref.key]

    def nbytes(self) -> int:
        seen, total = set(), 0
        for t in self._tensors.values():
            if t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        return total


def _convert_on_device(stored: torch.Tensor, part: torch.Tensor, transposed: bool = False) -> None:
    """The file's bytes go up as they are stored; the transpose of a matrix that the checkpoint keeps the other way
    round, the conversion into the kept type and the placing into the parameter's rows are the device's (the
    reference converts and joins when it packs a model, models/qwen3.py:125-160)."""
    up = stored.to(part.device)
    ops.convert_into(up.t().contiguous() if transposed else up, part)


def _taken(tensor: torch.Tensor, how) -> torch.Tensor:
    """The rows of a stored tensor that a piece takes (a view; a transpose is left to ``place``)."""
    if how is None or how.rows is None:
        return tensor
    return tensor[how.rows[0]:how.rows[1]]


def load_weights(spec: ModelSpec, files: ModelFiles, mode: torch.dtype, device, place=_convert_on_device,
                 strict: bool = True, warn=None) -> Weights:
    """``place(stored tensor of the file, rows of the parameter, transposed)`` puts a checkpoint tensor (or the rows
    taken of it) where it belongs; the default converts on the device.  (Tests of the binding alone, which run
    without a GPU, hand in a stand-in.)  ``strict=False``: tensors the model does not name are reported through
    ``warn(names)`` (default: one line on standard error) instead of refused."""
    names = files.names()
    where = str(files.files[0].path.parent)
    extra = check_names(spec, {n: files.shape(n) for n in names}, {n: files.dtype_name(n) for n in names},
                        where=where, strict=strict)
    if extra:
        if warn is None:
            print(f"[palm_infra_amd] {where}: {len(extra)} tensors that the model does not name are left alone: "
                  + ", ".join(extra), file=sys.stderr, flush=True)
        else:
            warn(extra)
    out = {}
    for ref in spec.tensor_refs():
        dt = kept_dtype(ref, [files.dtype_name(n) for n in ref.names], mode)
        dst = torch.empty(ref.shape, dtype=dt, device=device)
        row = 0
        for name, shape, how in ref.pieces():
            part = dst[row:row + shape[0]] if shape else dst
            stored = _taken(files.tensor(name), how)
            transposed = how is not None and how.transposed
            if ref.role == "integer":
                part.copy_((stored.t() if transposed else stored).to(torch.int32))
            elif transposed:
                place(stored, part, True)
            else:
                place(stored, part)
            row += shape[0] if shape else 0
        out[ref.key] = dst
    return Weights(out)


def random_weights(spec: ModelSpec, seed: int, mode: torch.dtype, device) -> Weights:
    """Random parameters made on the device without a file (for measurements at sizes whose folder would be
    tens of gigabytes).  They are, bit for bit, what ``load_weights`` gives for the folder that
    ``write_random_model(config, seed, folder, "bfloat16")`` writes: both take element i of checkpoint tensor
    ``name`` from ``random_numbers``' function of (seed, name, i), rounded to bfloat16 as the folder stores it,
    and kept as the mode keeps it (vectors, and everything in the float32 mode, widened to float32)."""
    out = {}
    for ref in spec.tensor_refs():
        dt = kept_dtype(ref, ["BF16"], mode)
        dst = torch.zeros(ref.shape, dtype=dt, device=device)
        row = 0
        for name, shape, how in ref.pieces():
            if ref.role != "integer":
                _, mean, std = ref.init
                part = dst[row:row + shape[0]] if shape else dst
                if how is None and dt == torch.bfloat16:
                    ops.random_fill(part, tensor_key(seed, name), mean, std)
                else:
                    # the tensor as a folder would store it (element i of tensor `name`), then what a load does with it
                    stored = torch.empty(how.shape if how is not None else part.shape, dtype=torch.bfloat16, device=device)
                    ops.random_fill(stored, tensor_key(seed, name), mean, std)
                    _convert_on_device(_taken(stored, how), part, how is not None and how.transposed)
            row += shape[0] if shape else 0
        out[ref.key] = dst
    return Weights(out)

"""Binding a checkpoint's tensors to a model's parameters by name.

The reference renames, re-types and merges tensors in its converter (models/qwen3.py:57-168): q, k
and v rows are joined into one matrix, gate and up likewise, norm weights are kept in 32-bit, and
``lm_head.weight`` stands for the head if the file has it, else the embedding.  Here the model's
description names the checkpoint tensors of every parameter (``TensorRef``), and this loader
checks all of them before it copies anything.

Precision of what is kept: in the ``bfloat16`` mode matrices and tables are bfloat16 unless the file
stores them in 32-bit (those stay 32-bit; float16 is re-rounded to bfloat16), vectors are widened to
float32 (exact), integer tables are int32.  In the ``float32`` mode every float tensor is float32.
"""
from __future__ import annotations

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


def check_names(spec: ModelSpec, shapes: dict[str, tuple], dtypes: dict[str, str] | None = None, where="checkpoint"):
    """Compare the tensors a checkpoint holds (name -> shape) with the model's; raise one error that
    lists all missing and unexpected tensors and all wrong shapes."""
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
    if missing or unexpected or wrong or wrong_dtype:
        raise WeightError(where, missing, unexpected, wrong, wrong_dtype)


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
        return self._tensors[ref.names]

    def nbytes(self) -> int:
        seen, total = set(), 0
        for t in self._tensors.values():
            if t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        return total


def _convert_on_device(stored: torch.Tensor, part: torch.Tensor) -> None:
    """The file's bytes go up as they are stored; the conversion into the kept type and into the parameter's
    rows is the device's (the reference converts and joins when it packs a model, models/qwen3.py:125-160)."""
    ops.convert_into(stored.to(part.device), part)


def load_weights(spec: ModelSpec, files: ModelFiles, mode: torch.dtype, device, place=_convert_on_device) -> Weights:
    """``place(stored tensor of the file, rows of the parameter)`` puts a checkpoint tensor where it belongs; the
    default converts on the device.  (Tests of the binding alone, which run without a GPU, hand in a stand-in.)"""
    names = files.names()
    check_names(spec, {n: files.shape(n) for n in names}, {n: files.dtype_name(n) for n in names},
                where=str(files.files[0].path.parent))
    out = {}
    for ref in spec.tensor_refs():
        dt = kept_dtype(ref, [files.dtype_name(n) for n in ref.names], mode)
        dst = torch.empty(ref.shape, dtype=dt, device=device)
        row = 0
        for name, shape in zip(ref.names, ref.shapes):
            part = dst[row:row + shape[0]] if shape else dst
            if ref.role == "integer":
                part.copy_(files.tensor(name).to(torch.int32))
            else:
                place(files.tensor(name), part)
            row += shape[0] if shape else 0
        out[ref.names] = dst
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
        for name, shape in zip(ref.names, ref.shapes):
            if ref.role != "integer":
                _, mean, std = ref.init
                part = dst[row:row + shape[0]] if shape else dst
                if dt == torch.bfloat16:
                    ops.random_fill(part, tensor_key(seed, name), mean, std)
                else:
                    stored = torch.empty(part.shape, dtype=torch.bfloat16, device=device)
                    ops.random_fill(stored, tensor_key(seed, name), mean, std)
                    ops.convert_into(stored, part)
            row += shape[0] if shape else 0
        out[ref.names] = dst
    return Weights(out)

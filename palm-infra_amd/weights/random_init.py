"""The random-weights mode: write a model folder (config.json, model.safetensors) from a
configuration and a seed.

The reference has this only as a test fixture (tests/run_tiny_qwen3_cpu_e2e.py:52-95).  Here matrices
and the embedding are N(0, 0.02) and norm weights 1 + N(0, 0.02), as each parameter's description
says.  A tensor's values depend on the seed, on the tensor's name and on the element's index only
(``random_numbers``), so a model with more layers starts with the same layers, and the folder written here
holds the same numbers as ``loader.random_weights`` makes on the device.
"""
from __future__ import annotations

import json
from pathlib import Path

import torch

from ..config.registry import config_from_dict, config_source
from .random_numbers import normal, tensor_key
from .safetensors_io import write_safetensors

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def random_tensors(spec, seed: int, dtype: str = "bfloat16") -> dict[str, torch.Tensor]:
    if dtype not in _STORE:
        raise ValueError(f"dtype {dtype!r} is not one of {sorted(_STORE)}")
    out = {}
    for ref in spec.tensor_refs():
        for name, shape in ref.stored_shapes():          # the tensors as the checkpoint stores them, each once
            if name in out:
                continue
            if ref.role == "integer":
                out[name] = torch.zeros(shape, dtype=torch.int32)
                continue
            _, mean, std = ref.init
            count = 1
            for extent in shape:
                count *= int(extent)
            t = torch.from_numpy(normal(tensor_key(seed, name), count, mean, std)).reshape(shape)
            out[name] = t.to(_STORE[dtype])
    return out


def write_random_model(config, seed: int, out_dir, dtype: str = "bfloat16") -> Path:
    """``config`` is a typed configuration or the dict of a config.json."""
    if isinstance(config, dict):
        config = config_from_dict(config)
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    raw = config.to_dict()
    raw["torch_dtype"] = dtype
    (out_dir / "config.json").write_text(json.dumps(raw, indent=2))
    write_safetensors(out_dir / "model.safetensors", random_tensors(config.spec(), seed, dtype),
                      metadata={"format": "pt", "seed": seed})
    return out_dir


def main(argv=None) -> int:
    """``python -m palm_infra_amd.weights.random_init --config config.json --seed 0 --out DIR``"""
    import argparse
    ap = argparse.ArgumentParser(prog="palm_random_model",
                                 description="Write a model folder (config.json, model.safetensors) with random weights.")
    ap.add_argument("--config", required=True, help="a config.json of a registered architecture, or a named size")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--out", required=True, help="folder to write")
    ap.add_argument("--dtype", default="bfloat16", choices=sorted(_STORE), help="how the tensors are stored")
    args = ap.parse_args(argv)
    raw = config_source(args.config)
    out = write_random_model(raw, args.seed, args.out, args.dtype)
    print(out)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())

"""The random-weights mode on the device against the same mode's folder: one function of (seed, tensor name,
element index) makes both, so they hold the same bits; and ``trace_run --random`` against the plain
implementation reading that folder."""
import json
import subprocess
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_qwen3 as P

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
DEV = "cuda:0"


@pytest.mark.parametrize("preset", ["tiny-a", "tiny-b"])
@pytest.mark.parametrize("mode", ["bfloat16", "float32"])
def test_device_weights_are_the_folder_s_weights_bit_for_bit(tmp_path, preset, mode):
    from palm_infra_amd.config import config_from_dict, config_source
    from palm_infra_amd.engine.engine import resolve_dtype
    from palm_infra_amd.weights import ModelFiles, load_weights, random_weights, write_random_model
    cfg = config_from_dict(config_source(preset))
    folder = write_random_model(cfg, 11, tmp_path / "m")
    files = ModelFiles(folder)
    spec = cfg.spec(files.names())
    dt = resolve_dtype(mode)
    from_file = load_weights(spec, files, dt, DEV)
    on_device = random_weights(cfg.spec(), 11, dt, DEV)
    other_seed = random_weights(cfg.spec(), 12, dt, DEV)
    refs = spec.tensor_refs()
    assert len(refs) > 5
    for ref in refs:
        a, b = from_file.get(ref), on_device.get(ref)
        assert a.dtype == b.dtype and a.shape == b.shape
        assert torch.equal(a, b), ref.names
        assert not torch.equal(a, other_seed.get(ref)), ref.names


def test_a_layer_does_not_depend_on_how_many_layers_follow():
    from palm_infra_amd.config import config_from_dict, config_source
    from palm_infra_amd.weights import random_weights
    raw = config_source("tiny-b")
    shallow = config_from_dict(dict(raw, num_hidden_layers=2)).spec()
    deep = config_from_dict(dict(raw, num_hidden_layers=3)).spec()
    ws, wd = random_weights(shallow, 4, torch.bfloat16, DEV), random_weights(deep, 4, torch.bfloat16, DEV)
    deep_by_name = {r.names: r for r in deep.tensor_refs()}
    for ref in shallow.tensor_refs():
        assert torch.equal(ws.get(ref), wd.get(deep_by_name[ref.names])), ref.names


def test_one_layer_of_large_sizes_matches_the_host_function_in_windows():
    """Qwen3-8B's layer sizes (a small vocabulary keeps the test short): windows of rows of every tensor, the
    last rows included, against the host function; the joined q/k/v and gate/up are their parts one after the
    other."""
    from palm_infra_amd.config import config_from_dict, config_source
    from palm_infra_amd.weights import random_numbers as R
    from palm_infra_amd.weights import random_weights
    cfg = config_from_dict(dict(config_source("qwen3-8b"), num_hidden_layers=1, vocab_size=2000))
    spec = cfg.spec()
    w = random_weights(spec, 0, torch.bfloat16, DEV)
    checked = 0
    for ref in spec.tensor_refs():
        t = w.get(ref)
        row = 0
        for name, shape in zip(ref.names, ref.shapes):
            part = t[row:row + shape[0]].reshape(-1).cpu()
            row += shape[0]
            _, mean, std = ref.init
            n = part.numel()
            for first in sorted({0, max(0, n // 2 - 777), max(0, n - 60_000)}):
                count = min(60_000, n - first)
                want = torch.from_numpy(R.standard_normal(R.tensor_key(0, name), first, count)) * torch.tensor(np.float32(std)) \
                    + torch.tensor(np.float32(mean))
                assert torch.equal(part[first:first + count], want.to(torch.bfloat16).to(part.dtype)), (name, first)
                checked += count
    assert checked > 1_000_000


def test_trace_run_with_random_weights_of_a_named_size(tmp_path):
    from palm_infra_amd.config import config_source
    from palm_infra_amd.weights import write_random_model
    folder = write_random_model(config_source("tiny-a"), 3, tmp_path / "m")
    cfg, w = P.read_model(folder)
    g = torch.Generator().manual_seed(5)
    req = torch.randint(0, cfg["vocab_size"], (40,), generator=g).tolist()
    steps = [{"step": 0, "entries": [{"id": "r", "tokens": req[:30], "want": [0, 29]}], "end": []}]
    steps += [{"step": 1 + i, "entries": [{"id": "r", "tokens": [req[30 + i]], "want": [0]}], "end": ["r"] if i == 9 else []}
              for i in range(10)]
    out = tmp_path / "o"
    proc = subprocess.run([str(ROOT / "bin" / "trace_run"), "--random", "tiny-a", "--seed", "3", "--dtype", "float32", "--out", str(out),
                           "--max-tokens", "64"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                          text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr
    assert proc.stdout.split("\n")[:11] == [f"done {i}" for i in range(11)]
    ref = P.logits(cfg, w, req)
    V = cfg["vocab_size"]
    first = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V).copy())
    assert float((first.double() - ref[[0, 29]]).abs().max()) <= 1e-4
    for i in range(10):
        row = torch.from_numpy(np.fromfile(out / f"{1 + i}.f32", dtype="<f4").reshape(-1, V).copy())
        assert float((row.double() - ref[30 + i:31 + i]).abs().max()) <= 1e-4, i

"""bin/trace_run as a user runs it: a child process fed JSON lines, writing <step>.f32 files.  The same
requests are replayed whole, with the last 32 tokens one by one, and in batches of unequal lengths, in
float32 and in bfloat16, and compared with the plain implementation."""
import json
import subprocess
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_qwen3 as P
import tiny

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


def run_trace(model_dir, dtype, steps, out_dir, max_tokens):
    """Feeds one step at a time and waits for its `done` line, as the protocol says."""
    proc = subprocess.Popen([str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype, "--out", str(out_dir),
                             "--max-tokens", str(max_tokens)], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for rec in steps:
            proc.stdin.write(json.dumps(rec) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {rec['step']}", f"step {rec['step']}: got {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()


def read_logits(out_dir, step, vocab):
    return torch.from_numpy(np.fromfile(Path(out_dir) / f"{step}.f32", dtype="<f4").reshape(-1, vocab).copy())


def schedule_steps(reqs):
    """Three schedules over the same requests in one trace; returns (steps, checks) where a check is
    (step, row range, request, first place, number of places)."""
    steps, checks, no = [], [], 0
    # 1. each alone and whole
    for i, r in enumerate(reqs):
        steps.append({"step": no, "entries": [{"id": f"w{i}", "tokens": r, "want": list(range(len(r)))}], "end": [f"w{i}"]})
        checks.append((no, 0, i, 0, len(r)))
        no += 1
    # 2. whole minus the last 32, then one by one
    for i, r in enumerate(reqs):
        if len(r) <= 32:
            continue
        cut = len(r) - 32
        steps.append({"step": no, "entries": [{"id": f"d{i}", "tokens": r[:cut], "want": [cut - 1]}], "end": []})
        checks.append((no, 0, i, cut - 1, 1))
        no += 1
        for t in range(cut, len(r)):
            steps.append({"step": no, "entries": [{"id": f"d{i}", "tokens": [r[t]], "want": [0]}], "end": [f"d{i}"] if t == len(r) - 1 else []})
            checks.append((no, 0, i, t, 1))
            no += 1
    # 3. two batches of unequal lengths, the shorter requests ending earlier, one batch after the other
    for b, members in enumerate(([0, 1, 2], [3, 4, 5, 0])):
        tail = 4
        cuts = {i: max(1, len(reqs[i]) - tail - 2 * k) for k, i in enumerate(members)}
        ents, row = [], 0
        for i in members:
            ents.append({"id": f"b{b}_{i}", "tokens": reqs[i][:cuts[i]], "want": [0, cuts[i] - 1] if cuts[i] > 1 else [0]})
            checks.append((no, row, i, 0, 1))
            if cuts[i] > 1:
                checks.append((no, row + 1, i, cuts[i] - 1, 1))
            row += 2 if cuts[i] > 1 else 1
        steps.append({"step": no, "entries": ents, "end": [f"b{b}_{i}" for i in members if cuts[i] == len(reqs[i])]})
        no += 1
        fed = dict(cuts)
        while any(fed[i] < len(reqs[i]) for i in members):
            live = [i for i in members if fed[i] < len(reqs[i])]
            ents = [{"id": f"b{b}_{i}", "tokens": [reqs[i][fed[i]]], "want": [0] if (fed[i] + i) % 3 else []} for i in live]
            row = 0
            for i, e in zip(live, ents):
                if e["want"]:
                    checks.append((no, row, i, fed[i], 1))
                    row += 1
                fed[i] += 1
            steps.append({"step": no, "entries": ents, "end": [f"b{b}_{i}" for i in live if fed[i] == len(reqs[i])]})
            no += 1
    return steps, checks


# the last three: a folder stored in one precision and run in the other (a tensor stored in 32-bit stays so in
# the bfloat16 mode; bfloat16 and float16 widen exactly for the float32 mode; float16 is re-rounded for bfloat16)
@pytest.mark.parametrize("name,dtype,store", [("A", "float32", None), ("A", "bfloat16", None), ("B", "float32", None),
                                              ("B", "bfloat16", None), ("D", "bfloat16", None), ("B", "bfloat16", "float32"),
                                              ("A", "float32", "bfloat16"), ("B", "float32", "float16"),
                                              ("A", "bfloat16", "float16")])
def test_replay_schedules(model_dirs, tmp_path, name, dtype, store):
    lengths = {"A": [5, 17, 9, 70, 40, 33], "B": [1, 31, 12, 64, 100, 45], "D": [64, 3, 97, 65, 128, 33]}[name]
    reqs = tiny.prompts(name, lengths, seed=8)
    steps, checks = schedule_steps(reqs)
    # the most that is live at once: the second batch, each request rounded up to 64
    max_tokens = max(sum(-(-len(reqs[i]) // 64) * 64 for i in m) for m in ([0, 1, 2], [3, 4, 5, 0]))
    out = tmp_path / "out"
    store = store or dtype
    model_dir = model_dirs[name][store] if store in model_dirs[name] else tiny.write_model(name, tmp_path / "model", store)
    run_trace(model_dir, dtype, steps, out, max_tokens)
    cfg, w = P.read_model(model_dir)
    V = cfg["vocab_size"]
    refs = [P.logits(cfg, w, r) for r in reqs]
    files = {}
    for step, row, i, place, count in checks:
        if step not in files:
            files[step] = read_logits(out, step, V)
        tiny.assert_logits_close(files[step][row:row + count], refs[i][place:place + count], dtype,
                                 f"{name} {dtype} step {step} request {i} place {place}")
    wanted_steps = {c[0] for c in checks}
    for rec in steps:
        has = (out / f"{rec['step']}.f32").exists()
        assert has == (rec["step"] in wanted_steps), rec["step"]       # no file for a step in which nothing is wanted
        if has:
            n_want = sum(len(e["want"]) for e in rec["entries"])
            assert files.get(rec["step"], read_logits(out, rec["step"], V)).shape == (n_want, V)


def test_replay_drives_the_framework_s_own_step(model_dirs, tmp_path):
    """The replay tool has no forward pass of its own: what it writes is bit for bit what Engine.step
    returns for the same steps."""
    from palm_infra_amd.engine import Engine, StepEntry
    reqs = tiny.prompts("A", [20, 7], seed=9)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": reqs[0][:15], "want": [14]}, {"id": "y", "tokens": reqs[1], "want": [0, 6]}], "end": ["y"]},
             {"step": 1, "entries": [{"id": "x", "tokens": reqs[0][15:16], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": reqs[0][16:], "want": []}], "end": ["x"]}]
    out = tmp_path / "o"
    run_trace(model_dirs["A"]["bfloat16"], "bfloat16", steps, out, 128)
    eng = Engine.from_dir(model_dirs["A"]["bfloat16"], dtype="bfloat16", max_tokens=128)
    x, y = eng.open(), eng.open()
    s0 = eng.step([StepEntry(x, reqs[0][:15], [14]), StepEntry(y, reqs[1], [0, 6])]).cpu()
    eng.close(y)
    s1 = eng.step([StepEntry(x, reqs[0][15:16], [0])]).cpu()
    assert torch.equal(read_logits(out, 0, 256), s0) and torch.equal(read_logits(out, 1, 256), s1)
    assert not (out / "2.f32").exists()


def test_a_step_that_cannot_run_ends_the_replay_with_one_line(model_dirs, tmp_path):
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3], "want": [2]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [1] * 200, "want": []}], "end": []}]
    proc = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(model_dirs["A"]["float32"]), "--dtype", "float32",
                           "--out", str(tmp_path / "o"), "--max-tokens", "128"], input="".join(json.dumps(s) + "\n" for s in steps),
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode == 1 and proc.stdout.strip() == "done 0"
    assert "CacheFull" in proc.stderr and "Traceback" not in proc.stderr
    assert (tmp_path / "o" / "0.f32").exists()

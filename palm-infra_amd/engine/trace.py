"""Trace replay: feed given token ids through a model step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: it drives the engine's
``step``, the one that generation uses.  The reference's nearest tools are ``prefill_hidden`` /
``decode_hidden`` / ``run_lmhead_raw(all_positions)`` (engine/engine.cpp:1062-1246, 1669-1720,
487-555), which its chunked-prefill test drives (tests/test_e2e.cpp:413-529).

Input, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``<out>/<step>.f32`` holds the logits at the wanted places in
the order of the entries and of ``want``, little-endian float32 [wanted, vocab].  After every step a
line ``done <step>`` is printed and flushed.
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


def replay(engine, lines, out_dir, report=print) -> None:
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    from .engine import StepEntry
    slots: dict[str, int] = {}
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step_no = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid = str(e["id"])
            if rid not in slots:
                slots[rid] = engine.open()
            entries.append(StepEntry(slots[rid], list(e["tokens"]), list(e.get("want", []))))
        if entries:
            logits = engine.step(entries)
            if logits.shape[0] > 0:
                arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                arr.tofile(out_dir / f"{step_no}.f32")
        for rid in rec.get("end", []):
            rid = str(rid)
            if rid in slots:
                engine.close(slots.pop(rid))
        report(f"done {step_no}")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description="Replay token ids through a model and write logits.")
    src = ap.add_mutually_exclusive_group(required=True)
    src.add_argument("--model", help="folder with config.json and model.safetensors")
    src.add_argument("--random", metavar="CONFIG", help="instead of --model: a config.json, or a named size (tiny-a, "
                     "qwen3-8b, ..), filled on the device with the random-weights mode's numbers for --seed")
    ap.add_argument("--seed", type=int, default=0, help="seed of --random (default 0)")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="the most tokens that live requests hold at any time (each rounded up to 64)")
    args = ap.parse_args(argv)
    from ..cache import CacheFull
    from .engine import Engine
    try:
        if args.random:
            from ..config import config_source
            engine = Engine.from_config(config_source(args.random), seed=args.seed, dtype=args.dtype, max_tokens=args.max_tokens)
        else:
            engine = Engine.from_dir(args.model, dtype=args.dtype, max_tokens=args.max_tokens)
    except (ValueError, FileNotFoundError, RuntimeError) as e:
        print(f"trace_run: {type(e).__name__}: {e}", file=sys.stderr)
        return 1

    def report(msg):
        print(msg, flush=True)

    try:
        replay(engine, sys.stdin, args.out, report)
    except (ValueError, KeyError, CacheFull) as e:
        # a line that is no JSON object of the form above, a token outside the vocabulary, more tokens than
        # --max-tokens holds: the steps before it are done and reported, this one changed nothing
        print(f"trace_run: {type(e).__name__}: {e}", file=sys.stderr)
        return 1
    return 0

"""Measures generation with random weights of Qwen3-8B's layer sizes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One JSON line: ``value`` is decoded tokens a second at batch 8 with 2,048-token contexts (a step is one
decode step of the whole batch: the model's forward pass from the cache, greedy choice on the device and
the copy of the chosen tokens to the host, as the generation loop does it).  The same line holds the
prefill of 2,048 tokens, the decode step's fraction of the HBM roofline, and decode at batch 1 and 64.

``points`` also holds (flat, every figure under a name of its own) the other workloads that the baseline names and
the lengths at which other kernels matter, each with tokens a second, milliseconds and its fraction of the same
roofline by the same formulas: decode at 128 sequences and at 8 sequences of 8,192 tokens, a prompt of 32,768
tokens, the time to the first token of prompts of 64, 128, 256 and 512 tokens (Qwen3-8B sizes); 16 prompts of unequal
lengths drawn from 64..2,048 and 256 decode steps at Qwen3-14B sizes; 32 prompts of 4,096 tokens and 512 decode
steps at Qwen3-32B sizes (the decode steps of these two scale with ``--steps``: twice and four times as many).
``--only 8b`` (or ``14b``, ``32b``, a comma-separated list) measures a part.

The protocol is the reference's (examples/bench.cpp:564-590, docs/performance.md:127-131): synthetic
token ids, no stop token, warm-up before the timed run, decode timed from an existing context.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X, published: HBM3E 8 TB/s; dense matrix cores 2.5 PFLOP/s for bfloat16
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}

# the measured configuration: Qwen3-8B sizes, kept as data beside the configuration code
from palm_infra_amd.config import preset_dict  # noqa: E402

QWEN3_8B = preset_dict("qwen3-8b")
CONTEXT = 2048          # tokens every sequence holds when decoding starts
PREFILL_TOKENS = 2048
BATCH = 8
FULL_LAYERS = 36


def layer_params(c) -> int:
    q, kv = c["num_attention_heads"] * c["head_dim"], c["num_key_value_heads"] * c["head_dim"]
    H, I = c["hidden_size"], c["intermediate_size"]
    return (q + 2 * kv) * H + H * q + 3 * H * I


def decode_bytes(c, batch: int, context: float, itemsize: int = 2) -> float:
    """What one decode step has to read: every weight it uses once (layers and head; the embedding only
    its batch rows) and the keys and values of the live requests (``batch`` of them holding ``context`` tokens
    each, or in the mean)."""
    L = c["num_hidden_layers"]
    weights = (L * layer_params(c) + c["vocab_size"] * c["hidden_size"]) * itemsize
    kv = 2 * c["num_key_value_heads"] * c["head_dim"] * itemsize * L * context * batch
    return weights + kv


def prefill_flops(c, tokens) -> float:
    """Linear layers for every token, causal attention (half of the square), the head for one row a prompt.
    ``tokens``: a prompt's length, or the lengths of the prompts that go through together."""
    lengths = [tokens] if isinstance(tokens, int) else list(tokens)
    L = c["num_hidden_layers"]
    linear = 2.0 * sum(lengths) * L * layer_params(c)
    attention = L * 4.0 * c["num_attention_heads"] * c["head_dim"] * sum(n * n for n in lengths) / 2.0
    return linear + attention + 2.0 * c["hidden_size"] * c["vocab_size"] * len(lengths)


def random_ids(n: int, vocab: int, seed: int) -> list:
    import torch
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def fill_contexts(engine, batch: int, context: int, vocab: int, group: int = 8):
    """Open `batch` sequences and put `context` tokens into each, a few sequences a step."""
    from palm_infra_amd.engine import StepEntry
    slots = [engine.open() for _ in range(batch)]
    for g in range(0, batch, group):
        engine.step([StepEntry(s, random_ids(context, vocab, 100 + g + j), []) for j, s in enumerate(slots[g:g + group])])
    return slots


def time_decode(engine, sampler, slots, steps: int, warmup: int, vocab: int):
    """ms per decode step over `steps` steps after `warmup` (the mean by the host's clock around all of them, and
    the median of the steps by the device's), tokens chosen greedily and fed back, as the generation loop does it: a
    step is launched with the tokens the step before left on the device, and the host takes that step's tokens
    while the next one runs."""
    import torch
    from palm_infra_amd.engine import FedTokens, StepEntry
    from palm_infra_amd.engine.generate import TokenFetch
    from palm_infra_amd.sampling import SequenceSampling
    states = [SequenceSampling(i) for i in range(len(slots))]
    first = [random_ids(1, vocab, 7 + i)[0] for i in range(len(slots))]
    rows = list(range(len(slots)))
    logits = engine.step([StepEntry(s, [t], [0]) for s, t in zip(slots, first)])
    pending = TokenFetch(sampler.sample(logits, states))
    taken = []

    def one():
        nonlocal pending
        logits = engine.step([StepEntry(s, [0], [0]) for s in slots], fed=FedTokens(pending.ids, rows))
        following = TokenFetch(sampler.sample(logits, states))
        taken.append(pending.tokens())
        pending = following

    for _ in range(warmup):
        one()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        one()
        marks[i + 1].record()
    torch.cuda.synchronize()
    mean_ms = (time.perf_counter() - t0) * 1000.0 / steps
    # the device's own clock between the ends of consecutive steps, and its median (the reference's protocol reports
    # a median, docs/performance.md:38-41): a step that the host or another tenant of the machine delayed does not
    # move it
    each = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    median_ms = each[len(each) // 2] if len(each) % 2 else 0.5 * (each[len(each) // 2 - 1] + each[len(each) // 2])
    return mean_ms, median_ms


def time_prefill(engine, tokens: int, vocab: int, repeats: int = 3) -> float:
    """Best ms of `repeats` for one fresh sequence of `tokens` tokens, logits at the last place."""
    import torch
    from palm_infra_amd.engine import StepEntry
    best = float("inf")
    for r in range(repeats + 1):            # the first run warms up
        ids = random_ids(tokens, vocab, 500 + r)
        slot = engine.open()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([StepEntry(slot, ids, [tokens - 1])])
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1000.0
        engine.close(slot)
        if r > 0:
            best = min(best, ms)
    return best


def kernel_table(engine, cfg, slots, batch: int, context: int) -> dict:
    """The decode step's dominant kernels one by one: each launched once for every layer (so that no weight is read
    twice from a cache) inside a recorded graph, timed with events around its replays; the bytes each has to
    read, the time of one launch, and the fraction of the HBM peak that makes."""
    import torch
    from palm_infra_amd.kernels import ops
    from palm_infra_amd.parts import ResidualSink
    model, cache = engine.model, engine.cache
    layers = model.layers
    L = len(layers)
    H, I = cfg["hidden_size"], cfg["intermediate_size"]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    dev, bf16 = engine.device, torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(1)
    h = torch.randn(batch, H, device=dev, dtype=bf16, generator=g)
    attn = torch.randn(batch, nh * hd, device=dev, dtype=bf16, generator=g)
    act = torch.randn(batch, I, device=dev, dtype=bf16, generator=g)
    resid = torch.zeros(batch, H, device=dev, dtype=torch.float32)
    kv = cache.layer_caches[0].kv           # the store of the first layer's group (all layers of this model share it)
    seq_slot = torch.tensor(slots, dtype=torch.int32, device=dev)
    seq_start = torch.tensor([cache.lengths[s] - 1 for s in slots], dtype=torch.int32, device=dev)
    n_slices = ops.decode_slices(batch, nh, nkv, engine._length_bucket(context + 1))
    # what the attention part runs after its q/k/v projection in a decode step: the projection's planes of partial
    # sums in, per-head norms, rotation, the new key and value into the cache, attention, the merge of the slices
    mixer0 = layers[0].mixer
    qkv = mixer0.qkv(h, planes_ok=True).clone()
    cos, sin = ops.rope_table(seq_start, mixer0.position.inv_freq)

    def attention_of(i):
        m = layers[i].mixer
        return ops.attention_decode_fused(qkv, kv.k[i], kv.v[i], kv.table_dev, seq_slot, seq_start, nh, nkv, hd, m.scale, None,
                                          n_slices, q_norm_w=m.q_norm.weight, k_norm_w=m.k_norm.weight, eps=m.q_norm.eps,
                                          cos=cos, sin=sin, rotary_dim=hd, pairing=0)

    def each_layer(fn):
        return lambda: [fn(i) for i in range(L)]
    work = {
        "qkv_proj": (each_layer(lambda i: layers[i].mixer.qkv(h, planes_ok=True)), (nh + 2 * nkv) * hd * H * 2, L),
        "attention": (each_layer(attention_of), 2 * nkv * hd * 2 * context * batch, L),
        "o_proj": (each_layer(lambda i: layers[i].mixer.out(attn, sink=ResidualSink(resid, layers[i].feed_forward_norm))),
                   nh * hd * H * 2, L),
        "gate_up_proj": (each_layer(lambda i: layers[i].feed_forward.gate_up.gated(h)), 2 * I * H * 2, L),
        "down_proj": (each_layer(lambda i: layers[i].feed_forward.down(act, sink=ResidualSink(resid, layers[i].mixer_norm))),
                      I * H * 2, L),
        "lm_head": (lambda: [model.head.forward(h)], cfg["vocab_size"] * H * 2, 1),
    }
    table = {}
    for name, (fn, nbytes, launches) in work.items():
        fn()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        graph.replay()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) * 1000.0 / launches)
        gbs = nbytes / best / 1e3
        table[name] = {"bytes": int(nbytes), "us": round(best, 2), "gbs": round(gbs, 1), "frac": round(gbs / PEAK_HBM_GBS, 4)}
        del graph
    return table


def prefill_kernel_table(engine, cfg, tokens: int) -> dict:
    """The prompt step's dominant kernels one by one at `tokens` rows, as kernel_table does it: the four products
    of a layer (the library's), the prompt attention, the norm with the residual add and the gated activation;
    flops (or bytes) each has to do, the time of one launch and the fraction of the peak that makes."""
    import torch
    from palm_infra_amd.engine import StepEntry
    from palm_infra_amd.kernels import ops
    model, cache = engine.model, engine.cache
    layers = model.layers
    L = len(layers)
    H, I = cfg["hidden_size"], cfg["intermediate_size"]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    dev, bf16 = engine.device, torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(2)
    h = torch.randn(tokens, H, device=dev, dtype=bf16, generator=g)
    attn = torch.randn(tokens, nh * hd, device=dev, dtype=bf16, generator=g)
    act = torch.randn(tokens, I, device=dev, dtype=bf16, generator=g)
    gate_up = torch.randn(tokens, 2 * I, device=dev, dtype=bf16, generator=g)
    resid = torch.zeros(tokens, H, device=dev, dtype=torch.float32)
    slot = engine.open()
    engine.step([StepEntry(slot, random_ids(tokens, cfg["vocab_size"], 900), [])])       # keys and values to attend over
    kv = cache.layer_caches[0].kv           # the store of the first layer's group (all layers of this model share it)
    i32 = lambda xs: torch.tensor(xs, dtype=torch.int32, device=dev)
    seq_slot, seq_start, seq_new, cu = i32([slot]), i32([0]), i32([tokens]), i32([0, tokens])
    mfma, hbm = PEAK_FLOPS["bf16"], PEAK_HBM_GBS * 1e9
    # as the attention part hands them over: queries that carry the scale where the kernel of this head size takes them so
    q_scale = ops.prefill_q_scale(hd, bf16, hd ** -0.5)
    queries = (attn.float() * q_scale).to(bf16)

    def each_layer(fn):
        return lambda: [fn(i) for i in range(L)]
    work = {
        "qkv_proj": (each_layer(lambda i: layers[i].mixer.qkv(h)), 2.0 * tokens * (nh + 2 * nkv) * hd * H, mfma),
        "attention": (each_layer(lambda i: ops.attention_prefill(queries, kv.k[i], kv.v[i], kv.table_dev, seq_slot, seq_start, seq_new, cu,
                                                                 tokens, nh, nkv, hd, hd ** -0.5, None, q_prescaled=q_scale != 1.0)),
                      4.0 * nh * hd * tokens * (tokens + 1) / 2.0, mfma),
        "o_proj": (each_layer(lambda i: layers[i].mixer.out(attn)), 2.0 * tokens * nh * hd * H, mfma),
        "gate_up_proj": (each_layer(lambda i: layers[i].feed_forward.gate_up(h)), 2.0 * tokens * 2 * I * H, mfma),
        "down_proj": (each_layer(lambda i: layers[i].feed_forward.down(act)), 2.0 * tokens * I * H, mfma),
        # memory-bound passes: bytes instead of flops, against the HBM peak
        "norm_with_add": (each_layer(lambda i: layers[i].feed_forward_norm(resid, delta=h, update=True)), tokens * H * (4 + 2 + 4 + 2.0), hbm),
        "gated_activation": (each_layer(lambda i: ops.swiglu(gate_up)), tokens * I * (4 + 2.0), hbm),
    }
    table = {}
    for name, (fn, amount, peak) in work.items():
        fn()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):                     # launched one by one, as a prompt step launches them
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) * 1000.0 / L)
        table[name] = {"us": round(best, 1), "frac": round(amount / (best * 1e-6) / peak, 4),
                       "of": "mfma" if peak == mfma else "hbm"}
    engine.close(slot)
    return table


def other_sizes(name: str, args, sampler) -> dict:
    """The baseline's workloads at Qwen3-14B and Qwen3-32B sizes, flat: prompts together in one step (timed once,
    after a short warm-up prompt), then decode steps from those contexts."""
    import torch
    from palm_infra_amd.engine import Engine, StepEntry
    cfg = preset_dict(name)
    vocab = cfg["vocab_size"]
    if name == "qwen3-14b":
        import random
        rng = random.Random(3)
        lengths = [rng.randint(64, 2048) for _ in range(16)]
        steps, label = 2 * args.steps, "qwen3_14b_b16_unequal"
    else:
        lengths = [4096] * 32
        steps, label = 4 * args.steps, "qwen3_32b_b32_ctx8192"
    room = sum((n + steps + args.warmup + 64 + 63) // 64 * 64 for n in lengths) + 256
    t0 = time.perf_counter()
    engine = Engine.from_config(cfg, seed=0, dtype="bfloat16", max_tokens=room, max_seqs=len(lengths) + 1)
    torch.cuda.synchronize()
    load_s = time.perf_counter() - t0
    warm = engine.open()
    engine.step([StepEntry(warm, random_ids(256, vocab, 1), [255])])
    engine.close(warm)
    slots = [engine.open() for _ in lengths]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    engine.step([StepEntry(s, random_ids(n, vocab, 200 + i), [n - 1]) for i, (s, n) in enumerate(zip(slots, lengths))])
    torch.cuda.synchronize()
    prefill_ms = (time.perf_counter() - t0) * 1000.0
    mean_ms, median_ms = time_decode(engine, sampler, slots, steps, args.warmup, vocab)
    held = sum(lengths) + len(lengths) * (1 + args.warmup + steps / 2.0)          # tokens in the cache at the middle step
    nbytes = decode_bytes(cfg, 1, held)
    out = {
        f"{label}_decode": round(len(lengths) * 1000.0 / mean_ms, 2), f"{label}_decode_ms": round(mean_ms, 4),
        f"{label}_decode_ms_median": round(median_ms, 4), f"{label}_decode_steps": steps,
        f"{label}_decode_frac": round(nbytes / (mean_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
        f"{label}_prefill": round(sum(lengths) * 1000.0 / prefill_ms, 1), f"{label}_prefill_ms": round(prefill_ms, 2),
        f"{label}_prefill_tokens": sum(lengths),
        f"{label}_prefill_frac": round(prefill_flops(cfg, lengths) / (prefill_ms * 1e-3) / PEAK_FLOPS["bf16"], 4),
        f"{label}_load_s": round(load_s, 1),
    }
    for s in slots:
        engine.close(s)
    del engine
    torch.cuda.empty_cache()
    return out


def sizes_text(c) -> str:
    return (f"{c['num_hidden_layers']} layers, hidden {c['hidden_size']}, {c['num_attention_heads']} heads, "
            f"{c['num_key_value_heads']} kv heads, head_dim {c['head_dim']}, intermediate {c['intermediate_size']}, "
            f"vocab {c['vocab_size']}, random bf16 weights")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128, help="timed decode steps (the workload's 128)")
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=FULL_LAYERS, help="fewer layers than the model has, for a quick look")
    ap.add_argument("--batch", type=int, default=BATCH)
    ap.add_argument("--no-points", action="store_true", help="only the headline: batch 8, and the prefill of 2,048 tokens")
    ap.add_argument("--only", default="8b,14b,32b", help="which sizes' points to measure (8b is always measured)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="tokens of the timed prompt (2,048 is the workload's; others serve profiles of longer prompts)")
    args = ap.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not measured")
        return 2

    import torch
    from palm_infra_amd.engine import Engine, StepEntry
    from palm_infra_amd.sampling import GREEDY, DeviceSampler

    only = set() if args.no_points else {x.strip() for x in args.only.split(",")}
    cfg = dict(QWEN3_8B, num_hidden_layers=args.layers)
    vocab = cfg["vocab_size"]
    room = CONTEXT + args.warmup + args.steps + 64
    LONG, LONG_CONTEXT, LONG_BATCH, MANY = 32768, 8192, 8, 128
    prompt_tokens = args.prefill_tokens
    if args.no_points:
        cache_tokens = args.batch * room + prompt_tokens + 64
    else:
        cache_tokens = max(MANY * room, LONG_BATCH * (LONG_CONTEXT + room), LONG + 64) + prompt_tokens + 64
    t_load = time.perf_counter()
    engine = Engine.from_config(cfg, seed=0, dtype="bfloat16", max_tokens=cache_tokens, max_seqs=max(args.batch, MANY) + 1)
    torch.cuda.synchronize()
    load_s = time.perf_counter() - t_load
    sampler = DeviceSampler(GREEDY)

    kernels = {}

    def decode_at(batch: int, steps: int, warmup: int, table: bool = False, context: int = CONTEXT):
        slots = fill_contexts(engine, batch, context, vocab)
        ms = time_decode(engine, sampler, slots, steps, warmup, vocab)
        if table:
            kernels.update(kernel_table(engine, cfg, slots, batch, context + warmup + steps))
        for s in slots:
            engine.close(s)
        return ms

    def frac_of(batch: int, context: float, ms: float) -> float:
        return round(decode_bytes(cfg, batch, context) / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)

    ms_step, ms_median = decode_at(args.batch, args.steps, args.warmup, table=True)
    value = args.batch * 1000.0 / ms_step
    mid_context = CONTEXT + args.warmup + args.steps / 2.0
    points, fracs = {}, {}
    if not args.no_points:
        for name, b, steps, context in (("decode_b1", 1, args.steps, CONTEXT), ("decode_b64", 64, max(16, args.steps // 4), CONTEXT),
                                        ("decode_b128", MANY, max(16, args.steps // 4), CONTEXT),
                                        ("decode_b8_ctx8192", LONG_BATCH, max(16, args.steps // 2), LONG_CONTEXT)):
            ms, med = decode_at(b, steps, args.warmup, context=context)
            points[name] = round(b * 1000.0 / ms, 2)
            points[name + "_ms"], points[name + "_ms_median"] = round(ms, 4), round(med, 4)
            fracs[name] = points[name + "_frac"] = frac_of(b, context + args.warmup + steps / 2.0, ms)

    # The prompts last: a second of a prompt's large products back to back (the per-kernel table) leaves the chip at a
    # lower clock for some 0.2 s afterwards (the first 40 decode steps after it took 4.12 ms instead of 3.98), which
    # would be charged to the decode step if that were measured next.
    prefill_ms = time_prefill(engine, prompt_tokens, vocab)
    pf = prefill_flops(cfg, prompt_tokens)
    prefill_kernels = prefill_kernel_table(engine, cfg, prompt_tokens)
    if not args.no_points:
        for n in (64, 128, 256, 512):        # time to the first token: one prompt, logits at its last place
            points[f"ttft_{n}_ms"] = round(time_prefill(engine, n, vocab, repeats=5), 3)
        long_ms = time_prefill(engine, LONG, vocab, repeats=2)
        points["prefill_32768"] = round(LONG * 1000.0 / long_ms, 1)
        points["prefill_32768_ms"] = round(long_ms, 2)
        points["prefill_32768_frac"] = round(prefill_flops(cfg, LONG) / (long_ms * 1e-3) / PEAK_FLOPS["bf16"], 4)
    cache_room = engine.cache.max_tokens
    del engine
    torch.cuda.empty_cache()

    points_config = {}
    for name in ("qwen3-14b", "qwen3-32b"):
        if name.split("-")[1] in only:
            points.update(other_sizes(name, args, sampler))
            points_config[name.replace("-", "_")] = sizes_text(preset_dict(name))

    bytes_step = decode_bytes(cfg, args.batch, mid_context)
    achieved = bytes_step / (ms_step * 1e-3) / 1e9
    record = {
        "metric": "decode tok/s at batch 8, 2048-token contexts (Qwen3-8B sizes, bf16)",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "ms_per_step_median": round(ms_median, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic: random weights, uniform random token ids, no stop token",
        "config": {"model": "Qwen3-8B sizes, random weights", "global_batch": args.batch, "seq_len": CONTEXT,
                   "parallelism": "single GPU", "layers": args.layers, "layers_of_model": FULL_LAYERS,
                   "hidden_size": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate_size": cfg["intermediate_size"], "vocab_size": vocab, "rope_theta": cfg["rope_theta"],
                   "rms_norm_eps": cfg["rms_norm_eps"], "tied_head": False,
                   # the cache is one pool of pages for all live sequences; a sequence may take all of it
                   "cache_tokens": cache_room,
                   "prefill_tokens": prompt_tokens, "decode_steps": args.steps, "load_s": round(load_s, 1)},
        "prefill": {"value": round(prompt_tokens * 1000.0 / prefill_ms, 1), "tokens": prompt_tokens,
                    "ms": round(prefill_ms, 3), "frac": round(pf / (prefill_ms * 1e-3) / PEAK_FLOPS["bf16"], 4),
                    # the step's dominant kernels alone (a launch for each layer, event-timed): us a layer, and the
                    # fraction of the matrix cores' (or, for the two memory-bound passes, of HBM's) peak
                    "kernels": prefill_kernels},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4),
                     # the step's dominant kernels alone (a launch for each layer in a recorded graph, event-timed)
                     "kernels": kernels, **{f"frac_{k}": v["frac"] for k, v in kernels.items()},
                     # the same fraction for the other decode points (their bytes over their time)
                     **{f"frac_{name}": f for name, f in fracs.items()}},
        "points": points,
        # the sizes behind the points that are not of the headline's model
        "points_config": points_config,
    }
    print(json.dumps(record), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

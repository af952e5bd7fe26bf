"""Decode steps replayed from HIP graphs give what the same steps give when launched one by one: over many
replays, with other work and synchronisations between them, with batches that shrink and are padded, and
with slots and pages used again."""
import pytest
import torch

import tiny

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "bfloat16"), ("D", "bfloat16")])
def test_replays_equal_plain_launches(model_dirs, name, dtype):
    from palm_infra_amd.engine import Engine, StepEntry
    g = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 40, graphs=True)
    e = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 40, graphs=False)
    assert g.model.capturable
    n_req = 11
    reqs = tiny.prompts(name, [3 + 7 * i for i in range(n_req)], seed=30)
    decoded = tiny.prompts(name, [60] * n_req, seed=31)
    pool = tiny.LogitsPool(dtype, f"{name}: recorded steps against plain launches")
    for round_no in range(2):                                   # the second round reuses slots, pages and graphs
        sg = [g.open() for _ in reqs]
        se = [e.open() for _ in reqs]
        a = g.step([StepEntry(s, r, [len(r) - 1]) for s, r in zip(sg, reqs)])
        b = e.step([StepEntry(s, r, [len(r) - 1]) for s, r in zip(se, reqs)])
        assert torch.equal(a, b)                                # prompts never go through a graph
        live = list(range(n_req))
        for t in range(50):
            if t in (5, 9, 20, 21, 33, 40):                     # sequences end: 11 -> 10 -> 9 (a padded 16) -> .. -> 5
                gone = live.pop(t % len(live))
                g.close(sg[gone]); e.close(se[gone])
            a = g.step([StepEntry(sg[i], [decoded[i][t]], [0]) for i in live])
            b = e.step([StepEntry(se[i], [decoded[i][t]], [0]) for i in live])
            if t % 7 == 3:                                      # other work and a synchronisation between replays
                torch.cuda.synchronize()
                extra = g.open()
                g.step([StepEntry(extra, reqs[2], [0])])
                g.close(extra)
            if dtype == "float32":
                assert torch.equal(a, b), (round_no, t)         # padding and recording change no bit
            else:
                # the recorded step cuts a key range into slices sized for a rounded-up length: another order of sums
                pool.add(a, b.double().cpu(), f"{name} round {round_no} step {t}")
                assert float((a - b).abs().max()) < 0.05 * float(b.abs().max())
        for i in live:
            g.close(sg[i]); e.close(se[i])
        g.cache.check(); e.cache.check()
    if dtype != "float32":
        pool.check()                                            # a few rows a step: all of them together, too
    keys = sorted(k for k in g._decode_graphs if k[0] != "prompt")        # (the extra prompt between replays is recorded too)
    assert len(keys) >= 4 and all(st["graph"] is not None for k, st in g._decode_graphs.items() if st["calls"] > 1)
    assert not e._decode_graphs


@pytest.mark.parametrize("name,dtype", [("B", "bfloat16"), ("D", "bfloat16"), ("A", "float32")])
def test_recorded_steps_of_65_to_128_sequences(model_dirs, name, dtype):
    """Steps of more than 64 sequences are recorded too (their products go through the kernel that shares up to 128
    rows through LDS, their logits through the tiled one): against the plain implementation, with sequences that
    end on the way, so that the batch passes through several padded sizes, and each size is replayed."""
    import plain_qwen3 as P
    from palm_infra_amd.engine import Engine, StepEntry
    n_seqs = 128
    eng = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 2 * n_seqs, max_seqs=n_seqs)
    reqs = tiny.prompts(name, [9 + (7 * i) % 60 for i in range(n_seqs)], seed=36)
    cfg, w = P.read_model(model_dirs[name][dtype])
    refs = [P.logits(cfg, w, r) for r in reqs]
    slots = [eng.open() for _ in reqs]
    eng.step([StepEntry(s, r[:-8], []) for s, r in zip(slots, reqs)])
    live = list(range(n_seqs))
    pool = tiny.LogitsPool(dtype, f"{name}: recorded steps of many sequences")
    for t in range(8, 0, -1):
        if t in (6, 4, 2):                                          # 128 -> 106 -> 88 -> 73
            gone, live = live[::6], [i for k, i in enumerate(live) if k % 6]
            for i in gone:
                eng.close(slots[i])
        got = eng.step([StepEntry(slots[i], [reqs[i][-t]], [0]) for i in live])
        pool.add(got, torch.stack([refs[i][len(reqs[i]) - t] for i in live]), f"{len(live)} sequences, {t} before the end")
    pool.check()
    sizes = sorted(k[0] for k, st in eng._decode_graphs.items() if k[0] != "prompt" and st["graph"] is not None)
    assert sizes == [80, 88, 112, 128], sizes                       # each size ran twice: once plain, once recorded and replayed
    for i in live:
        eng.close(slots[i])
    eng.cache.check()


def test_a_wanted_subset_and_an_empty_one(model_dirs):
    from palm_infra_amd.engine import Engine, StepEntry
    g = Engine.from_dir(model_dirs["A"]["bfloat16"], dtype="bfloat16", max_tokens=64 * 8)
    reqs = tiny.prompts("A", [5, 6, 7], seed=32)
    slots = [g.open() for _ in reqs]
    g.step([StepEntry(s, r, []) for s, r in zip(slots, reqs)])
    for t in range(4):
        full = g.step([StepEntry(s, [t + 1], [0]) for s in slots])
        assert full.shape == (3, 256)
    some = g.step([StepEntry(slots[0], [9], []), StepEntry(slots[1], [9], [0]), StepEntry(slots[2], [9], [])])
    none = g.step([StepEntry(s, [3], []) for s in slots])
    assert some.shape == (1, 256) and none.shape == (0, 256)
    assert [g.length(s) for s in slots] == [11, 12, 13]


def test_a_model_with_a_part_that_plans_on_the_host_is_not_recorded(model_dirs):
    import test_toy_parts as toy
    from palm_infra_amd.config import config_from_dir
    from palm_infra_amd.engine import Engine
    from palm_infra_amd.weights import ModelFiles, load_weights
    toy.register_toy_mixer()
    d = model_dirs["A"]["float32"]
    config, files = config_from_dir(d), ModelFiles(d)
    base = config.spec(files.names())
    w = toy.ExtraWeights(load_weights(base, files, torch.float32, "cuda:0"),
                         {("toy.w_in",): torch.zeros(24, 64, device="cuda:0"), ("toy.w_out",): torch.zeros(64, 24, device="cuda:0")})
    eng = Engine(config, toy.toy_spec(base), w, torch.float32, max_tokens=256)
    assert not eng.model.capturable


@pytest.mark.parametrize("name", ["B", "C"])
def test_replays_of_steps_with_17_to_64_sequences(model_dirs, name):
    """From 17 sequences on a tiny model's products go to the BLAS library (its matrices have too few rows for
    the kernel that shares the activations through LDS), so these recorded steps hold library calls: every
    replay is checked against plain launches, with other work and synchronisations between the replays."""
    from palm_infra_amd.engine import Engine, StepEntry
    dtype = "bfloat16"
    g = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 64, graphs=True)
    e = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 64, graphs=False)
    n_req = 40
    reqs = tiny.prompts(name, [2 + (5 * i) % 23 for i in range(n_req)], seed=40)
    decoded = tiny.prompts(name, [30] * n_req, seed=41)
    sg = [g.open() for _ in reqs]
    se = [e.open() for _ in reqs]
    g.step([StepEntry(s, r, []) for s, r in zip(sg, reqs)])
    e.step([StepEntry(s, r, []) for s, r in zip(se, reqs)])
    live = list(range(n_req))
    for t in range(30):
        if t in (6, 12, 18, 24):                                    # 40 -> 33 -> 26 -> 19 -> 12 sequences
            for _ in range(7):
                gone = live.pop((3 * t) % len(live))
                g.close(sg[gone]); e.close(se[gone])
        a = g.step([StepEntry(sg[i], [decoded[i][t]], [0]) for i in live])
        b = e.step([StepEntry(se[i], [decoded[i][t]], [0]) for i in live])
        if t % 5 == 2:
            torch.cuda.synchronize()
            extra = g.open()
            g.step([StepEntry(extra, reqs[3], [0])])
            g.close(extra)
        tiny.assert_logits_close(a, b.double().cpu(), dtype, f"{name} {len(live)} sequences, step {t}")
        assert float((a - b).abs().max()) < 0.05 * float(b.abs().max()), (len(live), t)
    for i in live:
        g.close(sg[i]); e.close(se[i])
    g.cache.check(); e.cache.check()
    assert sum(st["graph"] is not None for st in g._decode_graphs.values()) >= 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sequences_that_grow_across_length_buckets_and_few_recordings_are_kept(model_dirs, dtype):
    """Recorded steps are keyed by the longest sequence rounded up to a power of two (256, 512, 1,024): three
    sequences grow from under 256 to over 512 tokens, every step checked against plain launches and pooled
    against the plain implementation; and an engine keeps no more recordings than its limit, dropping the one
    used longest ago."""
    import plain_qwen3 as P
    from palm_infra_amd.engine import Engine, StepEntry
    name = "C"
    g = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 40, graphs=True)
    e = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 40, graphs=False)
    g.GRAPH_LIMIT = 2
    reqs = tiny.prompts(name, [530, 300, 270], seed=35)
    starts = [245, 100, 5]
    cfg, w = P.read_model(model_dirs[name][dtype])
    refs = [P.logits(cfg, w, r) for r in reqs]
    sg, se = [g.open() for _ in reqs], [e.open() for _ in reqs]
    for eng, slots in ((g, sg), (e, se)):
        eng.step([StepEntry(s, r[:c], []) for s, r, c in zip(slots, reqs, starts)])
    pool = tiny.LogitsPool(dtype, "growing across length buckets")
    fed = list(starts)
    seen = set()
    for t in range(285):
        live = [i for i in range(3) if fed[i] < len(reqs[i])]
        a = g.step([StepEntry(sg[i], [reqs[i][fed[i]]], [0]) for i in live])
        b = e.step([StepEntry(se[i], [reqs[i][fed[i]]], [0]) for i in live])
        seen |= set(g._decode_graphs)
        assert len(g._decode_graphs) <= 2
        if dtype == "float32":
            assert torch.equal(a, b), t
        if t % 9 == 0 or 8 <= t <= 14 or 262 <= t <= 270:            # around the edges at 256 and 512, and now and then
            pool.add(a, torch.stack([refs[i][fed[i]] for i in live]), f"step {t}")
        for i in live:
            fed[i] += 1
    pool.check()
    assert {k[1] for k in seen} == {256, 512, 1024} and len(seen) >= 4      # more shapes than are kept at once
    for i in range(3):
        g.close(sg[i]); e.close(se[i])
    g.cache.check()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "bfloat16"), ("B", "float32")])
def test_short_prompts_of_one_sequence_are_recorded_too(model_dirs, name, dtype):
    """A prompt (or a further piece) of 2 to 63 tokens of one sequence with one place wanted runs as a recorded
    step, padded to a multiple of 8 tokens by a sequence of its own: every length three times (as it is,
    recorded, replayed), at the start of a sequence and on top of what it already holds, against plain launches
    and against the plain implementation."""
    import plain_qwen3 as P
    from palm_infra_amd.engine import Engine, StepEntry
    g = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 12, graphs=True)
    e = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 12, graphs=False)
    cfg, w = P.read_model(model_dirs[name][dtype])
    pool = tiny.LogitsPool(dtype, f"{name} {dtype}: short prompts as recorded steps")
    lengths = [2, 7, 8, 9, 15, 16, 17, 31, 40, 63]
    for round_no in range(3):
        for n in lengths:
            ids = tiny.prompts(name, [n + 1 + 5], seed=50 + n + 100 * round_no)[0]
            ref = P.logits(cfg, w, ids)
            sg, se = g.open(), e.open()
            a = g.step([StepEntry(sg, ids[:n], [n - 1])])
            b = e.step([StepEntry(se, ids[:n], [n - 1])])
            a1 = g.step([StepEntry(sg, ids[n:n + 1], [0])])               # a decode step on what the recorded prompt left
            b1 = e.step([StepEntry(se, ids[n:n + 1], [0])])
            a2 = g.step([StepEntry(sg, ids[n + 1:], [2])])                # a further piece of five tokens, recorded as well
            b2 = e.step([StepEntry(se, ids[n + 1:], [2])])
            if dtype == "float32":
                assert torch.equal(a, b) and torch.equal(a1, b1) and torch.equal(a2, b2), (round_no, n)
            pool.add(torch.cat([a, a1, a2]), ref[[n - 1, n, n + 3]], f"round {round_no}, {n} tokens")
            assert g.length(sg) == n + 6
            g.close(sg); e.close(se)
    pool.check()
    recorded = {k: st for k, st in g._decode_graphs.items() if k[0] == "prompt"}
    assert set(recorded) == {("prompt", b) for b in (8, 16, 24, 32, 48, 64)}
    assert all(st["graph"] is not None and st["calls"] >= 3 for st in recorded.values())
    assert not e._decode_graphs
    # what is not served: two sequences, more than one place wanted, 64 tokens or more
    s1, s2 = g.open(), g.open()
    before = {k: st["calls"] for k, st in g._decode_graphs.items()}
    g.step([StepEntry(s1, [1, 2, 3], [2]), StepEntry(s2, [4, 5], [1])])
    g.step([StepEntry(s1, [1, 2, 3], [0, 2])])
    g.step([StepEntry(s2, list(range(1, 65)), [63])])
    assert {k: st["calls"] for k, st in g._decode_graphs.items()} == before
    g.cache.check()

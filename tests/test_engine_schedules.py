"""The engine against the plain implementation under every way of cutting and batching the same
requests: each alone and whole; whole minus the last 32 tokens, which then come one by one; batches of
unequal lengths whose shorter requests end earlier, one batch after another so that slots and pages are
used again; long decoding; the first tokens of a sequence.  In float32 and in bfloat16."""
import pytest
import torch

import plain_qwen3 as P
import tiny
from palm_infra_amd.cache import KVNeed, StateNeed

pytestmark = pytest.mark.gpu

CASES = [(name, dtype) for name in ("A", "B", "C", "D") for dtype in ("float32", "bfloat16")]
LENGTHS = {"A": [5, 17, 9, 64, 100, 33], "B": [1, 31, 12, 64, 65, 200], "C": [48, 7, 129, 2, 300, 70],
           "D": [64, 3, 65, 129, 1, 40]}

_engines = {}
_refs = {}


def engine_for(model_dirs, name, dtype):
    from palm_infra_amd.engine import Engine
    key = (name, dtype)
    if key not in _engines:
        _engines[key] = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 24)
    return _engines[key]


def reference(model_dirs, name, dtype, ids):
    """Plain logits [n, V] of one whole sequence, from the same stored weights."""
    key = (name, dtype, tuple(ids))
    if key not in _refs:
        cfg, w = P.read_model(model_dirs[name][dtype])
        _refs[key] = P.logits(cfg, w, ids)
    return _refs[key]


@pytest.mark.parametrize("name,dtype", CASES)
def test_each_request_alone_and_whole(model_dirs, name, dtype):
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(model_dirs, name, dtype)
    for ids in tiny.prompts(name, LENGTHS[name]):
        slot = eng.open()
        got = eng.step([StepEntry(slot, ids, list(range(len(ids))))])
        eng.close(slot)
        tiny.assert_logits_close(got, reference(model_dirs, name, dtype, ids), dtype, f"{name} whole {len(ids)}")
    eng.cache.check()


@pytest.mark.parametrize("name,dtype", CASES)
def test_last_32_tokens_one_by_one(model_dirs, name, dtype):
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(model_dirs, name, dtype)
    for ids in tiny.prompts(name, [n for n in LENGTHS[name] if n > 32], seed=1):
        ref = reference(model_dirs, name, dtype, ids)
        cut = len(ids) - 32
        slot = eng.open()
        got = [eng.step([StepEntry(slot, ids[:cut], list(range(cut)))])]
        for t in range(cut, len(ids)):
            got.append(eng.step([StepEntry(slot, [ids[t]], [0])]))
            assert eng.length(slot) == t + 1
        eng.close(slot)
        tiny.assert_logits_close(torch.cat(got), ref, dtype, f"{name} {len(ids)} tokens, last 32 one by one")


@pytest.mark.parametrize("name,dtype", CASES)
def test_batches_of_unequal_lengths_one_after_another(model_dirs, name, dtype):
    """Two batches through the same slots and pages.  In a batch all prompts go in one step minus their
    last `tail` tokens, which come one a step; a request with no tokens left ends (its slot goes back at
    once), so later steps are smaller."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(model_dirs, name, dtype)
    held_before = eng.cache.groups_of(KVNeed)[0].table.pages.held_count
    for round_no, (seed, tails) in enumerate([(2, [3, 0, 9, 1, 20, 5]), (3, [1, 12, 0, 2, 7, 30])]):
        reqs = tiny.prompts(name, LENGTHS[name] if round_no == 0 else LENGTHS[name][::-1], seed=seed)
        tails = [min(t, len(r) - 1) for t, r in zip(tails, reqs)]
        slots = [eng.open() for _ in reqs]
        assert sorted(slots) == list(range(len(reqs)))                # the second batch gets the first one's slots
        got = {i: [] for i in range(len(reqs))}
        cuts = [len(r) - t for r, t in zip(reqs, tails)]
        out = eng.step([StepEntry(s, r[:c], list(range(c))) for s, r, c in zip(slots, reqs, cuts)])
        o = 0
        for i, c in enumerate(cuts):
            got[i].append(out[o:o + c])
            o += c
        live = list(range(len(reqs)))
        fed = list(cuts)
        while True:
            for i in [i for i in live if fed[i] == len(reqs[i])]:
                eng.close(slots[i])
                live.remove(i)
            if not live:
                break
            out = eng.step([StepEntry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
            for r, i in enumerate(live):
                got[i].append(out[r:r + 1])
                fed[i] += 1
        for i, r in enumerate(reqs):
            tiny.assert_logits_close(torch.cat(got[i]), reference(model_dirs, name, dtype, r), dtype,
                                     f"{name} batch {round_no} request {i} ({len(r)} tokens, {tails[i]} one by one)")
        eng.cache.check()
        assert eng.cache.groups_of(KVNeed)[0].table.pages.held_count == held_before


@pytest.mark.parametrize("name,dtype", [("C", "float32"), ("C", "bfloat16"), ("B", "float32"), ("D", "bfloat16")])
def test_long_decoding(model_dirs, name, dtype):
    """A short prompt, then every further token one by one, across several pages."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(model_dirs, name, dtype)
    n = 250 if name == "B" else 420
    ids = tiny.prompts(name, [n], seed=4)[0]
    ref = reference(model_dirs, name, dtype, ids)
    other = eng.open()                                                # a neighbour that decodes along, then leaves
    eng.step([StepEntry(other, ids[5:40], [])])
    slot = eng.open()
    got = [eng.step([StepEntry(slot, ids[:3], [0, 1, 2])])]
    for t in range(3, n):
        entries = [StepEntry(slot, [ids[t]], [0])]
        if t < 200:
            entries.insert(0, StepEntry(other, [ids[t]], []))
        elif t == 200:
            eng.close(other)
        got.append(eng.step(entries))
    eng.close(slot)
    tiny.assert_logits_close(torch.cat(got), ref, dtype, f"{name} long decoding")
    eng.cache.check()


@pytest.mark.parametrize("name,dtype", CASES)
def test_first_tokens_of_a_sequence(model_dirs, name, dtype):
    """Prompts of one and two tokens, and a sequence fed one token at a time from its first."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(model_dirs, name, dtype)
    ids = tiny.prompts(name, [6], seed=5)[0]
    ref = reference(model_dirs, name, dtype, ids)
    a, b, c = eng.open(), eng.open(), eng.open()
    first = eng.step([StepEntry(a, ids[:1], [0]), StepEntry(b, ids[:2], [0, 1]), StepEntry(c, ids[:6], [5])])
    tiny.assert_logits_close(first[0:1], ref[0:1], dtype, "one-token prompt")
    tiny.assert_logits_close(first[1:3], ref[0:2], dtype, "two-token prompt")
    tiny.assert_logits_close(first[3:4], ref[5:6], dtype, "last place only")
    got = [first[0:1]]
    for t in range(1, 6):
        got.append(eng.step([StepEntry(a, [ids[t]], [0])]))
    tiny.assert_logits_close(torch.cat(got), ref, dtype, "token by token from the first")
    for s in (a, b, c):
        eng.close(s)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_padding_and_companions_change_no_result(model_dirs, dtype):
    """The same request alone, among longer and shorter companions, and in another slot."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(model_dirs, "B", dtype)
    reqs = tiny.prompts("B", [40, 3, 130, 64], seed=6)
    s = eng.open()
    alone = eng.step([StepEntry(s, reqs[0], list(range(40)))]).cpu()
    eng.close(s)
    slots = [eng.open() for _ in range(4)]
    order = [2, 1, 0, 3]
    out = eng.step([StepEntry(slots[j], reqs[j], list(range(len(reqs[j])))) for j in order]).cpu()
    for sl in slots:
        eng.close(sl)
    together = out[130 + 3:130 + 3 + 40]
    if dtype == "float32":
        # every output element adds its products in the same order whatever else is in the batch
        assert torch.equal(alone, together)
    else:
        tiny.assert_logits_close(together, alone.double(), dtype, "with companions")


def test_a_refused_step_changes_nothing(model_dirs):
    from palm_infra_amd.cache import CacheFull
    from palm_infra_amd.engine import StepEntry, StepError
    eng = engine_for(model_dirs, "A", "float32")
    s = eng.open()
    ids = tiny.prompts("A", [10], seed=7)[0]
    eng.step([StepEntry(s, ids[:4], [])])
    for bad, err in (([StepEntry(s, [256], [0])], StepError), ([StepEntry(s, [1], [1])], StepError),
                     ([StepEntry(s, [], [])], StepError), ([StepEntry(s, [1], []), StepEntry(s, [2], [])], StepError),
                     ([StepEntry(31, [1], [])], StepError), ([StepEntry(s, [1] * 2000, [])], CacheFull), ([], StepError)):
        with pytest.raises(err):
            eng.step(bad)
        assert eng.length(s) == 4
    got = eng.step([StepEntry(s, ids[4:], list(range(6)))])           # the cache has 24 pages: 2,000 more do not fit
    tiny.assert_logits_close(got, reference(model_dirs, "A", "float32", ids)[4:], "float32", "after refused steps")
    eng.close(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_sequence_longer_than_max_position_embeddings(model_dirs, dtype):
    """The reference never reads ``max_position_embeddings`` (models/qwen3.py:175-184); a sequence is bounded by
    the cache alone.  Configuration A names 128 positions; 150 tokens run, the last 10 one by one."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(model_dirs, "A", dtype)
    ids = tiny.prompts("A", [150], seed=21)[0]
    s = eng.open()
    got = [eng.step([StepEntry(s, ids[:140], list(range(140)))])]
    got += [eng.step([StepEntry(s, [t], [0])]) for t in ids[140:]]
    eng.close(s)
    tiny.assert_logits_close(torch.cat(got), reference(model_dirs, "A", dtype, ids), dtype, "150 tokens with 128 positions named")


@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("C", "bfloat16")])
def test_a_step_with_more_tokens_than_run_at_once_goes_through_in_pieces(model_dirs, name, dtype):
    """``max_step_tokens`` bounds the tokens that run through the layers together (the memory of a step's
    activations); a longer step is cut, within sequences and between them, and gives the same logits at the same
    places.  A step that the cache cannot hold is refused before its first piece."""
    from palm_infra_amd.cache import CacheFull
    from palm_infra_amd.engine import Engine, StepEntry
    eng = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 12, max_step_tokens=50)
    reqs = tiny.prompts(name, [130, 7, 61, 50, 3], seed=17)
    slots = [eng.open() for _ in reqs]
    wants = [[0, 49, 50, 64, 100, 129], [6], [], [0, 49], [1, 2]]
    got = eng.step([StepEntry(s, r, w) for s, r, w in zip(slots, reqs, wants)])
    assert [eng.length(s) for s in slots] == [len(r) for r in reqs]
    row = 0
    pool = tiny.LogitsPool(dtype, f"{name}: a step in pieces and one more token each")
    for r, w in zip(reqs, wants):
        if w:
            pool.add(got[row:row + len(w)], reference(model_dirs, name, dtype, r)[w], f"pieces, {len(r)} tokens")
        row += len(w)
    assert got.shape[0] == row
    # one more token each, from what the pieces left in the cache
    nxt = tiny.prompts(name, [1] * len(reqs), seed=18)
    one = eng.step([StepEntry(s, t, [0]) for s, t in zip(slots, nxt)])
    for b, (r, t) in enumerate(zip(reqs, nxt)):
        pool.add(one[b:b + 1], reference(model_dirs, name, dtype, r + t)[-1:], f"after pieces, request {b}")
    pool.check()
    # 12 pages hold 768 tokens; five sequences hold 7 pages: a step of 400 more tokens for one of them does not fit
    before = [eng.length(s) for s in slots]
    with pytest.raises(CacheFull):
        eng.step([StepEntry(slots[1], tiny.prompts(name, [400], seed=19)[0], [])])
    assert [eng.length(s) for s in slots] == before
    for s in slots:
        eng.close(s)
    eng.cache.check()


@pytest.mark.parametrize("name,dtype", [(n, d) for n in ("A", "B") for d in ("float32", "bfloat16")])
def test_a_mixed_step_of_running_sequences_a_fresh_prompt_and_a_continuation(model_dirs, name, dtype):
    """One step that brings, side by side: two running sequences with one token each, a fresh prompt, and a
    further piece of a prompt whose first piece an earlier step brought; then a second mixed step in which a
    new sequence starts in the slot that a finished one gave back."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(model_dirs, name, dtype)
    r0, r1, r2, r3, r4 = tiny.prompts(name, [40, 23, 50, 70, 9], seed=33)
    ref = [reference(model_dirs, name, dtype, r) for r in (r0, r1, r2, r3, r4)]
    s0, s1, s2, s3 = (eng.open() for _ in range(4))
    eng.step([StepEntry(s0, r0[:30], []), StepEntry(s1, r1[:10], []), StepEntry(s3, r3[:33], [])])
    out = eng.step([StepEntry(s0, [r0[30]], [0]), StepEntry(s2, r2, list(range(50))), StepEntry(s1, [r1[10]], [0]),
                    StepEntry(s3, r3[33:53], list(range(20)))])
    assert out.shape[0] == 1 + 50 + 1 + 20
    pool = tiny.LogitsPool(dtype, f"{name} {dtype} mixed steps")
    pool.add(out[0:1], ref[0][30:31], "running sequence 0")
    pool.add(out[1:51], ref[2], "fresh prompt among running sequences")
    pool.add(out[51:52], ref[1][10:11], "running sequence 1")
    pool.add(out[52:72], ref[3][33:53], "continuation piece")
    eng.close(s2)
    s4 = eng.open()
    assert s4 == s2                                                 # the slot (and its pages) are used again
    out = eng.step([StepEntry(s3, r3[53:], list(range(17))), StepEntry(s0, [r0[31]], [0]), StepEntry(s4, r4, [0, 8]),
                    StepEntry(s1, [r1[11]], [0])])
    pool.add(out[0:17], ref[3][53:], "last piece")
    pool.add(out[17:18], ref[0][31:32], "running sequence 0, next token")
    pool.add(out[18:20], ref[4][[0, 8]], "a new sequence in a slot given back")
    pool.add(out[20:21], ref[1][11:12], "running sequence 1, next token")
    pool.check()
    assert [eng.length(s) for s in (s0, s1, s3, s4)] == [32, 12, 70, 9]
    for s in (s0, s1, s3, s4):
        eng.close(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_seqs", [150, 290])
def test_decode_steps_of_more_sequences_than_a_recorded_step_takes(model_dirs, dtype, n_seqs):
    """150 and 290 sequences one token each: beyond the batch sizes that are recorded into graphs, so these are
    plain launches with the products of more than 128 rows and an attention grid of as many sequences.
    Unequal lengths; some of the sequences end between the steps."""
    from palm_infra_amd.engine import Engine, StepEntry
    name = "B"
    eng = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 2 * n_seqs)
    assert n_seqs > eng.GRAPH_MAX_BATCH
    reqs = tiny.prompts(name, [4 + (11 * i) % 90 for i in range(n_seqs)], seed=34)
    cfg, w = P.read_model(model_dirs[name][dtype])
    refs = [P.logits(cfg, w, r) for r in reqs]
    slots = [eng.open() for _ in reqs]
    eng.step([StepEntry(s, r[:-3], []) for s, r in zip(slots, reqs)])
    live = list(range(n_seqs))
    pool = tiny.LogitsPool(dtype, f"{n_seqs} sequences a step")
    for t in (3, 2, 1):
        if t == 1:                                                  # 290 -> 193, 150 -> 139: still more than a recorded step takes
            every = 3 if n_seqs == 290 else 14
            gone, live = live[::every], [i for k, i in enumerate(live) if k % every]
            for i in gone:
                eng.close(slots[i])
        got = eng.step([StepEntry(slots[i], [reqs[i][-t]], [0]) for i in live])
        pool.add(got, torch.stack([refs[i][len(reqs[i]) - t] for i in live]), f"{len(live)} sequences, {t} before the end")
    pool.check()
    assert not eng._decode_graphs
    for i in live:
        eng.close(slots[i])
    eng.cache.check()


def test_which_decode_steps_take_the_attention_that_starts_from_the_projection(model_dirs, monkeypatch):
    """Heads of 64 in bfloat16 do (once a layer), heads of 48 and float32 steps do not; prompts never."""
    from palm_infra_amd.engine import Engine, StepEntry
    from palm_infra_amd.kernels import ops
    calls = []
    real = ops.attention_decode_fused
    monkeypatch.setattr(ops, "attention_decode_fused", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    for name, dtype, expected in (("D", "bfloat16", tiny.CONFIGS["D"]["num_hidden_layers"]), ("D", "float32", 0), ("C", "bfloat16", 0)):
        eng = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 4, graphs=False)
        slot = eng.open()
        eng.step([StepEntry(slot, [1, 2, 3], [2])])
        assert not calls
        eng.step([StepEntry(slot, [4], [0])])
        assert len(calls) == expected, (name, dtype)
        calls.clear()
        eng.close(slot)

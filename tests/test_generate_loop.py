"""The generation loop's decisions, with stand-ins for the engine and the sampler (no GPU)."""
import pytest
import torch

from palm_infra_amd.engine.generate import RequestTooLong, compute_metrics, generate, plan_batches, GenerationResult


class ScriptedEngine:
    """Its "logits" put all weight on the token that a script names for (request, how many tokens it has
    seen); it keeps the engine's books so the loop's use of slots can be checked."""

    def __init__(self, script, vocab=50, max_tokens=64 * 64, max_seq_tokens=4096, n_slots=8):
        self.script, self.vocab = script, vocab
        self.cache = type("C", (), {"max_tokens": max_tokens, "max_seq_tokens": max_seq_tokens})()
        self.free = list(range(n_slots - 1, -1, -1))
        self.seen = {}            # slot -> tokens consumed
        self.steps = []           # [(slot, n tokens), ...] of every step
        self.closed = []

    def open(self):
        s = self.free.pop()
        self.seen[s] = []
        return s

    def close(self, slot):
        assert slot in self.seen, "closed twice"
        del self.seen[slot]
        self.closed.append(slot)
        self.free.append(slot)
        self.free.sort(reverse=True)

    def step(self, entries):
        self.steps.append([(e.slot, len(e.tokens)) for e in entries])
        rows = []
        for e in entries:
            assert e.slot in self.seen
            self.seen[e.slot].extend(e.tokens)
            assert len(e.want) == 1 and e.want[0] == len(e.tokens) - 1
            row = torch.zeros(self.vocab)
            row[self.script(tuple(self.seen[e.slot]))] = 1.0
            rows.append(row)
        return torch.stack(rows)


class ArgmaxSampler:
    def __init__(self):
        self.histories = []

    def sample(self, logits, states):
        self.histories.append([list(s.history) for s in states])
        return logits.argmax(-1)


def test_unequal_prompts_stop_tokens_and_early_endings():
    # a prompt is [how many tokens to generate before the stop token, filler..., 0]; the stop token is 9
    prompts = [[3, 1, 1, 0], [1, 0], [5, 7, 7, 7, 7, 7, 0]]

    def script2(seen):
        n_gen = len(seen) - (seen.index(0) + 1)
        return 9 if n_gen >= seen[0] else 20 + n_gen
    eng, smp = ScriptedEngine(script2), ArgmaxSampler()
    seen_tokens = []
    results, metrics = generate(eng, smp, prompts, max_new_tokens=5, stop_token_ids=[9],
                                on_token=lambda i, t: seen_tokens.append((i, t)))
    assert [r.token_ids for r in results] == [[20, 21, 22, 9], [20, 9], [20, 21, 22, 23, 24]]
    assert [r.finish_reason for r in results] == ["stop", "stop", "length"]
    assert results[0].hit_eos and not results[2].hit_eos
    # one step with all prompts, then one token for each sequence that still runs
    assert eng.steps[0] == [(0, 4), (1, 2), (2, 7)]
    assert eng.steps[1:] == [[(0, 1), (1, 1), (2, 1)], [(0, 1), (2, 1)], [(0, 1), (2, 1)], [(2, 1)]]
    assert sorted(eng.closed) == [0, 1, 2] and eng.closed[0] == 1           # the shortest left first
    assert not eng.seen
    # sampling history follows what the model has consumed (engine/engine.cpp:977, 1451)
    assert smp.histories[0] == prompts and smp.histories[1][0] == prompts[0] + [20]
    assert seen_tokens[:3] == [(0, 20), (1, 20), (2, 20)]
    # the reference's metrics (examples/cli_common.cpp:418-436), summed
    assert metrics.prompt_tokens == 13 and metrics.generated_tokens == 11 and metrics.decode_tokens == 8


def test_stop_at_the_first_token_runs_no_decode_step():
    eng = ScriptedEngine(lambda seen: 9)
    results, _ = generate(eng, ArgmaxSampler(), [[1, 2], [3]], max_new_tokens=8, stop_token_ids=[9])
    assert [r.token_ids for r in results] == [[9], [9]] and len(eng.steps) == 1 and not eng.seen


def test_batches_follow_one_another_and_slots_are_used_again():
    eng = ScriptedEngine(lambda seen: 30 + len(seen), n_slots=2)
    prompts = [[1] * n for n in (3, 5, 2, 4, 6)]
    results, _ = generate(eng, ArgmaxSampler(), prompts, max_new_tokens=2, max_batch=2)
    assert [r.token_ids for r in results] == [[33, 34], [35, 36], [32, 33], [34, 35], [36, 37]]
    firsts = [s for s in eng.steps if any(n > 1 for _, n in s)]
    assert firsts == [[(0, 3), (1, 5)], [(0, 2), (1, 4)], [(0, 6)]]
    assert not eng.seen


def test_a_sequence_that_fills_its_context_ends():
    eng = ScriptedEngine(lambda seen: 1, max_seq_tokens=6)
    results, _ = generate(eng, ArgmaxSampler(), [[2, 2, 2, 2]], max_new_tokens=50)
    # 4 prompt tokens; tokens 1 and 2 can still be fed (lengths 5, 6); the third cannot
    assert results[0].finish_reason == "context" and len(results[0].token_ids) == 3
    assert len(eng.steps) == 3 and not eng.seen


def test_slots_come_back_when_a_step_fails():
    class Failing(ScriptedEngine):
        def step(self, entries):
            if len(self.steps) == 2:
                raise RuntimeError("boom")
            return super().step(entries)
    eng = Failing(lambda seen: 1)
    with pytest.raises(RuntimeError, match="boom"):
        generate(eng, ArgmaxSampler(), [[1], [2]], max_new_tokens=9)
    assert not eng.seen and sorted(eng.closed) == [0, 1]


def test_plan_batches():
    # 64-token pages: 60+10 -> 2 pages, 10+10 -> 1 page
    assert plan_batches([60, 10, 10, 10], 10, max_batch=8, cache_tokens=64 * 3, max_seq_tokens=4096) == [[0, 1], [2, 3]]
    assert plan_batches([1, 1, 1, 1, 1], 1, max_batch=2, cache_tokens=64 * 100, max_seq_tokens=4096) == [[0, 1], [2, 3], [4]]
    with pytest.raises(RequestTooLong, match="request 1"):
        plan_batches([5, 200], 1, 4, 64 * 100, max_seq_tokens=128)
    with pytest.raises(RequestTooLong, match="do not fit"):
        plan_batches([5, 200], 100, 4, 64 * 2, max_seq_tokens=4096)
    with pytest.raises(RequestTooLong, match="empty"):
        plan_batches([0], 1, 4, 64, 64)
    with pytest.raises(ValueError):
        generate(ScriptedEngine(lambda s: 1), ArgmaxSampler(), [[1]], max_new_tokens=0)   # examples/cli_common.cpp:451-454


def test_metrics_follow_the_reference_definitions():
    rs = [GenerationResult(prompt_tokens=10, token_ids=[1, 2, 3]), GenerationResult(prompt_tokens=6, token_ids=[4])]
    m = compute_metrics(rs, prefill_ms=8.0, decode_ms=4.0)
    assert (m.prompt_tokens, m.generated_tokens, m.decode_tokens) == (16, 4, 2)
    assert m.ttft_ms == 8.0 and m.tpot_ms == 2.0 and m.prefill_tps == 2000.0 and m.decode_tps == 500.0 and m.total_ms == 12.0
    m0 = compute_metrics([GenerationResult(prompt_tokens=3, token_ids=[1])], 1.0, 0.0)
    assert m0.decode_tokens == 0 and m0.tpot_ms == 0.0 and m0.decode_tps == 0.0


def test_a_conversation_feeds_only_what_is_new_and_keeps_its_slot():
    from palm_infra_amd.engine.generate import Conversation
    # the model counts upwards from the last token it saw; the stop token is 9
    eng = ScriptedEngine(lambda seen: min(seen[-1] + 1, 9), max_seq_tokens=64)
    eng.length = lambda slot: len(eng.seen[slot])
    sampler = ArgmaxSampler()
    talk = Conversation(eng, sampler, stop_token_ids=(9,))
    first = talk.say([1, 2, 5], max_new_tokens=10)
    assert first.token_ids == [6, 7, 8, 9] and first.finish_reason == "stop" and first.prompt_tokens == 3
    slot = talk.slot
    assert eng.seen[slot] == [1, 2, 5, 6, 7, 8] and talk.pending == [9]          # the stop token is not fed yet
    second = talk.say([3], max_new_tokens=2)
    assert second.token_ids == [4, 5] and second.finish_reason == "length" and second.prompt_tokens == 2
    assert talk.slot == slot and eng.seen[slot] == [1, 2, 5, 6, 7, 8, 9, 3, 4] and talk.pending == [5]
    # a turn's first step brings only the new tokens (and the pending one), never the conversation again
    assert eng.steps[0] == [(slot, 3)] and eng.steps[4] == [(slot, 2)] and all(st == [(slot, 1)] for st in eng.steps[1:4] + eng.steps[5:])
    # penalties see the whole conversation
    assert sampler.histories[-1] == [[1, 2, 5, 6, 7, 8, 9, 3, 4]]
    # a turn may consist of the pending token alone
    third = talk.say([], max_new_tokens=1)
    assert third.token_ids == [6] and eng.seen[slot][-1] == 5
    talk.reset()
    assert talk.slot is None and eng.closed == [slot] and talk.length == 0 and talk.pending == []
    with pytest.raises(ValueError, match="at least one token"):
        talk.say([])
    # the cache's end: a turn that does not fit is refused, a turn that reaches it ends for "context"
    with pytest.raises(RequestTooLong):
        talk.say([1] * 65)
    assert talk.slot is None
    full = talk.say([1] * 62, max_new_tokens=50)
    assert full.finish_reason == "context" and talk.length == 64 and len(full.token_ids) == 3
    talk.reset()


def test_a_batch_holds_no_more_sequences_than_the_cache_has_slots_and_a_refused_slot_leaks_none():
    eng = ScriptedEngine(lambda seen: 1, n_slots=3)
    eng.cache.max_seqs = 3
    results, _ = generate(eng, ArgmaxSampler(), [[1], [2], [3], [4], [5]], max_new_tokens=2, max_batch=8)
    assert [len(r.token_ids) for r in results] == [2] * 5
    assert len(eng.steps[0]) == 3 and max(len(s) for s in eng.steps) == 3          # batches of three, then two
    assert not eng.seen and len(eng.free) == 3

    # an engine that runs out of slots part-way (its cache does not say how many it has): those taken go back
    class NoSlots(RuntimeError):
        pass

    class Short(ScriptedEngine):
        def open(self):
            if not self.free:
                raise NoSlots("no free slot")
            return super().open()
    eng = Short(lambda seen: 1, n_slots=2)
    with pytest.raises(NoSlots):
        generate(eng, ArgmaxSampler(), [[1], [2], [3]], max_new_tokens=2, max_batch=8)
    assert not eng.seen and sorted(eng.free) == [0, 1] and not eng.steps


# ---- the loop that runs one step ahead of itself ------------------------------------------------------

class FedScriptedEngine(ScriptedEngine):
    """The same stand-in, which also takes a step's tokens from what an earlier draw left "on the device" (here a
    tensor like any other): the loop may then launch a step before it has looked at the tokens it feeds."""
    takes_fed = True

    def __init__(self, *a, **k):
        super().__init__(*a, **k)
        self.fed_steps = 0

    def step(self, entries, fed=None):
        if fed is not None:
            self.fed_steps += 1
            ids = fed.ids.tolist()
            assert len(fed.rows) == len(entries) and all(len(e.tokens) == 1 for e in entries)
            entries = [type(e)(e.slot, [ids[r]], e.want) for e, r in zip(entries, fed.rows)]
        for e in entries:
            assert len(self.seen[e.slot]) + len(e.tokens) <= self.cache.max_seq_tokens, "stepped beyond the longest sequence"
        return super().step(entries)


class StatelessSampler(ArgmaxSampler):
    needs_history = False


@pytest.mark.parametrize("max_new", [1, 2, 5, 9])
def test_the_loop_that_runs_ahead_gives_the_same_results_and_keeps_the_same_books(max_new):
    prompts = [[3, 1, 1, 0], [1, 0], [5, 7, 7, 7, 7, 7, 0], [0, 0], [8, 0]]

    def script(seen):
        n_gen = len(seen) - (seen.index(0) + 1)
        return 9 if n_gen >= seen[0] else 20 + n_gen
    plain, ahead = ScriptedEngine(script), FedScriptedEngine(script)
    tokens_plain, tokens_ahead = [], []
    want, m0 = generate(plain, ArgmaxSampler(), prompts, max_new_tokens=max_new, stop_token_ids=[9],
                        on_token=lambda i, t: tokens_plain.append((i, t)))
    got, m1 = generate(ahead, StatelessSampler(), prompts, max_new_tokens=max_new, stop_token_ids=[9],
                       on_token=lambda i, t: tokens_ahead.append((i, t)))
    assert [r.token_ids for r in got] == [r.token_ids for r in want]
    assert [r.finish_reason for r in got] == [r.finish_reason for r in want]
    assert tokens_ahead == tokens_plain                         # every token reported once, in the same order
    assert (m1.generated_tokens, m1.decode_tokens) == (m0.generated_tokens, m0.decode_tokens)
    assert not ahead.seen and sorted(ahead.closed) == sorted(plain.closed)      # every slot given back once
    # it did run ahead (where there was a second decode step to run), and a sequence that ended on a stop token was
    # stepped at most once more than in the plain loop; one that ended by its length never
    if max_new > 2:
        assert ahead.fed_steps > 0
    fed_plain = sum(n for s in plain.steps[1:] for _, n in s)
    fed_ahead = sum(n for s in ahead.steps[1:] for _, n in s)
    stopped = sum(1 for r in want if r.finish_reason == "stop" and len(r.token_ids) > 1)
    assert fed_plain <= fed_ahead <= fed_plain + stopped


def test_the_loop_that_runs_ahead_never_steps_beyond_the_longest_sequence():
    eng = FedScriptedEngine(lambda seen: 1, max_seq_tokens=6)
    results, _ = generate(eng, StatelessSampler(), [[2, 2, 2, 2], [2, 2]], max_new_tokens=50)
    assert [r.finish_reason for r in results] == ["context", "context"]
    assert [len(r.token_ids) for r in results] == [3, 5] and not eng.seen


def test_a_sampler_that_needs_the_history_keeps_the_plain_loop():
    eng = FedScriptedEngine(lambda seen: 30 + len(seen))
    results, _ = generate(eng, ArgmaxSampler(), [[1, 2, 3]], max_new_tokens=4)
    assert results[0].token_ids == [33, 34, 35, 36] and eng.fed_steps == 0


def test_slots_come_back_when_a_step_launched_ahead_fails():
    class Failing(FedScriptedEngine):
        def step(self, entries, fed=None):
            if len(self.steps) == 3:
                raise RuntimeError("boom")
            return super().step(entries, fed)
    eng = Failing(lambda seen: 1)
    with pytest.raises(RuntimeError, match="boom"):
        generate(eng, StatelessSampler(), [[1, 2], [3]], max_new_tokens=8)
    assert not eng.seen and sorted(eng.closed) == [0, 1]

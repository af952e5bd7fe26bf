"""Generation through the entry points: greedy tokens equal the plain implementation's; temperature
sampling is reproducible and a sequence's tokens do not depend on its batch companions."""
import subprocess
from pathlib import Path

import pytest
import torch

import plain_qwen3 as P
import tiny

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def engine_a(model_dirs):
    import palm_infra_amd
    return palm_infra_amd.load(model_dirs["A"]["float32"], dtype="float32", max_tokens=64 * 16)


def test_greedy_generation_equals_the_plain_implementation(model_dirs, engine_a):
    from palm_infra_amd.sampling import GREEDY
    cfg, w = P.read_model(model_dirs["A"]["float32"])
    prompts = tiny.prompts("A", [5, 17, 9], seed=10)                 # the workload of the first tiny configuration
    results, metrics = engine_a.generate(prompts, GREEDY, max_new_tokens=8, ignore_eos=True)
    for p, r in zip(prompts, results):
        assert r.token_ids == P.greedy(cfg, w, p, 8) and r.finish_reason == "length"
    assert metrics.prompt_tokens == 31 and metrics.generated_tokens == 24 and metrics.decode_tokens == 21
    assert metrics.prefill_tps > 0 and metrics.decode_tps > 0
    engine_a.cache.check()
    assert engine_a.cache.slots.held_count == 0
    # sampling options by name: temperature 0 is the greedy choice whatever the other options say
    named, _ = engine_a.generate(prompts, temperature=0.0, seed=3, max_new_tokens=8, ignore_eos=True)
    assert [r.token_ids for r in named] == [r.token_ids for r in results]
    with pytest.raises(TypeError, match="unknown options \\['temprature'\\]"):
        engine_a.generate(prompts, temprature=0.0)


def test_stop_tokens_end_sequences_early_and_batches_follow(model_dirs, engine_a):
    from palm_infra_amd.sampling import GREEDY
    cfg, w = P.read_model(model_dirs["A"]["float32"])
    prompts = tiny.prompts("A", [6, 3, 11, 4, 8], seed=11)
    free_run = [P.greedy(cfg, w, p, 12) for p in prompts]
    stop = free_run[0][3]                                            # a token the first request emits fourth
    results, _ = engine_a.generate(prompts, GREEDY, max_new_tokens=12, stop_token_ids=[stop], max_batch=2)
    for p, r, free in zip(prompts, results, free_run):
        expect = P.greedy(cfg, w, p, 12, stop=(stop,))
        assert r.token_ids == expect
        assert r.finish_reason == ("stop" if expect[-1] == stop else "length")
    assert results[0].hit_eos and len(results[0].token_ids) <= 4
    # config.json's eos_token_id is the default stop token
    eos = 7
    results, _ = engine_a.generate(prompts, GREEDY, max_new_tokens=12)
    for p, r in zip(prompts, results):
        assert r.token_ids == P.greedy(cfg, w, p, 12, stop=(eos,))
    assert engine_a.cache.slots.held_count == 0


def test_bfloat16_greedy_follows_the_oracle_where_the_margin_is_clear(model_dirs):
    """bfloat16 may pick another token where two logits are close; on the oracle's own path (teacher
    forcing) its argmax must agree wherever the oracle's top-2 margin exceeds the rounding bound."""
    from palm_infra_amd.engine import Engine, StepEntry
    cfg, w = P.read_model(model_dirs["B"]["bfloat16"])
    eng = Engine.from_dir(model_dirs["B"]["bfloat16"], dtype="bfloat16", max_tokens=64 * 8)
    ids = tiny.prompts("B", [250], seed=12)[0]
    ref = P.logits(cfg, w, ids)
    s = eng.open()
    got = eng.step([StepEntry(s, ids, list(range(250)))]).cpu().double()
    eng.close(s)
    top2 = ref.topk(2, dim=-1).values
    clear = (top2[:, 0] - top2[:, 1]) > 2 * tiny.BFLOAT16_MAX_REL * float(ref.pow(2).mean().sqrt())  # both logits may move
    assert int(clear.sum()) >= 5
    assert torch.equal(got.argmax(-1)[clear], ref.argmax(-1)[clear])


def test_temperature_sampling_is_reproducible_and_independent_of_companions(model_dirs):
    from palm_infra_amd.engine import Engine
    from palm_infra_amd.sampling import SamplingParams
    eng = Engine.from_dir(model_dirs["B"]["float32"], dtype="float32", max_tokens=64 * 16)
    prompts = tiny.prompts("B", [1, 31, 12, 64], seed=13)            # the workload of the second tiny configuration
    sp = SamplingParams(temperature=0.7, top_k=0, top_p=0.0, seed=1)
    a, _ = eng.generate(prompts, sp, max_new_tokens=16, ignore_eos=True)
    b, _ = eng.generate(prompts, sp, max_new_tokens=16, ignore_eos=True)
    assert [r.token_ids for r in a] == [r.token_ids for r in b]      # same seed, same stream
    c, _ = eng.generate(prompts, SamplingParams(temperature=0.7, top_k=0, top_p=0.0, seed=2), max_new_tokens=16, ignore_eos=True)
    assert [r.token_ids for r in a] != [r.token_ids for r in c]
    # request 0 alone draws the same tokens as in the batch: its stream is its own
    alone, _ = eng.generate(prompts[:1], sp, max_new_tokens=16, ignore_eos=True)
    assert alone[0].token_ids == a[0].token_ids
    one_by_one, _ = eng.generate(prompts, sp, max_new_tokens=16, ignore_eos=True, max_batch=1)
    assert [r.token_ids for r in one_by_one] == [r.token_ids for r in a]
    # every token drawn has positive probability under the plain distribution of its own context
    cfg, w = P.read_model(model_dirs["B"]["float32"])
    r = a[2]
    ctx = list(prompts[2])
    for tok in r.token_ids[:6]:
        probs = P.probabilities(P.logits(cfg, w, ctx)[-1].numpy(), 0.7)
        assert probs[tok] > 0
        ctx.append(tok)


def test_all_sampling_options_together(model_dirs):
    from palm_infra_amd.engine import Engine
    from palm_infra_amd.sampling import SamplingParams
    eng = Engine.from_dir(model_dirs["A"]["bfloat16"], dtype="bfloat16", max_tokens=64 * 8)
    sp = SamplingParams(temperature=0.9, top_k=20, top_p=0.8, min_p=0.02, repeat_penalty=1.3, repeat_last_n=8,
                        presence_penalty=0.5, frequency_penalty=0.2, seed=3)
    prompts = tiny.prompts("A", [4, 9], seed=14)
    a, _ = eng.generate(prompts, sp, max_new_tokens=20, ignore_eos=True)
    b, _ = eng.generate(prompts, sp, max_new_tokens=20, ignore_eos=True)
    assert [r.token_ids for r in a] == [r.token_ids for r in b] and all(len(r.token_ids) == 20 for r in a)
    # a strong penalty forbids an immediate repeat under greedy choice
    greedy_pen = SamplingParams(temperature=0.0, repeat_penalty=1.0, presence_penalty=2.0, frequency_penalty=2.0, repeat_last_n=-1)
    out, _ = eng.generate(prompts, greedy_pen, max_new_tokens=12, ignore_eos=True)
    plain, _ = eng.generate(prompts, SamplingParams(temperature=0.0), max_new_tokens=12, ignore_eos=True)
    assert [r.token_ids for r in out] != [r.token_ids for r in plain]


def test_command_line_generates_and_reports(model_dirs):
    cfg, w = P.read_model(model_dirs["A"]["float32"])
    prompt = tiny.prompts("A", [6], seed=15)[0]
    r = subprocess.run([str(ROOT / "bin" / "palm_chat"), "--package", str(model_dirs["A"]["float32"]), "--dtype", "float32",
                        "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--temperature", "0", "--n-ctx", "256"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [int(t) for t in r.stdout.split()] == P.greedy(cfg, w, prompt, 6, stop=(7,))
    b = subprocess.run([str(ROOT / "bin" / "palm_bench"), "--package", str(model_dirs["A"]["bfloat16"]), "--prompt-tokens", "20",
                        "--batch", "3", "--max-new-tokens", "5", "--temperature", "0", "--n-ctx", "512", "--warmup", "1"],
                       capture_output=True, text=True, timeout=120)
    assert b.returncode == 0, b.stderr[-2000:]
    kv = dict(line.split("=", 1) for line in b.stdout.strip().splitlines())
    assert kv["prompt_tokens"] == "60" and kv["generated_tokens"] == "15" and kv["decode_tokens"] == "12" and kv["hit_eos"] == "0"
    assert float(kv["decode_tps"]) > 0 and float(kv["prefill_tps"]) > 0
    # stop tokens given on the command line, and stopping switched off
    free = P.greedy(cfg, w, prompt, 12)
    common = [str(ROOT / "bin" / "palm_chat"), "--package", str(model_dirs["A"]["float32"]), "--dtype", "float32", "--prompt-ids",
              ",".join(map(str, prompt)), "--max-new-tokens", "12", "--temperature", "0", "--n-ctx", "256"]
    r = subprocess.run(common + ["--ignore-eos"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and [int(t) for t in r.stdout.split()] == free, r.stderr[-2000:]
    r = subprocess.run(common + ["--stop-token-ids", f"{free[4]},999"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and [int(t) for t in r.stdout.split()] == free[:free.index(free[4]) + 1], r.stderr[-2000:]
    # what cannot run ends with one line and status 1, not with a traceback
    for extra, says in ((["--prompt-ids", "1,2,900"], "outside the vocabulary"), (["--prompt-ids", ",".join(["1"] * 300)], "300")):
        r = subprocess.run([str(ROOT / "bin" / "palm_chat"), "--package", str(model_dirs["A"]["float32"]), "--n-ctx", "128",
                            "--max-new-tokens", "4"] + extra, capture_output=True, text=True, timeout=120)
        assert r.returncode == 1 and says in r.stderr and "Traceback" not in r.stderr, r.stderr[-2000:]
    r = subprocess.run([str(ROOT / "bin" / "palm_chat"), "--package", str(ROOT / "no_such_folder"), "--prompt-ids", "1"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 1 and "no config.json" in r.stderr and "Traceback" not in r.stderr
    bad = subprocess.run([str(ROOT / "bin" / "palm_chat"), "--package", str(model_dirs["A"]["float32"]), "--temperature", "3"],
                         capture_output=True, text=True, timeout=120)
    assert bad.returncode == 1 and "temperature must be between 0 and 2" in bad.stderr


def test_command_line_profile_and_trace(tmp_path):
    """``--profile`` prints a table per phase whose launches are the timed run's; ``--trace`` writes them as a
    Chrome trace; the model is a named size with random weights."""
    import json
    trace = tmp_path / "t.json"
    b = subprocess.run([str(ROOT / "bin" / "palm_bench"), "--random", "tiny-b", "--prompt-tokens", "20", "--batch", "2",
                        "--max-new-tokens", "4", "--temperature", "0", "--n-ctx", "512", "--warmup", "1", "--profile",
                        "--trace", str(trace)], capture_output=True, text=True, timeout=120)
    assert b.returncode == 0, b.stderr[-2000:]
    out = b.stdout
    assert "[prefill_profile]" in out and "[decode_profile]" in out and "generated_tokens=8" in out
    decode = out.split("[decode_profile]")[1]
    rows = {line.split()[0]: int(line.split()[1]) for line in decode.strip().splitlines()[2:]}
    # tiny-b has three layers; three decode steps of two sequences follow the prompts' step
    assert rows["palm_attention_decode"] == 3 * 3 and rows["palm_argmax"] == 3
    events = json.loads(trace.read_text())["traceEvents"]
    steps = [e for e in events if e.get("ph") == "X" and e["tid"] == 0]
    assert [e["cat"] for e in steps] == ["prefill", "decode", "decode", "decode"]
    kernels = [e for e in events if e.get("ph") == "X" and e["tid"] == 1]
    assert all(e["dur"] >= 0 for e in kernels) and sum(e["name"] == "palm_attention_decode" for e in kernels) == 9
    # every launch of a step lies inside the step
    first = steps[0]
    inside = [e for e in kernels if first["ts"] <= e["ts"] and e["ts"] + e["dur"] <= first["ts"] + first["dur"] + 1.0]
    assert len(inside) >= 3 * 4
    empty = subprocess.run([str(ROOT / "bin" / "palm_bench"), "--random", "tiny-b", "--trace", ""], capture_output=True,
                           text=True, timeout=120)
    assert empty.returncode == 1 and "--trace path must not be empty" in empty.stderr


def test_a_conversation_continues_from_the_cache(model_dirs, engine_a):
    """Turn by turn on one slot gives what the whole token sequence gives at once (greedy, float32), and the
    command line's loop of turns does the same."""
    from palm_infra_amd.sampling import GREEDY
    cfg, w = P.read_model(model_dirs["A"]["float32"])
    turns = tiny.prompts("A", [6, 3, 4], seed=33)
    talk = engine_a.conversation(GREEDY, ignore_eos=True)
    history, lines = [], []
    for turn in turns:
        r = talk.say(turn, max_new_tokens=5)
        history += turn
        want = P.greedy(cfg, w, history, 5)                     # the oracle reads the whole conversation again
        assert r.token_ids == want and r.finish_reason == "length"
        history += want
        lines.append(want)
    assert talk.length == len(history) - 1                      # the last chosen token is not fed yet
    talk.reset()
    assert engine_a.cache.slots.held_count == 0
    engine_a.cache.check()
    text = "".join(" ".join(map(str, t)) + "\n" for t in turns) + "/reset\n" + " ".join(map(str, turns[0])) + "\n/quit\n"
    r = subprocess.run([str(ROOT / "bin" / "palm_chat"), "--package", str(model_dirs["A"]["float32"]), "--dtype", "float32",
                        "--max-new-tokens", "5", "--temperature", "0", "--n-ctx", "256", "--ignore-eos"],
                       input=text, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    got = [[int(t) for t in line.split()] for line in r.stdout.strip().splitlines()]
    assert got == lines + [lines[0]]                            # after /reset the first turn gives its first answer again


# ---- tokens fed from the device, and the loop that runs one step ahead ---------------------------------

@pytest.mark.parametrize("name,dtype,graphs", [("A", "float32", True), ("D", "bfloat16", True), ("B", "bfloat16", False)])
def test_a_step_fed_from_the_device_is_the_step_fed_from_the_host(model_dirs, name, dtype, graphs):
    """The same single-token steps with the tokens as host integers and as rows of a device tensor (in order, and
    picked out of a longer one): the same bits; without recorded steps the tokens come to the host first."""
    from palm_infra_amd.engine import Engine, FedTokens, StepEntry, StepError
    a = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 12, graphs=graphs)
    b = Engine.from_dir(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 12, graphs=graphs)
    reqs = tiny.prompts(name, [9, 3, 30, 64], seed=40)
    sa, sb = [a.open() for _ in reqs], [b.open() for _ in reqs]
    for eng, slots in ((a, sa), (b, sb)):
        eng.step([StepEntry(s, r, []) for s, r in zip(slots, reqs)])
    V = tiny.CONFIGS[name]["vocab_size"]
    g = torch.Generator().manual_seed(5)
    for t in range(6):
        toks = torch.randint(0, V, (len(reqs),), generator=g).tolist()
        if t % 2 == 0:                                          # row k for entry k
            ids, rows = torch.tensor(toks, dtype=torch.int32).to("cuda:0"), list(range(len(reqs)))
        else:                                                   # picked out of a longer tensor, not in order
            spread = [V - 1] * (2 * len(reqs) + 1)
            rows = [2 * k + 1 for k in range(len(reqs))][::-1]
            for k, r in enumerate(rows):
                spread[r] = toks[k]
            ids = torch.tensor(spread, dtype=torch.int32).to("cuda:0")
        host = a.step([StepEntry(s, [tok], [0]) for s, tok in zip(sa, toks)])
        fed = b.step([StepEntry(s, [0], [0]) for s in sb], fed=FedTokens(ids, rows))
        assert torch.equal(host, fed), t
    with pytest.raises(StepError, match="one token for each sequence"):
        b.step([StepEntry(sb[0], [1, 2], [1])], fed=FedTokens(ids, [0]))
    with pytest.raises(StepError, match="outside"):
        b.step([StepEntry(sb[0], [0], [0])], fed=FedTokens(ids, [ids.shape[0]]))
    for eng, slots in ((a, sa), (b, sb)):
        for s in slots:
            eng.close(s)
        eng.cache.check()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("D", "bfloat16")])
@pytest.mark.parametrize("temperature", [0.0, 0.9])
def test_the_loop_that_runs_ahead_generates_what_the_plain_loop_does(model_dirs, name, dtype, temperature):
    """The engine's generation (whose loop launches a step before it has seen the last one's tokens) against the
    same loop made to wait for every step's tokens: the same tokens and endings, with stop tokens that end
    sequences at different steps, in batches that follow one another."""
    import palm_infra_amd
    from palm_infra_amd.engine.generate import generate
    from palm_infra_amd.sampling import DeviceSampler, SamplingParams

    class Waiting(DeviceSampler):
        needs_history = True

    eng = palm_infra_amd.load(model_dirs[name][dtype], dtype=dtype, max_tokens=64 * 16)
    params = SamplingParams(temperature=temperature, top_k=20, seed=4)
    prompts = tiny.prompts(name, [6, 3, 11, 70, 8, 1, 40], seed=41)
    free, _ = generate(eng, Waiting(params), prompts, max_new_tokens=24, stop_token_ids=(), max_batch=3)
    # stop tokens that some requests emit early, some late, some never
    stop = {free[0].token_ids[2], free[3].token_ids[10], free[5].token_ids[-1]}
    want, _ = generate(eng, Waiting(params), prompts, max_new_tokens=24, stop_token_ids=stop, max_batch=3)
    seen = []
    got, metrics = generate(eng, DeviceSampler(params), prompts, max_new_tokens=24, stop_token_ids=stop, max_batch=3,
                            on_token=lambda i, t: seen.append((i, t)))
    assert [r.token_ids for r in got] == [r.token_ids for r in want]
    assert [r.finish_reason for r in got] == [r.finish_reason for r in want]
    assert {r.finish_reason for r in got} == {"stop", "length"}
    assert sorted(seen) == sorted((i, t) for i, r in enumerate(got) for t in r.token_ids)
    assert metrics.generated_tokens == sum(len(r.token_ids) for r in want)
    eng.cache.check()
    assert eng.cache.slots.held_count == 0

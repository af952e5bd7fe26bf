"""The engine at the layer sizes that are measured (Qwen3-8B's: width 4096, 32 heads in 8 groups of head size
128, feed-forward width 12288; and Qwen3-14B's and 32B's) against the plain implementation: one layer and a short, odd vocabulary keep it
quick.  The tiny configurations cannot show what only long sums and the kernels' fast paths do: K of 4096 and
12288 in the thin and the library products, the folded norms, head size 128 in the matrix-core attention.
In float32 (1e-4 absolute, as everywhere) and in bfloat16."""
import pytest
import torch

import plain_qwen3 as P
import tiny

pytestmark = pytest.mark.gpu

LENGTHS = [70, 5, 33, 300]
DECODED = 8


# Qwen3-14B's sizes bring a down projection too long to fold the add and the norm in (K 17,408, cut into planes),
# Qwen3-32B's twice as many query rows as the width (64 heads of 128 over 5,120) and K 25,600
@pytest.fixture(scope="module", params=["qwen3-8b", "qwen3-14b", "qwen3-32b"])
def real(request):
    return one_layer_of(request.param)


@pytest.fixture(scope="module")
def real_8b():
    return one_layer_of("qwen3-8b")


def one_layer_of(size):
    from palm_infra_amd.config import config_from_dict, preset_dict
    from palm_infra_amd.weights import random_weights
    raw = dict(preset_dict(size), num_hidden_layers=1, vocab_size=3001, max_position_embeddings=4096)
    cfg = config_from_dict(raw)
    spec = cfg.spec()
    # values that bfloat16 holds exactly, so that both modes and the oracle start from the same numbers.  At this
    # width the usual spread already gives logits of order one; the q norm is four times larger, so that scores
    # are of order four and a wrong or missing key moves the logits by their own order
    # (made on the device, whose numbers are the random-weights mode's: hundreds of millions of them take the host
    # function half a minute)
    made = random_weights(spec, 11, torch.bfloat16, "cuda:0")
    tensors = {}
    for ref in spec.tensor_refs():
        row, joined = 0, made.get(ref).cpu()
        for name, shape in zip(ref.names, ref.shapes):
            t = joined[row:row + shape[0]].float()
            row += shape[0]
            if name.endswith("q_norm.weight"):
                t = t * 4.0
            tensors[name] = t.to(torch.bfloat16)
    del made
    oracle = {k: v.double() for k, v in tensors.items()}
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, raw["vocab_size"], (n,), generator=g).tolist() for n in LENGTHS]
    refs = [P.logits(raw, oracle, ids) for ids in prompts]
    del oracle
    return raw, cfg, spec, tensors, prompts, refs


def engine_of(real, dtype, pages=16):
    from palm_infra_amd.engine import Engine
    from palm_infra_amd.weights.loader import Weights, kept_dtype
    raw, cfg, spec, tensors, _, _ = real
    mode = torch.float32 if dtype == "float32" else torch.bfloat16
    held = {}
    for ref in spec.tensor_refs():
        dt = kept_dtype(ref, ["BF16"] * len(ref.names), mode)
        held[ref.names] = torch.cat([tensors[n] for n in ref.names]).to("cuda:0", dt)
    return Engine(cfg, spec, Weights(held), mode, max_tokens=64 * pages)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts_then_tokens_one_by_one_and_a_batch(real, dtype):
    from palm_infra_amd.engine import StepEntry
    _, _, _, _, prompts, refs = real
    eng = engine_of(real, dtype)
    # each alone: all but the last tokens in one step, the last ones one by one
    for ids, ref in zip(prompts, refs):
        cut = max(1, len(ids) - DECODED)
        slot = eng.open()
        got = [eng.step([StepEntry(slot, ids[:cut], list(range(cut)))])]
        for t in range(cut, len(ids)):
            got.append(eng.step([StepEntry(slot, [ids[t]], [0])]))
        eng.close(slot)
        tiny.assert_logits_close(torch.cat(got), ref, dtype, f"8B-size layer, {len(ids)} tokens, last {len(ids) - cut} one by one")
    # all together: prompts of unequal lengths in one step (each without its last token), then one token each
    slots = [eng.open() for _ in prompts]
    got = eng.step([StepEntry(s, ids[:-1], list(range(len(ids) - 1))) for s, ids in zip(slots, prompts)])
    last = eng.step([StepEntry(s, [ids[-1]], [0]) for s, ids in zip(slots, prompts)])
    row = 0
    for b, (ids, ref) in enumerate(zip(prompts, refs)):
        n = len(ids) - 1
        tiny.assert_logits_close(torch.cat([got[row:row + n], last[b:b + 1]]), ref, dtype, f"8B-size layer, batch, request {b}")
        row += n
    for s in slots:
        eng.close(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_of_many_sequences(real, dtype):
    """40 sequences, then 24 of them, each one token further: in bfloat16 these are the kernels for 17 to 64
    rows at the measured widths (the gated product over 24,576 weight rows, products cut along K into planes
    that the norms and the q/k/v pass add up), recorded into a graph on their second step."""
    from palm_infra_amd.engine import StepEntry
    raw = real[0]
    eng = engine_of(real, dtype, pages=48)
    oracle = {k: v.double() for k, v in real[3].items()}
    g = torch.Generator().manual_seed(6)
    seqs = [torch.randint(0, raw["vocab_size"], (2 + b % 4 + 3,), generator=g).tolist() for b in range(40)]
    refs = [P.logits(raw, oracle, ids) for ids in seqs]
    slots = [eng.open() for _ in seqs]
    eng.step([StepEntry(s, ids[:-3], []) for s, ids in zip(slots, seqs)])
    live = list(range(40))
    for t in (3, 2, 1):                                  # 40 sequences twice (the second step is a replay), then 24
        if t == 1:
            for b in live[24:]:
                eng.close(slots[b])
            live = live[:24]
        got = eng.step([StepEntry(slots[b], [seqs[b][-t]], [0]) for b in live])
        ref = torch.stack([refs[b][len(seqs[b]) - t] for b in live])
        tiny.assert_logits_close(got, ref, dtype, f"{len(live)} sequences, {t} tokens before the end")
    for b in live:
        eng.close(slots[b])
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_and_the_tokens_after_it(real_8b, dtype):
    """2,100 tokens in one step (34 pages; in bfloat16 the prompt kernels of the measured run: library products
    of thousands of rows, the q/k/v pass that holds heads in registers, matrix-core attention with query tiles
    paired from both ends), then three tokens one by one over 33 and 34 pages in slices."""
    from palm_infra_amd.engine import StepEntry
    real = real_8b
    raw = real[0]
    eng = engine_of(real, dtype, pages=40)
    oracle = {k: v.double() for k, v in real[3].items()}
    ids = torch.randint(0, raw["vocab_size"], (2103,), generator=torch.Generator().manual_seed(8)).tolist()
    places = [0, 63, 64, 1000, 2047, 2048, 2099]
    ref = P.logits(raw, oracle, ids)
    s = eng.open()
    got = [eng.step([StepEntry(s, ids[:2100], places)])]
    got += [eng.step([StepEntry(s, [t], [0])]) for t in ids[2100:]]
    eng.close(s)
    tiny.assert_logits_close(torch.cat(got), ref[places + [2100, 2101, 2102]], dtype, "2,100-token prompt and three more tokens")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixed_step_at_large_sizes(real_8b, dtype):
    """Two running sequences with one token each, a fresh prompt and a continuation piece in one step."""
    from palm_infra_amd.engine import StepEntry
    _, _, _, _, prompts, refs = real_8b
    eng = engine_of(real_8b, dtype, pages=24)
    r0, r1, r2, r3 = prompts                                   # 70, 5, 33, 300 tokens
    s0, s1, s2, s3 = (eng.open() for _ in range(4))
    eng.step([StepEntry(s0, r0[:60], []), StepEntry(s1, r1[:3], []), StepEntry(s3, r3[:130], [])])
    out = eng.step([StepEntry(s0, [r0[60]], [0]), StepEntry(s2, r2, list(range(33))), StepEntry(s1, [r1[3]], [0]),
                    StepEntry(s3, r3[130:250], list(range(120)))])
    pool = tiny.LogitsPool(dtype, "mixed step at large sizes")
    pool.add(out[0:1], refs[0][60:61], "running sequence")
    pool.add(out[1:34], refs[2], "fresh prompt")
    pool.add(out[34:35], refs[1][3:4], "short running sequence")
    pool.add(out[35:155], refs[3][130:250], "continuation piece")
    out = eng.step([StepEntry(s3, r3[250:], [0, 49]), StepEntry(s0, [r0[61]], [0]), StepEntry(s1, [r1[4]], [0])])
    pool.add(out[0:2], refs[3][[250, 299]], "last piece")
    pool.add(out[2:3], refs[0][61:62])
    pool.add(out[3:4], refs[1][4:5])
    pool.check()
    for s in (s0, s1, s2, s3):
        eng.close(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_of_70_and_130_sequences_at_large_sizes(real_8b, dtype):
    """130 sequences are beyond the batch sizes that are recorded (plain launches, library products of 130 rows);
    70 are within them, served by the kernel that shares up to 128 rows through LDS (a first step runs plain, the
    recording comes with the second); decode attention over more than 64 sequences either way."""
    from palm_infra_amd.engine import StepEntry
    raw = real_8b[0]
    eng = engine_of(real_8b, dtype, pages=140)
    oracle = {k: v.double() for k, v in real_8b[3].items()}
    g = torch.Generator().manual_seed(16)
    seqs = [torch.randint(0, raw["vocab_size"], (3 + b % 5,), generator=g).tolist() for b in range(130)]
    refs = [P.logits(raw, oracle, ids) for ids in seqs]
    slots = [eng.open() for _ in seqs]
    eng.step([StepEntry(s, ids[:-2], []) for s, ids in zip(slots, seqs)])
    live = list(range(130))
    pool = tiny.LogitsPool(dtype, "decode steps of 130 and 70 sequences")
    for t in (2, 1):
        if t == 1:
            for b in live[70:]:
                eng.close(slots[b])
            live = live[:70]
        got = eng.step([StepEntry(slots[b], [seqs[b][-t]], [0]) for b in live])
        pool.add(got, torch.stack([refs[b][len(seqs[b]) - t] for b in live]), f"{len(live)} sequences")
    pool.check()
    assert all(st["graph"] is None for st in eng._decode_graphs.values())
    for b in live:
        eng.close(slots[b])
    eng.cache.check()


@pytest.fixture(scope="module")
def long_sequence(real_8b):
    """9,000 tokens and the plain logits at the places the test asks for (the float64 attention of 32 heads over
    9,000 x 9,000 scores takes most of a minute: made once for both precisions)."""
    raw = real_8b[0]
    oracle = {k: v.double() for k, v in real_8b[3].items()}
    ids = torch.randint(0, raw["vocab_size"], (9000,), generator=torch.Generator().manual_seed(17)).tolist()
    places = [0, 63, 64, 4095, 4096, 8189] + list(range(8190, 8200)) + [8999]
    S = P.sizes(raw)
    n = len(ids)
    x = P.embedding(oracle["model.embed_tokens.weight"], ids)
    x = P.decoder_layer(x, oracle, 0, S, list(range(n)))
    ref = P.linear(P.rms_norm(x[places], oracle["model.norm.weight"], S["eps"]), P.head_weight(oracle))
    return ids, places, ref


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_sequence_that_grows_across_8192_tokens(real_8b, long_sequence, dtype):
    """8,190 tokens in one step (logits at a handful of places), then ten tokens one by one across the edge at
    8,192 where the recorded step's length bucket and the cut of the key range into slices change, then the
    rest of the 9,000 in one piece."""
    from palm_infra_amd.engine import StepEntry
    ids, places, ref = long_sequence
    eng = engine_of(real_8b, dtype, pages=144)
    s = eng.open()
    first = [p for p in places if p < 8190]
    got = [eng.step([StepEntry(s, ids[:8190], first)])]
    for t in range(8190, 8200):
        got.append(eng.step([StepEntry(s, [ids[t]], [0])]))
    got.append(eng.step([StepEntry(s, ids[8200:], [799])]))
    assert eng.length(s) == 9000
    tiny.assert_logits_close(torch.cat(got), ref, dtype, "9,000 tokens")
    eng.close(s)
    eng.cache.check()

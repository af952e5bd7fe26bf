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
    from palm_infra_amd.weights import random_tensors
    raw = dict(preset_dict(size), num_hidden_layers=1, vocab_size=3001, max_position_embeddings=4096)
    cfg = config_from_dict(raw)
    spec = cfg.spec()
    # values that bfloat16 holds exactly, so that both modes and the oracle start from the same numbers.  At this
    # width the usual spread already gives logits of order one; the q norm is four times larger, so that scores
    # are of order four and a wrong or missing key moves the logits by their own order
    tensors = {}
    for name, t in random_tensors(spec, 11, "float32").items():
        if name.endswith("q_norm.weight"):
            t = t * 4.0
        tensors[name] = t.to(torch.bfloat16)
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

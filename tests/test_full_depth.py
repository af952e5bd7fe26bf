"""The whole of Qwen3-8B's sizes (36 layers, the full vocabulary) against the plain implementation: prompts of
unequal lengths in one step, then their last 32 tokens one by one as recorded decode steps, then a second, shorter
batch through the slots and pages the first gave back, in float32 and in bfloat16.  What only depth shows
(rounding that adds up over 36 layers, every layer's kernels at the measured sizes one after the other) is not in
the tiny configurations; and the sequences are long enough that depth meets paging: every sequence crosses a page
border while it is decoded, a decode step's key ranges are cut into several slices that a second kernel merges, and
the slice that owns the new position's page changes on the way.  The same tokens in another cut give the same
logits (the reference's chunk invariant, tests/test_e2e.cpp:413-529).

The oracle runs layer by layer on the CPU in 64-bit from the very numbers the engine holds (random values that
bfloat16 represents exactly), one layer's tensors in memory at a time."""
import pytest
import torch

import plain_qwen3 as P
import tiny

pytestmark = pytest.mark.gpu

LENGTHS = [150, 70, 200]       # whole sequences; the last DECODED tokens of each go in one by one
DECODED = 32
SECOND = [45, 80]              # the batch that follows in the same slots, its last SECOND_DECODED tokens one by one
SECOND_DECODED = 4


def oracle_logits(raw, spec, weights, sequences):
    """Plain logits of whole sequences; ``weights`` is the engine's own (bfloat16 on the device)."""
    S = P.sizes(raw)
    q_rows, kv_rows, inter = S["nh"] * S["hd"], S["nkv"] * S["hd"], S["I"]

    def host(ref):
        return weights.get(ref).to("cpu").double()

    table = weights.get(spec.embedding.tensors["table"])
    xs = [table[torch.tensor(ids, device=table.device)].to("cpu").double() for ids in sequences]
    for i, layer in enumerate(spec.layers):
        mixer, ff = layer.parts["mixer"], layer.parts["feed_forward"]
        qkv, gate_up = host(mixer.tensors["qkv"]), host(ff.tensors["gate_up"])
        p = f"model.layers.{i}."
        w = {p + "input_layernorm.weight": host(layer.parts["mixer_norm"].tensors["weight"]),
             p + "post_attention_layernorm.weight": host(layer.parts["feed_forward_norm"].tensors["weight"]),
             p + "self_attn.q_proj.weight": qkv[:q_rows], p + "self_attn.k_proj.weight": qkv[q_rows:q_rows + kv_rows],
             p + "self_attn.v_proj.weight": qkv[q_rows + kv_rows:],
             p + "self_attn.q_norm.weight": host(mixer.parts["q_norm"].tensors["weight"]),
             p + "self_attn.k_norm.weight": host(mixer.parts["k_norm"].tensors["weight"]),
             p + "self_attn.o_proj.weight": host(mixer.tensors["out"]),
             p + "mlp.gate_proj.weight": gate_up[:inter], p + "mlp.up_proj.weight": gate_up[inter:],
             p + "mlp.down_proj.weight": host(ff.tensors["down"])}
        xs = [P.decoder_layer(x, w, i, S, list(range(x.shape[0]))) for x in xs]
        del w, qkv, gate_up
    norm_w, head = host(spec.final_norm.tensors["weight"]), host(spec.head.tensors["weight"])
    return [P.linear(P.rms_norm(x, norm_w, S["eps"]), head) for x in xs]


@pytest.fixture(scope="module")
def full():
    from palm_infra_amd.config import config_from_dict, preset_dict
    from palm_infra_amd.weights import random_weights
    raw = preset_dict("qwen3-8b")
    cfg = config_from_dict(raw)
    spec = cfg.spec()
    weights = random_weights(spec, 3, torch.bfloat16, "cuda:0")
    g = torch.Generator().manual_seed(9)
    seqs = [torch.randint(0, raw["vocab_size"], (n,), generator=g).tolist() for n in LENGTHS + SECOND]
    refs = oracle_logits(raw, spec, weights, seqs)
    return raw, cfg, spec, weights, seqs, refs


class Widened:
    """The same parameters in float32 (every bfloat16 value is a float32 value)."""

    def __init__(self, weights):
        self.weights, self.made = weights, {}

    def get(self, ref):
        if ref.names not in self.made:
            self.made[ref.names] = self.weights.get(ref).float()
        return self.made[ref.names]

    def nbytes(self):
        return sum(t.numel() * t.element_size() for t in self.made.values())


def run_batch(eng, slots, seqs, refs, decoded, dtype, what):
    """All but the last `decoded` tokens of every sequence in one step, the rest one by one; every position's
    logits against the plain implementation's."""
    from palm_infra_amd.engine import StepEntry
    first = eng.step([StepEntry(s, ids[:-decoded], list(range(len(ids) - decoded))) for s, ids in zip(slots, seqs)])
    later = [eng.step([StepEntry(s, [ids[len(ids) - decoded + t]], [0]) for s, ids in zip(slots, seqs)]) for t in range(decoded)]
    row = 0
    for b, (ids, ref) in enumerate(zip(seqs, refs)):
        n = len(ids) - decoded
        got = torch.cat([first[row:row + n]] + [step[b:b + 1] for step in later])
        tiny.assert_logits_close(got[:n], ref[:n], dtype, f"36 layers, {what}, request {b}: its first {n} tokens in one step")
        tiny.assert_logits_close(got[n:], ref[n:], dtype, f"36 layers, {what}, request {b}: its last {decoded} tokens one by one")
        row += n


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompts_together_then_the_last_tokens_one_by_one_then_a_second_batch_in_the_same_slots(full, dtype):
    from palm_infra_amd.engine import Engine
    raw, cfg, spec, weights, seqs, refs = full
    # room for the first batch and not much more: the second batch gets the pages the first one held
    room = sum((n + 63) // 64 for n in LENGTHS) * 64
    if dtype == "float32":
        eng = Engine(cfg, spec, Widened(weights), torch.float32, max_tokens=room, max_seqs=3)
    else:
        eng = Engine(cfg, spec, weights, torch.bfloat16, max_tokens=room, max_seqs=3)
    n1 = len(LENGTHS)
    slots = [eng.open() for _ in range(n1)]
    run_batch(eng, slots, seqs[:n1], refs[:n1], DECODED, dtype, "first batch")
    recorded = [key for key, st in eng._decode_graphs.items() if st["graph"] is not None]
    assert recorded, "the single tokens ran as replays of a recorded step"
    kv = eng.cache.layer_caches[0].kv
    held = {p for s in slots for p in kv.table.slot_pages[s]}
    for s in slots:
        eng.close(s)
    again = [eng.open() for _ in SECOND]
    assert set(again) <= set(slots)
    run_batch(eng, again, seqs[n1:], refs[n1:], SECOND_DECODED, dtype, "second batch")
    assert {p for s in again for p in kv.table.slot_pages[s]} <= held        # pages used again, uncleared
    for s in again:
        eng.close(s)
    eng.cache.check()
    del eng
    torch.cuda.empty_cache()

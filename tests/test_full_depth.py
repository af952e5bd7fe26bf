"""The whole of Qwen3-8B's sizes (36 layers, the full vocabulary) against the plain implementation: prompts of
unequal lengths in one step, then tokens one by one as recorded decode steps, in float32 and in bfloat16.
What only depth shows (rounding that adds up over 36 layers, every layer's kernels at the measured sizes one
after the other) is not in the tiny configurations.

The oracle runs layer by layer on the CPU in 64-bit from the very numbers the engine holds (random values that
bfloat16 represents exactly), one layer's tensors in memory at a time."""
import pytest
import torch

import plain_qwen3 as P
import tiny

pytestmark = pytest.mark.gpu

PROMPTS = [40, 9, 21]
DECODED = 4


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
    seqs = [torch.randint(0, raw["vocab_size"], (n + DECODED,), generator=g).tolist() for n in PROMPTS]
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompts_together_then_recorded_decode_steps(full, dtype):
    from palm_infra_amd.engine import Engine, StepEntry
    raw, cfg, spec, weights, seqs, refs = full
    if dtype == "float32":
        eng = Engine(cfg, spec, Widened(weights), torch.float32, max_tokens=64 * 8)
    else:
        eng = Engine(cfg, spec, weights, torch.bfloat16, max_tokens=64 * 8)
    slots = [eng.open() for _ in seqs]
    first = eng.step([StepEntry(s, ids[:-DECODED], list(range(len(ids) - DECODED))) for s, ids in zip(slots, seqs)])
    later = [eng.step([StepEntry(s, [ids[len(ids) - DECODED + t]], [0]) for s, ids in zip(slots, seqs)]) for t in range(DECODED)]
    if dtype == "bfloat16":
        assert any(st["graph"] is not None for st in eng._decode_graphs.values())       # the later steps were replays
    row = 0
    for b, (ids, ref) in enumerate(zip(seqs, refs)):
        n = len(ids) - DECODED
        got = torch.cat([first[row:row + n]] + [step[b:b + 1] for step in later])
        tiny.assert_logits_close(got, ref, dtype, f"36 layers, request {b} of {len(ids)} tokens")
        row += n
    for s in slots:
        eng.close(s)
    del eng
    torch.cuda.empty_cache()

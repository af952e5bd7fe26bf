"""Sizes that fit none of the fast paths, or only some: a width that is no multiple of 8 (rows of the matrices
do not start on 16 bytes: the exact product), head sizes that are no multiple of 16 (the exact attention
kernel), as many groups as heads.  Prompts of unequal lengths in one step, then single tokens."""
import pytest
import torch

import plain_qwen3 as P
import tiny

pytestmark = pytest.mark.gpu

_BASE = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", max_position_embeddings=512, tie_word_embeddings=False,
             rope_theta=10000.0, rms_norm_eps=1e-6)
ODD = {
    "width_100_heads_of_20": dict(vocab_size=301, hidden_size=100, num_hidden_layers=2, num_attention_heads=7, num_key_value_heads=7,
                                  head_dim=20, intermediate_size=172),
    "width_104_heads_of_40": dict(vocab_size=777, hidden_size=104, num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=3,
                                  head_dim=40, intermediate_size=200),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ODD))
def test_sizes_off_the_fast_paths(name, dtype, tmp_path):
    import palm_infra_amd
    from palm_infra_amd.engine import StepEntry
    from palm_infra_amd.weights import write_random_model
    cfg = dict(_BASE, **ODD[name])
    write_random_model(cfg, 4, tmp_path, dtype=dtype)
    c, w = P.read_model(tmp_path)
    eng = palm_infra_amd.load(str(tmp_path), dtype=dtype, max_tokens=64 * 16)
    g = torch.Generator().manual_seed(1)
    reqs = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (70, 5, 33)]
    slots = [eng.open() for _ in reqs]
    cuts = [50, 2, 33]
    out = eng.step([StepEntry(s, r[:k], list(range(k))) for s, r, k in zip(slots, reqs, cuts)])
    got, o = {i: [] for i in range(3)}, 0
    for i, k in enumerate(cuts):
        got[i].append(out[o:o + k]); o += k
    fed = list(cuts)
    while any(fed[i] < len(reqs[i]) for i in range(3)):
        live = [i for i in range(3) if fed[i] < len(reqs[i])]
        out = eng.step([StepEntry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
        for row, i in enumerate(live):
            got[i].append(out[row:row + 1]); fed[i] += 1
    for i in range(3):
        tiny.assert_logits_close(torch.cat(got[i]), P.logits(c, w, reqs[i]), dtype, f"{name} request {i}")
        eng.close(slots[i])
    eng.cache.check()

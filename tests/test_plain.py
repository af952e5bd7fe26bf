"""Pins the plain implementation (the oracle of the GPU tests) by what fixes it beside the reference's
text: vectors from the reference's own tests, special cases that reduce to a library routine, and
invariants, each chosen so that a plausible mistake fails it (no GPU)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as P
import tiny

F64 = torch.float64


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64) * scale


# ---- RMSNorm ------------------------------------------------------------------------------------

def test_rms_norm_with_unit_weight_is_the_library_routine():
    x = rand(5, 17, seed=1)
    assert torch.allclose(P.rms_norm(x, torch.ones(17, dtype=F64), 1e-6), F.rms_norm(x, (17,), eps=1e-6), atol=1e-12)


def test_rms_norm_eps_is_inside_the_root_and_weight_is_not_one_plus_w():
    # tiny x: eps inside the root gives x/sqrt(eps); outside it would give ~x/|x|
    x = torch.full((1, 4), 1e-6, dtype=F64)
    y = P.rms_norm(x, torch.ones(4, dtype=F64), 1e-6)
    assert torch.allclose(y, x / math.sqrt(1e-12 + 1e-6), rtol=1e-9)
    w = rand(4, seed=2)
    assert torch.allclose(P.rms_norm(rand(3, 4), w, 1e-6), P.rms_norm(rand(3, 4), torch.ones(4, dtype=F64), 1e-6) * w)
    assert float(P.rms_norm(torch.zeros(2, 32, dtype=F64), rand(32), 1e-6).abs().max()) == 0.0   # tests/test_norm.cpp:152-160
    # no mean subtraction: a constant row stays a constant, not zero
    assert torch.allclose(P.rms_norm(torch.full((1, 8), 3.0, dtype=F64), torch.ones(8, dtype=F64), 0.0 + 1e-30), torch.ones(1, 8, dtype=F64))


# ---- rotation -----------------------------------------------------------------------------------

def test_rope_table_matches_the_closed_form_of_the_reference_test():
    # tests/test_engine.cpp:90-105: cos(0)=1, sin(0)=0; sin(pos / theta^(2i/d))
    cos, sin = P.rope_table([0, 1, 2, 3], 64, 500000.0)
    assert abs(float(cos[0, 0]) - 1) < 1e-5 and abs(float(sin[0, 0])) < 1e-5 and cos.shape == (4, 32)
    for pos, i in ((1, 0), (2, 1), (3, 30)):
        assert abs(float(sin[pos, i]) - math.sin(pos / 500000.0 ** (2 * i / 64))) < 1e-6


def test_rope_pairs_are_half_split_not_interleaved():
    # a one-hot input at dim 1 must mix with dim 1 + half, not with dim 0 (tests/test_rope.cpp:22-53)
    hd = 8
    x = torch.zeros(1, 1, hd, dtype=F64)
    x[0, 0, 1] = 1.0
    cos, sin = P.rope_table([5], hd, 10000.0)
    y = P.rope_half_split(x, cos, sin)[0, 0]
    assert abs(float(y[1]) - float(cos[0, 1])) < 1e-12 and abs(float(y[1 + hd // 2]) - float(sin[0, 1])) < 1e-12
    assert float(y[0]) == 0.0 and float(y[2]) == 0.0


def test_rope_is_a_complex_multiplication_and_keeps_norms():
    hd, n = 16, 6
    x = rand(n, 3, hd, seed=3)
    pos = [0, 1, 7, 30, 31, 100]
    cos, sin = P.rope_table(pos, hd, 10000.0)
    y = P.rope_half_split(x, cos, sin)
    z = torch.complex(x[..., :hd // 2], x[..., hd // 2:]) * torch.complex(cos, sin)[:, None, :]
    assert torch.allclose(y[..., :hd // 2], z.real, atol=1e-12) and torch.allclose(y[..., hd // 2:], z.imag, atol=1e-12)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-12)
    assert torch.equal(P.rope_half_split(x[:1], *P.rope_table([0], hd, 10000.0)), x[:1])     # position 0 is the identity


def test_rope_scores_depend_on_distance_only():
    hd = 32
    q, k = rand(1, 1, hd, seed=4), rand(1, 1, hd, seed=5)

    def score(m, n):
        return float((P.rope_half_split(q, *P.rope_table([m], hd, 1e4)) * P.rope_half_split(k, *P.rope_table([n], hd, 1e4))).sum())
    assert abs(score(9, 4) - score(25, 20)) < 1e-4 and abs(score(9, 4) - score(4, 9)) > 1e-3   # sign of the angle matters


# ---- attention ----------------------------------------------------------------------------------

@pytest.mark.parametrize("nh,nkv", [(4, 4), (4, 2), (6, 1)])
def test_attention_is_the_library_routine_with_repeated_kv_heads(nh, nkv):
    n, hd = 11, 8
    q, k, v = rand(n, nh, hd, seed=6), rand(n, nkv, hd, seed=7), rand(n, nkv, hd, seed=8)
    got = P.causal_attention(q, k, v, hd ** -0.5)
    kr, vr = k.repeat_interleave(nh // nkv, dim=1), v.repeat_interleave(nh // nkv, dim=1)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), kr.transpose(0, 1), vr.transpose(0, 1), is_causal=True)
    assert torch.allclose(got, ref.transpose(0, 1), atol=1e-12)
    assert torch.allclose(got[0], vr[0], atol=1e-12)          # the first token attends only itself


def test_attention_head_to_kv_head_map():
    # consecutive query heads share a kv head (kernels/attention.cpp:1161): make every kv head's v a constant
    n, nh, nkv, hd = 3, 6, 3, 4
    v = torch.stack([torch.full((n, hd), float(g + 1), dtype=F64) for g in range(nkv)], dim=1)
    out = P.causal_attention(rand(n, nh, hd), rand(n, nkv, hd, seed=1), v, 0.5)
    assert [float(out[2, h, 0]) for h in range(nh)] == pytest.approx([1, 1, 2, 2, 3, 3])


def test_attention_window_and_mask_semantics():
    # engine/input_prep.cpp:8-15: key j is visible to query i iff j <= i
    n, hd = 6, 4
    q, k = rand(n, 1, hd, seed=2), rand(n, 1, hd, seed=3)
    v = torch.eye(n, dtype=F64)[:, None, :]                    # output row = the attention weights
    w = P.causal_attention(q, k, v, 1.0)[:, 0, :]
    assert float(w.triu(1).abs().max()) == 0.0 and torch.allclose(w.sum(-1), torch.ones(n, dtype=F64))
    ww = P.causal_attention(q, k, v, 1.0, window=2)[:, 0, :]
    assert float(ww[4, 2]) == 0.0 and float(ww[4, 3]) > 0 and float(ww[4, 4]) > 0


# ---- feed-forward, linear -----------------------------------------------------------------------

def test_swiglu_is_silu_of_gate_times_up():
    h, wg, wu, wd = rand(4, 6, seed=1), rand(10, 6, seed=2), rand(10, 6, seed=3), rand(6, 10, seed=4)
    ref = F.linear(F.silu(F.linear(h, wg)) * F.linear(h, wu), wd)
    assert torch.allclose(P.swiglu_mlp(h, wg, wu, wd), ref, atol=1e-12)
    assert not torch.allclose(P.swiglu_mlp(h, wu, wg, wd), ref, atol=1e-3)       # swapping the halves changes it


def test_linear_layout_is_out_by_in():
    x, w = rand(3, 5), rand(7, 5, seed=1)
    assert torch.allclose(P.linear(x, w), F.linear(x, w), atol=1e-12)


# ---- the whole model ----------------------------------------------------------------------------

def _model(name="A"):
    cfg = tiny.CONFIGS[name]
    w = {k: v.double() for k, v in tiny.sharpened_tensors(name, "float32").items()}
    return cfg, w


def test_branches_add_to_the_residual_stream():
    cfg, w = _model("A")
    ids = [5, 9, 200, 31]
    for i in range(cfg["num_hidden_layers"]):
        w[f"model.layers.{i}.self_attn.o_proj.weight"].zero_()
        w[f"model.layers.{i}.mlp.down_proj.weight"].zero_()
    x = P.embedding(w["model.embed_tokens.weight"], ids)
    assert torch.allclose(P.hidden_states(cfg, w, ids), P.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]), atol=1e-12)


def test_only_attention_mixes_positions():
    cfg, w = _model("A")
    a, b = P.hidden_states(cfg, w, [5, 9, 200, 31]), P.hidden_states(cfg, w, [6, 9, 200, 31])
    assert not torch.allclose(a[3], b[3], atol=1e-6)
    for i in range(cfg["num_hidden_layers"]):
        w[f"model.layers.{i}.self_attn.o_proj.weight"].zero_()
    a, b = P.hidden_states(cfg, w, [5, 9, 200, 31]), P.hidden_states(cfg, w, [6, 9, 200, 31])
    assert torch.allclose(a[3], b[3], atol=1e-12)


def test_scale_is_head_dim_not_hidden_over_heads():
    # B has head_dim 32 and hidden/heads = 12: the two scales differ
    cfg, w = _model("B")
    S = P.sizes(cfg)
    assert S["hd"] == 32 and S["H"] // S["nh"] == 12
    ids = tiny.prompts("B", [9])[0]
    x = P.embedding(w["model.embed_tokens.weight"], ids)
    h = P.rms_norm(x, w["model.layers.0.input_layernorm.weight"], S["eps"])
    got = P.attention_block(h, w, "model.layers.0.self_attn.", S, list(range(9)))
    n = 9
    q = P.rms_norm(P.linear(h, w["model.layers.0.self_attn.q_proj.weight"]).reshape(n, 8, 32), w["model.layers.0.self_attn.q_norm.weight"], S["eps"])
    k = P.rms_norm(P.linear(h, w["model.layers.0.self_attn.k_proj.weight"]).reshape(n, 1, 32), w["model.layers.0.self_attn.k_norm.weight"], S["eps"])
    v = P.linear(h, w["model.layers.0.self_attn.v_proj.weight"]).reshape(n, 1, 32)
    cos, sin = P.rope_table(list(range(n)), 32, S["theta"])
    q, k = P.rope_half_split(q, cos, sin), P.rope_half_split(k, cos, sin)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k.expand(n, 8, 32).transpose(0, 1), v.expand(n, 8, 32).transpose(0, 1),
                                         is_causal=True, scale=32 ** -0.5).transpose(0, 1).reshape(n, 256)
    assert torch.allclose(got, P.linear(ref, w["model.layers.0.self_attn.o_proj.weight"]), atol=1e-10)


def _attention_inputs(name="B", n=9, seed=0):
    cfg, w = _model(name)
    S = P.sizes(cfg)
    ids = tiny.prompts(name, [n], seed=seed)[0]
    x = P.embedding(w["model.embed_tokens.weight"], ids)
    h = P.rms_norm(x, w["model.layers.0.input_layernorm.weight"], S["eps"])
    return cfg, w, S, h


def test_q_and_k_are_normed_before_they_are_rotated():
    """models/qwen3.py:315-334: RMSNorm of q and k per head, then the rotation.  With a norm weight that differs
    from element to element the two orders differ (the rotation mixes element i with i + half, which carry
    different weights); with a constant weight they would not, which is why the weight is made uneven here."""
    cfg, w, S, h = _attention_inputs("B")
    a = "model.layers.0.self_attn."
    hd, nh, nkv, n = S["hd"], S["nh"], S["nkv"], h.shape[0]
    w[a + "q_norm.weight"] = torch.linspace(0.2, 3.0, hd, dtype=F64)
    w[a + "k_norm.weight"] = torch.linspace(2.5, 0.3, hd, dtype=F64)
    got = P.attention_block(h, w, a, S, list(range(n)))
    q = P.linear(h, w[a + "q_proj.weight"]).reshape(n, nh, hd)
    k = P.linear(h, w[a + "k_proj.weight"]).reshape(n, nkv, hd)
    v = P.linear(h, w[a + "v_proj.weight"]).reshape(n, nkv, hd)
    cos, sin = P.rope_table(list(range(n)), hd, S["theta"])

    def finish(q, k):
        return P.linear(P.causal_attention(q, k, v, hd ** -0.5).reshape(n, nh * hd), w[a + "o_proj.weight"])
    norm_then_rotate = finish(P.rope_half_split(P.rms_norm(q, w[a + "q_norm.weight"], S["eps"]), cos, sin),
                              P.rope_half_split(P.rms_norm(k, w[a + "k_norm.weight"], S["eps"]), cos, sin))
    rotate_then_norm = finish(P.rms_norm(P.rope_half_split(q, cos, sin), w[a + "q_norm.weight"], S["eps"]),
                              P.rms_norm(P.rope_half_split(k, cos, sin), w[a + "k_norm.weight"], S["eps"]))
    assert torch.allclose(got, norm_then_rotate, atol=1e-12)
    assert float((got - rotate_then_norm).abs().max()) > 1e-2 * float(got.abs().max())


def test_one_q_norm_weight_serves_all_heads():
    """The q norm's weight has head_dim elements and every head uses it (models/qwen3.py:315-324): so renumbering
    the query heads of a kv group (rows of q_proj, columns of o_proj) changes nothing.  A weight of its own for
    each head, or a norm over all heads together, would not commute with the renumbering."""
    cfg, w, S, h = _attention_inputs("B")
    a = "model.layers.0.self_attn."
    hd, nh, n = S["hd"], S["nh"], h.shape[0]
    w[a + "q_norm.weight"] = torch.linspace(0.2, 3.0, hd, dtype=F64)
    before = P.attention_block(h, w, a, S, list(range(n)))
    perm = torch.tensor([3, 0, 7, 1, 6, 2, 5, 4])                    # B has one kv head: all eight heads are one group
    rows = (perm[:, None] * hd + torch.arange(hd)[None, :]).reshape(-1)
    w2 = dict(w)
    w2[a + "q_proj.weight"] = w[a + "q_proj.weight"][rows]
    w2[a + "o_proj.weight"] = w[a + "o_proj.weight"][:, rows]
    assert torch.allclose(P.attention_block(h, w2, a, S, list(range(n))), before, atol=1e-12)
    # and the norm is over one head's elements, not over all heads: scaling one head's rows of q_proj changes nothing
    w3 = dict(w)
    w3[a + "q_proj.weight"] = w[a + "q_proj.weight"].clone()
    w3[a + "q_proj.weight"][2 * hd:3 * hd] *= 7.0
    # (up to eps, which weighs 49 times less beside the larger mean square)
    assert torch.allclose(P.attention_block(h, w3, a, S, list(range(n))), before, atol=1e-4 * float(before.abs().max()))


def test_the_q_and_k_norms_use_the_model_s_eps_and_v_is_not_normed():
    """models/qwen3.py:315-324 hands rms_norm_eps to both head norms; v goes to the cache as it is."""
    cfg, w, S, h = _attention_inputs("B")
    a = "model.layers.0.self_attn."
    hd, nh, nkv, n = S["hd"], S["nh"], S["nkv"], h.shape[0]
    for key in ("q_proj.weight", "k_proj.weight"):
        w[a + key] = w[a + key] * 1e-3                               # mean squares of the order of eps (1e-5): eps counts
    got = P.attention_block(h, w, a, S, list(range(n)))
    q = P.linear(h, w[a + "q_proj.weight"]).reshape(n, nh, hd)
    k = P.linear(h, w[a + "k_proj.weight"]).reshape(n, nkv, hd)
    v = P.linear(h, w[a + "v_proj.weight"]).reshape(n, nkv, hd)
    cos, sin = P.rope_table(list(range(n)), hd, S["theta"])

    def with_eps(eps):
        qn = (q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps)) * w[a + "q_norm.weight"]
        kn = (k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps)) * w[a + "k_norm.weight"]
        o = P.causal_attention(P.rope_half_split(qn, cos, sin), P.rope_half_split(kn, cos, sin), v, hd ** -0.5)
        return P.linear(o.reshape(n, nh * hd), w[a + "o_proj.weight"])
    assert torch.allclose(got, with_eps(cfg["rms_norm_eps"]), atol=1e-12)
    assert float((got - with_eps(1e-6)).abs().max()) > 1e-3 * float(got.abs().max())         # another eps shows
    # v is used as it is: three times v gives three times the output (a normed v would give the same output)
    w2 = dict(w)
    w2[a + "v_proj.weight"] = w[a + "v_proj.weight"] * 3.0
    assert torch.allclose(P.attention_block(h, w2, a, S, list(range(n))), 3.0 * got, atol=1e-10)


def test_tied_and_untied_heads():
    cfg, w = _model("A")
    ids = [1, 2, 3]
    assert torch.allclose(P.logits(cfg, w, ids), P.hidden_states(cfg, w, ids) @ w["model.embed_tokens.weight"].T)
    cfgb, wb = _model("B")
    h0, l0 = P.hidden_states(cfgb, wb, ids), P.logits(cfgb, wb, ids)
    wb["lm_head.weight"] = wb["lm_head.weight"] * 2
    assert torch.allclose(P.hidden_states(cfgb, wb, ids), h0) and torch.allclose(P.logits(cfgb, wb, ids), 2 * l0)


def test_a_shift_of_all_positions_changes_nothing():
    # only distances count: the same tokens at positions 40.. give the same hidden states (up to the float32 table)
    cfg, w = _model("A")
    ids = tiny.prompts("A", [12])[0]
    assert torch.allclose(P.hidden_states(cfg, w, ids, 0), P.hidden_states(cfg, w, ids, 40), atol=2e-4)


def test_causality_of_the_whole_model():
    cfg, w = _model("B")
    ids = tiny.prompts("B", [10])[0]
    assert torch.allclose(P.logits(cfg, w, ids)[:6], P.logits(cfg, w, ids[:6]), atol=1e-10)


def test_plain_greedy_stops_on_a_stop_token_and_keeps_it():
    cfg, w = _model("A")
    out = P.greedy(cfg, w, [3, 4, 5], 6)
    assert len(out) == 6
    stop = out[2]
    first = out.index(stop)
    assert P.greedy(cfg, w, [3, 4, 5], 6, stop=(stop,)) == out[:first + 1]


# ---- sampling -----------------------------------------------------------------------------------

def test_sampling_vectors_of_the_reference():
    # tests/test_sampler.cpp:19-60
    assert P.draw([0.5, 3.0, 2.0], 0.3, temperature=0.0) == 1
    assert P.draw([0.5, 3.0, 2.0], 0.99, temperature=1.0, top_k=1) == 1
    for u in (0.0, 0.5, 0.999):
        assert P.draw([4.0, 0.0, -1.0], u, temperature=1.0, min_p=0.5) == 0
        assert P.draw([4.0, 0.0, -1.0], u, temperature=1.0, top_p=0.5) == 0
    # tests/test_sampler.cpp:170-181
    p = P.probabilities([0.0, math.log(2.0), math.log(3.0)], 1.0, top_k=0, top_p=1.0)
    assert np.allclose(p, [1 / 6, 2 / 6, 3 / 6], atol=1e-5)


def test_candidates_ties_and_filters():
    ids, w = P.candidates([1.0, 2.0, 2.0, 0.0], 1.0, top_k=2)
    assert ids == [1, 2]                                        # ties to the lower id (engine/sampler.cpp:93-119)
    ids, w = P.candidates([1.0, 2.0, 2.0, 0.0], 1.0, top_k=1)
    assert ids == [1]
    ids, _ = P.candidates([0.0, math.log(2), math.log(3), math.log(4)], 1.0, top_p=0.65)
    assert ids == [3, 2]                                        # 0.4, then 0.7 >= 0.65
    lg = P.apply_penalties([2.0, -2.0, 1.0, 0.5], [0, 1, 1, 7], repeat_penalty=2.0, repeat_last_n=3, presence_penalty=0.5, frequency_penalty=0.25)
    # window of 3: tokens 1 (twice) and 7 (out of range); token 0 is outside the window
    assert np.allclose(lg, [2.0, -2.0 * 2 - 0.5 - 0.5, 1.0, 0.5])
    assert np.allclose(P.apply_penalties([2.0, -2.0], [0], repeat_penalty=2.0, repeat_last_n=-1), [1.0, -2.0])
    assert np.allclose(P.apply_penalties([2.0, -2.0], [0, 1], repeat_penalty=2.0, repeat_last_n=0), [2.0, -2.0])

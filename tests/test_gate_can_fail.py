"""Shows that the bfloat16 gate of the engine tests (tiny.assert_logits_close) can fail: the plain implementation
with one deliberate mistake each, confined to one kv head of one layer, is fed to the gate in place of the
engine's logits, and the gate must reject every one, at every tiny configuration, both for many rows checked
together and for rows collected a few at a time.  (No GPU: both sides are the plain implementation.)

The mistakes are those a cache or a step function would make:
  page      the head reads the keys and values of positions 0..63 where those of 64..127 belong, and the reverse
            (a wrong entry in a page table)
  stale     a query at position i also sees a key at i + 1 that another sequence left behind (a read beyond the
            sequence's length)
  rotation  the head's queries are rotated by position + 1 (a decoded token given the wrong position)
"""
import math

import pytest
import torch

import plain_qwen3 as P
import tiny

F64 = torch.float64
FAULTS = ("page", "stale", "rotation")


def attention_with_a_fault(h, w, prefix, S, n, fault, kv_head):
    nh, nkv, hd = S["nh"], S["nkv"], S["hd"]
    group = nh // nkv
    q = P.rms_norm(P.linear(h, w[prefix + "q_proj.weight"]).reshape(n, nh, hd), w[prefix + "q_norm.weight"], S["eps"])
    k = P.rms_norm(P.linear(h, w[prefix + "k_proj.weight"]).reshape(n, nkv, hd), w[prefix + "k_norm.weight"], S["eps"])
    v = P.linear(h, w[prefix + "v_proj.weight"]).reshape(n, nkv, hd)
    cos, sin = P.rope_table(list(range(n)), hd, S["theta"])
    q_good = P.rope_half_split(q, cos, sin)
    k = P.rope_half_split(k, cos, sin)
    if fault == "rotation":
        cos1, sin1 = P.rope_table(list(range(1, n + 1)), hd, S["theta"])
        q_bad = P.rope_half_split(q, cos1, sin1)
    out = torch.zeros(n, nh, hd, dtype=F64)
    idx = torch.arange(n)
    causal = idx[None, :] <= idx[:, None]
    for head in range(nh):
        g = head // group
        faulty = g == kv_head
        qh, kh, vh, visible = q_good[:, head], k[:, g], v[:, g], causal
        if faulty and fault == "rotation":
            qh = q_bad[:, head]
        if faulty and fault == "page":
            perm = torch.arange(n)
            m = min(64, n - 64)
            perm[:m], perm[64:64 + m] = torch.arange(64, 64 + m), torch.arange(m)
            kh, vh = kh[perm], vh[perm]
        if faulty and fault == "stale":
            # n more keys: key n + j stands at position j and holds what position n - 1 - j of this head holds;
            # query i sees it only where j == i + 1
            kh, vh = torch.cat([kh, kh.flip(0)]), torch.cat([vh, vh.flip(0)])
            visible = torch.cat([causal, idx[None, :] == idx[:, None] + 1], dim=1)
        s = (qh @ kh.T) * hd ** -0.5
        s = s.masked_fill(~visible, -math.inf)
        p = torch.softmax(s, dim=-1)
        out[:, head] = p @ vh
    return P.linear(out.reshape(n, nh * hd), w[prefix + "o_proj.weight"])


def logits_with_a_fault(cfg, w, ids, fault, layer, kv_head):
    S = P.sizes(cfg)
    n = len(ids)
    x = P.embedding(w["model.embed_tokens.weight"], ids)
    for i in range(S["L"]):
        p = f"model.layers.{i}."
        h = P.rms_norm(x, w[p + "input_layernorm.weight"], S["eps"])
        if i == layer:
            x = x + attention_with_a_fault(h, w, p + "self_attn.", S, n, fault, kv_head)
        else:
            x = x + P.attention_block(h, w, p + "self_attn.", S, list(range(n)))
        h = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], S["eps"])
        x = x + P.swiglu_mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.linear(P.rms_norm(x, w["model.norm.weight"], S["eps"]), P.head_weight(w))


def model(name):
    cfg = tiny.CONFIGS[name]
    return cfg, {k: v.double() for k, v in tiny.sharpened_tensors(name, "bfloat16").items()}


def test_the_faulty_functions_are_the_plain_ones_without_their_fault():
    cfg, w = model("A")
    ids = tiny.prompts("A", [70], seed=1)[0]
    assert torch.allclose(logits_with_a_fault(cfg, w, ids, None, 0, 0), P.logits(cfg, w, ids), atol=1e-10)


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("fault", FAULTS)
def test_the_bfloat16_gate_rejects_a_fault_in_one_kv_head_of_one_layer(name, fault):
    cfg, w = model(name)
    n = 120
    ids = tiny.prompts(name, [n], seed=3)[0]
    ref = P.logits(cfg, w, ids)
    last_layer, last_head = cfg["num_hidden_layers"] - 1, cfg["num_key_value_heads"] - 1
    for layer, kv_head in ((0, 0), (last_layer, last_head)):
        bad = logits_with_a_fault(cfg, w, ids, fault, layer, kv_head)
        # "page" and "stale" change what the later positions see: those are the rows a decode test checks
        rows = slice(64, n) if fault == "page" else slice(0, n - 1)
        with pytest.raises(AssertionError):
            tiny.assert_logits_close(bad[rows], ref[rows], "bfloat16", f"{name} {fault}")
        # and a few rows at a time, pooled, as the decode tests do it
        with pytest.raises(AssertionError):
            pool = tiny.LogitsPool("bfloat16", f"{name} {fault}")
            for t in range(rows.start, rows.stop - 1, 2)[:24]:
                pool.add(bad[t:t + 2], ref[t:t + 2])
            pool.check()
    # the gate itself is not a coin: the plain logits, rounded as a bfloat16 run rounds its output, pass
    tiny.assert_logits_close(ref.to(torch.bfloat16).double(), ref, "bfloat16", "rounded logits")

"""A plain, slow implementation of the dense Qwen3 decoder, used only as the oracle of the tests.

Whole sequences, no cache, no batching, one function for each part.  It is written from the
formulas of the reference engine (each function cites where the reference has them) and shares no
code with the package under test: it reads config.json and the safetensors file with its own few
lines, and computes in float64 on the CPU (the rotation table is built in float32 like the
reference builds it).

Citations are paths under the reference checkout, as ``file:line``.
"""
from __future__ import annotations

import json
import math
import struct
from pathlib import Path

import numpy as np
import torch

F64 = torch.float64


# --------------------------------------------------------------------------------------------
# files
# --------------------------------------------------------------------------------------------

def read_safetensors(path) -> dict[str, torch.Tensor]:
    """8-byte little-endian header length, a JSON header with dtype/shape/data_offsets for each
    tensor, then the raw bytes (models/qwen35.py:95-123).  Every tensor is widened to float64."""
    raw = Path(path).read_bytes()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + hlen])
    base = 8 + hlen
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        a, b = meta["data_offsets"]
        buf = raw[base + a:base + b]
        dt = meta["dtype"]
        if dt == "F32":
            arr = np.frombuffer(buf, dtype="<f4").astype(np.float64)
        elif dt == "F16":
            arr = np.frombuffer(buf, dtype="<f2").astype(np.float64)
        elif dt == "BF16":
            # bf16 is the upper half of a float32 (models/qwen35.py:118-120)
            u = np.frombuffer(buf, dtype="<u2").astype(np.uint32) << 16
            arr = u.view(np.float32).astype(np.float64)
        else:
            raise ValueError(f"{name}: dtype {dt}")
        out[name] = torch.from_numpy(arr.reshape(meta["shape"]).copy())
    return out


def read_model(model_dir):
    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    return cfg, read_safetensors(model_dir / "model.safetensors")


def sizes(cfg: dict) -> dict:
    """The keys and defaults that the reference reads (models/qwen3.py:175-184)."""
    nh = cfg["num_attention_heads"]
    return dict(
        H=cfg["hidden_size"], L=cfg["num_hidden_layers"], eps=cfg.get("rms_norm_eps", 1e-6),
        theta=cfg.get("rope_theta", 1000000.0), nh=nh, nkv=cfg.get("num_key_value_heads", nh),
        hd=cfg.get("head_dim", cfg["hidden_size"] // nh), I=cfg["intermediate_size"],
        V=cfg["vocab_size"],
    )


# --------------------------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------------------------

def embedding(table: torch.Tensor, ids) -> torch.Tensor:
    """x[t, :] = E[id_t, :] (engine/engine.cpp:332-357)."""
    return table[torch.as_tensor(ids, dtype=torch.long)].to(F64)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * (1 / sqrt(mean(x^2) + eps)) * w over the last dim; eps inside the root, the weight
    multiplies as it is (kernels/norm.cpp:13-31)."""
    x = x.to(F64)
    r = 1.0 / torch.sqrt((x * x).sum(-1, keepdim=True) / x.shape[-1] + eps)
    return x * r * w.to(F64)


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """y = x W^T with W stored [out, in], no bias (kernels/matmul_dense.cpp:939-953)."""
    return x.to(F64) @ w.to(F64).T


def rope_table(positions, rope_dim: int, theta: float):
    """cos/sin [n, rope_dim/2]: inv_i = 1 / theta^(2i/rope_dim), angle = pos * inv_i, all in
    float32 as the reference computes them (engine/input_prep.cpp:17-30)."""
    half = rope_dim // 2
    i = np.arange(half, dtype=np.float32)
    inv = (np.float32(1.0) / np.power(np.float32(theta), np.float32(2.0) * i / np.float32(rope_dim))
           ).astype(np.float32)
    pos = np.asarray(positions, dtype=np.float32)
    ang = (pos[:, None] * inv[None, :]).astype(np.float32)
    return torch.from_numpy(np.cos(ang).astype(np.float64)), torch.from_numpy(np.sin(ang).astype(np.float64))


def rope_half_split(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [n, heads, hd]; pairs are (i, i + hd/2): y_i = x_i c - x_{i+h} s, y_{i+h} = x_i s + x_{i+h} c
    (kernels/rope.cpp:38-48, the interleave=false branch; models/qwen3.py:333-334)."""
    half = cos.shape[-1]
    x = x.to(F64)
    x0, x1, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat([x0 * c - x1 * s, x0 * s + x1 * c, rest], dim=-1)


def causal_attention(q, k, v, scale: float, window: int | None = None) -> torch.Tensor:
    """q [n, nh, hd], k/v [n, nkv, hd] of one whole sequence -> [n, nh, hd].

    Head h reads kv head h // (nh/nkv) (kernels/attention.cpp:1161); s_ij = scale * q_i.k_j, key j
    is visible to query i iff j <= i (engine/input_prep.cpp:8-15) and, with a window w, j > i - w;
    softmax with the maximum subtracted, then the weighted sum of v (kernels/attention.cpp:937-962).
    """
    n, nh, hd = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    out = torch.zeros(n, nh, v.shape[-1], dtype=F64)
    idx = torch.arange(n)
    visible = idx[None, :] <= idx[:, None]
    if window is not None:
        visible &= idx[None, :] > idx[:, None] - window
    for h in range(nh):
        g = h // group
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        s = s.masked_fill(~visible, -math.inf)
        s = s - s.max(dim=-1, keepdim=True).values
        p = torch.exp(s)
        p = p / p.sum(-1, keepdim=True)
        out[:, h, :] = p @ v[:, g, :]
    return out


def attention_block(h, w, prefix, S, positions, window=None) -> torch.Tensor:
    """Projections, per-head RMSNorm of q and k over head_dim with one weight vector for all heads
    and the model's eps, rotation of both, attention with scale head_dim^-0.5, output projection
    (models/qwen3.py:290-349).  v is neither normed nor rotated."""
    n = h.shape[0]
    q = linear(h, w[prefix + "q_proj.weight"]).reshape(n, S["nh"], S["hd"])
    k = linear(h, w[prefix + "k_proj.weight"]).reshape(n, S["nkv"], S["hd"])
    v = linear(h, w[prefix + "v_proj.weight"]).reshape(n, S["nkv"], S["hd"])
    q = rms_norm(q, w[prefix + "q_norm.weight"], S["eps"])
    k = rms_norm(k, w[prefix + "k_norm.weight"], S["eps"])
    cos, sin = rope_table(positions, S["hd"], S["theta"])
    q = rope_half_split(q, cos, sin)
    k = rope_half_split(k, cos, sin)
    o = causal_attention(q, k, v, S["hd"] ** -0.5, window)
    return linear(o.reshape(n, S["nh"] * S["hd"]), w[prefix + "o_proj.weight"])


def swiglu_mlp(h, w_gate, w_up, w_down) -> torch.Tensor:
    """down( silu(gate(h)) * up(h) ), silu(z) = z / (1 + exp(-z)) (models/qwen3.py:276-287,
    kernels/elementwise.cpp:578-582)."""
    g = linear(h, w_gate)
    u = linear(h, w_up)
    return linear(g / (1.0 + torch.exp(-g)) * u, w_down)


def decoder_layer(x, w, i, S, positions, window=None) -> torch.Tensor:
    """x += attn(norm(x)); x += mlp(norm(x)) (models/qwen3.py:254-287)."""
    p = f"model.layers.{i}."
    h = rms_norm(x, w[p + "input_layernorm.weight"], S["eps"])
    x = x + attention_block(h, w, p + "self_attn.", S, positions, window)
    h = rms_norm(x, w[p + "post_attention_layernorm.weight"], S["eps"])
    return x + swiglu_mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                          w[p + "mlp.down_proj.weight"])


def hidden_states(cfg, w, ids, first_position: int = 0) -> torch.Tensor:
    """The final-norm output for every position (models/qwen3.py:237-248)."""
    S = sizes(cfg)
    positions = [first_position + t for t in range(len(ids))]
    x = embedding(w["model.embed_tokens.weight"], ids)
    for i in range(S["L"]):
        x = decoder_layer(x, w, i, S, positions)
    return rms_norm(x, w["model.norm.weight"], S["eps"])


def head_weight(w) -> torch.Tensor:
    """lm_head.weight if the file has it, else the embedding table (models/qwen3.py:89-95, 162-165)."""
    return w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]


def logits(cfg, w, ids) -> torch.Tensor:
    """[n, V] for every position of one whole sequence (engine/engine.cpp:487-555)."""
    return linear(hidden_states(cfg, w, ids), head_weight(w))


def greedy(cfg, w, prompt, n_new: int, stop=()) -> list[int]:
    """Prefill, then one token at a time, each time over the whole sequence; the lowest index wins
    a tie (engine/sampler.cpp:72-77); the stop token is kept (examples/cli_common.cpp:486-519)."""
    ids = list(prompt)
    out = []
    for _ in range(n_new):
        nxt = int(torch.argmax(logits(cfg, w, ids)[-1]))
        out.append(nxt)
        ids.append(nxt)
        if nxt in stop:
            break
    return out


# --------------------------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------------------------

def apply_penalties(lg: np.ndarray, history, repeat_penalty=1.0, repeat_last_n=64,
                    presence_penalty=0.0, frequency_penalty=0.0) -> np.ndarray:
    """Tokens seen in the last repeat_last_n of the history (-1: all, 0: off): l>0 ? l/r : l*r,
    then l -= presence, l -= frequency * count (engine/sampler.cpp:304-343)."""
    lg = np.array(lg, dtype=np.float64)
    on = repeat_last_n != 0 and (repeat_penalty != 1.0 or presence_penalty != 0.0 or frequency_penalty != 0.0)
    if not on:
        return lg
    window = len(history) if repeat_last_n < 0 else min(len(history), repeat_last_n)
    counts: dict[int, int] = {}
    for t in history[len(history) - window:]:
        if 0 <= t < len(lg):
            counts[t] = counts.get(t, 0) + 1
    for t, c in counts.items():
        if repeat_penalty != 1.0:
            lg[t] = lg[t] / repeat_penalty if lg[t] > 0 else lg[t] * repeat_penalty
        lg[t] -= presence_penalty
        lg[t] -= frequency_penalty * c
    return lg


def candidates(lg, temperature: float, top_k: int = 0, top_p: float = 0.0, min_p: float = 0.0):
    """The candidate list of the reference (engine/sampler.cpp:90-157): the k largest logits (ties to
    the lower id), sorted; p = exp((l - l_max)/T); min_p drops p < min_p * p_best; top_p keeps the
    shortest prefix whose mass reaches top_p * sum.  Returns (ids, weights) in that order."""
    lg = np.asarray(lg, dtype=np.float64)
    order = sorted(range(len(lg)), key=lambda i: (-lg[i], i))
    if top_k > 0:
        order = order[:min(top_k, len(lg))]
    p = np.exp((lg[order] - lg[order[0]]) / temperature)
    active = len(order)
    if min_p > 0.0:
        active = 1
        while active < len(order) and p[active] >= min_p * p[0]:
            active += 1
    total = p[:active].sum()
    if 0.0 < top_p < 1.0:
        cum = 0.0
        for i in range(active):
            cum += p[i]
            if cum >= top_p * total:
                active = i + 1
                break
    return order[:active], p[:active]


def probabilities(lg, temperature, top_k=0, top_p=0.0, min_p=0.0) -> np.ndarray:
    """The distribution that sampling draws from (engine/sampler.cpp:190-216); one-hot at the
    first maximum when temperature <= 0 or top_k == 1 (engine/sampler.cpp:171-172)."""
    out = np.zeros(len(lg))
    if temperature <= 0.0 or top_k == 1:
        out[int(np.argmax(np.asarray(lg)))] = 1.0
        return out
    ids, p = candidates(lg, temperature, top_k, top_p, min_p)
    out[ids] = p / p.sum()
    return out


def draw(lg, u: float, temperature, top_k=0, top_p=0.0, min_p=0.0) -> int:
    """Walk the cumulative weights of the sorted candidates until u * sum is reached
    (engine/sampler.cpp:180-187)."""
    if temperature <= 0.0 or top_k == 1:
        return int(np.argmax(np.asarray(lg)))
    ids, p = candidates(lg, temperature, top_k, top_p, min_p)
    target = u * p.sum()
    cum = 0.0
    for i, w in zip(ids, p):
        cum += w
        if target <= cum:
            return i
    return ids[-1]

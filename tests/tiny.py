"""The tiny configurations of the tests and helpers to make model folders and prompts.

A and B differ in every size and option (layers, width, heads and groups, head size, heads*head_dim equal
to the width or not, a feed-forward width that is no power of two, vocabulary, rotation base, eps, tied or
untied head); C adds head sizes and widths that are no power of two at all, one kv head per head, and
room for long sequences; D has heads of 64, the smallest size at which a bfloat16 decode step takes the attention
kernel that starts from the joined projection's rows, and two heads a kv head.

The weights are the random-weights mode's, then sharpened so that faults show: matrices are four times
larger (logits of order one instead of a tenth) and the q norm's weight is four times larger, which makes
attention scores of order four, so that a wrong or missing key changes the output by much more than
rounding does.
"""
from __future__ import annotations

import json
from pathlib import Path

import torch

from palm_infra_amd.config import config_from_dict
from palm_infra_amd.weights import random_tensors, write_safetensors

_BASE = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3")

CONFIGS = {
    "A": dict(_BASE, vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
              head_dim=16, intermediate_size=128, tie_word_embeddings=True, rope_theta=10000.0, rms_norm_eps=1e-6,
              max_position_embeddings=128, eos_token_id=7),
    "B": dict(_BASE, vocab_size=1000, hidden_size=96, num_hidden_layers=3, num_attention_heads=8, num_key_value_heads=1,
              head_dim=32, intermediate_size=224, tie_word_embeddings=False, rope_theta=1000000.0, rms_norm_eps=1e-5,
              max_position_embeddings=256, eos_token_id=[3, 11]),
    "C": dict(_BASE, vocab_size=515, hidden_size=80, num_hidden_layers=2, num_attention_heads=5, num_key_value_heads=5,
              head_dim=48, intermediate_size=176, tie_word_embeddings=False, rope_theta=500000.0, rms_norm_eps=3e-6,
              max_position_embeddings=2048),
    "D": dict(_BASE, vocab_size=300, hidden_size=88, num_hidden_layers=2, num_attention_heads=6, num_key_value_heads=3,
              head_dim=64, intermediate_size=200, tie_word_embeddings=True, rope_theta=20000.0, rms_norm_eps=2e-6,
              max_position_embeddings=512, eos_token_id=5),
}
SEEDS = {"A": 0, "B": 1, "C": 2, "D": 3}


def sharpened_tensors(name: str, store: str) -> dict[str, torch.Tensor]:
    cfg = config_from_dict(CONFIGS[name])
    tensors = random_tensors(cfg.spec(), SEEDS[name], "float32")
    out = {}
    for k, t in tensors.items():
        if t.dim() == 2:
            t = t * 4.0
        elif k.endswith("q_norm.weight"):
            t = t * 4.0
        out[k] = t.to({"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}[store])
    return out


def write_model(name: str, path, store: str) -> Path:
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(CONFIGS[name]))
    write_safetensors(path / "model.safetensors", sharpened_tensors(name, store))
    return path


def prompts(name: str, lengths, seed: int = 0) -> list[list[int]]:
    g = torch.Generator().manual_seed(1000 + seed)
    V = CONFIGS[name]["vocab_size"]
    return [torch.randint(0, V, (n,), generator=g).tolist() for n in lengths]


# What "equal" means for logits.
#   float32: the engine differs from the float64 oracle by the rounding of 32-bit sums: 1e-4 absolute
#            on logits of order one.  This is the gate that shows faults: a wrong, missing or stale key, a
#            wrong position or pairing moves a row of logits by the order of the logits themselves.
#   bfloat16: the same code paths with activations rounded to 8 bits (relative 2^-9) about ten times a layer.
#            The sharpened q norm makes scores of order 4, so rounding q and k moves a score by about 0.01 and a
#            softmax weight by as many percent; with the other roundings a row of logits is off by a few percent
#            of the logits' scale, more at positions where two keys compete.  Measured on paths whose float32
#            twin is exact (configuration B, one kv head and three layers, is the worst): up to 3.2 % for the root
#            mean square over all logits, up to 11 % for one position's row, up to 25 % for one element.  The
#            gates are twice the largest row and element errors seen and 1.5 times the overall one; a fault moves
#            a row by the order of the scale itself, and every bfloat16 case has a float32 twin held to 1e-4.
#            (The reference's own CPU-vs-GPU gate for float16, which has three bits more, is 2e-3 on unsharpened
#            logits, tests/test_tiny_cpu_inference.cpp:152-172.)
FLOAT32_ABS = 1e-4
BFLOAT16_RMS_REL = 5e-2
BFLOAT16_ROW_RMS_REL = 2e-1
BFLOAT16_MAX_REL = 5e-1


def assert_logits_close(got, ref, dtype: str, what: str = "") -> None:
    got = torch.as_tensor(got).double().cpu().reshape(ref.shape)
    ref = ref.double()
    err = (got - ref).abs()
    assert torch.isfinite(got).all(), f"{what}: logits are not finite"
    if dtype == "float32":
        worst = float(err.max()) if err.numel() else 0.0
        assert worst <= FLOAT32_ABS, f"{what}: float32 logits differ by {worst:.3e} at {divmod(int(err.argmax()), ref.shape[-1])}"
        return
    if err.numel() == 0:
        return
    scale = float(ref.pow(2).mean().sqrt())
    rms = float(err.pow(2).mean().sqrt())
    worst = float(err.max())
    rows = err.reshape(-1, ref.shape[-1]).pow(2).mean(-1).sqrt()
    if rows.numel() >= 16:      # the gate over all logits is for many positions together; a few rows are held to the row gate
        assert rms <= BFLOAT16_RMS_REL * scale, f"{what}: bfloat16 rms error {rms:.3e} vs logits rms {scale:.3e}"
    assert float(rows.max()) <= BFLOAT16_ROW_RMS_REL * scale, (f"{what}: bfloat16 rms error {float(rows.max()):.3e} in row "
                                                               f"{int(rows.argmax())} vs logits rms {scale:.3e}")
    assert worst <= BFLOAT16_MAX_REL * scale, (f"{what}: bfloat16 max error {worst:.3e} vs logits rms {scale:.3e} at "
                                                f"{divmod(int(err.argmax()), ref.shape[-1])}")
    # the same first choice wherever the plain implementation's is clear: its best logit leads the second by more
    # than a row may be off (the reference's own gate between its CPU and GPU runs demands the same top-1,
    # tests/test_tiny_cpu_inference.cpp:152-172)
    ref2, got2 = ref.reshape(-1, ref.shape[-1]), got.reshape(-1, ref.shape[-1])
    top2 = ref2.topk(2, dim=-1)
    clear = (top2.values[:, 0] - top2.values[:, 1]) > BFLOAT16_ROW_RMS_REL * scale
    wrong = clear & (got2.argmax(-1) != top2.indices[:, 0])
    assert not bool(wrong.any()), (f"{what}: bfloat16 picks token {int(got2.argmax(-1)[wrong][0])} where the plain implementation "
                                   f"picks {int(top2.indices[wrong][0, 0])} by a clear margin (row {int(wrong.nonzero()[0, 0])})")


class LogitsPool:
    """Collects the rows that a test checks a few at a time (a decode step gives one row a sequence) so that the
    gate over all logits, which needs many rows, applies to them together: ``add`` holds each piece to the row
    gates at once, ``check`` holds the collection to all of them."""

    def __init__(self, dtype: str, what: str = ""):
        self.dtype, self.what, self.got, self.ref = dtype, what, [], []

    def add(self, got, ref, what: str = "") -> None:
        got = torch.as_tensor(got).double().cpu().reshape(ref.shape)
        assert_logits_close(got, ref, self.dtype, what or self.what)
        self.got.append(got.reshape(-1, ref.shape[-1]))
        self.ref.append(ref.double().reshape(-1, ref.shape[-1]))

    def check(self, least_rows: int = 16) -> None:
        got, ref = torch.cat(self.got), torch.cat(self.ref)
        assert got.shape[0] >= least_rows, f"{self.what}: only {got.shape[0]} rows were collected"
        assert_logits_close(got, ref, self.dtype, f"{self.what} (all {got.shape[0]} rows together)")

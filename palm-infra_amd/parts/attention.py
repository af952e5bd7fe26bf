"""Causal grouped-query attention over the cache, with optional per-head RMSNorm of q and k, a
rotation of both, and an optional window.

Order of operations as the reference builds it (models/qwen3.py:290-349): one joined q/k/v projection;
per-head norm of q and k over head_dim with one weight vector for all heads; rotation of q and k; the
step's k and v are appended to the cache; every query attends the cached keys of its own sequence up
to its own position with scale ``scale`` (head_dim^-0.5 for Qwen3); head h reads kv head
h // (heads / kv_heads) (kernels/attention.cpp:1161); output projection.  The reference's projections have no
bias; a specification that names tensors ``qkv_bias`` / ``out_bias`` (float32 vectors) gets them added.
"""
from __future__ import annotations

from ..cache import KVNeed
from ..kernels import ops
from .base import register_part
from .linear import Linear
from .position import PAIRINGS


@register_part("mixer", "attention")
class Attention:
    capturable = True

    def __init__(self, spec, builder):
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nh, self.nkv, self.hd = int(p["num_heads"]), int(p["num_kv_heads"]), int(p["head_dim"])
        self.scale = float(p["scale"])
        self.window = int(p["window"]) if p.get("window") else None
        if self.nh % self.nkv:
            raise ValueError(f"{self.nh} heads are not a multiple of {self.nkv} kv heads")
        bias = lambda name: builder.tensor(spec, name) if name in spec.tensors else None
        self.qkv = Linear(builder.tensor(spec, "qkv"), bias("qkv_bias"))
        self.out = Linear(builder.tensor(spec, "out"), bias("out_bias"))
        if self.qkv.weight.shape != ((self.nh + 2 * self.nkv) * self.hd, self.hidden):
            raise ValueError(f"attention: joined q/k/v weight {tuple(self.qkv.weight.shape)} does not fit "
                             f"{self.nh}+2*{self.nkv} heads of {self.hd} over hidden {self.hidden}")
        if self.out.weight.shape != (self.hidden, self.nh * self.hd):
            raise ValueError(f"attention: output weight {tuple(self.out.weight.shape)} does not fit")
        self.q_norm = builder.build(spec.parts["q_norm"]) if "q_norm" in spec.parts else None
        self.k_norm = builder.build(spec.parts["k_norm"]) if "k_norm" in spec.parts else None
        if (self.q_norm is None) != (self.k_norm is None):
            raise ValueError("attention: q_norm and k_norm come together")
        if self.q_norm is not None and (self.q_norm.width != self.hd or self.k_norm.width != self.hd
                                        or self.q_norm.eps != self.k_norm.eps):
            raise ValueError("attention: q_norm and k_norm must be over head_dim with one eps")
        self.position = builder.build(spec.parts["position"]) if "position" in spec.parts else None
        self.dtype = builder.dtype

    @staticmethod
    def cache_needs(spec):
        p = spec.params
        return [KVNeed(int(p["num_kv_heads"]), int(p["head_dim"]), int(p["window"]) if p.get("window") else None)]

    takes_sink = True

    def forward(self, h, ctx, sink=None):
        lc = ctx.layer_cache
        if lc is None or lc.kv is None:
            raise RuntimeError("attention needs the keys and values of its layer; the step gave it no cache")
        qkv = self.qkv(h, planes_ok=True)
        tables = self.position.tables(ctx) if self.position is not None else None
        cos, sin = tables if tables is not None else (None, None)
        rotary_dim = self.position.rotary_dim if tables is not None else 0
        pairing = PAIRINGS[self.position.pairing] if tables is not None else 0
        if ctx.is_decode and ops.decode_fused_serves(qkv, self.hd, self.dtype, rotary_dim, pairing):
            # one token a sequence: its slot and position are the sequence's, and the q/k/v pass rides in the
            # attention kernel
            o = ops.attention_decode_fused(
                qkv, lc.k, lc.v, lc.kv.table_dev, ctx.seq_slot, ctx.seq_start, self.nh, self.nkv, self.hd, self.scale,
                self.window, ops.slices_of_step(ctx, self.nh, self.nkv, self.window),
                q_norm_w=self.q_norm.weight if self.q_norm else None, k_norm_w=self.k_norm.weight if self.k_norm else None,
                eps=self.q_norm.eps if self.q_norm else 0.0, cos=cos, sin=sin, rotary_dim=rotary_dim, pairing=pairing,
                write_cache=lc.writes)
            return self.out(o, sink=sink)
        # a prompt's queries carry the scale (times log2 e) into their one rounding where the prompt kernel of this
        # head size takes them so: a score then leaves the matrix cores as the exponent of its weight
        q_scale = 1.0 if ctx.is_decode else ops.prefill_q_scale(self.hd, self.dtype, self.scale)
        q = ops.qk_norm_rope_store(
            qkv, self.nh, self.nkv, self.hd, ctx.positions,
            q_norm_w=self.q_norm.weight if self.q_norm else None, k_norm_w=self.k_norm.weight if self.k_norm else None,
            eps=self.q_norm.eps if self.q_norm else 0.0, cos=cos, sin=sin,
            rotary_dim=rotary_dim, pairing=pairing,
            k_cache=lc.k, v_cache=lc.v, block_table=lc.kv.table_dev, tok_slot=ctx.tok_slot, write_cache=lc.writes,
            out_dtype=self.dtype, q_scale=q_scale)
        o = ops.attention(q, lc.k, lc.v, lc.kv.table_dev, ctx, self.nh, self.nkv, self.hd, self.scale, self.window,
                          q_prescaled=q_scale != 1.0)
        return self.out(o, sink=sink)

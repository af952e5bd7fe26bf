"""The typed configuration of the dense Qwen3 decoder and its description as parts.

Keys and defaults follow the reference's reader (models/qwen3.py:175-184): ``hidden_size``,
``num_hidden_layers``, ``rms_norm_eps`` (1e-6), ``rope_theta`` (1e6), ``num_attention_heads``,
``num_key_value_heads`` (= heads), ``head_dim`` (= hidden/heads), ``intermediate_size``,
``vocab_size``.  Keys that the reference does not read but that would change the computation if set
(attention bias, a sliding window, scaled rotation, another activation) are checked and refused.
"""
from __future__ import annotations

from dataclasses import dataclass, asdict

from .registry import ConfigError, register_architecture
from .spec import LayerCall, ModelSpec, PartSpec, joined, tensor

_NORM_INIT = ("normal", 1.0, 0.02)


def _need(raw: dict, key: str, typ=int):
    if key not in raw or raw[key] is None:
        raise ConfigError(f"config.json: required key {key!r} is missing")
    try:
        return typ(raw[key])
    except (TypeError, ValueError):
        raise ConfigError(f"config.json: {key!r} = {raw[key]!r} is not {typ.__name__}") from None


@register_architecture("Qwen3ForCausalLM", model_type="qwen3")
@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1000000.0
    max_position_embeddings: int = 32768
    # None: the checkpoint decides (a stored lm_head.weight means untied), as the reference does
    # (models/qwen3.py:89-95, 162-165)
    tie_word_embeddings: bool | None = None
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen3Config":
        nh = _need(raw, "num_attention_heads")
        hidden = _need(raw, "hidden_size")
        nkv = int(raw["num_key_value_heads"]) if raw.get("num_key_value_heads") is not None else nh
        hd = int(raw["head_dim"]) if raw.get("head_dim") is not None else hidden // max(nh, 1)
        eos = raw.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        tie = raw.get("tie_word_embeddings")
        # newer checkpoints keep the rotation's base in a ``rope_parameters`` table; the top-level key, which the
        # reference reads (models/qwen3.py:179), comes first
        nested = raw.get("rope_parameters") if isinstance(raw.get("rope_parameters"), dict) else {}
        theta = raw.get("rope_theta", nested.get("rope_theta", 1000000.0))
        cfg = cls(
            vocab_size=_need(raw, "vocab_size"), hidden_size=hidden,
            num_hidden_layers=_need(raw, "num_hidden_layers"), num_attention_heads=nh,
            num_key_value_heads=nkv, head_dim=hd, intermediate_size=_need(raw, "intermediate_size"),
            rms_norm_eps=float(raw.get("rms_norm_eps", 1e-6)), rope_theta=float(theta),
            max_position_embeddings=int(raw.get("max_position_embeddings", 32768)),
            tie_word_embeddings=None if tie is None else bool(tie), eos_token_ids=eos_ids,
        )
        cfg.validate()
        # what the reference never reads but a checkpoint may set
        if raw.get("attention_bias"):
            raise ConfigError("config.json: attention_bias=true is not supported (Qwen3 projections have no bias)")
        if raw.get("use_sliding_window") and raw.get("sliding_window"):
            raise ConfigError("config.json: a sliding window is not part of this architecture "
                              f"(use_sliding_window=true, sliding_window={raw['sliding_window']})")
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError(f"config.json: rope_scaling={raw['rope_scaling']!r} is not supported (plain rotation only)")
        if nested.get("rope_type", nested.get("type", "default")) not in (None, "default"):
            raise ConfigError(f"config.json: rope_parameters={nested!r} is not supported (plain rotation only)")
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"config.json: hidden_act={raw['hidden_act']!r}; the feed-forward of this architecture uses silu")
        return cfg

    def validate(self) -> None:
        for key in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                    "num_key_value_heads", "head_dim", "intermediate_size", "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"config.json: {key} = {getattr(self, key)} must be positive")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            # models/qwen3.py:186-190
            raise ConfigError("config.json: num_attention_heads must be divisible by num_key_value_heads: "
                              f"{self.num_attention_heads} vs {self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim = {self.head_dim} must be even (rotation works on pairs)")
        if not self.rms_norm_eps > 0.0:
            raise ConfigError(f"config.json: rms_norm_eps = {self.rms_norm_eps} must be positive")
        if not self.rope_theta > 0.0:
            raise ConfigError(f"config.json: rope_theta = {self.rope_theta} must be positive")

    def to_dict(self) -> dict:
        d = asdict(self)
        eos = d.pop("eos_token_ids")
        if d["tie_word_embeddings"] is None:
            d.pop("tie_word_embeddings")
        if eos:
            d["eos_token_id"] = eos[0] if len(eos) == 1 else list(eos)
        d["architectures"] = [self.architecture]
        d["model_type"] = self.model_type
        d["hidden_act"] = "silu"
        d["attention_bias"] = False
        return d

    # ------------------------------------------------------------------------------------------
    def spec(self, tensor_names=None) -> ModelSpec:
        """The model as parts.  ``tensor_names`` (the names a checkpoint holds) settles the head as the reference
        does (models/qwen3.py:89-95, 162-165): ``lm_head.weight`` if the checkpoint has it, else the embedding,
        whatever ``tie_word_embeddings`` says (the reference never reads that key).  Without a checkpoint
        (random weights) the key decides."""
        H, nh, nkv, hd, I, V = (self.hidden_size, self.num_attention_heads, self.num_key_value_heads,
                                self.head_dim, self.intermediate_size, self.vocab_size)
        eps = self.rms_norm_eps
        if tensor_names is not None:
            tied = "lm_head.weight" not in tensor_names
        else:
            tied = bool(self.tie_word_embeddings)

        def norm(name: str, width: int) -> PartSpec:
            return PartSpec("norm", "rms", {"width": width, "eps": eps},
                            {"weight": tensor(name, (width,), "vector", _NORM_INIT)})

        layers = []
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}."
            a = p + "self_attn."
            mixer = PartSpec(
                "mixer", "attention",
                {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": hd,
                 "scale": hd ** -0.5, "window": None},
                {"qkv": joined((a + "q_proj.weight", a + "k_proj.weight", a + "v_proj.weight"),
                               ((nh * hd, H), (nkv * hd, H), (nkv * hd, H))),
                 "out": tensor(a + "o_proj.weight", (H, nh * hd))},
                {"q_norm": norm(a + "q_norm.weight", hd), "k_norm": norm(a + "k_norm.weight", hd),
                 "position": PartSpec("position", "rotary", {"rotary_dim": hd, "theta": self.rope_theta,
                                                             "pairing": "half_split"})},
            )
            ff = PartSpec(
                "feed_forward", "gated_silu", {"hidden_size": H, "intermediate_size": I},
                {"gate_up": joined((p + "mlp.gate_proj.weight", p + "mlp.up_proj.weight"), ((I, H), (I, H))),
                 "down": tensor(p + "mlp.down_proj.weight", (H, I))},
            )
            layers.append(PartSpec(
                "block", "pre_norm", {"hidden_size": H}, {},
                {"mixer_norm": norm(p + "input_layernorm.weight", H), "mixer": mixer,
                 "feed_forward_norm": norm(p + "post_attention_layernorm.weight", H), "feed_forward": ff},
            ))

        embed_ref = tensor("model.embed_tokens.weight", (V, H), "table")
        head_ref = embed_ref if tied else tensor("lm_head.weight", (V, H), "matrix")
        return ModelSpec(
            architecture=self.architecture, vocab_size=V, hidden_size=H,
            # the reference never reads max_position_embeddings (models/qwen3.py:175-184): its limit is the cache's
            # rows (engine/engine.cpp:969-976), and rotation angles are computed, not looked up
            max_positions=None,
            embedding=PartSpec("embedding", "token_table", {"vocab_size": V, "hidden_size": H}, {"table": embed_ref}),
            layers=tuple(layers),
            order=tuple(LayerCall(i) for i in range(self.num_hidden_layers)),
            final_norm=norm("model.norm.weight", H),
            head=PartSpec("head", "linear", {"vocab_size": V, "hidden_size": H}, {"weight": head_ref}),
            stop_token_ids=self.eos_token_ids,
        )

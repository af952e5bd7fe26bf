"""A whole architecture defined here, outside the framework: its configuration class (its own config.json keys and
its own tensor names), registered by name, describes a model made of shipped and toy parts with a run order that
names a layer twice; a folder is written for it with the random-weights mode, loaded through the public entry
point (which picks the class by config.json, as for any model), stepped under several schedules and generated
from, against a plain computation written here.  No file of the framework changes.  (A toy, not a model of
anyone's: sizes and rules are made up for the test.)"""
import dataclasses
import json

import pytest
import torch

import plain_qwen3 as P
import test_toy_parts as toy
import tiny

pytestmark = pytest.mark.gpu
NAME = "ToyMixedForCausalLM"


def register():
    from palm_infra_amd.config import (LayerCall, ModelSpec, PartSpec, Stored, joined, register_architecture,
                                       registered_architectures, tensor)
    toy.register_toy_mixer()
    if NAME in registered_architectures():
        return

    @register_architecture(NAME, model_type="toy_mixed")
    @dataclasses.dataclass(frozen=True)
    class ToyMixedConfig:
        vocab: int
        width: int
        blocks: tuple            # of dicts: {"mixer": "attention", "heads", "kv_heads", "head_size", "rotary", "ff"} or {"mixer": "decay", "state", "decay", "ff"}
        order: tuple             # the run order: indices into blocks, repeats allowed
        eps: float
        theta: float
        tied: bool
        stop: tuple = ()

        @classmethod
        def from_dict(cls, raw):
            return cls(vocab=int(raw["vocab"]), width=int(raw["width"]), blocks=tuple(dict(b) for b in raw["blocks"]),
                       order=tuple(int(i) for i in raw["order"]), eps=float(raw.get("eps", 1e-5)), theta=float(raw.get("theta", 1e4)),
                       tied=bool(raw.get("tied", False)), stop=tuple(raw.get("stop", ())))

        def to_dict(self):
            return {"architectures": [NAME], "model_type": "toy_mixed", "vocab": self.vocab, "width": self.width,
                    "blocks": [dict(b) for b in self.blocks], "order": list(self.order), "eps": self.eps, "theta": self.theta,
                    "tied": self.tied, "stop": list(self.stop)}

        def spec(self, tensor_names=None):
            H = self.width
            unit = ("normal", 1.0, 0.05)

            def norm(name, width):
                return PartSpec("norm", "rms", {"width": width, "eps": self.eps}, {"weight": tensor(name, (width,), "vector", unit)})
            layers = []
            for i, b in enumerate(self.blocks):
                p = f"blocks.{i}."
                if b["mixer"] == "attention":
                    nh, nkv, hd = b["heads"], b["kv_heads"], b["head_size"]
                    mixer = PartSpec("mixer", "attention",
                                     {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": hd, "scale": hd ** -0.5, "window": None},
                                     # the checkpoint keeps v, k and q fused in one tensor, in that order, and the output
                                     # matrix as [in, out]: the description says so, the loader needs no change
                                     {"qkv": joined((p + "attn.wvkq",) * 3, ((nh * hd, H), (nkv * hd, H), (nkv * hd, H)), init=("normal", 0.0, 0.1),
                                                    stored=(Stored(((nh + 2 * nkv) * hd, H), rows=(2 * nkv * hd, (nh + 2 * nkv) * hd)),
                                                            Stored(((nh + 2 * nkv) * hd, H), rows=(nkv * hd, 2 * nkv * hd)),
                                                            Stored(((nh + 2 * nkv) * hd, H), rows=(0, nkv * hd)))),
                                      "out": tensor(p + "attn.wo_t", (H, nh * hd), init=("normal", 0.0, 0.1),
                                                    stored=Stored((nh * hd, H), transposed=True))},
                                     {"position": PartSpec("position", "rotary", {"rotary_dim": b["rotary"], "theta": self.theta,
                                                                                  "pairing": "interleaved"})})      # no q/k norm here
                else:
                    mixer = PartSpec("mixer", "toy_decay", {"decay": b["decay"], "state_size": b["state"]},
                                     {"w_in": tensor(p + "mix.w_in", (b["state"], H), init=("normal", 0.0, 0.2)),
                                      "w_out": tensor(p + "mix.w_out", (H, b["state"]), init=("normal", 0.0, 0.2))})
                ff = PartSpec("feed_forward", "gated_silu", {"hidden_size": H, "intermediate_size": b["ff"]},
                              {"gate_up": tensor(p + "ff.w13", (2 * b["ff"], H), init=("normal", 0.0, 0.1)),      # stored joined already
                               "down": tensor(p + "ff.w2", (H, b["ff"]), init=("normal", 0.0, 0.1))})
                layers.append(PartSpec("block", "pre_norm", {"hidden_size": H}, {},
                                       {"mixer_norm": norm(p + "n1.weight", H), "mixer": mixer,
                                        "feed_forward_norm": norm(p + "n2.weight", H), "feed_forward": ff}))
            table = tensor("tok.weight", (self.vocab, H), "table", init=("normal", 0.0, 1.0))
            head = table if self.tied else tensor("unembed.weight", (self.vocab, H), init=("normal", 0.0, 0.1))
            return ModelSpec(architecture=NAME, vocab_size=self.vocab, hidden_size=H, max_positions=None,
                             embedding=PartSpec("embedding", "token_table", {"vocab_size": self.vocab, "hidden_size": H}, {"table": table}),
                             layers=tuple(layers), order=tuple(LayerCall(i) for i in self.order), final_norm=norm("out_norm.weight", H),
                             head=PartSpec("head", "linear", {"vocab_size": self.vocab, "hidden_size": H}, {"weight": head}),
                             stop_token_ids=self.stop)


RAW = {"architectures": [NAME], "vocab": 300, "width": 64,
       "blocks": [{"mixer": "attention", "heads": 4, "kv_heads": 2, "head_size": 32, "rotary": 16, "ff": 96},
                  {"mixer": "decay", "state": 24, "decay": 0.7, "ff": 80}],
       "order": [0, 1, 0], "eps": 2e-5, "theta": 5000.0, "tied": False, "stop": [7]}


def plain_logits(raw, w, ids):
    """The toy architecture by its own rules, whole sequence, float64."""
    n, H, eps = len(ids), raw["width"], raw["eps"]
    x = P.embedding(w["tok.weight"], ids)
    for i in raw["order"]:
        b, p = raw["blocks"][i], f"blocks.{i}."
        h = P.rms_norm(x, w[p + "n1.weight"], eps)
        if b["mixer"] == "attention":
            nh, nkv, hd, rot = b["heads"], b["kv_heads"], b["head_size"], b["rotary"]
            vkq = w[p + "attn.wvkq"]                     # rows: v heads, then k heads, then q heads
            v = P.linear(h, vkq[:nkv * hd]).reshape(n, nkv, hd)
            k = P.linear(h, vkq[nkv * hd:2 * nkv * hd]).reshape(n, nkv, hd)
            q = P.linear(h, vkq[2 * nkv * hd:]).reshape(n, nh, hd)
            cos, sin = P.rope_table(list(range(n)), rot, raw["theta"])
            q, k = toy._rope_interleaved(q, cos, sin, rot), toy._rope_interleaved(k, cos, sin, rot)
            x = x + P.causal_attention(q, k, v, hd ** -0.5).reshape(n, nh * hd) @ w[p + "attn.wo_t"].double()     # stored [in, out]
        else:
            u = h @ w[p + "mix.w_in"].double().T
            s, mixed = torch.zeros(b["state"], dtype=torch.float64), []
            for t in range(n):
                s = b["decay"] * s + u[t]
                mixed.append(s)
            x = x + torch.stack(mixed) @ w[p + "mix.w_out"].double().T
        h = P.rms_norm(x, w[p + "n2.weight"], eps)
        I = b["ff"]
        x = x + P.swiglu_mlp(h, w[p + "ff.w13"][:I], w[p + "ff.w13"][I:], w[p + "ff.w2"])
    return P.linear(P.rms_norm(x, w["out_norm.weight"], eps), w["unembed.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_an_architecture_registered_from_outside_loads_steps_and_generates(tmp_path, dtype):
    import palm_infra_amd
    from palm_infra_amd.config import ConfigError, config_from_dir, registered_architectures
    from palm_infra_amd.engine import StepEntry
    from palm_infra_amd.sampling import GREEDY
    from palm_infra_amd.weights import WeightError, write_random_model
    register()
    assert NAME in registered_architectures()
    folder = write_random_model(RAW, 9, tmp_path / "toy", dtype)             # the random-weights mode knows no architecture either
    assert json.loads((folder / "config.json").read_text())["blocks"][1]["mixer"] == "decay"
    assert type(config_from_dir(folder)).__name__ == "ToyMixedConfig"
    engine = palm_infra_amd.load(folder, dtype=dtype, max_tokens=64 * 8)
    # three runs of two layers: two key/value stores for the layer that runs twice, one state for the toy mixer
    kinds = sorted((type(g.need).__name__, g.n_entries) for g in engine.cache.groups)
    assert kinds == [("KVNeed", 2), ("StateNeed", 1)]
    assert not engine.model.capturable                                          # the toy mixer plans on the host
    raw, w = P.read_model(folder)
    reqs = [torch.randint(0, raw["vocab"], (n,), generator=torch.Generator().manual_seed(60 + n)).tolist() for n in (70, 9, 33)]
    refs = [plain_logits(raw, w, r) for r in reqs]
    slots = [engine.open() for _ in reqs]
    cuts = [50, 9, 1]
    out = engine.step([StepEntry(s, r[:c], list(range(c))) for s, r, c in zip(slots, reqs, cuts)])
    got, o = {i: [] for i in range(3)}, 0
    for i, c in enumerate(cuts):
        got[i].append(out[o:o + c]); o += c
    fed = list(cuts)
    while any(fed[i] < len(reqs[i]) for i in range(3)):
        live = [i for i in range(3) if fed[i] < len(reqs[i])]
        out = engine.step([StepEntry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
        for r_, i in enumerate(live):
            got[i].append(out[r_:r_ + 1]); fed[i] += 1
    for i in range(3):
        tiny.assert_logits_close(torch.cat(got[i]), refs[i], dtype, f"toy architecture, request {i}")
        engine.close(slots[i])
    engine.cache.check()
    # generation through the public entry point, stop token from the architecture's own config key
    if dtype == "float32":
        results, _ = engine.generate([reqs[1], reqs[2][:5]], GREEDY, max_new_tokens=6, ignore_eos=True)
        for r, prompt in zip(results, (reqs[1], reqs[2][:5])):
            ids = list(prompt)
            for tok in r.token_ids:
                assert tok == int(torch.argmax(plain_logits(raw, w, ids)[-1]))
                ids.append(tok)
        assert engine.spec.stop_token_ids == (7,)
    # its checkpoint errors are the loader's: a missing and an unexpected tensor named together
    from palm_infra_amd.weights import ModelFiles, load_weights, write_safetensors
    broken = {k: v for k, v in w.items() if k != "blocks.1.mix.w_in"}
    broken["surplus"] = torch.zeros(3)
    (tmp_path / "broken").mkdir()
    (tmp_path / "broken" / "config.json").write_text((folder / "config.json").read_text())
    write_safetensors(tmp_path / "broken" / "model.safetensors", {k: v.float() for k, v in broken.items()})
    with pytest.raises(WeightError) as err:
        palm_infra_amd.load(tmp_path / "broken", dtype=dtype, max_tokens=128)
    assert err.value.missing == ["blocks.1.mix.w_in"] and err.value.unexpected == ["surplus"]
    with pytest.raises(ConfigError, match="unknown architecture"):
        from palm_infra_amd.config import config_from_dict
        config_from_dict({"architectures": ["NoSuchForCausalLM"]})

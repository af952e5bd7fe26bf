"""Safetensors files, the loader's errors and the random-weights mode (no GPU)."""
import json
import struct

import pytest
import torch

import plain_qwen3 as P
import tiny
from palm_infra_amd.config import config_from_dict, config_from_dir
from palm_infra_amd.weights import (ModelFiles, SafetensorsError, SafetensorsFile, WeightError, load_weights,
                                    random_tensors, write_random_model, write_safetensors)


def host_copy(stored, part, transposed=False):
    """Stands in for the device's conversion kernel where only the binding is tested (no GPU here)."""
    part.copy_(stored.t() if transposed else stored)


def test_round_trip_is_bit_exact(tmp_path):
    g = torch.Generator().manual_seed(0)
    tensors = {"a": torch.randn(3, 5, generator=g), "b": torch.randn(7, generator=g).to(torch.bfloat16),
               "c": torch.randn(2, 2, generator=g).to(torch.float16), "d": torch.arange(6, dtype=torch.int32).reshape(2, 3)}
    write_safetensors(tmp_path / "m.safetensors", tensors)
    f = SafetensorsFile(tmp_path / "m.safetensors")
    for k, t in tensors.items():
        got = f.tensor(k)
        assert got.dtype == t.dtype and got.shape == t.shape
        assert torch.equal(got.view(torch.uint8) if t.dtype != torch.int32 else got, t.view(torch.uint8) if t.dtype != torch.int32 else t)
    # and the oracle's own reader agrees
    write_safetensors(tmp_path / "f.safetensors", {k: t for k, t in tensors.items() if t.is_floating_point()})
    mine = P.read_safetensors(tmp_path / "f.safetensors")
    assert torch.equal(mine["b"], tensors["b"].double())


def _raw_file(path, header: dict, payload: bytes, hlen=None):
    raw = json.dumps(header).encode()
    path.write_bytes(struct.pack("<Q", len(raw) if hlen is None else hlen) + raw + payload)


def test_bad_files_are_refused(tmp_path):
    # the checks of models/safetensors_stream.py:71-118
    p = tmp_path / "x.safetensors"
    _raw_file(p, {"t": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 12]}}, b"\0" * 12)
    with pytest.raises(SafetensorsError, match="needs 16"):
        SafetensorsFile(p)
    _raw_file(p, {"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 4)
    with pytest.raises(SafetensorsError, match="outside the file"):
        SafetensorsFile(p)
    _raw_file(p, {"t": {"dtype": "F8_E4M3", "shape": [2], "data_offsets": [0, 2]}}, b"\0" * 2)
    with pytest.raises(SafetensorsError, match="not supported"):
        SafetensorsFile(p)
    _raw_file(p, {}, b"", hlen=1 << 40)
    with pytest.raises(SafetensorsError, match="exceeds"):
        SafetensorsFile(p)
    _raw_file(p, {}, b"", hlen=500)
    with pytest.raises(SafetensorsError, match="cut off"):
        SafetensorsFile(p)
    with pytest.raises(FileNotFoundError, match="No safetensors"):
        ModelFiles(tmp_path / "nowhere")


def test_one_error_lists_missing_unexpected_and_misshapen(tmp_path):
    tensors = tiny.sharpened_tensors("A", "float32")
    del tensors["model.layers.1.self_attn.k_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.mlp.down_proj.weight"] = torch.zeros(64, 100)
    tensors["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(32)
    tensors["model.layers.7.mlp.up_proj.weight"] = torch.zeros(2, 2)
    tensors["rotary.inv_freq"] = torch.zeros(8)
    (tmp_path / "config.json").write_text(json.dumps(tiny.CONFIGS["A"]))
    write_safetensors(tmp_path / "model.safetensors", tensors)
    cfg = config_from_dir(tmp_path)
    files = ModelFiles(tmp_path)
    with pytest.raises(WeightError) as e:
        load_weights(cfg.spec(files.names()), files, torch.float32, "cpu", place=host_copy)
    err = e.value
    assert sorted(err.missing) == ["model.layers.1.self_attn.k_proj.weight", "model.norm.weight"]
    assert sorted(err.unexpected) == ["model.layers.7.mlp.up_proj.weight", "rotary.inv_freq"]
    assert sorted(n for n, _, _ in err.wrong_shape) == ["model.layers.0.mlp.down_proj.weight", "model.layers.0.self_attn.q_norm.weight"]
    text = str(err)
    for word in ("missing", "unexpected", "wrong shapes", "k_proj", "inv_freq", "expected [64, 128], file has [64, 100]"):
        assert word in text, word


def test_tensors_the_model_does_not_name_are_a_warning_list_when_asked(tmp_path):
    """The reference's converter passes over names it does not know (models/qwen3.py:105-106).  Here they are an
    error by default; with strict=False they come back as a list and the model loads; what is missing or
    misshapen stays an error either way."""
    tensors = tiny.sharpened_tensors("A", "float32")
    tensors["rotary.inv_freq"] = torch.zeros(8)
    tensors["model.layers.7.mlp.up_proj.weight"] = torch.zeros(2, 2)
    (tmp_path / "config.json").write_text(json.dumps(tiny.CONFIGS["A"]))
    write_safetensors(tmp_path / "model.safetensors", tensors)
    files = ModelFiles(tmp_path)
    spec = config_from_dir(tmp_path).spec(files.names())
    with pytest.raises(WeightError) as e:
        load_weights(spec, files, torch.float32, "cpu", place=host_copy)
    assert sorted(e.value.unexpected) == ["model.layers.7.mlp.up_proj.weight", "rotary.inv_freq"] and not e.value.missing
    told = []
    w = load_weights(spec, files, torch.float32, "cpu", place=host_copy, strict=False, warn=told.extend)
    assert sorted(told) == ["model.layers.7.mlp.up_proj.weight", "rotary.inv_freq"]
    assert torch.equal(w.get(spec.final_norm.tensors["weight"]), tensors["model.norm.weight"])
    del tensors["model.norm.weight"]
    write_safetensors(tmp_path / "model.safetensors", tensors)
    files = ModelFiles(tmp_path)
    with pytest.raises(WeightError) as e:
        load_weights(spec, files, torch.float32, "cpu", place=host_copy, strict=False, warn=told.extend)
    assert e.value.missing == ["model.norm.weight"]


def test_a_parameter_may_be_rows_of_a_stored_tensor_or_its_transpose(tmp_path):
    """A checkpoint that stores q, k and v fused in one tensor (here in the order v, k, q) and a matrix as [in, out]
    is a matter of the model's description, not of the loader: pieces say which rows of which stored tensor they
    are, and whether what is stored is their transpose."""
    from palm_infra_amd.config import Stored, joined, tensor
    from palm_infra_amd.config.spec import LayerCall, ModelSpec, PartSpec
    g = torch.Generator().manual_seed(3)
    fused, w_io = torch.randn(4 + 4 + 8, 6, generator=g), torch.randn(6, 10, generator=g)
    qkv = joined(("att.fused",) * 3, ((8, 6), (4, 6), (4, 6)),
                 stored=(Stored((16, 6), rows=(8, 16)), Stored((16, 6), rows=(4, 8)), Stored((16, 6), rows=(0, 4))))
    out = tensor("att.out_io", (10, 6), stored=Stored((6, 10), transposed=True))
    assert qkv.shape == (16, 6) and out.shape == (10, 6) and qkv.key != joined(("att.fused",) * 3, ((8, 6), (4, 6), (4, 6))).key
    with pytest.raises(ValueError, match="expects"):
        tensor("x", (5, 6), stored=Stored((6, 10), transposed=True))
    with pytest.raises(ValueError, match="rows"):
        tensor("x", (5, 6), stored=Stored((4, 6), rows=(0, 5)))
    part = PartSpec("mixer", "anything", {}, {"qkv": qkv, "out": out})
    norm = PartSpec("norm", "rms", {}, {"weight": tensor("n", (6,), "vector")})
    spec = ModelSpec("T", 3, 6, None, PartSpec("embedding", "token_table", {}, {"table": tensor("emb", (3, 6), "table")}),
                     (part,), (LayerCall(0),), norm, PartSpec("head", "linear", {}, {"weight": tensor("emb", (3, 6), "table")}))
    assert spec.expected_tensors()["att.fused"] == ((16, 6), "matrix") and spec.expected_tensors()["att.out_io"] == ((6, 10), "matrix")
    write_safetensors(tmp_path / "model.safetensors", {"att.fused": fused, "att.out_io": w_io, "n": torch.ones(6), "emb": torch.zeros(3, 6)})
    w = load_weights(spec, ModelFiles(tmp_path), torch.float32, "cpu", place=host_copy)
    assert torch.equal(w.get(qkv), torch.cat([fused[8:16], fused[4:8], fused[0:4]]))
    assert torch.equal(w.get(out), w_io.t())
    # the random-weights mode writes the tensors as the checkpoint stores them, each once
    from palm_infra_amd.weights import random_tensors
    made = random_tensors(spec, 1, "float32")
    assert made["att.fused"].shape == (16, 6) and made["att.out_io"].shape == (6, 10) and set(made) == {"att.fused", "att.out_io", "n", "emb"}
    # a wrong stored shape is named like any other
    write_safetensors(tmp_path / "model.safetensors", {"att.fused": fused[:12], "att.out_io": w_io, "n": torch.ones(6), "emb": torch.zeros(3, 6)})
    with pytest.raises(WeightError) as e:
        load_weights(spec, ModelFiles(tmp_path), torch.float32, "cpu", place=host_copy)
    assert [n for n, _, _ in e.value.wrong_shape] == ["att.fused"]


def test_a_stored_head_is_used_whatever_the_config_says(tmp_path):
    """models/qwen3.py:89-95, 162-165: lm_head.weight if the checkpoint has it, else the embedding; the reference
    never reads tie_word_embeddings."""
    tensors = tiny.sharpened_tensors("A", "float32")
    tensors["lm_head.weight"] = torch.full((256, 64), 0.5)
    (tmp_path / "config.json").write_text(json.dumps(tiny.CONFIGS["A"]))      # tie_word_embeddings: true
    write_safetensors(tmp_path / "model.safetensors", tensors)
    files = ModelFiles(tmp_path)
    spec = config_from_dir(tmp_path).spec(files.names())
    w = load_weights(spec, files, torch.float32, "cpu", place=host_copy)
    assert torch.equal(w.get(spec.head.tensors["weight"]), tensors["lm_head.weight"])
    # and the other way round: the key says untied, the checkpoint has no head of its own
    d = tmp_path / "b"
    d.mkdir()
    tensors = {k: v for k, v in tiny.sharpened_tensors("B", "float32").items() if k != "lm_head.weight"}
    (d / "config.json").write_text(json.dumps(tiny.CONFIGS["B"]))             # tie_word_embeddings: false
    write_safetensors(d / "model.safetensors", tensors)
    files = ModelFiles(d)
    spec = config_from_dir(d).spec(files.names())
    w = load_weights(spec, files, torch.float32, "cpu", place=host_copy)
    assert w.get(spec.head.tensors["weight"]).data_ptr() == w.get(spec.embedding.tensors["table"]).data_ptr()


def test_what_is_kept_in_which_precision(tmp_path):
    cfg = config_from_dict(tiny.CONFIGS["B"])
    d = tiny.write_model("B", tmp_path / "bf", "bfloat16")
    files = ModelFiles(d)
    spec = cfg.spec(files.names())
    w = load_weights(spec, files, torch.bfloat16, "cpu", place=host_copy)
    mixer = spec.layers[0].parts["mixer"]
    assert w.get(mixer.tensors["qkv"]).dtype == torch.bfloat16
    assert w.get(mixer.tensors["qkv"]).shape == (8 * 32 + 2 * 32, 96)
    assert w.get(mixer.parts["q_norm"].tensors["weight"]).dtype == torch.float32      # vectors are widened
    assert w.get(spec.embedding.tensors["table"]).dtype == torch.bfloat16
    w32 = load_weights(spec, files, torch.float32, "cpu", place=host_copy)
    assert w32.get(mixer.tensors["qkv"]).dtype == torch.float32
    # a tensor stored in 32-bit stays so in the bfloat16 mode
    d32 = tiny.write_model("B", tmp_path / "f32", "float32")
    f32 = ModelFiles(d32)
    wmix = load_weights(spec, f32, torch.bfloat16, "cpu", place=host_copy)
    assert wmix.get(mixer.tensors["qkv"]).dtype == torch.float32
    # the joined matrix is q rows, k rows, v rows
    q = f32.tensor("model.layers.0.self_attn.q_proj.weight")
    v = f32.tensor("model.layers.0.self_attn.v_proj.weight")
    joined = wmix.get(mixer.tensors["qkv"])
    assert torch.equal(joined[:256], q) and torch.equal(joined[-32:], v)


def test_tied_head_is_the_embedding_itself(tmp_path):
    d = tiny.write_model("A", tmp_path / "a", "float32")
    files = ModelFiles(d)
    spec = config_from_dir(d).spec(files.names())
    w = load_weights(spec, files, torch.float32, "cpu", place=host_copy)
    assert w.get(spec.head.tensors["weight"]).data_ptr() == w.get(spec.embedding.tensors["table"]).data_ptr()


def test_sharded_checkpoint_with_index(tmp_path):
    tensors = tiny.sharpened_tensors("A", "float32")
    names = list(tensors)
    half = len(names) // 2
    write_safetensors(tmp_path / "model-00001-of-00002.safetensors", {n: tensors[n] for n in names[:half]})
    write_safetensors(tmp_path / "model-00002-of-00002.safetensors", {n: tensors[n] for n in names[half:]})
    index = {"weight_map": {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
                            for i, n in enumerate(names)}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    files = ModelFiles(tmp_path)
    assert sorted(files.names()) == sorted(names)
    assert torch.equal(files.tensor(names[-1]), tensors[names[-1]])
    (tmp_path / "model.safetensors.index.json").unlink()       # the glob patterns of models/qwen3.py:39-54
    assert sorted(ModelFiles(tmp_path).names()) == sorted(names)


def test_random_weights_mode_writes_a_loadable_folder(tmp_path):
    cfg = config_from_dict(tiny.CONFIGS["B"])
    d1 = write_random_model(cfg, 5, tmp_path / "one")
    d2 = write_random_model(tiny.CONFIGS["B"], 5, tmp_path / "two")
    d3 = write_random_model(cfg, 6, tmp_path / "three")
    assert (d1 / "config.json").is_file() and (d1 / "model.safetensors").is_file()
    assert config_from_dir(d1) == cfg
    a, b, c = (ModelFiles(d) for d in (d1, d2, d3))
    n = "model.layers.2.mlp.up_proj.weight"
    assert a.dtype_name(n) == "BF16"
    assert torch.equal(a.tensor(n).float(), b.tensor(n).float())            # the seed decides
    assert not torch.equal(a.tensor(n).float(), c.tensor(n).float())
    load_weights(cfg.spec(a.names()), a, torch.bfloat16, "cpu", place=host_copy)
    t = random_tensors(cfg.spec(), 5, "float32")
    assert abs(float(t[n].std()) - 0.02) < 2e-3 and abs(float(t["model.norm.weight"].mean()) - 1.0) < 2e-2
    # a tensor depends on the seed and its name only: a model with fewer layers starts the same
    small = config_from_dict(dict(tiny.CONFIGS["B"], num_hidden_layers=1))
    assert torch.equal(random_tensors(small.spec(), 5, "float32")["model.layers.0.mlp.up_proj.weight"],
                       t["model.layers.0.mlp.up_proj.weight"])


def test_random_numbers_are_a_function_of_seed_name_and_index():
    from palm_infra_amd.weights import random_numbers as R
    key = R.tensor_key(5, "model.layers.1.mlp.up_proj.weight")
    assert key == R.tensor_key(5, "model.layers.1.mlp.up_proj.weight") and 0 <= key < 1 << 64
    assert len({R.tensor_key(s, n) for s in (0, 1, 5) for n in ("a", "b", "model.layers.1.mlp.up_proj.weight")}) == 9
    z = R.standard_normal(key, 0, 400_000)
    # cutting the stream anywhere gives the same elements
    assert (R.standard_normal(key, 1234, 1000) == z[1234:2234]).all()
    assert (R.normal(key, 5000, 0.0, 1.0, chunk=777) == z[:5000]).all()
    # standard normal: moments, tails, no correlation between neighbours or with another key's stream
    import numpy as np
    assert abs(float(z.mean())) < 6e-3 and abs(float(z.std()) - 1) < 5e-3
    assert abs(float((z ** 4).mean()) - 3) < 0.1 and abs(float((np.abs(z) > 2).mean()) - 0.0455) < 2e-3
    assert abs(float(np.corrcoef(z[:-1], z[1:])[0, 1])) < 6e-3
    other = R.standard_normal(R.tensor_key(5, "model.layers.2.mlp.up_proj.weight"), 0, 400_000)
    assert abs(float(np.corrcoef(z, other)[0, 1])) < 6e-3
    assert np.isfinite(z).all() and float(np.abs(z).max()) < 6.0

"""Each part alone: built from its description and a few tensors, stepped with a hand-made context,
compared with the plain function of the same part."""
import pytest
import torch

import plain_qwen3 as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16


class Tensors:
    """Stands in for loaded weights: TensorRef -> tensor."""

    def __init__(self):
        self.by_names = {}

    def add(self, ref, t):
        self.by_names[ref.names] = t.to(DEV)
        return ref

    def get(self, ref):
        return self.by_names[ref.names]


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def build(spec, tensors, dtype):
    from palm_infra_amd.parts import Builder
    return Builder(tensors, dtype, DEV).build(spec)


def tol(dtype):
    return 3e-5 if dtype == F32 else 5e-2


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_norm_part(dtype):
    from palm_infra_amd.config import PartSpec, tensor
    T = Tensors()
    w = rand(80, seed=1) + 1
    spec = PartSpec("norm", "rms", {"width": 80, "eps": 3e-6}, {"weight": T.add(tensor("n.weight", (80,), "vector"), w)})
    norm = build(spec, T, dtype)
    x, d = rand(6, 80, seed=2), rand(6, 80, seed=3).to(dtype)
    xd = x.to(DEV)
    y = norm(xd, delta=d.to(DEV), update=True)
    assert y.dtype == dtype and torch.equal(xd.cpu(), x + d.float())
    assert torch.allclose(y.cpu().double(), P.rms_norm(x.double() + d.double(), w, 3e-6), atol=tol(dtype))
    assert torch.allclose(norm(x.to(DEV), out_dtype=F32).cpu().double(), P.rms_norm(x, w, 3e-6), atol=3e-5)


def test_position_part_makes_its_tables_once_per_step():
    from palm_infra_amd.config import PartSpec
    from palm_infra_amd.parts import make_context
    rot = build(PartSpec("position", "rotary", {"rotary_dim": 48, "theta": 500000.0, "pairing": "half_split"}), Tensors(), F32)
    ctx = make_context([0, 1], [10, 0], [[1, 2, 3], [4]], F32, DEV)
    cos, sin = rot.tables(ctx)
    rc, rs = P.rope_table([10, 11, 12, 0], 48, 500000.0)
    assert torch.allclose(cos.cpu().double(), rc, atol=1e-6) and torch.allclose(sin.cpu().double(), rs, atol=1e-6)
    assert rot.tables(ctx)[0] is cos
    same = build(PartSpec("position", "rotary", {"rotary_dim": 48, "theta": 500000.0}), Tensors(), F32)
    other = build(PartSpec("position", "rotary", {"rotary_dim": 48, "theta": 10000.0}), Tensors(), F32)
    assert same.tables(ctx)[0] is cos and other.tables(ctx)[0] is not cos
    assert build(PartSpec("position", "none"), Tensors(), F32).tables(ctx) is None
    with pytest.raises(ValueError, match="pairing"):
        build(PartSpec("position", "rotary", {"rotary_dim": 8, "theta": 1.0, "pairing": "spiral"}), Tensors(), F32)


def attention_spec(T, H, nh, nkv, hd, eps, theta, window=None, qk_norm=True, position=True, seed=0, bias=False):
    from palm_infra_amd.config import PartSpec, joined, tensor
    # without a q/k norm the scores' spread is set by these scales: kept near one so that bfloat16 rounding
    # cannot flip which key leads
    w = {"q": rand(nh * hd, H, seed=seed + 1, scale=0.1), "k": rand(nkv * hd, H, seed=seed + 2, scale=0.1),
         "v": rand(nkv * hd, H, seed=seed + 3, scale=0.3), "o": rand(H, nh * hd, seed=seed + 4, scale=0.3),
         "qn": rand(hd, seed=seed + 5) * 0.2 + 2.0, "kn": rand(hd, seed=seed + 6) * 0.2 + 1.0}
    parts = {}
    if qk_norm:
        parts["q_norm"] = PartSpec("norm", "rms", {"width": hd, "eps": eps}, {"weight": T.add(tensor("qn", (hd,), "vector"), w["qn"])})
        parts["k_norm"] = PartSpec("norm", "rms", {"width": hd, "eps": eps}, {"weight": T.add(tensor("kn", (hd,), "vector"), w["kn"])})
    if position:
        parts["position"] = PartSpec("position", "rotary", {"rotary_dim": hd, "theta": theta, "pairing": "half_split"})
    tensors = {"qkv": T.add(joined(("q", "k", "v"), ((nh * hd, H), (nkv * hd, H), (nkv * hd, H))), torch.cat([w["q"], w["k"], w["v"]])),
               "out": T.add(tensor("o", (H, nh * hd)), w["o"])}
    if bias:           # a projection with a bias is no part of Qwen3; the part takes one if its specification names it
        w.update(qb=rand(nh * hd, seed=seed + 7, scale=0.5), kb=rand(nkv * hd, seed=seed + 8, scale=0.5),
                 vb=rand(nkv * hd, seed=seed + 9, scale=0.5), ob=rand(H, seed=seed + 10, scale=0.5))
        tensors["qkv_bias"] = T.add(tensor("qkvb", ((nh + 2 * nkv) * hd,), "vector"), torch.cat([w["qb"], w["kb"], w["vb"]]))
        tensors["out_bias"] = T.add(tensor("ob", (H,), "vector"), w["ob"])
    spec = PartSpec("mixer", "attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": hd,
                                           "scale": hd ** -0.5, "window": window}, tensors, parts)
    return spec, w


def plain_attention(h, w, nh, nkv, hd, eps, theta, window, qk_norm, position):
    n = h.shape[0]
    zero = torch.zeros(1, dtype=torch.float64)
    q = (P.linear(h, w["q"]) + w.get("qb", zero).double()).reshape(n, nh, hd)
    k = (P.linear(h, w["k"]) + w.get("kb", zero).double()).reshape(n, nkv, hd)
    v = (P.linear(h, w["v"]) + w.get("vb", zero).double()).reshape(n, nkv, hd)
    if qk_norm:
        q, k = P.rms_norm(q, w["qn"], eps), P.rms_norm(k, w["kn"], eps)
    if position:
        cos, sin = P.rope_table(list(range(n)), hd, theta)
        q, k = P.rope_half_split(q, cos, sin), P.rope_half_split(k, cos, sin)
    return P.linear(P.causal_attention(q, k, v, hd ** -0.5, window).reshape(n, nh * hd), w["o"]) + w.get("ob", zero).double()


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("kw", [dict(), dict(window=40), dict(qk_norm=False), dict(position=False), dict(qk_norm=False, position=False),
                                dict(hd=64), dict(hd=64, window=40), dict(hd=64, qk_norm=False), dict(hd=64, position=False),
                                dict(hd=128, nkv=1, window=3), dict(bias=True), dict(hd=64, bias=True)])
def test_attention_part_in_pieces_against_whole_sequences(dtype, kw):
    """Plain attention without rotation or norm is one of the cases; each switch is a parameter of the part.  With
    heads of 64 or 128 the single-token steps in bfloat16 take the kernel that starts from the projection's rows."""
    from palm_infra_amd.cache import ModelCache
    from palm_infra_amd.parts import cache_needs, make_context
    H, nh, nkv, hd, eps, theta = 72, 6, kw.get("nkv", 3), kw.get("hd", 48), 1e-5, 10000.0
    window, qk_norm, position = kw.get("window"), kw.get("qk_norm", True), kw.get("position", True)
    T = Tensors()
    spec, w = attention_spec(T, H, nh, nkv, hd, eps, theta, window, qk_norm, position, bias=kw.get("bias", False))
    att = build(spec, T, dtype)
    needs = cache_needs(spec)
    assert needs[0].num_kv_heads == nkv and needs[0].head_dim == hd and needs[0].window == window
    cache = ModelCache([needs], [None], 64 * 8, None, 4096, dtype, DEV)
    seqs = [rand(157, H, seed=11), rand(77, H, seed=12)]
    slots = [cache.open(), cache.open()]
    outs = [[], []]
    done = [0, 0]
    # a prompt each, one token for the first only, a further piece, then both token by token (the second sequence's
    # first single token opens a page)
    for pieces in ([100, 64], [1, 0], [49, 0]) + ([1, 1],) * 7 + ([0, 6],):
        live = [b for b in range(2) if pieces[b] > 0]
        growth = [(slots[b], pieces[b]) for b in live]
        cache.reserve(growth)
        ctx = make_context([slots[b] for b in live], [done[b] for b in live], [[0] * pieces[b] for b in live], dtype, DEV)
        ctx.layer_cache = cache.layer_caches[0]
        h = torch.cat([seqs[b][done[b]:done[b] + pieces[b]] for b in live]).to(dtype).to(DEV)
        out = att.forward(h, ctx).cpu()
        cache.commit(growth)
        o = 0
        for b in live:
            outs[b].append(out[o:o + pieces[b]])
            o += pieces[b]
            done[b] += pieces[b]
    for b in range(2):
        ref = plain_attention(seqs[b].to(dtype), w_as(w, dtype), nh, nkv, hd, eps, theta, window, qk_norm, position)
        got = torch.cat(outs[b]).double()
        scale = float(ref.abs().max())
        assert torch.allclose(got, ref, atol=tol(dtype) * max(scale, 1.0)), (b, float((got - ref).abs().max()), scale)


def w_as(w, dtype):
    """The weights as the part holds them: matrices in the run's precision, norm vectors in float32."""
    return {k: (v if k in ("qn", "kn", "qb", "kb", "vb", "ob") else v.to(dtype)) for k, v in w.items()}


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_feed_forward_part(dtype):
    from palm_infra_amd.config import PartSpec, joined, tensor
    H, I = 80, 176
    T = Tensors()
    wg, wu, wd = rand(I, H, seed=1, scale=0.2), rand(I, H, seed=2, scale=0.2), rand(H, I, seed=3, scale=0.2)
    spec = PartSpec("feed_forward", "gated_silu", {"hidden_size": H, "intermediate_size": I},
                    {"gate_up": T.add(joined(("g", "u"), ((I, H), (I, H))), torch.cat([wg, wu]).to(dtype)),
                     "down": T.add(tensor("d", (H, I)), wd.to(dtype))})
    ff = build(spec, T, dtype)
    h = rand(9, H, seed=4).to(dtype)
    got = ff.forward(h.to(DEV), None).cpu().double()
    ref = P.swiglu_mlp(h, wg.to(dtype), wu.to(dtype), wd.to(dtype))
    assert torch.allclose(got, ref, atol=tol(dtype) * float(ref.abs().max()))
    # with biases (no part of Qwen3; the part takes them if its specification names them)
    bg, bd = rand(2 * I, seed=5, scale=0.5), rand(H, seed=6, scale=0.5)
    biased = PartSpec("feed_forward", "gated_silu", {"hidden_size": H, "intermediate_size": I},
                      dict(spec.tensors, gate_up_bias=T.add(tensor("gub", (2 * I,), "vector"), bg), down_bias=T.add(tensor("db", (H,), "vector"), bd)))
    for rows in (9, 70):
        h2 = rand(rows, H, seed=7).to(dtype)
        g, u = P.linear(h2, wg.to(dtype)) + bg[:I].double(), P.linear(h2, wu.to(dtype)) + bg[I:].double()
        ref2 = (g / (1 + torch.exp(-g)) * u) @ wd.to(dtype).double().T + bd.double()
        got2 = build(biased, T, dtype).forward(h2.to(DEV), None).cpu().double()
        assert torch.allclose(got2, ref2, atol=tol(dtype) * float(ref2.abs().max())), float((got2 - ref2).abs().max())
    # one expert of a routed feed-forward is this feed-forward: nothing else to reduce to here
    with pytest.raises(ValueError, match="do not fit"):
        build(PartSpec("feed_forward", "gated_silu", {"hidden_size": H, "intermediate_size": I + 1}, spec.tensors), T, dtype)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_embedding_and_head_parts(dtype):
    from palm_infra_amd.config import PartSpec, tensor
    V, H = 515, 80
    T = Tensors()
    table = rand(V, H, seed=1).to(dtype)
    ref_t = T.add(tensor("emb", (V, H), "table"), table)
    emb = build(PartSpec("embedding", "token_table", {"vocab_size": V, "hidden_size": H}, {"table": ref_t}), T, dtype)
    ids = torch.tensor([0, 514, 3], dtype=torch.int32)
    assert torch.equal(emb.forward(ids.to(DEV)).cpu(), table[ids.long()].float())
    head = build(PartSpec("head", "linear", {"vocab_size": V, "hidden_size": H}, {"weight": ref_t}), T, dtype)   # tied
    h = rand(4, H, seed=2).to(dtype)
    lg = head.forward(h.to(DEV)).cpu()
    assert lg.dtype == F32 and torch.allclose(lg.double(), P.linear(h, table), atol=1e-4 if dtype == F32 else 2e-2)


@pytest.mark.parametrize("n_rows", [70, 5])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_block_part_is_a_plain_decoder_layer(dtype, n_rows, model_dirs):
    """One layer of tiny model C, built as a block from the model's description and run alone: with many rows
    (the norms run as kernels of their own) and with few (in bfloat16 the products fold them in)."""
    from palm_infra_amd.cache import ModelCache
    from palm_infra_amd.config import config_from_dir
    from palm_infra_amd.parts import Builder, Prenormed, ResidualSink, as_tensor, cache_needs, make_context
    from palm_infra_amd.weights import ModelFiles, load_weights
    name = "float32" if dtype == F32 else "bfloat16"
    d = model_dirs["C"][name]
    files = ModelFiles(d)
    spec = config_from_dir(d).spec(files.names())
    weights = load_weights(spec, files, dtype, DEV)
    block = Builder(weights, dtype, DEV).build(spec.layers[1])
    cache = ModelCache([cache_needs(spec.layers[1])], [None], 64 * 4, None, 2048, dtype, DEV)
    slot = cache.open()
    cfg, w = P.read_model(d)
    S = P.sizes(cfg)
    x0 = rand(n_rows, S["H"], seed=5)
    cache.reserve([(slot, n_rows)])
    ctx = make_context([slot], [0], [[0] * n_rows], dtype, DEV)
    ctx.layer_cache = cache.layer_caches[0]
    xd = x0.to(DEV)
    h = block.entry_norm(xd)
    out = block.forward(xd, h, ctx, ResidualSink(xd, block.entry_norm))      # the reader after it: the same norm again
    assert isinstance(out, Prenormed) == (dtype == BF16 and n_rows <= 16)
    ref = P.decoder_layer(x0.double(), w, 1, S, list(range(n_rows)))
    assert xd.dtype == F32 and torch.allclose(xd.cpu().double(), ref, atol=tol(dtype) * float(ref.abs().max()))   # in place, 32-bit
    ref_out = P.rms_norm(ref, w["model.layers.1.input_layernorm.weight"].double(), S["eps"])
    got_out = as_tensor(out).cpu().double()
    assert torch.allclose(got_out, ref_out, atol=tol(dtype) * float(ref_out.abs().max()))
    # rows picked by the reader: nothing is written back, only those rows come out
    x2 = x0.to(DEV)
    rows = torch.tensor([n_rows - 1, 0], dtype=torch.int32).to(DEV)
    picked = as_tensor(block.forward(x2, block.entry_norm(x2), ctx, ResidualSink(x2, block.entry_norm, rows=rows))).cpu().double()
    assert torch.allclose(picked, ref_out[[n_rows - 1, 0]], atol=tol(dtype) * float(ref_out.abs().max()))


def test_unknown_kind_names_the_registered_ones():
    from palm_infra_amd.config import PartSpec
    with pytest.raises(KeyError, match="attention"):
        build(PartSpec("mixer", "convolution"), Tensors(), F32)

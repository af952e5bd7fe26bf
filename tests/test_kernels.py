"""Each kernel alone against its plain reference, at other sizes than the engine's tiny models use."""
import math

import numpy as np
import pytest
import torch

import plain_qwen3 as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16


@pytest.fixture(scope="module")
def ops():
    from palm_infra_amd.kernels import ops
    return ops


def rand(*shape, seed=0, scale=1.0, dtype=F32):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


def tol(dtype):
    return 2e-5 if dtype == F32 else 2e-2


# ---- embedding, norm, swiglu, cast --------------------------------------------------------------

@pytest.mark.parametrize("dtype", [F32, BF16])
def test_embed(ops, dtype):
    table = rand(515, 80, seed=1, dtype=dtype)
    ids = torch.tensor([0, 514, 7, 7, 300], dtype=torch.int32)
    got = ops.embed(table.to(DEV), ids.to(DEV)).cpu()
    assert got.dtype == F32 and torch.equal(got, table[ids.long()].float())
    bad = ops.embed(table.to(DEV), torch.tensor([3, 515, -1], dtype=torch.int32).to(DEV)).cpu()
    assert torch.equal(bad[0], table[3].float()) and torch.isnan(bad[1:]).all()      # visible, never a wrong row


@pytest.mark.parametrize("width", [8, 17, 64, 2048, 5120])
@pytest.mark.parametrize("eps", [1e-6, 1e-5])
def test_rmsnorm_widths_of_the_reference_test(ops, width, eps):       # tests/test_norm.cpp:43-256
    x, w = rand(5, width, seed=width), rand(width, seed=1) + 1.0
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), eps, F32).cpu()
    assert torch.allclose(got.double(), P.rms_norm(x, w, eps), atol=1e-5 if width < 2048 else 1e-4)


def test_rmsnorm_eps_inside_the_root_and_zero_rows(ops):
    x = torch.full((2, 32), 1e-4)
    x[1] = 0.0
    got = ops.rmsnorm(x.to(DEV), torch.ones(32).to(DEV), 1e-6, F32).cpu()
    assert torch.allclose(got[0], x[0] / math.sqrt(1e-8 + 1e-6), rtol=1e-5) and float(got[1].abs().max()) == 0.0


@pytest.mark.parametrize("out_dtype,delta_dtype", [(F32, F32), (BF16, BF16), (BF16, F32)])
def test_rmsnorm_adds_the_pending_branch_in_32_bit(ops, out_dtype, delta_dtype):
    x, d, w = rand(7, 96, seed=2), rand(7, 96, seed=3, dtype=delta_dtype), rand(96, seed=4) + 1.0
    xd = x.to(DEV)
    got = ops.rmsnorm(xd, w.to(DEV), 1e-5, out_dtype, delta=d.to(DEV), update_x=True).cpu()
    assert torch.equal(xd.cpu(), x + d.float())                        # the residual stream holds the exact 32-bit sum
    assert torch.allclose(got.double(), P.rms_norm(x.double() + d.double(), w, 1e-5), atol=tol(out_dtype))
    # row selection reads x + delta without touching x
    xd2 = x.to(DEV)
    rows = torch.tensor([6, 0, 3], dtype=torch.int32).to(DEV)
    sel = ops.rmsnorm(xd2, w.to(DEV), 1e-5, F32, delta=d.to(DEV), rows=rows).cpu()
    assert torch.equal(xd2.cpu(), x)
    assert torch.allclose(sel.double(), P.rms_norm(x.double() + d.double(), w, 1e-5)[[6, 0, 3]], atol=2e-5)


@pytest.mark.parametrize("width", [2048, 4096, 5120, 8200, 5000])
@pytest.mark.parametrize("dtypes", [(BF16, BF16), (F32, F32), (BF16, F32), (None, BF16)])
def test_rmsnorm_of_many_rows(ops, width, dtypes):
    """Prompts: hundreds of rows of the widths that models have, with and without a pending branch, whole and
    through a row selection."""
    delta_dtype, out_dtype = dtypes
    n = 300
    x, w = rand(n, width, seed=width), rand(width, seed=4) + 1.0
    d = rand(n, width, seed=3, dtype=delta_dtype) if delta_dtype is not None else None
    xd = x.to(DEV)
    got = ops.rmsnorm(xd, w.to(DEV), 1e-6, out_dtype, delta=None if d is None else d.to(DEV), update_x=d is not None).cpu()
    total = x if d is None else x + d.float()
    assert torch.equal(xd.cpu(), total)                               # the stream holds the exact 32-bit sum (or is untouched)
    assert torch.allclose(got.double(), P.rms_norm(total.double(), w, 1e-6), atol=1e-4 if out_dtype == F32 else 2e-2, rtol=0 if out_dtype == F32 else 1e-2)
    rows = torch.arange(n - 1, -1, -1, dtype=torch.int32).to(DEV)       # a selection of as many rows, backwards
    sel = ops.rmsnorm(x.to(DEV), w.to(DEV), 1e-6, F32, delta=None if d is None else d.to(DEV), rows=rows).cpu()
    assert torch.allclose(sel.double(), P.rms_norm(total.double(), w, 1e-6).flip(0), atol=1e-4)


@pytest.mark.parametrize("planes", [2, 3, 4])
@pytest.mark.parametrize("width", [96, 4096, 5000])
def test_rmsnorm_adds_planes_of_partial_sums_in_their_order(ops, planes, width):
    x, w = rand(5, width, seed=2), rand(width, seed=4) + 1.0
    d = rand(planes, 5, width, seed=3) * torch.tensor([1.0, 1e3, 1e-3, 7.0])[:planes, None, None]   # the order of the sum shows
    want_x = x.clone()
    for p in range(planes):
        want_x = want_x + d[p]
    xd = x.to(DEV)
    got = ops.rmsnorm(xd, w.to(DEV), 1e-5, BF16, delta=d.to(DEV), update_x=True).cpu()
    assert torch.equal(xd.cpu(), want_x)
    assert torch.allclose(got.double(), P.rms_norm(want_x.double(), w, 1e-5), atol=2e-2, rtol=1e-2)
    rows = torch.tensor([4, 0], dtype=torch.int32).to(DEV)
    sel = ops.rmsnorm(x.to(DEV), w.to(DEV), 1e-5, F32, delta=d.to(DEV), rows=rows).cpu()
    assert torch.allclose(sel.double(), P.rms_norm(want_x.double(), w, 1e-5)[[4, 0]], atol=1e-4)
    with pytest.raises(Exception, match="planes"):
        ops.rmsnorm(x.to(DEV), w.to(DEV), 1e-5, F32, delta=torch.zeros(5, 5, width, device=DEV))
    with pytest.raises(Exception, match="planes"):
        ops.rmsnorm(x.to(DEV), w.to(DEV), 1e-5, F32, delta=torch.zeros(2, 5, width, device=DEV, dtype=BF16))


def test_qk_norm_rope_store_adds_planes(ops):
    nh, nkv, hd, n = 6, 2, 80, 5
    planes = rand(3, n, (nh + 2 * nkv) * hd, seed=11)
    whole = (planes[0] + planes[1]) + planes[2]
    qw, kw = rand(hd, seed=1) + 1.0, rand(hd, seed=2) + 1.0
    pos = torch.arange(60, 60 + n, dtype=torch.int32).to(DEV)
    table = torch.tensor([[2, 1]], dtype=torch.int32).to(DEV)
    slot = torch.zeros(n, dtype=torch.int32).to(DEV)
    inv = torch.from_numpy((1.0 / np.power(np.float32(1e4), 2.0 * np.arange(hd // 2, dtype=np.float32) / hd)).astype(np.float32))
    cos, sin = ops.rope_table(pos, inv.to(DEV))
    results = []
    for qkv, kw_extra in ((whole.to(BF16).to(DEV), {}), (planes.to(DEV), {"out_dtype": BF16})):
        kc, vc = _paged(4, nkv, hd, BF16)
        q = ops.qk_norm_rope_store(qkv, nh, nkv, hd, pos, q_norm_w=qw.to(DEV), k_norm_w=kw.to(DEV), eps=1e-6, cos=cos, sin=sin,
                                   rotary_dim=hd, pairing=0, k_cache=kc, v_cache=vc, block_table=table, tok_slot=slot, **kw_extra)
        results.append((q.cpu().float(), kc.cpu().float(), vc.cpu().float()))
    # the planes are added in 32-bit, the single input was rounded to bfloat16 first: equal within that rounding
    for a, b in zip(*results):
        assert torch.allclose(a, b, atol=6e-2, rtol=2e-2)
    assert float(results[1][1].abs().max()) > 0.5
    with pytest.raises(Exception, match="planes"):
        ops.qk_norm_rope_store(planes.to(DEV), nh, nkv, hd, pos, write_cache=False)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_swiglu(ops, dtype):
    gu = rand(9, 2 * 176, seed=5, scale=3.0, dtype=dtype)
    got = ops.swiglu(gu.to(DEV)).cpu()
    g, u = gu[:, :176].double(), gu[:, 176:].double()
    assert torch.allclose(got.double(), g / (1 + torch.exp(-g)) * u, atol=tol(dtype), rtol=tol(dtype))
    swapped = u / (1 + torch.exp(-u)) * g
    assert not torch.allclose(got.double(), swapped, atol=0.1)


def test_swiglu_of_bfloat16_rows_far_from_zero(ops):
    """The prompt kernel for bfloat16 uses the hardware's 2^x and reciprocal: gates from -100 (where 2^x overflows
    and the weight must come out as zero, not as a NaN) to +100, rounded to the nearest bfloat16."""
    gate = torch.tensor([-100.0, -90.0, -40.0, -20.0, -5.0, -1.0, -0.0, 0.0, 0.5, 1.0, 3.0, 10.0, 30.0, 88.0, 90.0, 100.0])
    gu = torch.cat([gate.repeat(3, 4), rand(3, 64, seed=9, scale=5.0, dtype=F32)], dim=1).to(BF16)         # [3, 2 * 64]
    got = ops.swiglu(gu.to(DEV)).cpu()
    g, u = gu[:, :64].double(), gu[:, 64:].double()
    want = (g / (1 + torch.exp(-g)) * u).to(BF16)
    assert torch.isfinite(got.float()).all()
    # at most one step of bfloat16 away from the rounded exact value (a product that lies next to a rounding border);
    # where 2^x overflows (a gate below -88) the exact weight is below 1e-36 and the kernel's is zero
    steps = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs()
    tiny_ones = (want.float().abs() < 1e-30) & (got.float().abs() < 1e-30)
    steps = torch.where(tiny_ones, torch.zeros_like(steps), steps)
    assert int(steps.max()) <= 1 and float((steps > 0).float().mean()) < 0.05, (int(steps.max()), float((steps > 0).float().mean()))
    assert int(tiny_ones.sum()) >= 6


def test_conversion_at_load_rounds_to_nearest_even_from_every_stored_type(ops):
    x = torch.tensor([1.0, 1.00390625, 1.01171875, -3.1415927, 1e-40, 65504.0, float("inf"), 0.3, -7.7e-3])
    for stored in (F32, BF16, torch.float16, torch.float64):
        src = x.to(stored)
        for kept in (F32, BF16):
            # into the middle rows of a larger tensor, as the loader joins q, k and v
            dst = torch.full((3, x.numel()), 9.0, dtype=kept, device=DEV)
            ops.convert_into(src.to(DEV), dst[1])
            assert torch.equal(dst[1].cpu(), src.to(kept)), (stored, kept)
            assert bool((dst[0] == 9.0).all()) and bool((dst[2] == 9.0).all())
    with pytest.raises(Exception, match="stored as"):
        ops.convert_into(torch.zeros(4, dtype=torch.int32, device=DEV), torch.zeros(4, dtype=F32, device=DEV))


def test_random_fill_gives_the_host_function_s_bits(ops):
    """The device kernel and weights/random_numbers.py are the same function of (key, index): float32 and
    bfloat16, a count that is no multiple of anything, several keys, mean and scale as the model's tensors use."""
    from palm_infra_amd.weights import random_numbers as R
    for key, n, mean, std in ((R.tensor_key(0, "model.embed_tokens.weight"), 1_000_003, 0.0, 0.02),
                              (R.tensor_key(7, "model.norm.weight"), 4099, 1.0, 0.02), ((1 << 64) - 1, 70_001, -3.0, 1.0),
                              (0, 65, 0.0, 1.0)):
        want = torch.from_numpy(R.normal(key, n, mean, std))
        for dtype in (F32, BF16):
            got = torch.empty(n, dtype=dtype, device=DEV)
            ops.random_fill(got, key, mean, std)
            assert torch.equal(got.cpu(), want.to(dtype)), (key, n, dtype, int((got.cpu() != want.to(dtype)).sum()))
    # a window far into a long stream (what a large tensor's later rows are)
    key = R.tensor_key(3, "model.layers.0.mlp.down_proj.weight")
    n, first, count = 50_331_648, 50_000_000, 100_000
    got = torch.empty(n, dtype=BF16, device=DEV)
    ops.random_fill(got, key, 0.0, 0.02)
    want = torch.from_numpy(R.standard_normal(key, first, count)) * torch.tensor(0.02) + torch.tensor(0.0)
    assert torch.equal(got[first:first + count].cpu(), want.to(BF16))


# ---- linear -------------------------------------------------------------------------------------

@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (3, 130, 67), (65, 64, 16), (70, 515, 80), (129, 96, 224)])
@pytest.mark.parametrize("ta,tw,tc", [(F32, F32, F32), (BF16, BF16, BF16), (BF16, F32, BF16), (BF16, BF16, F32)])
def test_linear_exact(ops, M, N, K, ta, tw, tc):
    a, w = rand(M, K, seed=M, dtype=ta), rand(N, K, seed=N, dtype=tw)
    got = ops.linear_exact(a.to(DEV), w.to(DEV), tc).cpu()
    ref = P.linear(a, w)
    assert got.dtype == tc
    assert torch.allclose(got.double(), ref, atol=1e-4 if tc == F32 else 0.1, rtol=1e-5 if tc == F32 else 1e-2)


def test_linear_exact_result_of_a_row_does_not_depend_on_the_other_rows(ops):
    a, w = rand(70, 80, seed=1), rand(130, 80, seed=2)
    whole = ops.linear_exact(a.to(DEV), w.to(DEV)).cpu()
    for r in (0, 33, 69):
        alone = ops.linear_exact(a[r:r + 1].contiguous().to(DEV), w.to(DEV)).cpu()
        assert torch.equal(alone[0], whole[r])


def test_linear_refuses_what_does_not_fit(ops):
    from palm_infra_amd.kernels import KernelError
    with pytest.raises(KernelError, match="inner size"):
        ops.linear_exact(rand(2, 5).to(DEV), rand(3, 6).to(DEV))
    with pytest.raises(KernelError, match="GPU only"):
        ops.linear_exact(rand(2, 5), rand(3, 5))
    with pytest.raises(KernelError, match="contiguous"):
        ops.linear_exact(rand(5, 2).t().to(DEV), rand(3, 5).to(DEV))


# ---- rotation, q/k norm and the cache write -----------------------------------------------------

def _paged(n_pages, nkv, hd, dtype):
    """Empty key and value caches; values are kept transposed, [pages, nkv, hd, 64]."""
    return (torch.zeros(n_pages, nkv, 64, hd, dtype=dtype, device=DEV), torch.zeros(n_pages, nkv, hd, 64, dtype=dtype, device=DEV))


@pytest.mark.parametrize("theta,half", [(10000.0, 8), (1000000.0, 24), (500000.0, 64)])
def test_rope_table(ops, theta, half):
    pos = [0, 1, 2, 63, 64, 1000, 40000]
    i = np.arange(half, dtype=np.float32)
    inv = (np.float32(1.0) / np.power(np.float32(theta), np.float32(2.0) * i / np.float32(2 * half))).astype(np.float32)
    cos, sin = ops.rope_table(torch.tensor(pos, dtype=torch.int32).to(DEV), torch.from_numpy(inv).to(DEV))
    rc, rs = P.rope_table(pos, 2 * half, theta)
    # the angle is a float32 product on both sides; pow may differ in the last bit, which the position multiplies
    assert torch.allclose(cos.cpu().double(), rc, atol=2e-3) and torch.allclose(sin.cpu().double(), rs, atol=2e-3)
    assert torch.allclose(cos.cpu().double()[:5], rc[:5], atol=1e-5) and torch.allclose(sin.cpu().double()[:5], rs[:5], atol=1e-5)
    assert float(cos[0, 0]) == 1.0 and float(sin[0, 0]) == 0.0         # tests/test_engine.cpp:90-91


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("nh,nkv,hd", [(5, 5, 48), (6, 2, 80), (3, 1, 128)])
def test_qk_norm_rope_store(ops, dtype, nh, nkv, hd):
    # two sequences in slots 2 and 0, the first continuing at position 60 (so it crosses a page border)
    starts, counts, slots = [60, 0], [9, 5], [2, 0]
    n = sum(counts)
    pos = [s + j for s, c in zip(starts, counts) for j in range(c)]
    tslot = [sl for sl, c in zip(slots, counts) for _ in range(c)]
    qkv = rand(n, (nh + 2 * nkv) * hd, seed=hd, dtype=dtype)
    qw, kw = rand(hd, seed=1) + 1.0, rand(hd, seed=2) + 1.0
    eps, theta = 1e-5, 10000.0
    table = torch.full((4, 3), 7, dtype=torch.int32)
    table[2, :2] = torch.tensor([5, 1])
    table[0, :1] = torch.tensor([3])
    kc, vc = _paged(8, nkv, hd, dtype)
    inv = torch.from_numpy((1.0 / np.power(np.float32(theta), 2.0 * np.arange(hd // 2, dtype=np.float32) / hd)).astype(np.float32))
    cos, sin = ops.rope_table(torch.tensor(pos, dtype=torch.int32).to(DEV), inv.to(DEV))
    q = ops.qk_norm_rope_store(qkv.to(DEV), nh, nkv, hd, torch.tensor(pos, dtype=torch.int32).to(DEV), q_norm_w=qw.to(DEV),
                               k_norm_w=kw.to(DEV), eps=eps, cos=cos, sin=sin, rotary_dim=hd, pairing=0, k_cache=kc, v_cache=vc,
                               block_table=table.to(DEV), tok_slot=torch.tensor(tslot, dtype=torch.int32).to(DEV)).cpu()
    x = qkv.double()
    rq = x[:, :nh * hd].reshape(n, nh, hd)
    rk = x[:, nh * hd:(nh + nkv) * hd].reshape(n, nkv, hd)
    rv = x[:, (nh + nkv) * hd:].reshape(n, nkv, hd)
    c64, s64 = P.rope_table(pos, hd, theta)
    rq = P.rope_half_split(P.rms_norm(rq, qw, eps), c64, s64)
    rk = P.rope_half_split(P.rms_norm(rk, kw, eps), c64, s64)
    t = 5e-5 if dtype == F32 else 4e-2
    assert torch.allclose(q.double().reshape(n, nh, hd), rq, atol=t)
    kc, vc = kc.cpu().double(), vc.cpu().double()
    for i in range(n):
        page = int(table[tslot[i], pos[i] // 64])
        assert torch.allclose(kc[page, :, pos[i] % 64], rk[i], atol=t), i
        assert torch.allclose(vc[page, :, :, pos[i] % 64], rv[i], atol=1e-12 if dtype == F32 else 0), i   # v is stored as it is
    written = {(int(table[tslot[i], pos[i] // 64]), pos[i] % 64) for i in range(n)}
    for page in range(8):
        for r in range(64):
            if (page, r) not in written:
                assert float(kc[page, :, r].abs().max()) == 0.0 and float(vc[page, :, :, r].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("nh,nkv,hd", [(5, 5, 48), (6, 2, 80), (3, 1, 128), (8, 2, 16), (4, 4, 32), (9, 3, 64), (2, 1, 256), (3, 1, 144)])
def test_qk_norm_rope_store_of_many_tokens(ops, dtype, nh, nkv, hd):
    """Prompts go through kernels of their own (heads held in registers, v written tile by tile): three
    sequences that start inside pages, cross page borders, and fill no tile of 64 tokens."""
    starts, counts, slots = [60, 0, 130], [250, 141, 3], [2, 0, 3]
    n = sum(counts)
    pos = [s + j for s, c in zip(starts, counts) for j in range(c)]
    tslot = [sl for sl, c in zip(slots, counts) for _ in range(c)]
    qkv = rand(n, (nh + 2 * nkv) * hd, seed=hd, dtype=dtype)
    qw, kw = rand(hd, seed=1) + 1.0, rand(hd, seed=2) + 1.0
    eps, theta = 1e-5, 10000.0
    table = torch.full((4, 5), 9, dtype=torch.int32)
    table[2] = torch.tensor([5, 1, 7, 2, 4])
    table[0, :3] = torch.tensor([3, 6, 8])
    table[3, 2] = 0
    kc, vc = _paged(10, nkv, hd, dtype)
    inv = torch.from_numpy((1.0 / np.power(np.float32(theta), 2.0 * np.arange(hd // 2, dtype=np.float32) / hd)).astype(np.float32))
    pos_d = torch.tensor(pos, dtype=torch.int32).to(DEV)
    cos, sin = ops.rope_table(pos_d, inv.to(DEV))
    q = ops.qk_norm_rope_store(qkv.to(DEV), nh, nkv, hd, pos_d, q_norm_w=qw.to(DEV), k_norm_w=kw.to(DEV), eps=eps, cos=cos, sin=sin,
                               rotary_dim=hd, pairing=0, k_cache=kc, v_cache=vc, block_table=table.to(DEV),
                               tok_slot=torch.tensor(tslot, dtype=torch.int32).to(DEV)).cpu()
    x = qkv.double()
    rq = x[:, :nh * hd].reshape(n, nh, hd)
    rk = x[:, nh * hd:(nh + nkv) * hd].reshape(n, nkv, hd)
    rv = x[:, (nh + nkv) * hd:].reshape(n, nkv, hd)
    c64, s64 = P.rope_table(pos, hd, theta)
    rq = P.rope_half_split(P.rms_norm(rq, qw, eps), c64, s64)
    rk = P.rope_half_split(P.rms_norm(rk, kw, eps), c64, s64)
    t = 5e-5 if dtype == F32 else 4e-2
    assert torch.allclose(q.double().reshape(n, nh, hd), rq, atol=t)
    kc, vc = kc.cpu().double(), vc.cpu().double()
    written = torch.zeros(10, 64, dtype=torch.bool)
    for i in range(n):
        page = int(table[tslot[i], pos[i] // 64])
        assert torch.allclose(kc[page, :, pos[i] % 64], rk[i], atol=t), i
        assert torch.allclose(vc[page, :, :, pos[i] % 64], rv[i], atol=1e-12 if dtype == F32 else 0), i   # v is stored as it is
        written[page, pos[i] % 64] = True
    rest = ~written
    assert float(kc.permute(0, 2, 1, 3)[rest].abs().max()) == 0.0 and float(vc.permute(0, 3, 1, 2)[rest].abs().max()) == 0.0
    # the same tokens a few at a time (the kernel for few tokens) leave the same cache, up to the last bit of a sum
    kc2, vc2 = _paged(10, nkv, hd, dtype)
    for a in range(0, n, 9):
        sl = slice(a, a + 9)
        ops.qk_norm_rope_store(qkv[sl].contiguous().to(DEV), nh, nkv, hd, pos_d[sl].contiguous(), q_norm_w=qw.to(DEV), k_norm_w=kw.to(DEV),
                               eps=eps, cos=cos[sl].contiguous(), sin=sin[sl].contiguous(), rotary_dim=hd, pairing=0, k_cache=kc2,
                               v_cache=vc2, block_table=table.to(DEV), tok_slot=torch.tensor(tslot[sl], dtype=torch.int32).to(DEV))
    assert torch.allclose(kc2.cpu().double(), kc, atol=1e-5 if dtype == F32 else 4e-2) and torch.equal(vc2.cpu().double(), vc)
    # a factor on the queries (what a prompt's attention kernel wants folded in before they are rounded): q times
    # the factor, keys and values as before; through the kernel for many tokens and the one for few
    for sl in (slice(0, n), slice(0, 9)):
        kc3, vc3 = _paged(10, nkv, hd, dtype)
        q3 = ops.qk_norm_rope_store(qkv[sl].contiguous().to(DEV), nh, nkv, hd, pos_d[sl].contiguous(), q_norm_w=qw.to(DEV), k_norm_w=kw.to(DEV),
                                    eps=eps, cos=cos[sl].contiguous(), sin=sin[sl].contiguous(), rotary_dim=hd, pairing=0, k_cache=kc3,
                                    v_cache=vc3, block_table=table.to(DEV), tok_slot=torch.tensor(tslot[sl], dtype=torch.int32).to(DEV),
                                    q_scale=0.375).cpu()
        m = q3.shape[0]
        assert torch.allclose(q3.double().reshape(m, nh, hd), 0.375 * rq[sl], atol=t)
        if m == n:
            assert torch.allclose(kc3.cpu().double(), kc, atol=1e-5 if dtype == F32 else 4e-2) and torch.equal(vc3.cpu().double(), vc)


def test_qk_norm_rope_store_of_many_tokens_whole_or_in_planes_and_other_rotations(ops):
    nh, nkv, hd, n = 6, 2, 64, 430           # enough tokens for the kernels that take many
    i32 = lambda xs: torch.tensor(xs, dtype=torch.int32).to(DEV)
    pos, slot = i32(list(range(30, 30 + n))), i32([1] * n)
    table = i32([[9] * 8, [4, 2, 6, 1, 8, 3, 7, 5]])
    qw, kw = (rand(hd, seed=1) + 1.0).to(DEV), (rand(hd, seed=2) + 1.0).to(DEV)
    planes = rand(3, n, (nh + 2 * nkv) * hd, seed=11)
    whole = ((planes[0] + planes[1]) + planes[2]).to(BF16)
    for pairing, rot, norms, writes in ((0, hd, True, True), (1, hd, True, True), (1, 24, False, True), (0, 0, True, True),
                                        (0, 32, True, True), (0, hd, True, False)):
        cos = sin = None
        if rot:
            inv = torch.from_numpy((1.0 / np.power(np.float32(1e6), 2.0 * np.arange(rot // 2, dtype=np.float32) / rot)).astype(np.float32))
            cos, sin = ops.rope_table(pos, inv.to(DEV))
        kw_args = dict(q_norm_w=qw if norms else None, k_norm_w=kw if norms else None, eps=1e-6, cos=cos, sin=sin, rotary_dim=rot,
                       pairing=pairing, block_table=table, tok_slot=slot, write_cache=writes)
        results = []
        # all at once (the kernels for many tokens where they serve), all at once from planes, and 47 at a time
        kc, vc = _paged(10, nkv, hd, BF16)
        q = ops.qk_norm_rope_store(whole.to(DEV), nh, nkv, hd, pos, k_cache=kc, v_cache=vc, **kw_args)
        kc3, vc3 = _paged(10, nkv, hd, BF16)
        q3 = ops.qk_norm_rope_store(planes.to(DEV), nh, nkv, hd, pos, k_cache=kc3, v_cache=vc3, out_dtype=BF16, **kw_args)
        kc2, vc2 = _paged(10, nkv, hd, BF16)
        qs = []
        for a in range(0, n, 47):
            sl = slice(a, a + 47)
            args = dict(kw_args, cos=None if cos is None else cos[sl].contiguous(), sin=None if sin is None else sin[sl].contiguous(),
                        tok_slot=slot[sl].contiguous())
            qs.append(ops.qk_norm_rope_store(whole[sl].contiguous().to(DEV), nh, nkv, hd, pos[sl].contiguous(), k_cache=kc2, v_cache=vc2, **args))
        case = (pairing, rot, norms, writes)
        assert torch.allclose(q.float(), torch.cat(qs).float(), atol=6e-2, rtol=2e-2), case
        assert torch.allclose(kc.float(), kc2.float(), atol=6e-2, rtol=2e-2) and torch.allclose(vc.float(), vc2.float(), atol=2e-2, rtol=1e-2), case
        assert torch.allclose(q3.float(), torch.cat(qs).float(), atol=6e-2, rtol=2e-2), case
        assert torch.allclose(kc3.float(), kc2.float(), atol=6e-2, rtol=2e-2) and torch.allclose(vc3.float(), vc2.float(), atol=2e-2, rtol=1e-2), case
        assert (float(kc.abs().max()) > 0.5) == writes, case


def test_rotation_variants_interleaved_partial_and_none(ops):
    n, nh, nkv, hd, rot = 4, 2, 1, 32, 16
    pos = [3, 4, 5, 6]
    qkv = rand(n, (nh + 2 * nkv) * hd, seed=9)
    inv = torch.from_numpy((1.0 / np.power(np.float32(1e4), 2.0 * np.arange(rot // 2, dtype=np.float32) / rot)).astype(np.float32))
    posd = torch.tensor(pos, dtype=torch.int32).to(DEV)
    cos, sin = ops.rope_table(posd, inv.to(DEV))
    x = qkv.double()[:, :nh * hd].reshape(n, nh, hd)
    c, s = P.rope_table(pos, rot, 1e4)
    # partial rotation, half-split: the tail passes (kernels/rope.cpp:26-29)
    q = ops.qk_norm_rope_store(qkv.to(DEV), nh, nkv, hd, posd, cos=cos, sin=sin, rotary_dim=rot, pairing=0, write_cache=False).cpu()
    assert torch.allclose(q.double().reshape(n, nh, hd), P.rope_half_split(x, c, s), atol=1e-5)
    # interleaved pairs (2i, 2i+1) (kernels/rope.cpp:31-40)
    q = ops.qk_norm_rope_store(qkv.to(DEV), nh, nkv, hd, posd, cos=cos, sin=sin, rotary_dim=rot, pairing=1, write_cache=False).cpu()
    ref = x.clone()
    ev, od = x[..., 0:rot:2], x[..., 1:rot:2]
    ref[..., 0:rot:2] = ev * c[:, None] - od * s[:, None]
    ref[..., 1:rot:2] = ev * s[:, None] + od * c[:, None]
    assert torch.allclose(q.double().reshape(n, nh, hd), ref, atol=1e-5)
    # no norm, no rotation: q comes through unchanged
    q = ops.qk_norm_rope_store(qkv.to(DEV), nh, nkv, hd, posd, write_cache=False).cpu()
    assert torch.equal(q.reshape(n, nh, hd), qkv[:, :nh * hd].reshape(n, nh, hd))


# ---- attention ----------------------------------------------------------------------------------

def _fill_cache(kc, vc, table, slot, k, v):
    """k, v [len, nkv, hd] into the pages of `slot`."""
    for p in range(k.shape[0]):
        page = int(table[slot, p // 64])
        kc[page, :, p % 64] = k[p].to(kc.dtype)
        vc[page, :, :, p % 64] = v[p].to(vc.dtype)


def _poison(t):
    """What a request whose activations overflowed may leave in its pages: NaN, +inf and -inf in turn."""
    flat = t.view(-1)
    flat[0::3], flat[1::3], flat[2::3] = float("nan"), float("inf"), float("-inf")
    return t


def _attention_case(ops, fn, dtype, nh, nkv, hd, lens_new, window, seed=0, scale=None, poison=False):
    """Sequences (total length, new tokens): queries are the last `new` positions.  Every place of the cache that
    belongs to no sequence (other pages, the last page's tail) holds stale values: random numbers, or with
    ``poison`` NaN and infinities."""
    scale = scale if scale is not None else hd ** -0.5
    B = len(lens_new)
    n_pages = sum((L + 63) // 64 for L, _ in lens_new) + 2
    perm = torch.randperm(n_pages - 1, generator=torch.Generator().manual_seed(seed)).tolist()
    max_pages = max((L + 63) // 64 for L, _ in lens_new) + 1
    slots = torch.randperm(B + 4, generator=torch.Generator().manual_seed(seed + 7)).tolist()[:B]      # distinct, not in order
    table = torch.full((B + 4, max_pages), n_pages - 1, dtype=torch.int32)
    kc = rand(n_pages, nkv, 64, hd, seed=seed + 50, dtype=dtype).to(DEV)      # stale values everywhere
    vc = rand(n_pages, nkv, hd, 64, seed=seed + 51, dtype=dtype).to(DEV)
    if poison:
        _poison(kc), _poison(vc)
    qs, refs, o = [], [], 0
    for b, (L, new) in enumerate(lens_new):
        npg = (L + 63) // 64
        table[slots[b], :npg] = torch.tensor(perm[o:o + npg], dtype=torch.int32)
        o += npg
        k, v = rand(L, nkv, hd, seed=seed + 10 * b + 1, dtype=dtype), rand(L, nkv, hd, seed=seed + 10 * b + 2, dtype=dtype)
        q = rand(L, nh, hd, seed=seed + 10 * b + 3, scale=2.0, dtype=dtype)
        _fill_cache(kc, vc, table, slots[b], k.to(DEV), v.to(DEV))
        refs.append(P.causal_attention(q, k, v, scale, window)[L - new:])
        qs.append(q[L - new:])
    qcat = torch.cat(qs).reshape(-1, nh * hd).contiguous()
    i32 = lambda xs: torch.tensor(xs, dtype=torch.int32).to(DEV)
    cu = [0]
    for _, new in lens_new:
        cu.append(cu[-1] + new)
    got = fn(qcat.to(DEV), kc, vc, table.to(DEV), i32(slots), i32([L - new for L, new in lens_new]),
             i32([new for _, new in lens_new]), i32(cu), max(new for _, new in lens_new), nh, nkv, hd, scale, window)
    return got.cpu().double().reshape(-1, nh, hd), torch.cat(refs)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("nh,nkv,hd", [(8, 4, 16), (5, 5, 48), (6, 1, 80), (4, 2, 128)])
def test_attention_exact_prompts_decode_and_mixed_lengths(ops, dtype, nh, nkv, hd):
    # tests/test_attention.cpp:186-217: GQA, past > 0, tails that do not fill a tile, 256 keys
    cases = [[(20, 20)], [(256, 256)], [(300, 1)], [(1, 1)], [(64, 64), (65, 1), (130, 70), (7, 7)]]
    for lens in cases:
        got, ref = _attention_case(ops, ops.attention_exact, dtype, nh, nkv, hd, lens, None, seed=len(lens))
        assert torch.allclose(got, ref, atol=1e-5 if dtype == F32 else 2e-2), lens


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_attention_exact_takes_nothing_from_what_lies_beyond_a_sequence(ops, dtype):
    """Pages are handed out uncleared: NaN and infinities beyond a sequence's length must not reach its output."""
    got, ref = _attention_case(ops, ops.attention_exact, dtype, 4, 2, 32, [(64, 64), (65, 1), (130, 70), (7, 7)], None, seed=5, poison=True)
    assert torch.isfinite(got).all() and torch.allclose(got, ref, atol=1e-5 if dtype == F32 else 2e-2)
    got, ref = _attention_case(ops, ops.attention_exact, dtype, 4, 2, 32, [(200, 1), (150, 150), (3, 1)], 70, seed=6, poison=True)
    assert torch.isfinite(got).all() and torch.allclose(got, ref, atol=1e-5 if dtype == F32 else 2e-2)


def test_attention_exact_over_thousands_of_keys(ops):
    """The float32 path's attention keeps its 1e-5 where a query sees thousands of keys (a prompt's continuation
    far into a sequence, single queries)."""
    for lens in ([(3000, 40)], [(2048, 1), (4500, 1), (70, 70)]):
        got, ref = _attention_case(ops, ops.attention_exact, F32, 8, 2, 64, lens, None, seed=len(lens))
        assert torch.allclose(got, ref, atol=1e-5), (lens, float((got - ref).abs().max()))


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_attention_exact_window(ops, dtype):
    for window in (1, 5, 64, 100):
        got, ref = _attention_case(ops, ops.attention_exact, dtype, 4, 2, 32, [(200, 200), (150, 1), (70, 3)], window, seed=window)
        assert torch.allclose(got, ref, atol=1e-5 if dtype == F32 else 2e-2), window


def _spike_case(ops, fn, dtype, L, spike_at, window=None, hd=32):
    """One key among L is made to dominate the last query; the output must be that key's value."""
    nh, nkv = 2, 1
    k = rand(L, nkv, hd, seed=1, scale=0.1, dtype=dtype)
    v = rand(L, nkv, hd, seed=2, dtype=dtype)
    q = rand(1, nh, hd, seed=3, scale=0.1, dtype=dtype)
    k[spike_at, 0, :] = 0
    k[spike_at, 0, 5] = 8.0
    q[0, :, 5] = 8.0                         # score 64 * scale at the spike, ~0 elsewhere
    table = torch.arange((L + 63) // 64 + 1, dtype=torch.int32).flip(0)[None, :].contiguous()
    n_pages = table.shape[1]
    kc, vc = _paged(n_pages, nkv, hd, dtype)
    _fill_cache(kc, vc, table, 0, k.to(DEV), v.to(DEV))
    i32 = lambda xs: torch.tensor(xs, dtype=torch.int32).to(DEV)
    got = fn(q.reshape(1, nh * hd).to(DEV), kc, vc, table.to(DEV), i32([0]), i32([L - 1]), i32([1]), i32([0, 1]), 1, nh, nkv, hd,
             1.0, window)
    return got.cpu().float().reshape(nh, hd), v


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_a_far_key_among_hundreds_is_found(ops, dtype):
    for L, at in ((700, 13), (700, 0), (700, 699), (513, 448), (64, 63), (65, 64)):
        got, v = _spike_case(ops, ops.attention_exact, dtype, L, at)
        assert torch.allclose(got, v[at, 0].float().expand(2, -1), atol=1e-2), (L, at)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_the_edge_of_a_window(ops, dtype):
    L, w = 300, 70
    inside, outside = L - w, L - w - 1       # the last query sits at L-1 and reads keys L-w .. L-1
    got, v = _spike_case(ops, ops.attention_exact, dtype, L, inside, window=w)
    assert torch.allclose(got, v[inside, 0].float().expand(2, -1), atol=1e-2)
    got, v = _spike_case(ops, ops.attention_exact, dtype, L, outside, window=w)
    assert not torch.allclose(got, v[outside, 0].float().expand(2, -1), atol=0.2)   # the spike is out of reach


# ---- sampling -----------------------------------------------------------------------------------

def test_argmax_takes_the_first_maximum(ops):
    lg = rand(6, 1000, seed=3)
    lg[1, 17] = lg[1, 900] = 50.0
    lg[2, :] = 0.0
    lg[3, 999] = 60.0
    lg[4, 0] = 60.0
    got = ops.argmax(lg.to(DEV)).cpu().tolist()
    assert got == [int(lg[0].argmax()), 17, 0, 999, 0, int(lg[5].argmax())]
    assert ops.argmax(torch.tensor([[0.5, 3.0, 2.0]]).to(DEV)).item() == 1       # tests/test_sampler.cpp:26-27
    # rows that do not start on 16 bytes, a width that is no multiple of four, ties at both ends of a wide row
    for V in (1003, 151937, 5):
        lg = rand(5, V, seed=V)
        lg[1, 2] = lg[1, V - 1] = 70.0
        lg[2, V - 1] = 70.0
        lg[3, V - 2] = lg[3, V // 2] = 70.0
        lg[4, :] = float("-inf")
        want = [int(lg[0].argmax()), 2, V - 1, min(V - 2, V // 2), 0]
        assert ops.argmax(lg.to(DEV)).cpu().tolist() == want, V


def _sample(ops, lg, u, **kw):
    lg = torch.as_tensor(lg, dtype=F32).reshape(1, -1)
    return ops.sample(lg.to(DEV), torch.tensor([u], dtype=F32).to(DEV), **kw).item()


def test_sampling_vectors_of_the_reference(ops):
    # tests/test_sampler.cpp:19-60
    assert _sample(ops, [0.5, 3.0, 2.0], 0.7, temperature=0.0) == 1
    assert _sample(ops, [0.5, 3.0, 2.0], 0.99, temperature=1.0, top_k=1) == 1
    for u in (0.0, 0.5, 0.999):
        assert _sample(ops, [4.0, 0.0, -1.0], u, temperature=1.0, min_p=0.5) == 0
        assert _sample(ops, [4.0, 0.0, -1.0], u, temperature=1.0, top_p=0.5) == 0
        assert _sample(ops, [4.0, 0.0, -1.0], u, temperature=1.0, top_k=2, top_p=0.5) == 0
    # tests/test_sampler.cpp:170-181
    lg = torch.tensor([[0.0, math.log(2.0), math.log(3.0)]])
    _, probs = ops.sample(lg.to(DEV), torch.zeros(1).to(DEV), 1.0, 0, 1.0, 0.0, want_probs=True)
    assert torch.allclose(probs.cpu(), torch.tensor([[1 / 6, 2 / 6, 3 / 6]]), atol=1e-5)


@pytest.mark.parametrize("kw", [
    dict(temperature=0.7), dict(temperature=1.3, min_p=0.05), dict(temperature=1.0, top_p=0.8), dict(temperature=0.9, top_p=0.3, min_p=0.01),
    dict(temperature=0.8, top_k=50), dict(temperature=1.0, top_k=5, top_p=0.7), dict(temperature=1.5, top_k=1024, top_p=0.9, min_p=0.02),
    dict(temperature=0.6, top_k=50, top_p=0.9),          # the reference's defaults
])
def test_the_distribution_drawn_from_is_the_plain_one(ops, kw):
    V = 5003
    lg = rand(3, V, seed=11, scale=2.0)
    lg[1, 100] = lg[1, 4000] = lg[1, 7] = float(lg[1].max()) + 0.5       # ties at the top, to be taken by lower id first
    lg[2, :] = torch.round(lg[2, :] * 2) / 2                              # many ties everywhere
    full = dict(temperature=1.0, top_k=0, top_p=0.0, min_p=0.0)
    full.update(kw)
    _, probs = ops.sample(lg.to(DEV), torch.zeros(3).to(DEV), full["temperature"], full["top_k"], full["top_p"], full["min_p"], want_probs=True)
    probs = probs.cpu().double().numpy()
    for r in range(3):
        ref = P.probabilities(lg[r].double().numpy(), **full)
        kept, kept_ref = set(np.nonzero(probs[r])[0]), set(np.nonzero(ref)[0])
        # a candidate exactly at a filter's threshold may fall on either side of a 32-bit sum; nothing else may differ
        assert len(kept ^ kept_ref) <= 1, (r, sorted(kept ^ kept_ref))
        if kept == kept_ref:
            assert np.allclose(probs[r], ref, atol=1e-5), r


def test_draws_walk_the_kept_set_and_follow_u(ops):
    V = 3001
    lg = rand(1, V, seed=5, scale=1.5)
    # without top-k the walk is in index order
    ref = P.probabilities(lg[0].double().numpy(), temperature=0.9, top_p=0.6)
    cdf = np.cumsum(ref)
    for u in (0.0, 0.1, 0.37, 0.5, 0.81, 0.999):
        tok = ops.sample(lg.to(DEV), torch.tensor([u], dtype=F32).to(DEV), 0.9, 0, 0.6, 0.0).item()
        assert ref[tok] > 0
        lo = cdf[tok] - ref[tok]
        assert lo - 1e-4 <= u <= cdf[tok] + 1e-4, (u, tok)
    # many ties at the threshold (logits on a grid of halves): the draw, which searches among a few elements set
    # aside, lands where the kernel's own probabilities (written from the whole row) put u
    tied = torch.round(rand(1, 5003, seed=6, scale=2.0, dtype=F32) * 2) / 2
    for top_p, t in ((0.8, 1.0), (0.35, 0.7), (0.97, 1.3)):
        probs = ops.sample(tied.to(DEV), torch.zeros(1).to(DEV), t, 0, top_p, 0.0, want_probs=True)[1].cpu().double()[0]
        cdf = torch.cumsum(probs, 0)
        for u in (0.0, 0.123, 0.5, 0.77, 0.9999):
            tok = ops.sample(tied.to(DEV), torch.tensor([u], dtype=F32).to(DEV), t, 0, top_p, 0.0).item()
            assert float(probs[tok]) > 0 and float(cdf[tok] - probs[tok]) - 1e-4 <= u <= float(cdf[tok]) + 1e-4, (top_p, t, u, tok)
    # with top-k the walk is over the sorted candidates, as the reference's (engine/sampler.cpp:180-187)
    for u in (0.0, 0.2, 0.55, 0.93, 0.9999):
        tok = ops.sample(lg.to(DEV), torch.tensor([u], dtype=F32).to(DEV), 0.9, 40, 0.95, 0.0).item()
        assert tok == P.draw(lg[0].double().numpy(), u, temperature=0.9, top_k=40, top_p=0.95), u


def test_top_k_where_the_candidates_do_not_stand_out(ops):
    """Rows whose k largest are not a few elements near the top: all equal, half of them equal to the maximum, and
    a maximum far above a flat rest (the kernel's coarse cut does not thin these out, so its slow way runs)."""
    V = 9001
    flat = torch.zeros(V)
    half = rand(V, seed=3, dtype=F32)
    half[::2] = float(half.max()) + 1.0
    spike = rand(V, seed=4, dtype=F32) * 1e-3
    spike[4321] = 500.0
    for lg in (flat, half, spike):
        for k in (1, 5, 300):
            for u in (0.0, 0.3, 0.77, 0.9999):
                tok = ops.sample(lg.reshape(1, -1).to(DEV), torch.tensor([u], dtype=F32).to(DEV), 0.9, k, 1.0, 0.0).item()
                assert tok == P.draw(lg.double().numpy(), u, temperature=0.9, top_k=k), (k, u)


def test_rows_are_sampled_independently(ops):
    lg = rand(4, 2000, seed=8)
    u = torch.tensor([0.1, 0.5, 0.9, 0.3])
    together = ops.sample(lg.to(DEV), u.to(DEV), 1.0, 20, 0.9, 0.0).cpu().tolist()
    alone = [ops.sample(lg[r:r + 1].to(DEV), u[r:r + 1].to(DEV), 1.0, 20, 0.9, 0.0).item() for r in range(4)]
    assert together == alone
    # without top-k, on a wide row of an odd width, and again and again: weights are added as integers, so not
    # a bit depends on the order in which the block's waves arrive
    lg = rand(4, 151937, seed=9, scale=3.0)
    for args in ((0.8, 0, 0.9, 0.0), (1.2, 0, 1.0, 0.02), (1.0, 0, 1.0, 0.0)):
        together = ops.sample(lg.to(DEV), u.to(DEV), *args).cpu().tolist()
        alone = [ops.sample(lg[r:r + 1].to(DEV), u[r:r + 1].to(DEV), *args).item() for r in range(4)]
        assert together == alone and together == ops.sample(lg.to(DEV), u.to(DEV), *args).cpu().tolist(), args
        probs = ops.sample(lg.to(DEV), u.to(DEV), *args, want_probs=True)[1].cpu().double()
        assert all(float(probs[r, together[r]]) > 0 for r in range(4)), args
        for r in range(4):           # the token is where the kept weights, added up in index order, pass u
            cdf = torch.cumsum(probs[r], 0)
            assert float(cdf[together[r]] - probs[r, together[r]]) - 1e-4 <= float(u[r]) <= float(cdf[together[r]]) + 1e-4, (args, r)


def test_penalties(ops):
    lg = torch.tensor([[2.0, -2.0, 1.0, 0.5], [1.0, 1.0, 1.0, 1.0]])
    d = lg.to(DEV)
    i32 = lambda xs: torch.tensor(xs, dtype=torch.int32).to(DEV)
    ops.apply_penalties(d, i32([0, 0, 1]), i32([0, 1, 3]), i32([1, 2, 4]), 2.0, 0.5, 0.25)
    ref0 = P.apply_penalties(lg[0].numpy(), [0, 1, 1], repeat_penalty=2.0, repeat_last_n=-1, presence_penalty=0.5, frequency_penalty=0.25)
    assert np.allclose(d.cpu().numpy()[0], ref0) and np.allclose(d.cpu().numpy()[1], [1, 1, 1, 1 / 2 - 0.5 - 1.0])


def test_sampling_refuses_bad_options(ops):
    from palm_infra_amd.kernels import KernelError
    lg, u = rand(1, 5000).to(DEV), torch.zeros(1).to(DEV)
    with pytest.raises(KernelError, match="temperature"):
        ops.sample(lg, u, 3.0)
    with pytest.raises(KernelError, match="at most 1024"):
        ops.sample(lg, u, 1.0, top_k=2000)
    with pytest.raises(KernelError, match="uniform"):
        ops.sample(lg, None, 1.0)

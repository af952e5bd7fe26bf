"""The matrix-core kernels alone against their plain references: the thin linear product (with and
without the gated epilogue) and the bfloat16 attention kernels, at sizes other than the tiny models'."""

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


def rand(*shape, seed=0, scale=1.0, dtype=BF16):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 33, 64, 70, 128, 150])
@pytest.mark.parametrize("N,K", [(7, 8), (130, 64), (515, 80), (1000, 224), (96, 4096), (4096, 1536), (300, 12288),
                                 (1000, 2048), (515, 2056), (130, 5000), (9000, 2048), (8200, 3080), (64, 8192), (48, 7000),
                                 (4200, 5120)])
def test_linear_thin_against_the_plain_product(ops, M, N, K):
    a, w = rand(M, K, seed=M + K), rand(N, K, seed=N, scale=0.5)
    ref = P.linear(a, w)
    got32 = ops.linear_thin(a.to(DEV), w.to(DEV), F32).cpu()
    # exact products of bfloat16 values, added in 32-bit: only the order of the sum differs
    assert torch.allclose(got32.double(), ref, atol=2e-4 * (K ** 0.5), rtol=1e-5), float((got32.double() - ref).abs().max())
    got16 = ops.linear_thin(a.to(DEV), w.to(DEV), BF16).cpu()
    if 64 < M <= 128 and K % 8 == 0:
        # the float32 result of so many rows comes from the tiled kernel, the bfloat16 one from the kernel that shares
        # up to 128 rows through LDS: sums in another order, so the rounding may fall the other way
        assert torch.allclose(got16.double(), ref, atol=2e-4 * (K ** 0.5), rtol=2.0 ** -8)
    else:
        assert torch.equal(got16, got32.to(BF16))                      # one rounding at the end


@pytest.mark.parametrize("M", [1, 8, 16])
@pytest.mark.parametrize("N,K,planes", [(4096, 4096, 2), (2048, 12288, 3), (1000, 12288, 3), (6144, 4096, 2), (4096, 6000, 2),
                                        (4096, 2048, 2), (16384, 4096, 1), (515, 520, 1), (5120, 17408, 3), (2048, 25600, 4)])
def test_linear_thin_as_planes_of_partial_sums(ops, M, N, K, planes):
    a, w = rand(M, K, seed=M, dtype=BF16), rand(N, K, seed=N + K, dtype=BF16)
    got = ops.linear_thin(a.to(DEV), w.to(DEV), F32, planes_ok=True).cpu()
    want = P.linear(a, w)
    if planes == 1:
        assert got.shape == (M, N)
    else:
        assert got.shape == (planes, M, N) and got.dtype == F32
        assert all(float(got[p].abs().max()) > 0 for p in range(planes))
        got = got.double().sum(0)
    assert torch.allclose(got.double(), want, atol=2e-4 * (K ** 0.5), rtol=1e-5)
    # bfloat16 results and gated products never come in planes
    assert ops.linear_thin(a.to(DEV), w.to(DEV), BF16, planes_ok=False).shape == (M, N)


@pytest.mark.parametrize("M", [17, 40, 64, 65, 100, 128])
@pytest.mark.parametrize("N,K,cut", [(4096, 12288, True), (4096, 4096, True), (6144, 4096, True), (1000, 3000, True),
                                     (24576, 4096, False), (4096, 1000, False), (300, 12296, True)])
def test_linear_for_17_to_128_rows_as_planes_of_partial_sums(ops, M, N, K, cut):
    a, w = rand(M, K, seed=M, dtype=BF16), rand(N, K, seed=N + K, dtype=BF16)
    got = ops.linear_thin(a.to(DEV), w.to(DEV), F32, planes_ok=True).cpu()
    want = P.linear(a, w)
    if cut or (M > 64 and got.dim() == 3):          # (more than 64 rows go by in shorter steps of K, so a short K is cut too)
        assert got.dim() == 3 and 2 <= got.shape[0] <= 4 and got.shape[1:] == (M, N) and got.dtype == F32
        assert all(float(got[p].abs().max()) > 0 for p in range(got.shape[0]))       # no range of K is empty
        got = got.double().sum(0)
    else:
        assert got.shape == (M, N)
    assert torch.allclose(got.double(), want, atol=2e-4 * (K ** 0.5), rtol=1e-5)
    assert ops.linear_thin(a.to(DEV), w.to(DEV), BF16, planes_ok=False).shape == (M, N)


@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("N,K", [(80, 64), (4096, 4096), (1000, 1096), (515, 12288), (8200, 2048), (5120, 5120), (8200, 4224)])
def test_linear_thin_into_the_residual_stream_and_on_with_the_row_factor(ops, M, N, K):
    """A product that adds its result to the residual stream and leaves the next norm's output but for the row
    factor; then a product (plain, in planes, gated) that takes such rows: together they are
    x += a W1^T;  y = rms_norm(x, w) W2^T."""
    eps = 1e-5
    a, w1 = rand(M, K, seed=M), rand(N, K, seed=N, scale=0.1)
    x0, nw = rand(M, N, seed=3, dtype=F32) * 3, rand(N, seed=4, dtype=F32) + 1.0
    xd = x0.to(DEV)
    values, ss = ops.linear_thin_into_residual(a.to(DEV), w1.to(DEV), xd, nw.to(DEV))
    x_ref = x0.double() + P.linear(a, w1)
    assert torch.allclose(xd.cpu().double(), x_ref, atol=2e-4 * (K ** 0.5), rtol=1e-5)          # 32-bit, in place
    assert values.dtype == BF16 and ss.shape == (M, (N + 15) // 16)
    assert torch.allclose(ss.cpu().double().sum(1), (x_ref ** 2).sum(1), rtol=1e-4)
    assert torch.allclose(values.cpu().double(), x_ref * nw.double(), atol=3e-2, rtol=1e-2)
    whole = ops.scale_rows(values, ss, eps).cpu().double()
    normed = P.rms_norm(x_ref, nw.double(), eps)
    assert torch.allclose(whole, normed, atol=3e-2, rtol=1e-2)
    # the reader: the same rows go in with and without their factor
    # (rows whose length is no multiple of 8 go the way of the exact kernel, made whole first)
    for N2, gated in ((96, False), (6144, False), (2 * 176, True), (2 * 4500, True)) if N % 8 == 0 else ():
        w2 = rand(N2, N, seed=N2, scale=0.2)
        for planes_ok in (False, True):
            if gated and planes_ok:
                continue
            got = ops.linear_thin(values, w2.to(DEV), F32, gated=gated, planes_ok=planes_ok, row_ss=ss, row_eps=eps).cpu().double()
            want = ops.linear_thin(ops.scale_rows(values, ss, eps), w2.to(DEV), F32, gated=gated).cpu().double()
            if got.dim() == 3:
                got = got.sum(0)
            scale = float(want.abs().max())
            # scale_rows rounds the rows to bfloat16 once more than the fold does: a few parts in a thousand
            assert torch.allclose(got, want, atol=1.5e-2 * scale), (N2, gated, planes_ok, float((got - want).abs().max()), scale)
    # and both at once: rows without their factor in, residual stream and the next such rows out
    if N % 8 == 0:
        w3 = rand(N, N, seed=9, scale=0.05)
        x1 = xd.clone()
        v2, ss2 = ops.linear_thin_into_residual(values, w3.to(DEV), x1, nw.to(DEV), row_ss=ss, row_eps=eps)
        x1_ref = x_ref + P.linear(normed.to(BF16), w3)
        assert torch.allclose(x1.cpu().double(), x1_ref, atol=2e-2 * float(x1_ref.abs().max()))
        assert torch.allclose(ss2.cpu().double().sum(1), (x1.cpu().double() ** 2).sum(1), rtol=1e-4)


def test_the_folded_norm_refuses_what_it_does_not_serve(ops):
    from palm_infra_amd.kernels import KernelError
    a, w, x, nw = rand(17, 64).to(DEV), rand(32, 64).to(DEV), torch.zeros(17, 32, device=DEV), torch.ones(32, device=DEV)
    with pytest.raises(KernelError, match="16"):
        ops.linear_thin_into_residual(a, w, x, nw)
    with pytest.raises(KernelError, match="residual"):
        ops.linear_thin_into_residual(a[:4].contiguous(), w, x[:4, :8].contiguous(), nw)
    with pytest.raises(KernelError, match="sums of squares"):
        ops.linear_thin(a[:4].contiguous(), w, F32, row_ss=torch.zeros(5, 2, device=DEV), row_eps=1e-6)
    with pytest.raises(KernelError, match="at most 16"):          # the kernel for 17 to 64 rows applies no row factor
        ops.linear_thin(a, w, F32, row_ss=torch.ones(17, 2, device=DEV), row_eps=1e-6)


def test_linear_thin_orientation(ops):
    """One weight row and one token stand out: the product must land at [token, feature], not transposed,
    and every k must be used exactly once."""
    M, N, K = 5, 40, 256
    a, w = torch.zeros(M, K, dtype=BF16), torch.zeros(N, K, dtype=BF16)
    a[3] = torch.arange(K).to(BF16) % 7
    w[29] = 1.0
    w[11, 100] = 2.0
    got = ops.linear_thin(a.to(DEV), w.to(DEV), F32).cpu()
    ref = torch.zeros(M, N)
    ref[3, 29] = float((torch.arange(K) % 7).sum())
    ref[3, 11] = 2.0 * (100 % 7)
    assert torch.equal(got, ref)


@pytest.mark.parametrize("M", [1, 8, 20, 64, 90, 128])
@pytest.mark.parametrize("I,K", [(5, 16), (176, 80), (224, 96), (1536, 512), (4500, 2048), (300, 3000), (100, 6000), (2200, 5120),
                                 (40, 8192)])
def test_linear_thin_gated(ops, M, I, K):
    a, w = rand(M, K, seed=M), rand(2 * I, K, seed=I, scale=0.3)
    g, u = P.linear(a, w[:I]), P.linear(a, w[I:])
    ref = g / (1 + torch.exp(-g)) * u
    got = ops.linear_thin(a.to(DEV), w.to(DEV), F32, gated=True).cpu()
    assert got.shape == (M, I)
    # the two sums are exact products added in 32-bit: an error of about sqrt(K) roundings of their size in each,
    # which silu(g) * u hands on with |u| (silu's slope is at most 1.1) and |silu(g)|
    eps32 = 2.0 ** -24
    err_g, err_u = (4 * eps32 * K ** 0.5 * float(t.abs().max()) for t in (g, u))
    bound = 1.1 * u.abs() * err_g + (g / (1 + torch.exp(-g))).abs() * err_u + 1e-6
    assert bool(((got.double() - ref).abs() <= bound).all()), float(((got.double() - ref).abs() / bound).max())
    swapped = u / (1 + torch.exp(-u)) * g
    assert not torch.allclose(got.double(), swapped, atol=1e-2) or I * M < 8
    got16 = ops.linear_thin(a.to(DEV), w.to(DEV), BF16, gated=True).cpu()
    if M > 64:          # bfloat16 from the kernel for up to 128 rows, float32 from the tiled one: sums in another order
        assert bool(((got16.double() - ref).abs() <= bound + 2.0 ** -8 * ref.abs()).all())
    else:
        assert torch.equal(got16, got.to(BF16))


def test_linear_thin_is_the_same_bits_every_time_and_for_every_companion(ops):
    a, w = rand(40, 1024, seed=1), rand(200, 1024, seed=2)
    ad, wd = a.to(DEV), w.to(DEV)
    first = ops.linear_thin(ad, wd, F32).cpu()
    for _ in range(3):
        assert torch.equal(ops.linear_thin(ad, wd, F32).cpu(), first)
    # a row's result does not depend on which rows are computed with it (within one kernel shape)
    assert torch.equal(ops.linear_thin(a[32:40].contiguous().to(DEV), wd, F32).cpu(),
                       ops.linear_thin(a[25:40].contiguous().to(DEV), wd, F32).cpu()[7:])


def test_linear_thin_falls_back_when_rows_do_not_start_on_16_bytes(ops):
    a, w = rand(3, 12, seed=1), rand(9, 12, seed=2)          # K = 12: the exact kernel takes it
    assert torch.allclose(ops.linear_thin(a.to(DEV), w.to(DEV), F32).cpu().double(), P.linear(a, w), atol=1e-4)
    a32 = rand(3, 16, seed=1, dtype=F32)
    assert torch.allclose(ops.linear_thin(a32.to(DEV), rand(9, 16, seed=2, dtype=F32).to(DEV), F32).cpu().double(),
                          P.linear(a32, rand(9, 16, seed=2, dtype=F32)), atol=1e-4)


# ---- the product for some hundred rows, both operands through rings in LDS -----------------------------

@pytest.mark.parametrize("M", [1, 17, 33, 64, 65, 100, 128, 129, 200, 256, 257, 300, 512, 515])
@pytest.mark.parametrize("N,K", [(96, 64), (7, 128), (1000, 192), (515, 320), (4096, 4096), (300, 12288), (6144, 1024), (8200, 448)])
def test_linear_mid_against_the_plain_product(ops, M, N, K):
    a, w = rand(M, K, seed=M + K), rand(N, K, seed=N, scale=0.5)
    ref = P.linear(a, w)
    got32 = ops.linear_mid(a.to(DEV), w.to(DEV), F32).cpu()
    assert got32.shape == (M, N)
    assert torch.allclose(got32.double(), ref, atol=2e-4 * (K ** 0.5), rtol=1e-5), float((got32.double() - ref).abs().max())
    got16 = ops.linear_mid(a.to(DEV), w.to(DEV), BF16).cpu()
    assert torch.equal(got16, got32.to(BF16))                          # one rounding at the end


@pytest.mark.parametrize("M", [20, 64, 90, 128, 129, 256, 300])
@pytest.mark.parametrize("N,K,cut", [(4096, 12288, True), (4096, 4096, True), (6144, 4096, True), (1000, 3072, True),
                                     (24576, 4096, False), (4096, 448, False)])
def test_linear_mid_as_planes_of_partial_sums(ops, M, N, K, cut):
    a, w = rand(M, K, seed=M), rand(N, K, seed=N + K, scale=0.5)
    got = ops.linear_mid(a.to(DEV), w.to(DEV), F32, planes_ok=True).cpu()
    want = P.linear(a, w)
    parts = ops.core().palm_linear_mid_parts(M, N, K, 0)
    assert parts > 1 if cut else (parts == 1 or M <= 128)       # (few rows may be cut although weight rows are many: whole rounds of blocks)
    if parts > 1:
        assert got.shape == (parts, M, N) and parts <= 4 and got.dtype == F32
        assert all(float(got[p].abs().max()) > 0 for p in range(parts))              # no range of K is empty
        got = got.double().sum(0)
    else:
        assert got.shape == (M, N)
    assert torch.allclose(got.double(), want, atol=2e-4 * (K ** 0.5), rtol=1e-5)
    assert ops.linear_mid(a.to(DEV), w.to(DEV), BF16, planes_ok=False).shape == (M, N)


def test_linear_mid_orientation_and_every_k_once(ops):
    M, N, K = 300, 520, 448
    a, w = torch.zeros(M, K, dtype=BF16), torch.zeros(N, K, dtype=BF16)
    a[3] = (torch.arange(K) % 7).to(BF16)
    a[299, 447] = 3.0
    w[29] = 1.0
    w[511, 100] = 2.0
    w[519, 447] = 5.0
    got = ops.linear_mid(a.to(DEV), w.to(DEV), F32).cpu()
    ref = torch.zeros(M, N)
    ref[3, 29] = float((torch.arange(K) % 7).sum())
    ref[3, 511] = 2.0 * (100 % 7)
    ref[3, 519] = 5.0 * (447 % 7)
    ref[299, 29] = 3.0
    ref[299, 519] = 15.0
    assert torch.equal(got, ref)


@pytest.mark.parametrize("M", [17, 40, 64, 100, 128, 129, 256, 300])
@pytest.mark.parametrize("I,K", [(128, 64), (176, 128), (1536, 512), (4500, 2048), (301, 3008), (12288, 4096)])
def test_linear_mid_gated(ops, M, I, K):
    a, w = rand(M, K, seed=M), rand(2 * I, K, seed=I, scale=0.3)
    g, u = P.linear(a, w[:I]), P.linear(a, w[I:])
    ref = g / (1 + torch.exp(-g)) * u
    got = ops.linear_mid(a.to(DEV), w.to(DEV), BF16, gated=True).cpu()
    assert got.shape == (M, I)
    scale = float(ref.abs().max())
    assert torch.allclose(got.double(), ref, atol=2.0 ** -8 * scale), float((got.double() - ref).abs().max()) / scale
    swapped = u / (1 + torch.exp(-u)) * g
    assert not torch.allclose(got.double(), swapped, atol=1e-2 * scale)


def test_linear_mid_refuses_what_it_does_not_serve(ops):
    from palm_infra_amd.kernels.library import KernelError
    a, w = rand(130, 72).to(DEV), rand(96, 72).to(DEV)
    with pytest.raises((KernelError, ValueError), match="64"):
        ops.linear_mid(a, w, BF16)
    assert not ops.mid_pays(130, 96, 72) and not ops.mid_pays(16, 4096, 4096, planes_ok=True)
    assert not ops.mid_pays(300, 4096, 4096, planes_ok=True)
    assert ops.mid_pays(200, 4096, 4096, planes_ok=True) and not ops.mid_pays(200, 4096, 4096, planes_ok=False)
    assert not ops.mid_pays(200, 24576, 4096, planes_ok=True)           # weight rows enough: no planes, the library's
    # 17 to 128 rows: wherever the blocks fill the chip
    assert ops.mid_pays(64, 24576, 4096, gated=True) and ops.mid_pays(100, 4096, 4096, planes_ok=True)
    assert not ops.mid_pays(100, 4096, 4096, planes_ok=False) and not ops.mid_pays(64, 96, 128)
    assert ops.mid_pays(128, 151936, 4096, out_dtype=F32) and ops.mid_pays(64, 151936, 4096, out_dtype=F32)


def test_a_short_prompts_projections_take_the_kernel_with_rings(ops, monkeypatch):
    """The linear part sends bfloat16 products of 129 to 256 rows to this kernel where its blocks fill the chip, and to
    the library otherwise; either way the result is the plain product."""
    from palm_infra_amd.parts.linear import Linear
    calls = []
    real = ops.linear_mid
    monkeypatch.setattr(ops, "linear_mid", lambda *a, **k: (calls.append(a[0].shape[0]), real(*a, **k))[1])
    w = rand(6144, 1024, seed=1, scale=0.5)
    lin = Linear(w.to(DEV))
    for M, expect in ((200, True), (256, True), (128, True), (40, True), (17, True), (16, False), (257, False)):
        x = rand(M, 1024, seed=M)
        calls.clear()
        got = lin(x.to(DEV), planes_ok=True)
        assert bool(calls) == expect, (M, calls)
        got = got.double().sum(0) if got.dim() == 3 else got.double()
        assert torch.allclose(got.cpu(), P.linear(x, w), atol=2e-4 * 32 + 2.0 ** -8 * float(P.linear(x, w).abs().max()))


# ---- the tiled product for many rows -----------------------------------------------------------------

@pytest.mark.parametrize("M", [65, 128, 130, 257, 700])
@pytest.mark.parametrize("N,K", [(256, 64), (1000, 128), (515, 192), (4096, 4096), (300, 12288), (6144, 1024), (8200, 320)])
def test_linear_tile_against_the_plain_product(ops, M, N, K):
    a, w = rand(M, K, seed=M + K), rand(N, K, seed=N, scale=0.5)
    ref = P.linear(a, w)
    got32 = ops.linear_tile(a.to(DEV), w.to(DEV), F32).cpu()
    assert got32.shape == (M, N)
    assert torch.allclose(got32.double(), ref, atol=2e-4 * (K ** 0.5), rtol=1e-5), float((got32.double() - ref).abs().max())
    got16 = ops.linear_tile(a.to(DEV), w.to(DEV), BF16).cpu()
    assert torch.equal(got16, got32.to(BF16))                          # one rounding at the end
    # and through the dispatcher: a float32 result for more than 64 rows takes this kernel
    assert torch.equal(ops.linear_thin(a.to(DEV), w.to(DEV), F32).cpu(), got32)


@pytest.mark.parametrize("M", [70, 256, 300])
@pytest.mark.parametrize("N,K,cut", [(4096, 12288, True), (4096, 4096, True), (1000, 3072, True), (24576, 4096, False),
                                     (4096, 1024, False)])
def test_linear_tile_as_planes_of_partial_sums(ops, M, N, K, cut):
    """Few tiles and a long K: K is cut into ranges, each block writes its range's sums to a float32 plane, and the
    planes add up to the product; a product with tiles enough comes whole."""
    a, w = rand(M, K, seed=M), rand(N, K, seed=N + K, scale=0.5)
    got = ops.linear_tile(a.to(DEV), w.to(DEV), F32, planes_ok=True).cpu()
    want = P.linear(a, w)
    parts = ops.core().palm_linear_tile_parts(M, N, K)
    assert parts > 1 if cut else parts >= 1
    if parts > 1:
        assert got.shape == (parts, M, N) and parts <= 4 and got.dtype == F32
        assert all(float(got[p].abs().max()) > 0 for p in range(parts))              # no range of K is empty
        got = got.double().sum(0)
    else:
        assert got.shape == (M, N)
    assert torch.allclose(got.double(), want, atol=2e-4 * (K ** 0.5), rtol=1e-5)
    assert ops.linear_tile(a.to(DEV), w.to(DEV), BF16, planes_ok=False).shape == (M, N)


def test_linear_tile_orientation_and_every_k_once(ops):
    M, N, K = 300, 520, 256
    a, w = torch.zeros(M, K, dtype=BF16), torch.zeros(N, K, dtype=BF16)
    a[3] = torch.arange(K).to(BF16) % 7
    a[299, 255] = 3.0
    w[29] = 1.0
    w[511, 100] = 2.0
    w[519, 255] = 5.0
    got = ops.linear_tile(a.to(DEV), w.to(DEV), F32).cpu()
    ref = torch.zeros(M, N)
    ref[3, 29] = float((torch.arange(K) % 7).sum())
    ref[3, 511] = 2.0 * (100 % 7)
    ref[3, 519] = 5.0 * (255 % 7)
    ref[299, 29] = 3.0
    ref[299, 519] = 15.0
    assert torch.equal(got, ref)


def test_linear_tile_refuses_what_it_does_not_serve(ops):
    from palm_infra_amd.kernels import KernelError
    with pytest.raises(KernelError, match="multiple of 64"):
        ops.linear_tile(rand(70, 72).to(DEV), rand(32, 72).to(DEV), F32)
    with pytest.raises(KernelError, match="bfloat16"):
        ops.linear_tile(rand(70, 64, dtype=F32).to(DEV), rand(32, 64).to(DEV), F32)
    # the dispatcher takes the other way where this kernel does not serve
    a, w = rand(70, 72), rand(40, 72)
    assert torch.allclose(ops.linear_thin(a.to(DEV), w.to(DEV), F32).cpu().double(), P.linear(a, w), atol=2e-3)


# ---- attention on the matrix cores ------------------------------------------------------------------

from test_kernels import _attention_case, _fill_cache, _poison, _spike_case  # noqa: E402  (the cases and the cache filling are shared)


def decode_fn(ops, n_slices):
    def fn(q, kc, vc, table, slots, starts, news, cu, max_new, nh, nkv, hd, scale, window):
        assert max_new == 1
        return ops.attention_decode(q, kc, vc, table, slots, starts, nh, nkv, hd, scale, window, n_slices)
    return fn


# 192 and 112: rows of 24 and 14 chunks, which do not divide an instruction's 64 (a page must then go through
# registers into LDS); 144 and 240: two pages that need more LDS than the smaller sizes
HEADS = [(8, 4, 16), (5, 5, 48), (6, 1, 80), (4, 2, 128), (32, 8, 128), (40, 2, 32), (3, 3, 256), (4, 2, 192), (6, 3, 112),
         (2, 1, 144), (2, 2, 240)]


@pytest.mark.parametrize("nh,nkv,hd", HEADS)
def test_attention_prefill_mfma(ops, nh, nkv, hd):
    # whole prompts, a prompt's continuation (past > 0), single tokens among prompts, tails that fill no tile
    cases = [[(20, 20)], [(256, 256)], [(1, 1)], [(300, 44)], [(64, 64), (65, 1), (130, 70), (7, 7), (200, 17)]]
    for lens in cases:
        got, ref = _attention_case(ops, ops.attention_prefill, BF16, nh, nkv, hd, lens, None, seed=len(lens) + hd)
        assert torch.allclose(got, ref, atol=2e-2), (lens, float((got - ref).abs().max()))


@pytest.mark.parametrize("nh,nkv,hd", HEADS)
@pytest.mark.parametrize("n_slices", [1, 3, 8])
def test_attention_decode_mfma(ops, nh, nkv, hd, n_slices):
    for lens in ([(300, 1)], [(1, 1)], [(64, 1), (65, 1), (700, 1), (7, 1), (128, 1)]):
        got, ref = _attention_case(ops, decode_fn(ops, n_slices), BF16, nh, nkv, hd, lens, None, seed=len(lens) + hd)
        assert torch.allclose(got, ref, atol=2e-2), (lens, float((got - ref).abs().max()))


@pytest.mark.parametrize("nh,nkv,hd", [(32, 8, 128), (6, 3, 64), (2, 1, 128), (3, 3, 64)])
def test_attention_prefill_with_the_scale_folded_into_the_queries(ops, nh, nkv, hd):
    """The prompt kernel of the head sizes 64 and 128 takes queries that come multiplied by scale * log2(e): the
    same attention as with plain queries and the scale applied inside.  (Other head sizes say that they do not.)"""
    assert ops.prefill_q_scale(hd, BF16, 0.25) == pytest.approx(0.25 * 1.4426950408889634)
    assert ops.prefill_q_scale(80, BF16, 0.25) == 1.0 and ops.prefill_q_scale(hd, F32, 0.25) == 1.0

    def folded(q, kc, vc, table, slots, starts, news, cu, max_new, nh_, nkv_, hd_, scale, window):
        qs = (q.float() * ops.prefill_q_scale(hd, BF16, scale)).to(BF16)
        return ops.attention_prefill(qs, kc, vc, table, slots, starts, news, cu, max_new, nh, nkv, hd, scale, window, q_prescaled=True)
    for window in (None, 70):
        for lens in ([(20, 20)], [(300, 44)], [(64, 64), (65, 1), (130, 70), (7, 7), (200, 17)], [(1100, 1100)], [(2304, 300), (70, 70)]):
            got, ref = _attention_case(ops, folded, BF16, nh, nkv, hd, lens, window, seed=len(lens) + hd, poison=True)
            assert torch.isfinite(got).all() and torch.allclose(got, ref, atol=3e-2), (lens, window, float((got - ref).abs().max()))
    from palm_infra_amd.kernels import KernelError
    with pytest.raises(KernelError, match="applies the scale itself"):
        _attention_case(ops, lambda q, kc, vc, table, slots, starts, news, cu, max_new, a, b, c, scale, window: ops.attention_prefill(
            q, kc, vc, table, slots, starts, news, cu, max_new, 6, 1, 80, scale, window, q_prescaled=True), BF16, 6, 1, 80, [(20, 20)], None)


@pytest.mark.parametrize("nh,nkv,hd", [(32, 8, 128), (4, 2, 64), (6, 1, 80)])
def test_attention_mfma_long_sequences(ops, nh, nkv, hd):
    """The measured lengths and beyond: a 2,048-token prompt (32 pages, query tiles paired from both ends, a
    running maximum that is followed only now and then), a prompt's continuation far into a sequence, unequal
    prompts together, and single queries over thousands of keys in few and in many slices."""
    for lens in ([(2048, 2048)], [(4100, 1000)], [(1500, 1500), (70, 70), (2304, 300)]):
        got, ref = _attention_case(ops, ops.attention_prefill, BF16, nh, nkv, hd, lens, None, seed=len(lens) + hd)
        assert torch.allclose(got, ref, atol=2e-2), (lens, float((got - ref).abs().max()))
    for n_slices in (2, 12, 64):
        got, ref = _attention_case(ops, decode_fn(ops, n_slices), BF16, nh, nkv, hd, [(5000, 1), (2049, 1), (3, 1)], None, seed=hd)
        assert torch.allclose(got, ref, atol=2e-2), (n_slices, float((got - ref).abs().max()))


@pytest.mark.parametrize("window", [1, 5, 64, 100, 1000])
def test_attention_mfma_window(ops, window):
    got, ref = _attention_case(ops, ops.attention_prefill, BF16, 4, 2, 32, [(200, 200), (150, 1), (70, 3), (90, 30)], window, seed=window)
    assert torch.allclose(got, ref, atol=2e-2), float((got - ref).abs().max())
    for n_slices in (1, 4):
        got, ref = _attention_case(ops, decode_fn(ops, n_slices), BF16, 4, 2, 32, [(200, 1), (150, 1), (3, 1)], window, seed=window)
        assert torch.allclose(got, ref, atol=2e-2), (n_slices, float((got - ref).abs().max()))


def test_attention_mfma_finds_a_far_key_and_respects_the_window_edge(ops):
    for fn in (ops.attention_prefill, decode_fn(ops, 1), decode_fn(ops, 5)):
        for L, at in ((700, 13), (700, 0), (700, 699), (513, 448), (64, 63), (65, 64), (129, 31)):
            got, v = _spike_case(ops, fn, BF16, L, at)
            assert torch.allclose(got, v[at, 0].float().expand(2, -1), atol=1e-2), (L, at)
        for hd in (192, 112):
            got, v = _spike_case(ops, fn, BF16, 200, 77, hd=hd)
            assert torch.allclose(got, v[77, 0].float().expand(2, -1), atol=1e-2), hd
        L, w = 300, 70
        got, v = _spike_case(ops, fn, BF16, L, L - w, window=w)
        assert torch.allclose(got, v[L - w, 0].float().expand(2, -1), atol=1e-2)
        got, v = _spike_case(ops, fn, BF16, L, L - w - 1, window=w)
        assert not torch.allclose(got, v[L - w - 1, 0].float().expand(2, -1), atol=0.2)


@pytest.mark.parametrize("nh,nkv,hd", [(32, 8, 128), (6, 3, 64), (6, 1, 80), (3, 3, 256), (4, 2, 192), (40, 2, 32)])
def test_attention_mfma_takes_nothing_from_what_lies_beyond_a_sequence(ops, nh, nkv, hd):
    """Pages are handed out uncleared, and a key beyond a sequence's length has weight zero: but zero times the NaN
    or the infinity that an earlier request may have left as its value is NaN.  Every place of the cache that
    belongs to no sequence is filled with NaN and infinities; the outputs must be finite and right.  (Every head
    size's way of bringing a page into LDS, prompts whose last page is partly filled and exactly filled, a
    continuation, single queries in one and in several slices, with and without a window.)"""
    prompts = [[(20, 20)], [(64, 64)], [(1, 1)], [(300, 44)], [(64, 64), (65, 1), (130, 70), (7, 7), (200, 17), (129, 129)]]
    for window in (None, 70):
        for lens in prompts:
            got, ref = _attention_case(ops, ops.attention_prefill, BF16, nh, nkv, hd, lens, window, seed=len(lens) + hd, poison=True)
            assert torch.isfinite(got).all(), (lens, window)
            assert torch.allclose(got, ref, atol=2e-2), (lens, window, float((got - ref).abs().max()))
        for n_slices in (1, 3, 8):
            for lens in ([(300, 1)], [(1, 1)], [(64, 1), (65, 1), (700, 1), (7, 1), (128, 1)]):
                got, ref = _attention_case(ops, decode_fn(ops, n_slices), BF16, nh, nkv, hd, lens, window, seed=len(lens) + hd, poison=True)
                assert torch.isfinite(got).all(), (lens, window, n_slices)
                assert torch.allclose(got, ref, atol=2e-2), (lens, window, n_slices, float((got - ref).abs().max()))


def test_attention_decode_reads_no_record_of_a_slice_without_pages(ops):
    """A step is cut into slices for its longest sequence; a shorter sequence's last slices hold no page, write no
    record, and the merge must read none of theirs: the workspace is handed in full of NaN."""
    nh, nkv, hd = 8, 2, 64
    for n_slices in (4, 9, 40):
        def fn(q, kc, vc, table, slots, starts, news, cu, max_new, nh_, nkv_, hd_, scale, window):
            work = torch.full((q.shape[0] * nh * n_slices * (hd + 4),), float("nan"), device=DEV)
            return ops.attention_decode(q, kc, vc, table, slots, starts, nh, nkv, hd, scale, window, n_slices, work=work)
        for window in (None, 100):
            got, ref = _attention_case(ops, fn, BF16, nh, nkv, hd, [(2000, 1), (3, 1), (65, 1), (700, 1)], window, seed=n_slices)
            assert torch.isfinite(got).all() and torch.allclose(got, ref, atol=2e-2), (n_slices, window)


def test_attention_mfma_agrees_with_the_exact_kernel_on_the_same_cache(ops):
    """Both read the same cache (keys as rows, values transposed): the layouts cannot drift apart."""
    got_m, ref = _attention_case(ops, ops.attention_prefill, BF16, 8, 2, 64, [(190, 190), (64, 5)], None, seed=3)
    got_e, _ = _attention_case(ops, ops.attention_exact, BF16, 8, 2, 64, [(190, 190), (64, 5)], None, seed=3)
    assert torch.allclose(got_m, got_e, atol=2e-2) and torch.allclose(got_e, ref, atol=2e-2)


def test_attention_mfma_refuses_what_it_was_not_built_for(ops):
    from palm_infra_amd.kernels import KernelError
    with pytest.raises(KernelError, match="steps of 16"):
        ops.attention_lib(24)
    q = torch.zeros(1, 2 * 32, dtype=F32, device=DEV)
    kc, vc = torch.zeros(2, 1, 64, 32, dtype=F32, device=DEV), torch.zeros(2, 1, 32, 64, dtype=F32, device=DEV)
    i32 = lambda xs: torch.tensor(xs, dtype=torch.int32).to(DEV)
    with pytest.raises(KernelError, match="bfloat16"):
        ops.attention_decode(q, kc, vc, i32([[0, 1]]), i32([0]), i32([3]), 2, 1, 32, 1.0, None, 1)


# ---- decode attention that starts from the joined projection's rows -----------------------------------

def _fused_case(ops, nh, nkv, hd, lengths, n_slices, planes, window=None, norm=True, rotate=True, seed=0, poison=False):
    """Sequences whose last token is new: its q/k/v row goes (a) through qk_norm_rope_store and attention_decode and
    (b) through attention_decode_fused, each on its own copy of a cache that holds the earlier tokens and stale
    values elsewhere.  Returns both outputs and both pairs of caches."""
    B, W = len(lengths), (nh + 2 * nkv) * hd
    n_pages = sum((L + 63) // 64 for L in lengths) + 2
    perm = torch.randperm(n_pages - 1, generator=torch.Generator().manual_seed(seed)).tolist()
    max_pages = max((L + 63) // 64 for L in lengths) + 1
    slots = torch.randperm(B + 3, generator=torch.Generator().manual_seed(seed + 7)).tolist()[:B]
    table = torch.full((B + 3, max_pages), n_pages - 1, dtype=torch.int32)
    kc = rand(n_pages, nkv, 64, hd, seed=seed + 50).to(DEV)
    vc = rand(n_pages, nkv, hd, 64, seed=seed + 51).to(DEV)
    if poison:
        _poison(kc), _poison(vc)
    o = 0
    for b, L in enumerate(lengths):
        npg = (L + 63) // 64
        table[slots[b], :npg] = torch.tensor(perm[o:o + npg], dtype=torch.int32)
        o += npg
        if L > 1:
            _fill_cache(kc, vc, table, slots[b], rand(L - 1, nkv, hd, seed=seed + 10 * b + 1).to(DEV),
                        rand(L - 1, nkv, hd, seed=seed + 10 * b + 2).to(DEV))
    if planes == 0:
        qkv = rand(B, W, seed=seed + 3, scale=1.5).to(DEV)
    else:
        qkv = rand(planes, B, W, seed=seed + 3, scale=1.5, dtype=F32).to(DEV)
    i32 = lambda xs: torch.tensor(xs, dtype=torch.int32).to(DEV)
    pos, slot = i32([L - 1 for L in lengths]), i32(slots)
    kw = dict(q_norm_w=(1 + 0.3 * rand(hd, seed=seed + 4, dtype=F32)).to(DEV) if norm else None,
              k_norm_w=(1 + 0.3 * rand(hd, seed=seed + 5, dtype=F32)).to(DEV) if norm else None, eps=1e-5 if norm else 0.0)
    if rotate:
        inv = torch.from_numpy((1.0 / np.power(10000.0, np.arange(hd // 2, dtype=np.float32) * 2 / hd)).astype(np.float32))
        cos, sin = ops.rope_table(pos, inv.to(DEV))
        kw.update(cos=cos, sin=sin, rotary_dim=hd, pairing=0)
    ka, va, kb, vb = kc.clone(), vc.clone(), kc.clone(), vc.clone()
    tab = table.to(DEV)
    apart = torch.cat([qkv, torch.zeros_like(qkv)]) if planes == 1 else qkv          # the pass alone takes two planes or more
    q = ops.qk_norm_rope_store(apart, nh, nkv, hd, pos, k_cache=ka, v_cache=va, block_table=tab, tok_slot=slot, out_dtype=BF16, **kw)
    two = ops.attention_decode(q, ka, va, tab, slot, pos, nh, nkv, hd, hd ** -0.5, window, n_slices)
    one = ops.attention_decode_fused(qkv, kb, vb, tab, slot, pos, nh, nkv, hd, hd ** -0.5, window, n_slices, **kw)
    return one.float().cpu(), two.float().cpu(), (ka.cpu(), va.cpu()), (kb.cpu(), vb.cpu()), (kc.cpu(), vc.cpu())


def _one_ulp(a, b):
    """Both are rounded to bfloat16 from sums made in another order: a step of the last bit (2^-8 of the value, and
    values here reach 8) on top of the attention kernels' own tolerance."""
    return torch.allclose(a, b, rtol=2 ** -7, atol=2e-2)


def _same_caches(a, b):
    """Keys and values written by the two paths: the same but for an element's last bit now and then (the sums of
    squares are added in another order)."""
    for x, y in zip(a, b):
        x, y = x.float(), y.float()
        assert torch.allclose(x, y, rtol=2 ** -7, atol=1e-6), float((x - y).abs().max())
        assert float((x != y).float().mean()) < 1e-3


@pytest.mark.parametrize("nh,nkv,hd", [(4, 2, 128), (32, 8, 128), (6, 3, 64), (40, 2, 64), (3, 3, 256), (4, 1, 192)])
@pytest.mark.parametrize("n_slices", [1, 3, 8])
def test_attention_decode_fused_is_the_two_kernels_in_one(ops, nh, nkv, hd, n_slices):
    """Lengths around page borders (the new token first in its page, last in it, the only one of its sequence), rows
    as bfloat16 and as one to five planes."""
    for planes, lengths in ((0, [300]), (1, [1]), (2, [64, 65, 700, 7, 128, 129, 1]), (3, [193, 2]), (4, [130, 64, 1]), (5, [66])):
        one, two, ca, cb, before = _fused_case(ops, nh, nkv, hd, lengths, n_slices, planes, seed=hd + planes)
        assert _one_ulp(one, two), (planes, lengths, float((one - two).abs().max()))
        _same_caches(ca, cb)
        assert not torch.equal(cb[0], before[0]) and not torch.equal(cb[1], before[1])      # it did write


def test_attention_decode_fused_takes_nothing_from_what_lies_beyond_a_sequence(ops):
    """As for the other attention kernels: NaN and infinities wherever the cache belongs to no sequence, also at the
    new token's own place, which the kernel may read before or after it writes it."""
    for nh, nkv, hd in ((32, 8, 128), (6, 3, 64), (3, 3, 256)):
        for n_slices in (1, 3, 8):
            for window in (None, 70):
                one, two, *_ = _fused_case(ops, nh, nkv, hd, [64, 65, 700, 7, 128, 129, 1, 300], n_slices, 2, window=window,
                                           seed=hd, poison=True)
                assert torch.isfinite(one).all() and torch.isfinite(two).all(), (hd, n_slices, window)
                assert _one_ulp(one, two), (hd, n_slices, window, float((one - two).abs().max()))


def test_attention_decode_fused_with_a_window_without_norm_and_without_rotation(ops):
    for window in (1, 5, 64, 100):
        for n_slices in (1, 4):
            one, two, ca, cb, _ = _fused_case(ops, 4, 2, 64, [200, 150, 3, 65], n_slices, 2, window=window, seed=window)
            assert _one_ulp(one, two), (window, n_slices, float((one - two).abs().max()))
            _same_caches(ca, cb)
    for norm, rotate in ((False, True), (True, False), (False, False)):
        one, two, ca, cb, _ = _fused_case(ops, 8, 2, 128, [200, 64, 65], 3, 2, norm=norm, rotate=rotate, seed=9)
        assert _one_ulp(one, two), (norm, rotate, float((one - two).abs().max()))
        _same_caches(ca, cb)


def test_attention_decode_fused_sees_its_own_key_and_leaves_a_read_only_cache_alone(ops):
    """The new token's key is made to dominate: the output is its value, which only the step's row holds.  A layer
    that reads another layer's cache writes nothing and reads the position from the cache."""
    nh, nkv, hd = 4, 2, 128
    W = (nh + 2 * nkv) * hd
    i32 = lambda xs: torch.tensor(xs, dtype=torch.int32).to(DEV)
    for L in (1, 64, 65, 300):
        for n_slices in (1, 4):
            table = torch.arange((L + 63) // 64 + 1, dtype=torch.int32).flip(0)[None, :].contiguous()
            kc, vc = 0.1 * rand(table.shape[1], nkv, 64, hd, seed=1), rand(table.shape[1], nkv, hd, 64, seed=2)
            row = 0.1 * rand(1, W, seed=3)
            row[0, : (nh + nkv) * hd].reshape(nh + nkv, hd)[:, 5] = 8.0          # every q and k head: one large element
            kd, vd = kc.to(DEV), vc.to(DEV)
            got = ops.attention_decode_fused(row.to(DEV), kd, vd, table.to(DEV), i32([0]), i32([L - 1]), nh, nkv, hd, 1.0, None, n_slices)
            v_new = row[0, (nh + nkv) * hd:].reshape(nkv, hd).float()
            want = v_new.repeat_interleave(nh // nkv, 0).reshape(1, nh * hd)
            assert torch.allclose(got.float().cpu(), want, atol=1e-2), (L, n_slices)
            page = int(table[0, (L - 1) // 64])
            assert torch.equal(vd[page, :, :, (L - 1) % 64].cpu(), row[0, (nh + nkv) * hd:].reshape(nkv, hd))
            assert torch.equal(kd[page, :, (L - 1) % 64].cpu(), row[0, nh * hd:(nh + nkv) * hd].reshape(nkv, hd))
            # read only: the cache as the writing call left it gives the same result, and stays as it is
            k2, v2 = kd.clone(), vd.clone()
            other = 0.1 * rand(1, W, seed=4)
            other[0, : nh * hd] = row[0, : nh * hd]
            again = ops.attention_decode_fused(other.to(DEV), k2, v2, table.to(DEV), i32([0]), i32([L - 1]), nh, nkv, hd, 1.0, None,
                                               n_slices, write_cache=False)
            assert torch.allclose(again.float().cpu(), want, atol=1e-2)
            assert torch.equal(k2, kd) and torch.equal(v2, vd)


def test_attention_decode_fused_says_what_it_serves(ops):
    from palm_infra_amd.kernels import KernelError
    planes = torch.zeros(2, 1, 4 * 128, dtype=F32, device=DEV)
    assert ops.decode_fused_serves(planes, 128, BF16, 128, 0) and ops.decode_fused_serves(planes, 64, BF16, 0, 0)
    assert not ops.decode_fused_serves(planes, 128, BF16, 64, 0)          # a rotation over half the head
    assert not ops.decode_fused_serves(planes, 128, BF16, 128, 1)         # pairs side by side
    assert not ops.decode_fused_serves(planes, 80, BF16, 80, 0)           # a pair would lie in two lanes
    assert not ops.decode_fused_serves(planes, 128, F32, 128, 0)
    qkv = torch.zeros(1, 4 * 80, dtype=BF16, device=DEV)
    kc, vc = torch.zeros(2, 1, 64, 80, dtype=BF16, device=DEV), torch.zeros(2, 1, 80, 64, dtype=BF16, device=DEV)
    i32 = lambda xs: torch.tensor(xs, dtype=torch.int32).to(DEV)
    with pytest.raises(KernelError, match="multiple of 64"):
        ops.attention_decode_fused(qkv, kc, vc, i32([[0, 1]]), i32([0]), i32([3]), 2, 1, 80, 1.0, None, 1)


def test_attention_decode_fused_finds_a_far_key_and_respects_the_window_edge(ops):
    """One cached key among hundreds dominates the new token's query (the new token's own key does not): the output
    is that key's value, wherever it lies (first, last before the new one, on a page's border, in any slice); just
    outside a window it is out of reach."""
    nh, nkv, hd = 4, 2, 128
    W = (nh + 2 * nkv) * hd
    i32 = lambda xs: torch.tensor(xs, dtype=torch.int32).to(DEV)

    def run(L, at, n_slices, window=None):
        k = rand(L - 1, nkv, hd, seed=1, scale=0.1)
        v = rand(L - 1, nkv, hd, seed=2)
        k[at] = 0
        k[at, :, 5] = 8.0
        row = rand(1, W, seed=3, scale=0.1)
        row[0, : nh * hd].reshape(nh, hd)[:, 5] = 8.0                    # every query head looks for element 5
        table = torch.arange((L + 63) // 64 + 1, dtype=torch.int32).flip(0)[None, :].contiguous()
        kc = rand(table.shape[1], nkv, 64, hd, seed=4).to(DEV)           # stale values everywhere else
        vc = rand(table.shape[1], nkv, hd, 64, seed=5).to(DEV)
        _fill_cache(kc, vc, table, 0, k.to(DEV), v.to(DEV))
        got = ops.attention_decode_fused(row.to(DEV), kc, vc, table.to(DEV), i32([0]), i32([L - 1]), nh, nkv, hd, 1.0, window,
                                         n_slices)
        return got.float().cpu().reshape(nh, hd), v[at].float().repeat_interleave(nh // nkv, 0)

    for n_slices in (1, 5):
        for L, at in ((700, 13), (700, 0), (700, 698), (513, 448), (65, 63), (66, 64), (130, 31), (2, 0)):
            got, want = run(L, at, n_slices)
            assert torch.allclose(got, want, atol=1e-2), (L, at, n_slices)
        L, w = 300, 70                                                   # the query sits at L-1 and reads keys L-w .. L-1
        got, want = run(L, L - w, n_slices, window=w)
        assert torch.allclose(got, want, atol=1e-2), n_slices
        got, want = run(L, L - w - 1, n_slices, window=w)
        assert not torch.allclose(got, want, atol=0.2), n_slices

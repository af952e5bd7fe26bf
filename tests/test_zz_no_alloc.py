"""The decode attention entry point that allocates nothing (``palm_attention_decode_static``), called through
ctypes as a caller without torch would call it, against the existing entry point with a workspace of the
caller's and against a plain computation of the same attention: two calls in a row on one stream, the second with a
smaller input (fewer sequences, fewer slices), so that what the first call left in the library's buffer must not show
in the second's result; then a request beyond the buffer's limit, which must be refused before anything is launched."""
import ctypes
from ctypes import c_float, c_int, c_longlong, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF16 = torch.bfloat16

ARGS_STATIC = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
               c_float, c_int, c_int, c_void_p]
ARGS_WORK = ARGS_STATIC[:-1] + [c_void_p, c_void_p]


def load(hd):
    from palm_infra_amd.kernels import library
    lib = ctypes.CDLL(str(library.build(f"attention_hd{hd}")))       # a handle of the test's own, by the file's path
    lib.palm_attention_decode_static.argtypes, lib.palm_attention_decode_static.restype = ARGS_STATIC, c_int
    lib.palm_attention_decode.argtypes, lib.palm_attention_decode.restype = ARGS_WORK, c_int
    lib.palm_attention_decode_static_limit.restype = c_longlong
    lib.palm_last_error.restype = ctypes.c_char_p
    return lib


def case(n_seqs, nh, nkv, hd, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    pages_of = [(L + 63) // 64 for L in lengths]
    n_pages = sum(pages_of) + 1
    max_pages = max(pages_of)
    perm = torch.randperm(n_pages, generator=g).tolist()
    table = torch.full((n_seqs, max_pages), perm[-1], dtype=torch.int32)
    o = 0
    for b, n in enumerate(pages_of):
        table[b, :n] = torch.tensor(perm[o:o + n], dtype=torch.int32)
        o += n
    kc = torch.randn(n_pages, nkv, 64, hd, generator=g).to(BF16).to(DEV)
    vc = torch.randn(n_pages, nkv, hd, 64, generator=g).to(BF16).to(DEV)
    q = (torch.randn(n_seqs, nh * hd, generator=g) * 2).to(BF16).to(DEV)
    slots = torch.arange(n_seqs, dtype=torch.int32).to(DEV)
    starts = torch.tensor([L - 1 for L in lengths], dtype=torch.int32).to(DEV)
    return q, kc, vc, table.to(DEV), max_pages, slots, starts


def plain(q, kc, vc, table, lengths, nh, nkv, hd):
    """One query a sequence (at its last position) over the keys of its pages, in 64-bit: softmax(q.k / sqrt(hd)) v,
    head h reading kv head h // (nh / nkv)."""
    q, kc, vc, table = q.cpu().double(), kc.cpu().double(), vc.cpu().double(), table.cpu()
    out = torch.zeros(len(lengths), nh, hd, dtype=torch.float64)
    for b, L in enumerate(lengths):
        pages = table[b, :(L + 63) // 64].long()
        k = kc[pages].permute(1, 0, 2, 3).reshape(nkv, -1, hd)[:, :L]              # [nkv, L, hd]
        v = vc[pages].permute(1, 2, 0, 3).reshape(nkv, hd, -1)[:, :, :L]           # values are kept transposed
        for h in range(nh):
            g = h // (nh // nkv)
            w = torch.softmax(k[g] @ q[b].reshape(nh, hd)[h] * hd ** -0.5, dim=0)
            out[b, h] = v[g] @ w
    return out.reshape(len(lengths), nh * hd)


def run_both(lib, n_seqs, nh, nkv, hd, lengths, n_slices, seed):
    q, kc, vc, table, max_pages, slots, starts = case(n_seqs, nh, nkv, hd, lengths, seed)
    stream = torch.cuda.current_stream().cuda_stream
    scale = hd ** -0.5
    out_static = torch.full_like(q, float("nan"))
    out_work = torch.full_like(q, float("nan"))
    work = torch.empty(n_seqs * nh * n_slices * (hd + 4), dtype=torch.float32, device=DEV)
    common = (stream, q.data_ptr(), kc.data_ptr(), vc.data_ptr(), table.data_ptr(), max_pages, slots.data_ptr(),
              starts.data_ptr(), n_seqs, nh, nkv, hd, scale, 0, n_slices)
    rc = lib.palm_attention_decode_static(*common, out_static.data_ptr())
    assert rc == 0, lib.palm_last_error().decode()
    rc = lib.palm_attention_decode(*common, work.data_ptr(), out_work.data_ptr())
    assert rc == 0, lib.palm_last_error().decode()
    torch.cuda.synchronize()
    return out_static.cpu(), out_work.cpu(), plain(q, kc, vc, table, lengths, nh, nkv, hd)


@pytest.mark.parametrize("nh,nkv,hd", [(32, 8, 128), (6, 3, 64)])
def test_decode_attention_without_a_workspace_argument(nh, nkv, hd):
    lib = load(hd)
    # the first call fills much of the buffer; the second is smaller in every way and reuses its beginning
    a_static, a_work, a_plain = run_both(lib, 9, nh, nkv, hd, [700, 64, 65, 1, 2049, 300, 128, 4000, 17], 12, seed=1)
    b_static, b_work, b_plain = run_both(lib, 3, nh, nkv, hd, [130, 5, 1000], 5, seed=2)
    for got, want, ref in ((a_static, a_work, a_plain), (b_static, b_work, b_plain)):
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got, want)                                            # the same bits through either door
        assert torch.allclose(got.double(), ref, atol=2e-2), float((got.double() - ref).abs().max())      # and the right ones
    # one slice: no buffer is touched at all
    c_static, c_work, c_plain = run_both(lib, 2, nh, nkv, hd, [90, 200], 1, seed=3)
    assert torch.equal(c_static, c_work) and torch.allclose(c_static.double(), c_plain, atol=2e-2)


def test_a_request_beyond_the_buffer_is_refused_and_nothing_runs():
    hd, nh, nkv = 128, 32, 8
    lib = load(hd)
    limit = lib.palm_attention_decode_static_limit()
    assert limit == 2 * 1024 * 1024
    n_seqs, n_slices = 64, 16
    assert n_seqs * nh * n_slices * (hd + 4) > limit
    q, kc, vc, table, max_pages, slots, starts = case(n_seqs, nh, nkv, hd, [70] * n_seqs, seed=4)
    out = torch.full_like(q, 7.0)
    rc = lib.palm_attention_decode_static(torch.cuda.current_stream().cuda_stream, q.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                          table.data_ptr(), max_pages, slots.data_ptr(), starts.data_ptr(), n_seqs, nh, nkv, hd,
                                          hd ** -0.5, 0, n_slices, out.data_ptr())
    torch.cuda.synchronize()
    assert rc != 0 and b"exceed" in lib.palm_last_error()
    assert bool((out == 7.0).all())                                   # nothing was launched

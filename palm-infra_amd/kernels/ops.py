"""The kernels as functions on torch tensors.

Every function checks on the host what its kernel assumes (device, element types, contiguity, shapes
that fit each other) before it launches anything, and launches on torch's current stream.  Tensors
are memory here; the one computation that torch does on the product path is the library matrix product of
``linear_library`` (bfloat16 products of more rows than the kernels here stream weights past).
"""
from __future__ import annotations

from ctypes import c_float, c_int, c_longlong, c_ulonglong, c_void_p

import torch

from . import library, profile
from .library import KernelError

F32, BF16 = torch.float32, torch.bfloat16
_CODES = {F32: 0, BF16: 1}
PAGE_TOKENS = 64

_SIGNATURES = {
    "palm_embed": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p],
    "palm_rmsnorm": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_float, c_void_p, c_int, c_int,
                     c_void_p, c_int, c_int, c_longlong],
    "palm_swiglu": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int],
    "palm_add_bias": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int],
    "palm_convert": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_longlong],
    "palm_random_fill": [c_void_p, c_void_p, c_int, c_longlong, c_ulonglong, c_float, c_float],
    "palm_linear": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int],
    "palm_qk_norm_rope_store": [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                c_int, c_int, c_int, c_float],
    "palm_rope_table": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int],
    "palm_attention_simple": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                              c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    "palm_linear_thin": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                         c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p],
    "palm_scale_rows": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_int, c_void_p],
    "palm_linear_thin_parts": [c_int, c_int, c_int],
    "palm_linear_wide": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int],
    "palm_linear_wide_parts": [c_int, c_int, c_int, c_int],
    "palm_linear_wide_blocks": [c_int, c_int, c_int, c_int, c_int],
    "palm_linear_mid": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int],
    "palm_linear_mid_parts": [c_int, c_int, c_int, c_int],
    "palm_linear_mid_blocks": [c_int, c_int, c_int, c_int, c_int],
    "palm_linear_tile": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int],
    "palm_linear_tile_parts": [c_int, c_int, c_int],
    "palm_argmax": [c_void_p, c_void_p, c_int, c_int, c_void_p],
    "palm_apply_penalties": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_float, c_float, c_float],
    "palm_sample": [c_void_p, c_void_p, c_int, c_int, c_void_p, c_float, c_int, c_float, c_float, c_void_p, c_void_p],
}

_core = None


def core():
    """The core library, with the argument types of its entry points declared."""
    global _core
    if _core is None:
        lib = library.load("core")
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = argtypes, c_int      # (the *_parts and *_blocks functions return a count, not a status)
        if lib.palm_page_tokens() != PAGE_TOKENS:
            raise KernelError(f"the kernels were built for pages of {lib.palm_page_tokens()} tokens, "
                              f"the cache uses {PAGE_TOKENS}")
        _core = lib
    return _core


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _p(t):
    return None if t is None else t.data_ptr()


def _code(t: torch.Tensor, what: str) -> int:
    if t.dtype not in _CODES:
        raise KernelError(f"{what}: element type {t.dtype} is neither float32 nor bfloat16")
    return _CODES[t.dtype]


def _dev(what: str, *tensors) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError(f"{what}: a tensor lies on {t.device}; the kernels run on the GPU only "
                              "(there is no CPU path)")
        if not t.is_contiguous():
            raise KernelError(f"{what}: a tensor of shape {tuple(t.shape)} is not contiguous")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise KernelError(f"{what}: tensors lie on {dev} and {t.device}")


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _i32(what: str, *tensors) -> None:
    for t in tensors:
        if t is not None and t.dtype != torch.int32:
            raise KernelError(f"{what}: an index tensor has element type {t.dtype}, not int32")


# ---- elementwise ----------------------------------------------------------------------------------

def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[t, :] = table[ids[t], :] as float32."""
    _dev("embed", table, ids, out)
    _i32("embed", ids)
    _need(table.dim() == 2 and ids.dim() == 1, f"embed: table {tuple(table.shape)}, ids {tuple(ids.shape)}")
    vocab, hidden = table.shape
    n = ids.shape[0]
    if out is None:
        out = torch.empty((n, hidden), dtype=F32, device=table.device)
    _need(out.shape == (n, hidden) and out.dtype == F32, f"embed: out {tuple(out.shape)} {out.dtype}")
    library.call(core(), "palm_embed", _stream(), _p(table), _code(table, "embed table"), _p(ids), n, hidden, vocab, _p(out))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype, delta: torch.Tensor | None = None,
            update_x: bool = False, rows: torch.Tensor | None = None) -> torch.Tensor:
    """out[r] = norm(x[src] + delta[src]) * weight, src = rows[r] or r; with update_x the sum is written
    back to x (the residual stream).  x is [n, width]; statistics in float32.  delta may also be float32
    planes [P, n, width], which are added one after the other."""
    _dev("rmsnorm", x, weight, delta, rows)
    _i32("rmsnorm", rows)
    _need(x.dim() == 2, f"rmsnorm: x {tuple(x.shape)} is not [rows, width]")
    n, width = x.shape
    _need(weight.shape == (width,) and weight.dtype == F32, f"rmsnorm: weight {tuple(weight.shape)} {weight.dtype}, "
          f"width {width} (norm weights are float32)")
    planes = 1
    if delta is not None and delta.dim() == 3:
        planes = delta.shape[0]
        _need(delta.dtype == F32 and delta.shape[1:] == x.shape and delta.is_contiguous(),
              f"rmsnorm: delta planes {tuple(delta.shape)} {delta.dtype} for x {tuple(x.shape)} (planes are contiguous float32)")
    else:
        _need(delta is None or delta.shape == x.shape, "rmsnorm: delta and x differ in shape")
    _need(not update_x or (delta is not None and rows is None), "rmsnorm: update_x needs a delta and no row selection")
    n_out = n if rows is None else rows.shape[0]
    out = torch.empty((n_out, width), dtype=out_dtype, device=x.device)
    library.call(core(), "palm_rmsnorm", _stream(), _p(x), _code(x, "rmsnorm x"), _p(delta),
                 _code(delta, "rmsnorm delta") if delta is not None else 0, planes, _p(weight), float(eps), _p(rows), n_out, width,
                 _p(out), _code(out, "rmsnorm out"), int(update_x), n)
    return out


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """[n, 2I] -> [n, I]: silu(first half) * second half."""
    _dev("swiglu", gate_up)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, f"swiglu: input {tuple(gate_up.shape)}")
    n, two_i = gate_up.shape
    out = torch.empty((n, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    library.call(core(), "palm_swiglu", _stream(), _p(gate_up), _code(gate_up, "swiglu"), _p(out), n, two_i // 2)
    return out


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """y[r, :] += bias, in place; y [n, out] float32 or bfloat16, bias [out] float32.  Returns y."""
    _dev("add_bias", y, bias)
    _need(y.dim() == 2 and y.is_contiguous() and bias.shape == (y.shape[1],) and bias.dtype == F32 and bias.is_contiguous(),
          f"add_bias: y {tuple(y.shape)}, bias {tuple(bias.shape)} {bias.dtype} is not float32 [{y.shape[-1]}]")
    library.call(core(), "palm_add_bias", _stream(), _p(y), _code(y, "add_bias"), _p(bias), y.shape[0], y.shape[1])
    return y


_STORED_CODES = {F32: 0, BF16: 1, torch.float16: 2, torch.float64: 3}


def convert_into(src: torch.Tensor, dst: torch.Tensor) -> None:
    """dst = src in dst's element type (float32 or bfloat16); src is as a checkpoint stores it (float32, bfloat16,
    float16 or float64).  One rounding to nearest where dst is narrower.  dst may be a run of rows of a larger
    tensor: what a checkpoint's tensors go through when they are joined into one parameter."""
    _dev("convert", src, dst)
    _need(src.dtype in _STORED_CODES, f"convert: a tensor stored as {src.dtype} is not float32, bfloat16, float16 or float64")
    _need(src.numel() == dst.numel(), f"convert: {tuple(src.shape)} into {tuple(dst.shape)}")
    library.call(core(), "palm_convert", _stream(), _p(src), _STORED_CODES[src.dtype], _p(dst), _code(dst, "convert dst"),
                 src.numel())


def random_fill(out: torch.Tensor, key: int, mean: float, std: float) -> None:
    """out[i] = normal(key, i) * std + mean, the counter-based numbers of weights/random_numbers.py (same bits)."""
    _dev("random_fill", out)
    _need(0 <= int(key) < 1 << 64, "random_fill: the key is 64 bits")
    library.call(core(), "palm_random_fill", _stream(), _p(out), _code(out, "random_fill out"), out.numel(), int(key),
                 float(mean), float(std))


# ---- linear ---------------------------------------------------------------------------------------

def linear_exact(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype | None = None, out: torch.Tensor | None = None,
                 accumulate: bool = False) -> torch.Tensor:
    """a [M, K] . w [N, K]^T with plain 32-bit FMA; any mix of float32 and bfloat16 operands."""
    _dev("linear", a, w, out)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1],
          f"linear: a {tuple(a.shape)} and w {tuple(w.shape)} do not share the inner size")
    M, K = a.shape
    N = w.shape[0]
    if out is None:
        _need(not accumulate, "linear: accumulate needs an output to add to")
        out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
    _need(out.shape == (M, N), f"linear: out {tuple(out.shape)} is not {(M, N)}")
    library.call(core(), "palm_linear", _stream(), _p(a), _code(a, "linear a"), _p(w), _code(w, "linear w"), _p(out),
                 _code(out, "linear out"), M, N, K, int(accumulate))
    return out


# ---- attention ------------------------------------------------------------------------------------

def _check_cache(what, k_cache, v_cache, block_table, nkv, hd):
    _need(k_cache.dim() == 4 and k_cache.shape[1:] == (nkv, PAGE_TOKENS, hd),
          f"{what}: key cache {tuple(k_cache.shape)} is not [pages, {nkv}, {PAGE_TOKENS}, {hd}]")
    _need(v_cache.shape == (k_cache.shape[0], nkv, hd, PAGE_TOKENS) and v_cache.dtype == k_cache.dtype,
          f"{what}: value cache {tuple(v_cache.shape)} is not [pages, {nkv}, {hd}, {PAGE_TOKENS}] (values are kept transposed)")
    _need(block_table.dim() == 2, f"{what}: page table {tuple(block_table.shape)} is not [slots, pages]")


def qk_norm_rope_store(qkv: torch.Tensor, nh: int, nkv: int, hd: int, positions: torch.Tensor, *, q_norm_w=None,
                       k_norm_w=None, eps: float = 0.0, cos=None, sin=None, rotary_dim: int = 0, pairing: int = 0,
                       k_cache=None, v_cache=None, block_table=None, tok_slot=None, write_cache: bool = True,
                       out_dtype: torch.dtype | None = None, q_scale: float = 1.0) -> torch.Tensor:
    """qkv [n, (nh + 2 nkv) hd] -> q [n, nh hd], normed and rotated by the cos/sin rows [n, rotary_dim/2];
    k (normed, rotated) and v go to the cache page of (tok_slot[t], positions[t]).  qkv may also be float32
    planes [P, n, (nh + 2 nkv) hd] to be added up; ``out_dtype`` then names the type of q and of the cache.
    ``q_scale``: a factor on q (not k), applied before the rounding (see ``prefill_q_scale``)."""
    _dev("qk_norm_rope_store", qkv, positions, q_norm_w, k_norm_w, cos, sin, k_cache, v_cache, block_table, tok_slot)
    _i32("qk_norm_rope_store", positions, block_table, tok_slot)
    planes = 1
    if qkv.dim() == 3:
        planes = qkv.shape[0]
        _need(qkv.dtype == F32 and qkv.is_contiguous() and out_dtype is not None,
              "qk_norm_rope_store: planes are contiguous float32 and come with the type of the result")
        _need(planes >= 2 or out_dtype == F32, "qk_norm_rope_store: a single plane comes as rows of the result's type")
        n = qkv.shape[1]
    else:
        _need(qkv.dim() == 2, f"qk_norm_rope_store: qkv {tuple(qkv.shape)}")
        n = qkv.shape[0]
        out_dtype = out_dtype or qkv.dtype
        _need(out_dtype == qkv.dtype, "qk_norm_rope_store: q and the cache have the type of qkv unless qkv comes in planes")
    _need(qkv.shape[-1] == (nh + 2 * nkv) * hd, f"qk_norm_rope_store: qkv {tuple(qkv.shape)} is not "
          f"[n, ({nh} + 2*{nkv}) * {hd}]")
    _need(positions.shape == (n,), "qk_norm_rope_store: one position for each token")
    for w, nm in ((q_norm_w, "q"), (k_norm_w, "k")):
        _need(w is None or (w.shape == (hd,) and w.dtype == F32), f"qk_norm_rope_store: {nm} norm weight must be float32 [{hd}]")
    _need((cos is None) == (sin is None), "qk_norm_rope_store: cos and sin come together")
    if cos is not None:
        _need(0 < rotary_dim <= hd and rotary_dim % 2 == 0, f"qk_norm_rope_store: rotary_dim {rotary_dim}, head_dim {hd}")
        for tab in (cos, sin):
            _need(tab.dtype == F32 and tab.shape == (n, rotary_dim // 2),
                  f"qk_norm_rope_store: rotation table {tuple(tab.shape)} {tab.dtype} is not float32 [{n}, {rotary_dim // 2}]")
    max_pages = 0
    if write_cache:
        _need(k_cache is not None and v_cache is not None and block_table is not None and tok_slot is not None,
              "qk_norm_rope_store: writing the cache needs cache, page table and slots")
        _check_cache("qk_norm_rope_store", k_cache, v_cache, block_table, nkv, hd)
        _need(k_cache.dtype == out_dtype, f"qk_norm_rope_store: cache is {k_cache.dtype}, activations are {out_dtype}")
        _need(tok_slot.shape == (n,), "qk_norm_rope_store: one slot for each token")
        max_pages = block_table.shape[1]
    q_out = torch.empty((n, nh * hd), dtype=out_dtype, device=qkv.device)
    library.call(core(), "palm_qk_norm_rope_store", _stream(), _p(qkv), _code(q_out, "qkv"), planes, _p(q_out), _p(k_cache), _p(v_cache),
                 _p(block_table), max_pages, _p(tok_slot), _p(positions), _p(q_norm_w), _p(k_norm_w), float(eps),
                 _p(cos), _p(sin), int(rotary_dim if cos is not None else 0), int(pairing), n, nh, nkv, hd, int(write_cache),
                 float(q_scale))
    return q_out


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor):
    """cos, sin [n, half] float32 of positions[t] * inv_freq[i]."""
    _dev("rope_table", positions, inv_freq)
    _i32("rope_table", positions)
    _need(positions.dim() == 1 and inv_freq.dim() == 1 and inv_freq.dtype == F32, "rope_table: positions [n] int32, inv_freq [half] float32")
    n, half = positions.shape[0], inv_freq.shape[0]
    cos = torch.empty((n, half), dtype=F32, device=positions.device)
    sin = torch.empty_like(cos)
    library.call(core(), "palm_rope_table", _stream(), _p(positions), _p(inv_freq), _p(cos), _p(sin), n, half)
    return cos, sin


def attention_exact(q: torch.Tensor, k_cache, v_cache, block_table, seq_slot, seq_start, seq_new, cu_new, max_new: int,
                    nh: int, nkv: int, hd: int, scale: float, window: int | None) -> torch.Tensor:
    """Causal attention of the step's queries over the cache, 32-bit arithmetic, any head size.
    q [n, nh hd]; sequence b has seq_new[b] queries starting at row cu_new[b] and position seq_start[b]."""
    _dev("attention", q, k_cache, v_cache, block_table, seq_slot, seq_start, seq_new, cu_new)
    _i32("attention", block_table, seq_slot, seq_start, seq_new, cu_new)
    n = q.shape[0]
    _need(q.dim() == 2 and q.shape[1] == nh * hd, f"attention: q {tuple(q.shape)} is not [n, {nh}*{hd}]")
    _check_cache("attention", k_cache, v_cache, block_table, nkv, hd)
    _need(k_cache.dtype == q.dtype, f"attention: cache is {k_cache.dtype}, queries are {q.dtype}")
    B = seq_slot.shape[0]
    _need(seq_start.shape == (B,) and seq_new.shape == (B,) and cu_new.shape == (B + 1,),
          "attention: per-sequence arrays differ in length")
    out = torch.empty((n, nh * hd), dtype=q.dtype, device=q.device)
    library.call(core(), "palm_attention_simple", _stream(), _p(q), _code(q, "attention q"), _p(k_cache), _p(v_cache),
                 _p(block_table), block_table.shape[1], _p(seq_slot), _p(seq_start), _p(seq_new), _p(cu_new), B, int(max_new),
                 nh, nkv, hd, float(scale), int(window or 0), _p(out))
    return out


# ---- sampling -------------------------------------------------------------------------------------

def argmax(logits: torch.Tensor) -> torch.Tensor:
    _dev("argmax", logits)
    _need(logits.dim() == 2 and logits.dtype == F32, f"argmax: logits {tuple(logits.shape)} {logits.dtype}")
    out = torch.empty((logits.shape[0],), dtype=torch.int32, device=logits.device)
    library.call(core(), "palm_argmax", _stream(), _p(logits), logits.shape[0], logits.shape[1], _p(out))
    return out


def apply_penalties(logits: torch.Tensor, rows, tokens, counts, repeat_penalty: float, presence: float, frequency: float) -> None:
    """In place, for each (row, token, count)."""
    _dev("penalties", logits, rows, tokens, counts)
    _i32("penalties", rows, tokens, counts)
    _need(logits.dim() == 2 and logits.dtype == F32, "penalties: logits must be float32 [rows, vocab]")
    _need(rows.shape == tokens.shape == counts.shape and rows.dim() == 1, "penalties: rows, tokens, counts differ in length")
    library.call(core(), "palm_apply_penalties", _stream(), _p(logits), logits.shape[1], _p(rows), _p(tokens), _p(counts),
                 rows.shape[0], float(repeat_penalty), float(presence), float(frequency))


def sample(logits: torch.Tensor, uniforms: torch.Tensor | None, temperature: float, top_k: int = 0, top_p: float = 0.0,
           min_p: float = 0.0, want_probs: bool = False):
    """One token for each row.  ``uniforms`` [rows] float32 in [0, 1).  With want_probs also the
    distribution that was drawn from, [rows, vocab]."""
    _dev("sample", logits, uniforms)
    _need(logits.dim() == 2 and logits.dtype == F32, f"sample: logits {tuple(logits.shape)} {logits.dtype}")
    n, V = logits.shape
    _need(uniforms is None or (uniforms.shape == (n,) and uniforms.dtype == F32), "sample: uniforms must be float32 [rows]")
    out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    probs = torch.empty((n, V), dtype=F32, device=logits.device) if want_probs else None
    library.call(core(), "palm_sample", _stream(), _p(logits), n, V, _p(uniforms), float(temperature), int(top_k), float(top_p),
                 float(min_p), _p(out), _p(probs))
    return (out, probs) if want_probs else out


# ---- dispatch: which kernel serves a call -----------------------------------------------------------

def linear_library(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """bfloat16 a [M, K] . w [N, K]^T through the BLAS library (hipBLASLt under torch.matmul), 32-bit
    accumulation, bfloat16 result: the one place where a library computes on the product path."""
    _dev("linear", a, w)
    _need(a.dtype == BF16 and w.dtype == BF16, "linear_library serves bfloat16 operands only")
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1],
          f"linear: a {tuple(a.shape)} and w {tuple(w.shape)} do not share the inner size")
    recorder = profile.active()
    if recorder is not None:
        return recorder.around("library_matmul", lambda: torch.matmul(a, w.t()))
    return torch.matmul(a, w.t())


THIN_TOKENS = 16      # up to here every wave fetches its own activations; above, a block shares them through LDS
WIDE_TOKENS = 128     # as many rows as that block holds
WIDE_FLOAT32_TOKENS = 64   # a float32 result (logits) of more rows than this goes through the tiled kernel instead


COMPUTE_UNITS = 256     # of an MI355X; a folded product's blocks come in rounds of this many


def fold_pays(M: int, N: int, K: int) -> bool:
    """Whether a product of M <= 16 rows that is a branch's output should fold the residual add and the next norm
    in, or rather be cut along K into planes that the norm's own kernel adds up.  A fold needs all of K in one
    block.  Up to K = 8192 the block keeps the activations in registers and the fold won at every width measured
    (N 1024 to 5120: 8 to 28 us against 8 to 36).  Beyond that it reads them beside the weights and wins only
    where whole rounds of blocks fill the compute units: N 4096 at K 12288 and 14336 (25 to 42 us against 32 to
    41), not N 2560 or 5120 (a quarter of a second round: 55 to 125 us against 40 to 66), and nowhere measured
    beyond K 14336."""
    if K <= 8192:
        return True
    strips = (N + 15) // 16
    rounds = (strips + COMPUTE_UNITS - 1) // COMPUTE_UNITS
    return K <= 14336 and strips >= 0.75 * rounds * COMPUTE_UNITS


WIDE_MIN_BLOCKS = 128   # of 256 compute units


def wide_pays(M: int, N: int, K: int, gated: bool = False, planes_ok: bool = False) -> bool:
    """Whether the kernel for 17 to 128 rows has enough blocks for this product to beat the library: with few
    weight rows it does only if the reader takes planes of partial sums.  Measured at Qwen3-8B's shapes with 64
    rows (us, own against library): q/k/v 18 and 18, output projection 14 and 16, down 27 and 37 as planes (76
    whole), gate/up 45 gated against 46 with the activation's own pass; with 32 rows 14/17, 11/13, 23/26, 40/47;
    with 128 rows q/k/v 22 and 26, output projection 17 and 25, down 37 and 65, gate/up 65 gated against 53 and the
    activation's pass of 8 (kept all the same: a step of up to 128 sequences then runs no library code and can be
    recorded)."""
    return THIN_TOKENS < M <= WIDE_TOKENS and core().palm_linear_wide_blocks(
        M, N, K, 1 if gated else 0, 1 if planes_ok else 0) >= WIDE_MIN_BLOCKS


MID_TOKENS = 256      # rows of one block of the kernel whose operands both cross LDS
MID_FROM = 16         # above this many rows it serves (up to 16: the stream whose activations stay in registers)
MID_CHUNK = 64        # it walks over K in steps of this many


def mid_pays(M: int, N: int, K: int, planes_ok: bool = False, gated: bool = False,
             out_dtype: torch.dtype = BF16) -> bool:
    """Whether the kernel that brings both operands through rings in LDS serves this product of bfloat16 operands.

    17 to 128 rows (decode steps of many sequences, short prompts): wherever its blocks fill the chip (for few weight
    rows that needs a reader that takes planes).  Measured at Qwen3-8B's shapes (us, this kernel against that one): 64 rows gate/up gated 46
    and 49, down 25 and 27, output projection 11 and 14, q/k/v 16 and 17, head 231 and 275; 128 rows 47 and 67, 30 and
    36, 14 and 17, 19 and 21, 273 and 338 (the tiled kernel 289); 32 rows 42 and 40, 22 and 23, 10 and 11, 14 and 14,
    222 and 252 (a decode step of 32 sequences at Qwen3-32B's sizes 20.7 against 21.3 ms).

    129 to 256 rows (short prompts): where the weight rows are so few that it cuts K into planes; the library's tiles
    leave compute units idle there.  Own against library at 256 rows: q/k/v 29 and 40, output projection 23 and 24,
    down 46 and 53; at 129 rows (library at 192) 23 and 34, 18 and 33, 39 and 88; the planes cost their readers about
    4 us each.  Not a product with weight rows enough for all compute units (gate/up at 256 rows: 70 against 65, gated
    72 to 79 against 65 and the activation's pass of 8; every block then reads all rows again for 96 weight rows, and
    one wave a SIMD does not overlap those loads, the fragment reads from LDS and 39 us of arithmetic), and not more
    than 256 rows, where it ties (q/k/v 40 and 37, output projection 32 and 30, down 78 and 80 at 512 rows)."""
    if K % MID_CHUNK != 0 or not MID_FROM < M <= MID_TOKENS:
        return False
    planes = planes_ok and not gated
    blocks = core().palm_linear_mid_blocks(M, N, K, 1 if gated else 0, 1 if planes else 0)
    if M <= WIDE_TOKENS:
        return blocks >= WIDE_MIN_BLOCKS
    return planes and out_dtype == BF16 and core().palm_linear_mid_parts(M, N, K, 0) > 1 and blocks >= WIDE_MIN_BLOCKS


def linear_mid(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, gated: bool = False,
               planes_ok: bool = False) -> torch.Tensor:
    """bfloat16 a [M, K] . w [N, K]^T for some hundred rows, K a multiple of 64: both operands go through rings in
    LDS, a block of four waves holding 256 rows against 96 or 64 weight rows.  The result is [M, N] in bfloat16 or
    float32 ([M, N/2] bfloat16 when ``gated``), or, if ``planes_ok`` and the weight rows are few, float32 planes
    [P, M, N] over ranges of K."""
    _dev("linear_mid", a, w)
    _need(a.dtype == BF16 and w.dtype == BF16 and a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1]
          and a.is_contiguous() and w.is_contiguous(),
          f"linear_mid: a {tuple(a.shape)} {a.dtype} and w {tuple(w.shape)} {w.dtype} (bfloat16, one inner size)")
    M, K = a.shape
    N = w.shape[0]
    _need(K % MID_CHUNK == 0, f"linear_mid: K = {K} is no multiple of {MID_CHUNK}")
    _need(not gated or (N % 2 == 0 and out_dtype == BF16), "linear_mid: a gated product has an even number of weight rows and a bfloat16 result")
    planes = core().palm_linear_mid_parts(M, N, K, 0) if planes_ok and not gated else 1
    if planes > 1:
        out = torch.empty((planes, M, N), dtype=F32, device=a.device)
    else:
        out = torch.empty((M, N // 2 if gated else N), dtype=out_dtype, device=a.device)
    library.call(core(), "palm_linear_mid", _stream(), _p(a), _p(w), _p(out), _code(out, "linear_mid out"), M, N, K,
                 1 if gated else 0, planes)
    return out


def thin_serves(a: torch.Tensor, w: torch.Tensor) -> bool:
    """The matrix-core kernel for thin products takes bfloat16 operands whose rows start on 16 bytes."""
    return a.dtype == BF16 and w.dtype == BF16 and a.shape[1] % 8 == 0


def _row_ss(what: str, a: torch.Tensor, row_ss) -> int:
    """Checks the pieces of the rows' sums of squares that come with rows lacking their norm's factor."""
    if row_ss is None:
        return 0
    _dev(what, a, row_ss)
    _need(row_ss.dim() == 2 and row_ss.shape[0] == a.shape[0] and row_ss.dtype == F32 and row_ss.is_contiguous()
          and row_ss.shape[1] > 0, f"{what}: sums of squares {tuple(row_ss.shape)} {row_ss.dtype} for {a.shape[0]} rows")
    _need(a.shape[0] <= THIN_TOKENS and thin_serves(a, a), f"{what}: a norm is folded into products of at most {THIN_TOKENS} bfloat16 rows")
    return row_ss.shape[1]


def scale_rows(a: torch.Tensor, row_ss: torch.Tensor, eps: float) -> torch.Tensor:
    """a[r] / sqrt(sum of row_ss[r, :] / width + eps): rows that lack their norm's factor, made whole."""
    _dev("scale_rows", a, row_ss)
    _need(a.dim() == 2 and row_ss.dim() == 2 and row_ss.shape[0] == a.shape[0] and row_ss.dtype == F32 and row_ss.is_contiguous()
          and row_ss.shape[1] > 0, f"scale_rows: rows {tuple(a.shape)}, sums of squares {tuple(row_ss.shape)} {row_ss.dtype}")
    out = torch.empty_like(a)
    library.call(core(), "palm_scale_rows", _stream(), _p(a), _code(a, "scale_rows"), _p(row_ss), row_ss.shape[1], a.shape[0],
                 float(eps), a.shape[1], _p(out))
    return out


def linear_thin_into_residual(a: torch.Tensor, w: torch.Tensor, x: torch.Tensor, norm_w: torch.Tensor, row_ss=None,
                              row_eps: float = 0.0):
    """A branch's last product and what follows it, for up to 16 rows: x += a . w^T (x float32 [M, N], in
    place); returns (x * norm_w rounded to bfloat16, the pieces [M, N/16] of each row's sum of squares of x):
    the next norm's output but for the row factor.  row_ss / row_eps: a itself lacks a row factor."""
    _dev("linear_thin_into_residual", a, w, x, norm_w)
    M, K = a.shape
    N = w.shape[0]
    _need(thin_serves(a, w) and M <= THIN_TOKENS and w.shape[1] == K, f"linear_thin_into_residual: a {tuple(a.shape)} {a.dtype}, "
          f"w {tuple(w.shape)} {w.dtype} (bfloat16, at most {THIN_TOKENS} rows, K a multiple of 8)")
    _need(x.shape == (M, N) and x.dtype == F32 and x.is_contiguous(), f"linear_thin_into_residual: residual {tuple(x.shape)} {x.dtype}")
    _need(norm_w.shape == (N,) and norm_w.dtype == F32, "linear_thin_into_residual: the norm's weight is float32 [N]")
    pieces = _row_ss("linear_thin_into_residual", a, row_ss)
    values = torch.empty((M, N), dtype=BF16, device=a.device)
    ss = torch.empty((M, (N + 15) // 16), dtype=F32, device=a.device)
    library.call(core(), "palm_linear_thin", _stream(), _p(a), _p(w), _p(values), _code(values, "values"), M, N, K, 0, 1,
                 _p(row_ss), pieces, float(row_eps), _p(x), _p(norm_w), _p(ss))
    return values, ss


def linear_thin(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, gated: bool = False,
                planes_ok: bool = False, row_ss=None, row_eps: float = 0.0) -> torch.Tensor:
    """bfloat16 a [M, K] . w [N, K]^T on the matrix cores, the weight streamed once per 16 rows of a (64 above 16);
    result [M, N] in bfloat16 or float32.  With ``gated`` w is [gate rows | up rows] and the result is
    silu(a gate^T) * (a up^T), [M, N/2].

    ``planes_ok``: the caller can take the product as float32 planes [P, M, N] whose sum (in the order of the
    planes) it is: for a few rows and few weight rows the kernel then cuts K into P ranges to fill the chip.
    rmsnorm's ``delta`` and qk_norm_rope_store's ``qkv`` take such planes.

    ``row_ss`` [M, pieces] float32 with ``row_eps``: the rows of a lack the factor 1 / sqrt(mean square + eps) of
    their norm, whose sums of squares come in pieces; the result rows are multiplied by it (at most 16 rows)."""
    pieces = _row_ss("linear_thin", a, row_ss)
    if not thin_serves(a, w):
        out = linear_exact(a, w, out_dtype)
        return swiglu(out) if gated else out
    _dev("linear_thin", a, w)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1],
          f"linear: a {tuple(a.shape)} and w {tuple(w.shape)} do not share the inner size")
    M, K = a.shape
    N = w.shape[0]
    _need(not gated or N % 2 == 0, f"linear_thin: a gated product needs an even number of weight rows, got {N}")
    out = torch.empty((M, N // 2 if gated else N), dtype=out_dtype, device=a.device)
    if M <= THIN_TOKENS:
        planes = core().palm_linear_thin_parts(M, N, K) if planes_ok and not gated else 1
        if planes > 1:
            out = torch.empty((planes, M, N), dtype=F32, device=a.device)
        library.call(core(), "palm_linear_thin", _stream(), _p(a), _p(w), _p(out), _code(out, "linear_thin out"), M, N, K,
                     1 if gated else 0, planes, _p(row_ss), pieces, float(row_eps), None, None, None)
        return out
    _need(row_ss is None, f"linear_thin: rows that lack their norm's factor come at most {THIN_TOKENS} at a time, not {M}")
    if M > WIDE_TOKENS or (M > WIDE_FLOAT32_TOKENS and out_dtype == F32 and not planes_ok):
        # a float32 result for many rows (logits at many places): the tiled kernel, which reads the weight once for
        # every 256 rows; where K is no whole number of its stages, 64 rows at a time
        if tile_serves(a, w) and not gated:
            return linear_tile(a, w, out_dtype)
        return torch.cat([linear_thin(a[r0:r0 + WIDE_FLOAT32_TOKENS], w, out_dtype, gated=gated)
                          for r0 in range(0, M, WIDE_FLOAT32_TOKENS)])
    # more rows than one block of 16: the kernel that shares the activations through LDS
    planes = core().palm_linear_wide_parts(M, N, K, 0) if planes_ok and not gated else 1
    if planes > 1:
        out = torch.empty((planes, M, N), dtype=F32, device=a.device)
    library.call(core(), "palm_linear_wide", _stream(), _p(a), _p(w), _p(out), _code(out, "linear_wide out"), M, N, K,
                 1 if gated else 0, planes)
    return out


# ---- products of many rows ----------------------------------------------------------------------------

TILE_K = 64           # the tiled kernel walks over K in stages of this many


def tile_serves(a: torch.Tensor, w: torch.Tensor) -> bool:
    """The tiled matrix-core kernel takes bfloat16 operands whose K is a whole number of stages."""
    return a.dtype == BF16 and w.dtype == BF16 and a.shape[1] % TILE_K == 0 and a.shape[1] == w.shape[1]


def linear_tile(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, planes_ok: bool = False) -> torch.Tensor:
    """bfloat16 a [M, K] . w [N, K]^T for many rows, tiled over the matrix cores; result bfloat16 or float32.
    ``planes_ok``: the caller takes float32 planes [P, M, N] of partial sums (see linear_thin); the kernel then
    cuts K into ranges where the tiles alone would leave most of the chip without work."""
    _dev("linear_tile", a, w)
    _need(a.dim() == 2 and w.dim() == 2 and tile_serves(a, w), f"linear_tile: a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} "
          f"{w.dtype} (bfloat16, one inner size, a multiple of {TILE_K})")
    M, K = a.shape
    N = w.shape[0]
    parts = core().palm_linear_tile_parts(M, N, K) if planes_ok else 1
    if parts > 1:
        out = torch.empty((parts, M, N), dtype=F32, device=a.device)
    else:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    library.call(core(), "palm_linear_tile", _stream(), _p(a), _p(w), _p(out), _code(out, "linear_tile out"), M, N, K, parts)
    return out


# ---- attention on the matrix cores (one library for each head size) ---------------------------------

_ATTENTION_SIGNATURES = {
    "palm_attention_decode": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int,
                              c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p],
    "palm_attention_prefill": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p],
    "palm_attention_prefill_takes_prescaled": [],
    "palm_attention_decode_fused": [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int,
                                    c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int,
                                    c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p],
    "palm_attention_decode_fused_serves": [c_int, c_int],
}
_attention_libs: dict = {}
MFMA_HEAD_DIMS = tuple(range(16, 257, 16))
DECODE_WAVES_WANTED = 768         # slices of the key range are made until about this many waves run (measured best)


def attention_lib(hd: int):
    if hd not in _attention_libs:
        if hd not in MFMA_HEAD_DIMS:
            raise KernelError(f"the matrix-core attention kernels take head sizes in steps of 16 up to 256, not {hd}")
        lib = library.load(f"attention_hd{hd}")
        for name, argtypes in _ATTENTION_SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = argtypes, c_int
        if lib.palm_attention_head_dim() != hd:
            raise KernelError(f"library attention_hd{hd} was built for head size {lib.palm_attention_head_dim()}")
        if lib.palm_attention_page_tokens() != PAGE_TOKENS:
            raise KernelError(f"library attention_hd{hd} was built for pages of {lib.palm_attention_page_tokens()} tokens, "
                              f"the cache has pages of {PAGE_TOKENS}")
        _attention_libs[hd] = lib
    return _attention_libs[hd]


def mfma_attention_serves(q: torch.Tensor, hd: int) -> bool:
    return q.dtype == BF16 and hd in MFMA_HEAD_DIMS


def decode_slices(n_seqs: int, nh: int, nkv: int, max_keys: int) -> int:
    """Into how many slices each sequence's key range is cut, so that the launch fills the chip."""
    waves = n_seqs * nkv * ((nh // nkv + 15) // 16)
    pages = max(1, (max_keys + PAGE_TOKENS - 1) // PAGE_TOKENS)
    return max(1, min(pages, (DECODE_WAVES_WANTED + waves - 1) // waves))


def _attention_checks(what, q, k_cache, v_cache, block_table, nh, nkv, hd, *index):
    _dev(what, q, k_cache, v_cache, block_table, *index)
    _i32(what, block_table, *index)
    _need(q.dim() == 2 and q.shape[1] == nh * hd and q.dtype == BF16, f"{what}: q {tuple(q.shape)} {q.dtype} is not bfloat16 [n, {nh}*{hd}]")
    _need(nh % nkv == 0, f"{what}: {nh} heads are not a multiple of {nkv} kv heads")
    _check_cache(what, k_cache, v_cache, block_table, nkv, hd)
    _need(k_cache.dtype == BF16, f"{what}: the cache is {k_cache.dtype}, not bfloat16")


def _slices_workspace(what: str, work, B: int, nh: int, n_slices: int, hd: int, device):
    """Where the slices' partial results cross to the merging kernel: the caller's, or a new one."""
    need = B * nh * n_slices * (hd + 4)
    if n_slices <= 1:
        return None
    if work is None:
        return torch.empty((need,), dtype=F32, device=device)
    _dev(what, work)
    _need(work.dtype == F32 and work.numel() >= need, f"{what}: the workspace holds {work.numel()} {work.dtype}, "
          f"{B} sequences x {nh} heads x {n_slices} slices need {need} float32")
    return work


def attention_decode(q, k_cache, v_cache, block_table, seq_slot, seq_start, nh: int, nkv: int, hd: int, scale: float,
                     window: int | None, n_slices: int, work: torch.Tensor | None = None) -> torch.Tensor:
    """One query for each sequence (row b of q, at position seq_start[b]) over keys 0..seq_start[b].  ``work``: a
    float32 workspace of B * nh * n_slices * (hd + 4) elements for the slices' partial results (made here if None;
    nothing in it has to be cleared)."""
    _attention_checks("attention_decode", q, k_cache, v_cache, block_table, nh, nkv, hd, seq_slot, seq_start)
    B = seq_slot.shape[0]
    _need(q.shape[0] == B and seq_start.shape == (B,), "attention_decode: one query, slot and start for each sequence")
    out = torch.empty_like(q)
    work = _slices_workspace("attention_decode", work, B, nh, n_slices, hd, q.device)
    library.call(attention_lib(hd), "palm_attention_decode", _stream(), _p(q), _p(k_cache), _p(v_cache), _p(block_table),
                 block_table.shape[1], _p(seq_slot), _p(seq_start), B, nh, nkv, hd, float(scale), int(window or 0),
                 int(n_slices), _p(work), _p(out))
    return out


DECODE_FUSED_ROWS = 96      # sequences up to which the q/k/v pass rides in the decode attention kernel


def decode_fused_serves(qkv: torch.Tensor, hd: int, out_dtype, rotary_dim: int, pairing: int) -> bool:
    """Whether attention_decode_fused takes this step's q/k/v rows: bfloat16 attention on the matrix cores, a head
    size and a rotation for which a rotation pair lies in one lane, and not too many sequences: every wave of a
    sequence's slices makes the queries anew, which for many sequences costs more than the pass of its own that it
    saves (a step of Qwen3-8B's sizes, fused against apart: 64 sequences 7.80 and 7.93 ms, 96: 10.15 and 10.11,
    128: 12.23 and 11.87)."""
    if out_dtype != BF16 or hd not in MFMA_HEAD_DIMS or qkv.shape[-2] > DECODE_FUSED_ROWS:
        return False
    if not (qkv.dim() == 3 and qkv.dtype == F32 or qkv.dim() == 2 and qkv.dtype == BF16):
        return False
    return bool(attention_lib(hd).palm_attention_decode_fused_serves(int(rotary_dim), int(pairing)))


def attention_decode_fused(qkv, k_cache, v_cache, block_table, seq_slot, seq_start, nh: int, nkv: int, hd: int, scale: float,
                           window: int | None, n_slices: int, *, q_norm_w=None, k_norm_w=None, eps: float = 0.0, cos=None,
                           sin=None, rotary_dim: int = 0, pairing: int = 0, write_cache: bool = True,
                           work: torch.Tensor | None = None) -> torch.Tensor:
    """A decode step's attention from the joined projection's rows: qk_norm_rope_store and attention_decode in one
    launch.  qkv is [B, (nh + 2 nkv) hd] bfloat16 or float32 planes [P, B, (nh + 2 nkv) hd]; sequence b's token is
    row b, at position seq_start[b]; cos, sin are [B, hd / 2] rows of those positions.  Returns [B, nh hd] bfloat16."""
    what = "attention_decode_fused"
    _dev(what, qkv, k_cache, v_cache, block_table, seq_slot, seq_start, q_norm_w, k_norm_w, cos, sin)
    _i32(what, block_table, seq_slot, seq_start)
    as_planes = qkv.dim() == 3
    _need(qkv.is_contiguous() and (as_planes and qkv.dtype == F32 or qkv.dim() == 2 and qkv.dtype == BF16),
          f"{what}: qkv {tuple(qkv.shape)} {qkv.dtype} is neither bfloat16 rows nor float32 planes")
    B = seq_slot.shape[0]
    _need(qkv.shape[-2] == B and qkv.shape[-1] == (nh + 2 * nkv) * hd and seq_start.shape == (B,),
          f"{what}: qkv {tuple(qkv.shape)} is not [.., {B}, ({nh} + 2*{nkv}) * {hd}]")
    _need(nh % nkv == 0, f"{what}: {nh} heads are not a multiple of {nkv} kv heads")
    _check_cache(what, k_cache, v_cache, block_table, nkv, hd)
    _need(k_cache.dtype == BF16, f"{what}: the cache is {k_cache.dtype}, not bfloat16")
    for w, nm in ((q_norm_w, "q"), (k_norm_w, "k")):
        _need(w is None or (w.shape == (hd,) and w.dtype == F32), f"{what}: {nm} norm weight must be float32 [{hd}]")
    _need((cos is None) == (sin is None), f"{what}: cos and sin come together")
    for tab in (cos, sin):
        _need(tab is None or (tab.dtype == F32 and tab.shape == (B, hd // 2) and tab.is_contiguous() and rotary_dim == hd),
              f"{what}: a rotation table is float32 [{B}, {hd // 2}] over the whole head")
    out = torch.empty((B, nh * hd), dtype=BF16, device=qkv.device)
    work = _slices_workspace(what, work, B, nh, n_slices, hd, qkv.device)
    library.call(attention_lib(hd), "palm_attention_decode_fused", _stream(), _p(qkv), int(as_planes),
                 qkv.shape[0] if as_planes else 1, _p(q_norm_w), _p(k_norm_w), float(eps), _p(cos), _p(sin),
                 int(rotary_dim if cos is not None else 0), int(pairing), int(write_cache), _p(k_cache), _p(v_cache),
                 _p(block_table), block_table.shape[1], _p(seq_slot), _p(seq_start), B, nh, nkv, hd, float(scale),
                 int(window or 0), int(n_slices), _p(work), _p(out))
    return out


LOG2E = 1.4426950408889634


def prefill_q_scale(hd: int, dtype, scale: float) -> float:
    """What the pass that rounds a prompt's queries should multiply them by first: scale * log2(e) where the prompt
    attention kernel of this head size takes its queries so (a score is then the exponent of its weight as it leaves
    the matrix cores), else 1."""
    if dtype == BF16 and hd in MFMA_HEAD_DIMS and attention_lib(hd).palm_attention_prefill_takes_prescaled():
        return float(scale) * LOG2E
    return 1.0


def attention_prefill(q, k_cache, v_cache, block_table, seq_slot, seq_start, seq_new, cu_new, max_new: int, nh: int,
                      nkv: int, hd: int, scale: float, window: int | None, q_prescaled: bool = False) -> torch.Tensor:
    """The step's queries (several for each sequence) over the cache, on the matrix cores.  ``q_prescaled``: the
    queries come multiplied by ``prefill_q_scale`` already, and ``scale`` is not applied again."""
    _attention_checks("attention_prefill", q, k_cache, v_cache, block_table, nh, nkv, hd, seq_slot, seq_start, seq_new, cu_new)
    B = seq_slot.shape[0]
    _need(seq_start.shape == (B,) and seq_new.shape == (B,) and cu_new.shape == (B + 1,),
          "attention_prefill: per-sequence arrays differ in length")
    out = torch.empty_like(q)
    library.call(attention_lib(hd), "palm_attention_prefill", _stream(), _p(q), _p(k_cache), _p(v_cache), _p(block_table),
                 block_table.shape[1], _p(seq_slot), _p(seq_start), _p(seq_new), _p(cu_new), B, int(max_new), nh, nkv, hd,
                 float(scale), int(window or 0), int(bool(q_prescaled)), _p(out))
    return out


def slices_of_step(ctx, nh: int, nkv: int, window: int | None) -> int:
    """The slices of a decode step's key ranges: what a recorded step was cut for, else what fills the chip."""
    keys = min(ctx.max_total, window) if window else ctx.max_total
    return ctx.decode_slices or decode_slices(ctx.n_seqs, nh, nkv, keys)


def attention(q, k_cache, v_cache, block_table, ctx, nh: int, nkv: int, hd: int, scale: float, window: int | None,
              q_prescaled: bool = False):
    """The step's queries over the cache; picks the kernel by element type, head size and step shape.
    ``q_prescaled``: see ``attention_prefill`` (only a prompt step on the matrix cores takes such queries)."""
    if q_prescaled:
        _need(mfma_attention_serves(q, hd) and not ctx.is_decode, "attention: only the prompt kernel takes scaled queries")
        return attention_prefill(q, k_cache, v_cache, block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new,
                                 ctx.max_new, nh, nkv, hd, scale, window, q_prescaled=True)
    if mfma_attention_serves(q, hd):
        if ctx.is_decode:
            n_slices = slices_of_step(ctx, nh, nkv, window)
            return attention_decode(q, k_cache, v_cache, block_table, ctx.seq_slot, ctx.seq_start, nh, nkv, hd, scale,
                                    window, n_slices)
        return attention_prefill(q, k_cache, v_cache, block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new,
                                 ctx.max_new, nh, nkv, hd, scale, window)
    return attention_exact(q, k_cache, v_cache, block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new,
                           ctx.max_new, nh, nkv, hd, scale, window)

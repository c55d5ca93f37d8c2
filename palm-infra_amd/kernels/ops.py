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
    "palm_embed": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p, c_float],
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
    "palm_rope_table": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float],
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

def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor | None = None, scale: float = 1.0) -> torch.Tensor:
    """out[t, :] = table[ids[t], :] * scale as float32."""
    _dev("embed", table, ids, out)
    _i32("embed", ids)
    _need(table.dim() == 2 and ids.dim() == 1, f"embed: table {tuple(table.shape)}, ids {tuple(ids.shape)}")
    vocab, hidden = table.shape
    n = ids.shape[0]
    if out is None:
        out = torch.empty((n, hidden), dtype=F32, device=table.device)
    _need(out.shape == (n, hidden) and out.dtype == F32, f"embed: out {tuple(out.shape)} {out.dtype}")
    library.call(core(), "palm_embed", _stream(), _p(table), _code(table, "embed table"), _p(ids), n, hidden, vocab, _p(out),
                 float(scale))
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


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, magnitude: float = 1.0):
    """cos, sin [n, half] float32 of positions[t] * inv_freq[i], both times ``magnitude``."""
    _dev("rope_table", positions, inv_freq)
    _i32("rope_table", positions)
    _need(positions.dim() == 1 and inv_freq.dim() == 1 and inv_freq.dtype == F32, "rope_table: positions [n] int32, inv_freq [half] float32")
    n, half = positions.shape[0], inv_freq.shape[0]
    cos = torch.empty((n, half), dtype=F32, device=positions.device)
    sin = torch.empty_like(cos)
    library.call(core(), "palm_rope_table", _stream(), _p(positions), _p(inv_freq), _p(cos), _p(sin), n, half, float(magnitude))
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


# ---- mixers beside softmax attention, and blocks that norm a branch's output (library ``mixers``) -----------------

_MIXER_SIGNATURES = {
    "palm_add_normed": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_float, c_int, c_int, c_void_p, c_void_p, c_int,
                        c_longlong, c_void_p, c_int],
    "palm_xielu": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_longlong],
    "palm_causal_conv": [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                         c_int, c_int, c_int, c_void_p],
    "palm_selective_scan": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "palm_diff_qkv_store": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                            c_void_p, c_void_p, c_float, c_int, c_int, c_int, c_int, c_int, c_int],
    "palm_attention_diff": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                            c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_float, c_float, c_void_p, c_int,
                            c_void_p, c_int],
    "palm_add_normed_scaled": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_float, c_float, c_int, c_int, c_void_p, c_float,
                               c_void_p, c_int],
    "palm_softcap": [c_void_p, c_void_p, c_float, c_longlong],
    "palm_delta_pad": [c_int],
    "palm_delta_rule": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                        c_void_p, c_void_p, c_void_p, c_float, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                        c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p],
    "palm_latent_prep": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p,
                         c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p],
    "palm_latent_query": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "palm_latent_attention": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                              c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    "palm_latent_output": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
}
_mixers = None


def mixers():
    """The library of the other mixers' kernels, with the argument types of its entry points declared."""
    global _mixers
    if _mixers is None:
        lib = library.load("mixers")
        for name, argtypes in _MIXER_SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = argtypes, c_int
        _mixers = lib
    return _mixers


_RECURRENT_SIGNATURES = {
    "palm_retention": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p,
                       c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int,
                       c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    "palm_retention_pad": [c_int],
    "palm_joined_norm_gate": [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
}
_SINK_SIGNATURES = {
    "palm_sink_qkv_store": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                            c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                            c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int],
    "palm_sink_attention": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                            c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_float, c_void_p, c_void_p, c_int,
                            c_int, c_int, c_void_p, c_void_p],
}
_FEEDFORWARD_SIGNATURES = {
    "palm_moe_route": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p],
    "palm_moe_route_scored": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int, c_float, c_void_p, c_void_p],
    "palm_add_gated_rows": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int],
    "palm_moe_experts": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                         c_void_p, c_void_p, c_int],
    "palm_moe_tile_tokens": [],
    "palm_moe_grouped": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                         c_void_p, c_void_p, c_int],
    "palm_gather_rows": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    "palm_scatter_add": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "palm_activation": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_longlong],
}
_STREAMS_SIGNATURES = {
    "palm_streams_spread": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "palm_streams_mix_norm": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                              c_void_p, c_float, c_float, c_void_p, c_int, c_int, c_void_p, c_int],
}
_MLSTM_SIGNATURES = {
    "palm_mlstm_pad": [c_int],
    "palm_mlstm": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_float, c_void_p, c_float,
                   c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p,
                   c_int, c_void_p, c_void_p],
}
_BRANCH_SIGNATURES = {
    "palm_add_scaled_normed": [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_float, c_int, c_void_p, c_void_p, c_float, c_void_p,
                               c_int, c_int, c_int, c_void_p, c_int],
    "palm_capped_gate": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_float, c_float],
}
_small_libraries: dict = {}


def _small(name: str, signatures: dict):
    """A library of one mechanism, loaded (and built, if it never was) when a model first uses the mechanism."""
    lib = _small_libraries.get(name)
    if lib is None:
        lib = library.load(name)
        for fn_name, argtypes in signatures.items():
            fn = getattr(lib, fn_name)
            fn.argtypes, fn.restype = argtypes, c_int
        _small_libraries[name] = lib
    return lib


def recurrent():
    return _small("recurrent", _RECURRENT_SIGNATURES)


def sink_attention_lib():
    return _small("sink_attention", _SINK_SIGNATURES)


def branches():
    return _small("branches", _BRANCH_SIGNATURES)


def feedforward():
    return _small("feedforward", _FEEDFORWARD_SIGNATURES)


def streams_lib():
    return _small("streams", _STREAMS_SIGNATURES)


def mlstm_lib():
    return _small("mlstm", _MLSTM_SIGNATURES)


def add_normed(x: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
               results: torch.Tensor | None = None, mix: torch.Tensor | None = None) -> torch.Tensor:
    """x += delta / sqrt(mean(delta^2) + eps) * weight, row by row, in place (x float32 [n, width]).

    ``results`` float32 [P, n, width] with ``mix`` float32 [J + 1], J < P: the sum is also written to plane J, and x
    becomes sum_j mix[j] * results[j], j = 0 .. J (the planes below J hold earlier layers' results).

    Returns x in ``out_dtype`` for the branch that reads it next: x itself if that is float32, else a rounded copy
    made in the same pass."""
    _dev("add_normed", x, delta, weight, results, mix)
    _need(x.dim() == 2 and x.dtype == F32 and delta.shape == x.shape, f"add_normed: x {tuple(x.shape)} {x.dtype}, delta {tuple(delta.shape)}")
    n, width = x.shape
    _need(weight.shape == (width,) and weight.dtype == F32, f"add_normed: the norm's weight is float32 [{width}]")
    planes, stride = 0, 0
    if results is not None:
        _need(mix is not None and mix.dtype == F32 and mix.dim() == 1 and results.dtype == F32 and results.dim() == 3
              and results.shape[1:] == x.shape and 1 <= mix.shape[0] <= results.shape[0],
              f"add_normed: results {tuple(results.shape)} {results.dtype} and {None if mix is None else tuple(mix.shape)} weights")
        planes, stride = mix.shape[0], n * width
    else:
        _need(mix is None, "add_normed: weights without results")
    out = x if out_dtype == F32 else torch.empty((n, width), dtype=out_dtype, device=x.device)
    library.call(mixers(), "palm_add_normed", _stream(), _p(x), _p(delta), _code(delta, "add_normed delta"), _p(weight), float(eps),
                 n, width, _p(results), _p(mix), planes, stride, None if out is x else _p(out), _code(out, "add_normed out"))
    return out


def xielu(z: torch.Tensor, pq: torch.Tensor) -> torch.Tensor:
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2, with pq = [p, q] float32."""
    _dev("xielu", z, pq)
    _need(pq.shape == (2,) and pq.dtype == F32, f"xielu: the two numbers are float32 [2], not {pq.dtype} {tuple(pq.shape)}")
    out = torch.empty_like(z)
    library.call(mixers(), "palm_xielu", _stream(), _p(z), _p(out), _code(z, "xielu"), _p(pq), z.numel())
    return out


RETENTION_BLOCKS_WANTED = 512      # a long run of new tokens is cut into chunks until about this many blocks run
RETENTION_MIN_CHUNK = 32


def retention_chunk(n_seqs: int, heads: int, max_new: int) -> int:
    """Into chunks of how many tokens the retention kernel cuts the step's runs of new tokens (0: not at all).  One
    block per (head, sequence) walks over its tokens one after the other; where that leaves most of the chip idle and
    the runs are long, chunks run side by side at the price of walking over every token twice."""
    per_seq = RETENTION_BLOCKS_WANTED // max(1, heads * n_seqs)
    if max_new <= 2 * RETENTION_MIN_CHUNK or per_seq <= 1:
        return 0
    chunk = max(RETENTION_MIN_CHUNK, -(-max_new // per_seq))
    chunk = (chunk + 7) // 8 * 8
    return chunk if chunk < max_new else 0


def retention(qkvg: torch.Tensor, heads: int, dim: int, vdim: int, decay: torch.Tensor, k_scale: float, eps: float,
              state: torch.Tensor, ctx, cos=None, sin=None, rot: int = 0, chunk: int | None = None, input_silu: bool = False,
              joined_norm: torch.Tensor | None = None, gate_sigmoid: bool = False, col0: int = 0) -> torch.Tensor:
    """The step's tokens through a retention layer's recurrence.  qkvg [n, heads * (2 dim + 2 vdim)] holds q | k | v |
    gate; state float32 [slots, heads, dim, vdim] is read and left updated.  Returns [n, heads * vdim]: the heads'
    outputs, unit-normed per head and gated by silu of the gate.  ``chunk``: see ``retention_chunk`` (None: chosen here).

    ``input_silu``: q, k and v go through silu first.  ``joined_norm`` (float32 [heads * vdim]): instead of the unit norm
    per head, a token's joined heads are normed together and multiplied by this weight; ``gate_sigmoid``: the gate is then
    sigmoid of the gate values instead of silu.  ``col0``: q | k | v | gate begin at this column of wider rows (a product
    that several mixers share)."""
    _dev("retention", qkvg, decay, state, cos, sin, ctx.seq_slot, ctx.seq_new, ctx.cu_new)
    _i32("retention", ctx.seq_slot, ctx.seq_new, ctx.cu_new)
    n = qkvg.shape[0]
    _need(qkvg.dim() == 2 and col0 >= 0 and qkvg.shape[1] >= col0 + heads * (2 * dim + 2 * vdim) and (col0 or qkvg.shape[1] == heads * (2 * dim + 2 * vdim)),
          f"retention: rows {tuple(qkvg.shape)} from column {col0} are not [n, {heads} * (2*{dim} + 2*{vdim})]")
    _need(decay.shape == (heads,) and decay.dtype == F32, f"retention: one float32 decay for each of {heads} heads")
    _need(state.dim() == 4 and state.shape[1:] == (heads, dim, vdim) and state.dtype == F32,
          f"retention: state {tuple(state.shape)} {state.dtype} is not float32 [slots, {heads}, {dim}, {vdim}]")
    _need(n == ctx.n_tokens, "retention: one row for each token of the step")
    if rot:
        for tab in (cos, sin):
            _need(tab is not None and tab.dtype == F32 and tab.shape == (n, rot // 2), f"retention: rotation rows are float32 [{n}, {rot // 2}]")
    out = torch.empty((n, heads * vdim), dtype=qkvg.dtype, device=qkvg.device)
    raw = None
    if joined_norm is not None:
        _dev("retention", joined_norm)
        _need(joined_norm.shape == (heads * vdim,) and joined_norm.dtype == F32, f"retention: the joined heads' norm weight is float32 [{heads * vdim}]")
        raw = torch.empty((n, heads * vdim), dtype=F32, device=qkvg.device)
    else:
        _need(not gate_sigmoid, "retention: the per-head unit norm comes with a silu gate")
    chunk = retention_chunk(ctx.n_seqs, heads, ctx.max_new) if chunk is None else int(chunk)
    # q and k after the rotation, 32-bit, in rows padded to the key size that the kernel is compiled for
    rotated = torch.empty((n, heads, 2, recurrent().palm_retention_pad(dim)), dtype=F32, device=qkvg.device)
    starts = None
    if chunk:
        max_chunks = -(-ctx.max_new // chunk)
        starts = torch.empty((ctx.n_seqs * max_chunks, heads, dim, vdim), dtype=F32, device=qkvg.device)
    g_off = col0 + 2 * heads * dim + heads * vdim
    library.call(recurrent(), "palm_retention", _stream(), _p(qkvg), _code(qkvg, "retention"), qkvg.shape[1], col0, col0 + heads * dim,
                 col0 + 2 * heads * dim, g_off, _p(cos), _p(sin), int(rot), _p(decay), float(k_scale), float(eps),
                 _p(state), _p(ctx.seq_slot), _p(ctx.seq_new), _p(ctx.cu_new), ctx.n_seqs, heads, dim, vdim, _p(out),
                 int(ctx.max_new), chunk, _p(starts), n, _p(rotated), int(input_silu), int(raw is not None), _p(raw))
    if raw is not None:
        library.call(recurrent(), "palm_joined_norm_gate", _stream(), _p(raw), _p(joined_norm), float(eps),
                     qkvg.data_ptr() + g_off * qkvg.element_size(), _code(qkvg, "retention"), qkvg.shape[1], int(gate_sigmoid), n,
                     heads * vdim, _p(out))
    return out


def causal_conv(xz: torch.Tensor, channels: int, weight: torch.Tensor, bias: torch.Tensor | None, conv_state: torch.Tensor, ctx) -> torch.Tensor:
    """silu(bias + a causal convolution per channel) (``bias`` None: none) over the first ``channels`` columns of xz [n, >= channels];
    weight float32 [channels, taps] (last column: the current token), conv_state float32 [slots, taps - 1, channels]:
    each sequence's last inputs, read and left updated."""
    _dev("causal_conv", xz, weight, bias, conv_state, ctx.seq_slot, ctx.seq_new, ctx.cu_new)
    _i32("causal_conv", ctx.seq_slot, ctx.seq_new, ctx.cu_new)
    taps = weight.shape[1]
    _need(xz.dim() == 2 and xz.shape[1] >= channels and xz.shape[0] == ctx.n_tokens, f"causal_conv: input {tuple(xz.shape)}")
    _need(weight.shape == (channels, taps) and weight.dtype == F32 and (bias is None or (bias.shape == (channels,) and bias.dtype == F32)),
          f"causal_conv: weight {tuple(weight.shape)} {weight.dtype}, bias {None if bias is None else tuple(bias.shape)}")
    _need(conv_state.dim() == 3 and conv_state.shape[1:] == (max(taps - 1, 0), channels) and conv_state.dtype == F32,
          f"causal_conv: state {tuple(conv_state.shape)} is not float32 [slots, {taps - 1}, {channels}]")
    out = torch.empty((xz.shape[0], channels), dtype=xz.dtype, device=xz.device)
    library.call(mixers(), "palm_causal_conv", _stream(), _p(xz), _code(xz, "causal_conv"), xz.shape[1], _p(weight), _p(bias),
                 _p(conv_state), _p(ctx.seq_slot), _p(ctx.seq_new), _p(ctx.cu_new), ctx.n_seqs, ctx.max_new, channels, taps, _p(out))
    return out


def selective_scan(u: torch.Tensor, xz: torch.Tensor, bc: torch.Tensor, b_off: int, c_off: int, dt_linear: torch.Tensor,
                   dt_bias: torch.Tensor, a_log: torch.Tensor, d_skip: torch.Tensor, state: torch.Tensor, ctx) -> torch.Tensor:
    """u [n, C] (the convolution's output), the gate z = xz[:, C:2C], B = bc[:, b_off:b_off+N], C = bc[:, c_off:c_off+N],
    dt_linear float32 [n, C] (before bias and softplus), a_log float32 [C, N], state float32 [slots, C, N] read and
    left updated.  Returns y * silu(z), [n, C]."""
    _dev("selective_scan", u, xz, bc, dt_linear, dt_bias, a_log, d_skip, state, ctx.seq_slot, ctx.seq_new, ctx.cu_new)
    _i32("selective_scan", ctx.seq_slot, ctx.seq_new, ctx.cu_new)
    n, C = u.shape
    N = a_log.shape[1]
    _need(xz.shape == (n, 2 * C) and xz.dtype == u.dtype and bc.dtype == u.dtype and bc.dim() == 2 and bc.shape[0] == n
          and 0 <= b_off and b_off + N <= bc.shape[1] and 0 <= c_off and c_off + N <= bc.shape[1],
          f"selective_scan: u {tuple(u.shape)}, xz {tuple(xz.shape)}, bc {tuple(bc.shape)}")
    _need(dt_linear.shape == (n, C) and dt_linear.dtype == F32, f"selective_scan: step sizes {tuple(dt_linear.shape)} {dt_linear.dtype} are float32 [{n}, {C}]")
    for v, nm in ((dt_bias, "dt bias"), (d_skip, "D")):
        _need(v.shape == (C,) and v.dtype == F32, f"selective_scan: {nm} is float32 [{C}]")
    _need(a_log.shape == (C, N) and a_log.dtype == F32, f"selective_scan: A_log {tuple(a_log.shape)} {a_log.dtype}")
    _need(state.dim() == 3 and state.shape[1:] == (C, N) and state.dtype == F32, f"selective_scan: state {tuple(state.shape)} {state.dtype}")
    _need(n == ctx.n_tokens, "selective_scan: one row for each token of the step")
    out = torch.empty((n, C), dtype=u.dtype, device=u.device)
    library.call(mixers(), "palm_selective_scan", _stream(), _p(u), xz.data_ptr() + C * xz.element_size(), 2 * C, _p(bc), bc.shape[1],
                 int(b_off), int(c_off), _code(u, "selective_scan"), _p(dt_linear), _p(dt_bias), _p(a_log), _p(d_skip), _p(state),
                 _p(ctx.seq_slot), _p(ctx.seq_new), _p(ctx.cu_new), ctx.n_seqs, C, N, _p(out))
    return out


def _check_diff_cache(what, k_cache, v_cache, block_table, kv_heads, dim, vdim):
    _need(k_cache.dim() == 4 and k_cache.shape[1:] == (2 * kv_heads, PAGE_TOKENS, dim),
          f"{what}: key cache {tuple(k_cache.shape)} is not [pages, 2*{kv_heads}, {PAGE_TOKENS}, {dim}]")
    _need(v_cache.shape == (k_cache.shape[0], kv_heads, vdim, PAGE_TOKENS) and v_cache.dtype == k_cache.dtype,
          f"{what}: value cache {tuple(v_cache.shape)} is not [pages, {kv_heads}, {vdim}, {PAGE_TOKENS}]")
    _need(block_table.dim() == 2, f"{what}: page table {tuple(block_table.shape)} is not [slots, pages]")


def diff_qkv_store(qkv: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, q_norm_w, k_norm_w, eps: float,
                   k_cache, v_cache, block_table, ctx, write_cache: bool = True) -> torch.Tensor:
    """qkv [n, 2 heads dim + 2 kv_heads dim + kv_heads vdim] -> q [n, 2 heads dim], RMS-normed per head and map; k
    (normed likewise) and v go to the cache page of each token."""
    what = "diff_qkv_store"
    _dev(what, qkv, q_norm_w, k_norm_w, k_cache, v_cache, block_table, ctx.tok_slot, ctx.positions)
    _i32(what, block_table, ctx.tok_slot, ctx.positions)
    n = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == 2 * (heads + kv_heads) * dim + kv_heads * vdim, f"{what}: rows {tuple(qkv.shape)}")
    for w in (q_norm_w, k_norm_w):
        _need(w.shape == (dim,) and w.dtype == F32, f"{what}: a norm weight is float32 [{dim}]")
    _check_diff_cache(what, k_cache, v_cache, block_table, kv_heads, dim, vdim)
    _need(k_cache.dtype == qkv.dtype, f"{what}: cache is {k_cache.dtype}, activations are {qkv.dtype}")
    _need(n == ctx.n_tokens, f"{what}: one row for each token of the step")
    q = torch.empty((n, 2 * heads * dim), dtype=qkv.dtype, device=qkv.device)
    library.call(mixers(), "palm_diff_qkv_store", _stream(), _p(qkv), _code(qkv, what), _p(q), _p(k_cache), _p(v_cache), _p(block_table),
                 block_table.shape[1], _p(ctx.tok_slot), _p(ctx.positions), _p(q_norm_w), _p(k_norm_w), float(eps), n, heads, kv_heads,
                 dim, vdim, int(write_cache))
    return q


DIFF_BLOCKS_WANTED = 1024         # a decode step's key ranges are cut into slices until about this many blocks run


def diff_slices(ctx, heads: int) -> int:
    """Into how many slices the exact kernel cuts every key range: only a decode step's (few queries, long ranges)."""
    if not ctx.is_decode:
        return 1
    pages = max(1, (ctx.max_total + PAGE_TOKENS - 1) // PAGE_TOKENS)
    return max(1, min(pages, DIFF_BLOCKS_WANTED // max(1, ctx.n_seqs * heads), 64))


def attention_diff_exact(q: torch.Tensor, k_cache, v_cache, block_table, ctx, heads: int, kv_heads: int, dim: int, vdim: int,
                         scale: float, lam: float, gain: float, eps: float, n_slices: int | None = None) -> torch.Tensor:
    """Differential attention of the step's queries over the cache in 32-bit arithmetic: out [n, heads * vdim] =
    unit_rms(a1 - lam * a2) * gain per head.  ``n_slices``: see ``diff_slices`` (None: chosen here)."""
    what = "attention_diff"
    _dev(what, q, k_cache, v_cache, block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new)
    _i32(what, block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new)
    n = q.shape[0]
    _need(q.dim() == 2 and q.shape[1] == 2 * heads * dim and n == ctx.n_tokens, f"{what}: q {tuple(q.shape)} is not [n, 2*{heads}*{dim}]")
    _check_diff_cache(what, k_cache, v_cache, block_table, kv_heads, dim, vdim)
    _need(k_cache.dtype == q.dtype, f"{what}: cache is {k_cache.dtype}, queries are {q.dtype}")
    out = torch.empty((n, heads * vdim), dtype=q.dtype, device=q.device)
    n_slices = diff_slices(ctx, heads) if n_slices is None else int(n_slices)
    _need(n_slices == 1 or ctx.is_decode, f"{what}: only a decode step's key ranges are cut into slices")
    work = torch.empty((n * heads * n_slices * 2 * (vdim + 2),), dtype=F32, device=q.device) if n_slices > 1 else None
    library.call(mixers(), "palm_attention_diff", _stream(), _p(q), _code(q, what), _p(k_cache), _p(v_cache), _p(block_table),
                 block_table.shape[1], _p(ctx.seq_slot), _p(ctx.seq_start), _p(ctx.seq_new), _p(ctx.cu_new), ctx.n_seqs, int(ctx.max_new),
                 heads, kv_heads, dim, vdim, float(scale), float(lam), float(gain), float(eps), _p(out), n_slices, _p(work), n)
    return out


_DIFF_MFMA_SIGNATURE = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                        c_int, c_int, c_int, c_int, c_float, c_float, c_float, c_float, c_void_p]
_diff_libs: dict = {}
DIFF_MFMA_MAX_DIM, DIFF_MFMA_MAX_VDIM = 256, 256


def diff_mfma_serves(q: torch.Tensor, dim: int, vdim: int) -> bool:
    """The matrix-core kernel takes bfloat16, key sizes in steps of 8 and value sizes in steps of 4, up to 256."""
    return q.dtype == BF16 and dim % 8 == 0 and vdim % 4 == 0 and dim <= DIFF_MFMA_MAX_DIM and vdim <= DIFF_MFMA_MAX_VDIM


def diff_query_tiles(vdim: int) -> int:
    """Tiles of 16 queries a wave of the matrix-core kernel: two where the output tiles of both maps then still fit a
    lane's registers (measured: key size 64, value size 128: 224 us with two against 274 with one; 128 and 256: 1,025
    against 590).  ``PALM_DIFF_QUERY_TILES`` in the environment overrides the choice, for such measurements."""
    import os
    forced = os.environ.get("PALM_DIFF_QUERY_TILES")
    if forced:
        return int(forced)
    return 2 if (vdim + 15) // 16 <= 8 else 1


def attention_diff_lib(dim: int, vdim: int):
    key = ((dim + 31) // 32, (vdim + 15) // 16, diff_query_tiles(vdim))
    if key not in _diff_libs:
        lib = library.load(f"attention_diff_k{key[0]}_v{key[1]}_q{key[2]}")
        lib.palm_attention_diff_mfma.argtypes, lib.palm_attention_diff_mfma.restype = _DIFF_MFMA_SIGNATURE, c_int
        lib.palm_attention_diff_mfma_sizes.argtypes, lib.palm_attention_diff_mfma_sizes.restype = [c_int], c_int
        if tuple(lib.palm_attention_diff_mfma_sizes(i) for i in range(3)) != (key[0] * 32, key[1] * 16, key[2]):
            raise KernelError(f"library attention_diff_k{key[0]}_v{key[1]}_q{key[2]} was built for other sizes")
        _diff_libs[key] = lib
    return _diff_libs[key]


def attention_diff_mfma(q: torch.Tensor, k_cache, v_cache, block_table, ctx, heads: int, kv_heads: int, dim: int, vdim: int,
                        scale: float, lam: float, gain: float, eps: float) -> torch.Tensor:
    """As ``attention_diff_exact`` for bfloat16 prompts, both products on the matrix cores."""
    what = "attention_diff_mfma"
    _dev(what, q, k_cache, v_cache, block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new)
    _i32(what, block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new)
    n = q.shape[0]
    _need(diff_mfma_serves(q, dim, vdim), f"{what}: {q.dtype}, key size {dim}, value size {vdim}")
    _need(q.dim() == 2 and q.shape[1] == 2 * heads * dim and n == ctx.n_tokens, f"{what}: q {tuple(q.shape)} is not [n, 2*{heads}*{dim}]")
    _check_diff_cache(what, k_cache, v_cache, block_table, kv_heads, dim, vdim)
    _need(k_cache.dtype == BF16, f"{what}: the cache is {k_cache.dtype}, not bfloat16")
    out = torch.empty((n, heads * vdim), dtype=BF16, device=q.device)
    library.call(attention_diff_lib(dim, vdim), "palm_attention_diff_mfma", _stream(), _p(q), _p(k_cache), _p(v_cache), _p(block_table),
                 block_table.shape[1], _p(ctx.seq_slot), _p(ctx.seq_start), _p(ctx.seq_new), _p(ctx.cu_new), ctx.n_seqs, int(ctx.max_new),
                 heads, kv_heads, dim, vdim, float(scale), float(lam), float(gain), float(eps), _p(out))
    return out


def attention_diff(q, k_cache, v_cache, block_table, ctx, heads, kv_heads, dim, vdim, scale, lam, gain, eps):
    """The step's queries over the cache; picks the kernel by element type and step shape: prompts (and portions of
    them) in bfloat16 go to the matrix cores, single tokens and the float32 mode to the exact kernel."""
    if not ctx.is_decode and diff_mfma_serves(q, dim, vdim):
        return attention_diff_mfma(q, k_cache, v_cache, block_table, ctx, heads, kv_heads, dim, vdim, scale, lam, gain, eps)
    return attention_diff_exact(q, k_cache, v_cache, block_table, ctx, heads, kv_heads, dim, vdim, scale, lam, gain, eps)


# ---- blocks that norm a branch on both sides; a cap on the logits -------------------------------------------------

def add_normed_scaled(x: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor, eps: float, gain: float,
                      next_weight: torch.Tensor | None = None, next_eps: float = 0.0, out_dtype: torch.dtype | None = None):
    """x += gain * (delta / sqrt(mean(delta^2) + eps) * weight), row by row, in place (x float32 [n, width]).  With
    ``next_weight``: also returns x / sqrt(mean(x^2) + next_eps) * next_weight in ``out_dtype``, made in the same pass
    (what the norm that reads the stream next would give); else returns None."""
    _dev("add_normed_scaled", x, delta, weight, next_weight)
    _need(x.dim() == 2 and x.dtype == F32 and delta.shape == x.shape, f"add_normed_scaled: x {tuple(x.shape)} {x.dtype}, delta {tuple(delta.shape)}")
    n, width = x.shape
    for w in (weight, next_weight):
        _need(w is None or (w.shape == (width,) and w.dtype == F32), f"add_normed_scaled: a norm's weight is float32 [{width}]")
    out = None
    if next_weight is not None:
        out = torch.empty((n, width), dtype=out_dtype or F32, device=x.device)
    library.call(mixers(), "palm_add_normed_scaled", _stream(), _p(x), _p(delta), _code(delta, "add_normed_scaled delta"), _p(weight),
                 float(eps), float(gain), n, width, _p(next_weight), float(next_eps), _p(out),
                 _code(out, "add_normed_scaled out") if out is not None else 0)
    return out


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits <- cap * tanh(logits / cap), in place (float32).  Returns logits."""
    _dev("softcap", logits)
    _need(logits.dtype == F32 and cap > 0, f"softcap: float32 logits and a positive cap, not {logits.dtype} and {cap}")
    library.call(mixers(), "palm_softcap", _stream(), _p(logits), float(cap), logits.numel())
    return logits


# ---- the delta rule ------------------------------------------------------------------------------------------------

DELTA_BLOCKS_WANTED = 512          # a long run of new tokens is cut into chunks until about this many blocks run
DELTA_MIN_CHUNK = 64


def delta_chunk(n_seqs: int, heads: int, max_new: int) -> int:
    """Into chunks of how many tokens the delta rule's kernel cuts the step's runs of new tokens (0: not at all).  One block
    per (head, sequence) walks over its tokens one after the other; where that leaves most of the chip idle and the runs
    are long, chunks run side by side at the price of walking over every token twice, over the key size more columns the
    first time, and of a small product for every chunk between the two walks."""
    per_seq = DELTA_BLOCKS_WANTED // max(1, heads * n_seqs)
    if max_new <= 2 * DELTA_MIN_CHUNK or per_seq <= 1:
        return 0
    chunk = max(DELTA_MIN_CHUNK, -(-max_new // per_seq))
    chunk = (chunk + 7) // 8 * 8
    return chunk if chunk < max_new else 0


def delta_rule(u: torch.Tensor, offsets: tuple, b: torch.Tensor, a: torch.Tensor, gate: torch.Tensor, a_log: torch.Tensor,
               dt_bias: torch.Tensor, norm_w: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, q_scale: float,
               unit_eps: float, eps: float, state: torch.Tensor, ctx, chunk: int | None = None) -> torch.Tensor:
    """The step's tokens through the recurrence of a gated delta rule with one decay per key channel.

    u [n, >= 2 kv_heads dim + heads vdim]: the convolution's output with q, k, v at the columns ``offsets``; b [n, heads]
    (a view of rows is fine: its row stride is passed on): the write strengths before the sigmoid; a float32 [n, heads * dim]
    and gate float32 [n, heads * vdim] (views likewise): the decays' rows before bias and softplus, the output gate before
    its sigmoid; state float32 [slots, heads, dim, vdim], read and left updated.  Returns [n, heads * vdim]: the heads'
    outputs, each normed over vdim with ``norm_w`` and gated.  ``chunk``: see ``delta_chunk`` (None: chosen here)."""
    what = "delta_rule"
    _dev(what, u, a_log, dt_bias, norm_w, state, ctx.seq_slot, ctx.seq_new, ctx.cu_new)
    _i32(what, ctx.seq_slot, ctx.seq_new, ctx.cu_new)
    n = u.shape[0]
    q_off, k_off, v_off = (int(o) for o in offsets)
    _need(u.dim() == 2 and n == ctx.n_tokens and max(q_off, k_off) + kv_heads * dim <= u.shape[1] and v_off + heads * vdim <= u.shape[1],
          f"{what}: rows {tuple(u.shape)} do not hold q, k ({kv_heads} x {dim}) and v ({heads} x {vdim}) at {offsets}")
    for t, cols, dt, nm in ((b, heads, u.dtype, "write strengths"), (a, heads * dim, F32, "decay rows"), (gate, heads * vdim, F32, "gate rows")):
        _need(t.is_cuda and t.dim() == 2 and t.shape == (n, cols) and t.dtype == dt and (n == 0 or t.stride(1) == 1),
              f"{what}: the {nm} are {dt} [{n}, {cols}] with contiguous rows, not {t.dtype} {tuple(t.shape)}")
    _need(a_log.shape == (heads,) and a_log.dtype == F32 and dt_bias.shape == (heads * dim,) and dt_bias.dtype == F32
          and norm_w.shape == (vdim,) and norm_w.dtype == F32, f"{what}: A_log [{heads}], dt_bias [{heads * dim}] and the norm's weight [{vdim}] are float32")
    _need(state.dim() == 4 and state.shape[1:] == (heads, dim, vdim) and state.dtype == F32,
          f"{what}: state {tuple(state.shape)} {state.dtype} is not float32 [slots, {heads}, {dim}, {vdim}]")
    out = torch.empty((n, heads * vdim), dtype=u.dtype, device=u.device)
    prep = torch.empty((n, heads, 3, mixers().palm_delta_pad(dim)), dtype=F32, device=u.device)
    beta = torch.empty((n, heads), dtype=F32, device=u.device)
    chunk = delta_chunk(ctx.n_seqs, heads, ctx.max_new) if chunk is None else int(chunk)
    ext = starts = None
    if chunk:
        chunks = ctx.n_seqs * (-(-ctx.max_new // chunk))
        ext = torch.empty((chunks, heads, dim, vdim + dim), dtype=F32, device=u.device)
        starts = torch.empty((chunks, heads, dim, vdim), dtype=F32, device=u.device)
    library.call(mixers(), "palm_delta_rule", _stream(), _p(u), _code(u, what), u.stride(0), q_off, k_off, v_off, _p(b), b.stride(0),
                 _p(a), a.stride(0), _p(gate), gate.stride(0), _p(a_log), _p(dt_bias), _p(norm_w), float(q_scale), float(unit_eps),
                 float(eps), _p(state), _p(ctx.seq_slot), _p(ctx.seq_new), _p(ctx.cu_new), ctx.n_seqs, heads, kv_heads, dim, vdim,
                 _p(out), n, _p(prep), _p(beta), int(ctx.max_new), chunk, _p(ext), _p(starts))
    return out


# ---- attention over one compressed row per position -----------------------------------------------------------------

def latent_prep(down: torch.Tensor, q_rank: int, kv_off: int, kv_rank: int, rot_dim: int, q_norm_w, kv_norm_w, eps: float,
                cos, sin, rows_cache: torch.Tensor, block_table: torch.Tensor, ctx, write_cache: bool = True,
                rows_t: torch.Tensor | None = None, table_t: torch.Tensor | None = None) -> torch.Tensor:
    """down [n, >= kv_off + kv_rank + rot_dim]: the query latent at column 0, the key/value latent at ``kv_off`` and the key
    part to rotate behind it.  Returns the normed query latent [n, q_rank]; writes [normed latent | rotated key part] into
    each token's row of ``rows_cache`` [pages, PAGE_TOKENS, kv_rank + rot_dim] and, if given, the normed latent into
    ``rows_t`` (bfloat16 [pages, kv_rank, PAGE_TOKENS], with the page table ``table_t`` of its own)."""
    what = "latent_prep"
    _dev(what, down, q_norm_w, kv_norm_w, cos, sin, rows_cache, block_table, ctx.positions, ctx.tok_slot, rows_t, table_t)
    _i32(what, block_table, ctx.positions, ctx.tok_slot, table_t)
    _need(rows_t is None or (table_t is not None and rows_t.dtype == BF16 and rows_t.dim() == 3 and rows_t.shape[1:] == (kv_rank, PAGE_TOKENS)
                             and table_t.shape == block_table.shape),
          f"{what}: the transposed copy is bfloat16 [pages, {kv_rank}, {PAGE_TOKENS}] with a page table like the rows'")
    n = down.shape[0]
    _need(down.dim() == 2 and n == ctx.n_tokens, f"{what}: rows {tuple(down.shape)} for {ctx.n_tokens} tokens")
    _need(q_norm_w.shape == (q_rank,) and q_norm_w.dtype == F32 and kv_norm_w.shape == (kv_rank,) and kv_norm_w.dtype == F32,
          f"{what}: the norms' weights are float32 [{q_rank}] and [{kv_rank}]")
    _need(rows_cache.dim() == 3 and rows_cache.shape[1:] == (PAGE_TOKENS, kv_rank + rot_dim) and rows_cache.dtype == down.dtype,
          f"{what}: the cache {tuple(rows_cache.shape)} {rows_cache.dtype} is not {down.dtype} [pages, {PAGE_TOKENS}, {kv_rank + rot_dim}]")
    if rot_dim:
        for tab in (cos, sin):
            _need(tab is not None and tab.dtype == F32 and tab.shape == (n, rot_dim // 2), f"{what}: rotation rows are float32 [{n}, {rot_dim // 2}]")
    _need(block_table.dim() == 2, f"{what}: page table {tuple(block_table.shape)} is not [slots, pages]")
    cq = torch.empty((n, q_rank), dtype=down.dtype, device=down.device)
    library.call(mixers(), "palm_latent_prep", _stream(), _p(down), _code(down, what), down.shape[1], q_rank, kv_off, kv_rank, rot_dim,
                 _p(q_norm_w), _p(kv_norm_w), float(eps), _p(cos), _p(sin), _p(ctx.positions), _p(ctx.tok_slot), _p(block_table),
                 block_table.shape[1], _p(rows_cache), int(write_cache), _p(cq), n, _p(rows_t), _p(table_t))
    return cq


def latent_query(q: torch.Tensor, uk: torch.Tensor, cos, sin, heads: int, dim: int, rot_dim: int, kv_rank: int) -> torch.Tensor:
    """q [n, heads * (dim + rot_dim)], uk [heads * dim, kv_rank] -> float32 [n, heads, kv_rank + rot_dim]: each head's plain
    part taken through its key matrix, its rotated part behind it."""
    what = "latent_query"
    _dev(what, q, uk, cos, sin)
    n = q.shape[0]
    _need(q.dim() == 2 and q.shape[1] == heads * (dim + rot_dim) and uk.shape == (heads * dim, kv_rank),
          f"{what}: q {tuple(q.shape)}, key matrix {tuple(uk.shape)} for {heads} heads of {dim} + {rot_dim} and a latent of {kv_rank}")
    if rot_dim:
        for tab in (cos, sin):
            _need(tab is not None and tab.dtype == F32 and tab.shape == (n, rot_dim // 2), f"{what}: rotation rows are float32 [{n}, {rot_dim // 2}]")
    qa = torch.empty((n, heads, kv_rank + rot_dim), dtype=F32, device=q.device)
    library.call(mixers(), "palm_latent_query", _stream(), _p(q), _code(q, what), _p(uk), _code(uk, what + " key matrix"), _p(cos), _p(sin),
                 n, heads, dim, rot_dim, kv_rank, _p(qa))
    return qa


_LATENT_MFMA_SIGNATURE = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                          c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]
_latent_libs: dict = {}
LATENT_MFMA_MAX_ROW, LATENT_MFMA_MAX_RANK = 640, 512


def latent_mfma_serves(rows_cache: torch.Tensor, kv_rank: int, rot_dim: int) -> bool:
    """The matrix-core kernel takes bfloat16 rows whose sizes are multiples of eight, up to 640 values a row and a latent of 512."""
    return (rows_cache.dtype == BF16 and kv_rank % 8 == 0 and (kv_rank + rot_dim) % 8 == 0 and kv_rank + rot_dim <= LATENT_MFMA_MAX_ROW
            and kv_rank <= LATENT_MFMA_MAX_RANK)


def latent_attention_lib(kv_rank: int, rot_dim: int):
    key = ((kv_rank + rot_dim + 31) // 32, (kv_rank + 15) // 16)
    if key not in _latent_libs:
        lib = library.load(f"latent_attention_k{key[0]}_v{key[1]}")
        lib.palm_latent_attention_mfma.argtypes, lib.palm_latent_attention_mfma.restype = _LATENT_MFMA_SIGNATURE, c_int
        lib.palm_latent_attention_mfma_sizes.argtypes, lib.palm_latent_attention_mfma_sizes.restype = [c_int], c_int
        if tuple(lib.palm_latent_attention_mfma_sizes(i) for i in range(2)) != (key[0] * 32, key[1] * 16):
            raise KernelError(f"library latent_attention_k{key[0]}_v{key[1]} was built for other sizes")
        _latent_libs[key] = lib
    return _latent_libs[key]


def latent_attention(qa: torch.Tensor, rows_cache: torch.Tensor, block_table: torch.Tensor, ctx, heads: int, kv_rank: int,
                     rot_dim: int, scale: float, window: int | None, rows_t: torch.Tensor | None = None,
                     table_t: torch.Tensor | None = None) -> torch.Tensor:
    """Softmax attention of the step's queries (float32 [n, heads, kv_rank + rot_dim]) over the cached rows of their own
    sequences up to their own positions (the last ``window`` of them if set): float32 [n, heads, kv_rank], the weighted sums
    of the rows' latents.  Prompts (and portions of them) in bfloat16 go to the matrix cores if the caller keeps the
    transposed copy of the latents (``rows_t`` [pages, kv_rank, PAGE_TOKENS] with its page table); single tokens, the
    float32 mode and sizes that kernel does not take go to the exact kernel."""
    what = "latent_attention"
    _dev(what, qa, rows_cache, block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new, rows_t, table_t)
    _i32(what, block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new, table_t)
    n = qa.shape[0]
    _need(qa.shape == (n, heads, kv_rank + rot_dim) and qa.dtype == F32 and n == ctx.n_tokens, f"{what}: queries {tuple(qa.shape)} {qa.dtype}")
    _need(rows_cache.dim() == 3 and rows_cache.shape[1:] == (PAGE_TOKENS, kv_rank + rot_dim),
          f"{what}: the cache {tuple(rows_cache.shape)} is not [pages, {PAGE_TOKENS}, {kv_rank + rot_dim}]")
    _need(block_table.dim() == 2, f"{what}: page table {tuple(block_table.shape)} is not [slots, pages]")
    out = torch.empty((n, heads, kv_rank), dtype=F32, device=qa.device)
    if rows_t is not None and not ctx.is_decode and latent_mfma_serves(rows_cache, kv_rank, rot_dim):
        _need(table_t is not None and rows_t.dtype == BF16 and rows_t.dim() == 3 and rows_t.shape[1:] == (kv_rank, PAGE_TOKENS)
              and table_t.shape == block_table.shape, f"{what}: the transposed copy is bfloat16 [pages, {kv_rank}, {PAGE_TOKENS}] with a page "
              "table like the rows'")
        library.call(latent_attention_lib(kv_rank, rot_dim), "palm_latent_attention_mfma", _stream(), _p(qa), _p(rows_cache), _p(rows_t),
                     _p(block_table), _p(table_t), block_table.shape[1], _p(ctx.seq_slot), _p(ctx.seq_start), _p(ctx.seq_new), _p(ctx.cu_new),
                     ctx.n_seqs, int(ctx.max_new), heads, kv_rank, rot_dim, float(scale), int(window or 0), _p(out), None, None, 0, 0, None)
        return out
    library.call(mixers(), "palm_latent_attention", _stream(), _p(qa), _p(rows_cache), _code(rows_cache, what), _p(block_table),
                 block_table.shape[1], _p(ctx.seq_slot), _p(ctx.seq_start), _p(ctx.seq_new), _p(ctx.cu_new), ctx.n_seqs, int(ctx.max_new),
                 heads, kv_rank, rot_dim, float(scale), int(window or 0), _p(out))
    return out


def latent_fused_serves(qa: torch.Tensor, rows_cache: torch.Tensor, rows_t, uv: torch.Tensor, ctx, kv_rank: int, rot_dim: int, vdim: int) -> bool:
    """Whether the prompt kernel on the matrix cores also applies the value matrices: a prompt (or a portion) in bfloat16 with
    the transposed copy of the latents at hand, bfloat16 matrices, a value size that is a multiple of four."""
    return (rows_t is not None and not ctx.is_decode and uv.dtype == BF16 and vdim % 4 == 0 and latent_mfma_serves(rows_cache, kv_rank, rot_dim))


def latent_attention_fused(qa: torch.Tensor, rows_cache: torch.Tensor, block_table: torch.Tensor, ctx, heads: int, kv_rank: int,
                           rot_dim: int, scale: float, window: int | None, rows_t: torch.Tensor, table_t: torch.Tensor, uv: torch.Tensor,
                           gate: torch.Tensor | None, vdim: int) -> torch.Tensor:
    """``latent_attention`` on the matrix cores and ``latent_output`` in one kernel: bfloat16 [n, heads * vdim]."""
    what = "latent_attention_fused"
    _dev(what, qa, rows_cache, block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new, rows_t, table_t, uv)
    _i32(what, block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new, table_t)
    n = qa.shape[0]
    _need(latent_fused_serves(qa, rows_cache, rows_t, uv, ctx, kv_rank, rot_dim, vdim), f"{what}: a prompt in bfloat16 with sizes the kernel takes")
    _need(qa.shape == (n, heads, kv_rank + rot_dim) and qa.dtype == F32 and n == ctx.n_tokens, f"{what}: queries {tuple(qa.shape)} {qa.dtype}")
    _need(rows_cache.dim() == 3 and rows_cache.shape[1:] == (PAGE_TOKENS, kv_rank + rot_dim) and rows_t.dtype == BF16 and rows_t.dim() == 3
          and rows_t.shape[1:] == (kv_rank, PAGE_TOKENS) and block_table.dim() == 2 and table_t.shape == block_table.shape,
          f"{what}: the cache {tuple(rows_cache.shape)}, its transposed copy {tuple(rows_t.shape)}, page tables {tuple(block_table.shape)}")
    _need(uv.shape == (heads * vdim, kv_rank), f"{what}: value matrix {tuple(uv.shape)} for {heads} heads of {vdim} over a latent of {kv_rank}")
    _need(gate is None or (gate.is_cuda and gate.shape == (n, heads) and gate.dtype == BF16 and (n == 0 or gate.stride(1) == 1)),
          f"{what}: the gate is bfloat16 [{n}, {heads}] with contiguous rows")
    out = torch.empty((n, heads * vdim), dtype=BF16, device=qa.device)
    library.call(latent_attention_lib(kv_rank, rot_dim), "palm_latent_attention_mfma", _stream(), _p(qa), _p(rows_cache), _p(rows_t),
                 _p(block_table), _p(table_t), block_table.shape[1], _p(ctx.seq_slot), _p(ctx.seq_start), _p(ctx.seq_new), _p(ctx.cu_new),
                 ctx.n_seqs, int(ctx.max_new), heads, kv_rank, rot_dim, float(scale), int(window or 0), None, _p(uv), _p(gate),
                 gate.stride(0) if gate is not None else 0, vdim, _p(out))
    return out


def latent_output(o_lat: torch.Tensor, uv: torch.Tensor, gate: torch.Tensor | None, heads: int, kv_rank: int, vdim: int,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """o_lat float32 [n, heads, kv_rank], uv [heads * vdim, kv_rank], gate [n, heads] (a view of rows is fine) or None ->
    [n, heads * vdim]: head h's latent sum through its value matrix, times sigmoid(gate[:, h])."""
    what = "latent_output"
    _dev(what, o_lat, uv)
    n = o_lat.shape[0]
    _need(o_lat.shape == (n, heads, kv_rank) and o_lat.dtype == F32 and uv.shape == (heads * vdim, kv_rank),
          f"{what}: sums {tuple(o_lat.shape)} {o_lat.dtype}, value matrix {tuple(uv.shape)}")
    _need(gate is None or (gate.is_cuda and gate.shape == (n, heads) and gate.dtype == out_dtype and (n == 0 or gate.stride(1) == 1)),
          f"{what}: the gate is {out_dtype} [{n}, {heads}] with contiguous rows")
    out = torch.empty((n, heads * vdim), dtype=out_dtype, device=o_lat.device)
    library.call(mixers(), "palm_latent_output", _stream(), _p(o_lat), _p(uv), _code(uv, what + " value matrix"), _p(gate),
                 gate.stride(0) if gate is not None else 0, _code(out, what), n, heads, kv_rank, vdim, _p(out))
    return out


# ---- routed experts ----------------------------------------------------------------------------------------------------

def moe_route(logits: torch.Tensor, top: int):
    """logits float32 [n, experts] -> (chosen int32 [n, top], weight float32 [n, top]): the ``top`` largest logits of each
    row, largest first (the lower index wins a tie), and the softmax over them alone."""
    _dev("moe_route", logits)
    _need(logits.dim() == 2 and logits.dtype == F32, f"moe_route: router logits are float32 [n, experts], not {logits.dtype} {tuple(logits.shape)}")
    n, experts = logits.shape
    chosen = torch.empty((n, top), dtype=torch.int32, device=logits.device)
    weight = torch.empty((n, top), dtype=F32, device=logits.device)
    library.call(feedforward(), "palm_moe_route", _stream(), _p(logits), n, experts, int(top), _p(chosen), _p(weight))
    return chosen, weight


EXPERT_FORMS = {"gated_silu": 0, "gelu": 1}


def _expert_shapes(what, h, up, down, ff, form):
    """-> (experts, rows of an expert's first matrix): gated experts keep their gate rows before their up rows."""
    _need(form in EXPERT_FORMS, f"{what}: an expert's form {form!r} is not one of {sorted(EXPERT_FORMS)}")
    per = (2 if form == "gated_silu" else 1) * ff
    width = h.shape[1]
    _need(up.dim() == 2 and up.shape[1] == width and up.shape[0] % per == 0 and down.shape == (up.shape[0] // per * width, ff)
          and up.dtype == down.dtype, f"{what}: first matrices {tuple(up.shape)}, down {tuple(down.shape)} for width {width}, inner size {ff}")
    return up.shape[0] // per


def moe_route_scored(logits: torch.Tensor, experts: int, top: int, correction: torch.Tensor | None, groups: int, keep: int, scale: float):
    """logits float32 [n, >= experts] (the experts' columns first) -> (chosen int32 [n, top], weight float32 [n, top]).  The
    scores are sigmoid(logit); the choice is made by score + ``correction``; the experts lie in ``groups`` equal groups of
    neighbours, a group ranks by the sum of its two largest corrected scores, and only experts of the best ``keep`` groups can
    be chosen (the lower index wins a tie); the weights are the chosen scores over their sum (+ 1e-20), times ``scale``."""
    _dev("moe_route_scored", logits, correction)
    _need(logits.dim() == 2 and logits.dtype == F32 and logits.shape[1] >= experts, f"moe_route_scored: router logits are float32 [n, >= {experts}], "
          f"not {logits.dtype} {tuple(logits.shape)}")
    _need(correction is None or (correction.shape == (experts,) and correction.dtype == F32), f"moe_route_scored: the correction is float32 [{experts}]")
    n = logits.shape[0]
    chosen = torch.empty((n, top), dtype=torch.int32, device=logits.device)
    weight = torch.empty((n, top), dtype=F32, device=logits.device)
    library.call(feedforward(), "palm_moe_route_scored", _stream(), _p(logits), logits.shape[1], n, int(experts), int(top), _p(correction),
                 int(groups), int(keep), float(scale), _p(chosen), _p(weight))
    return chosen, weight


def add_gated_rows(out: torch.Tensor, y: torch.Tensor, logits: torch.Tensor, column: int) -> torch.Tensor:
    """out[t] += sigmoid(logits[t, column]) * y[t]: out float32 [n, width] in place, logits float32 [n, *]."""
    _dev("add_gated_rows", out, y, logits)
    _need(out.dim() == 2 and out.dtype == F32 and y.shape == out.shape and logits.dim() == 2 and logits.dtype == F32
          and logits.shape[0] == out.shape[0] and 0 <= column < logits.shape[1],
          f"add_gated_rows: out {tuple(out.shape)} {out.dtype}, y {tuple(y.shape)}, gate column {column} of {tuple(logits.shape)} {logits.dtype}")
    library.call(feedforward(), "palm_add_gated_rows", _stream(), _p(out), _p(y), _code(y, "add_gated_rows"),
                 logits.data_ptr() + column * 4, logits.shape[1], out.shape[0], out.shape[1])
    return out


ACTIVATIONS = {"relu_squared": 0, "gelu_erf": 1, "gelu_tanh": 2}


def activation(z: torch.Tensor, kind: str) -> torch.Tensor:
    """max(z, 0)^2, or the gelu with erf, or the gelu with tanh, elementwise, 32-bit inside."""
    _dev("activation", z)
    _need(kind in ACTIVATIONS, f"activation: {kind!r} is not one of {sorted(ACTIVATIONS)}")
    out = torch.empty_like(z)
    library.call(feedforward(), "palm_activation", _stream(), _p(z), _p(out), _code(z, "activation"), ACTIVATIONS[kind], z.numel())
    return out


def moe_experts(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, chosen: torch.Tensor, weight: torch.Tensor, ff: int,
                form: str = "gated_silu") -> torch.Tensor:
    """Every row through its chosen experts, nothing planned on the host: h [n, width]; gate_up [experts * 2 ff, width] (an
    expert's gate rows, then its up rows; ``form`` "gelu": [experts * ff, width], up rows alone, through the exact gelu);
    down [experts * width, ff].  Returns float32 [n, width], the weighted sum."""
    what = "moe_experts"
    _dev(what, h, gate_up, down, chosen, weight)
    _i32(what, chosen)
    n, width = h.shape
    top = chosen.shape[1]
    _expert_shapes(what, h, gate_up, down, ff, form)
    _need(chosen.shape == (n, top) and weight.shape == (n, top) and weight.dtype == F32, f"{what}: choices {tuple(chosen.shape)}, weights {tuple(weight.shape)}")
    mid = torch.empty((n, top, ff), dtype=F32, device=h.device)
    out = torch.empty((n, width), dtype=F32, device=h.device)
    library.call(feedforward(), "palm_moe_experts", _stream(), _p(h), _code(h, what), _p(gate_up), _p(down), _code(gate_up, what + " weights"),
                 _p(chosen), _p(weight), n, top, width, ff, _p(mid), _p(out), EXPERT_FORMS[form])
    return out


def moe_grouped_serves(h: torch.Tensor, gate_up: torch.Tensor, ff: int) -> bool:
    """The grouped products on the matrix cores take bfloat16 rows and weights whose sizes are multiples of eight."""
    return h.dtype == BF16 and gate_up.dtype == BF16 and h.shape[1] % 8 == 0 and ff % 8 == 0


def moe_grouped(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, chosen: torch.Tensor, weight: torch.Tensor, ff: int,
                form: str = "gated_silu") -> torch.Tensor:
    """Every row through its chosen experts, for many rows, planned on the device: the (row, choice) pairs grouped by expert,
    two grouped products on the matrix cores, the weighted sum in the order of the choices.  Shapes as ``moe_experts``;
    returns float32 [n, width]."""
    what = "moe_grouped"
    _dev(what, h, gate_up, down, chosen, weight)
    _i32(what, chosen)
    n, width = h.shape
    top = chosen.shape[1]
    _need(moe_grouped_serves(h, gate_up, ff), f"{what}: bfloat16 rows and weights, sizes in multiples of eight")
    experts = _expert_shapes(what, h, gate_up, down, ff, form)
    _need(down.dtype == BF16, f"{what}: bfloat16 weights")
    _need(chosen.shape == (n, top) and weight.shape == (n, top) and weight.dtype == F32, f"{what}: choices {tuple(chosen.shape)}, weights {tuple(weight.shape)}")
    tile = feedforward().palm_moe_tile_tokens()
    max_tiles = (n * top + tile - 1) // tile + experts
    slots = max_tiles * tile
    plan = torch.empty((2 * experts + 1 + max_tiles + slots + n * top,), dtype=torch.int32, device=h.device)
    mid = torch.empty((slots, ff), dtype=BF16, device=h.device)
    y = torch.empty((slots, width), dtype=BF16, device=h.device)
    out = torch.empty((n, width), dtype=F32, device=h.device)
    library.call(feedforward(), "palm_moe_grouped", _stream(), _p(h), _p(gate_up), _p(down), _p(chosen), _p(weight), n, top, experts, width, ff,
                 _p(plan), _p(mid), _p(y), _p(out), EXPERT_FORMS[form])
    return out


def gather_rows(h: torch.Tensor, src: torch.Tensor) -> torch.Tensor:
    """xs[p] = h[src[p]] (src int32)."""
    _dev("gather_rows", h, src)
    _i32("gather_rows", src)
    _need(h.dim() == 2 and src.dim() == 1, f"gather_rows: rows {tuple(h.shape)}, indices {tuple(src.shape)}")
    xs = torch.empty((src.shape[0], h.shape[1]), dtype=h.dtype, device=h.device)
    library.call(feedforward(), "palm_gather_rows", _stream(), _p(h), _code(h, "gather_rows"), _p(src), src.shape[0], h.shape[1], _p(xs))
    return xs


def scatter_add(out: torch.Tensor, y: torch.Tensor, rows: torch.Tensor, weight: torch.Tensor) -> None:
    """out[rows[i]] += weight[i] * y[i]; out float32; the rows must be distinct."""
    _dev("scatter_add", out, y, rows, weight)
    _i32("scatter_add", rows)
    _need(out.dtype == F32 and out.dim() == 2 and y.dim() == 2 and y.shape[1] == out.shape[1] and rows.shape == (y.shape[0],)
          and weight.shape == (y.shape[0],) and weight.dtype == F32, f"scatter_add: out {tuple(out.shape)} {out.dtype}, y {tuple(y.shape)}, "
          f"rows {tuple(rows.shape)}, weights {tuple(weight.shape)} {weight.dtype}")
    library.call(feedforward(), "palm_scatter_add", _stream(), _p(y), _code(y, "scatter_add"), _p(rows), _p(weight), y.shape[0], out.shape[1], _p(out))


# ---- softmax attention with a sink, a window and a gate (library ``sink_attention``) -------------------------------

SINK_NORMS = {None: 0, "projection": 1, "head": 2}
SINK_BLOCKS_WANTED = 1024         # a decode step's key ranges are cut into slices until about this many blocks run


ROTARY_PAIRINGS = {"half_split": 0, "interleaved": 1}


def sink_qkv_store(rows: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, bias, norm: str | None, q_w, k_w, eps: float,
                   cos, sin, rot: int, k_cache, v_cache, block_table, ctx, write_cache: bool = True, col0: int = 0,
                   pairing: str = "half_split", conv=None, conv_state=None) -> torch.Tensor:
    """q, k and v of the step's tokens from ``rows`` [n, >= heads*dim + kv_heads*dim + kv_heads*vdim] (q | k | v | whatever
    follows): ``bias`` (float32 over q | k | v, or None) is added, q and k are normed (``norm``: "projection": one RMS norm
    over the whole q row and one over the whole k row, weights of those sizes; "head": per head, weights of the key size;
    None), their first ``rot`` dimensions are rotated by the tokens' cos and sin rows (``pairing``: dimension i with i + rot/2,
    or 2i with 2i + 1), k and v go to their pages, and q comes back as [n, heads, dim].  ``col0``: q begins at this column of
    the rows.

    ``write_cache`` false: the layer reads another layer's keys and values; the rows hold q alone (| whatever follows) and
    bias, convolution and state cover q's channels only.

    ``conv`` (float32 [channels, taps], q | k | v) with ``conv_state`` (float32 [slots, taps - 1, channels]): right after
    the bias every channel goes through a short causal convolution over time, y_t = sum_j conv[c, j] u_(t - taps + 1 + j);
    the state holds each sequence's last taps - 1 inputs (zero for a new sequence) and is left updated."""
    _dev("sink_qkv_store", rows, bias, q_w, k_w, cos, sin, block_table, ctx.tok_slot, ctx.positions, conv, conv_state)
    _i32("sink_qkv_store", block_table, ctx.tok_slot, ctx.positions)
    n = rows.shape[0]
    q_size = heads * dim
    k_size, v_size = (kv_heads * dim, kv_heads * vdim) if write_cache else (0, 0)
    channels = q_size + k_size + v_size
    _need(rows.dim() == 2 and col0 >= 0 and rows.shape[1] >= col0 + channels and n == ctx.n_tokens,
          f"sink_qkv_store: rows {tuple(rows.shape)} for {ctx.n_tokens} tokens of {q_size} + {k_size} + {v_size}")
    _need(norm in SINK_NORMS, f"sink_qkv_store: norm {norm!r} is not one of {sorted(map(str, SINK_NORMS))}")
    _need(pairing in ROTARY_PAIRINGS, f"sink_qkv_store: pairing {pairing!r} is not one of {sorted(ROTARY_PAIRINGS)}")
    if bias is not None:
        _need(bias.shape == (channels,) and bias.dtype == F32, f"sink_qkv_store: the bias is float32 [{channels}]")
    if norm is not None:
        want = (q_size, kv_heads * dim) if norm == "projection" else (dim, dim)
        _need(q_w is not None and k_w is not None and q_w.shape == (want[0],) and k_w.shape == (want[1],) and q_w.dtype == F32
              and k_w.dtype == F32, f"sink_qkv_store: the norm weights are float32 [{want[0]}] and [{want[1]}]")
    if rot:
        for tab in (cos, sin):
            _need(tab is not None and tab.dtype == F32 and tab.shape == (n, rot // 2), f"sink_qkv_store: rotation rows are float32 [{n}, {rot // 2}]")
    if write_cache:
        _dev("sink_qkv_store", k_cache, v_cache)
        _need(k_cache.dtype == rows.dtype and v_cache.dtype == rows.dtype and k_cache.shape[1:] == (kv_heads, PAGE_TOKENS, dim)
              and v_cache.shape[1:] == (kv_heads, vdim, PAGE_TOKENS) and block_table.dim() == 2,
              f"sink_qkv_store: cache {tuple(k_cache.shape)} / {tuple(v_cache.shape)} {k_cache.dtype} for rows of {rows.dtype}")
    taps = 0
    if conv is not None:
        taps = conv.shape[1] if conv.dim() == 2 else -1
        _need(conv.shape == (channels, taps) and conv.dtype == F32 and taps >= 1, f"sink_qkv_store: the convolution is float32 [{channels}, taps], not {tuple(conv.shape)}")
        if taps > 1:
            _need(conv_state is not None and conv_state.dim() == 3 and conv_state.shape[1:] == (taps - 1, channels) and conv_state.dtype == F32,
                  f"sink_qkv_store: the convolution's state is float32 [slots, {taps - 1}, {channels}]")
            _dev("sink_qkv_store", ctx.seq_slot, ctx.seq_new, ctx.cu_new)
            _i32("sink_qkv_store", ctx.seq_slot, ctx.seq_new, ctx.cu_new)
    q = torch.empty((n, heads, dim), dtype=rows.dtype, device=rows.device)
    library.call(sink_attention_lib(), "palm_sink_qkv_store", _stream(), _p(rows), _code(rows, "sink_qkv_store"), rows.shape[1], col0, col0 + q_size,
                 col0 + q_size + k_size, _p(bias), _p(q), _p(k_cache) if write_cache else None, _p(v_cache) if write_cache else None,
                 _p(block_table), block_table.shape[1], _p(ctx.tok_slot),
                 _p(ctx.positions), SINK_NORMS[norm], _p(q_w), _p(k_w), float(eps), _p(cos), _p(sin), int(rot), n, heads, kv_heads, dim,
                 vdim, int(write_cache), ROTARY_PAIRINGS[pairing], _p(conv), int(taps), _p(conv_state) if taps > 1 else None,
                 _p(ctx.seq_slot), _p(ctx.seq_new), _p(ctx.cu_new), ctx.n_seqs)
    return q


def sink_slices(ctx, heads: int, kv_heads: int, window: int | None) -> int:
    """Into how many slices the exact kernel cuts a query's key range: one for prompts; for single tokens as many as
    fill the chip, each of at least two pages (measured with 8 sequences, 4 key/value heads and 17 pages: 1, 2, 4, 8 and 16
    slices took 35.8, 27.6, 23.1, 21.2 and 27.3 us)."""
    if not ctx.is_decode:
        return 1
    keys = min(ctx.max_total, window) if window else ctx.max_total
    pages = -(-keys // PAGE_TOKENS) + 1
    blocks = ctx.n_seqs * kv_heads * -(-(heads // kv_heads) // 8)
    return max(1, min(pages // 2, SINK_BLOCKS_WANTED // max(1, blocks)))


def sink_attention_exact(q: torch.Tensor, k_cache, v_cache, block_table, ctx, heads: int, kv_heads: int, dim: int, vdim: int,
                         scale: float, window: int | None, sink, gate: torch.Tensor | None, gate_off: int = 0,
                         slices: int | None = None, gate_per_head: bool = False) -> torch.Tensor:
    """Attention of the step's queries q [n, heads, dim] over the cached keys of their sequences up to their own positions
    (the last ``window`` if given), with a sink in the denominator: ``sink`` is its score for all heads, or a float32 tensor
    [heads] of learned scores, or None.  ``gate``: a tensor [n, >= gate_off + heads*vdim] whose columns from ``gate_off`` on
    gate the output through a sigmoid (None: no gate); with ``gate_per_head`` one column for each head.  Returns
    [n, heads * vdim].  32-bit arithmetic whatever the elements' type."""
    _dev("sink_attention", q, k_cache, v_cache, block_table, gate, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new)
    _i32("sink_attention", block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new)
    n = q.shape[0]
    _need(q.shape == (ctx.n_tokens, heads, dim), f"sink_attention: q {tuple(q.shape)} is not [{ctx.n_tokens}, {heads}, {dim}]")
    _need(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype and k_cache.shape[1:] == (kv_heads, PAGE_TOKENS, dim)
          and v_cache.shape[1:] == (kv_heads, vdim, PAGE_TOKENS), f"sink_attention: cache {tuple(k_cache.shape)} / {tuple(v_cache.shape)}")
    gate_ptr, gate_stride = _sink_gate("sink_attention", gate, gate_off, n, heads, vdim, q.dtype, gate_per_head)
    sink_score, sink_scores = _sink_scores("sink_attention", sink, heads, q.device)
    slices = sink_slices(ctx, heads, kv_heads, window) if slices is None else int(slices)
    work = torch.empty((n * heads * slices * (vdim + 2),), dtype=F32, device=q.device) if slices > 1 else None
    out = torch.empty((n, heads * vdim), dtype=q.dtype, device=q.device)
    library.call(sink_attention_lib(), "palm_sink_attention", _stream(), _p(q), _code(q, "sink_attention"), _p(k_cache), _p(v_cache),
                 _p(block_table), block_table.shape[1], _p(ctx.seq_slot), _p(ctx.seq_start), _p(ctx.seq_new), _p(ctx.cu_new), ctx.n_seqs,
                 int(ctx.max_new), n, heads, kv_heads, dim, vdim, float(scale), int(window or 0), int(sink is not None),
                 sink_score, _p(sink_scores), gate_ptr, gate_stride, int(gate_per_head), slices, _p(work), _p(out))
    return out


def _sink_gate(what: str, gate, gate_off: int, n: int, heads: int, vdim: int, dtype, per_head: bool):
    """(address of token 0's first gate value, elements between rows), or (None, 0)."""
    if gate is None:
        return None, 0
    cols = heads if per_head else heads * vdim
    _need(gate.dim() == 2 and gate.shape[0] == n and gate.shape[1] >= gate_off + cols and gate.dtype == dtype,
          f"{what}: gate rows {tuple(gate.shape)} {gate.dtype} with {cols} columns from column {gate_off}")
    return gate.data_ptr() + gate_off * gate.element_size(), gate.shape[1]


def _sink_scores(what: str, sink, heads: int, device):
    """(one score for all heads, a tensor of one for each or None)."""
    if isinstance(sink, torch.Tensor):
        _dev(what, sink)
        _need(sink.shape == (heads,) and sink.dtype == F32, f"{what}: learned sink scores are float32 [{heads}], not {sink.dtype} {tuple(sink.shape)}")
        return 0.0, sink
    return float(sink or 0.0), None


_SINK_MFMA_SIGNATURE = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                        c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_float, c_void_p, c_void_p, c_int, c_int, c_void_p]
_sink_mfma_libs: dict = {}


def sink_mfma_serves(q: torch.Tensor, dim: int, vdim: int) -> bool:
    """Whether the matrix-core kernel takes these queries: bfloat16, a key size in steps of 8 and a value size in steps of 4."""
    return q.dtype == BF16 and dim % 8 == 0 and vdim % 4 == 0 and dim <= 256 and vdim <= 256


def sink_attention_mfma_lib(dim: int, vdim: int):
    """The library compiled for this key and value size (built when a model of these sizes first runs a prompt)."""
    key = (-(-dim // 32), -(-vdim // 16))
    lib = _sink_mfma_libs.get(key)
    if lib is None:
        lib = library.load(f"sink_attention_k{key[0]}_v{key[1]}")
        lib.palm_sink_attention_mfma.argtypes, lib.palm_sink_attention_mfma.restype = _SINK_MFMA_SIGNATURE, c_int
        _sink_mfma_libs[key] = lib
    return lib


def sink_attention_mfma(q: torch.Tensor, k_cache, v_cache, block_table, ctx, heads: int, kv_heads: int, dim: int, vdim: int,
                        scale: float, window: int | None, sink, gate: torch.Tensor | None, gate_off: int = 0,
                        gate_per_head: bool = False) -> torch.Tensor:
    """``sink_attention_exact`` for prompts in bfloat16 on the matrix cores (scores, weights and sums 32-bit)."""
    _dev("sink_attention_mfma", q, k_cache, v_cache, block_table, gate, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new)
    _i32("sink_attention_mfma", block_table, ctx.seq_slot, ctx.seq_start, ctx.seq_new, ctx.cu_new)
    n = q.shape[0]
    _need(sink_mfma_serves(q, dim, vdim), f"sink_attention_mfma: {q.dtype} queries of key size {dim} and value size {vdim} are not served")
    _need(q.shape == (ctx.n_tokens, heads, dim), f"sink_attention_mfma: q {tuple(q.shape)} is not [{ctx.n_tokens}, {heads}, {dim}]")
    _need(k_cache.dtype == BF16 and v_cache.dtype == BF16 and k_cache.shape[1:] == (kv_heads, PAGE_TOKENS, dim)
          and v_cache.shape[1:] == (kv_heads, vdim, PAGE_TOKENS), f"sink_attention_mfma: cache {tuple(k_cache.shape)} / {tuple(v_cache.shape)}")
    gate_ptr, gate_stride = _sink_gate("sink_attention_mfma", gate, gate_off, n, heads, vdim, BF16, gate_per_head)
    sink_score, sink_scores = _sink_scores("sink_attention_mfma", sink, heads, q.device)
    out = torch.empty((n, heads * vdim), dtype=BF16, device=q.device)
    library.call(sink_attention_mfma_lib(dim, vdim), "palm_sink_attention_mfma", _stream(), _p(q), _p(k_cache), _p(v_cache), _p(block_table),
                 block_table.shape[1], _p(ctx.seq_slot), _p(ctx.seq_start), _p(ctx.seq_new), _p(ctx.cu_new), ctx.n_seqs, int(ctx.max_new),
                 heads, kv_heads, dim, vdim, float(scale), int(window or 0), int(sink is not None), sink_score, _p(sink_scores), gate_ptr,
                 gate_stride, int(gate_per_head), _p(out))
    return out


def sink_attention(q, k_cache, v_cache, block_table, ctx, heads, kv_heads, dim, vdim, scale, window, sink, gate, gate_off=0,
                   gate_per_head=False):
    """The kernel that serves: the matrix cores for prompts in bfloat16, the exact one for the float32 mode, for single
    tokens, and for sizes that the matrix-core kernel does not take."""
    if not ctx.is_decode and sink_mfma_serves(q, dim, vdim):
        return sink_attention_mfma(q, k_cache, v_cache, block_table, ctx, heads, kv_heads, dim, vdim, scale, window, sink, gate, gate_off,
                                   gate_per_head=gate_per_head)
    return sink_attention_exact(q, k_cache, v_cache, block_table, ctx, heads, kv_heads, dim, vdim, scale, window, sink, gate, gate_off,
                                gate_per_head=gate_per_head)


# ---- branches scaled by a learned vector; the capped feed-forward gate (library ``branches``) ---------------------

def add_scaled_normed(x: torch.Tensor, terms, weights, scale: torch.Tensor | None, norm_w: torch.Tensor | None, eps: float,
                      out_dtype: torch.dtype | None = None, rows: torch.Tensor | None = None):
    """x += scale * sum_i weights[i] * terms[i] (one or two terms [n, width] of one element type; scale float32 [width] or
    None; the sum in 32-bit, x float32 in place), and what the norm with weight ``norm_w`` makes of the sum, in
    ``out_dtype``.  With ``rows`` only those rows are summed and normed and x stays as it is.  ``norm_w`` None: the sum
    alone is made, and nothing is returned."""
    _need(1 <= len(terms) <= 2 and len(weights) == len(terms), f"add_scaled_normed: {len(terms)} terms with {len(weights)} weights (one or two)")
    _dev("add_scaled_normed", x, *terms, scale, norm_w, rows)
    _i32("add_scaled_normed", rows)
    n, width = x.shape
    _need(x.dtype == F32 and all(t.shape == x.shape and t.dtype == terms[0].dtype for t in terms),
          f"add_scaled_normed: x {tuple(x.shape)} {x.dtype}, terms {[tuple(t.shape) for t in terms]}")
    for v in (scale, norm_w):
        _need(v is None or (v.shape == (width,) and v.dtype == F32), f"add_scaled_normed: vectors are float32 [{width}]")
    _need(norm_w is not None or rows is None, "add_scaled_normed: a selection of rows is for the norm that reads them")
    n_out = n if rows is None else rows.shape[0]
    out = torch.empty((n_out, width), dtype=out_dtype or F32, device=x.device) if norm_w is not None else None
    library.call(branches(), "palm_add_scaled_normed", _stream(), _p(x), _p(terms[0]), float(weights[0]),
                 _p(terms[1]) if len(terms) > 1 else None, float(weights[1]) if len(terms) > 1 else 0.0, _code(terms[0], "add_scaled_normed"),
                 _p(scale), _p(norm_w), float(eps), _p(rows), n_out, width, int(rows is None), _p(out),
                 _code(out, "add_scaled_normed out") if out is not None else 0)
    return out


def capped_gate(gate_up: torch.Tensor, limit: float, slope: float, shift: float) -> torch.Tensor:
    """[n, 2 ff] (gate | up) -> [n, ff]: g * sigmoid(slope * g) * (u + shift), g = min(gate, limit), u = clamp(up, -limit, limit)."""
    _dev("capped_gate", gate_up)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, f"capped_gate: rows {tuple(gate_up.shape)} are not [n, 2 ff]")
    n, ff = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((n, ff), dtype=gate_up.dtype, device=gate_up.device)
    library.call(branches(), "palm_capped_gate", _stream(), _p(gate_up), _p(out), _code(gate_up, "capped_gate"), n, ff, float(limit),
                 float(slope), float(shift))
    return out


# ---- a residual stream in several copies, and its norms (library ``streams``) ------------------------------------

STREAM_NORMS = {None: 0, "dyt": 1, "rms": 2}


def streams_spread(x: torch.Tensor, streams: int) -> torch.Tensor:
    """x float32 [n, width] -> [n, streams, width]: every stream starts as a copy of x."""
    _dev("streams_spread", x)
    _need(x.dim() == 2 and x.dtype == F32 and streams >= 1, f"streams_spread: x {tuple(x.shape)} {x.dtype}, {streams} streams")
    xs = torch.empty((x.shape[0], streams, x.shape[1]), dtype=F32, device=x.device)
    library.call(streams_lib(), "palm_streams_spread", _stream(), _p(x), x.shape[0], int(streams), x.shape[1], _p(xs))
    return xs


def streams_mix_norm(xs: torch.Tensor, y: torch.Tensor | None, mix: torch.Tensor | None, out_w: torch.Tensor | None,
                     in_w: torch.Tensor | None, norm: str | None, norm_w=None, norm_b=None, alpha: float = 1.0, eps: float = 0.0,
                     rows: torch.Tensor | None = None, out_dtype: torch.dtype | None = None, read: bool = True):
    """One sublayer's write into the streams and the next reader's read, in one pass.  xs float32 [n, S, width].

    Write (``y`` [n, width] given): xs'[t] = sum_s mix[s, t] xs[s] + out_w[t] y, all streams at once, in place; with
    ``rows`` the stream stays as it is and only those rows are computed, for the reader.
    Read (``read``): u = sum_s in_w[s] xs'[s] (``in_w`` None: the plain sum), through ``norm``: "dyt" tanh(alpha u) w + b,
    "rms" u / sqrt(mean(u^2) + eps) w, None u itself; returned in ``out_dtype`` as [rows or n, width]."""
    what = "streams_mix_norm"
    _dev(what, xs, y, mix, out_w, in_w, norm_w, norm_b, rows)
    _i32(what, rows)
    _need(xs.dim() == 3 and xs.dtype == F32, f"{what}: the streams are float32 [n, S, width], not {xs.dtype} {tuple(xs.shape)}")
    n, S, width = xs.shape
    _need(norm in STREAM_NORMS, f"{what}: norm {norm!r} is not one of {sorted(map(str, STREAM_NORMS))}")
    if y is not None:
        _need(y.shape == (n, width) and mix is not None and mix.shape == (S, S) and mix.dtype == F32 and out_w is not None
              and out_w.shape == (S,) and out_w.dtype == F32, f"{what}: output {tuple(y.shape)} with weights {None if mix is None else tuple(mix.shape)}, "
              f"{None if out_w is None else tuple(out_w.shape)} for {S} streams of width {width}")
    _need(in_w is None or (in_w.shape == (S,) and in_w.dtype == F32), f"{what}: the reader's weights are float32 [{S}]")
    _need(y is not None or read, f"{what}: neither a write nor a read")
    out = None
    n_rows = n if rows is None else rows.shape[0]
    if read:
        if norm is not None:
            _need(norm_w is not None and norm_w.shape == (width,) and norm_w.dtype == F32 and (norm_b is None or (norm_b.shape == (width,) and norm_b.dtype == F32)),
                  f"{what}: the norm's vectors are float32 [{width}]")
        out = torch.empty((n_rows, width), dtype=out_dtype or F32, device=xs.device)
    if rows is not None and n_rows == 0:
        return out                                  # nothing is read, and a selection leaves the streams as they are
    library.call(streams_lib(), "palm_streams_mix_norm", _stream(), _p(xs), n, S, width, _p(y), _code(y, what) if y is not None else 0, _p(mix),
                 _p(out_w), _p(in_w), STREAM_NORMS[norm], _p(norm_w), _p(norm_b), float(alpha), float(eps), _p(rows), n_rows,
                 int(rows is None and y is not None), _p(out), _code(out, what + " out") if out is not None else 0)
    return out


# ---- a matrix memory with gates per head and token (library ``mlstm``) ----------------------------------------------

MLSTM_BLOCKS_WANTED = 512          # a long run of new tokens is cut into chunks until about this many blocks run
MLSTM_MIN_CHUNK = 32


def mlstm_chunk(n_seqs: int, heads: int, max_new: int) -> int:
    """Into chunks of how many tokens the kernel cuts the step's runs of new tokens (0: not at all): where one block per
    (head, sequence) leaves most of the chip idle and the runs are long, chunks run side by side at the price of walking
    over every token twice."""
    per_seq = MLSTM_BLOCKS_WANTED // max(1, heads * n_seqs)
    if max_new <= 2 * MLSTM_MIN_CHUNK or per_seq <= 1:
        return 0
    chunk = max(MLSTM_MIN_CHUNK, -(-max_new // per_seq))
    chunk = (chunk + 7) // 8 * 8
    return chunk if chunk < max_new else 0


def mlstm(rows: torch.Tensor, gates: torch.Tensor, gate_bias: torch.Tensor | None, heads: int, dim: int, vdim: int, cap: float,
          q_scale: float, norm_w: torch.Tensor, eps: float, state: torch.Tensor, m_state: torch.Tensor, ctx, col0: int = 0,
          chunk: int | None = None) -> torch.Tensor:
    """The step's tokens through a matrix memory.  rows [n, >= col0 + heads * (2 dim + 2 vdim)] hold q | k | v | gate; gates
    float32 [n, 2 heads] the input gates' rows and then the forget gates' (``gate_bias`` float32 [2 heads] is added); state
    float32 [slots, heads, dim, vdim + 1] (the memory and, as its last column, the normalizer) and m_state float32 [slots,
    heads] (the running maximum) are read and left updated.  Returns [n, heads * vdim]: every head's output over its
    denominator, unit-normed per head, times ``norm_w`` and the sigmoid of the gate.  ``chunk``: see ``mlstm_chunk``."""
    what = "mlstm"
    _dev(what, rows, gates, gate_bias, norm_w, state, m_state, ctx.seq_slot, ctx.seq_new, ctx.cu_new)
    _i32(what, ctx.seq_slot, ctx.seq_new, ctx.cu_new)
    n = rows.shape[0]
    in_rows = heads * (2 * dim + 2 * vdim)
    _need(rows.dim() == 2 and col0 >= 0 and rows.shape[1] >= col0 + in_rows and n == ctx.n_tokens, f"{what}: rows {tuple(rows.shape)} from column {col0} "
          f"are not [{ctx.n_tokens}, {heads} * (2*{dim} + 2*{vdim})]")
    _need(gates.shape == (n, 2 * heads) and gates.dtype == F32, f"{what}: the gates' rows are float32 [{n}, {2 * heads}], not {gates.dtype} {tuple(gates.shape)}")
    _need(gate_bias is None or (gate_bias.shape == (2 * heads,) and gate_bias.dtype == F32), f"{what}: the gates' bias is float32 [{2 * heads}]")
    _need(norm_w.shape == (heads * vdim,) and norm_w.dtype == F32, f"{what}: the norm's weight is float32 [{heads * vdim}]")
    _need(state.dim() == 4 and state.shape[1:] == (heads, dim, vdim + 1) and state.dtype == F32 and m_state.dim() == 2
          and m_state.shape == (state.shape[0], heads) and m_state.dtype == F32,
          f"{what}: state {tuple(state.shape)} {state.dtype} / {tuple(m_state.shape)} is not float32 [slots, {heads}, {dim}, {vdim + 1}] / [slots, {heads}]")
    lib = mlstm_lib()
    out = torch.empty((n, heads * vdim), dtype=rows.dtype, device=rows.device)
    chunk = mlstm_chunk(ctx.n_seqs, heads, ctx.max_new) if chunk is None else int(chunk)
    qk = torch.empty((n, heads, 2, lib.palm_mlstm_pad(dim)), dtype=F32, device=rows.device)
    coef = torch.empty((n, heads, 4), dtype=F32, device=rows.device)
    starts = keeps = None
    if chunk:
        max_chunks = -(-ctx.max_new // chunk)
        starts = torch.empty((ctx.n_seqs * max_chunks, heads, dim, vdim + 1), dtype=F32, device=rows.device)
        keeps = torch.empty((ctx.n_seqs * max_chunks, heads), dtype=F32, device=rows.device)
    library.call(lib, "palm_mlstm", _stream(), _p(rows), _code(rows, what), rows.shape[1], col0, col0 + heads * dim, col0 + 2 * heads * dim,
                 col0 + 2 * heads * dim + heads * vdim, _p(gates), _p(gate_bias), float(cap), float(q_scale), _p(norm_w), float(eps), _p(state),
                 _p(m_state), _p(ctx.seq_slot), _p(ctx.seq_new), _p(ctx.cu_new), ctx.n_seqs, heads, dim, vdim, _p(out), int(ctx.max_new),
                 chunk, _p(starts), _p(keeps), n, _p(qk), _p(coef))
    return out

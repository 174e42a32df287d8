"""ctypes bindings of the HIP library, with the host-side checks every launch needs.

Each wrapper checks, before anything reaches the GPU, that its tensors live on the
device, are contiguous where the kernel assumes it, have the dtypes and shapes the
kernel's indexing assumes, and that index tensors are int32. There is no CPU
fallback: without a GPU, or without the library, the call raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_uint32, c_void_p

import torch

from . import build as _build

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}
EPI_STORE, EPI_ADD, EPI_GATED = 0, 1, 2
ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}     # the gated epilogue's activation

_lib = None


class KernelError(RuntimeError):
    pass


def library():
    """The loaded library; built first if no build matches the sources."""
    global _lib
    if _lib is None:
        path = _build.library_path() or _build.build()
        lib = ctypes.CDLL(path)
        lib.gl3_last_error.restype = ctypes.c_char_p
        _declare(lib)
        _lib = lib
    return _lib


def library_file():
    library()
    return _build.library_path()


def _declare(lib):
    P, I, L, F = c_void_p, c_int, c_long, c_float
    sigs = {
        "gl3_abi_version": [],
        "gl3_fill_u32": [P, c_uint32, L, P],
        "gl3_embed": [P, I, P, P, I, I, P, P, P, F, P, P, I, P],
        "gl3_scale_f32": [P, F, L, P],
        "gl3_softcap_f32": [P, F, L, P],
        "gl3_rmsnorm": [P, P, P, I, P, I, I, I, F, P],
        "gl3_gather_rows": [P, P, P, I, I, I, P],
        "gl3_add_slices_rmsnorm": [P, P, P, I, L, L, P, I, P, I, I, I, F, P],
        "gl3_rope_cache_write": [P, I, P, P, P, I, P, P, P, P, I, I, I, I, I, I, I, I, P],
        "gl3_gemm_generic": [P, I, P, I, P, I, I, I, I, L, L, L, I, P, I, I, P, P],
        "gl3_attention_generic": [P, L, P, P, I, P, P, P, I, P, L, I, I, I, I, I, I, F, P],
        "gl3_sample": [P, L, P, P, P, P, P, I, I, P, I, P],
        "gl3_sample_work_floats": [I, I],
        "gl3_argmax": [P, L, P, P, I, I, P],
        "gl3_argmax_advance": [P, L, P, P, I, I, P, P, P, P, I, P, P],
        "gl3_argmax_static": [P, L, P, I, I, P],
        "gl3_decode_advance": [P, P, P, P, P, I, P, I, P],
        "gl3_gemm_skinny": [P, P, P, I, I, I, I, L, L, L, I, I, P, I, P, P, L, P, I, P, P, I, P],
        "gl3_gemm_skinny_wide": [P, P, P, I, I, I, I, L, L, L, I, I, L, I, P, I, P, I, F, I, I, P],
        "gl3_gemm_skinny_norm": [P, P, P, I, F, P, P, I, I, I, I, L, L, L, I, I, P, I, P, I, P],
        "gl3_qkv_rope_cache": [P, P, I, F, P, P, L, I, I, L, L, P, P, P, I, P, P, P, P, I, I, I, I, I, I, P, P, P, I, P],
        "gl3_token_facts": [P, P, P, I, I, P, P, I, P, P, P, I, P],
        "gl3_gemm_mfma": [P, P, P, I, I, I, I, L, L, L, I, I, P, L, L, P, I, I, I, P, P],
        "gl3_attention_decode_supports": [I, I],
        "gl3_attention_prefill_supports": [I, I],
        "gl3_attention_prefill": [P, L, P, P, P, P, P, P, I, P, L, I, I, I, I, I, I, I, F, I, P],
        "gl3_scatter_i32": [P, L, P, P, I, P],
        "gl3_upload": [P, P, L, P],
        "gl3_stage_decode": [P, I, I, P, P, P, I, P, P],
        "gl3_stage_step": [P, P, P, I, P, P, P, I, P, I, I, P],
        "gl3_graph_launch": [P, P],
        "gl3_attention_decode": [P, L, P, P, P, P, P, I, P, P, L, P, L, I, I, I, I, I, I, F, I, P],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name, None)
        if fn is None:
            continue
        fn.argtypes = args
        fn.restype = c_int
    lib.gl3_sample_work_floats.restype = ctypes.c_long
    lib._optional = set()


def has(name):
    return hasattr(library(), name)


def _check(rc, name):
    if rc != 0:
        raise KernelError(f"{name}: {library().gl3_last_error().decode()}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current stream of the current device (asked for at every launch: a graph capture changes it).
    The raw handle where this torch offers it: building a stream object costs as much as a launch."""
    if _raw_stream is not None and _raw_device is not None:
        return c_void_p(_raw_stream(_raw_device()))
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t, name, dtype=None, contiguous=True):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name} must be a tensor on the GPU (the kernels have no CPU path)")
    if dtype is not None and t.dtype not in (dtype if isinstance(dtype, tuple) else (dtype,)):
        raise KernelError(f"{name} has dtype {t.dtype}, expected {dtype}")
    if contiguous and not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    return t


def held_once(w):
    """Whether the matrix is kept in the matrix cores' order ALONE (``hold_once``): its memory is one of its
    copies (``w.tiled``, ``w.tiled8``), and only what reads such an order may touch it."""
    return getattr(w, "operand_order_only", False)


def _w_order(w):
    """How a weight lies, for the kernels that read any order: (0, the stored rows, no table), (1, the copy in
    the operands' order, each row's place in it or nothing), (2, the copy in packed strips of 8 rows, nothing)."""
    if not held_once(w):
        return 0, _ptr(w), c_void_p(0)
    t = getattr(w, "tiled", None)
    if t is not None:
        return 1, _ptr(t), _ptr(getattr(t, "row_pos", None))
    return 2, _ptr(w.tiled8), c_void_p(0)


def _code(t, name):
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"{name} has dtype {t.dtype}; the kernels take float32 and bfloat16") from None


def _ptr(t):
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(0)


def _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, who):
    """Keys [pages, kv heads, page, head_dim]; values transposed [pages, kv heads, head_dim, page]; inside a
    page both lie in the kernels' tiles (``cache/layout.py``), which needs pages of a multiple of 32 positions
    and heads of a multiple of 16 elements."""
    if (k_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (n_kv, page_size, head_dim)
            or tuple(v_cache.shape) != (k_cache.shape[0], n_kv, head_dim, page_size)):
        raise KernelError(f"{who}: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} for kv {n_kv} "
                          f"page {page_size} hs {head_dim}")
    if page_size % 32 or head_dim % 16:
        raise KernelError(f"{who}: the cache lies in tiles: pages of {page_size} positions must be a multiple of 32, "
                          f"heads of {head_dim} elements a multiple of 16")


# ------------------------------------------------------------------ ops
def fill_u32(t, value):
    _dev(t, "tensor")
    if t.element_size() * t.numel() % 4:
        raise KernelError("fill_u32 needs a multiple of 4 bytes")
    _check(library().gl3_fill_u32(_ptr(t), value, t.element_size() * t.numel() // 4, _stream()), "fill_u32")


def _check_next(next_weight, xg, rows, d, who):
    """The next norm's float weight [d] and the bfloat16 rows [rows, d] that receive weight * x."""
    if (next_weight is None) != (xg is None):
        raise KernelError(f"{who}: the next norm's weight and its rows come together")
    if xg is not None:
        _dev(next_weight, "next_weight", torch.float32); _dev(xg, "xg", torch.bfloat16, contiguous=False)
        if next_weight.shape != (d,) or xg.dim() != 2 or xg.shape != (rows, d) or xg.stride(1) != 1:
            raise KernelError(f"{who}: next weight {tuple(next_weight.shape)}, rows {tuple(xg.shape)} for [{rows}, {d}]")


def _bias(bias, n, who):
    """A bias per output column: float32 [n] on the device, or None."""
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.shape != (n,):
            raise KernelError(f"{who}: bias {tuple(bias.shape)} for {n} columns")
    return _ptr(bias)


def _act(act, who):
    try:
        return ACTIVATIONS[act]
    except KeyError:
        raise KernelError(f"{who}: activation {act!r} is not built ({sorted(ACTIVATIONS)})") from None


def scale_(t, factor):
    """t *= factor (float32, contiguous)."""
    _dev(t, "tensor", torch.float32)
    _check(library().gl3_scale_f32(_ptr(t), float(factor), t.numel(), _stream()), "scale_f32")


def softcap_(t, cap):
    """t = cap * tanh(t / cap) (float32, contiguous)."""
    _dev(t, "tensor", torch.float32)
    _check(library().gl3_softcap_f32(_ptr(t), float(cap), t.numel(), _stream()), "softcap_f32")


def _table_steps(table):
    """0, or the k-steps of 32 a strip of a table that is held once (in the operands' order, rows in order)."""
    if not held_once(table):
        return 0
    t = getattr(table, "tiled", None)
    if t is None or getattr(t, "row_pos", None) is not None or t.data_ptr() != table.data_ptr():
        raise KernelError("embed: a table that is held once must be its copy in the operands' order, rows in order")
    return -(-table.shape[1] // 32)


def embed(table, ids, out, ssq=None, next_weight=None, xg=None, scale=1.0, pos_table=None, positions=None):
    """out[t] = scale * table[ids[t]] (+ pos_table[positions[t]]) as float32. The caller has checked
    ids < rows and positions < rows of ``pos_table``. ``ssq`` (at least 64 floats, at most 64 tokens)
    receives each row's sum of squares; with it ``xg`` [T, d] bfloat16 may receive ``next_weight *
    out``, the rows as the product after the next norm reads them."""
    _dev(table, "table"); _dev(ids, "ids", torch.int32); _dev(out, "out", torch.float32)
    T, d = out.shape
    if table.dim() != 2 or table.shape[1] != d or ids.numel() != T:
        raise KernelError(f"embed: table {tuple(table.shape)}, ids {tuple(ids.shape)}, out {tuple(out.shape)}")
    if ssq is not None:
        _dev(ssq, "ssq", torch.float32)
        if ssq.numel() < 64 or T > 64:
            raise KernelError("embed: sums of squares need 64 floats and at most 64 tokens")
    _check_next(next_weight, xg, T, d, "embed")
    if xg is not None and (ssq is None or not xg.is_contiguous()):
        raise KernelError("embed: the next norm's rows come with the sums of squares, contiguous")
    if pos_table is not None:
        _dev(pos_table, "pos_table", table.dtype); _dev(positions, "positions", torch.int32)
        if pos_table.dim() != 2 or pos_table.shape[1] != d or positions.numel() != T:
            raise KernelError(f"embed: table of positions {tuple(pos_table.shape)} for rows of {d}")
    _check(library().gl3_embed(_ptr(table), _code(table, "table"), _ptr(ids), _ptr(out), T, d, _ptr(ssq),
                               _ptr(next_weight), _ptr(xg), float(scale), _ptr(pos_table),
                               _ptr(positions) if pos_table is not None else c_void_p(0), _table_steps(table),
                               _stream()), "embed")


def rmsnorm(x, weight, out, eps, rows=None):
    """out[r] = weight * x[rows[r]] / rms (rows None: every row in order)."""
    _dev(x, "x", torch.float32); _dev(weight, "weight"); _dev(out, "out")
    d = x.shape[-1]
    n = out.shape[0]
    if x.dim() != 2 or out.dim() != 2 or out.shape[1] != d or weight.shape != (d,):
        raise KernelError(f"rmsnorm: x {tuple(x.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    if rows is not None:
        _dev(rows, "rows", torch.int32)
        if rows.numel() != n:
            raise KernelError(f"rmsnorm: {rows.numel()} rows for {n} outputs")
    elif x.shape[0] != n:
        raise KernelError(f"rmsnorm: {x.shape[0]} inputs for {n} outputs")
    _check(library().gl3_rmsnorm(_ptr(x), _ptr(rows), _ptr(weight), _code(weight, "weight"), _ptr(out),
                                 _code(out, "out"), n, d, float(eps), _stream()), "rmsnorm")


def gather_rows(x, rows, out):
    """out[r] = x[rows[r]] in ``out``'s dtype (x float32; the caller has checked rows < rows of x)."""
    _dev(x, "x", torch.float32); _dev(rows, "rows", torch.int32); _dev(out, "out")
    if x.dim() != 2 or out.dim() != 2 or out.shape != (rows.numel(), x.shape[1]):
        raise KernelError(f"gather_rows: x {tuple(x.shape)}, {rows.numel()} rows, out {tuple(out.shape)}")
    _check(library().gl3_gather_rows(_ptr(x), _ptr(rows), _ptr(out), _code(out, "out"), out.shape[0], x.shape[1],
                                     _stream()), "gather_rows")


def add_slices_rmsnorm(x, slices, weight=None, out=None, eps=0.0, rows=None):
    """x += slices[0] + slices[1] + ... (in that order; ``slices`` [S, rows of x, d] float32), and
    out[r] = weight * x[r] / rms when ``out`` is given. With ``rows`` the listed rows are normalised
    and x keeps its values."""
    _dev(x, "x", torch.float32); _dev(slices, "slices", torch.float32, contiguous=False)
    d = x.shape[-1]
    if (x.dim() != 2 or slices.dim() != 3 or slices.shape[1:] != x.shape or slices.stride(2) != 1
            or (weight is None) != (out is None)):
        raise KernelError(f"add_slices_rmsnorm: x {tuple(x.shape)}, slices {tuple(slices.shape)}")
    n = x.shape[0]
    if out is not None:
        _dev(weight, "weight"); _dev(out, "out")
        n = out.shape[0]
        if out.dim() != 2 or out.shape[1] != d or weight.shape != (d,):
            raise KernelError(f"add_slices_rmsnorm: weight {tuple(weight.shape)}, out {tuple(out.shape)} for d={d}")
    if rows is not None:
        _dev(rows, "rows", torch.int32)
        if out is None or rows.numel() != n:
            raise KernelError("add_slices_rmsnorm: rows select the rows that are normalised, one per output row")
    elif x.shape[0] != n:
        raise KernelError(f"add_slices_rmsnorm: {x.shape[0]} inputs for {n} outputs")
    _check(library().gl3_add_slices_rmsnorm(
        _ptr(x), _ptr(rows), _ptr(slices), slices.shape[0], slices.stride(0), slices.stride(1), _ptr(weight),
        _code(weight, "weight") if weight is not None else 0, _ptr(out), _code(out, "out") if out is not None else 0,
        n, d, float(eps), _stream()), "add_slices_rmsnorm")


def rope_cache_write(qkv, positions, seq_of_token, block_table, cos, sin, k_cache, v_cache, n_heads, n_kv,
                     head_dim, rot_dim, adjacent, page_size, write_kv=True):
    """Rotate q (in place) and k, and write k and v into one layer's paged cache.

    qkv [T, (H+2K)*hs] (or [T, H*hs] when ``write_kv`` is false); caches
    [pages, K, page_size, hs]; block_table [B, width] int32.
    """
    _dev(qkv, "qkv"); _dev(positions, "positions", torch.int32)
    T = qkv.shape[0]
    width = (n_heads + (2 * n_kv if write_kv else 0)) * head_dim
    if qkv.dim() != 2 or qkv.shape[1] != width or positions.numel() != T:
        raise KernelError(f"rope_cache_write: qkv {tuple(qkv.shape)} for {n_heads}+2*{n_kv} heads of {head_dim}")
    if cos is not None:
        _dev(cos, "cos", torch.float32); _dev(sin, "sin", torch.float32)
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != rot_dim // 2:
            raise KernelError(f"rope_cache_write: table {tuple(cos.shape)} for rot_dim {rot_dim}")
    stride = 0
    if write_kv:
        _dev(seq_of_token, "seq_of_token", torch.int32); _dev(block_table, "block_table", torch.int32)
        _dev(k_cache, "k_cache", qkv.dtype); _dev(v_cache, "v_cache", qkv.dtype)
        if seq_of_token.numel() != T or block_table.dim() != 2:
            raise KernelError("rope_cache_write: seq_of_token / block_table shapes")
        _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, "rope_cache_write")
        stride = block_table.shape[1]
    _check(library().gl3_rope_cache_write(
        _ptr(qkv), _code(qkv, "qkv"), _ptr(positions), _ptr(seq_of_token), _ptr(block_table), stride,
        _ptr(cos), _ptr(sin), _ptr(k_cache), _ptr(v_cache), T, n_heads, n_kv, head_dim, rot_dim, int(adjacent),
        page_size, int(write_kv), _stream()), "rope_cache_write")


def gemm_generic(a, w, out, epilogue=EPI_STORE, bias=None, act="silu"):
    """out = a @ w.T with float multiply-adds; see gemm_generic.hip for the epilogues.
    ``a`` and ``out`` may be row-strided views (last dimension contiguous). ``bias``: float32, one
    per row of ``w``; ``act``: the gated epilogue's activation."""
    _dev(a, "a", contiguous=False); _dev(w, "w"); _dev(out, "out", contiguous=False)
    if a.dim() != 2 or w.dim() != 2 or out.dim() != 2 or a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: operands must be 2-d with a contiguous last dimension")
    M, K = a.shape
    N = out.shape[1]
    rows = 2 * N if epilogue == EPI_GATED else N
    if w.shape != (rows, K) or out.shape[0] != M:
        raise KernelError(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}, epilogue {epilogue}")
    order, wp, pos = _w_order(w)
    _check(library().gl3_gemm_generic(_ptr(a), _code(a, "a"), wp, _code(w, "w"), _ptr(out), _code(out, "out"),
                                      M, N, K, a.stride(0), w.stride(0), out.stride(0), epilogue,
                                      _bias(bias, rows, "gemm_generic"), _act(act, "gemm_generic"), order, pos, _stream()),
           "gemm_generic")


def attention_generic(q, k_cache, v_cache, positions, seq_of_token, block_table, out, n_heads, n_kv, head_dim,
                      page_size, window, scale):
    """q: a [T, >= H*hs] view whose first H*hs columns of each row are the queries."""
    _dev(q, "q", contiguous=False); _dev(out, "out", contiguous=False)
    _dev(k_cache, "k_cache", q.dtype); _dev(v_cache, "v_cache", q.dtype)
    _dev(positions, "positions", torch.int32); _dev(seq_of_token, "seq_of_token", torch.int32)
    _dev(block_table, "block_table", torch.int32)
    T = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < n_heads * head_dim or out.dtype != q.dtype:
        raise KernelError(f"attention: q {tuple(q.shape)} for {n_heads} heads of {head_dim}")
    if out.shape != (T, n_heads * head_dim) or out.stride(1) != 1:
        raise KernelError(f"attention: out {tuple(out.shape)}")
    _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, "attention")
    if positions.numel() != T or seq_of_token.numel() != T or block_table.dim() != 2:
        raise KernelError("attention: positions / seq_of_token / block_table shapes")
    _check(library().gl3_attention_generic(
        _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _code(q, "q"), _ptr(positions), _ptr(seq_of_token),
        _ptr(block_table), block_table.shape[1], _ptr(out), out.stride(0), T, n_heads, n_kv, head_dim, page_size,
        int(window or 0), float(scale), _stream()), "attention_generic")


def decode_advance(token_ids, positions, kv_before, sampled, history, step):
    """Feed the sampled tokens back, move every sequence on by one, log the tokens in row step[0]
    of ``history`` [rows, n], count the step."""
    n = token_ids.numel()
    for t, name in ((token_ids, "token_ids"), (positions, "positions"), (kv_before, "kv_before"),
                    (sampled, "sampled"), (history, "history"), (step, "step")):
        _dev(t, name, torch.int32)
    if positions.numel() != n or kv_before.numel() != n or sampled.numel() < n or history.dim() != 2 or history.shape[1] < n:
        raise KernelError("decode_advance: sizes")
    _check(library().gl3_decode_advance(_ptr(token_ids), _ptr(positions), _ptr(kv_before), _ptr(sampled),
                                        _ptr(history), history.stride(0), _ptr(step), n, _stream()), "decode_advance")


def argmax(logits, work, out):
    """Every row's first greatest logit; ``work``: at least 128 floats per row."""
    _dev(logits, "logits", torch.float32, contiguous=False); _dev(work, "work", torch.float32)
    _dev(out, "out", torch.int32)
    R, V = logits.shape
    if logits.stride(1) != 1 or work.numel() < 128 * R or out.numel() < R:
        raise KernelError("argmax: argument sizes")
    _check(library().gl3_argmax(_ptr(logits), logits.stride(0), _ptr(work), _ptr(out), R, V, _stream()), "argmax")


def argmax_advance(logits, work, out, token_ids, positions, kv_before, history, step):
    """``argmax`` into ``out`` and ``decode_advance`` with its result, in two launches instead of three."""
    _dev(logits, "logits", torch.float32, contiguous=False); _dev(work, "work", torch.float32)
    R, V = logits.shape
    for t, name in ((out, "out"), (token_ids, "token_ids"), (positions, "positions"), (kv_before, "kv_before"),
                    (history, "history"), (step, "step")):
        _dev(t, name, torch.int32)
    if (logits.stride(1) != 1 or work.numel() < 128 * R or out.numel() < R or token_ids.numel() != R
            or positions.numel() != R or kv_before.numel() != R or history.dim() != 2 or history.shape[1] < R or R > 1024):
        raise KernelError("argmax_advance: argument sizes")
    _check(library().gl3_argmax_advance(_ptr(logits), logits.stride(0), _ptr(work), _ptr(out), R, V, _ptr(token_ids),
                                        _ptr(positions), _ptr(kv_before), _ptr(history), history.stride(0), _ptr(step),
                                        _stream()), "argmax_advance")


def sample_work_size(rows, vocab):
    """Floats of scratch that `sample` and `argmax` need for `rows` rows."""
    return max(int(library().gl3_sample_work_floats(int(rows), int(vocab))), 128 * rows)


def sample(logits, work, temperature, top_p, uniform, out, step=None, uniform_stride=0):
    _dev(logits, "logits", torch.float32, contiguous=False); _dev(work, "work", torch.float32)
    for t, n in ((temperature, "temperature"), (top_p, "top_p"), (uniform, "uniform")):
        _dev(t, n, torch.float32)
    _dev(out, "out", torch.int32)
    R, V = logits.shape
    if logits.stride(1) != 1 or work.numel() < sample_work_size(R, V) or min(temperature.numel(), top_p.numel(), uniform.numel(),
                                                              out.numel()) < R:
        raise KernelError("sample: argument sizes")
    if step is not None:
        _dev(step, "step", torch.int32)
    _check(library().gl3_sample(_ptr(logits), logits.stride(0), _ptr(work), _ptr(temperature), _ptr(top_p),
                                _ptr(uniform), _ptr(out), R, V, _ptr(step), int(uniform_stride), _stream()), "sample")


# ------------------------------------------------------------------ bfloat16 product for few rows
def gemm_skinny_fits(a, w, out, epilogue):
    M, K = a.shape
    return (M <= 64 and K % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and (out.dtype == torch.float32 or (out.dtype == torch.bfloat16 and epilogue != EPI_ADD)))


def skinny_strip_rows(M, N, K, epilogue):
    """Rows of w that a block of the skinny kernel takes: 8 where strips of 16 would leave more than a
    third of the CUs without a block. With at most 8 rows of ``a`` the half-empty tile of such a strip
    takes the next 32 k instead (N=2048, 8 rows: K=8192 12.4 -> 9.7 us, K=2048 6.1 -> 4.3 us); with 9
    to 16 rows half the tile idles, which pays only where K is too long for the kernel that keeps its
    rows of ``a`` in registers (17.0 -> 15.8 us at N=2048, K=8192). Else 16."""
    if epilogue == EPI_GATED or -(-N // 16) > 160:
        return 16
    return 8 if M <= 8 or (M <= 16 and K > 4096) else 16


def skinny_keeps_operands(M, K):
    """Whether the skinny product (store epilogue, no folded norm) of ``M`` rows over ``K`` columns runs on
    the kernel whose waves keep their operands of ``a`` in registers: with 17 to 64 rows that is K up to
    2,048, with fewer rows up to 4,096. Beyond it the kernel that streams the rows of ``a`` for every strip
    runs, which a product of very many strips should leave to the tiled kernel."""
    return K <= (2048 if M > 16 else 4096)


def packed_rows(n_columns, dtype, device):
    """A buffer for at most 8 rows of ``n_columns`` elements in the order in which the products of strips of
    8 weight rows read them: [step of 64 columns][lane 16 q + r][8 elements], lane (r, q) holding row r % 8 at
    column 32 (r // 8) + 8 q. A product with ``pack_out`` writes it, one with ``a_packed`` reads it."""
    return torch.empty((-(-n_columns // 64), 64, 8), dtype=dtype, device=device)


def gemm_skinny(a, w, out, epilogue=EPI_STORE, waves=0, ssq_out=None, strip_rows=16, next_weight=None, xg=None,
                bias=None, act="silu", a_packed=False):
    """out (=, +=, gated) a @ w.T on the matrix cores for at most 64 rows of ``a``. ``ssq_out``
    [N/strip_rows, 64] float32 (add epilogue): partial sums of squares of the completed rows; with it
    ``xg`` [M, N] bfloat16 may receive ``next_weight * out``, the rows as the product after the next
    norm reads them. ``a_packed`` (strips of 8 rows, at most 8 rows): ``a`` is a ``packed_rows`` buffer."""
    _dev(a, "a", torch.bfloat16, contiguous=False); _dev(w, "w", torch.bfloat16); _dev(out, "out", contiguous=False)
    if a_packed:
        if (w.dim() != 2 or out.dim() != 2 or out.stride(1) != 1 or not a.is_contiguous()
                or a.numel() < -(-w.shape[1] // 64) * 512 or out.shape[0] > 8 or strip_rows != 8 or waves):
            raise KernelError("gemm_skinny: rows in the packed order go with strips of 8 weight rows and at most 8 rows")
        a = a.view(-1)[:8 * w.shape[1]].view(8, w.shape[1])[:out.shape[0]]     # (the shape only: the kernel knows the order)
    if a.dim() != 2 or w.dim() != 2 or out.dim() != 2 or a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: operands must be 2-d with a contiguous last dimension")
    M, K = a.shape
    N = out.shape[1]
    rows = 2 * N if epilogue == EPI_GATED else N
    if w.shape != (rows, K) or out.shape[0] != M:
        raise KernelError(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}, epilogue {epilogue}")
    if ssq_out is not None:
        _dev(ssq_out, "ssq_out", torch.float32)
        if epilogue != EPI_ADD or N % 16 or ssq_out.numel() < N // strip_rows * 64:
            raise KernelError("gemm_skinny: sums of squares need the add epilogue, N % 16 == 0 and 64 floats a strip")
    _check_next(next_weight, xg, M, N, "gemm_skinny")
    if xg is not None and ssq_out is None:
        raise KernelError("gemm_skinny: the next norm's rows come with the sums of squares")
    if held_once(w) and not (skinny_takes(w, M, strip_rows) and (strip_rows == 8 or _tiled(w, rows, K, n_out=N).value)
                             and a.stride(0) < 2 ** 24 and K < 2 ** 24):
        raise KernelError("gemm_skinny: a weight kept in the matrix cores' order alone is read through the copy whose strips "
                          f"the call names (strips of {strip_rows} rows, {M} rows of a)")
    _check(library().gl3_gemm_skinny(_ptr(a), _ptr(w), _ptr(out), _code(out, "out"), M, N, K, a.stride(0), w.stride(0),
                                     out.stride(0), epilogue, waves, _ptr(ssq_out), strip_rows, _ptr(next_weight),
                                     _ptr(xg), xg.stride(0) if xg is not None else 0, _bias(bias, rows, "gemm_skinny"),
                                     _act(act, "gemm_skinny"), _tiled(w, rows, K, n_out=N), _tiled8(w, rows, K), int(bool(a_packed)),
                                     _stream()), "gemm_skinny")


def strip_rows_of(n_rows, qkv=None):
    """Which row of W is row r of strip t of 16, as the kernels' ``sk_strip_row`` names them: rows
    16 t + r (the last strip repeats the last row), and for the stacked q, k, v rows with half-split
    pairing (``qkv`` = (n_heads, n_kv, head_dim, rotated, adjacent)) 8 rows of a rotated head and the
    8 half a head further, so that both elements of a pair lie in one tile."""
    n_strips = -(-n_rows // 16)
    rows = torch.arange(n_strips * 16).clamp(max=n_rows - 1).view(n_strips, 16)
    if qkv is not None:
        n_heads, n_kv, hs, rotated, adjacent = qkv
        if rotated and not adjacent:
            per_head = hs // 16
            t = torch.arange(n_strips).view(-1, 1)
            r = torch.arange(16).view(1, -1)
            hd, sub = t // per_head, t % per_head
            paired = hd * hs + 8 * sub + torch.where(r < 8, r, hs // 2 + r - 8)
            rows = torch.where(hd < n_heads + n_kv, paired, rows)
    return rows.reshape(-1)


def tile_weight(w, qkv=None):
    """A copy of ``w`` [N, K] (bfloat16, N % 16 == 0) in the order in which the matrix cores take it as an
    operand: [strip of 16 rows][k-step of 32][lane = 16 * (k block of 8) + row][8 elements], k padded with
    zeros to whole steps. The products of few rows whose kernels keep their rows of A in registers read
    it where a weight carries one (``w.tiled``): a load is then 1 KB of consecutive memory."""
    N, K = w.shape
    if N % 16 or w.dtype != torch.bfloat16:
        raise KernelError(f"tile_weight: {tuple(w.shape)} {w.dtype}")
    steps = -(-K // 32)
    rows = strip_rows_of(N, qkv).to(w.device)
    wp = torch.zeros(N, steps * 32, dtype=w.dtype, device=w.device)
    wp[:, :K] = w[rows]
    t = wp.view(N // 16, 16, steps, 4, 8).permute(0, 2, 3, 1, 4).contiguous()
    t.tiled_for = qkv
    if not torch.equal(rows, torch.arange(N, device=rows.device)):
        # the place of each stored row in the copy, for the kernels that read the copy row by row
        t.row_pos = torch.empty(N, dtype=torch.int32, device=w.device)
        t.row_pos[rows] = torch.arange(N, dtype=torch.int32, device=w.device)
    return t


def tile_weight8(w):
    """A copy of ``w`` [N, K] (bfloat16, N % 8 == 0) in the order of the packed tiles that the products of
    at most 8 rows use for strips of 8 weight rows: [strip of 8 rows][step of 64 k][lane][8 elements], lane
    16 q + r holding row r % 8 at k = 32 (r // 8) + 8 q, k padded with zeros to whole steps."""
    N, K = w.shape
    if N % 8 or w.dtype != torch.bfloat16:
        raise KernelError(f"tile_weight8: {tuple(w.shape)} {w.dtype}")
    steps = -(-K // 64)
    wp = torch.zeros(N, steps * 64, dtype=w.dtype, device=w.device)
    wp[:, :K] = w
    # [strip, row, step, half, q, element] -> [strip, step, q, half, row, element]
    return wp.view(N // 8, 8, steps, 2, 4, 8).permute(0, 2, 4, 3, 1, 5).contiguous()


def untile_weight(t, n_rows, K):
    """The rows of a matrix out of its copy in the matrix operands' order (``tile_weight``): a new tensor
    [n_rows, K] in the stored order."""
    steps = -(-K // 32)
    rows = t.view(n_rows // 16, steps, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(n_rows, steps * 32)[:, :K]
    pos = getattr(t, "row_pos", None)
    return (rows[pos.long()] if pos is not None else rows).contiguous()


def untile_weight8(t, n_rows, K):
    """The same out of the copy in packed strips of 8 rows (``tile_weight8``)."""
    steps = -(-K // 64)
    # [strip, step, q, half, row, element] -> [strip, row, step, half, q, element]
    return t.view(n_rows // 8, steps, 4, 2, 8, 8).permute(0, 4, 1, 3, 2, 5).reshape(n_rows, steps * 64)[:, :K].contiguous()


def stored_order(w):
    """``w`` as the rows lie in the model's file: ``w`` itself, or (held once) rebuilt from a copy, a new tensor."""
    if not held_once(w):
        return w
    t = getattr(w, "tiled", None)
    return untile_weight(t, *w.shape) if t is not None else untile_weight8(w.tiled8, *w.shape)


def can_hold_once(w):
    """Whether one of the copies that ``w`` carries has exactly the matrix's elements, over whole steps of 64 k
    (the tiled product's step), so that it can stand for the matrix."""
    N, K = w.shape
    t, t8 = getattr(w, "tiled", None), getattr(w, "tiled8", None)
    return K % 64 == 0 and ((t is not None and N % 16 == 0 and t.numel() == N * K)
                            or (t8 is not None and N % 8 == 0 and t8.numel() == N * K))


def hold_once(w):
    """``w`` (which carries ``w.tiled`` and/or ``w.tiled8``, over whole steps of k) as a matrix that is kept in
    the matrix cores' order alone: a tensor of the same shape and dtype whose memory IS a copy. Whoever drops
    ``w`` then frees the stored order. The kernels that read any order (the embedding, the generic and the tiled
    product, the kernel of whole lines, and those of few rows that take the copies anyway) are told by
    ``held_once``; the others refuse it."""
    if not can_hold_once(w):
        raise KernelError(f"hold_once: {tuple(w.shape)} has no copy in the matrix cores' order that could stand for it")
    N, K = w.shape
    t, t8 = getattr(w, "tiled", None), getattr(w, "tiled8", None)
    base = t if (t is not None and N % 16 == 0 and t.numel() == N * K) else t8
    alias = base.view(N, K)
    alias.operand_order_only = True
    if t is not None:
        alias.tiled = t
    if t8 is not None:
        alias.tiled8 = t8
    return alias


def skinny_takes(w, M, strip_rows, qkv=None):
    """Whether the products of few rows can read ``w`` in strips of ``strip_rows``: always when the stored order
    is there; a weight that is held once through the copy whose strips those are (rows in order, or for ``qkv``)."""
    if not held_once(w):
        return True
    N, K = w.shape
    if strip_rows == 8:
        return M <= 8 and bool(_tiled8(w, N, K).value)
    return bool(_tiled(w, N, K, qkv=qkv).value)


def _tiled8(w, n_rows, K):
    t = getattr(w, "tiled8", None)
    if t is None or n_rows % 8 or t.numel() != n_rows * -(-K // 64) * 64:
        return c_void_p(0)
    return _ptr(t)


def _tiled(w, n_rows, K, qkv=None, n_out=None):
    """The pointer to ``w.tiled`` if the weight carries a copy in the operands' order that fits this call
    (``n_out``: the output columns, where the gate rows and the up rows must each fill whole strips)."""
    t = getattr(w, "tiled", None)
    if (t is None or n_rows % 16 or (n_out is not None and n_out % 16) or t.numel() != n_rows * -(-K // 32) * 32
            or getattr(t, "tiled_for", None) != qkv):
        return c_void_p(0)
    return _ptr(t)


def gemm_skinny_wide_fits(a, w, out, epilogue):
    return (8 < a.shape[0] <= 64 and gemm_skinny_fits(a, w, out, epilogue)
            and not (held_once(w) and getattr(getattr(w, "tiled", None), "row_pos", None) is not None))


def wide_slices(N, K):
    """Into how many slices of K the wide kernel's product [*, K] x [N, K] is cut: enough blocks for
    the chip (a block takes 32 columns where they are few), at least one pair of k-steps (64 k) for
    each of a block's 8 waves."""
    return max(1, min(8, 256 // -(-N // 32), K // 512))


def gemm_skinny_wide(a, w, out, epilogue=EPI_STORE, strips=0, bias=None, act="silu"):
    """out (=, +=, gated) a @ w.T for 17 to 64 rows of ``a``. ``out`` with three axes [slices, M, N]
    (float32, store epilogue) takes the sums of one slice of K each: the caller adds them up; that form
    also takes 9 to 16 rows."""
    _dev(a, "a", torch.bfloat16, contiguous=False); _dev(w, "w", torch.bfloat16); _dev(out, "out", contiguous=False)
    M, K = a.shape
    slices, slice_stride = 1, 0
    rows = out
    if out.dim() == 3:
        slices, slice_stride, rows = out.shape[0], out.stride(0), out[0]
    N = rows.shape[1]
    wrows = 2 * N if epilogue == EPI_GATED else N
    if (w.shape != (wrows, K) or rows.shape[0] != M or rows.stride(1) != 1 or a.stride(1) != 1
            or not (16 < M <= 64 or (8 < M <= 16 and epilogue == EPI_STORE and out.dtype == torch.float32))):
        raise KernelError(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}, epilogue {epilogue}")
    order, wp, pos = _w_order(w)
    if pos.value:
        raise KernelError("gemm_skinny_wide: a copy whose strips hold the rows in another order is not read row by row")
    _check(library().gl3_gemm_skinny_wide(_ptr(a), wp, _ptr(out), _code(out, "out"), M, N, K, a.stride(0),
                                          w.stride(0), rows.stride(0), epilogue, slices, slice_stride, strips,
                                          _bias(bias, wrows, "gemm_skinny_wide"), _act(act, "gemm_skinny_wide"),
                                          None, 0, 0.0, 0, order, _stream()), "gemm_skinny_wide")


def _check_norm_args(xg, ssq, n_partials, K):
    _dev(xg, "xg", torch.bfloat16, contiguous=False); _dev(ssq, "ssq", torch.float32)
    if xg.dim() != 2 or xg.stride(1) != 1 or xg.shape[1] != K:
        raise KernelError(f"folded norm: rows {tuple(xg.shape)} for K={K}")
    if xg.shape[0] > 64 or n_partials < 1 or ssq.numel() < n_partials * 64:
        raise KernelError("folded norm: at most 64 rows, and n_partials * 64 partial sums")


def gemm_skinny_norm_fits(xg, w, out, epilogue):
    K = xg.shape[1]
    return (xg.shape[0] <= 64 and K % 8 == 0 and xg.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and xg.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and w.dtype == torch.bfloat16
            and ((epilogue == EPI_STORE and out.dtype in (torch.float32, torch.bfloat16))
                 or (epilogue == EPI_GATED and out.dtype == torch.bfloat16)))


def gemm_skinny_norm(xg, ssq, n_partials, eps, w, out, epilogue=EPI_STORE, rows=None, waves=0, bias=None, act="silu",
                     pack_out=False, whole_lines=False):
    """out (=, gated) RMSNorm(x)[rows] @ w.T, where ``xg`` = bfloat16(norm weight * x) was left by the
    kernel that completed the rows of x, together with their sums of squares as partial sums.
    ``pack_out`` (at most 8 rows, bfloat16): ``out`` is a ``packed_rows`` buffer. ``whole_lines`` (gated
    epilogue, at most 16 rows, all rows): the kernel that loads both operands as whole lines and takes
    several strips a block (``gemm_skinny_wide``'s) does the work."""
    _dev(w, "w", torch.bfloat16); _dev(out, "out", contiguous=False)
    K = w.shape[1]
    _check_norm_args(xg, ssq, n_partials, K)
    M = xg.shape[0]
    if rows is not None:
        _dev(rows, "rows", torch.int32)
        M = rows.numel()
    if pack_out:
        n_out = w.shape[0] // 2 if epilogue == EPI_GATED else w.shape[0]
        if M > 8 or out.dtype != torch.bfloat16 or not out.is_contiguous() or out.numel() < -(-n_out // 64) * 512:
            raise KernelError("gemm_skinny_norm: the packed order holds at most 8 rows of bfloat16")
        out = out.view(-1)[:8 * n_out].view(8, n_out)[:M]                      # (the shape only: the kernel knows the order)
    N = out.shape[1]
    wrows = 2 * N if epilogue == EPI_GATED else N
    if w.shape != (wrows, K) or out.shape[0] != M or out.stride(1) != 1 or M > 64:
        raise KernelError(f"gemm: rows {tuple(xg.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}, epilogue {epilogue}")
    if held_once(w) and not whole_lines and not _tiled(w, wrows, K, n_out=N).value:
        raise KernelError("gemm_skinny_norm: a weight kept in the matrix cores' order alone is read through its copy")
    if whole_lines:
        if epilogue != EPI_GATED or rows is not None or M > 16 or waves:
            raise KernelError("gemm_skinny_norm: whole lines go with the gated epilogue, at most 16 rows, all of them")
        order, wp, pos = _w_order(w)
        if pos.value or order == 2:
            raise KernelError("gemm_skinny_norm: the gated product of whole lines reads stored rows or the operands' order")
        return _check(library().gl3_gemm_skinny_wide(
            _ptr(xg), wp, _ptr(out), _code(out, "out"), M, N, K, xg.stride(0), w.stride(0), out.stride(0), epilogue,
            1, 0, 0, _bias(bias, wrows, "gemm_skinny_norm"), _act(act, "gemm_skinny_norm"), _ptr(ssq), n_partials,
            float(eps), int(bool(pack_out)), order, _stream()), "gemm_skinny_wide")
    _check(library().gl3_gemm_skinny_norm(
        _ptr(xg), _ptr(rows), _ptr(ssq), n_partials, float(eps), _ptr(w), _ptr(out), _code(out, "out"), M, N, K,
        xg.stride(0), w.stride(0), out.stride(0), epilogue, waves, _bias(bias, wrows, "gemm_skinny_norm"),
        _act(act, "gemm_skinny_norm"), _tiled(w, wrows, K, n_out=N), int(bool(pack_out)), _stream()), "gemm_skinny_norm")


def qkv_rope_cache_fits(a, w_qkv, head_dim, rot_dim):
    """a: normalised bfloat16 rows, or bfloat16(norm weight * x) with the sums of squares."""
    K = a.shape[1]
    return (a.shape[0] <= 64 and a.stride(1) == 1 and a.dtype == torch.bfloat16 and K % 8 == 0
            and a.stride(0) % 8 == 0 and w_qkv.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and w_qkv.data_ptr() % 16 == 0 and w_qkv.dtype == torch.bfloat16
            and head_dim % 16 == 0 and rot_dim in (0, head_dim))


def token_facts(positions, table_rows, block_table, page_size, cos, sin, pages, rot, tables=None):
    """What hangs on each token's position, looked up once for all layers of a step: ``pages`` [T] int32
    receives the page of the token's position (``block_table[table_rows[t]][positions[t] // page_size]``) and
    ``rot`` [T, 2 * half] float32 its rows of ``cos`` and ``sin`` one after the other (``cos``, ``sin``, ``rot``
    all None: no rotation, the pages alone). ``qkv_rope_cache`` takes both in place of its own look-ups.
    ``tables`` [T, width of ``block_table``] int32 (optional) receives each token's row of the block table up to
    its position's page: ``attention_decode`` reads it with ``seq_of_token=None``."""
    _dev(positions, "positions", torch.int32); _dev(table_rows, "table_rows", torch.int32)
    _dev(block_table, "block_table", torch.int32); _dev(pages, "pages", torch.int32)
    T = positions.numel()
    if table_rows.numel() != T or pages.numel() != T or block_table.dim() != 2:
        raise KernelError("token_facts: one row of the table and one page per token")
    half = 0
    if cos is not None:
        _dev(cos, "cos", torch.float32); _dev(sin, "sin", torch.float32); _dev(rot, "rot", torch.float32)
        half = cos.shape[1]
        if cos.shape != sin.shape or cos.dim() != 2 or rot.shape != (T, 2 * half):
            raise KernelError(f"token_facts: tables {tuple(cos.shape)}, rows {tuple(rot.shape)} for {T} tokens")
    elif sin is not None or rot is not None:
        raise KernelError("token_facts: the tables and the rows for them come together")
    if tables is not None:
        _dev(tables, "tables", torch.int32)
        if tables.shape != (T, block_table.shape[1]):
            raise KernelError(f"token_facts: the tokens' rows {tuple(tables.shape)} of a table {tuple(block_table.shape)}")
    _check(library().gl3_token_facts(_ptr(positions), _ptr(table_rows), _ptr(block_table), block_table.shape[1], int(page_size),
                                     _ptr(cos), _ptr(sin), half, _ptr(pages), _ptr(rot), _ptr(tables), T, _stream()),
           "token_facts")


def qkv_rope_cache(a, ssq, n_partials, eps, w_qkv, q_out, positions, seq_of_token, block_table, cos, sin,
                   k_cache, v_cache, n_heads, n_kv, head_dim, adjacent, page_size, waves=0, token_pages=None, token_rot=None):
    """a @ w_qkv.T, rotation, q into ``q_out`` [T, H*hs] bfloat16, k and v into the cache. ``ssq`` None:
    ``a`` holds the rows as they are; else ``a`` = bfloat16(norm weight * x) and the product is that
    of RMSNorm(x), the rows' sums of squares coming as partial sums. ``token_pages``, ``token_rot``: what
    ``token_facts`` made of the same positions, table and rotation (then the kernel does not look them up)."""
    _dev(w_qkv, "w_qkv", torch.bfloat16); _dev(q_out, "q_out", torch.bfloat16, contiguous=False)
    K = w_qkv.shape[1]
    if ssq is None:
        _dev(a, "a", torch.bfloat16, contiguous=False)
        if a.dim() != 2 or a.stride(1) != 1 or a.shape[1] != K or a.shape[0] > 64:
            raise KernelError(f"qkv_rope_cache: rows {tuple(a.shape)} for K={K}")
        n_partials = 0
    else:
        _check_norm_args(a, ssq, n_partials, K)
    T = a.shape[0]
    _dev(positions, "positions", torch.int32); _dev(seq_of_token, "seq_of_token", torch.int32)
    _dev(block_table, "block_table", torch.int32)
    _dev(k_cache, "k_cache", torch.bfloat16); _dev(v_cache, "v_cache", torch.bfloat16)
    _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, "qkv_rope_cache")
    if (w_qkv.shape[0] != (n_heads + 2 * n_kv) * head_dim or q_out.shape[0] != T or q_out.stride(1) != 1
            or q_out.shape[1] < n_heads * head_dim or positions.numel() != T or seq_of_token.numel() != T
            or block_table.dim() != 2):
        raise KernelError("qkv_rope_cache: shapes")
    if cos is not None:
        _dev(cos, "cos", torch.float32); _dev(sin, "sin", torch.float32)
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != head_dim // 2:
            raise KernelError(f"qkv_rope_cache: table {tuple(cos.shape)} for head_dim {head_dim}")
    # (the kernel reads the tables through 32-bit byte offsets)
    if block_table.numel() >= 2 ** 29 or (cos is not None and cos.numel() >= 2 ** 29):
        raise KernelError("qkv_rope_cache: a block table or rotation table of 2 GiB or more")
    if token_pages is not None:
        _dev(token_pages, "token_pages", torch.int32)
        if token_pages.numel() != T or (cos is not None and (token_rot is None or token_rot.dtype != torch.float32
                                                             or token_rot.shape != (T, head_dim) or not token_rot.is_cuda
                                                             or not token_rot.is_contiguous())):
            raise KernelError("qkv_rope_cache: a page per token, and with a rotation a row [head_dim] of cos and sin per token")
    copy = _tiled(w_qkv, w_qkv.shape[0], K, qkv=(n_heads, n_kv, head_dim, cos is not None, bool(adjacent)))
    if held_once(w_qkv) and not copy.value:
        raise KernelError("qkv_rope_cache: weights kept in the operands' order alone need the copy made for this rotation")
    _check(library().gl3_qkv_rope_cache(
        _ptr(a), _ptr(ssq), n_partials, float(eps), _ptr(w_qkv), _ptr(q_out), q_out.stride(0), T, K, a.stride(0),
        w_qkv.stride(0), _ptr(positions), _ptr(seq_of_token), _ptr(block_table), block_table.shape[1], _ptr(cos),
        _ptr(sin), _ptr(k_cache), _ptr(v_cache), n_heads, n_kv, head_dim, int(adjacent), page_size, waves,
        copy, _ptr(token_pages), _ptr(token_rot if token_pages is not None and cos is not None else None),
        int(held_once(w_qkv)), _stream()),
        "qkv_rope_cache")


# ------------------------------------------------------------------ bfloat16 attention of a decode step
def attention_decode_fits(head_dim, n_heads, n_kv, page_size):
    return bool(library().gl3_attention_decode_supports(head_dim, page_size)) and n_heads % n_kv == 0


def decode_splits(n_tokens, n_heads, n_kv, kv_len, head_dim=64):
    """Blocks that share a sequence's keys. A split costs a second kernel that merges the parts, which
    is worth its few microseconds only when a block would otherwise walk hundreds of KB of keys (more
    than 128 K elements, or 256 K and more where the step has more than 16 blocks anyway; ``kv_len`` is
    what the launch is sized for, in a replayed step the next power of two, so 4,096 stands for 2,049
    to 4,096 keys), then one split per 64 K elements (per 32 K where the step has at most 16 blocks: one
    sequence of the 1B layers at 4,000 keys, 0.865 -> 0.822 ms a step; the same within 1% at 8,000 to 32,768 keys),
    and only until every CU has a block: more splits than that were slower at every batch and context
    measured (heads of 64, 16 sequences at 8,200 keys: 54 us with 2 splits, 63 us with 8)."""
    blocks = n_tokens * n_kv * -(-(n_heads // n_kv) // 16)
    elements = kv_len * head_dim
    if elements <= 131072 or (blocks > 16 and elements < 262144):
        return 1
    return int(max(1, min(elements // (32768 if blocks <= 16 else 65536), 256 // blocks, 32)))


def attention_decode(q, k_cache, v_cache, positions, seq_of_token, block_table, out, n_heads, n_kv, head_dim,
                     page_size, window, scale, n_splits, part_o=None, part_ml=None):
    """One token per sequence. ``part_o`` [T, H, splits, hs] and ``part_ml`` [T, H, splits, 2] float32
    are needed when ``n_splits`` > 1 (contiguous, adjacent is not required). ``seq_of_token`` None: token t's
    pages are row t of ``block_table`` (a table of the step's own, as ``token_facts`` makes it)."""
    _dev(q, "q", torch.bfloat16, contiguous=False); _dev(out, "out", torch.bfloat16, contiguous=False)
    _dev(k_cache, "k_cache", torch.bfloat16); _dev(v_cache, "v_cache", torch.bfloat16)
    _dev(positions, "positions", torch.int32); _dev(block_table, "block_table", torch.int32)
    if seq_of_token is not None:
        _dev(seq_of_token, "seq_of_token", torch.int32)
    T = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < n_heads * head_dim:
        raise KernelError(f"attention: q {tuple(q.shape)} for {n_heads} heads of {head_dim}")
    if out.shape != (T, n_heads * head_dim) or out.stride(1) != 1:
        raise KernelError(f"attention: out {tuple(out.shape)}")
    _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, "attention")
    if (positions.numel() != T or block_table.dim() != 2
            or (seq_of_token.numel() != T if seq_of_token is not None else block_table.shape[0] < T)):
        raise KernelError("attention: positions / seq_of_token / block_table shapes")
    floats = 0
    if n_splits > 1:
        _dev(part_o, "part_o", torch.float32); _dev(part_ml, "part_ml", torch.float32)
        if part_o.numel() < T * n_heads * n_splits * head_dim or part_ml.numel() < T * n_heads * n_splits * 2:
            raise KernelError("attention: the workspace of the splits is too small")
        floats = T * n_heads * n_splits * (head_dim + 2)
    _check(library().gl3_attention_decode(
        _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(positions), _ptr(seq_of_token), _ptr(block_table),
        block_table.shape[1], _ptr(part_o), _ptr(part_ml), floats, _ptr(out), out.stride(0), T, n_heads, n_kv,
        head_dim, page_size, int(window or 0), float(scale), n_splits, _stream()), "attention_decode")


# ------------------------------------------------------------------ bfloat16 product for many rows
def gemm_mfma_fits(a, w, out, epilogue):
    M, K = a.shape
    return (K % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and (out.dtype == torch.float32 or (out.dtype == torch.bfloat16 and epilogue != EPI_ADD)))


def gemm_mfma(a, w, out, epilogue=EPI_STORE, more_slices=None, bias=None, act="silu", shape=0):
    """out (=, +=, gated) a @ w.T on the matrix cores, tiled for many rows of ``a``. With
    ``more_slices`` [S, M, N] float32 K is cut into S + 1 slices: the first goes into ``out``, the
    others' sums are stored there, for the caller to add to ``out`` in that order."""
    _dev(a, "a", torch.bfloat16, contiguous=False); _dev(w, "w", torch.bfloat16); _dev(out, "out", contiguous=False)
    slices, p_stride, ldp = 1, 0, 0
    if more_slices is not None:
        _dev(more_slices, "more_slices", torch.float32, contiguous=False)
        if (more_slices.dim() != 3 or more_slices.shape[1:] != out.shape or more_slices.stride(2) != 1
                or epilogue == EPI_GATED):
            raise KernelError(f"gemm: slices {tuple(more_slices.shape)} for out {tuple(out.shape)}, epilogue {epilogue}")
        slices, p_stride, ldp = more_slices.shape[0] + 1, more_slices.stride(0), more_slices.stride(1)
    if a.dim() != 2 or w.dim() != 2 or out.dim() != 2 or a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: operands must be 2-d with a contiguous last dimension")
    M, K = a.shape
    N = out.shape[1]
    rows = 2 * N if epilogue == EPI_GATED else N
    if w.shape != (rows, K) or out.shape[0] != M:
        raise KernelError(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}, epilogue {epilogue}")
    order, wp, pos = _w_order(w)
    _check(library().gl3_gemm_mfma(_ptr(a), wp, _ptr(out), _code(out, "out"), M, N, K, a.stride(0), w.stride(0),
                                   out.stride(0), epilogue, slices, _ptr(more_slices), p_stride, ldp,
                                   _bias(bias, rows, "gemm_mfma"), _act(act, "gemm_mfma"), int(shape), order, pos, _stream()),
           "gemm_mfma")


def mfma_slices(M, N, K):
    """Into how many slices of K the tiled product [M, K] x [N, K] into the residual stream is cut
    where the tiles of 128 x 128 are at most one for each of the chip's 512 places (two blocks a CU).
    A block's time is its walk along K (half a microsecond per 64 columns, whatever else runs), so few
    tiles over a long K are better cut, down to slices of 512 columns; the norm that follows adds the
    slices up."""
    tiles = -(-M // 128) * -(-N // 128)
    return max(1, min(8, 512 // tiles, K // 512))


def mfma_plan(M, N, K):
    """(tile shape, slices of K) for the tiled product [M, K] x [N, K] into the residual stream, whose
    slices the norm that follows adds up. Few tiles: tiles of 128 x 128 and ``mfma_slices``. More tiles
    than places: the plan with the least estimated time among tiles of 128 (512 places) or 256 (256
    places) with one to four slices and tiles of 128 rows x 256 (256 places) with one, the estimate being (rounds the blocks need on their places) x
    (steps of 64 columns a block walks) x (time of such a step with the chip full: 1.05 us and 1.7 us)
    + what the norm pays per slice (0.35 us per MB). What decides is the last, partly empty round:
    276 tiles of 256 take two rounds for the work of 1.08, and two slices of them 2.16 of 3. Fitted to
    60 sizes (300 to 8,192 rows, the output and down projections of three models) times ten plans: the
    plan chosen is on average 1.4% slower than the best one measured, 13% at worst; one slice and the
    tile by the number of tiles alone was 4.1% and 36%."""
    if -(-M // 128) * -(-N // 128) <= 256:
        return 1, mfma_slices(M, N, K)
    best = None
    # (tile rows, tile columns, places on the chip, time of a step of 64 columns with the chip full); the tile of 128
    # rows x 256, one block a CU, whole K only: 0.95 us a step. It is the plan where its tiles are one round and the
    # others need two rounds or slices: the output projection of 2,048 rows of the 3B layers 81 -> 68 us with its norm,
    # of the 8B layers 110 -> 97 us, of 5,886 rows 307 -> 280 us, of 4,096 rows of the 1B layers 64 -> 60 us.
    for shape, rows, cols, places, step_us in ((1, 128, 128, 512, 1.05), (2, 256, 256, 256, 1.7), (5, 128, 256, 256, 0.95)):
        for slices in ((1,) if shape == 5 else (1, 2, 3, 4)):
            if slices > 1 and K // slices < 512:
                continue
            blocks = -(-M // rows) * -(-N // cols) * slices
            estimate = -(-blocks // places) * -(-K // (64 * slices)) * step_us + 0.35e-6 * (slices + 1.5) * M * N * 4
            if best is None or estimate < best[0]:
                best = (estimate, shape, slices)
    return best[1], best[2]


# ------------------------------------------------------------------ bfloat16 attention of a prefill step
def attention_prefill_fits(head_dim, n_heads, n_kv, page_size):
    return bool(library().gl3_attention_prefill_supports(head_dim, page_size)) and n_heads % n_kv == 0


def attention_prefill(q, k_cache, v_cache, cu_seqlens, kv_before, block_table, out, max_q_len, n_heads, n_kv,
                      head_dim, page_size, window, scale, seq_rows=None, wide_from=0):
    """Any number of tokens per sequence; ``cu_seqlens`` [B+1] and ``kv_before`` [B] say which tokens
    of the packed ``q`` belong to which sequence and where they sit in it. ``seq_rows`` [B] (optional)
    names each sequence's row of ``block_table``; without it sequence b reads row b. ``wide_from``: from
    how many tokens of the step's longest sequence on the kernel with 128 queries a block runs
    (0: the library's choice; tests run both kernels on the same inputs)."""
    _dev(q, "q", torch.bfloat16, contiguous=False); _dev(out, "out", torch.bfloat16, contiguous=False)
    _dev(k_cache, "k_cache", torch.bfloat16); _dev(v_cache, "v_cache", torch.bfloat16)
    _dev(cu_seqlens, "cu_seqlens", torch.int32); _dev(kv_before, "kv_before", torch.int32)
    _dev(block_table, "block_table", torch.int32)
    T = q.shape[0]
    B = kv_before.numel()
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < n_heads * head_dim:
        raise KernelError(f"attention: q {tuple(q.shape)} for {n_heads} heads of {head_dim}")
    if out.shape != (T, n_heads * head_dim) or out.stride(1) != 1:
        raise KernelError(f"attention: out {tuple(out.shape)}")
    _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, "attention")
    if cu_seqlens.numel() != B + 1 or block_table.dim() != 2 or max_q_len < 1:
        raise KernelError("attention: cu_seqlens / kv_before / block_table shapes")
    if seq_rows is not None:
        _dev(seq_rows, "seq_rows", torch.int32)
        if seq_rows.numel() != B:
            raise KernelError("attention: one table row per sequence")
    elif block_table.shape[0] < B:
        raise KernelError("attention: the block table has fewer rows than there are sequences")
    _check(library().gl3_attention_prefill(
        _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(cu_seqlens), _ptr(kv_before), _ptr(block_table),
        _ptr(seq_rows), block_table.shape[1], _ptr(out), out.stride(0), B, int(max_q_len), n_heads, n_kv, head_dim,
        page_size, int(window or 0), float(scale), int(wide_from), _stream()), "attention_prefill")


# ------------------------------------------------------------------ host to device without tensor objects
def scatter_i32(dst, places, values):
    """dst.view(-1)[places[i]] = values[i]: the places and values travel in the launch itself."""
    _dev(dst, "dst", torch.int32)
    n = len(places)
    if n != len(values):
        raise KernelError("scatter_i32: as many places as values")
    if n == 0:
        return
    arr = (c_int * n)
    _check(library().gl3_scatter_i32(_ptr(dst), dst.numel(), arr(*places), arr(*values), n, _stream()), "scatter_i32")


def stage_decode(dst, n_pad, tokens, positions, slots, pad_slot, counter=None):
    """The input of a captured decode step into its device buffer ``dst`` (int32, 4 * n_pad at least):
    tokens | positions | tokens held before | slots of ``len(tokens)`` sequences, padded to ``n_pad``
    with one-token sequences in ``pad_slot``. The numbers travel inside the launch."""
    n = len(tokens)
    if len(positions) != n or len(slots) != n or n > n_pad or dst.numel() < 4 * n_pad:
        raise KernelError("stage_decode: sizes")
    arr = c_int * n
    _check(library().gl3_stage_decode(_ptr(dst), n_pad, n, arr(*tokens), arr(*positions), arr(*slots), pad_slot,
                                      _ptr(counter), _stream()), "stage_decode")


def stage_step_ints(T, B, W):
    """Elements of the device buffer that ``stage_step`` fills."""
    return 4 * T + 3 * B + 1 + W


def stage_step(dev, pinned, tokens, slots, starts, counts, want, vocab):
    """The input of a step of any shape into its device buffer ``dev`` (int32):
    tokens[T] | cu_seqlens[B+1] | kv_before[B] | slots[B] | wanted rows[W] | positions[T] | seq_of_token[T] | table_rows[T].
    ``tokens`` [T], ``want`` [W]: contiguous int32 numpy arrays (the entries' tokens one after another, packed
    rows); ``slots``, ``starts``, ``counts``: one int per entry. The host's part travels as one copy out of
    ``pinned`` (pinned int32 host tensor, free again once that copy has run), the per-token arrays are expanded
    on the device. Token ids are checked against ``vocab``, counts against ``tokens``, rows against T."""
    _dev(dev, "dev", torch.int32)
    T, B, W = int(tokens.size), len(slots), int(want.size)
    if len(starts) != B or len(counts) != B or B == 0 or T == 0:
        raise KernelError("stage_step: one slot, start and count per entry, and at least one token")
    if (tokens.dtype != "int32" or want.dtype != "int32" or not tokens.flags.c_contiguous or not want.flags.c_contiguous
            or tokens.ndim != 1 or want.ndim != 1):
        raise KernelError("stage_step: tokens and wanted rows are contiguous int32 arrays")
    if pinned.is_cuda or not pinned.is_pinned() or pinned.dtype != torch.int32 or pinned.numel() < T + 3 * B + 1 + W:
        raise KernelError("stage_step: the staging buffer must be pinned int32 host memory of T + 3 B + 1 + W elements")
    if dev.numel() < 4 * T + 3 * B + 1 + W:
        raise KernelError("stage_step: the device buffer is too small")
    arr = c_int * B
    _check(library().gl3_stage_step(_ptr(dev), c_void_p(pinned.data_ptr()), c_void_p(tokens.ctypes.data), T, arr(*slots),
                                    arr(*starts), arr(*counts), B, c_void_p(want.ctypes.data if W else 0), W, int(vocab),
                                    _stream()), "stage_step")


def graph_launch(graph_exec):
    """Launch an instantiated graph (its raw handle) on the current stream."""
    _check(library().gl3_graph_launch(c_void_p(graph_exec), _stream()), "graph_launch")


def upload(dst, src_pinned, n_bytes=None):
    """Copy from pinned host memory to the device on the current stream."""
    _dev(dst, "dst")
    if src_pinned.is_cuda or not src_pinned.is_pinned():
        raise KernelError("upload: the source must be pinned host memory")
    n = src_pinned.numel() * src_pinned.element_size() if n_bytes is None else int(n_bytes)
    if n > dst.numel() * dst.element_size() or n > src_pinned.numel() * src_pinned.element_size():
        raise KernelError("upload: more bytes than the tensors hold")
    _check(library().gl3_upload(_ptr(dst), c_void_p(src_pinned.data_ptr()), n, _stream()), "upload")

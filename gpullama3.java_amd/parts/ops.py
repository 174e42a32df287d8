"""Which kernel runs an operation: chosen by dtype and shape, never silently wrong.

float32 activations always take the 32-bit kernels (plain multiply-adds, accurate
exp and sqrt). bfloat16 activations take the matrix-core kernels where the shape
fits what they are written for and the generic kernels otherwise.
"""
from __future__ import annotations

import torch

from ..csrc import lib as K

EPI_STORE, EPI_ADD, EPI_GATED = K.EPI_STORE, K.EPI_ADD, K.EPI_GATED

# a norm is folded into the next product for steps of at most this many tokens (one token tile); larger
# steps take the kernels for 17 to 64 rows or the tiled ones, with a norm kernel of its own. (With 17 to 32
# rows the folded products lose to those kernels: a block of the skinny kernel reads the step's rows again
# for every strip of 16 weight rows. Decode steps of the 1B / 8B layers at batch 32: 0.474 -> 0.386 ms and
# 1.008 -> 0.814 ms for four layers and the head.)
FUSE_ROWS = 16
# a decode step of up to this many rows is worked on in pieces of at most 64 rows; from 129 rows on the
# tiled kernel's two row tiles are faster than three pieces (8B layers, 192 rows: 2.03 -> 1.69 ms for
# four layers and the head)
CHUNK_ROWS = 128

# Switches for tests and measurements: names of fast paths that an engine must not use (``Engine(without=...)``;
# a step reads them as ``ctx.disabled``, a part that makes copies of its weights as its attribute ``without``, which
# the decoder sets before ``load``). "skinny", "wide", "mfma", "attn_decode", "attn_prefill": a family of kernels;
# "fused": norms, rotation and cache write folded into products; "tiled", "packed": the weights' copies in operand
# order and the rows handed over in the packed tiles' order; "widefold", "wide916": the kernel of whole lines for
# the gated product with a folded norm and for products of 9 to 16 rows over a long K; "once": a weight whose
# readers all take the operands' order kept in that order alone (with any switch set, both orders are kept).
SWITCHES = frozenset({"skinny", "wide", "mfma", "attn_decode", "attn_prefill", "fused", "tiled", "packed", "widefold",
                      "wide916", "once"})
_NONE = frozenset()


def switches(names):
    """``names`` (a string with commas, or any collection) as a frozen set; an unknown name is an error."""
    if isinstance(names, str):
        names = [n for n in names.split(",") if n]
    names = frozenset(names or ())
    if names - SWITCHES:
        raise ValueError(f"unknown fast path {sorted(names - SWITCHES)}; known: {sorted(SWITCHES)}")
    return names


def _off(ctx):
    """The fast paths that the step's engine has switched off."""
    return getattr(ctx, "disabled", _NONE) if ctx is not None else _NONE


def for_few_rows(w, qkv=None, without=_NONE):
    """Gives a bfloat16 weight on the GPU whose products are often ones of few rows (a decode step's
    QKV, gate/up and head) a second copy in the order in which the matrix cores take it as an operand
    (``lib.tile_weight``): the kernels that keep the step's rows in registers then read 1 KB of
    consecutive memory per instruction, where rows of ``w`` itself put every lane on a line of its own
    (gate/up 20.7 -> 19.2 us, the head 118 -> 103 us alone at 8 rows). Costs the weight's size again.
    ``qkv``: the stacked q, k, v rows of an attention, ``(n_heads, n_kv, head_dim, rotated, adjacent)``."""
    if ("tiled" not in without and w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[0] % 16 == 0
            and w.is_contiguous()):
        w.tiled = K.tile_weight(w, qkv)
    return w


def can_hold_once(w, without=_NONE):
    """Whether a weight can be kept in the order of one of its copies alone (``lib.hold_once``): it carries a copy
    over whole steps of k, and the engine has no fast path switched off (a comparison wants both orders at hand;
    ``Engine(weight_copies="both")`` asks for exactly that). Every kernel that a step may take for such a weight
    reads the copies' orders: the embedding look-up, the products of few rows (through the copy whose strips they
    walk), the kernel of whole lines, the tiled product's store and add epilogues, the generic product."""
    # (a weight with packed strips of 8 only: steps of 9 to 64 rows must find the kernel of whole lines, which takes
    # it with K in slices; else they would fall back to the tiled product, which is right but slow for so few rows)
    strips_of_16 = getattr(w, "tiled", None) is not None and w.shape[0] % 16 == 0
    return not without and K.can_hold_once(w) and (strips_of_16 or K.wide_slices(w.shape[0], w.shape[1]) >= 2)


class StoredRows:
    """Rows ``lo .. hi`` of a matrix that a part keeps in another order than the stored one, under the name the
    model's file gives them: put together when somebody asks (``Engine.weights``)."""

    def __init__(self, part, attribute, lo, hi):
        self.part, self.attribute, self.lo, self.hi = part, attribute, lo, hi

    def stored(self):
        return K.stored_order(getattr(self.part, self.attribute))[self.lo:self.hi]


def stored(w):
    """What ``Engine.weights`` hands out for an entry of a model's weights: the tensor in the stored order."""
    return w.stored() if isinstance(w, StoredRows) else K.stored_order(w)


def for_gated(w, without=_NONE, alone=False):
    """The stacked gate and up rows of a feed-forward: the copy of ``for_few_rows`` where a product of few
    rows reads it (the kernel of whole lines, which takes the large ones, reads stored rows as well) or where the
    copy is to stand alone (``alone``: the caller may hold the weight once, and ``gated_alone`` says that it can)."""
    if gated_on_whole_lines(w, without) and not (alone and gated_alone(w, without)):
        return w
    return for_few_rows(w, without=without)


def gated_alone(w, without=_NONE):
    """Whether the stacked gate and up rows ``w`` (2N rows) can be kept in the operands' order alone: N a multiple
    of 16 (the up strips follow the gate strips), K in whole steps of 64, and every fast path switched on. Every
    kernel that takes a gated product reads that order (the kernel of whole lines 2 to 8% faster than stored rows:
    the weights then do not pass through shared memory)."""
    return (not without and w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous()
            and (w.shape[0] // 2) % 16 == 0 and w.shape[0] % 2 == 0 and w.shape[1] % 64 == 0 and w.numel() < 2 ** 30)


def gated_on_whole_lines(w, without=_NONE):
    """Whether the gated products of few rows over ``w`` (2N rows) run on the kernel that loads whole lines:
    where it has blocks enough for the chip, and 32-bit byte offsets reach all of ``w``."""
    return ("wide" not in without and "widefold" not in without and w.shape[0] // 2 >= 32 * 192
            and w.numel() < 2 ** 30)


def for_eight_rows(w, without=_NONE):
    """The same for a weight of a product into the residual stream (output and down projection): steps of
    at most 8 rows take it in strips of 8 weight rows with packed tiles where 16-row strips would leave CUs
    idle (``lib.skinny_strip_rows``, ``lib.tile_weight8``), everything else of few rows in strips of 16;
    the copy for those is left out where no step reads it (strips of 8 up to 8 rows, and a K so long that 9 to
    16 rows go to the kernel of whole lines)."""
    N, Kd = w.shape
    if K.skinny_strip_rows(8, N, Kd, EPI_ADD) == 16 or Kd <= 4096 or "wide" in without or "wide916" in without:
        for_few_rows(w, without=without)
    if ("tiled" not in without and w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[0] % 8 == 0
            and w.is_contiguous() and K.skinny_strip_rows(8, w.shape[0], w.shape[1], EPI_ADD) == 8):
        w.tiled8 = K.tile_weight8(w)
    return w


class Normed:
    """The RMSNorm of (rows of) the float residual stream, not computed yet.

    A norm hands this out instead of a tensor when the step is small enough for the
    product that follows to do the norm's work itself. The kernel that last wrote the rows
    left what that takes: the rows times this norm's weight in bfloat16 (``xg``), and the
    sum of squares of every row as partial sums; the product applies 1/rms to its sums.
    ``materialize`` runs the norm as a kernel of its own, for consumers that cannot."""

    def __init__(self, ctx, x, weight, eps, dtype, xg, ssq, n_partials, rows, name):
        self.ctx, self.x, self.weight, self.eps, self.dtype = ctx, x, weight, eps, dtype
        self.xg, self.ssq, self.n_partials, self.rows, self.name = xg, ssq, n_partials, rows, name
        self.shape = (x.shape[0] if rows is None else rows.numel(), x.shape[1])

    def materialize(self):
        out = self.ctx.buffer(self.name, self.shape, self.dtype)
        K.rmsnorm(self.x, self.weight, out, self.eps, self.rows)
        return out


def settle_residual(ctx, x):
    """A product of 17 to 64 rows into the residual stream may have left its sums as slices that the
    next norm adds up. Whoever else wants to READ the rows (adding to them is always fine) calls
    this first."""
    pending = getattr(ctx, "pending", None)
    if pending is not None and pending[0] == x.data_ptr():
        K.add_slices_rmsnorm(x, pending[1])
        ctx.pending = None


def residual_written(ctx, x, ssq=None, n_partials=0, xg=None, norm=None):
    """Every writer of the residual stream says so: what a folded norm would use (the partial sums
    of squares of the rows, and the rows times the weight of ``norm``) is the last writer's, or
    nothing."""
    if ctx is not None:
        ctx.ssq = (x.data_ptr(), ssq, n_partials, xg, norm) if ssq is not None and xg is not None else None


def _next_norm(ctx, N):
    """The norm that reads the residual rows next, if it is one whose work a product can take over:
    (its float weight, a buffer for the rows times that weight), else (None, None)."""
    norm = getattr(ctx, "next_norm", None)
    w = getattr(norm, "weight_f32", None)
    if norm is None or w is None or w.shape != (N,) or not getattr(norm, "folds", False):
        return None, None
    return norm, ctx.buffer("rows_times_norm_weight", (ctx.n_tokens, N), torch.bfloat16)


def row_chunks(M, ctx=None):
    """Steps of 66 to 128 rows are worked on in two pieces of 33 to 64 rows: the kernels for
    so few rows stream the weights at several times the rate of the tiled kernel, whose tiles of
    128 rows are too few for the chip at these sizes, and the pieces after the first find the
    weights in the memory-side cache. Only in a step that is replayed from a graph: elsewhere the host pays
    for every launch, and twice the launches cost more than the pieces gain (a prompt of 128 tokens, 1B
    layers: 2.83 ms in pieces, 2.22 ms tiled). None: no pieces."""
    if not 65 < M <= CHUNK_ROWS or (ctx is not None and not getattr(ctx, "replayed", False)):
        return None
    n = -(-M // 64)
    size = -(-M // n)
    return [(lo, min(M, lo + size)) for lo in range(0, M, size)]


def _linear_in_chunks(a, w, out, epilogue, ctx, chunks, bias=None, act="silu"):
    M, Kd = a.shape
    N = out.shape[1]
    if epilogue != EPI_ADD:
        for lo, hi in chunks:
            linear(a[lo:hi], w, out[lo:hi], epilogue, ctx, bias=bias, act=act)
        return
    slices = K.wide_slices(N, Kd) if bias is None else 1     # (a bias is added once: no slices of K with one)
    if slices < 2:
        for lo, hi in chunks:
            K.gemm_skinny(a[lo:hi], w, out[lo:hi], EPI_ADD, bias=bias)
        return residual_written(ctx, out)
    settle_residual(ctx, out)
    part = ctx.buffer(f"slices{slices}", (slices, M, N), torch.float32)
    for lo, hi in chunks:
        K.gemm_skinny_wide(a[lo:hi], w, part[:, lo:hi], EPI_STORE)
    residual_written(ctx, out)
    ctx.pending = (out.data_ptr(), part)


class _BF16_OUT:      # what the check of a product's output looks at
    dtype = torch.bfloat16


def packs_rows(ctx, h, w_first, w_second, x):
    """Whether a gated product of ``h`` and the product of its result into the residual rows ``x`` can hand
    the result over in the packed order (``lib.packed_rows``): a folded norm in front, at most 8 rows, the
    second product in strips of 8 weight rows. Every block of that product reads all of the step's rows;
    with a long K they are as many bytes as its weights, and in the packed order a CU's first-level
    cache takes them in a third of the time."""
    M = h.shape[0]
    F = w_second.shape[1]
    return (isinstance(h, Normed) and M <= 8 and not _off(ctx) & {"packed", "fused", "skinny"}
            and w_first.dtype == torch.bfloat16 and w_second.dtype == torch.bfloat16 and x.dtype == torch.float32
            and w_first.shape[0] == 2 * F and F % 8 == 0 and w_second.stride(0) % 8 == 0 and w_second.data_ptr() % 16 == 0
            and K.gemm_skinny_norm_fits(h.xg, w_first, _BF16_OUT, EPI_GATED)
            and K.skinny_strip_rows(M, x.shape[1], F, EPI_ADD) == 8)


def linear(a, w, out, epilogue=EPI_STORE, ctx=None, bias=None, act="silu", pack_out=False, a_packed=False):
    """out (=, +=, gated) a @ w.T. ``a`` may be a ``Normed``. With the add epilogue ``out`` is the
    residual stream. ``bias`` (float32, one per row of ``w``) is added to the sums before the
    epilogue's own rule; ``act`` is the gated epilogue's activation (``lib.ACTIVATIONS``).
    ``pack_out`` / ``a_packed``: ``out`` / ``a`` is a ``lib.packed_rows`` buffer (where ``packs_rows`` said so)."""
    disabled = _off(ctx if ctx is not None else getattr(a, "ctx", None))
    if pack_out:
        return K.gemm_skinny_norm(a.xg, a.ssq, a.n_partials, a.eps, w, out, epilogue, rows=a.rows, bias=bias, act=act,
                                  pack_out=True, whole_lines=_whole_lines(a, w, epilogue))
    if a_packed:
        M, N = out.shape
        if (epilogue == EPI_ADD and ctx is not None and getattr(ctx, "fuse", False) and N % 16 == 0
                and "fused" not in disabled and M == ctx.n_tokens <= FUSE_ROWS):
            norm, xg = _next_norm(ctx, N)
            if norm is not None:
                ssq = ctx.ssq_buffer(N // 8)
                K.gemm_skinny(a, w, out, epilogue, ssq_out=ssq, strip_rows=8, next_weight=norm.weight_f32, xg=xg, bias=bias,
                              a_packed=True)
                return residual_written(ctx, out, ssq, N // 8, xg, norm)
        K.gemm_skinny(a, w, out, epilogue, strip_rows=8, bias=bias, a_packed=True)
        if epilogue == EPI_ADD:
            residual_written(ctx, out)
        return
    if isinstance(a, Normed):
        if ("fused" not in disabled and w.dtype == torch.bfloat16 and K.gemm_skinny_norm_fits(a.xg, w, out, epilogue)
                and a.xg.shape[0] <= 64 and not _streams_rows_for_many_strips(out.shape[0], w, epilogue)
                and (_whole_lines(a, w, epilogue) or K.skinny_takes(w, out.shape[0], 16))):
            return K.gemm_skinny_norm(a.xg, a.ssq, a.n_partials, a.eps, w, out, epilogue, rows=a.rows, bias=bias, act=act,
                                      whole_lines=_whole_lines(a, w, epilogue))
        a = a.materialize()
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        chunks = row_chunks(a.shape[0], ctx)
        if (chunks and ctx is not None and getattr(ctx, "fuse", False) and not disabled & {"wide", "fused", "skinny"}
                and K.gemm_skinny_fits(a[:1], w, out[:1], epilogue)
                and not (epilogue == EPI_STORE and out.shape[1] >= 128 * 512)      # (the head: the tiled kernel)
                and (K.skinny_takes(w, 64, 16) or (epilogue == EPI_ADD and bias is None
                                                   and K.wide_slices(out.shape[1], a.shape[1]) >= 2))):
            return _linear_in_chunks(a, w, out, epilogue, ctx, chunks, bias, act)
        if (_streams_rows_for_many_strips(a.shape[0], w, epilogue) and "mfma" not in disabled
                and K.gemm_mfma_fits(a, w, out, epilogue)):
            return K.gemm_mfma(a, w, out, epilogue, bias=bias)
        if ("wide" not in disabled and (a.shape[0] > FUSE_ROWS or _long_k_of_9_to_16_rows(a, out, epilogue, bias, disabled))
                and K.gemm_skinny_wide_fits(a, w, out, epilogue) and _linear_wide(a, w, out, epilogue, ctx, bias, act)):
            return
        rows = K.skinny_strip_rows(a.shape[0], out.shape[1], a.shape[1], epilogue)
        if not K.skinny_takes(w, a.shape[0], rows):      # (held once: through the copy it has, if it has one for these rows)
            rows = 24 - rows if K.skinny_takes(w, a.shape[0], 24 - rows) and epilogue != EPI_GATED else 0
        if rows and "skinny" not in disabled and K.gemm_skinny_fits(a, w, out, epilogue):
            N = out.shape[1]
            if (epilogue == EPI_ADD and ctx is not None and getattr(ctx, "fuse", False) and N % 16 == 0
                    and "fused" not in disabled and out.shape[0] == ctx.n_tokens <= FUSE_ROWS):
                # the rows are complete after this product: leave what the norm that follows needs
                norm, xg = _next_norm(ctx, N)
                if norm is not None:
                    ssq = ctx.ssq_buffer(N // rows)
                    K.gemm_skinny(a, w, out, epilogue, ssq_out=ssq, strip_rows=rows, next_weight=norm.weight_f32, xg=xg,
                                  bias=bias)
                    return residual_written(ctx, out, ssq, N // rows, xg, norm)
            K.gemm_skinny(a, w, out, epilogue, strip_rows=rows, bias=bias, act=act)
            if epilogue == EPI_ADD:
                residual_written(ctx, out)
            return
        if "mfma" not in disabled and K.gemm_mfma_fits(a, w, out, epilogue):
            M, Kd = a.shape
            shape, slices = 0, 1
            if (epilogue == EPI_ADD and bias is None and ctx is not None and getattr(ctx, "fuse", False)
                    and "fused" not in disabled):
                shape, slices = K.mfma_plan(M, out.shape[1], Kd)
            if slices > 1:
                # the first slice adds into the rows, the norm that follows adds the others
                settle_residual(ctx, out)
                part = ctx.buffer(f"slices{slices - 1}", (slices - 1, M, out.shape[1]), torch.float32)
                K.gemm_mfma(a, w, out, epilogue, more_slices=part, shape=shape)
                residual_written(ctx, out)
                ctx.pending = (out.data_ptr(), part)
                return
            K.gemm_mfma(a, w, out, epilogue, bias=bias, act=act, shape=shape)
            if epilogue == EPI_ADD:
                residual_written(ctx, out)
            return
    K.gemm_generic(a, w, out, epilogue, bias=bias, act=act)
    if epilogue == EPI_ADD:
        residual_written(ctx, out)


def _long_k_of_9_to_16_rows(a, out, epilogue, bias, disabled=_NONE):
    """A product of 9 to 16 rows into the residual stream over a K too long for the kernel that keeps its rows
    in registers: strips of 8 weight rows leave half of every tile idle there, and the kernel of whole lines
    with K in slices is faster even with the norm kernel that then adds the slices."""
    return (epilogue == EPI_ADD and bias is None and 8 < a.shape[0] <= 16 and a.shape[1] > 4096
            and "wide916" not in disabled and out.dtype == torch.float32)


def _whole_lines(a, w, epilogue):
    """Whether a folded norm's gated product runs on the kernel that loads whole lines: where it has blocks
    enough for the chip, as for 17 to 64 rows."""
    return epilogue == EPI_GATED and a.rows is None and a.xg.shape[0] <= 16 and gated_on_whole_lines(w, _off(a.ctx))


def _streams_rows_for_many_strips(M, w, epilogue):
    """A head of more than 16 rows over a K beyond what the skinny kernel keeps in registers: that kernel
    would read the rows of ``a`` again for each of thousands of strips, and the tiled kernel, whose blocks
    share them, is the faster one (N = 128,256, K = 4,096: 32 rows 354 against 292 us, 64 rows 595 against
    273 us; K = 3,072: 32 rows 276 against 198 us)."""
    return (epilogue == EPI_STORE and w.shape[0] >= 128 * 512 and M > 16
            and not K.skinny_keeps_operands(M, w.shape[1]))


def _linear_wide(a, w, out, epilogue, ctx, bias=None, act="silu"):
    """Products of 17 to 64 rows where another kernel than the skinny one is faster. True when done."""
    disabled = _off(ctx)
    M, Kd = a.shape
    N = out.shape[1]
    if epilogue == EPI_GATED:
        if N < 32 * 192:          # too few blocks of two strip pairs for the chip
            return False
        K.gemm_skinny_wide(a, w, out, epilogue, bias=bias, act=act)
        return True
    if epilogue == EPI_STORE:
        # many columns (the head): the tiled kernel, whose blocks share their rows of a; where the weight has
        # a copy in the operands' order the skinny kernel is the faster one (64 rows: 131 against 152 us)
        if (N >= 128 * 512 and "mfma" not in disabled and getattr(w, "tiled", None) is None
                and K.gemm_mfma_fits(a, w, out, epilogue)):
            K.gemm_mfma(a, w, out, epilogue, bias=bias)
            return True
        return False
    if bias is not None:          # a bias is added once: no slices of K with one
        return False
    # into the residual stream: K in slices, added up by the norm that follows
    slices = K.wide_slices(N, Kd)
    if slices < 2 or ctx is None or not getattr(ctx, "fuse", False) or "fused" in disabled:
        return False
    settle_residual(ctx, out)
    part = ctx.buffer(f"slices{slices}", (slices, M, N), torch.float32)
    K.gemm_skinny_wide(a, w, part, EPI_STORE)
    residual_written(ctx, out)
    ctx.pending = (out.data_ptr(), part)
    return True


def _table_rows(ctx):
    """The block table's row of each token: what the context says, else the token's sequence number."""
    rows = getattr(ctx, "table_rows", None)
    return rows if rows is not None else ctx.seq_of_token


def _token_facts(ctx, block_table, cos, sin, page_size):
    """The page of each token's position and its rows of cos and sin, looked up once per step for all layers
    that share the block table and the rotation (``lib.token_facts``): in the QKV product of every layer they
    would be a second trip to memory behind the token's position. A step's context keeps them by the tables
    they were made from."""
    made = ctx.__dict__.setdefault("token_facts", {})
    key = (block_table.data_ptr(), cos.data_ptr() if cos is not None else 0, page_size)
    if key not in made:
        n = len(made)
        T = ctx.positions.numel()
        pages = ctx.buffer(f"token_pages{n}", (T,), torch.int32)
        rot = ctx.buffer(f"token_rot{n}", (T, 2 * cos.shape[1]), torch.float32) if cos is not None else None
        # a decode step's attention reads the tokens' own rows of the block table (row t: token t)
        tables = ctx.buffer(f"token_tables{n}", (T, block_table.shape[1]), torch.int32) if ctx.decode else None
        K.token_facts(ctx.positions, _table_rows(ctx), block_table, page_size, cos, sin, pages, rot, tables)
        made[key] = (pages, rot)
        if tables is not None:
            ctx.__dict__.setdefault("token_tables", {})[block_table.data_ptr()] = tables
    return made[key]


def qkv_project(ctx, h, w_qkv, w_q, rotary, k_cache, v_cache, block_table, n_heads, n_kv, head_dim, dtype, writes_kv,
                bias=None):
    """Queries, keys and values of the step's tokens: q rotated into a buffer whose rows start
    with the H*hs query columns (returned), k rotated and v into the cache. One kernel when
    ``h`` is a ``Normed`` and the shapes allow, else product and rotation apart (always apart with
    a ``bias``, float32 over the stacked q, k, v rows, which is added before the rotation)."""
    disabled = _off(ctx)
    T = h.shape[0]
    page = k_cache.shape[2]
    cos, sin = (rotary.cos, rotary.sin) if rotary is not None else (None, None)
    rot = rotary.rot_dim if rotary is not None else 0
    adjacent = rotary.adjacent if rotary is not None else False
    if (isinstance(h, Normed) and writes_kv and h.rows is None and "fused" not in disabled and bias is None
            and K.qkv_rope_cache_fits(h.xg, w_qkv, head_dim, rot)):
        q = ctx.buffer("q", (T, n_heads * head_dim), dtype)
        pages, rows_of_rotation = _token_facts(ctx, block_table, cos, sin, page)
        K.qkv_rope_cache(h.xg, h.ssq, h.n_partials, h.eps, w_qkv, q, ctx.positions, _table_rows(ctx),
                         block_table, cos, sin, k_cache, v_cache, n_heads, n_kv, head_dim, adjacent, page,
                         token_pages=pages, token_rot=rows_of_rotation)
        return q
    if isinstance(h, Normed):
        h = h.materialize()
    chunks = row_chunks(T, ctx) if getattr(ctx, "fuse", False) and "wide" not in disabled else None
    if (writes_kv and h.dtype == torch.bfloat16 and "fused" not in disabled and "skinny" not in disabled and bias is None
            and K.qkv_rope_cache_fits(h[:64], w_qkv, head_dim, rot) and (T <= 64 or chunks)):
        q = ctx.buffer("q", (T, n_heads * head_dim), dtype)
        for lo, hi in (chunks or [(0, T)]):
            K.qkv_rope_cache(h[lo:hi], None, 0, 0.0, w_qkv, q[lo:hi], ctx.positions[lo:hi], _table_rows(ctx)[lo:hi],
                             block_table, cos, sin, k_cache, v_cache, n_heads, n_kv, head_dim, adjacent, page)
        return q
    if writes_kv:
        qkv = ctx.buffer("qkv", (T, (n_heads + 2 * n_kv) * head_dim), dtype)
        linear(h, w_qkv, qkv, bias=bias)
    else:
        if w_q is None:
            raise ValueError("a layer that reads another entry's keys and values needs the query rows alone, which a "
                             "mixer that keeps its stacked rows in the operands' order only does not have")
        qkv = ctx.buffer("qkv", (T, n_heads * head_dim), dtype)
        linear(h, w_q, qkv, bias=None if bias is None else bias[:n_heads * head_dim])
    K.rope_cache_write(qkv, ctx.positions, _table_rows(ctx), block_table, cos, sin, k_cache, v_cache,
                       n_heads, n_kv, head_dim, rot, adjacent, page, write_kv=writes_kv)
    return qkv


def attention(ctx, q, k_cache, v_cache, block_table, out, n_heads, n_kv, head_dim, window, scale):
    page = k_cache.shape[2]          # keys are [page, kv head, position in page, head_dim]
    disabled = _off(ctx)
    if q.dtype == torch.bfloat16:
        if (ctx.decode and "attn_decode" not in disabled and K.has("gl3_attention_decode")
                and K.attention_decode_fits(head_dim, n_heads, n_kv, page)):
            T = q.shape[0]
            splits = K.decode_splits(T, n_heads, n_kv, ctx.kv_len_hint, head_dim)
            part_o = part_ml = None
            if splits > 1:
                part_o = ctx.buffer("attn_part_o", (T, n_heads, splits, head_dim), torch.float32)
                part_ml = ctx.buffer("attn_part_ml", (T, n_heads, splits, 2), torch.float32)
            own = getattr(ctx, "token_tables", {}).get(block_table.data_ptr())    # (made with the step's token facts)
            if own is not None:
                return K.attention_decode(q, k_cache, v_cache, ctx.positions, None, own, out, n_heads, n_kv, head_dim, page,
                                          window, scale, splits, part_o, part_ml)
            return K.attention_decode(q, k_cache, v_cache, ctx.positions, _table_rows(ctx), block_table, out, n_heads,
                                      n_kv, head_dim, page, window, scale, splits, part_o, part_ml)
        if (not ctx.decode and "attn_prefill" not in disabled and K.has("gl3_attention_prefill") and scale > 0
                and K.attention_prefill_fits(head_dim, n_heads, n_kv, page)):
            return K.attention_prefill(q, k_cache, v_cache, ctx.cu_seqlens, ctx.kv_before, block_table, out,
                                       ctx.max_q_len, n_heads, n_kv, head_dim, page, window, scale,
                                       seq_rows=getattr(ctx, "seq_rows", None))
    return K.attention_generic(q, k_cache, v_cache, ctx.positions, _table_rows(ctx), block_table, out, n_heads, n_kv,
                               head_dim, page, window, scale)

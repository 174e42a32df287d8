"""Each kernel alone against its plain reference, at sizes the engine's tests do not use."""
import math

import numpy as np
import pytest
import torch

import plain_llama as P
from cache_order import tile_keys, tile_values, untile_keys, untile_values
from gpullama3_java_amd.sampling import sample_host

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def K():
    from gpullama3_java_amd.csrc import lib
    return lib


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a)).to(DEV).to(dtype)


def rounded(a, dtype):
    """The values the kernel really sees after storage in ``dtype``."""
    return torch.as_tensor(np.asarray(a, np.float32)).to(TD[dtype]).float().numpy()


def tol(dtype, k=1):
    return {"float32": 2e-5, "bfloat16": 1e-2}[dtype]


# ------------------------------------------------------------------ embedding, norm
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed(dtype):
    rng = np.random.default_rng(0)
    table = rounded(rng.standard_normal((1000, 70)), dtype)
    ids = rng.integers(0, 1000, 37)
    out = torch.empty(37, 70, device=DEV)
    K().embed(dev(table, TD[dtype]), dev(ids, torch.int32), out)
    np.testing.assert_array_equal(out.cpu().numpy(), table[ids])
    # with the sums of squares and the rows times the next norm's weight, for a norm folded into a product
    nw = (1 + 0.2 * rng.standard_normal(70)).astype(np.float32)
    out2 = torch.empty(37, 70, device=DEV)
    ssq = torch.full((64,), -1.0, device=DEV)
    xg = torch.empty(37, 70, device=DEV, dtype=torch.bfloat16)
    K().embed(dev(table, TD[dtype]), dev(ids, torch.int32), out2, ssq, dev(nw), xg)
    assert torch.equal(out2, out)
    np.testing.assert_allclose(ssq[:37].cpu().numpy(), (table[ids].astype(np.float64) ** 2).sum(1), rtol=1e-5)
    assert torch.all(ssq[37:] == -1)
    assert torch.equal(xg, (dev(nw)[None, :] * out).to(torch.bfloat16))
    with pytest.raises(K().KernelError):
        K().embed(dev(table, TD[dtype]), dev(ids, torch.int32), out2, None, dev(nw), xg)


@pytest.mark.parametrize("d", [70, 2048, 5000])
@pytest.mark.parametrize("wdtype, odtype", [("float32", "float32"), ("bfloat16", "bfloat16"), ("float32", "bfloat16")])
def test_rmsnorm(d, wdtype, odtype):
    rng = np.random.default_rng(d)
    x = (rng.standard_normal((9, d)) * 3).astype(np.float32)
    w = rounded(1 + 0.2 * rng.standard_normal(d), wdtype)
    out = torch.empty(9, d, device=DEV, dtype=TD[odtype])
    K().rmsnorm(dev(x), dev(w, TD[wdtype]), out, 1e-6)
    ref = P.rmsnorm(x, w, 1e-6)
    np.testing.assert_allclose(out.float().cpu().numpy(), ref, rtol=1e-5 if odtype == "float32" else 5e-3, atol=1e-6)
    rows = np.array([7, 0, 7, 3])
    out2 = torch.empty(4, d, device=DEV, dtype=TD[odtype])
    K().rmsnorm(dev(x), dev(w, TD[wdtype]), out2, 1e-6, dev(rows, torch.int32))
    assert torch.equal(out2, out[torch.as_tensor(rows).to(DEV)])
    zero = torch.empty(1, d, device=DEV)
    K().rmsnorm(torch.zeros(1, d, device=DEV), dev(w), zero, 1e-5)
    assert torch.all(zero == 0)


# ------------------------------------------------------------------ generic product
@pytest.mark.parametrize("M, N, Kd", [(1, 130, 70), (37, 257, 129), (200, 64, 64), (3, 1000, 112)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gemm_generic_epilogues(M, N, Kd, dtype):
    rng = np.random.default_rng(M * N)
    a = rounded(rng.standard_normal((M, Kd)), dtype)
    w = rounded(rng.standard_normal((2 * N, Kd)) / math.sqrt(Kd), dtype)
    A, W = dev(a, TD[dtype]), dev(w, TD[dtype])
    lib = K()
    out = torch.empty(M, N, device=DEV, dtype=TD[dtype])
    lib.gemm_generic(A, W[:N], out, lib.EPI_STORE)
    ref = P.linear(a, w[:N])
    np.testing.assert_allclose(out.float().cpu().numpy(), ref, atol=tol(dtype) * np.abs(ref).max())
    logits = torch.empty(M, N, device=DEV)                         # float output from bfloat16 operands
    lib.gemm_generic(A, W[:N], logits, lib.EPI_STORE)
    np.testing.assert_allclose(logits.cpu().numpy(), ref, atol=2e-5 * np.abs(ref).max())
    res = rng.standard_normal((M, N)).astype(np.float32)
    x = dev(res)
    lib.gemm_generic(A, W[:N], x, lib.EPI_ADD)
    np.testing.assert_allclose(x.cpu().numpy(), res + ref, atol=2e-5 * np.abs(ref).max())
    gated = torch.empty(M, N, device=DEV, dtype=TD[dtype])
    lib.gemm_generic(A, W, gated, lib.EPI_GATED)
    refg = P.silu(P.linear(a, w[:N])) * P.linear(a, w[N:])
    np.testing.assert_allclose(gated.float().cpu().numpy(), refg, atol=tol(dtype) * max(np.abs(refg).max(), 1e-3))


def test_gemm_generic_rows_do_not_depend_on_their_company():
    rng = np.random.default_rng(3)
    a, w = dev(rng.standard_normal((130, 96))), dev(rng.standard_normal((77, 96)))
    lib = K()
    full = torch.empty(130, 77, device=DEV)
    lib.gemm_generic(a, w, full)
    one = torch.empty(1, 77, device=DEV)
    for r in (0, 63, 64, 129):
        lib.gemm_generic(a[r:r + 1], w, one)
        assert torch.equal(one[0], full[r])


def test_gemm_generic_mixed_storage_and_strides():
    rng = np.random.default_rng(4)
    a = rounded(rng.standard_normal((5, 40)), "bfloat16")
    w = rng.standard_normal((9, 40)).astype(np.float32)               # a matrix stored in 32-bit stays so
    lib = K()
    out = torch.empty(5, 9, device=DEV, dtype=torch.bfloat16)
    lib.gemm_generic(dev(a, torch.bfloat16), dev(w), out)
    np.testing.assert_allclose(out.float().cpu().numpy(), P.linear(a, w), atol=0.05)
    wide = torch.zeros(5, 30, device=DEV)                              # output is a view with a row stride
    lib.gemm_generic(dev(a), dev(w), wide[:, 3:12])
    np.testing.assert_allclose(wide[:, 3:12].cpu().numpy(), P.linear(a, w), atol=1e-4)
    assert torch.all(wide[:, :3] == 0) and torch.all(wide[:, 12:] == 0)
    with pytest.raises(lib.KernelError):
        lib.gemm_generic(dev(a), dev(w[:, :39]), wide[:, 3:12])


# ------------------------------------------------------------------ paged cache helpers
def paged(seqs_k, seqs_v, n_kv, hs, page, dtype, rng, n_pages=None):
    """Scatter per-sequence ``[len, n_kv, hs]`` keys and values into shuffled pages, in the order
    inside a page that the kernels use. ``untile_keys`` and ``untile_values`` give the plain order
    ``[page, kv head, position, hs]`` and ``[page, kv head, hs, position]`` back."""
    need = [-(-len(k) // page) for k in seqs_k]
    n_pages = n_pages or sum(need) + 3
    ids = rng.permutation(np.arange(1, n_pages))[:sum(need)].tolist()
    kc = torch.full((n_pages, n_kv, page, hs), 777.0, dtype=TD[dtype])        # garbage where nothing was written
    vc = torch.full((n_pages, n_kv, hs, page), -777.0, dtype=TD[dtype])       # values lie transposed in a page
    width = max(need)
    table = np.zeros((len(seqs_k), width), np.int32)
    for s, (k, v) in enumerate(zip(seqs_k, seqs_v)):
        for p in range(need[s]):
            pid = ids.pop()
            table[s, p] = pid
            chunk = slice(p * page, min(len(k), (p + 1) * page))
            n = chunk.stop - chunk.start
            kc[pid, :, :n] = torch.as_tensor(k[chunk]).to(TD[dtype]).transpose(0, 1)
            vc[pid, :, :, :n] = torch.as_tensor(v[chunk]).to(TD[dtype]).permute(1, 2, 0)
    # inside a page the kernels keep both in tiles; the tests think in the plain order of the shapes
    return tile_keys(kc).contiguous().to(DEV), tile_values(vc).contiguous().to(DEV), torch.as_tensor(table).to(DEV)


# ------------------------------------------------------------------ rotary + cache write
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("pairing", ["adjacent", "half"])
@pytest.mark.parametrize("H, Kh, hs", [(6, 2, 16), (5, 5, 48), (8, 1, 128)])
def test_rope_cache_write(dtype, pairing, H, Kh, hs):
    rng = np.random.default_rng(hs + H)
    page = 64
    lens_before, new = [70, 0, 129], [3, 40, 1]
    T = sum(new)
    qkv = rounded(rng.standard_normal((T, (H + 2 * Kh) * hs)), dtype)
    positions = np.concatenate([np.arange(b, b + n) for b, n in zip(lens_before, new)])
    seq_of = np.concatenate([[i] * n for i, n in enumerate(new)])
    total = [b + n for b, n in zip(lens_before, new)]
    zk = [np.zeros((t, Kh, hs), np.float32) for t in total]
    kc, vc, table = paged(zk, zk, Kh, hs, page, dtype, rng)
    before_k = kc.clone()
    cos, sin = P.rope_table(256, hs, 50000.0, dict(factor=4.0, low_freq_factor=1.0, high_freq_factor=2.0,
                                                   original_max_position_embeddings=64))
    buf = dev(qkv, TD[dtype])
    K().rope_cache_write(buf, dev(positions, torch.int32), dev(seq_of, torch.int32), table, dev(cos), dev(sin),
                         kc, vc, H, Kh, hs, hs, pairing == "adjacent", page)
    q = qkv[:, :H * hs].reshape(T, H, hs)
    k = qkv[:, H * hs:(H + Kh) * hs].reshape(T, Kh, hs)
    v = qkv[:, (H + Kh) * hs:].reshape(T, Kh, hs)
    qr = P.rope_rotate(q, positions, cos, sin, pairing)
    kr = P.rope_rotate(k, positions, cos, sin, pairing)
    out = buf.float().cpu().numpy()
    t = tol(dtype)
    np.testing.assert_allclose(out[:, :H * hs].reshape(T, H, hs), qr, atol=t * 4)
    np.testing.assert_array_equal(out[:, H * hs:], qkv[:, H * hs:])           # k and v in the buffer are left alone
    kcpu, vcpu, tab = untile_keys(kc).float().cpu().numpy(), untile_values(vc).float().cpu().numpy(), table.cpu().numpy()
    touched = np.zeros(kc.shape[0], bool)
    for i in range(T):
        pid = tab[seq_of[i], positions[i] // page]
        touched[pid] = True
        np.testing.assert_allclose(kcpu[pid, :, positions[i] % page], kr[i], atol=t * 4)
        np.testing.assert_array_equal(vcpu[pid, :, :, positions[i] % page], v[i])  # values are copied, never rotated
    # nothing else in the cache moved
    mask = torch.ones_like(kc, dtype=torch.bool)
    for i in range(T):
        mask[tab[seq_of[i], positions[i] // page], :, positions[i] % page] = False
    assert torch.equal(untile_keys(kc)[mask], untile_keys(before_k)[mask])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("pairing", ["adjacent", "half"])
def test_rope_of_a_part_of_the_head_and_of_queries_only(dtype, pairing):
    """Elements beyond the rotated part pass through, into the cache too; without the cache write a
    row holds queries only."""
    rng = np.random.default_rng(3)
    H, Kh, hs, rot, page = 3, 2, 64, 32, 64
    positions = np.array([5, 70, 0, 64, 127])
    T = len(positions)
    seq_of = np.array([0, 1, 2, 3, 3])
    zk = [np.zeros((6, Kh, hs), np.float32), np.zeros((71, Kh, hs), np.float32), np.zeros((1, Kh, hs), np.float32),
          np.zeros((128, Kh, hs), np.float32)]
    kc, vc, table = paged(zk, zk, Kh, hs, page, dtype, rng)
    cos, sin = P.rope_table(256, rot, 10000.0)
    qkv = rounded(rng.standard_normal((T, (H + 2 * Kh) * hs)), dtype)

    def rotated(x):                                                          # [T, heads, hs]
        out = x.copy()
        out[..., :rot] = P.rope_rotate(x[..., :rot], positions, cos, sin, pairing)
        return out
    buf = dev(qkv, TD[dtype])
    K().rope_cache_write(buf, dev(positions, torch.int32), dev(seq_of, torch.int32), table, dev(cos), dev(sin),
                         kc, vc, H, Kh, hs, rot, pairing == "adjacent", page)
    t = tol(dtype) * 4
    np.testing.assert_allclose(buf.float().cpu().numpy()[:, :H * hs].reshape(T, H, hs),
                               rotated(qkv[:, :H * hs].reshape(T, H, hs)), atol=t)
    kr = rotated(qkv[:, H * hs:(H + Kh) * hs].reshape(T, Kh, hs))
    kcpu, vcpu, tab = untile_keys(kc).float().cpu().numpy(), untile_values(vc).float().cpu().numpy(), table.cpu().numpy()
    for i in range(T):
        pid = tab[seq_of[i], positions[i] // page]
        np.testing.assert_allclose(kcpu[pid, :, positions[i] % page], kr[i], atol=t)
        np.testing.assert_array_equal(vcpu[pid, :, :, positions[i] % page], qkv[i, (H + Kh) * hs:].reshape(Kh, hs))
    q_only = dev(np.ascontiguousarray(qkv[:, :H * hs]), TD[dtype])
    k_before = kc.clone()
    K().rope_cache_write(q_only, dev(positions, torch.int32), dev(seq_of, torch.int32), table, dev(cos), dev(sin),
                         kc, vc, H, Kh, hs, rot, pairing == "adjacent", page, write_kv=False)
    np.testing.assert_allclose(q_only.float().cpu().numpy().reshape(T, H, hs),
                               rotated(qkv[:, :H * hs].reshape(T, H, hs)), atol=t)
    assert torch.equal(kc, k_before)


def test_rope_position_zero_and_no_table():
    rng = np.random.default_rng(1)
    qkv = rng.standard_normal((2, 4 * 16)).astype(np.float32)
    cos, sin = P.rope_table(8, 16, 10000.0)
    kc = torch.zeros(3, 1, 64, 16, device=DEV); vc = torch.zeros(3, 1, 16, 64, device=DEV)
    table = dev(np.array([[1], [2]]), torch.int32)
    for cs in ((dev(cos), dev(sin)), (None, None)):
        buf = dev(qkv)
        K().rope_cache_write(buf, dev([0, 0], torch.int32), dev([0, 1], torch.int32), table, cs[0], cs[1], kc, vc,
                             2, 1, 16, 16 if cs[0] is not None else 0, True, 64)
        np.testing.assert_array_equal(buf.cpu().numpy(), qkv)
        np.testing.assert_array_equal(untile_keys(kc)[1, 0, 0].cpu().numpy(), qkv[0, 32:48])


# ------------------------------------------------------------------ attention
def attention_case(rng, H, Kh, hs, lens_before, new, dtype, scale_hot=None):
    seqs_k, seqs_v, qs = [], [], []
    for b, n in zip(lens_before, new):
        seqs_k.append(rounded(rng.standard_normal((b + n, Kh, hs)), dtype))
        seqs_v.append(rounded(rng.standard_normal((b + n, Kh, hs)), dtype))
        qs.append(rounded(rng.standard_normal((b + n, H, hs)), dtype))
    return seqs_k, seqs_v, qs


def run_attention(fn, seqs_k, seqs_v, qs, lens_before, new, H, Kh, hs, dtype, rng, window=None, page=64):
    kc, vc, table = paged(seqs_k, seqs_v, Kh, hs, page, dtype, rng)
    positions = np.concatenate([np.arange(b, b + n) for b, n in zip(lens_before, new)])
    seq_of = np.concatenate([[i] * n for i, n in enumerate(new)])
    q = np.concatenate([qq[b:b + n] for qq, b, n in zip(qs, lens_before, new)]).reshape(len(positions), H * hs)
    wide = torch.zeros(len(positions), H * hs + 2 * Kh * hs, device=DEV, dtype=TD[dtype])   # q sits in a wider row
    wide[:, :H * hs] = dev(q, TD[dtype])
    out = torch.empty(len(positions), H * hs, device=DEV, dtype=TD[dtype])
    fn(wide, kc, vc, dev(positions, torch.int32), dev(seq_of, torch.int32), table, out, H, Kh, hs, page, window,
       1.0 / math.sqrt(hs))
    ref = np.concatenate([P.attention(qq, k, v, window=window)[b:b + n]
                          for qq, k, v, b, n in zip(qs, seqs_k, seqs_v, lens_before, new)])
    return out.float().cpu().numpy().reshape(-1, H, hs), ref


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, Kh, hs", [(6, 2, 16), (5, 5, 48), (8, 1, 128), (2, 1, 256), (4, 2, 80)])
def test_attention_generic(dtype, H, Kh, hs):
    rng = np.random.default_rng(H * hs)
    lens_before, new = [0, 70, 130, 5], [33, 1, 2, 1]          # a prompt, decodes at page edges, a short one
    sk, sv, qs = attention_case(rng, H, Kh, hs, lens_before, new, dtype)
    got, ref = run_attention(K().attention_generic, sk, sv, qs, lens_before, new, H, Kh, hs, dtype, rng)
    np.testing.assert_allclose(got, ref, atol=tol(dtype) * np.abs(ref).max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_generic_far_key_and_window_edge(dtype):
    """One far key among hundreds carries the whole weight; with a window the key just
    inside it counts and the key just outside does not."""
    rng = np.random.default_rng(9)
    H, Kh, hs, n = 4, 2, 32, 700
    k = rng.standard_normal((n, Kh, hs)).astype(np.float32) * 0.1
    v = rng.standard_normal((n, Kh, hs)).astype(np.float32)
    q = rng.standard_normal((n, H, hs)).astype(np.float32) * 0.1
    far = 13
    k[far, 1] = 0; k[far, 1, 5] = 30.0                                      # stands out for kv head 1 only
    q[n - 1, 2] = 0; q[n - 1, 2, 5] = 30.0                                  # head 2 -> kv head 1
    q[n - 1, 0] = 0; q[n - 1, 0, 5] = 30.0                                  # head 0 -> kv head 0: no hot key there
    k, v, q = (rounded(a, dtype) for a in (k, v, q))
    got, ref = run_attention(K().attention_generic, [k], [v], [q], [n - 1], [1], H, Kh, hs, dtype, rng)
    np.testing.assert_allclose(got, ref, atol=tol(dtype) * np.abs(ref).max())
    np.testing.assert_allclose(got[0, 2], v[far, 1], atol=tol(dtype) * 4)   # the far value, nothing else
    assert np.abs(got[0, 0] - v[far, 0]).max() > 0.3
    # window: the query at n-1 sees keys n-w .. n-1
    w = 100
    for hot, inside in ((n - w, True), (n - w - 1, False)):
        k2 = k.copy(); k2[far, 1] = 0.0; k2[hot, 1] = 0; k2[hot, 1, 5] = 30.0
        k2 = rounded(k2, dtype)
        got, ref = run_attention(K().attention_generic, [k2], [v], [q], [n - 1], [1], H, Kh, hs, dtype, rng, window=w)
        np.testing.assert_allclose(got, ref, atol=tol(dtype) * np.abs(ref).max())
        assert (np.abs(got[0, 2] - v[hot, 1]).max() < tol(dtype) * 4) == inside


def test_attention_generic_is_the_same_for_every_cut():
    rng = np.random.default_rng(11)
    H, Kh, hs, n = 4, 2, 48, 150
    sk, sv, qs = attention_case(rng, H, Kh, hs, [0], [n], "float32")
    whole, _ = run_attention(K().attention_generic, sk, sv, qs, [0], [n], H, Kh, hs, "float32", rng)
    for p in (0, 63, 64, 149):
        one, _ = run_attention(K().attention_generic, sk, sv, qs, [p], [1], H, Kh, hs, "float32", rng)
        np.testing.assert_array_equal(one[0], whole[p])


# ------------------------------------------------------------------ sampling
def check_draw(logits, temperature, top_p, u, tok):
    """The drawn token is the twin's, or u sits within rounding of the edge between them."""
    want = sample_host(logits, temperature, top_p, u)
    if tok == want:
        return
    for du in (-1e-6, 1e-6):
        if sample_host(logits, temperature, top_p, min(max(u + du, 0.0), 0.99999994)) == tok:
            return
    for dp in (-1e-6, 1e-6):
        if 0 < top_p < 1 and sample_host(logits, temperature, top_p + dp, u) == tok:
            return
    raise AssertionError(f"T={temperature} p={top_p} u={u}: kernel {tok}, twin {want}")


@pytest.mark.parametrize("V", [2, 50, 1000, 5000, 128256])
def test_sample_kernel(V):
    rng = np.random.default_rng(V)
    R = 24
    logits = (rng.standard_normal((R, V)) * rng.uniform(0.3, 4, (R, 1))).astype(np.float32)
    logits[3, : min(V, 7)] = logits[3].max() + 1.0                        # ties at the top
    temps = np.array([0, 0, 0.8, 1.0, 1.0, 0.3, 2.0, 1.0] * 3, np.float32)
    tops = np.array([0.95, 1.0, 0.95, 1.0, 0.0, 0.5, 0.9, 1e-6] * 3, np.float32)
    us = rng.random(R).astype(np.float32)
    us[4] = 0.0; us[6] = np.float32(0.99999994)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    K().sample(dev(logits), torch.empty(K().sample_work_size(R, V), device=DEV), dev(temps), dev(tops), dev(us), out)
    for r, tok in enumerate(out.tolist()):
        assert 0 <= tok < V
        check_draw(logits[r], float(temps[r]), float(tops[r]), float(us[r]), tok)
    assert out[3].item() == 0 if temps[3] == 0 else True


def test_sample_kernel_nucleus_from_the_short_list_and_from_the_whole_row():
    """A peaked row's nucleus lies among the few probabilities of 2^-13 or more, which the kernel
    gathers; a flat row's does not. Both must give the twin's token, with equal probabilities spread
    over the row, at the list's capacity and just beyond it."""
    rng = np.random.default_rng(8)
    V = 128256
    rows, temps, tops = [], [], []
    peaked = (rng.standard_normal(V) * 3).astype(np.float32)
    hot = rng.choice(V, 9, replace=False)
    peaked[hot] = peaked.max() + 2.0                                       # nine equal ones on top, anywhere in the row
    for tp in (0.3, 0.9, 0.999):
        rows.append(peaked); temps.append(0.5); tops.append(tp)
    flat = (rng.standard_normal(V) * 0.5).astype(np.float32)               # no probability reaches 2^-13
    rows.append(flat); temps.append(1.0); tops.append(0.9)
    # the list full, one more than it holds, few, and as many as the choosing block has threads, and one more
    for n_equal in (8192, 8193, 100, 1024, 1025):
        r = np.full(V, -np.inf, np.float32)
        r[rng.choice(V, n_equal, replace=False)] = 1.5
        rows.append(r); temps.append(1.0); tops.append(0.7)
    mixed = flat.copy()
    mixed[hot] += 9.0                                                       # most of the mass in nine, a long flat tail
    for tp in (0.5, 0.99):
        rows.append(mixed); temps.append(1.0); tops.append(tp)
    logits = np.stack(rows)
    R = len(rows)
    lib = K()
    for trial in range(6):
        us = rng.random(R).astype(np.float32)
        if trial == 0:
            us[:] = 0.0
        if trial == 1:
            us[:] = np.float32(0.99999994)
        out = torch.empty(R, dtype=torch.int32, device=DEV)
        lib.sample(dev(logits), torch.empty(lib.sample_work_size(R, V), device=DEV), dev(np.array(temps, np.float32)),
                   dev(np.array(tops, np.float32)), dev(us), out)
        for r, tok in enumerate(out.tolist()):
            check_draw(logits[r], temps[r], tops[r], float(us[r]), tok)


def test_sample_kernel_frequencies_and_rules():
    rng = np.random.default_rng(5)
    V, R = 12, 4000
    row = rng.standard_normal(V).astype(np.float32) * 1.5
    logits = np.tile(row, (R, 1))
    us = rng.random(R).astype(np.float32)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    lib = K()
    work = torch.empty(lib.sample_work_size(R, V), device=DEV)
    lib.sample(dev(logits), work, dev(np.full(R, 1.0)), dev(np.full(R, 1.0)), dev(us), out)
    p = P.probabilities(row, 1.0)
    counts = np.bincount(out.cpu().numpy(), minlength=V)
    assert np.sum((counts - R * p) ** 2 / (R * p)) < 40                 # 11 degrees of freedom
    lib.sample(dev(logits), work, dev(np.full(R, 1.0)), dev(np.full(R, 0.6)), dev(us), out)
    kept, _ = P.top_p_set(p, 0.6)
    assert set(out.cpu().numpy().tolist()) == set(kept)                 # the smallest prefix, all of it, only it
    lib.sample(dev(logits), work, dev(np.zeros(R)), dev(np.full(R, 0.6)), dev(us), out)
    assert torch.all(out == int(np.argmax(row)))
    lib.sample(dev(logits), work, dev(np.full(R, 1e-3)), dev(np.full(R, 1.0)), dev(us), out)
    assert torch.all(out == int(np.argmax(row)))                        # T -> 0+ is greedy


# ------------------------------------------------------------------ bfloat16 product for few rows (matrix cores)
@pytest.mark.parametrize("M", [1, 8, 17, 64])
# (the last case has strips enough for the blocks of four waves that very wide products take)
@pytest.mark.parametrize("N, Kd", [(2048, 2048), (130, 64), (48, 40), (3000, 512), (256, 8192), (33000, 136)])
def test_gemm_skinny(M, N, Kd):
    rng = np.random.default_rng(M + N)
    a = rounded(rng.standard_normal((M, Kd)), "bfloat16")
    w = rounded(rng.standard_normal((2 * N, Kd)) / math.sqrt(Kd), "bfloat16")
    A, W = dev(a, torch.bfloat16), dev(w, torch.bfloat16)
    lib = K()
    ref = P.linear(a, w[:N])
    scale = np.abs(ref).max()
    for waves in (0, 4, 8, 16):
        out = torch.zeros(M, N, device=DEV)
        lib.gemm_skinny(A, W[:N], out, lib.EPI_STORE, waves=waves)
        np.testing.assert_allclose(out.cpu().numpy(), ref, atol=2e-5 * scale * math.sqrt(Kd / 64), err_msg=f"waves {waves}")
        again = torch.zeros(M, N, device=DEV)
        lib.gemm_skinny(A, W[:N], again, lib.EPI_STORE, waves=waves)       # one order of summation: same bits
        assert torch.equal(out, again)
    ob = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
    lib.gemm_skinny(A, W[:N], ob)
    np.testing.assert_allclose(ob.float().cpu().numpy(), ref, atol=1e-2 * scale)
    res = rng.standard_normal((M, N)).astype(np.float32)
    x = dev(res)
    lib.gemm_skinny(A, W[:N], x, lib.EPI_ADD)
    np.testing.assert_allclose(x.cpu().numpy(), res + ref, atol=2e-5 * scale * math.sqrt(Kd / 64) + 1e-6)
    if M <= 16:                                                              # strips of 8 rows of w
        x8 = dev(res)
        ssq = torch.full((-(-N // 8), 64), -1.0, device=DEV) if N % 16 == 0 else None
        lib.gemm_skinny(A, W[:N], x8, lib.EPI_ADD, ssq_out=ssq, strip_rows=8)
        np.testing.assert_allclose(x8.cpu().numpy(), res + ref, atol=2e-5 * scale * math.sqrt(Kd / 64) + 1e-6)
        if ssq is not None:
            want = (x8.cpu().numpy().astype(np.float64) ** 2).reshape(M, N // 8, 8).sum(-1).T
            np.testing.assert_allclose(ssq[:, :M].cpu().numpy(), want, rtol=1e-5)
            assert torch.all(ssq[:, M:] == -1)
        o8 = torch.full((M, N + 2), -1.0, device=DEV)
        lib.gemm_skinny(A, W[:N], o8[:, :N], lib.EPI_STORE, strip_rows=8)
        np.testing.assert_allclose(o8[:, :N].cpu().numpy(), ref, atol=2e-5 * scale * math.sqrt(Kd / 64))
        assert torch.all(o8[:, N:] == -1)
    refg = P.silu(P.linear(a, w[:N])) * P.linear(a, w[N:])
    for waves in (0, 8):
        g_ = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
        lib.gemm_skinny(A, W, g_, lib.EPI_GATED, waves=waves)
        np.testing.assert_allclose(g_.float().cpu().numpy(), refg, atol=1e-2 * max(np.abs(refg).max(), 1e-3))


def test_gemm_skinny_refuses_what_it_cannot_do():
    lib = K()
    a = torch.zeros(65, 64, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(32, 64, device=DEV, dtype=torch.bfloat16)
    assert not lib.gemm_skinny_fits(a, w, torch.zeros(65, 32, device=DEV), lib.EPI_STORE)
    with pytest.raises(lib.KernelError, match="1..64"):
        lib.gemm_skinny(a, w, torch.zeros(65, 32, device=DEV))
    a2 = torch.zeros(4, 36, device=DEV, dtype=torch.bfloat16)
    assert not lib.gemm_skinny_fits(a2, w[:, :36], torch.zeros(4, 32, device=DEV), lib.EPI_STORE)   # K % 8


# ------------------------------------------------------------------ bfloat16 attention of a decode step
def decode_fn(splits):
    lib = K()

    def fn(q, kc, vc, positions, seq_of, table, out, H, Kh, hs, page, window, scale):
        T = q.shape[0]
        po = torch.empty(T, H, splits, hs, device=DEV) if splits > 1 else None
        pm = torch.empty(T, H, splits, 2, device=DEV) if splits > 1 else None
        lib.attention_decode(q, kc, vc, positions, seq_of, table, out, H, Kh, hs, page, window, scale, splits, po, pm)
    return fn


@pytest.mark.parametrize("splits", [1, 3, 8])
@pytest.mark.parametrize("H, Kh, hs", [(32, 8, 64), (6, 2, 32), (5, 5, 96), (8, 1, 128), (40, 2, 64)])
def test_attention_decode(H, Kh, hs, splits):
    rng = np.random.default_rng(H * hs + splits)
    lens_before, new = [0, 31, 32, 63, 64, 200, 511, 700], [1] * 8
    sk, sv, qs = attention_case(rng, H, Kh, hs, lens_before, new, "bfloat16")
    got, ref = run_attention(decode_fn(splits), sk, sv, qs, lens_before, new, H, Kh, hs, "bfloat16", rng)
    np.testing.assert_allclose(got, ref, atol=1e-2 * np.abs(ref).max())
    # pages of 32 positions (a chunk a page) and of 96 (no power of two: a chunk's page by division)
    for page in (32, 96):
        got, ref = run_attention(decode_fn(splits), sk, sv, qs, lens_before, new, H, Kh, hs, "bfloat16", rng, page=page)
        np.testing.assert_allclose(got, ref, atol=1e-2 * np.abs(ref).max(), err_msg=f"pages of {page}")


@pytest.mark.parametrize("hs", [96, 128])
def test_attention_decode_more_blocks_than_cus_and_many_splits(hs):
    """More (token, kv head) pairs than CUs (the blocks then have four waves, not eight), and more splits than
    chunks, so that most splits are empty and the merge reads more than a lane a split."""
    rng = np.random.default_rng(hs)
    H, Kh = 8, 4
    lens_before = [int(n) for n in rng.integers(0, 300, 70)]
    new = [1] * 70
    sk, sv, qs = attention_case(rng, H, Kh, hs, lens_before, new, "bfloat16")
    got, ref = run_attention(decode_fn(1), sk, sv, qs, lens_before, new, H, Kh, hs, "bfloat16", rng)
    np.testing.assert_allclose(got, ref, atol=1e-2 * np.abs(ref).max())
    lens_before, new = [5, 700, 2500], [1] * 3
    sk, sv, qs = attention_case(rng, H, Kh, hs, lens_before, new, "bfloat16")
    for splits in (70, 200):
        got, ref = run_attention(decode_fn(splits), sk, sv, qs, lens_before, new, H, Kh, hs, "bfloat16", rng)
        np.testing.assert_allclose(got, ref, atol=1e-2 * np.abs(ref).max())


@pytest.mark.parametrize("hs, far", [(64, 13), (128, 13), (128, 170), (96, 235)])
@pytest.mark.parametrize("splits", [1, 4, 40])
def test_attention_decode_far_key_and_window_edge(splits, hs, far):
    """One key among hundreds carries the weight: in the first wave's chunk, and (heads over 64) in a chunk of
    the upper waves, whose sums reach the result through the lower waves."""
    rng = np.random.default_rng(19)
    H, Kh, n = 4, 2, 700
    k = rng.standard_normal((n, Kh, hs)).astype(np.float32) * 0.1
    v = rng.standard_normal((n, Kh, hs)).astype(np.float32)
    q = rng.standard_normal((n, H, hs)).astype(np.float32) * 0.1
    k[far, 1] = 0; k[far, 1, 5] = 30.0
    q[n - 1, 2] = 0; q[n - 1, 2, 5] = 30.0
    q[n - 1, 0] = 0; q[n - 1, 0, 5] = 30.0
    k, v, q = (rounded(a, "bfloat16") for a in (k, v, q))
    got, ref = run_attention(decode_fn(splits), [k], [v], [q], [n - 1], [1], H, Kh, hs, "bfloat16", rng)
    np.testing.assert_allclose(got, ref, atol=1e-2 * np.abs(ref).max())
    np.testing.assert_allclose(got[0, 2], v[far, 1], atol=4e-2)
    assert np.abs(got[0, 0] - v[far, 0]).max() > 0.3
    w = 100
    for hot, inside in ((n - w, True), (n - w - 1, False)):
        k2 = k.copy(); k2[far, 1] = 0.0; k2[hot, 1] = 0; k2[hot, 1, 5] = 30.0
        k2 = rounded(k2, "bfloat16")
        got, ref = run_attention(decode_fn(splits), [k2], [v], [q], [n - 1], [1], H, Kh, hs, "bfloat16", rng, window=w)
        np.testing.assert_allclose(got, ref, atol=1e-2 * np.abs(ref).max())
        assert (np.abs(got[0, 2] - v[hot, 1]).max() < 4e-2) == inside


# ------------------------------------------------------------------ bfloat16 product for many rows (matrix cores)
# the last case is large enough for the 256 x 256 tiles, with edges in both directions
@pytest.mark.parametrize("M, N, Kd", [(65, 130, 64), (128, 128, 64), (200, 257, 136), (300, 64, 2048), (1000, 1000, 112),
                                      (4100, 8200, 72)])
def test_gemm_mfma(M, N, Kd):
    rng = np.random.default_rng(M + N + Kd)
    a = rounded(rng.standard_normal((M, Kd)), "bfloat16")
    w = rounded(rng.standard_normal((2 * N, Kd)) / math.sqrt(Kd), "bfloat16")
    A, W = dev(a, torch.bfloat16), dev(w, torch.bfloat16)
    lib = K()
    ref = P.linear(a, w[:N])
    scale = np.abs(ref).max()
    out = torch.zeros(M, N, device=DEV)
    lib.gemm_mfma(A, W[:N], out)
    np.testing.assert_allclose(out.cpu().numpy(), ref, atol=2e-5 * scale * math.sqrt(Kd / 64))
    ob = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
    lib.gemm_mfma(A, W[:N], ob)
    np.testing.assert_allclose(ob.float().cpu().numpy(), ref, atol=1e-2 * scale)
    res = rng.standard_normal((M, N)).astype(np.float32)
    x = dev(res)
    lib.gemm_mfma(A, W[:N], x, lib.EPI_ADD)
    np.testing.assert_allclose(x.cpu().numpy(), res + ref, atol=2e-5 * scale * math.sqrt(Kd / 64) + 1e-6)
    refg = P.silu(P.linear(a, w[:N])) * P.linear(a, w[N:])
    g_ = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
    lib.gemm_mfma(A, W, g_, lib.EPI_GATED)
    np.testing.assert_allclose(g_.float().cpu().numpy(), refg, atol=1e-2 * max(np.abs(refg).max(), 1e-3))
    if Kd > 64:                                                          # K in slices: the first adds, the others are stored
        for extra in [e for e in (1, 2) if e + 1 <= -(-Kd // 64)]:
            x2 = dev(res)
            part = torch.full((extra, M, N), 7.0, device=DEV)
            lib.gemm_mfma(A, W[:N], x2, lib.EPI_ADD, more_slices=part)
            per = -(-(-(-Kd // 64)) // (extra + 1)) * 64
            np.testing.assert_allclose(x2.cpu().numpy(), res + P.linear(a[:, :per], w[:N, :per]),
                                       atol=2e-5 * scale * math.sqrt(Kd / 64) + 1e-6)
            np.testing.assert_allclose((x2 + part.sum(0)).cpu().numpy(), res + ref,
                                       atol=2e-5 * scale * math.sqrt(Kd / 64) + 1e-6, err_msg=f"{extra + 1} slices")
    wide = torch.zeros(M, N + 24, device=DEV, dtype=torch.bfloat16)      # a view with a row stride as output
    lib.gemm_mfma(A, W[:N], wide[:, 8:8 + N])
    assert torch.equal(wide[:, 8:8 + N], ob) and torch.all(wide[:, :8] == 0) and torch.all(wide[:, 8 + N:] == 0)


# ------------------------------------------------------------------ bfloat16 attention of a prefill step
WIDE_FROM = {"64 queries a block": 1 << 30, "128 queries a block": 1}


def prefill_fn(lens_before, new, kernel, shuffled_rows=False):
    lib = K()

    def fn(q, kc, vc, positions, seq_of, table, out, H, Kh, hs, page, window, scale):
        cu = dev(np.concatenate([[0], np.cumsum(new)]), torch.int32)
        seq_rows = None
        if shuffled_rows:
            # the table's rows in another order, with rows of the sink page between them: sequence b reads row seq_rows[b]
            B = table.shape[0]
            order = np.random.default_rng(B).permutation(2 * B)[:B]
            big = torch.zeros((2 * B, table.shape[1]), dtype=torch.int32, device=table.device)
            big[torch.as_tensor(order, device=table.device)] = table
            table, seq_rows = big, dev(order, torch.int32)
        lib.attention_prefill(q, kc, vc, cu, dev(lens_before, torch.int32), table, out, max(new), H, Kh, hs, page,
                              window, scale, seq_rows=seq_rows, wide_from=WIDE_FROM[kernel])
    return fn


@pytest.fixture(params=["64 queries a block", "128 queries a block"])
def prefill_kernel(request):
    """Both kernels of the prefill attention on the same inputs, whatever the step's length."""
    return request.param


@pytest.mark.parametrize("H, Kh, hs", [(32, 8, 64), (6, 2, 32), (5, 5, 96), (8, 1, 128), (12, 2, 64), (3, 1, 128)])
def test_attention_prefill(H, Kh, hs, prefill_kernel):
    rng = np.random.default_rng(H * hs)
    lens_before, new = [0, 70, 0, 130, 5], [33, 1, 200, 17, 64]      # prompts, chunks after a prefix, one token
    sk, sv, qs = attention_case(rng, H, Kh, hs, lens_before, new, "bfloat16")
    got, ref = run_attention(prefill_fn(lens_before, new, prefill_kernel), sk, sv, qs, lens_before, new, H, Kh, hs, "bfloat16", rng)
    np.testing.assert_allclose(got, ref, atol=1e-2 * np.abs(ref).max())
    got, ref = run_attention(prefill_fn(lens_before, new, prefill_kernel, shuffled_rows=True), sk, sv, qs, lens_before, new, H, Kh, hs,
                             "bfloat16", rng)
    np.testing.assert_allclose(got, ref, atol=1e-2 * np.abs(ref).max(), err_msg="table rows named by seq_rows")
    # pages of 32 and of 96 positions: chunks of 32 keys, several pages or a part of one to a chunk's page
    for page in (32, 96):
        got, ref = run_attention(prefill_fn(lens_before, new, prefill_kernel), sk, sv, qs, lens_before, new, H, Kh, hs, "bfloat16",
                                 rng, page=page)
        np.testing.assert_allclose(got, ref, atol=1e-2 * np.abs(ref).max(), err_msg=f"pages of {page}")


def test_attention_prefill_far_key_and_window_edge(prefill_kernel):
    rng = np.random.default_rng(29)
    H, Kh, hs, n = 4, 2, 64, 700
    k = rng.standard_normal((n, Kh, hs)).astype(np.float32) * 0.1
    v = rng.standard_normal((n, Kh, hs)).astype(np.float32)
    q = rng.standard_normal((n, H, hs)).astype(np.float32) * 0.1
    far = 13
    k[far, 1] = 0; k[far, 1, 5] = 30.0
    q[n - 1, 2] = 0; q[n - 1, 2, 5] = 30.0
    k, v, q = (rounded(a, "bfloat16") for a in (k, v, q))
    for before, new in ((0, n), (500, 200)):                       # the whole prompt; a chunk after a prefix
        got, ref = run_attention(prefill_fn([before], [new], prefill_kernel), [k], [v], [q], [before], [new], H, Kh, hs, "bfloat16", rng)
        np.testing.assert_allclose(got, ref, atol=1e-2 * np.abs(ref).max())
        np.testing.assert_allclose(got[-1, 2], v[far, 1], atol=4e-2)
    w = 100
    for hot, inside in ((n - w, True), (n - w - 1, False)):
        k2 = k.copy(); k2[far, 1] = 0.0; k2[hot, 1] = 0; k2[hot, 1, 5] = 30.0
        k2 = rounded(k2, "bfloat16")
        got, ref = run_attention(prefill_fn([0], [n], prefill_kernel), [k2], [v], [q], [0], [n], H, Kh, hs, "bfloat16", rng, window=w)
        np.testing.assert_allclose(got, ref, atol=1e-2 * np.abs(ref).max())
        assert (np.abs(got[-1, 2] - v[hot, 1]).max() < 4e-2) == inside


# ------------------------------------------------------------------ norms and rotation folded into the products
def ssq_partials(x, n_partials):
    """Partial sums of squares as a producer leaves them: [n_partials, 64], rows of x in the columns."""
    M, d = x.shape
    out = np.zeros((n_partials, 64), np.float32)
    for p, cols in enumerate(np.array_split(np.arange(d), n_partials)):
        out[p, :M] = (x[:, cols] ** 2).sum(1)
    return out


def times_weight(x, nw):
    """The rows as a folded norm's product reads them: bfloat16(weight * x), computed in float."""
    return (torch.as_tensor(nw.astype(np.float32))[None, :] * torch.as_tensor(x)).to(torch.bfloat16)


@pytest.mark.parametrize("M", [1, 8, 33, 64])
@pytest.mark.parametrize("N, Kd, P_", [(2048, 2048, 128), (130, 64, 1), (1000, 112, 7), (96, 4096, 256), (64, 8192, 300)])
def test_gemm_skinny_with_folded_norm(M, N, Kd, P_):
    rng = np.random.default_rng(M + N)
    extra = 3 if M + 3 <= 64 else 0
    x = (rng.standard_normal((M + extra, Kd)) * 2).astype(np.float32)       # more rows than are used, where they fit
    nw = rounded(1 + 0.2 * rng.standard_normal(Kd), "float32")
    w = rounded(rng.standard_normal((2 * N, Kd)) / math.sqrt(Kd), "bfloat16")
    lib = K()
    XG, W = times_weight(x, nw).to(DEV), dev(w, torch.bfloat16)
    ssq = dev(ssq_partials(x, P_))
    h = P.rmsnorm(x, nw, 1e-5)
    rows = np.arange(M)[::-1].copy() + extra                                 # a gather of rows
    ref = P.linear(h[rows], w[:N])
    out = torch.zeros(M, N, device=DEV)
    lib.gemm_skinny_norm(XG, ssq, P_, 1e-5, W[:N], out, lib.EPI_STORE, rows=dev(rows, torch.int32))
    np.testing.assert_allclose(out.cpu().numpy(), ref, atol=1e-2 * np.abs(ref).max())   # x*w is rounded to bfloat16
    refg = P.silu(P.linear(h[:M], w[:N])) * P.linear(h[:M], w[N:])
    g_ = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
    lib.gemm_skinny_norm(XG[:M], ssq, P_, 1e-5, W, g_, lib.EPI_GATED)
    np.testing.assert_allclose(g_.float().cpu().numpy(), refg, atol=1.5e-2 * max(np.abs(refg).max(), 1e-3))


@pytest.mark.parametrize("M", [1, 7, 8, 16])
@pytest.mark.parametrize("N, Kd, P_", [(8192, 2048, 256), (6144, 136, 3), (130, 64, 1), (1000, 1544, 7), (24, 8192, 40)])
def test_gated_product_with_folded_norm_through_whole_lines(M, N, Kd, P_):
    """The folded norm's gated product on the kernel that loads whole lines, plain rows and rows in the packed
    tiles' order, against the plain implementation and against the kernel that keeps its rows in registers."""
    rng = np.random.default_rng(M + N)
    x = (rng.standard_normal((M + 2, Kd)) * 2).astype(np.float32)
    nw = rounded(1 + 0.2 * rng.standard_normal(Kd), "float32")
    w = rounded(rng.standard_normal((2 * N, Kd)) / math.sqrt(Kd), "bfloat16")
    bias = rng.standard_normal(2 * N).astype(np.float32)
    lib = K()
    XG, W = times_weight(x, nw).to(DEV), dev(w, torch.bfloat16)
    ssq = dev(ssq_partials(x, P_))
    h = P.rmsnorm(x, nw, 1e-5)[:M]
    for b in (None, bias):
        g, u = P.linear(h, w[:N]), P.linear(h, w[N:])
        if b is not None:
            g, u = g + b[:N], u + b[N:]
        ref = P.silu(g) * u
        out = torch.full((M + 1, N + 8), -1.0, device=DEV, dtype=torch.bfloat16)      # a view with a row stride
        lib.gemm_skinny_norm(XG[:M], ssq, P_, 1e-5, W, out[:M, :N], lib.EPI_GATED, bias=None if b is None else dev(b),
                             whole_lines=True)
        np.testing.assert_allclose(out[:M, :N].float().cpu().numpy(), ref, atol=1.5e-2 * max(np.abs(ref).max(), 1e-3))
        assert torch.all(out[M] == -1) and torch.all(out[:, N:] == -1)
        other = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
        lib.gemm_skinny_norm(XG[:M], ssq, P_, 1e-5, W, other, lib.EPI_GATED, bias=None if b is None else dev(b))
        np.testing.assert_allclose(out[:M, :N].float().cpu().numpy(), other.float().cpu().numpy(),
                                   atol=1e-2 * max(np.abs(ref).max(), 1e-3))            # (another order of summation)
    if M <= 8:
        packed = lib.packed_rows(N, torch.bfloat16, DEV)
        packed.fill_(777.0)
        lib.gemm_skinny_norm(XG[:M], ssq, P_, 1e-5, W, packed, lib.EPI_GATED, bias=dev(bias), pack_out=True, whole_lines=True)
        flat = packed.reshape(-1).cpu()
        m, k = np.meshgrid(np.arange(M), np.arange(N), indexing="ij")
        at = (((k // 64) * 64 + ((k % 32) // 8) * 16 + ((k % 64) // 32) * 8 + m) * 8) + k % 8
        assert torch.equal(flat[torch.as_tensor(at)], out[:M, :N].cpu())
        untouched = np.ones(flat.numel(), bool)
        untouched[at.reshape(-1)] = False
        assert torch.all(flat[torch.as_tensor(untouched)] == 777.0)
    with pytest.raises(lib.KernelError):
        lib.gemm_skinny_norm(XG[:M], ssq, P_, 1e-5, W[:N], torch.zeros(M, N, device=DEV), lib.EPI_STORE, whole_lines=True)


@pytest.mark.parametrize("M", [1, 8, 40])
def test_gemm_skinny_leaves_sums_of_squares(M):
    rng = np.random.default_rng(M)
    N, Kd = 208, 96
    a = rounded(rng.standard_normal((M, Kd)), "bfloat16")
    w = rounded(rng.standard_normal((N, Kd)) / 10, "bfloat16")
    res = rng.standard_normal((M, N)).astype(np.float32)
    x = dev(res)
    ssq = torch.full((N // 16, 64), -1.0, device=DEV)
    K().gemm_skinny(dev(a, torch.bfloat16), dev(w, torch.bfloat16), x, K().EPI_ADD, ssq_out=ssq)
    new = res + P.linear(a, w)
    np.testing.assert_allclose(x.cpu().numpy(), new, atol=1e-4)
    got = ssq.cpu().numpy()
    np.testing.assert_allclose(got[:, :M], ssq_partials(new, N // 16)[:, :M], rtol=1e-4)
    assert np.all(got[:, M:] == -1.0)                                        # rows that do not exist are not written
    # the same with the rows times the next norm's weight, in strips of 16 and (few rows) of 8
    nw = (1 + 0.2 * rng.standard_normal(N)).astype(np.float32)
    for strip in ((16, 8) if M <= 16 else (16,)):
        x2 = dev(res)
        ssq2 = torch.full((N // strip, 64), -1.0, device=DEV)
        xg = torch.full((M, N + 8), 9.0, device=DEV, dtype=torch.bfloat16)   # a view with a row stride
        K().gemm_skinny(dev(a, torch.bfloat16), dev(w, torch.bfloat16), x2, K().EPI_ADD, ssq_out=ssq2, strip_rows=strip,
                        next_weight=dev(nw), xg=xg[:, :N])
        np.testing.assert_allclose(x2.cpu().numpy(), new, atol=1e-4)         # (another order of summation per strip size)
        assert torch.equal(xg[:, :N], (dev(nw)[None, :] * x2).to(torch.bfloat16)) and torch.all(xg[:, N:] == 9.0)
        np.testing.assert_allclose(ssq2[:, :M].cpu().numpy(), ssq_partials(new, N // strip)[:, :M], rtol=1e-4)
    with pytest.raises(K().KernelError):
        K().gemm_skinny(dev(a, torch.bfloat16), dev(w, torch.bfloat16), x, K().EPI_ADD, next_weight=dev(nw),
                        xg=torch.empty(M, N, device=DEV, dtype=torch.bfloat16))          # not without the sums of squares


@pytest.mark.parametrize("folded_norm, more_rows", [(True, 0), (False, 45), (False, 21), (False, 0)])
@pytest.mark.parametrize("pairing", ["adjacent", "half", None])
@pytest.mark.parametrize("H, Kh, hs", [(32, 8, 64), (6, 2, 16), (5, 5, 48), (8, 1, 128), (32, 8, 128), (21, 7, 112)])
def test_qkv_rope_cache_in_one_kernel(pairing, H, Kh, hs, folded_norm, more_rows):
    rng = np.random.default_rng(hs + H)
    d, page = 96, 64
    lens_before = [70, 0, 129, 63, 64] + list(range(3, 3 + more_rows))     # 5, 26 and 50 rows: every kernel
    T = len(lens_before)
    x = (rng.standard_normal((T, d)) * 2).astype(np.float32)
    nw = rounded(1 + 0.2 * rng.standard_normal(d), "bfloat16")
    w = rounded(rng.standard_normal(((H + 2 * Kh) * hs, d)) / math.sqrt(d), "bfloat16")
    positions = np.array(lens_before)
    seq_of = np.arange(T)
    zk = [np.zeros((b + 1, Kh, hs), np.float32) for b in lens_before]
    kc, vc, table = paged(zk, zk, Kh, hs, page, "bfloat16", rng)
    before_k, before_v = kc.clone(), vc.clone()
    cos, sin = P.rope_table(256, hs, 50000.0)
    q_out = torch.zeros(T, H * hs, device=DEV, dtype=torch.bfloat16)
    if folded_norm:
        K().qkv_rope_cache(times_weight(x, nw).to(DEV), dev(ssq_partials(x, 6)), 6, 1e-5, dev(w, torch.bfloat16), q_out,
                           dev(positions, torch.int32), dev(seq_of, torch.int32), table,
                           dev(cos) if pairing else None, dev(sin) if pairing else None, kc, vc, H, Kh, hs,
                           pairing == "adjacent", page)
        qkv = P.linear(P.rmsnorm(x, nw, 1e-5), w)
    else:                                                                     # rows that are normalised already
        h = rounded(x, "bfloat16")
        K().qkv_rope_cache(dev(h, torch.bfloat16), None, 0, 0.0, dev(w, torch.bfloat16), q_out,
                           dev(positions, torch.int32), dev(seq_of, torch.int32), table,
                           dev(cos) if pairing else None, dev(sin) if pairing else None, kc, vc, H, Kh, hs,
                           pairing == "adjacent", page)
        qkv = P.linear(h, w)
    q = qkv[:, :H * hs].reshape(T, H, hs)
    k = qkv[:, H * hs:(H + Kh) * hs].reshape(T, Kh, hs)
    v = qkv[:, (H + Kh) * hs:].reshape(T, Kh, hs)
    if pairing:
        q = P.rope_rotate(q, positions, cos, sin, pairing)
        k = P.rope_rotate(k, positions, cos, sin, pairing)
    tol_ = 1.5e-2 * np.abs(qkv).max()
    np.testing.assert_allclose(q_out.float().cpu().numpy().reshape(T, H, hs), q, atol=tol_)
    kcpu, vcpu, tab = untile_keys(kc).float().cpu().numpy(), untile_values(vc).float().cpu().numpy(), table.cpu().numpy()
    mk, mv = torch.ones_like(kc, dtype=torch.bool), torch.ones_like(vc, dtype=torch.bool)
    for i in range(T):
        pid = tab[i, positions[i] // page]
        np.testing.assert_allclose(kcpu[pid, :, positions[i] % page], k[i], atol=tol_)
        np.testing.assert_allclose(vcpu[pid, :, :, positions[i] % page], v[i], atol=tol_)
        mk[pid, :, positions[i] % page] = False
        mv[pid, :, :, positions[i] % page] = False
    assert torch.equal(untile_keys(kc)[mk], untile_keys(before_k)[mk])                # nothing else moved
    assert torch.equal(untile_values(vc)[mv], untile_values(before_v)[mv])


# ------------------------------------------------------------------ the wide kernel for 17 to 64 rows, K in slices
@pytest.mark.parametrize("M", [17, 32, 33, 48, 64])
@pytest.mark.parametrize("N, Kd", [(2048, 2048), (130, 72), (40, 40), (1000, 1544), (6144, 256)])
def test_gemm_skinny_wide(M, N, Kd):
    rng = np.random.default_rng(M + N)
    a = rounded(rng.standard_normal((M, Kd)), "bfloat16")
    w = rounded(rng.standard_normal((2 * N, Kd)) / math.sqrt(Kd), "bfloat16")
    A, W = dev(a, torch.bfloat16), dev(w, torch.bfloat16)
    lib = K()
    ref = P.linear(a, w[:N])
    scale = np.abs(ref).max()
    tol32 = 2e-5 * scale * math.sqrt(Kd / 64)
    for strips in (0, 2, 4):
        out = torch.full((M + 1, N + 3), -1.0, device=DEV)                  # a view with a row stride, a row beyond
        lib.gemm_skinny_wide(A, W[:N], out[:M, :N], lib.EPI_STORE, strips=strips)
        np.testing.assert_allclose(out[:M, :N].cpu().numpy(), ref, atol=tol32, err_msg=f"strips {strips}")
        assert torch.all(out[M] == -1) and torch.all(out[:, N:] == -1)
        for slices in sorted({s_ for s_ in (2, 3, 8) if s_ <= (Kd + 63) // 64}):
            part = torch.full((slices, M, N), 7.0, device=DEV)
            lib.gemm_skinny_wide(A, W[:N], part, lib.EPI_STORE, strips=strips)
            np.testing.assert_allclose(part.sum(0).cpu().numpy(), ref, atol=tol32, err_msg=f"{slices} slices")
            per = -(-((Kd + 63) // 64) // slices) * 64                        # each slice is its own range of K
            for s_ in range(slices):
                lo, hi = min(s_ * per, Kd), min((s_ + 1) * per, Kd)
                np.testing.assert_allclose(part[s_].cpu().numpy(), P.linear(a[:, lo:hi], w[:N, lo:hi]) if hi > lo
                                           else np.zeros((M, N), np.float32), atol=tol32)
    ob = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
    lib.gemm_skinny_wide(A, W[:N], ob)
    np.testing.assert_allclose(ob.float().cpu().numpy(), ref, atol=1e-2 * scale)
    res = rng.standard_normal((M, N)).astype(np.float32)
    x = dev(res)
    lib.gemm_skinny_wide(A, W[:N], x, lib.EPI_ADD)
    np.testing.assert_allclose(x.cpu().numpy(), res + ref, atol=tol32 + 1e-6)
    refg = P.silu(P.linear(a, w[:N])) * P.linear(a, w[N:])
    for strips in (0, 1, 2):
        g_ = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
        lib.gemm_skinny_wide(A, W, g_, lib.EPI_GATED, strips=strips)
        np.testing.assert_allclose(g_.float().cpu().numpy(), refg, atol=1e-2 * max(np.abs(refg).max(), 1e-3))


@pytest.mark.parametrize("M", [9, 16])
@pytest.mark.parametrize("N, Kd", [(2048, 8192), (130, 200), (40, 4104)])
def test_gemm_skinny_wide_slices_of_9_to_16_rows(M, N, Kd):
    """9 to 16 rows: only what a long K into the residual stream needs, a float output stored, in slices or whole."""
    rng = np.random.default_rng(M + N)
    a = rounded(rng.standard_normal((M, Kd)), "bfloat16")
    w = rounded(rng.standard_normal((N, Kd)) / math.sqrt(Kd), "bfloat16")
    A, W = dev(a, torch.bfloat16), dev(w, torch.bfloat16)
    lib = K()
    ref = P.linear(a, w)
    tol32 = 2e-5 * np.abs(ref).max() * math.sqrt(Kd / 64)
    for slices in (1, 2, 4):
        part = torch.full((slices, M + 1, N + 3), 7.0, device=DEV)
        lib.gemm_skinny_wide(A, W, part[:, :M, :N], lib.EPI_STORE)
        np.testing.assert_allclose(part[:, :M, :N].sum(0).cpu().numpy(), ref, atol=tol32, err_msg=f"{slices} slices")
        assert torch.all(part[:, M] == 7.0) and torch.all(part[:, :, N:] == 7.0)
    with pytest.raises(lib.KernelError):
        lib.gemm_skinny_wide(A, W, torch.zeros(M, N, device=DEV), lib.EPI_ADD)
    with pytest.raises(lib.KernelError):
        lib.gemm_skinny_wide(A, W, torch.zeros(M, N, device=DEV, dtype=torch.bfloat16))


def test_gemm_skinny_wide_refuses_what_it_cannot_do():
    lib = K()
    a = torch.zeros(40, 64, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(32, 64, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(lib.KernelError):
        lib.gemm_skinny_wide(a[:8], w, torch.zeros(8, 32, device=DEV))                         # the skinny kernel's rows
    with pytest.raises(lib.KernelError, match="slices"):
        lib.gemm_skinny_wide(a, w, torch.zeros(2, 40, 32, device=DEV), lib.EPI_ADD)            # slices are stored, not added
    with pytest.raises(lib.KernelError, match="slices"):
        lib.gemm_skinny_wide(a, w, torch.zeros(3, 40, 32, device=DEV))                         # more slices than pairs of k-steps
    assert lib.wide_slices(2048, 8192) == 4 and lib.wide_slices(2048, 2048) == 4 and lib.wide_slices(128256, 2048) == 1


@pytest.mark.parametrize("d, wdtype, odtype, S", [(2048, "bfloat16", "bfloat16", 8), (100, "float32", "float32", 5),
                                                  (7, "float32", "bfloat16", 3), (9000, "float32", "float32", 11)])
def test_add_slices_rmsnorm(d, wdtype, odtype, S):
    rng = np.random.default_rng(d)
    M = 37
    x = (rng.standard_normal((M, d)) * 3).astype(np.float32)
    parts = rng.standard_normal((S, M, d)).astype(np.float32)
    w = rounded(1 + 0.2 * rng.standard_normal(d), wdtype)
    total = x.copy()
    for s_ in range(S):
        total = total + parts[s_]                                            # the kernel's order of summation
    lib = K()
    X = dev(x)
    out = torch.empty(M, d, device=DEV, dtype=TD[odtype])
    lib.add_slices_rmsnorm(X, dev(parts), dev(w, TD[wdtype]), out, 1e-6)
    assert np.array_equal(X.cpu().numpy(), total)
    np.testing.assert_allclose(out.float().cpu().numpy(), P.rmsnorm(total, w, 1e-6),
                               rtol=1e-5 if odtype == "float32" else 5e-3, atol=1e-6)
    X2 = dev(x)
    lib.add_slices_rmsnorm(X2, dev(parts))                                   # the sums alone
    assert np.array_equal(X2.cpu().numpy(), total)
    rows = np.array([7, 0, 7, 36])                                           # listed rows: x stays as it was
    X3 = dev(x)
    out3 = torch.empty(4, d, device=DEV, dtype=TD[odtype])
    lib.add_slices_rmsnorm(X3, dev(parts), dev(w, TD[wdtype]), out3, 1e-6, dev(rows, torch.int32))
    assert np.array_equal(X3.cpu().numpy(), x)
    assert torch.equal(out3, out[torch.as_tensor(rows).to(DEV)])
    with pytest.raises(lib.KernelError):
        lib.add_slices_rmsnorm(X, dev(parts[:, :5]))


@pytest.mark.parametrize("V", [2, 63, 1000, 128256])
def test_argmax_kernel_takes_the_first_of_the_greatest(V):
    rng = np.random.default_rng(V)
    R = 9
    logits = rng.standard_normal((R, V)).astype(np.float32)
    logits[2, [V // 3, V - 1]] = 50.0                       # ties: the lower index, across slices
    logits[5, :] = -np.inf                                    # nothing greater than -inf: index 0
    logits[6, 0] = 60.0
    logits[7, V - 1] = 60.0
    wide = torch.zeros(R, V + 5, device=DEV)                  # rows with a stride
    wide[:, :V] = dev(logits)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    K().argmax(wide[:, :V], torch.empty(128 * R, device=DEV), out)
    assert out.tolist() == [P.argmax(row) for row in logits]


@pytest.mark.parametrize("R, V", [(1, 1000), (9, 63), (40, 128256), (64, 5000)])
def test_greedy_pick_and_the_run_s_bookkeeping_in_one(R, V):
    """``argmax_advance`` is ``argmax`` followed by ``decode_advance``: the winners (first of the greatest) become the
    next tokens, go into the history row that the step counter names, every sequence moves on by one, the counter
    goes up; more rows than the block has waves, two steps in a row."""
    rng = np.random.default_rng(R + V)
    lib = K()
    work = torch.empty(128 * R, device=DEV)
    tok = torch.full((R,), -1, dtype=torch.int32, device=DEV)
    pos = dev(rng.integers(0, 500, R), torch.int32)
    before = pos.clone()
    pos0 = pos.cpu().numpy().copy()
    hist = torch.full((4, R + 2), -3, dtype=torch.int32, device=DEV)
    step = torch.tensor([1], dtype=torch.int32, device=DEV)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    for n in range(2):
        logits = rng.standard_normal((R, V)).astype(np.float32)
        logits[0, [V // 3, V - 1]] = 50.0                      # a tie: the lower index
        if R > 2:
            logits[2, :] = -np.inf                               # nothing greater than -inf: index 0
        want = [P.argmax(row) for row in logits]
        lib.argmax_advance(dev(logits), work, out, tok, pos, before, hist, step)
        assert out.tolist() == want and tok.tolist() == want
        assert hist[1 + n, :R].tolist() == want and torch.all(hist[1 + n, R:] == -3)
        assert step.item() == 2 + n
        assert np.array_equal(pos.cpu().numpy(), pos0 + n + 1) and torch.equal(before, pos)
    assert torch.all(hist[0] == -3) and torch.all(hist[3] == -3)


# ------------------------------------------------------------------ biases and the other activation in the products' epilogues
def gelu_tanh(v):
    return 0.5 * v * (1 + np.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3)))


def epilogue_reference(a, w, epilogue, bias, act, before=None):
    """What a product's end makes of a @ w.T in float64: bias first, then store / add / act(gate) * up."""
    s = a.astype(np.float64) @ w.astype(np.float64).T
    if bias is not None:
        s = s + bias.astype(np.float64)
    if epilogue == 2:
        n = s.shape[1] // 2
        g = s[:, :n]
        return (g / (1 + np.exp(-g)) if act == "silu" else gelu_tanh(g)) * s[:, n:]
    return s + before if epilogue == 1 else s


PRODUCTS = ["generic float32", "generic bfloat16", "tiled", "few rows", "few rows, folded norm",
            "few rows, folded norm, whole lines", "17 to 32 rows", "33 to 64 rows"]


@pytest.mark.parametrize("which", PRODUCTS)
@pytest.mark.parametrize("epilogue, act", [(0, "silu"), (1, "silu"), (2, "silu"), (2, "gelu_tanh")])
def test_products_with_bias_and_activation(which, epilogue, act):
    """Every product kernel with a bias per output column (the gated epilogue: the gate's, then the
    up's) and both activations, against the same in float64. The bias is large next to the sums, so
    that one added twice, to the wrong half or after the activation shows."""
    lib = K()
    rng = np.random.default_rng(len(which) * 7 + epilogue)
    M = {"tiled": 150, "33 to 64 rows": 40, "17 to 32 rows": 21}.get(which, 9)
    N, Kd = 200, 136                                               # output columns: no tile divides them
    dtype = "float32" if which == "generic float32" else "bfloat16"
    wrows = 2 * N if epilogue == 2 else N
    a = rounded(rng.standard_normal((M, Kd)), dtype)
    w = rounded(rng.standard_normal((wrows, Kd)) * 0.1, dtype)
    bias = (rng.standard_normal(wrows) * 2).astype(np.float32)
    before = rng.standard_normal((M, N)).astype(np.float32)
    out_dtype = torch.float32 if epilogue == 1 or dtype == "float32" else torch.bfloat16
    out = dev(before, out_dtype) if epilogue == 1 else torch.zeros(M, N, device=DEV, dtype=out_dtype)
    A, W, B = dev(a, TD[dtype]), dev(w, TD[dtype]), dev(bias)
    ref_a = a
    if which.startswith("generic"):
        lib.gemm_generic(A, W, out, epilogue, bias=B, act=act)
    elif which == "tiled":
        lib.gemm_mfma(A, W, out, epilogue, bias=B, act=act)
    elif which == "few rows":
        lib.gemm_skinny(A, W, out, epilogue, bias=B, act=act)
    elif which in ("33 to 64 rows", "17 to 32 rows"):
        lib.gemm_skinny_wide(A, W, out, epilogue, bias=B, act=act)
    else:
        if epilogue == 1:
            pytest.skip("a folded norm feeds store and gated products only")
        if which.endswith("whole lines") and epilogue != 2:
            pytest.skip("whole lines take the gated product only")
        x = (rng.standard_normal((M, Kd)) * 2).astype(np.float32)
        nw = (1 + 0.2 * rng.standard_normal(Kd)).astype(np.float32)
        xg = times_weight(x, nw).to(DEV)
        ssq = dev(ssq_partials(x, 3))
        lib.gemm_skinny_norm(xg, ssq, 3, 1e-5, W, out, epilogue, bias=B, act=act, whole_lines=which.endswith("whole lines"))
        ref_a = xg.float().cpu().numpy() / np.sqrt((x.astype(np.float64) ** 2).mean(1, keepdims=True) + 1e-5)
    ref = epilogue_reference(ref_a, w, epilogue, bias, act, before)
    np.testing.assert_allclose(out.float().cpu().numpy(), ref, atol=tol(dtype) * np.abs(ref).max())
    with pytest.raises(lib.KernelError):
        lib.gemm_generic(A, W, out, epilogue, bias=B[:-1])
    with pytest.raises(lib.KernelError, match="activation"):
        lib.gemm_generic(A, W, out, epilogue, act="relu")


def test_embed_with_a_multiplier_and_a_table_of_positions():
    rng = np.random.default_rng(3)
    for dtype, d in (("float32", 70), ("bfloat16", 256)):          # scalar and 16-byte paths
        table = rounded(rng.standard_normal((300, d)), dtype)
        ptab = rounded(rng.standard_normal((50, d)), dtype)
        ids, pos = rng.integers(0, 300, 21), rng.integers(0, 50, 21)
        out = torch.empty(21, d, device=DEV)
        K().embed(dev(table, TD[dtype]), dev(ids, torch.int32), out, scale=3.5, pos_table=dev(ptab, TD[dtype]),
                  positions=dev(pos, torch.int32))
        np.testing.assert_allclose(out.cpu().numpy(), 3.5 * table[ids] + ptab[pos], rtol=1e-6, atol=1e-6)
        K().embed(dev(table, TD[dtype]), dev(ids, torch.int32), out, scale=0.25)
        np.testing.assert_array_equal(out.cpu().numpy(), 0.25 * table[ids])
    t = dev(rng.standard_normal((5, 33)))
    before = t.clone()
    K().scale_(t, 1.5)
    assert torch.equal(t, before * 1.5)


def test_scatter_of_table_entries():
    lib = K()
    t = torch.zeros(6, 50, dtype=torch.int32, device=DEV)
    rng = np.random.default_rng(0)
    places = rng.permutation(300)[:200].tolist()                  # more than one launch holds
    values = rng.integers(1, 1000, 200).tolist()
    lib.scatter_i32(t, places, values)
    want = np.zeros(300, np.int32)
    want[places] = values
    assert t.view(-1).cpu().numpy().tolist() == want.tolist()
    with pytest.raises(lib.KernelError, match="outside"):
        lib.scatter_i32(t, [300], [1])


@pytest.mark.parametrize("M", [1, 5, 8, 9, 16])
@pytest.mark.parametrize("N, Kd", [(2048, 2048), (2048, 8192), (130, 40), (24, 136), (1000, 72), (8, 64)])
def test_gemm_skinny_strips_of_eight_rows(M, N, Kd):
    """Strips of 8 rows of the weights. With at most 8 rows of ``a`` the tile's second half takes the
    next 32 k (K of no multiple of 64 ends inside such a step); with 9 to 16 rows it idles. One
    column of the weights is large, so that a half of the sum that is dropped or taken twice shows."""
    lib = K()
    rng = np.random.default_rng(M * 1000 + N + Kd)
    a = rounded(rng.standard_normal((M, Kd)), "bfloat16")
    w = rounded(rng.standard_normal((N, Kd)) / 10, "bfloat16")
    w[:, Kd - 1] *= 20; w[:, min(Kd - 1, 37)] *= 20                         # in the last step, and in a second half
    w = rounded(w, "bfloat16")
    ref = a.astype(np.float64) @ w.astype(np.float64).T
    A, W = dev(a, torch.bfloat16), dev(w, torch.bfloat16)
    out = torch.full((M, N), 7.0, device=DEV)
    lib.gemm_skinny(A, W, out, lib.EPI_STORE, strip_rows=8)
    np.testing.assert_allclose(out.cpu().numpy(), ref, atol=2e-5 * np.abs(ref).max() + 1e-5)
    before = rng.standard_normal((M, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    x = dev(before)
    ssq = torch.full((-(-N // 8), 64), -1.0, device=DEV)
    if N % 16 == 0:
        lib.gemm_skinny(A, W, x, lib.EPI_ADD, ssq_out=ssq, strip_rows=8, bias=dev(bias))
        new = before + ref + bias
        np.testing.assert_allclose(ssq[:N // 8, :M].cpu().numpy(), ssq_partials(new.astype(np.float32), N // 8)[:, :M], rtol=1e-4)
    else:
        lib.gemm_skinny(A, W, x, lib.EPI_ADD, strip_rows=8, bias=dev(bias))
        new = before + ref + bias
    np.testing.assert_allclose(x.cpu().numpy(), new, atol=2e-5 * np.abs(new).max() + 1e-5)


# ------------------------------------------------------------------ weights in the operands' order
@pytest.mark.parametrize("N, Kd", [(48, 72), (2048, 2048), (160, 1544), (6144, 256), (1008, 4104)])
@pytest.mark.parametrize("M", [1, 8, 16, 29])
def test_products_read_a_weight_copy_in_operand_order(M, N, Kd):
    """``tile_weight``: [strip][k-step][lane][8] with k padded to whole steps. The kernels that keep the
    step's rows in registers read it in place of the rows of W; the sums are the same sums, bit for bit."""
    rng = np.random.default_rng(M + N + Kd)
    lib = K()
    w = dev(rounded(rng.standard_normal((2 * N, Kd)) / math.sqrt(Kd), "bfloat16"), torch.bfloat16)
    t = lib.tile_weight(w)
    steps = -(-Kd // 32)
    flat = t.reshape(-1).float().cpu().numpy()
    wn = w.float().cpu().numpy()
    for (n, k) in [(0, 0), (17, 9), (2 * N - 1, Kd - 1), (N + 5, Kd // 2), (31, 40 % Kd)]:
        strip, r, step, q, e = n // 16, n % 16, k // 32, (k % 32) // 8, k % 8
        assert flat[((strip * steps + step) * 64 + q * 16 + r) * 8 + e] == wn[n, k]
    x = (rng.standard_normal((M, Kd)) * 2).astype(np.float32)
    nw = rounded(1 + 0.2 * rng.standard_normal(Kd), "bfloat16")
    xg, ssq = times_weight(x, nw).to(DEV), dev(ssq_partials(x, 5))
    a = dev(rounded(x, "bfloat16"), torch.bfloat16)
    res = {}
    for tiled in (False, True):
        if tiled:
            w.tiled = t
        outs = []
        for waves in (0, 8, 16):            # the library's choice; the kernels that stream the rows of A, 8 and 16 waves
            g_ = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
            lib.gemm_skinny_norm(xg, ssq, 5, 1e-5, w, g_, lib.EPI_GATED, waves=waves)
            s_ = torch.zeros(M, 2 * N, device=DEV)
            lib.gemm_skinny_norm(xg, ssq, 5, 1e-5, w, s_, lib.EPI_STORE, waves=waves)
            p_ = torch.zeros(M, 2 * N, device=DEV)
            lib.gemm_skinny(a, w, p_, lib.EPI_STORE, waves=waves)
            outs += [g_, s_, p_]
        res[tiled] = tuple(outs)
    for u, v in zip(res[False], res[True]):
        assert torch.equal(u, v)
    np.testing.assert_allclose(res[True][2].cpu().numpy(), P.linear(rounded(x, "bfloat16"), wn),
                               atol=2e-5 * np.abs(wn).max() * np.abs(x).max() * Kd)
    # a copy that does not belong to the call's rows is not used
    w.tiled = lib.tile_weight(w[:N].contiguous())
    p2 = torch.zeros(M, 2 * N, device=DEV)
    lib.gemm_skinny(a, w, p2, lib.EPI_STORE)
    assert torch.equal(p2, res[False][2])


@pytest.mark.parametrize("N, Kd", [(48, 64), (2048, 2048), (272, 1600), (8208, 192)])
def test_a_weight_kept_in_operand_order_alone(N, Kd):
    """``hold_once``: the matrix's memory is its copy in the operands' order. The embedding look-up, the generic
    product, the tiled product (store epilogue, both tiles) and the products of few rows give what they give
    for the stored order, bit for bit; ``untile_weight`` gives the stored order back; what cannot read it refuses."""
    rng = np.random.default_rng(N + Kd)
    lib = K()
    w = dev(rounded(rng.standard_normal((N, Kd)) / math.sqrt(Kd), "bfloat16"), torch.bfloat16)
    w.tiled = lib.tile_weight(w)
    once = lib.hold_once(w)
    assert lib.held_once(once) and not lib.held_once(w) and once.shape == w.shape and once.data_ptr() == w.tiled.data_ptr()
    assert torch.equal(lib.untile_weight(once.tiled, N, Kd), w)
    # the embedding look-up, with and without what a folded norm wants
    ids = torch.tensor(rng.integers(0, N, 19), dtype=torch.int32, device=DEV)
    e1, e2 = torch.zeros(19, Kd, device=DEV), torch.zeros(19, Kd, device=DEV)
    lib.embed(w, ids, e1); lib.embed(once, ids, e2)
    assert torch.equal(e1, e2) and torch.equal(e1, w[ids.long()].float())
    nw = dev(1 + 0.1 * rng.standard_normal(Kd))
    got = []
    for table in (w, once):
        o, q, g_ = torch.zeros(19, Kd, device=DEV), torch.zeros(64, device=DEV), torch.zeros(19, Kd, device=DEV, dtype=torch.bfloat16)
        lib.embed(table, ids, o, q, nw, g_, scale=1.5)
        got.append((o, q, g_))
    assert all(torch.equal(u, v) for u, v in zip(*got))
    # products of many rows: the generic kernel and both tiles of the tiled one, odd row counts
    for M in (3, 65, 300):
        a = dev(rounded(rng.standard_normal((M, Kd)), "bfloat16"), torch.bfloat16)
        ref = P.linear(a.float().cpu().numpy(), w.float().cpu().numpy())
        g1, g2 = torch.zeros(M, N, device=DEV), torch.zeros(M, N, device=DEV)
        lib.gemm_generic(a, w, g1); lib.gemm_generic(a, once, g2)
        assert torch.equal(g1, g2)
        for shape in (1, 2, 0):
            m1, m2 = torch.zeros(M, N, device=DEV), torch.full((M, N + 3), -7.0, device=DEV)
            lib.gemm_mfma(a, w, m1, shape=shape); lib.gemm_mfma(a, once, m2[:, :N], shape=shape)
            assert torch.equal(m1, m2[:, :N]) and torch.all(m2[:, N:] == -7.0), (M, shape)
            np.testing.assert_allclose(m1.cpu().numpy(), ref, atol=2e-5 * np.abs(ref).max() * math.sqrt(Kd))
        b1, b2 = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16), torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
        lib.gemm_mfma(a, w, b1, shape=1); lib.gemm_mfma(a, once, b2, shape=1)
        assert torch.equal(b1, b2)
    # products of few rows read the copy as before
    for M in (1, 8, 16, 40, 64):
        a = dev(rounded(rng.standard_normal((M, Kd)), "bfloat16"), torch.bfloat16)
        s1, s2 = torch.zeros(M, N, device=DEV), torch.zeros(M, N, device=DEV)
        lib.gemm_skinny(a, w, s1); lib.gemm_skinny(a, once, s2)
        assert torch.equal(s1, s2), M
    x = (rng.standard_normal((9, Kd)) * 2).astype(np.float32)
    xg, ssq = times_weight(x, rounded(1 + 0.2 * rng.standard_normal(Kd), "bfloat16")).to(DEV), dev(ssq_partials(x, 3))
    n1, n2 = torch.zeros(9, N, device=DEV), torch.zeros(9, N, device=DEV)
    lib.gemm_skinny_norm(xg, ssq, 3, 1e-5, w, n1); lib.gemm_skinny_norm(xg, ssq, 3, 1e-5, once, n2)
    assert torch.equal(n1, n2)
    # what reads the stored order only says so
    a = dev(rounded(rng.standard_normal((8, Kd)), "bfloat16"), torch.bfloat16)
    with pytest.raises(lib.KernelError, match="matrix cores' order alone"):
        lib.gemm_skinny(a, once, torch.zeros(8, N, device=DEV), strip_rows=8)          # it has no copy in strips of 8
    with pytest.raises(lib.KernelError, match="hold_once"):
        lib.hold_once(dev(np.zeros((16, 40)), torch.bfloat16))              # no copy
    odd = dev(np.zeros((16, 96)), torch.bfloat16)
    odd.tiled = lib.tile_weight(odd)
    assert not lib.can_hold_once(odd)                                       # K is no whole number of the tiled product's steps


@pytest.mark.parametrize("F, Kd", [(48, 64), (4096, 2048), (272, 1600), (6160, 192)])
def test_stacked_gate_and_up_rows_kept_in_operand_order_alone(F, Kd):
    """The gate rows and the up rows of a feed-forward, stacked and held once: in the copy the up strips follow the
    F / 16 gate strips. The tiled product (all three tiles, whole and cut tiles), the kernel of whole lines, the
    products of few rows and the generic product give, with the gated epilogue, what they give over the stored
    rows, bit for bit."""
    rng = np.random.default_rng(F + Kd)
    lib = K()
    w = dev(rounded(rng.standard_normal((2 * F, Kd)) / math.sqrt(Kd), "bfloat16"), torch.bfloat16)
    w.tiled = lib.tile_weight(w)
    once = lib.hold_once(w)
    assert lib.held_once(once) and torch.equal(lib.stored_order(once), w)
    for M in (1, 8, 13, 24, 64, 65, 300, 1100):
        a = dev(rounded(rng.standard_normal((M, Kd)), "bfloat16"), torch.bfloat16)
        g, u = P.linear(a.float().cpu().numpy(), w[:F].float().cpu().numpy()), P.linear(a.float().cpu().numpy(), w[F:].float().cpu().numpy())
        ref = g / (1 + np.exp(-g)) * u
        if M in (1, 13, 65):
            g1, g2 = torch.zeros(M, F, device=DEV), torch.zeros(M, F, device=DEV)
            lib.gemm_generic(a, w, g1, lib.EPI_GATED); lib.gemm_generic(a, once, g2, lib.EPI_GATED)
            assert torch.equal(g1, g2)
        if M >= 65:
            for shape in (1, 2, 5, 0):
                m1 = torch.zeros(M, F, device=DEV, dtype=torch.bfloat16)
                m2 = torch.full((M, F + 3), -7.0, device=DEV, dtype=torch.bfloat16)
                lib.gemm_mfma(a, w, m1, lib.EPI_GATED, shape=shape); lib.gemm_mfma(a, once, m2[:, :F], lib.EPI_GATED, shape=shape)
                assert torch.equal(m1, m2[:, :F]) and torch.all(m2[:, F:] == -7.0), (M, shape)
                np.testing.assert_allclose(m1.float().cpu().numpy(), ref, atol=2e-2 * np.abs(ref).max())
            f1, f2 = torch.zeros(M, F, device=DEV), torch.zeros(M, F, device=DEV)
            lib.gemm_mfma(a, w, f1, lib.EPI_GATED); lib.gemm_mfma(a, once, f2, lib.EPI_GATED)
            assert torch.equal(f1, f2)
        if 16 < M <= 64:
            s1, s2 = torch.zeros(M, F, device=DEV, dtype=torch.bfloat16), torch.zeros(M, F, device=DEV, dtype=torch.bfloat16)
            lib.gemm_skinny_wide(a, w, s1, lib.EPI_GATED); lib.gemm_skinny_wide(a, once, s2, lib.EPI_GATED)
            assert torch.equal(s1, s2), M
        if M <= 64:
            s1, s2 = torch.zeros(M, F, device=DEV, dtype=torch.bfloat16), torch.zeros(M, F, device=DEV, dtype=torch.bfloat16)
            lib.gemm_skinny(a, w, s1, lib.EPI_GATED); lib.gemm_skinny(a, once, s2, lib.EPI_GATED)
            assert torch.equal(s1, s2), M
    # a folded norm in front, on the kernel of few rows and on the kernel of whole lines
    x = (rng.standard_normal((9, Kd)) * 2).astype(np.float32)
    xg, ssq = times_weight(x, rounded(1 + 0.2 * rng.standard_normal(Kd), "bfloat16")).to(DEV), dev(ssq_partials(x, 3))
    for whole in (False, True):
        n1, n2 = torch.zeros(9, F, device=DEV, dtype=torch.bfloat16), torch.zeros(9, F, device=DEV, dtype=torch.bfloat16)
        lib.gemm_skinny_norm(xg, ssq, 3, 1e-5, w, n1, lib.EPI_GATED, whole_lines=whole)
        lib.gemm_skinny_norm(xg, ssq, 3, 1e-5, once, n2, lib.EPI_GATED, whole_lines=whole)
        assert torch.equal(n1, n2), whole


@pytest.mark.parametrize("pairing", ["adjacent", "half", None])
@pytest.mark.parametrize("H, Kh, hs", [(32, 8, 64), (6, 2, 16), (5, 5, 48), (8, 1, 128)])
def test_qkv_rope_cache_reads_a_weight_copy_in_operand_order(pairing, H, Kh, hs):
    """The stacked q, k, v rows in the operands' order hold, for half-split pairing, 8 rows of a head and
    the 8 half a head further in one strip (``strip_rows_of``), as the kernel's strips do."""
    rng = np.random.default_rng(hs + H)
    lib = K()
    d, page, T = 96, 64, 7
    x = (rng.standard_normal((T, d)) * 2).astype(np.float32)
    nw = rounded(1 + 0.2 * rng.standard_normal(d), "bfloat16")
    w = dev(rounded(rng.standard_normal(((H + 2 * Kh) * hs, d)) / math.sqrt(d), "bfloat16"), torch.bfloat16)
    positions = np.array([70, 0, 129, 63, 64, 5, 31])
    zk = [np.zeros((b + 1, Kh, hs), np.float32) for b in positions]
    cos, sin = P.rope_table(256, hs, 50000.0)
    got = {}
    for tiled in (False, True):
        if tiled:
            w.tiled = lib.tile_weight(w, qkv=(H, Kh, hs, pairing is not None, pairing == "adjacent"))
        kc, vc, table = paged(zk, zk, Kh, hs, page, "bfloat16", np.random.default_rng(1))
        q_out = torch.zeros(T, H * hs, device=DEV, dtype=torch.bfloat16)
        lib.qkv_rope_cache(times_weight(x, nw).to(DEV), dev(ssq_partials(x, 6)), 6, 1e-5, w, q_out,
                           dev(positions, torch.int32), dev(np.arange(T), torch.int32), table,
                           dev(cos) if pairing else None, dev(sin) if pairing else None, kc, vc, H, Kh, hs,
                           pairing == "adjacent", page)
        got[tiled] = (q_out, kc, vc)
    for u, v in zip(got[False], got[True]):
        assert torch.equal(u, v)
    # a copy made for another pairing is not used
    w.tiled = lib.tile_weight(w, qkv=(H, Kh, hs, pairing is None, False))
    kc, vc, table = paged(zk, zk, Kh, hs, page, "bfloat16", np.random.default_rng(1))
    q2 = torch.zeros(T, H * hs, device=DEV, dtype=torch.bfloat16)
    lib.qkv_rope_cache(times_weight(x, nw).to(DEV), dev(ssq_partials(x, 6)), 6, 1e-5, w, q2,
                       dev(positions, torch.int32), dev(np.arange(T), torch.int32), table,
                       dev(cos) if pairing else None, dev(sin) if pairing else None, kc, vc, H, Kh, hs,
                       pairing == "adjacent", page)
    assert torch.equal(q2, got[False][0])


@pytest.mark.parametrize("N, Kd", [(48, 64), (2048, 2048), (272, 1600), (2048, 8192), (136, 320)])
def test_a_weight_kept_in_either_copy_s_order_alone(N, Kd):
    """A weight of a product into the residual stream that is held once, as its copy in the operands' order
    (strips of 16) or in packed strips of 8: the kernel of whole lines (17 to 64 rows, 9 to 16 into slices),
    the tiled product's add epilogue with K in slices, the generic product and the products of few rows give what
    they give for the stored rows, bit for bit; ``stored_order`` gives the rows back."""
    rng = np.random.default_rng(N * 3 + Kd)
    lib = K()
    w = dev(rounded(rng.standard_normal((N, Kd)) / math.sqrt(Kd), "bfloat16"), torch.bfloat16)
    holders = {}
    if N % 16 == 0:
        w16 = w.clone(); w16.tiled = lib.tile_weight(w16); holders["strips of 16"] = lib.hold_once(w16)
    if N % 8 == 0 and Kd % 64 == 0:
        w8 = w.clone(); w8.tiled8 = lib.tile_weight8(w8); holders["strips of 8"] = lib.hold_once(w8)
        assert holders["strips of 8"].data_ptr() == w8.tiled8.data_ptr()
    for how, once in holders.items():
        assert lib.held_once(once) and torch.equal(lib.stored_order(once), w), how
        # (over the packed strips of 8 the kernel of whole lines deals the k-steps to its waves in runs, not in turn:
        # the same products summed in another order)
        same = (lambda u, v: torch.equal(u, v)) if how == "strips of 16" else (
            lambda u, v: bool(((u.float() - v.float()).abs().max() <= 2e-2 * max(1e-6, float(u.float().abs().max())))))
        for M in (9, 16, 17, 40, 64):
            a = dev(rounded(rng.standard_normal((M, Kd)), "bfloat16"), torch.bfloat16)
            assert lib.gemm_skinny_wide_fits(a, once, torch.zeros(M, N, device=DEV), lib.EPI_STORE)
            slices = max(2, min(4, Kd // 64)) if Kd >= 128 else 1
            if M > 16 or slices > 1:
                shape = (slices, M, N) if slices > 1 else (M, N)
                p1, p2 = torch.zeros(shape, device=DEV), torch.zeros(shape, device=DEV)
                lib.gemm_skinny_wide(a, w, p1); lib.gemm_skinny_wide(a, once, p2)
                assert same(p1.sum(0) if slices > 1 else p1, p2.sum(0) if slices > 1 else p2), (how, M, "slices")
            if M > 16:
                res = rng.standard_normal((M, N)).astype(np.float32)
                x1, x2 = dev(res), dev(res)
                lib.gemm_skinny_wide(a, w, x1, lib.EPI_ADD); lib.gemm_skinny_wide(a, once, x2, lib.EPI_ADD)
                assert same(x1, x2), (how, M, "add")
                b1, b2 = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16), torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
                lib.gemm_skinny_wide(a, w, b1); lib.gemm_skinny_wide(a, once, b2)
                assert same(b1, b2), (how, M, "store")
        for M in (5, 130, 300):
            a = dev(rounded(rng.standard_normal((M, Kd)), "bfloat16"), torch.bfloat16)
            res = rng.standard_normal((M, N)).astype(np.float32)
            g1, g2 = dev(res), dev(res)
            lib.gemm_generic(a, w, g1, lib.EPI_ADD); lib.gemm_generic(a, once, g2, lib.EPI_ADD)
            assert torch.equal(g1, g2), (how, M, "generic")
            for shape in (1, 2, 0):
                for n_more in (0, 1, 2):
                    if n_more and Kd // (n_more + 1) < 64:
                        continue
                    x1, x2 = dev(res), dev(res)
                    m1 = torch.zeros(n_more, M, N, device=DEV) if n_more else None
                    m2 = torch.zeros(n_more, M, N, device=DEV) if n_more else None
                    lib.gemm_mfma(a, w, x1, lib.EPI_ADD, more_slices=m1, shape=shape)
                    lib.gemm_mfma(a, once, x2, lib.EPI_ADD, more_slices=m2, shape=shape)
                    assert torch.equal(x1, x2) and (m1 is None or torch.equal(m1, m2)), (how, M, shape, n_more)
        for M in (1, 8, 12):                                # the products of few rows, in the strips the copy has
            a = dev(rounded(rng.standard_normal((M, Kd)), "bfloat16"), torch.bfloat16)
            rows = 8 if how == "strips of 8" else 16
            res = rng.standard_normal((M, N)).astype(np.float32)
            if lib.skinny_takes(once, M, rows):
                x1, x2 = dev(res), dev(res)
                lib.gemm_skinny(a, w if rows == 16 else w8, x1, lib.EPI_ADD, strip_rows=rows)
                lib.gemm_skinny(a, once, x2, lib.EPI_ADD, strip_rows=rows)
                assert torch.equal(x1, x2), (how, M, "skinny")
            else:
                assert rows == 8 and M > 8
                with pytest.raises(lib.KernelError, match="matrix cores' order alone"):
                    lib.gemm_skinny(a, once, dev(res), lib.EPI_ADD, strip_rows=rows)


@pytest.mark.parametrize("pairing", ["adjacent", "half", None])
@pytest.mark.parametrize("H, Kh, hs, d", [(32, 8, 64, 128), (6, 2, 16, 64), (5, 5, 48, 3200), (8, 1, 128, 4096)])
def test_stacked_qkv_rows_kept_in_operand_order_alone(pairing, H, Kh, hs, d):
    """The stacked q, k, v rows held once, as the copy whose strips pair up what the rotation's end pairs: the fused
    product of 1 to 64 rows (the kernels of few rows, and the kernel of whole lines for 17 rows and more and for a
    folded norm over a long K), and the plain product through the tiled and the generic kernels, which find each
    row's place in the copy, all give what the stored rows give, bit for bit."""
    rng = np.random.default_rng(hs + H + d)
    lib = K()
    page = 64
    N = (H + 2 * Kh) * hs
    w = dev(rounded(rng.standard_normal((N, d)) / math.sqrt(d), "bfloat16"), torch.bfloat16)
    wq = w.clone()
    wq.tiled = lib.tile_weight(wq, qkv=(H, Kh, hs, pairing is not None, pairing == "adjacent"))
    once = lib.hold_once(wq)
    assert torch.equal(lib.stored_order(once), w)
    cos, sin = P.rope_table(256, hs, 50000.0)
    nw = rounded(1 + 0.2 * rng.standard_normal(d), "bfloat16")
    for T in (7, 16, 30, 64):
        x = (rng.standard_normal((T, d)) * 2).astype(np.float32)
        positions = rng.integers(0, 200, T)
        zk = [np.zeros((b + 1, Kh, hs), np.float32) for b in positions]
        for folded in ((True, False) if T <= 16 else (False,)):
            got = []
            for weight in (w, once):
                kc, vc, table = paged(zk, zk, Kh, hs, page, "bfloat16", np.random.default_rng(1))
                q_out = torch.zeros(T, H * hs, device=DEV, dtype=torch.bfloat16)
                rows = times_weight(x, nw).to(DEV) if folded else dev(rounded(x, "bfloat16"), torch.bfloat16)
                lib.qkv_rope_cache(rows, dev(ssq_partials(x, 6)) if folded else None, 6 if folded else 0, 1e-5, weight, q_out,
                                   dev(positions, torch.int32), dev(np.arange(T), torch.int32), table,
                                   dev(cos) if pairing else None, dev(sin) if pairing else None, kc, vc, H, Kh, hs,
                                   pairing == "adjacent", page)
                got.append((q_out, kc, vc))
            for u, v in zip(*got):
                assert torch.equal(u, v), (T, folded)
    for M in (3, 200):
        a = dev(rounded(rng.standard_normal((M, d)), "bfloat16"), torch.bfloat16)
        g1, g2 = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16), torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
        lib.gemm_generic(a, w, g1); lib.gemm_generic(a, once, g2)
        assert torch.equal(g1, g2)
        for shape in (0, 1, 2, 5):
            m1, m2 = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16), torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
            lib.gemm_mfma(a, w, m1, shape=shape); lib.gemm_mfma(a, once, m2, shape=shape)
            assert torch.equal(m1, m2), (M, shape)
    a = dev(rounded(rng.standard_normal((4, d)), "bfloat16"), torch.bfloat16)
    if pairing == "half" and hs > 16:                       # (rows in another order: the plain products of few rows cannot read it)
        assert not lib.skinny_takes(once, 4, 16)
        with pytest.raises(lib.KernelError, match="matrix cores' order alone"):
            lib.gemm_skinny(a, once, torch.zeros(4, N, device=DEV))


@pytest.mark.parametrize("N, Kd", [(2048, 2048), (2048, 8192), (40, 72), (136, 1544), (3072, 200)])
@pytest.mark.parametrize("M", [1, 5, 8])
def test_strips_of_eight_rows_read_a_weight_copy_in_their_tiles_order(M, N, Kd):
    """``tile_weight8``: [strip of 8 rows][step of 64 k][lane][8], lane 16 q + r holding row r % 8 at
    k = 32 (r // 8) + 8 q. The products of at most 8 rows into the residual stream read it; same sums."""
    rng = np.random.default_rng(M + N + Kd)
    lib = K()
    wn = rounded(rng.standard_normal((N, Kd)) / math.sqrt(Kd), "bfloat16")
    w = dev(wn, torch.bfloat16)
    t = lib.tile_weight8(w)
    steps = -(-Kd // 64)
    flat = t.reshape(-1).float().cpu().numpy()
    for (n, k) in [(0, 0), (17, 9), (N - 1, Kd - 1), (5, Kd // 2), (31, 40 % Kd), (12, 63 % Kd)]:
        strip, row, step, half, q, e = n // 8, n % 8, k // 64, (k % 64) // 32, (k % 32) // 8, k % 8
        assert flat[((strip * steps + step) * 64 + q * 16 + half * 8 + row) * 8 + e] == wn[n, k]
    a = dev(rounded(rng.standard_normal((M, Kd)), "bfloat16"), torch.bfloat16)
    res0 = rng.standard_normal((M, N)).astype(np.float32)
    got = {}
    for tiled in (False, True):
        if tiled:
            w.tiled8 = t
        x = dev(res0)
        ssq = torch.zeros(N // 8, 64, device=DEV)
        lib.gemm_skinny(a, w, x, lib.EPI_ADD, strip_rows=8, ssq_out=ssq if N % 16 == 0 else None)
        s_ = torch.zeros(M, N, device=DEV)
        lib.gemm_skinny(a, w, s_, lib.EPI_STORE, strip_rows=8)
        got[tiled] = (x, ssq, s_)
    for u, v in zip(got[False], got[True]):
        assert torch.equal(u, v)
    np.testing.assert_allclose(got[True][2].cpu().numpy(), P.linear(a.float().cpu().numpy(), wn), atol=2e-5 * Kd)


@pytest.mark.parametrize("d, F", [(2048, 8192), (64, 200), (136, 72), (96, 1544)])
@pytest.mark.parametrize("M", [1, 5, 8])
def test_rows_handed_over_in_the_packed_order(M, d, F):
    """A gated product that leaves its rows in the order of the packed tiles (``pack_out``) and a product of
    strips of 8 weight rows that reads them there (``a_packed``) give what the two give through plain rows."""
    rng = np.random.default_rng(M + d + F)
    lib = K()
    x = (rng.standard_normal((M, d)) * 2).astype(np.float32)
    nw = rounded(1 + 0.2 * rng.standard_normal(d), "bfloat16")
    w1 = dev(rounded(rng.standard_normal((2 * F, d)) / math.sqrt(d), "bfloat16"), torch.bfloat16)
    w2 = dev(rounded(rng.standard_normal((d, F)) / math.sqrt(F), "bfloat16"), torch.bfloat16)
    xg, ssq = times_weight(x, nw).to(DEV), dev(ssq_partials(x, 4))
    res0 = rng.standard_normal((M, d)).astype(np.float32)
    act = torch.zeros(M, F, device=DEV, dtype=torch.bfloat16)
    lib.gemm_skinny_norm(xg, ssq, 4, 1e-5, w1, act, lib.EPI_GATED)
    plain = dev(res0)
    lib.gemm_skinny(act, w2, plain, lib.EPI_ADD, strip_rows=8)
    packed = lib.packed_rows(F, torch.bfloat16, DEV)
    packed.fill_(777.0)                                                      # what is not written is not read
    lib.gemm_skinny_norm(xg, ssq, 4, 1e-5, w1, packed, lib.EPI_GATED, pack_out=True)
    flat = packed.reshape(-1).float().cpu().numpy()
    an = act.float().cpu().numpy()
    for (m, k) in [(0, 0), (M - 1, F - 1), (M // 2, F // 2), (0, 37 % F), (M - 1, 63 % F)]:
        assert flat[(((k // 64) * 64 + ((k % 32) // 8) * 16 + ((k % 64) // 32) * 8 + m) * 8) + k % 8] == an[m, k]
    for tiled in (False, True):
        if tiled:
            w2.tiled8 = lib.tile_weight8(w2)
        got = dev(res0)
        lib.gemm_skinny(packed, w2, got, lib.EPI_ADD, strip_rows=8, a_packed=True)
        assert torch.equal(got, plain)
    with pytest.raises(lib.KernelError):
        lib.gemm_skinny(packed, w2, dev(res0), lib.EPI_ADD, strip_rows=16, a_packed=True)

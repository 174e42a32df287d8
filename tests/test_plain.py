"""Pins of the plain implementation: what fixes each formula beside the reference's text.

The reference holds no test vectors (it has no tests at all), so each part is
fixed by a special case that reduces to a library routine and by invariants
chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong
place, the wrong kv head) fails.
"""
import math

import numpy as np
import pytest
import torch

import plain_llama as P
from tiny import TINY_A, TINY_B, TINY_C, TINY_D, dims, make_weights, tokens


# ------------------------------------------------------------------ rmsnorm
def test_rmsnorm_is_the_library_formula():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 96)).astype(np.float32) * 3
    w = (1 + 0.1 * rng.standard_normal(96)).astype(np.float32)
    xt = torch.from_numpy(x)
    ref = xt * torch.rsqrt(xt.pow(2).mean(-1, keepdim=True) + 1e-6) * torch.from_numpy(w)
    np.testing.assert_allclose(P.rmsnorm(x, w, 1e-6), ref.numpy(), rtol=2e-6, atol=1e-7)


def test_rmsnorm_invariants():
    rng = np.random.default_rng(1)
    x = rng.standard_normal(64).astype(np.float32)
    one = np.ones(64, np.float32)
    y = P.rmsnorm(x, one, 0.0)
    assert abs(np.mean(y * y) - 1) < 1e-5              # unit mean square, no mean subtraction
    np.testing.assert_allclose(P.rmsnorm(7.5 * x, one, 0.0), y, rtol=1e-5)
    assert np.all(P.rmsnorm(np.zeros(64, np.float32), one, 1e-5) == 0)   # eps keeps 0 finite
    # weight multiplies (w), it is not (1 + w)
    np.testing.assert_allclose(P.rmsnorm(x, 2 * one, 0.0), 2 * y, rtol=1e-6)
    # eps sits inside the root, after the mean
    big = P.rmsnorm(x, one, 3.0)
    np.testing.assert_allclose(big, x / math.sqrt(np.mean(x * x) + 3.0), rtol=1e-5)


# ------------------------------------------------------------------ rope
def test_rope_frequencies_without_scaling():
    f = P.rope_frequencies(16, 10000.0)
    np.testing.assert_allclose(f, 10000.0 ** (-np.arange(0, 16, 2) / 16), rtol=1e-6)
    assert f[0] == 1.0


def test_rope_scaling_factor_one_is_identity_and_branches():
    sc = dict(factor=1.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    np.testing.assert_allclose(P.rope_frequencies(32, 5e5, sc), P.rope_frequencies(32, 5e5), rtol=1e-6)
    sc = TINY_B["rope_scaling"]
    base = P.rope_frequencies(32, 5e5)
    got = P.rope_frequencies(32, 5e5, sc)
    wavelen = 2 * math.pi / base
    hi_w, lo_w = 64 / 4.0, 64 / 1.0
    kept = wavelen < hi_w
    divided = wavelen > lo_w
    mid = ~kept & ~divided
    assert kept.any() and divided.any() and mid.any()      # all three branches occur
    np.testing.assert_array_equal(got[kept], base[kept])   # high frequencies untouched
    np.testing.assert_allclose(got[divided], base[divided] / 8.0, rtol=1e-6)
    assert np.all(got[mid] < base[mid]) and np.all(got[mid] > base[mid] / 8.0)


def _scaled_over_base(fn, wavelen, sc):
    """``fn``'s scaled frequency over the unscaled one for a head of 4 whose second pair has the
    wavelength ``wavelen``: theta is chosen so that ``theta ** -0.5 == 2 pi / wavelen``."""
    theta = (wavelen / (2 * math.pi)) ** 2
    return float(fn(4, theta, sc)[1]) / float(fn(4, theta, None)[1])


# J/inference/operation/RoPE.java:20-27 worked by hand for old=64, lo=1, hi=4 (the band is 16..64):
# smooth = (old/wavelen - lo)/(hi - lo); scaled/base = (1 - smooth)/factor + smooth.
#   wavelen 32   -> old/wavelen 2   -> smooth 1/3 -> (2/3)/8 + 1/3 = 5/12
#   wavelen 25.6 -> old/wavelen 2.5 -> smooth 1/2 -> (1/2)/8 + 1/2 = 9/16
#   wavelen 64/3 -> old/wavelen 3   -> smooth 2/3 -> (1/3)/8 + 2/3 = 17/24
# (smooth and 1 - smooth exchanged would give 17/24, 9/16, 5/12: the first and last tell them apart)
# and for factor 32, old 8192 (the band is 2048..8192): wavelen 4096 -> smooth 1/3 -> (2/3)/32 + 1/3 = 17/48.
SC_8 = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
SC_32 = dict(factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)
HAND_VALUES = [(SC_8, 32.0, 5 / 12), (SC_8, 25.6, 9 / 16), (SC_8, 64 / 3, 17 / 24), (SC_32, 4096.0, 17 / 48)]


@pytest.mark.parametrize("sc, wavelen, expect", HAND_VALUES)
def test_rope_interpolation_at_points_worked_by_hand(sc, wavelen, expect):
    assert abs(_scaled_over_base(P.rope_frequencies, wavelen, sc) - expect) < 2e-6


def test_rope_interpolation_falls_from_one_to_one_over_factor_across_the_band():
    # through the function itself: continuous at both edges of the band, monotone inside it, and
    # linear in the frequency (smooth is linear in old/wavelen = old * freq / 2 pi)
    ratio = lambda w: _scaled_over_base(P.rope_frequencies, w, SC_8)
    assert ratio(15.99) == 1.0 and abs(ratio(16.01) - 1.0) < 1e-3            # old/hi = 16
    assert abs(ratio(63.99) - 1 / 8) < 1e-4 and abs(ratio(64.01) - 1 / 8) < 1e-6   # old/lo = 64
    ws = np.linspace(16.5, 63.5, 48)
    rs = np.array([ratio(w) for w in ws])
    assert np.all(np.diff(rs) < 0) and rs[0] < 1.0 and rs[-1] > 1 / 8
    fs = 64.0 / ws                                                           # old/wavelen
    np.testing.assert_allclose(rs, (1 - (fs - 1) / 3) / 8 + (fs - 1) / 3, atol=2e-6)


def _library_forward(cfg, W, toks):
    """The whole model out of library routines only (torch's rms_norm, scaled_dot_product_attention,
    silu, complex multiplication for the rotation), float64: an implementation that shares no line
    with ``plain_llama.forward``. Adjacent pairing rotates the complex numbers (x[2j], x[2j+1]),
    half pairing (x[j], x[j + hs/2]). The frequencies are ``P.rope_frequencies``, pinned above."""
    import torch.nn.functional as F
    d, H, K, hs, Fdim, V, L = dims(cfg)
    t = lambda n: torch.from_numpy(np.asarray(W[n])).double()
    T = len(toks)
    freq = torch.from_numpy(P.rope_frequencies(hs, cfg.get("rope_theta", 10000.0), cfg.get("rope_scaling"))).double()
    ang = torch.arange(T, dtype=torch.float64)[:, None] * freq[None, :]
    rot = torch.polar(torch.ones_like(ang), ang)                             # [T, hs/2]
    adjacent = cfg.get("rope_pairing", "half") == "adjacent"

    def rotate(x):                                                           # [T, heads, hs]
        pairs = x.reshape(T, -1, hs // 2, 2) if adjacent else torch.stack((x[..., :hs // 2], x[..., hs // 2:]), -1)
        z = torch.view_as_real(torch.view_as_complex(pairs.contiguous()) * rot[:, None, :])
        return z.reshape(T, -1, hs) if adjacent else torch.cat((z[..., 0], z[..., 1]), -1)

    eps = cfg.get("rms_norm_eps", 1e-5)
    x = t("model.embed_tokens.weight")[torch.tensor(toks)]
    for i in range(L):
        n = P.layer_names(i)
        h = F.rms_norm(x, (d,), t(n["attn_norm"]), eps)
        q = rotate((h @ t(n["q"]).T).reshape(T, H, hs)).transpose(0, 1)     # [H, T, hs]
        k = rotate((h @ t(n["k"]).T).reshape(T, K, hs)).transpose(0, 1)
        v = (h @ t(n["v"]).T).reshape(T, K, hs).transpose(0, 1)
        k, v = k.repeat_interleave(H // K, 0), v.repeat_interleave(H // K, 0)
        a = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
        x = x + a.transpose(0, 1).reshape(T, H * hs) @ t(n["o"]).T
        h = F.rms_norm(x, (d,), t(n["ffn_norm"]), eps)
        x = x + (F.silu(h @ t(n["gate"]).T) * (h @ t(n["up"]).T)) @ t(n["down"]).T
    head = t("model.embed_tokens.weight") if cfg.get("tie_word_embeddings", False) else t("lm_head.weight")
    return (F.rms_norm(x, (d,), t("model.norm.weight"), eps) @ head.T).numpy()


@pytest.mark.parametrize("cfg", [TINY_A, {**TINY_A, "rope_pairing": "half"}, TINY_B, TINY_C, TINY_D],
                         ids=["A", "A-half", "B", "C", "D"])
def test_whole_model_is_a_composition_of_library_routines(cfg):
    W = make_weights(cfg, 21, norm_std=0.1)
    toks = tokens(cfg, 21, 29)
    got = P.forward(cfg, W, toks)
    want = _library_forward(cfg, W, toks)
    scale = float(np.abs(want).max())
    assert float(np.abs(got - want).max()) < 3e-6 * scale


def test_rope_rotation_is_a_complex_multiplication():
    rng = np.random.default_rng(2)
    T, H, hs = 7, 3, 32
    q = rng.standard_normal((T, H, hs)).astype(np.float32)
    pos = np.array([0, 1, 2, 5, 9, 30, 31])
    cos, sin = P.rope_table(32, hs, 5e5, TINY_B["rope_scaling"])
    freq = P.rope_frequencies(hs, 5e5, TINY_B["rope_scaling"])
    ang = torch.from_numpy((pos[:, None].astype(np.float32) * freq[None]).astype(np.float32))
    z = torch.view_as_complex(torch.from_numpy(q).reshape(T, H, hs // 2, 2).contiguous())
    ref = torch.view_as_real(z * torch.polar(torch.ones_like(ang), ang)[:, None, :]).reshape(T, H, hs)
    np.testing.assert_allclose(P.rope_rotate(q, pos, cos, sin, "adjacent"), ref.numpy(), atol=2e-6)


@pytest.mark.parametrize("pairing", ["adjacent", "half"])
def test_rope_invariants(pairing):
    rng = np.random.default_rng(3)
    hs = 16
    cos, sin = P.rope_table(200, hs, 10000.0)
    q = rng.standard_normal((1, 1, hs)).astype(np.float32)
    k = rng.standard_normal((1, 1, hs)).astype(np.float32)
    np.testing.assert_array_equal(P.rope_rotate(q, np.array([0]), cos, sin, pairing), q)  # p = 0
    r = P.rope_rotate(q, np.array([13]), cos, sin, pairing)
    np.testing.assert_allclose(np.linalg.norm(r), np.linalg.norm(q), rtol=1e-6)
    # only the distance counts, and its sign matters
    def score(m, n):
        return float(np.sum(P.rope_rotate(q, np.array([m]), cos, sin, pairing)
                            * P.rope_rotate(k, np.array([n]), cos, sin, pairing)))
    assert abs(score(17, 5) - score(112, 100)) < 1e-4
    assert abs(score(17, 5) - score(5, 17)) > 1e-3


def test_pairings_are_linked_by_the_row_permutation():
    cfg = dict(TINY_B)
    W = make_weights(cfg, 5, norm_std=0.1)
    toks = tokens(cfg, 5, 23)
    d, H, K, hs, F, V, L = dims(cfg)
    half = P.forward({**cfg, "rope_pairing": "half"}, W, toks)
    W2 = dict(W)
    for i in range(L):
        n = P.layer_names(i)
        W2[n["q"]] = P.interleave_rows(W[n["q"]], H, hs)
        W2[n["k"]] = P.interleave_rows(W[n["k"]], K, hs)
    adj = P.forward({**cfg, "rope_pairing": "adjacent"}, W2, toks)
    np.testing.assert_allclose(adj, half, atol=2e-6)
    # and without the permutation the two differ: the pairing is not a no-op
    assert np.abs(P.forward({**cfg, "rope_pairing": "adjacent"}, W, toks) - half).max() > 1e-4


# ------------------------------------------------------------------ attention
def test_attention_is_library_sdpa_with_repeated_kv_heads():
    rng = np.random.default_rng(4)
    T, H, K, hs = 19, 6, 2, 16
    q = rng.standard_normal((T, H, hs)).astype(np.float32)
    k = rng.standard_normal((T, K, hs)).astype(np.float32)
    v = rng.standard_normal((T, K, hs)).astype(np.float32)
    tq = torch.from_numpy(q).transpose(0, 1)
    tk = torch.from_numpy(k).transpose(0, 1).repeat_interleave(H // K, 0)
    tv = torch.from_numpy(v).transpose(0, 1).repeat_interleave(H // K, 0)
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True)
    np.testing.assert_allclose(P.attention(q, k, v), ref.transpose(0, 1).numpy(), atol=2e-6)


def test_attention_special_cases():
    rng = np.random.default_rng(5)
    T, H, K, hs = 9, 4, 2, 16
    q = rng.standard_normal((T, H, hs)).astype(np.float32)
    k = rng.standard_normal((T, K, hs)).astype(np.float32)
    v = rng.standard_normal((T, K, hs)).astype(np.float32)
    out = P.attention(q, k, v)
    # first token sees itself only: out = v of its kv head (h // g, not h % K)
    for h in range(H):
        np.testing.assert_allclose(out[0, h], v[0, h // 2], atol=1e-7)
    # equal keys -> running mean of the values
    same = np.broadcast_to(k[:1], k.shape).copy()
    m = P.attention(q, same, v)
    np.testing.assert_allclose(m[5, 3], v[:6, 1].mean(0), atol=1e-6)
    # causality: a change of a later token leaves earlier rows alone
    k2, v2 = k.copy(), v.copy()
    k2[6:] += 1.0
    v2[6:] -= 2.0
    np.testing.assert_array_equal(P.attention(q, k2, v2)[:6], out[:6])
    # scale is 1/sqrt(hs): with one dominant key the weight follows exp(q.k/sqrt(hs))
    q1 = np.zeros((2, 1, 16), np.float32); q1[1, 0, 0] = 4.0
    k1 = np.zeros((2, 1, 16), np.float32); k1[1, 0, 0] = 2.0
    v1 = np.zeros((2, 1, 16), np.float32); v1[1, 0, 0] = 1.0
    w = P.attention(q1, k1, v1)[1, 0, 0]
    assert abs(w - math.exp(2.0) / (1 + math.exp(2.0))) < 1e-6
    # window keeps the last w keys only
    win = P.attention(q, k, v, window=3)
    np.testing.assert_allclose(win[:3], out[:3], atol=1e-7)
    assert np.abs(win[8] - out[8]).max() > 1e-4
    np.testing.assert_allclose(win[8], P.attention(q[6:], k[6:], v[6:])[2], atol=1e-6)


def test_softmax_rows_sum_to_one_and_ignore_a_shift():
    x = np.array([[1.0, 2.0, 3.0], [1000.0, 1001.0, 999.0]], np.float32)
    s = P.softmax(x)
    np.testing.assert_allclose(s.sum(-1), 1.0, rtol=1e-6)
    np.testing.assert_allclose(P.softmax(x + 50.0), s, rtol=1e-5)


# ------------------------------------------------------------------ feed-forward
def test_silu_glu():
    x = np.array([0.0, 30.0, -30.0, -200.0, 1.5], np.float32)
    s = P.silu(x)
    assert s[0] == 0 and abs(s[1] - 30) < 1e-5 and abs(s[2]) < 1e-10 and s[3] == 0 and np.isfinite(s).all()
    np.testing.assert_allclose(s, torch.nn.functional.silu(torch.from_numpy(x)).numpy(), atol=1e-6)
    rng = np.random.default_rng(6)
    xx = rng.standard_normal((3, 8)).astype(np.float32)
    g, u, dn = (rng.standard_normal(s).astype(np.float32) for s in ((12, 8), (12, 8), (8, 12)))
    t = torch.from_numpy
    ref = torch.nn.functional.linear(torch.nn.functional.silu(torch.nn.functional.linear(t(xx), t(g)))
                                     * torch.nn.functional.linear(t(xx), t(u)), t(dn))
    np.testing.assert_allclose(P.feed_forward(xx, g, u, dn), ref.numpy(), atol=1e-5)
    # gate and up are not interchangeable
    assert np.abs(P.feed_forward(xx, u, g, dn) - ref.numpy()).max() > 1e-3


# ------------------------------------------------------------------ whole model
@pytest.mark.parametrize("cfg", [TINY_A, TINY_B, TINY_C, TINY_D], ids=["A", "B", "C", "D"])
def test_zero_output_projections_leave_the_embedding(cfg):
    W = make_weights(cfg, 7, norm_std=0.1)
    for i in range(cfg["num_hidden_layers"]):
        n = P.layer_names(i)
        W[n["o"]][:] = 0
        W[n["down"]][:] = 0
    toks = tokens(cfg, 7, 9)
    E = W["model.embed_tokens.weight"]
    head = E if cfg["tie_word_embeddings"] else W["lm_head.weight"]
    ref = P.rmsnorm(E[toks], W["model.norm.weight"], cfg["rms_norm_eps"]) @ head.T
    np.testing.assert_allclose(P.forward(cfg, W, toks), ref, atol=1e-6)


def test_tied_head_is_an_untied_copy():
    W = make_weights(TINY_A, 8)
    toks = tokens(TINY_A, 8, 11)
    tied = P.forward(TINY_A, W, toks)
    W2 = dict(W); W2["lm_head.weight"] = W["model.embed_tokens.weight"].copy()
    np.testing.assert_array_equal(P.forward({**TINY_A, "tie_word_embeddings": False}, W2, toks), tied)


def test_prefix_logits_do_not_depend_on_later_tokens():
    W = make_weights(TINY_B, 9, norm_std=0.1)
    toks = tokens(TINY_B, 9, 30)
    full = P.forward(TINY_B, W, toks)
    np.testing.assert_allclose(P.forward(TINY_B, W, toks[:12]), full[:12], atol=1e-6)


def test_shifting_all_positions_changes_nothing_without_scaling():
    # a norm placed after the rotation, or a rotation of v, would break this
    W = make_weights(TINY_A, 10, std=0.3)
    toks = tokens(TINY_A, 10, 20)
    np.testing.assert_allclose(P.forward(TINY_A, W, toks, position_offset=57), P.forward(TINY_A, W, toks), atol=2e-4)


def test_schedule_default_and_repeats():
    W = make_weights(TINY_A, 11, std=0.2)
    toks = tokens(TINY_A, 11, 10)
    base = P.forward(TINY_A, W, toks)
    np.testing.assert_array_equal(P.forward(TINY_A, W, toks, schedule=[(0, None), (1, None)]), base)
    again = P.forward(TINY_A, W, toks, schedule=[(0, None), (1, None), (1, None)])
    shared = P.forward(TINY_A, W, toks, schedule=[(0, None), (1, None), (1, 1)])
    assert np.abs(again - base).max() > 1e-4 and np.abs(shared - again).max() > 1e-5


# ------------------------------------------------------------------ sampling
def test_argmax_first_of_ties():
    assert P.argmax(np.array([1.0, 5.0, 5.0, 2.0], np.float32)) == 1


def test_top_p_matches_sort_and_cumsum():
    rng = np.random.default_rng(12)
    logits = rng.standard_normal(50).astype(np.float32) * 2
    p = P.probabilities(logits, 0.8)
    order = np.argsort(-p.astype(np.float64), kind="stable")
    csum = np.cumsum(p[order].astype(np.float64))
    n_keep = int(np.argmax(csum > 0.9)) + 1
    kept, mass = P.top_p_set(p, 0.9)
    assert kept == order[:n_keep].tolist() and abs(mass - csum[n_keep - 1]) < 1e-12
    assert csum[n_keep - 1] > 0.9 and (n_keep == 1 or csum[n_keep - 2] <= 0.9)   # smallest prefix exceeding p
    for r in (0.0, 0.3, 0.77, 0.999999):
        tok = P.sample_top_p(p, 0.9, r)
        j = kept.index(tok)
        before = csum[j - 1] if j else 0.0
        assert before <= r * mass < csum[j]


def test_sampler_modes():
    rng = np.random.default_rng(13)
    logits = rng.standard_normal(40).astype(np.float32)
    assert P.sample(logits, 0.0, 0.95, 0.5) == int(np.argmax(logits))
    assert P.sample(logits, 1e-4, 0.0, 0.5) == int(np.argmax(logits))          # T -> 0+
    assert P.sample(logits, 1.0, 1e-6, 0.9) == int(np.argmax(logits))          # tiny top-p
    p = P.probabilities(logits, 1.0)
    for r in (0.1, 0.6, 0.95):
        assert P.sample(logits, 1.0, 1.0, r) == P.sample_categorical(p, r) == P.sample(logits, 1.0, 0.0, r)
    # frequencies follow the probabilities
    draws = np.random.default_rng(14).random(20000)
    counts = np.bincount([P.sample_categorical(p, r) for r in draws], minlength=40)
    chi2 = np.sum((counts - 20000 * p) ** 2 / (20000 * p))
    assert chi2 < 90    # 39 degrees of freedom: mean 39, this is far in the tail

"""Plain, slow Llama 3 in numpy: whole sequences, no cache, one function per part.

Written from the formulas of the reference's CPU path (the numerically
authoritative text). ``J/`` below stands for
``src/main/java/org/beehive/gpullama3/`` of the reference. Nothing here is
shared with the product path: it is the oracle the engine is compared with.

Every array is float32 unless said otherwise; where the reference evaluates a
transcendental in double and casts to float, so does this file.
"""
from __future__ import annotations

import math

import numpy as np

F32 = np.float32


# --------------------------------------------------------------------------- norms
def rmsnorm(x, weight, eps):
    """``out_i = w_i * (ss * x_i)``, ``ss = 1/sqrt(mean(x^2) + eps)``.

    J/inference/InferenceCore.java:47-56 (sum of squares, ``/= size``,
    ``+= eps``, ``1/sqrt`` in double cast to float, weight multiplies the
    normalised value directly, no ``1 + w``, no mean subtraction).
    Works on the last axis of ``x``.
    """
    x = np.asarray(x, dtype=F32)
    ss = np.sum(x * x, axis=-1, keepdims=True, dtype=F32)
    ss = ss / F32(x.shape[-1])
    ss = ss + F32(eps)
    ss = (1.0 / np.sqrt(ss.astype(np.float64))).astype(F32)
    return np.asarray(weight, dtype=F32) * (ss * x)


# --------------------------------------------------------------------------- rope
def rope_frequencies(head_size, theta, scaling=None):
    """Per-pair rotation frequency, float32 ``[head_size/2]``.

    J/inference/operation/RoPE.java:13-28: ``freq = 1/theta^(i/hs)`` for even
    ``i`` (pow in double, cast to float); with the llama3 rule a wavelength
    below ``old/hi`` keeps its frequency, above ``old/lo`` is divided by the
    factor, and in between is interpolated with
    ``smooth = (old/wavelen - lo)/(hi - lo)``.
    ``scaling`` is ``None`` or a dict with ``factor``, ``low_freq_factor``,
    ``high_freq_factor``, ``original_max_position_embeddings`` (the reference
    fixes 8, 1, 3, 8192 in J/model/loader/ModelLoader.java:235-239; here they
    are parameters).
    """
    assert head_size % 2 == 0
    out = np.zeros(head_size // 2, dtype=F32)
    for n, i in enumerate(range(0, head_size, 2)):
        freq = F32(1.0 / math.pow(float(theta), i / float(head_size)))
        if scaling is not None:
            scale = F32(scaling["factor"])
            lo = F32(scaling["low_freq_factor"])
            hi = F32(scaling["high_freq_factor"])
            old = F32(scaling["original_max_position_embeddings"])
            lo_wavelen = F32(old / lo)
            hi_wavelen = F32(old / hi)
            wavelen = F32(2.0 * math.pi / float(freq))
            if wavelen < hi_wavelen:
                pass
            elif wavelen > lo_wavelen:
                freq = F32(freq / scale)
            else:
                smooth = F32(F32(F32(old / wavelen) - lo) / F32(hi - lo))
                freq = F32(F32(F32(F32(1.0) - smooth) * freq / scale) + F32(smooth * freq))
        out[n] = freq
    return out


def rope_table(n_positions, head_size, theta, scaling=None):
    """cos and sin tables ``[n_positions, head_size/2]``.

    J/inference/operation/RoPE.java:29-31: the angle is ``pos * freq`` in
    float; cos and sin are evaluated in double on that float and cast.
    """
    freq = rope_frequencies(head_size, theta, scaling)
    pos = np.arange(n_positions, dtype=F32)[:, None]
    val = (pos * freq[None, :]).astype(F32)
    return np.cos(val.astype(np.float64)).astype(F32), np.sin(val.astype(np.float64)).astype(F32)


def rope_rotate(vec, positions, cos, sin, pairing="adjacent"):
    """Rotate ``vec [T, heads, hs]`` by the angles of ``positions [T]``.

    J/inference/InferenceCore.java:83-95: within each head the pair
    ``(2j, 2j+1)`` is rotated by the table entry ``j``:
    ``v0' = v0*c - v1*s``, ``v1' = v0*s + v1*c``. ``pairing="half"`` pairs
    ``(j, j + hs/2)`` instead, which is what the same weights need when their
    q/k rows are stored de-interleaved (the two are linked by a row
    permutation, see ``interleave_rows``).
    """
    vec = np.asarray(vec, dtype=F32)
    hs = vec.shape[-1]
    c = cos[positions][:, None, :]  # [T,1,hs/2]
    s = sin[positions][:, None, :]
    out = np.empty_like(vec)
    if pairing == "adjacent":
        v0, v1 = vec[..., 0::2], vec[..., 1::2]
        out[..., 0::2] = v0 * c - v1 * s
        out[..., 1::2] = v0 * s + v1 * c
    elif pairing == "half":
        v0, v1 = vec[..., : hs // 2], vec[..., hs // 2:]
        out[..., : hs // 2] = v0 * c - v1 * s
        out[..., hs // 2:] = v0 * s + v1 * c
    else:
        raise ValueError(pairing)
    return out


def interleave_rows(w, n_heads, head_size):
    """Row permutation that turns half-split q/k weights into adjacent-pair ones.

    ``new_row[2j] = old_row[j]``, ``new_row[2j+1] = old_row[j + hs/2]`` within
    every head. A model with ``pairing="half"`` and ``w`` equals a model with
    ``pairing="adjacent"`` and ``interleave_rows(w)``.
    """
    w = np.asarray(w)
    rest = w.shape[1:]
    w = w.reshape(n_heads, 2, head_size // 2, *rest)
    w = np.swapaxes(w, 1, 2)
    return np.ascontiguousarray(w).reshape(n_heads * head_size, *rest)


# --------------------------------------------------------------------------- attention
def softmax(x):
    """J/core/model/tensor/FloatTensor.java:211-219: subtract the max, exp
    (double, cast to float), sum, divide. Last axis."""
    x = np.asarray(x, dtype=F32)
    m = np.max(x, axis=-1, keepdims=True)
    e = np.exp((x - m).astype(np.float64)).astype(F32)
    return e / np.sum(e, axis=-1, keepdims=True, dtype=F32)


def attention(q, k, v, window=None, scale=None):
    """Causal grouped-query attention over one whole sequence.

    ``q [T, H, hs]``, ``k, v [T, K, hs]`` (k already rotated) -> ``[T, H, hs]``.
    J/inference/InferenceCore.java:106-145: query head ``h`` uses kv head
    ``h // (H/K)``; ``score_t = dot(q, k_t) / sqrt(hs)`` for ``t <= p`` (the
    mask is the loop bound), softmax over those, weighted sum of the values.
    ``window`` (not in the reference: every Llama 3 layer sees all keys)
    keeps only the last ``window`` keys, ``t > p - window``.
    """
    q = np.asarray(q, dtype=F32)
    T, H, hs = q.shape
    K = k.shape[1]
    g = H // K
    out = np.zeros((T, H, hs), dtype=F32)
    div = F32(math.sqrt(hs)) if scale is None else None
    for h in range(H):
        c = h // g
        for p in range(T):
            lo = 0 if window is None else max(0, p - window + 1)
            keys = k[lo:p + 1, c, :].astype(F32)
            score = keys @ q[p, h, :]
            score = score / div if scale is None else score * F32(scale)
            a = softmax(score)
            out[p, h, :] = a @ v[lo:p + 1, c, :].astype(F32)
    return out


# --------------------------------------------------------------------------- feed-forward
def silu(x):
    """``x / (1 + exp(-x))`` with exp in double cast to float
    (J/inference/InferenceCore.java:163)."""
    x = np.asarray(x, dtype=F32)
    with np.errstate(over="ignore"):
        return x / (1.0 + np.exp(-x.astype(np.float64))).astype(F32)


def feed_forward(x, w_gate, w_up, w_down):
    """``W2 . (silu(W1 . x) * (W3 . x))`` (J/inference/InferenceCore.java:158-169).
    Matrices are row-major ``[out, in]`` (J/core/model/tensor/FloatTensor.java:98-100)."""
    hb = linear(x, w_gate)
    hb2 = linear(x, w_up)
    return linear(silu(hb) * hb2, w_down)


def linear(x, w):
    """``out[i] = sum_j W[i, j] * x[j]``, no bias
    (J/core/model/tensor/FloatTensor.java:98-100)."""
    return np.asarray(x, dtype=F32) @ np.asarray(w, dtype=F32).T


# --------------------------------------------------------------------------- whole model
def layer_names(i):
    p = f"model.layers.{i}."
    return {
        "attn_norm": p + "input_layernorm.weight",
        "q": p + "self_attn.q_proj.weight",
        "k": p + "self_attn.k_proj.weight",
        "v": p + "self_attn.v_proj.weight",
        "o": p + "self_attn.o_proj.weight",
        "ffn_norm": p + "post_attention_layernorm.weight",
        "gate": p + "mlp.gate_proj.weight",
        "up": p + "mlp.up_proj.weight",
        "down": p + "mlp.down_proj.weight",
    }


def forward(cfg, weights, tokens, schedule=None, return_hidden=False, position_offset=0):
    """Logits ``[T, V]`` of one whole token sequence.

    ``cfg`` is the dict of config.json; ``weights`` maps tensor names to
    arrays. Order inside a layer as J/inference/InferenceCore.java:72-173:
    norm -> q,k,v -> rope(q,k) -> attention over 0..p -> Wo -> add -> norm ->
    gate, up -> silu(gate)*up -> down -> add; then the final norm and the LM
    head (:175-177), which is the embedding table when no separate head exists
    (J/model/loader/ModelLoader.java:252-253).

    ``schedule`` (not in the reference, whose layers run 0..L-1 once) is a list
    of ``(layer, source)``: run ``layer``'s weights; if ``source`` is not None
    the run computes no keys and values of its own and reads those that the
    earlier run number ``source`` made. ``position_offset`` shifts every
    position (the reference's ``startPosition``,
    J/inference/InferenceEngine.java:83-88, without the cached prefix): with
    rotary encoding only distances count, so it must not change the logits
    when no frequency scaling depends on absolute length.
    """
    d = cfg["hidden_size"]
    H = cfg["num_attention_heads"]
    K = cfg.get("num_key_value_heads", H)
    hs = cfg.get("head_dim") or d // H
    L = cfg["num_hidden_layers"]
    eps = cfg.get("rms_norm_eps", 1e-5)
    theta = cfg.get("rope_theta", 10000.0)
    pairing = cfg.get("rope_pairing", "half")
    tokens = np.asarray(tokens, dtype=np.int64)
    T = len(tokens)
    positions = np.arange(T) + position_offset
    cos, sin = rope_table(T + position_offset, hs, theta, cfg.get("rope_scaling"))
    W = {n: np.asarray(a, dtype=F32) for n, a in weights.items()}

    x = W["model.embed_tokens.weight"][tokens].astype(F32)  # InferenceCore.java:69
    if schedule is None:
        schedule = [(l, None) for l in range(L)]
    made = []
    for layer, source in schedule:
        n = layer_names(layer)
        xb = rmsnorm(x, W[n["attn_norm"]], eps)
        q = linear(xb, W[n["q"]]).reshape(T, H, hs)
        q = rope_rotate(q, positions, cos, sin, pairing)
        if source is None:
            k = linear(xb, W[n["k"]]).reshape(T, K, hs)
            v = linear(xb, W[n["v"]]).reshape(T, K, hs)
            k = rope_rotate(k, positions, cos, sin, pairing)
        else:
            k, v = made[source]
        made.append((k, v))
        att = attention(q, k, v).reshape(T, H * hs)
        x = x + linear(att, W[n["o"]])
        xb = rmsnorm(x, W[n["ffn_norm"]], eps)
        x = x + feed_forward(xb, W[n["gate"]], W[n["up"]], W[n["down"]])
    hidden = x
    x = rmsnorm(x, W["model.norm.weight"], eps)
    head = W["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else W["lm_head.weight"]
    logits = linear(x, head)
    return (logits, hidden) if return_hidden else logits


# --------------------------------------------------------------------------- sampling
def argmax(logits):
    """First index of the strictly greatest value
    (J/inference/sampler/Sampler.java:144-157)."""
    best, idx = -np.inf, 0
    for i, v in enumerate(np.asarray(logits)):
        if v > best:
            best, idx = v, i
    return idx


def probabilities(logits, temperature):
    """``softmax(logits / temperature)`` (J/inference/sampler/Sampler.java:87-89)."""
    return softmax(np.asarray(logits, dtype=F32) / F32(temperature))


def sample_categorical(probs, r):
    """First ``i`` with ``r < cdf_i``, else the last index
    (J/inference/sampler/CategoricalSampler.java:31-42). ``r`` in [0, 1)."""
    cdf = 0.0
    for i, p in enumerate(np.asarray(probs, dtype=np.float64)):
        cdf += p
        if r < cdf:
            return i
    return len(probs) - 1


def top_p_set(probs, top_p):
    """Indices kept by nucleus sampling, in descending order of probability
    (ties: lower index first), and their total mass.

    J/inference/sampler/ToppSampler.java:94-136: candidates below
    ``(1 - top_p)/(n - 1)`` can never be needed; the rest in descending order;
    the list is cut after the first element at which the running sum exceeds
    ``top_p``.
    """
    probs = np.asarray(probs, dtype=np.float64)
    order = sorted(range(len(probs)), key=lambda i: (-probs[i], i))
    kept, mass = [], 0.0
    for i in order:
        kept.append(i)
        mass += probs[i]
        if mass > top_p:
            break
    return kept, mass


def sample_top_p(probs, top_p, r):
    """J/inference/sampler/ToppSampler.java:139-155: ``r * mass``, walk the kept
    list in descending order, return the first whose running sum exceeds it;
    fallback is the last kept."""
    kept, mass = top_p_set(probs, top_p)
    target = r * mass
    cdf = 0.0
    for i in kept:
        cdf += float(probs[i])
        if target < cdf:
            return i
    return kept[-1]


def sample(logits, temperature, top_p, r):
    """Selection rule of J/inference/sampler/Sampler.java:56-104."""
    if temperature == 0.0:
        return argmax(logits)
    p = probabilities(logits, temperature)
    if top_p <= 0 or top_p >= 1:
        return sample_categorical(p, r)
    return sample_top_p(p, top_p, r)

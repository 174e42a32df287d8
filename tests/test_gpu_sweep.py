"""Seeded random configurations of the architecture through the engine, against the plain implementation.

Each configuration draws every size that config.json gives (head sizes in steps of 16 up to 128, one kv
head for many query heads up to as many kv heads as heads, widths and vocabularies that no tile divides,
tied and separate heads, frequency scaling on and off, both pairings) and runs, in 32-bit and in bfloat16:
a request alone and whole, its last 8 tokens one by one, a batch of three unequal requests whose shorter
ones end earlier, and a batch of many short sequences (the kernels for 9 to 80 rows, decode steps
replayed from graphs). The sweep stops at the first failure (``-x``), which names its seed.
"""
import os
import shutil
import tempfile

import numpy as np
import pytest
from safetensors.torch import load_file

import plain_llama as P

pytestmark = pytest.mark.gpu

TOL = {"float32": 2e-5, "bfloat16": 2e-2}          # as tests/gpu_helpers.py; never widened to pass
HEAD_SIZES = [16, 32, 48, 64, 80, 96, 112, 128, 48, 80, 112, 64]      # one per seed: every step of 16 is met


def draw(seed):
    rng = np.random.default_rng([seed, 2024])
    hs = HEAD_SIZES[seed % len(HEAD_SIZES)]
    K = int(rng.integers(1, 5))
    G = [1, 2, 3, 4, 5, 7, 8, 6, 1, 4, 8, 2][seed % 12]          # seeds 0 and 8: as many kv heads as heads; MQA where K == 1
    if seed in (2, 9):
        K = 1                                                     # one kv head for all query heads
    H = K * G
    d = int(rng.choice([8 * int(rng.integers(3, 40)), H * hs]))
    F = 8 * int(rng.integers(3, 90))
    V = int(rng.integers(40, 3000))
    L = int(rng.integers(1, 4))
    ctx = int(rng.choice([128, 320, 700]))
    scaling = None
    if seed % 2 == 0:
        scaling = {"rope_type": "llama3", "factor": float(rng.choice([2.0, 8.0, 32.0])), "low_freq_factor": 1.0,
                   "high_freq_factor": float(rng.choice([2.0, 4.0])),
                   "original_max_position_embeddings": int(rng.choice([32, 64, 256]))}
    cfg = {"architectures": ["LlamaForCausalLM"], "hidden_size": d, "intermediate_size": F, "num_hidden_layers": L,
           "num_attention_heads": H, "num_key_value_heads": K, "head_dim": hs, "vocab_size": V,
           "max_position_embeddings": ctx, "rms_norm_eps": float(rng.choice([1e-5, 1e-6, 3e-5])),
           "rope_theta": float(rng.choice([10000.0, 500000.0])), "rope_scaling": scaling,
           "tie_word_embeddings": seed % 3 != 0, "hidden_act": "silu"}
    if seed % 4 == 1:
        cfg["rope_pairing"] = "adjacent"
    return cfg, rng


def check(got, ref, dtype, what):
    scale = max(float(np.abs(ref).max()), 1e-3)
    assert got.shape == ref.shape and np.isfinite(got).all(), what
    err = np.abs(got - ref).max(axis=-1) / scale
    bad = np.flatnonzero(~(err <= TOL[dtype]))
    assert len(bad) == 0, f"{what}: first wrong row {int(bad[0])} of {len(ref)}, error {err.max():.3e} of the logit scale"


@pytest.mark.parametrize("seed", range(12))
def test_a_random_configuration(seed):
    import gpullama3_java_amd as g
    from gpullama3_java_amd.engine import Engine
    cfg, rng = draw(seed)
    what = (f"seed {seed}: head_dim {cfg['head_dim']}, {cfg['num_attention_heads']} heads, {cfg['num_key_value_heads']} kv, "
            f"hidden {cfg['hidden_size']}, ffn {cfg['intermediate_size']}, vocab {cfg['vocab_size']}, "
            f"{cfg['num_hidden_layers']} layers, context {cfg['max_position_embeddings']}")
    print(what, flush=True)
    ctx, V = cfg["max_position_embeddings"], cfg["vocab_size"]
    folder = tempfile.mkdtemp(prefix="gl3-sweep-")
    try:
        g.write_random_model(folder, g.config_from_dict(cfg), seed, std=min(0.05, 0.6 / cfg["hidden_size"] ** 0.5),
                             norm_std=0.1)
        W = {k: v.float().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
        lens = [int(x) for x in rng.integers(9, ctx - 20, size=3)]
        new = [int(x) for x in rng.integers(1, 12, size=3)]
        seqs = [rng.integers(0, V, size=p + n).tolist() for p, n in zip(lens, new)]
        refs = [P.forward(cfg, W, q) for q in seqs]
        B = int(rng.choice([9, 12, 16, 17, 24, 32, 33, 48, 64, 65, 80]))
        plen = [int(x) for x in rng.integers(1, 6, size=B)]
        many = [rng.integers(0, V, size=p + 3).tolist() for p in plen]
        many_refs = [P.forward(cfg, W, q) for q in many]
        for dtype in ("float32", "bfloat16"):
            eng = Engine.from_folder(folder, dtype=dtype, max_tokens=3 * 64 * (-(-ctx // 64)), n_slots=3)
            # the first request alone and whole; then again with its last 8 tokens one by one
            q, ref = seqs[0], refs[0]
            s = eng.take_slot()
            check(eng.step([(s, q)], want="all").cpu().numpy(), ref, dtype, f"{what}; {dtype}, whole")
            eng.give_back_slot(s)
            s = eng.take_slot()
            rows = [eng.step([(s, q[:-8])], want="all").cpu().numpy()]
            rows += [eng.step([(s, [t])]).cpu().numpy() for t in q[-8:]]
            eng.give_back_slot(s)
            check(np.concatenate(rows), ref, dtype, f"{what}; {dtype}, the last 8 one by one (prompt ends at {len(q) - 8})")
            # the three as a batch of unequal prompts, then one token each; the shorter ones end earlier
            slots = [eng.take_slot() for _ in seqs]
            got = [[] for _ in seqs]
            out = eng.step([(s, q[:p]) for s, q, p in zip(slots, seqs, lens)], want="all").cpu().numpy()
            o = 0
            for j, p in enumerate(lens):
                got[j].append(out[o:o + p])
                o += p
            k = 0
            while True:
                live = [j for j in range(3) if k < new[j]]
                for j in range(3):
                    if j not in live and slots[j] is not None:
                        eng.give_back_slot(slots[j])
                        slots[j] = None
                if not live:
                    break
                out = eng.step([(slots[j], [seqs[j][lens[j] + k]]) for j in live]).cpu().numpy()
                for r, j in enumerate(live):
                    got[j].append(out[r:r + 1])
                k += 1
            for j in range(3):
                check(np.concatenate(got[j]), refs[j], dtype,
                      f"{what}; {dtype}, batch of three, request {j} (prompt {lens[j]}, total {len(seqs[j])})")
            del eng
            # many short sequences in one batch
            eng = Engine.from_folder(folder, dtype=dtype, max_tokens=B * 64, n_slots=B)
            slots = [eng.take_slot() for _ in many]
            outs = [eng.step([(sl, q[:p]) for sl, q, p in zip(slots, many, plen)]).cpu().numpy()]
            for k in range(3):
                outs.append(eng.step([(sl, [q[p + k]]) for sl, q, p in zip(slots, many, plen)]).cpu().numpy())
            for j in range(B):
                check(np.stack([o[j] for o in outs]), many_refs[j][plen[j] - 1:], dtype,
                      f"{what}; {dtype}, batch of {B}, request {j}")
            del eng
    finally:
        shutil.rmtree(folder, ignore_errors=True)

"""The engines at the layer sizes of real models.

The tiny configurations of the other tests are too small for several choices that the
product path makes by size: products of a prompt cut into slices of K, tiles of 256 x 256,
strips of 8 rows, the kernels for 33 to 64 rows with their slices, the tiled kernel for the
head. Here the layers have the sizes of Llama-3.2-1B (what bench.py measures), Llama-3.2-3B and Llama-3.1-8B
(two layers each, to keep the test short). Every kind of step is run on the bfloat16 and the
float32 engine with the same weights, both engines are compared with the plain implementation
at these sizes, and runs of decode steps that sample on the device are compared with the
host's twin of the sampler on the logits of single steps."""
import numpy as np
import pytest
import torch

from gpu_helpers import TOL

pytestmark = pytest.mark.gpu

COMMON = {"architectures": ["LlamaForCausalLM"], "num_hidden_layers": 2, "vocab_size": 128256,
          "max_position_embeddings": 4096, "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "hidden_act": "silu"}
SHAPES = {
    # the layers of Llama-3.2-1B: head size 64, tied head
    "1B": {**COMMON, "hidden_size": 2048, "intermediate_size": 8192, "num_attention_heads": 32, "num_key_value_heads": 8,
           "head_dim": 64, "tie_word_embeddings": True,
           "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                            "original_max_position_embeddings": 8192}},
    # the layers of Llama-3.2-3B: three query heads to a kv head, head size 128, a width of 3072
    "3B": {**COMMON, "hidden_size": 3072, "intermediate_size": 8192, "num_attention_heads": 24, "num_key_value_heads": 8,
           "head_dim": 128, "tie_word_embeddings": True,
           "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                            "original_max_position_embeddings": 8192}},
    # the layers of Llama-3.1-8B: head size 128, longer rows, a head of its own
    "8B": {**COMMON, "hidden_size": 4096, "intermediate_size": 14336, "num_attention_heads": 32, "num_key_value_heads": 8,
           "head_dim": 128, "tie_word_embeddings": False,
           "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                            "original_max_position_embeddings": 8192}},
}


def steps(eng, vocab):
    """Logits of every kind of step: a long prompt, single tokens after it, batches of 8, 12, 20, 40 and 100
    sequences (short prompts, then decode steps that are replayed from graphs), prompts of 50, a prompt
    of 2,600 tokens and single tokens after it."""
    rng = np.random.default_rng(0)
    out = []
    s = eng.take_slot()
    toks = rng.integers(0, vocab, 603).tolist()
    out.append(eng.step([(s, toks[:600])]).cpu().numpy())
    for t in toks[600:]:
        out.append(eng.step([(s, [t])]).cpu().numpy())
    eng.give_back_slot(s)
    for B in (8, 12, 20, 40, 100):
        slots = [eng.take_slot() for _ in range(B)]
        seqs = [rng.integers(0, vocab, 7).tolist() for _ in range(B)]
        out.append(eng.step([(sl, q[:4]) for sl, q in zip(slots, seqs)]).cpu().numpy())
        for k in (4, 5, 6):
            out.append(eng.step([(sl, [q[k]]) for sl, q in zip(slots, seqs)]).cpu().numpy())
        for sl in slots:
            eng.give_back_slot(sl)
    five = [eng.take_slot() for _ in range(5)]
    out.append(eng.step([(sl, rng.integers(0, vocab, 50).tolist()) for sl in five]).cpu().numpy())
    for sl in five:
        eng.give_back_slot(sl)
    # a long prompt (the largest tiles), then tokens whose attention is split over the keys
    s = eng.take_slot()
    toks = rng.integers(0, vocab, 2603).tolist()
    out.append(eng.step([(s, toks[:2600])]).cpu().numpy())
    for t in toks[2600:]:
        out.append(eng.step([(s, [t])]).cpu().numpy())
    return out


@pytest.mark.parametrize("shape", ["1B", "3B", "8B"])
def test_real_layer_sizes_bfloat16_against_float32(tmp_path, shape):
    import gpullama3_java_amd as g
    from gpullama3_java_amd.engine import Engine
    cfg = g.config_from_dict(SHAPES[shape])
    folder = str(tmp_path / "shape")
    g.write_random_model(folder, cfg, 11, std=0.02, norm_std=0.1)
    results = {}
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_folder(folder, dtype=dtype, max_context=4096, max_tokens=128 * 64, n_slots=128)
        results[dtype] = steps(eng, cfg.vocab_size)
        if dtype == "bfloat16":
            assert eng._graphs, "the decode steps were not replayed from graphs"
        del eng
        torch.cuda.empty_cache()
    for i, (ref, got) in enumerate(zip(results["float32"], results["bfloat16"])):
        scale = float(np.abs(ref).max())
        err = float(np.abs(ref - got).max())
        assert err <= TOL["bfloat16"] * scale, f"step {i} ({ref.shape[0]} rows): {err / scale:.4f} of the logit scale"


def test_runs_of_decode_steps_at_real_layer_sizes_pick_the_tokens_of_single_steps(tmp_path):
    """Generation runs several decode steps on the device with one wait at the end; the tokens must
    be those that single steps with a host-side argmax give, for 40 sequences (the kernels for 33 to
    64 rows) and for 3."""
    import gpullama3_java_amd as g
    from gpullama3_java_amd.engine import Engine
    cfg = g.config_from_dict(SHAPES["1B"])
    folder = str(tmp_path / "shape")
    g.write_random_model(folder, cfg, 12, std=0.02, norm_std=0.1)
    eng = Engine.from_folder(folder, dtype="bfloat16", max_context=256, max_tokens=64 * 64, n_slots=64)
    rng = np.random.default_rng(1)
    for B in (40, 3):
        prompts = [rng.integers(0, cfg.vocab_size, 3 + i % 4).tolist() for i in range(B)]
        res = eng.generate(prompts, max_new_tokens=21, temperature=0.0, stop_ids=())
        slots = [eng.take_slot() for _ in range(B)]
        logits = eng.step(list(zip(slots, prompts)))
        want = [[] for _ in range(B)]
        for _ in range(21):
            toks = logits.argmax(-1).tolist()
            for i, t in enumerate(toks):
                want[i].append(t)
            logits = eng.step([(sl, [t]) for sl, t in zip(slots, toks)])
        for sl in slots:
            eng.give_back_slot(sl)
        for i in range(B):
            assert res[i].tokens == want[i], f"batch {B}, request {i}"


@pytest.mark.parametrize("shape", ["1B", "3B", "8B"])
def test_real_layer_sizes_against_the_plain_implementation(tmp_path, shape):
    """The kernels that only real widths select (tiles of 256 x 256, strips of 8 rows, the resident
    kernels of sixteen waves, the head through the tiled kernel, products cut into slices of K) inside
    a whole model against the plain implementation itself (J/inference/InferenceCore.java:58-180), not
    against another path of the engine: a prompt of 300 tokens with every row wanted, four single
    tokens after it, and a batch of 40 short prompts with three decode steps (the kernels for 33 to
    64 rows, replayed from graphs), in float32 and in bfloat16. Then batches of 12, 24 and 100 sequences
    (products of 9 to 16 rows over a long K, the variant for two token tiles, steps worked on in pieces
    of 64 rows), of which the sequences at the edges of the token tiles are compared."""
    from safetensors.torch import load_file

    import gpullama3_java_amd as g
    import plain_llama as P
    from gpullama3_java_amd.engine import Engine
    cfgd = SHAPES[shape]
    cfg = g.config_from_dict(cfgd)
    folder = str(tmp_path / "shape")
    g.write_random_model(folder, cfg, 13, std=0.02, norm_std=0.1)
    W = {k: v.float().numpy() for k, v in load_file(folder + "/model.safetensors").items()}
    rng = np.random.default_rng(2)
    long_toks = rng.integers(0, cfg.vocab_size, 304).tolist()
    short = [rng.integers(0, cfg.vocab_size, 7).tolist() for _ in range(40)]
    ref_long = P.forward(cfgd, W, long_toks)
    ref_short = [P.forward(cfgd, W, q)[3:] for q in short]                   # rows of the tokens 3, 4, 5, 6
    more = {B: [rng.integers(0, cfg.vocab_size, 7).tolist() for _ in range(B)] for B in (12, 24, 100)}
    watched = {12: [0, 7, 8, 11], 24: [0, 15, 16, 23], 100: [0, 31, 32, 49, 50, 63, 64, 99]}
    ref_more = {B: {i: P.forward(cfgd, W, more[B][i])[3:] for i in watched[B]} for B in more}
    del W
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_folder(folder, dtype=dtype, max_context=512, max_tokens=128 * 64, n_slots=128)
        s = eng.take_slot()
        got = [eng.step([(s, long_toks[:300])], want="all").cpu().numpy()]
        got += [eng.step([(s, [t])]).cpu().numpy() for t in long_toks[300:]]
        eng.give_back_slot(s)
        got = np.concatenate(got)
        scale = float(np.abs(ref_long).max())
        err = np.abs(got - ref_long).max(axis=1)
        assert err.max() <= TOL[dtype] * scale, f"{dtype}: row {int(err.argmax())} of the long sequence is off by {err.max() / scale:.2e}"
        slots = [eng.take_slot() for _ in short]
        rows = [eng.step([(sl, q[:4]) for sl, q in zip(slots, short)]).cpu().numpy()]
        rows += [eng.step([(sl, [q[k]]) for sl, q in zip(slots, short)]).cpu().numpy() for k in (4, 5, 6)]
        for sl in slots:
            eng.give_back_slot(sl)
        got = np.stack(rows, axis=1)                                         # [40, 4, vocab]
        for i, r in enumerate(ref_short):
            sc = float(np.abs(r).max())
            e = float(np.abs(got[i] - r).max())
            assert e <= TOL[dtype] * sc, f"{dtype}: sequence {i} of the batch of 40 is off by {e / sc:.2e}"
        for B, seqs in more.items():
            slots = [eng.take_slot() for _ in seqs]
            rows = [eng.step([(sl, q[:4]) for sl, q in zip(slots, seqs)]).cpu().numpy()]
            rows += [eng.step([(sl, [q[k]]) for sl, q in zip(slots, seqs)]).cpu().numpy() for k in (4, 5, 6)]
            for sl in slots:
                eng.give_back_slot(sl)
            got = np.stack(rows, axis=1)                                     # [B, 4, vocab]
            for i, r in ref_more[B].items():
                sc = float(np.abs(r).max())
                e = float(np.abs(got[i] - r).max())
                assert e <= TOL[dtype] * sc, f"{dtype}: sequence {i} of the batch of {B} is off by {e / sc:.2e}"
        if dtype == "bfloat16":
            assert eng._graphs
        del eng
        torch.cuda.empty_cache()


def test_a_long_context_at_real_layer_sizes_against_the_plain_implementation(tmp_path):
    """A prompt of 2,600 tokens (the largest tiles of the products, the longest blocks of the prompt's attention)
    and three single tokens after it, whose attention is split over the keys and merged (heads of 64 at a
    context beyond 2,048), with the layers of Llama-3.2-1B against the plain implementation itself, in float32
    and in bfloat16: the prompt's first, middle and last row and the three tokens' rows."""
    from safetensors.torch import load_file

    import gpullama3_java_amd as g
    import plain_llama as P
    from gpullama3_java_amd.csrc import lib
    from gpullama3_java_amd.engine import Engine
    cfgd = SHAPES["1B"]
    cfg = g.config_from_dict(cfgd)
    folder = str(tmp_path / "shape")
    g.write_random_model(folder, cfg, 14, std=0.02, norm_std=0.1)
    W = {k: v.float().numpy() for k, v in load_file(folder + "/model.safetensors").items()}
    toks = np.random.default_rng(3).integers(0, cfg.vocab_size, 2603).tolist()
    watched = [0, 1299, 2599, 2600, 2601, 2602]
    _, hidden = P.forward(cfgd, W, toks, return_hidden=True)
    ref = P.linear(P.rmsnorm(hidden[watched], W["model.norm.weight"], cfgd["rms_norm_eps"]), W["model.embed_tokens.weight"])
    del W, hidden
    assert lib.decode_splits(1, 32, 8, 4096, 64) > 1           # the case is the one it claims to be
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_folder(folder, dtype=dtype, max_context=4096, max_tokens=2688, n_slots=1)
        s = eng.take_slot()
        got = [eng.step([(s, toks[:2600])], want=[[0, 1299, 2599]]).cpu().numpy()]
        got += [eng.step([(s, [t])]).cpu().numpy() for t in toks[2600:]]
        got = np.concatenate(got)
        scale = float(np.abs(ref).max())
        err = np.abs(got - ref).max(axis=1)
        assert err.max() <= TOL[dtype] * scale, f"{dtype}: row {watched[int(err.argmax())]} is off by {err.max() / scale:.2e}"
        del eng
        torch.cuda.empty_cache()


def _share_of(logits, temperature, top_p, token, u):
    """How far the uniform number ``u`` lies from the share of [0, 1) that ``token`` has in the sampler's
    order of the candidates (by falling probability, the kept ones rescaled to 1): 0 when u draws it.
    With probabilities this flat the neighbours in that order are tokens from anywhere in the
    vocabulary, so a draw next to an edge is told by this distance and not by the token's number."""
    s = np.asarray(logits, np.float32) / np.float32(temperature)
    e = np.exp(s - s.max()).astype(np.float64)
    p = e / e.sum()
    order = np.lexsort((np.arange(len(p)), -p))
    csum = np.cumsum(p[order])
    mass = 1.0
    if 0 < top_p < 1:
        over = np.flatnonzero(csum > top_p)
        mass = csum[int(over[0])] if len(over) else csum[-1]
    else:
        order = np.arange(len(p))
        csum = np.cumsum(p)
    rank = int(np.flatnonzero(order == token)[0])
    lo, hi = (csum[rank - 1] if rank else 0.0) / mass, csum[rank] / mass
    return 0.0 if lo <= u < hi else min(abs(u - lo), abs(u - hi))


@pytest.mark.parametrize("B", [40, 9])
def test_sampled_runs_of_decode_steps_in_bfloat16_draw_what_single_steps_draw(tmp_path, B):
    """Runs of decode steps that sample on the device (temperature and top-p, per-row parameters and
    uniform numbers read by a step counter on the device) at real layer sizes in bfloat16: 40
    sequences take the kernels for 33 to 64 rows, 9 a bucket of 16. Every token of a run must be
    the one that the host's twin of the sampler draws, with the same uniform number, from the logits
    that a single step of the same engine returns for the same sequence so far."""
    import gpullama3_java_amd as g
    from gpullama3_java_amd.engine import Engine
    from gpullama3_java_amd.sampling import sample_host, uniform
    cfg = g.config_from_dict(SHAPES["1B"])
    folder = str(tmp_path / "shape")
    g.write_random_model(folder, cfg, 14, std=0.02, norm_std=0.1)
    eng = Engine.from_folder(folder, dtype="bfloat16", max_context=256, max_tokens=2 * B * 64, n_slots=2 * B)
    rng = np.random.default_rng(3)
    prompts = [rng.integers(0, cfg.vocab_size, 3 + i % 5).tolist() for i in range(B)]
    temps = [0.0 if i % 7 == 3 else 0.6 + 0.1 * (i % 5) for i in range(B)]          # some rows greedy, the rest at several temperatures
    tops = [1.0 if i % 4 == 0 else 0.9 for i in range(B)]
    n = 11
    us = [[uniform(5, i, k) for i in range(B)] for k in range(n)]
    slots = [eng.take_slot() for _ in range(B)]
    first = eng.step(list(zip(slots, prompts))).argmax(-1).tolist()
    run = eng.decode_run(list(zip(slots, first)), n, temps, tops, us)            # [n][B], sampled on the device
    assert any(key[2] == "sampled" for key in eng._graphs)
    again = [eng.take_slot() for _ in range(B)]
    eng.step(list(zip(again, prompts)), want="none")
    cur = first
    for k in range(n):
        logits = eng.step([(s, [t]) for s, t in zip(again, cur)]).cpu().numpy()
        for i in range(B):
            want = sample_host(logits[i], temps[i], tops[i], us[k][i])
            if run[k][i] != want:        # allowed only at an edge of the running sum (the two paths' logits differ in the last bits)
                assert _share_of(logits[i], temps[i], tops[i], run[k][i], us[k][i]) < 1e-4, \
                    f"step {k}, row {i}: {run[k][i]} drawn on the device, {want} by the host"
        cur = run[k]                     # go on with the device's tokens, so that both follow the same sequences

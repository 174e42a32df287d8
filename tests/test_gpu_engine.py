"""The engine against the plain implementation under every way of cutting the work."""
import numpy as np
import pytest
import torch

from gpu_helpers import CONFIGS, DTYPES, close, first_bad_row, model, plain_logits, rand_tokens

pytestmark = pytest.mark.gpu

CASES = [(n, d) for n in ("A", "B", "C", "D") for d in DTYPES]


def engine(name, dtype, **kw):
    from gpullama3_java_amd.engine import Engine
    folder, _, _ = model(name)
    kw.setdefault("max_tokens", 2048)
    return Engine.from_folder(folder, dtype=dtype, **kw)


def lengths(name):
    return {"A": [5, 11, 64, 100], "B": [3, 17, 40, 129, 200], "C": [1, 63, 65, 300], "D": [2, 33, 70, 257]}[name]


@pytest.mark.parametrize("name, dtype", CASES)
def test_each_request_alone_and_whole(name, dtype):
    eng = engine(name, dtype)
    for i, n in enumerate(lengths(name)):
        toks = rand_tokens(name, i, n)
        s = eng.take_slot()
        got = eng.step([(s, toks)], want="all").cpu().numpy()
        eng.give_back_slot(s)
        close(got, plain_logits(name, toks), dtype, f"{name} {dtype} whole n={n}")


@pytest.mark.parametrize("name, dtype", CASES)
def test_last_32_tokens_one_by_one(name, dtype):
    eng = engine(name, dtype)
    for i, n in enumerate(lengths(name)):
        if n <= 33:
            continue
        toks = rand_tokens(name, 10 + i, n)
        ref = plain_logits(name, toks)
        s = eng.take_slot()
        rows = [eng.step([(s, toks[:n - 32])], want="all").cpu().numpy()]
        rows += [eng.step([(s, [t])], want="all").cpu().numpy() for t in toks[n - 32:]]
        eng.give_back_slot(s)
        got = np.concatenate(rows)
        bad = first_bad_row(got, ref, dtype)
        assert bad is None, f"{name} {dtype} n={n}: first wrong row {bad} (prompt ends at {n - 32})"
        close(got, ref, dtype)


@pytest.mark.parametrize("name, dtype", CASES)
def test_unequal_batches_one_after_another_reuse_slots(name, dtype):
    """Batches start together with unequal prompts, decode one token each, shorter
    requests end earlier; three batches run over three slots and a cache that holds
    one batch only, so slots and pages are used again with old data in them."""
    cfgd = CONFIGS[name]
    limit = cfgd["max_position_embeddings"]
    eng = engine(name, dtype, n_slots=3, max_tokens=3 * 64 * (-(-min(limit, 200) // 64)))
    rng = np.random.default_rng(5)
    for batch in range(3):
        prompt_lens = [int(x) for x in rng.integers(1, min(limit, 200) - 40, size=3)]
        new = [int(x) for x in rng.integers(1, 30, size=3)]
        seqs = [rand_tokens(name, 100 * batch + j, p + n) for j, (p, n) in enumerate(zip(prompt_lens, new))]
        slots = [eng.take_slot() for _ in seqs]
        got = [[] for _ in seqs]
        out = eng.step([(s, q[:p]) for s, q, p in zip(slots, seqs, prompt_lens)], want="all").cpu().numpy()
        o = 0
        for j, p in enumerate(prompt_lens):
            got[j].append(out[o:o + p]); o += p
        live = list(range(3))
        k = 0
        while live:
            live = [j for j in live if k < new[j]]
            for j in range(3):                       # a request that has ended gives its slot back at once
                if j not in live and slots[j] is not None and k >= new[j]:
                    eng.give_back_slot(slots[j]); slots[j] = None
            if not live:
                break
            out = eng.step([(slots[j], [seqs[j][prompt_lens[j] + k]]) for j in live]).cpu().numpy()
            for r, j in enumerate(live):
                got[j].append(out[r:r + 1])
            k += 1
        for j, q in enumerate(seqs):
            g_ = np.concatenate(got[j])
            ref = plain_logits(name, q)
            bad = first_bad_row(g_, ref, dtype)
            assert bad is None, (f"{name} {dtype} batch {batch} request {j}: first wrong row {bad} "
                                 f"(prompt {prompt_lens[j]}, total {len(q)})")
    assert eng.cache.slots.live == set()


@pytest.mark.parametrize("name, dtype", [("B", "float32"), ("B", "bfloat16"), ("C", "float32"), ("C", "bfloat16"),
                                         ("D", "bfloat16")])
def test_long_decoding(name, dtype):
    n = {"B": 250, "C": 400, "D": 330}[name]
    toks = rand_tokens(name, 77, n)
    ref = plain_logits(name, toks)
    eng = engine(name, dtype)
    s = eng.take_slot()
    rows = [eng.step([(s, toks[:3])], want="all").cpu().numpy()]
    rows += [eng.step([(s, [t])]).cpu().numpy() for t in toks[3:]]
    got = np.concatenate(rows)
    bad = first_bad_row(got, ref, dtype)
    assert bad is None, f"first wrong row {bad}"


@pytest.mark.parametrize("name, dtype", CASES)
def test_first_tokens_of_a_sequence(name, dtype):
    eng = engine(name, dtype)
    toks = rand_tokens(name, 5, 6)
    ref = plain_logits(name, toks)
    s = eng.take_slot()                                          # from the very first token, one by one
    got = np.concatenate([eng.step([(s, [t])]).cpu().numpy() for t in toks])
    eng.give_back_slot(s)
    close(got, ref, dtype, "one by one from position 0")
    slots = [eng.take_slot() for _ in range(3)]
    # prompts of 1, 2, 3 tokens in one batch
    out = eng.step([(slots[i], toks[:i + 1]) for i in range(3)], want="all").cpu().numpy()
    close(out, np.concatenate([ref[:1], ref[:2], ref[:3]]), dtype, "prompts of 1, 2, 3")


@pytest.mark.parametrize("dtype", DTYPES)
def test_batch_mates_order_and_slot_change_nothing(dtype):
    name = "B"
    a, b, c = rand_tokens(name, 1, 50), rand_tokens(name, 2, 7), rand_tokens(name, 3, 120)
    eng = engine(name, dtype, n_slots=8)
    s = eng.take_slot()
    alone = eng.step([(s, a)], want="all").cpu().numpy()
    eng.give_back_slot(s)
    for _ in range(3):
        eng.take_slot()                                           # other slots, other pages
    sb, sa, sc = eng.take_slot(), eng.take_slot(), eng.take_slot()
    out = eng.step([(sc, c), (sa, a), (sb, b)], want="all").cpu().numpy()
    mixed = out[120:170]
    if dtype == "float32":
        np.testing.assert_array_equal(mixed, alone)               # same kernels, same order of sums
    else:
        close(mixed, alone, dtype)
    close(mixed, plain_logits(name, a), dtype)


@pytest.mark.parametrize("name, dtype", [("A", "bfloat16"), ("B", "float32"), ("B", "bfloat16"), ("C", "bfloat16"),
                                         ("D", "bfloat16")])
@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("B", [41, 23])
def test_decode_steps_of_17_to_64_sequences(name, dtype, graphs, B, monkeypatch):
    """Between 17 and 64 tokens a step the products into the residual stream leave their sums in
    slices of K that the next norm adds up, and rotation and cache write ride on the QKV product.
    The tiny models' K is too short for the rule that cuts it, so the rule is replaced by one that
    always cuts."""
    from gpullama3_java_amd.csrc import lib
    cut = []

    def always(N, Kd):
        n = 3 if Kd >= 192 else 2 if Kd >= 128 else 1      # (a slice is at least a pair of k-steps, 64 k)
        cut.append(n)
        return n
    monkeypatch.setattr(lib, "wide_slices", always)
    eng = engine(name, dtype, n_slots=64, max_tokens=64 * 64, use_graphs=graphs)
    seqs = [rand_tokens(name, 200 + i, 2 + i % 5 + 6) for i in range(B)]
    slots = [eng.take_slot() for _ in range(B)]
    first = eng.step([(s, q[:2 + i % 5]) for i, (s, q) in enumerate(zip(slots, seqs))]).cpu().numpy()
    rows = [[first[i]] for i in range(B)]
    for k in range(5):
        o = eng.step([(s, [q[2 + i % 5 + k]]) for i, (s, q) in enumerate(zip(slots, seqs))]).cpu().numpy()
        for i in range(B):
            rows[i].append(o[i])
    assert dtype == "float32" or max(cut) > 1
    for i in range(B):
        n0 = 2 + i % 5
        close(np.stack(rows[i]), plain_logits(name, seqs[i])[n0 - 1:n0 + 5], dtype, f"request {i}")


@pytest.mark.parametrize("name", ["B", "C", "D"])
def test_prompt_products_cut_into_slices_of_k(name, monkeypatch):
    """Products of a prompt into the residual stream cut K into slices when K is long and the tiles
    are few; the tiny models' K is short, so the rule is replaced here by one that always cuts.
    (Steps of more than 192 tokens: fewer are worked on by the kernels for few rows.)"""
    from gpullama3_java_amd.csrc import lib
    calls = []

    def always(M, N, Kd):
        n = 3 if Kd >= 192 else 2 if Kd >= 128 else 1
        calls.append(n)
        return n
    monkeypatch.setattr(lib, "mfma_slices", always)
    eng = engine(name, "bfloat16")
    toks = rand_tokens(name, 77, 240)
    s = eng.take_slot()
    got = eng.step([(s, toks[:200])], want="all").cpu().numpy()
    got2 = eng.step([(s, toks[200:])], want="all").cpu().numpy()
    assert max(calls) > 1
    close(np.concatenate([got, got2]), plain_logits(name, toks), "bfloat16", f"{name} in slices")


@pytest.mark.parametrize("dtype", DTYPES)
def test_wanted_places_and_errors(dtype):
    from gpullama3_java_amd.engine import CacheFull
    name = "A"
    eng = engine(name, dtype, max_tokens=128, n_slots=2)
    a, b = rand_tokens(name, 1, 20), rand_tokens(name, 2, 9)
    sa, sb = eng.take_slot(), eng.take_slot()
    out = eng.step([(sa, a), (sb, b)], want=[[0, 19, 7], []]).cpu().numpy()
    ref = plain_logits(name, a)
    close(out, ref[[0, 19, 7]], dtype)
    assert eng.step([(sb, [1])], want="none").shape == (0, 256)
    with pytest.raises(ValueError, match="vocabulary"):
        eng.step([(sa, [256])])
    with pytest.raises(ValueError, match="twice"):
        eng.step([(sa, [1]), (sa, [2])])
    with pytest.raises(CacheFull):
        eng.step([(sa, [1] * 60)])                                 # 20 + 60 needs a second page; b holds it
    assert eng.cache.length(sa) == 20                              # a refused step changed nothing
    more = eng.step([(sa, [5])]).cpu().numpy()
    close(more, plain_logits(name, a + [5])[-1:], dtype)
    with pytest.raises(CacheFull, match="longest"):
        eng.step([(sb, [1] * 200)])


def test_float32_and_bfloat16_pick_the_same_greedy_tokens():
    for name in ("A", "B"):
        prompts = [rand_tokens(name, 1, 5), rand_tokens(name, 2, 11)]
        out = {}
        for dtype in DTYPES:
            out[dtype] = [r.tokens for r in engine(name, dtype).generate(prompts, max_new_tokens=8)]
        # where they differ, the two logits must be a near tie in the plain implementation
        for p, x, y in zip(prompts, out["float32"], out["bfloat16"]):
            seq = list(p)
            for tx, ty in zip(x, y):
                if tx != ty:
                    l = plain_logits(name, seq)[-1]
                    assert abs(l[tx] - l[ty]) < 2e-2 * np.abs(l).max()
                    break
                seq.append(tx)


def test_no_gpu_library_no_engine(monkeypatch):
    """Without the device library the engine must fail, not fall back."""
    from gpullama3_java_amd.csrc import lib
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib._build, "library_path", lambda: None)
    monkeypatch.setattr(lib._build, "build", lambda: (_ for _ in ()).throw(RuntimeError("hipcc not found")))
    with pytest.raises(RuntimeError, match="hipcc"):
        lib.rmsnorm(torch.zeros(1, 8, device="cuda"), torch.zeros(8, device="cuda"),
                    torch.zeros(1, 8, device="cuda"), 1e-5)


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "bfloat16"), ("D", "bfloat16")])
def test_replayed_graphs_equal_plain_launches(name, dtype):
    """Decode steps replayed from captured graphs, with the batch padded to its bucket and other
    work of the same engine between the replays, give what the same kernels give when launched
    one by one."""
    eager = engine(name, dtype, use_graphs=False, n_slots=16)
    graph = engine(name, dtype, use_graphs=True, n_slots=16)
    assert graph.use_graphs and not eager.use_graphs
    B = 11                                                         # padded to a bucket of 16
    seqs = [rand_tokens(name, 60 + i, 8 + 5 * i + 12) for i in range(B)]
    outs = []
    for eng in (eager, graph):
        slots = [eng.take_slot() for _ in range(B)]
        rows = [[] for _ in range(B)]
        eng.step([(s, q[:8 + 5 * i]) for i, (s, q) in enumerate(zip(slots, seqs))], want="none")
        for k in range(12):
            o = eng.step([(s, [q[8 + 5 * i + k]]) for i, (s, q) in enumerate(zip(slots, seqs))]).cpu().numpy()
            for i in range(B):
                rows[i].append(o[i])
            if k % 4 == 1:                                         # eager work between replays: a prompt elsewhere
                extra = eng.take_slot()
                eng.step([(extra, rand_tokens(name, k, 30))])
                eng.give_back_slot(extra)
        outs.append(rows)
    assert len(graph._graphs) >= 1
    for i in range(B):
        got = np.stack(outs[1][i])
        np.testing.assert_array_equal(got, np.stack(outs[0][i]))
        n0 = 8 + 5 * i
        close(got, plain_logits(name, seqs[i])[n0:n0 + 12], dtype, f"request {i}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_logits_of_a_step_outlive_the_steps_after_it(dtype):
    """A caller may keep what ``step`` returned while it runs further steps of the same batch size
    and context bucket: decode steps are replayed from a captured graph whose own logits buffer
    the next replay overwrites, so ``step`` hands out a tensor of its own."""
    name = "B"
    eng = engine(name, dtype)
    assert eng.use_graphs
    a, b = rand_tokens(name, 40, 30), rand_tokens(name, 41, 21)
    ref_a, ref_b = plain_logits(name, a), plain_logits(name, b)
    sa, sb = eng.take_slot(), eng.take_slot()
    eng.step([(sa, a[:20]), (sb, b[:11])], want="none")
    kept = [eng.step([(sa, [a[20 + i]]), (sb, [b[11 + i]])]) for i in range(10)]    # ten results held at once
    torch.cuda.synchronize()
    assert len({k.data_ptr() for k in kept}) == 10
    for i, k in enumerate(kept):
        close(k.cpu().numpy(), np.stack([ref_a[20 + i], ref_b[11 + i]]), dtype, f"step {i} read after step 9")


def test_a_decode_step_costs_the_host_little():
    """The host's share of a decode step at batch 8 with the context of a real Llama 3.2 config.json
    (131072 positions: 2,048 pages a sequence): no page number is uploaded per step (the block tables
    live on the device, a row per slot), the step's tokens, positions and slots travel in one launch.
    A one-layer model, so that the device is not what the loop waits for. The bound is three times
    what the box measures, not the figure itself (it is printed)."""
    import time
    from gpullama3_java_amd.engine import Engine
    cfg = {"architectures": ["LlamaForCausalLM"], "hidden_size": 256, "intermediate_size": 512, "num_hidden_layers": 1,
           "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 64, "vocab_size": 1024,
           "max_position_embeddings": 131072, "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "tie_word_embeddings": True}
    eng = Engine.random(cfg, 0, dtype="bfloat16", max_tokens=8 * 4096, n_slots=8)
    assert eng.cache.max_pages_per_seq == 2048
    slots = [eng.take_slot() for _ in range(8)]
    eng.step([(s, [1, 2, 3]) for s in slots], want="none")
    entries = [(s, [5]) for s in slots]
    for _ in range(50):
        eng.step(entries)
    torch.cuda.synchronize()
    best = 1e9
    for _ in range(3):
        t0 = time.perf_counter()
        for _ in range(1000):
            eng.step(entries)
        best = min(best, (time.perf_counter() - t0) / 1000)
        torch.cuda.synchronize()
    print(f"host time of a decode step at batch 8: {best * 1e6:.1f} us")
    assert best < 120e-6

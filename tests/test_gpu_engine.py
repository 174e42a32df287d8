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


def test_what_a_step_costs_the_host():
    """The host's share of a step with the context of a real Llama 3.2 config.json (131072 positions: 2,048
    pages a sequence), on a one-layer model so that the device is not what the loop waits for. What is
    asserted is structure, not time: a decode step uploads no page numbers (the block tables live on the
    device, a row per slot; entries travel only when a sequence gets a page), and a prompt's per-token index
    arrays are made on the device from one small copy. The times are printed."""
    import time
    from gpullama3_java_amd.csrc import lib as K
    from gpullama3_java_amd.engine import Engine
    cfg = {"architectures": ["LlamaForCausalLM"], "hidden_size": 256, "intermediate_size": 512, "num_hidden_layers": 1,
           "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 64, "vocab_size": 1024,
           "max_position_embeddings": 131072, "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "tie_word_embeddings": True}
    eng = Engine.random(cfg, 0, dtype="bfloat16", max_tokens=8 * 4096 + 4096, n_slots=9)
    assert eng.cache.max_pages_per_seq == 2048
    slots = [eng.take_slot() for _ in range(8)]
    eng.step([(s, [1, 2, 3]) for s in slots], want="none")
    entries = [(s, [5]) for s in slots]
    for _ in range(50):
        eng.step(entries)
    torch.cuda.synchronize()
    sent = []
    real = K.scatter_i32
    K.scatter_i32 = lambda dst, places, values: sent.append(len(places)) or real(dst, places, values)
    try:
        best = 1e9
        for _ in range(3):
            t0 = time.perf_counter()
            for _ in range(1000):
                eng.step(entries)
            best = min(best, (time.perf_counter() - t0) / 1000)
            torch.cuda.synchronize()
    finally:
        K.scatter_i32 = real
    print(f"host time of a decode step at batch 8: {best * 1e6:.1f} us")
    # 3,053 tokens a sequence: 47 new pages each, sent when they were handed out and never again
    assert sum(sent) == 8 * (-(-3053 // 64) - 1) and len(sent) <= 47
    # a prompt of 2,048 tokens: the time from the call to the first kernel of the model
    s = eng.take_slot()
    toks = np.random.default_rng(0).integers(0, 1024, 2048).tolist()
    eng.step([(s, toks)])
    eng.give_back_slot(s)
    torch.cuda.synchronize()
    marks = []
    real_embed = K.embed
    K.embed = lambda *a, **k: marks.append(time.perf_counter()) or real_embed(*a, **k)
    try:
        s = eng.take_slot()
        t0 = time.perf_counter()
        eng.step([(s, toks)])
        t1 = time.perf_counter()
    finally:
        K.embed = real_embed
    torch.cuda.synchronize()
    print(f"a prompt of 2,048 tokens: {(marks[0] - t0) * 1e6:.0f} us on the host before the model's first kernel, "
          f"{(t1 - t0) * 1e6:.0f} us until the step returns")
    assert eng.cache.length(s) == 2048


def test_sizes_that_the_cache_cannot_hold_are_refused_before_the_weights_are_read(tmp_path, monkeypatch):
    """A head size that is no multiple of 16, or a page that is no multiple of 32 positions, is refused when the
    engine is built, by name, before a weight is read, not by the first kernel of the first step."""
    import gpullama3_java_amd as g
    from gpullama3_java_amd.engine import Engine, engine as engine_module
    cfg = dict(CONFIGS["A"], head_dim=24)
    folder = str(tmp_path / "hs24")
    g.write_random_model(folder, g.config_from_dict(cfg), 1)
    monkeypatch.setattr(engine_module, "load_weights", lambda *a, **k: pytest.fail("the weights were read"))
    with pytest.raises(ValueError, match="head_dim 24"):
        Engine.from_folder(folder, dtype="float32", max_tokens=256)
    with pytest.raises(ValueError, match="page_size 48"):
        Engine.from_folder(model("A")[0], dtype="float32", max_tokens=256, page_size=48)


def test_captured_steps_are_bounded_in_number_and_memory():
    """Every batch bucket and context bucket has a captured step of its own, with its logits and the
    sampler's scratch; an engine keeps ``max_graphs`` of them and drops the least recently used, so a process
    that walks many batch sizes and contexts levels off. Results stay right across the drops."""
    name, dtype = "C", "bfloat16"
    eng = engine(name, dtype, n_slots=8, max_tokens=8 * 1024, max_graphs=4)
    seqs = [rand_tokens(name, 400 + i, 600) for i in range(8)]
    refs = [plain_logits(name, q[:280]) for q in seqs[:2]]
    import gc
    import weakref
    held, keys, made = [], [], {}
    for B in (8, 7, 6, 5, 4, 3):                                # 12 buckets: six batch sizes at two contexts
        for start in (100, 270):
            slots = [eng.take_slot() for _ in range(B)]
            eng.step([(s, q[:start]) for s, q in zip(slots, seqs)], want="none")
            for k in range(3):
                out = eng.step([(s, [q[start + k]]) for s, q in zip(slots, seqs)])
            close(out[:2].cpu().numpy(), np.stack([r[start + 2] for r in refs]), dtype, f"batch {B} from {start}")
            for s in slots:
                eng.give_back_slot(s)
            torch.cuda.synchronize()
            held.append(torch.cuda.memory_allocated())
            keys.append(list(eng._graphs))
            made.update({k: weakref.ref(v) for k, v in eng._graphs.items() if k not in made})
            assert len(eng._graphs) <= 4
    assert len({k for ks in keys for k in ks}) == 12 and keys[-1] == [(4, 256, False), (4, 512, False), (3, 256, False),
                                                                     (3, 512, False)]
    gc.collect()
    assert sorted(k for k, r in made.items() if r() is not None) == sorted(keys[-1])   # the dropped ones are gone,
    assert held[-1] <= held[3] and max(held[4:]) <= held[3] + 65536    # and their memory with them (the first four are the largest)
    # a bucket that was dropped is captured again and gives the same logits
    slots = [eng.take_slot() for _ in range(8)]
    eng.step([(s, q[:100]) for s, q in zip(slots, seqs)], want="none")
    for k in range(3):
        out = eng.step([(s, [q[100 + k]]) for s, q in zip(slots, seqs)])
    close(out[:2].cpu().numpy(), np.stack([r[102] for r in refs]), dtype, "batch 8 again")
    assert (8, 256, False) in eng._graphs and len(eng._graphs) == 4


def test_a_slot_that_is_taken_again_reads_its_own_pages_only():
    """A slot's row of the device's block table keeps the page numbers of the sequence that held it before.
    After the slot is given back and taken again, the row's entries up to the new length are the new pages
    (what lies behind them is never read), the row of the padding entries is still all zero, and the logits
    are the plain implementation's."""
    name = "C"
    eng = engine(name, "float32", n_slots=2, max_tokens=1024)
    long, short = rand_tokens(name, 71, 300), rand_tokens(name, 72, 70)
    a = eng.take_slot()
    eng.step([(a, long)], want="none")
    other = eng.take_slot()
    eng.step([(other, rand_tokens(name, 73, 10))], want="none")
    old = list(eng.cache.slots.pages[a][0])
    eng.give_back_slot(a)
    b = eng.take_slot()
    assert b == a
    got = eng.step([(b, short)], want="all").cpu().numpy()
    got2 = eng.step([(b, [short[-1]])]).cpu().numpy()            # (a decode step from the captured graph reads the same row)
    table = eng.cache.device_table(0).cpu().numpy()
    new = eng.cache.slots.pages[b][0]
    assert len(new) == 2 and table[b, :2].tolist() == new and table[b, 2:5].tolist() == old[2:5]
    assert not table[eng.cache.sink_slot].any()
    close(got, plain_logits(name, short), "float32")
    close(got2, plain_logits(name, short + [short[-1]])[-1:], "float32")


@pytest.mark.parametrize("name", ["B", "D"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_one_step_with_a_decode_token_a_fresh_prompt_and_a_chunk(name, dtype):
    """One step may bring any mix: a single token of a sequence that the cache already holds, another
    sequence's whole prompt, and a chunk of a third that goes on. The generation loop never forms such a
    step; a caller of ``step`` (the replay program's users) can. Then a decode step of all three."""
    old, new, old2 = rand_tokens(name, 301, 70 + 2), rand_tokens(name, 302, 37 + 1), rand_tokens(name, 303, 130 + 5 + 1)
    eng = engine(name, dtype, n_slots=4)
    s_old, s_old2 = eng.take_slot(), eng.take_slot()
    eng.step([(s_old, old[:70]), (s_old2, old2[:130])], want="none")
    s_new = eng.take_slot()
    out = eng.step([(s_old, [old[70]]), (s_new, new[:37]), (s_old2, old2[130:135])], want="all").cpu().numpy()
    assert out.shape[0] == 1 + 37 + 5
    refs = [plain_logits(name, q) for q in (old, new, old2)]
    close(out[:1], refs[0][70:71], dtype, "the decode token among a prompt and a chunk")
    close(out[1:38], refs[1][:37], dtype, "the fresh prompt among a decode token and a chunk")
    close(out[38:], refs[2][130:135], dtype, "the chunk among a decode token and a prompt")
    assert [eng.cache.length(s) for s in (s_old, s_new, s_old2)] == [71, 37, 135]
    out = eng.step([(s_old, [old[71]]), (s_new, [new[37]]), (s_old2, [old2[135]])]).cpu().numpy()
    close(out, np.stack([refs[0][71], refs[1][37], refs[2][135]]), dtype, "the decode step after the mixed step")


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_weights_held_once_give_the_same_logits(name):
    """A bfloat16 engine keeps the matrices that decode steps read in the matrix cores' order ALONE where a copy
    can stand for them (whole steps of 64 k): the head (A: with the tied embedding), the stacked q, k, v rows, the
    output and the down projection. Every way a step reads them gives what an engine that keeps both orders gives,
    bit for bit: a prompt with all rows wanted (the tiled products), a chunk, single tokens (the folded norms), a
    batch of 12 and of 40 (the kernel of whole lines); ``weights()`` hands back the stored order under the stored names."""
    from gpullama3_java_amd.csrc import lib
    from safetensors.torch import load_file
    import os
    once, both = engine(name, "bfloat16", n_slots=64, max_tokens=8192), engine(name, "bfloat16", weight_copies="both",
                                                                                n_slots=64, max_tokens=8192)
    cfg = CONFIGS[name]
    d, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    mixer, ffn = once.model.blocks[0].mixer, once.model.blocks[0].ffn
    # which matrices a copy can stand for follows from the sizes alone
    assert lib.held_once(once.model.head) == (d % 64 == 0 and V % 16 == 0)
    assert lib.held_once(mixer.w_qkv) == (d % 64 == 0 and mixer.w_qkv.shape[0] % 16 == 0)
    from gpullama3_java_amd.parts import ops
    assert lib.held_once(mixer.w_o) == ops.can_hold_once(both.model.blocks[0].mixer.w_o)
    assert lib.held_once(ffn.w_down) == ops.can_hold_once(both.model.blocks[0].ffn.w_down)
    if name == "A":
        assert lib.held_once(once.model.head) and lib.held_once(mixer.w_qkv) and lib.held_once(mixer.w_o) and lib.held_once(ffn.w_down)
        assert (once.model.embedding is once.model.head) == cfg["tie_word_embeddings"]
        assert once.model.head.data_ptr() == once.model.head.tiled.data_ptr() and mixer.w_q is None
    for m in (both.model.head, both.model.blocks[0].mixer.w_qkv, both.model.blocks[0].ffn.w_down):
        assert not lib.held_once(m)
    folder, _, _ = model(name)
    stored = load_file(os.path.join(folder, "model.safetensors"))
    given = once.weights()
    assert set(given) == set(stored)
    for k, v in stored.items():
        assert torch.equal(given[k].cpu(), v.to(given[k].dtype)), k
    n = min(100, cfg["max_position_embeddings"] - 8)
    toks = rand_tokens(name, 5, n)
    outs = []
    for eng in (once, both):
        s = eng.take_slot()
        got = [eng.step([(s, toks[:n - 10])], want="all"), eng.step([(s, toks[n - 10:n - 5])]), eng.step([(s, toks[n - 5:n - 4])])]
        got += [eng.step([(s, [t])]) for t in toks[n - 4:]]
        for B in (12, 40):
            many = [eng.take_slot() for _ in range(B)]
            eng.step([(m, toks[i:i + 3]) for i, m in enumerate(many)], want="none")
            got.append(eng.step([(m, [toks[i]]) for i, m in enumerate(many)]))
            for m in many:
                eng.give_back_slot(m)
        outs.append([g_.clone() for g_ in got])
    for i, (u, v) in enumerate(zip(*outs)):
        assert torch.equal(u, v), f"{name}: result {i} differs between weights held once and both orders"
    close(outs[0][0].cpu().numpy(), plain_logits(name, toks[:n - 10]), "bfloat16", f"{name} held once, whole")

"""The generation loop's decisions, with a backend that needs no GPU."""
import numpy as np
import pytest

import plain_llama as P
from gpullama3_java_amd.cache import Cache, CacheFull, KVNeed
from gpullama3_java_amd.engine.generate import Request, RunMetrics, generate, plan_batch
from gpullama3_java_amd.sampling import SamplingParams, sample_host, uniform

V = 50


class FakeBackend:
    """Logits are a fixed function of a sequence's tokens, so every request has one
    right answer whatever it is batched with. The real cache does the bookkeeping."""

    def __init__(self, max_tokens=1024, max_context=64, n_slots=4):
        import torch
        self.cache = Cache([KVNeed(1, 16)], [None], max_tokens, max_context, n_slots, torch.float32, "cpu", 32)
        self.max_context, self.n_slots, self.page_size = max_context, n_slots, 32
        self.seqs = {}
        self.steps = []          # per step: list of (slot, n tokens)
        self.taken = []

    def tokens_capacity(self):
        return self.cache.tokens_free()

    def slots_free(self):
        return self.cache.slots.n_free

    def take_slot(self):
        s = self.cache.take_slot()
        assert s not in self.seqs
        self.seqs[s] = []
        self.taken.append(s)
        return s

    def give_back_slot(self, s):
        self.cache.give_back_slot(s)
        del self.seqs[s]

    @staticmethod
    def logits_of(seq):
        rng = np.random.default_rng([len(seq), sum(seq) % 9973, seq[-1]])
        return rng.standard_normal(V).astype(np.float32) * 3

    def step(self, entries):
        self.cache.reserve({s: len(t) for s, t in entries})
        rows = []
        for s, toks in entries:
            self.cache.advance(s, len(toks))
            self.seqs[s].extend(toks)
            rows.append(self.logits_of(self.seqs[s]))
        self.steps.append([(s, len(t)) for s, t in entries])
        return np.stack(rows)

    def sample(self, logits, temperatures, top_ps, uniforms):
        return [sample_host(l, t, p, u) for l, t, p, u in zip(logits, temperatures, top_ps, uniforms)]


class RunBackend(FakeBackend):
    """Runs several decode steps before it reports, as an engine that samples on the device does."""
    decode_run_length = 4

    def decode_run(self, entries, n, temperatures, top_ps, uniforms):
        assert 1 <= n <= self.decode_run_length
        out = []
        cur = list(entries)
        self.runs.append(n)
        for k in range(n):
            logits = self.step([(s, [t]) for s, t in cur])
            toks = self.sample(logits, temperatures, top_ps, uniforms[k])
            out.append(toks)
            cur = [(s, t) for (s, _), t in zip(cur, toks)]
        return out

    def __init__(self, *a, **kw):
        super().__init__(*a, **kw)
        self.runs = []


def alone(prompt, n, sampling=SamplingParams(), stops=(), index=0, max_context=64):
    seq, out = list(prompt), []
    while len(out) < n:
        tok = P.sample(FakeBackend.logits_of(seq), sampling.temperature, sampling.top_p,
                       uniform(sampling.seed, index, len(prompt) + len(out)))
        out.append(tok)
        if tok in stops or len(seq) >= max_context:
            break
        seq.append(tok)
    return out


def prompts(lens, seed=0):
    rng = np.random.default_rng(seed)
    return [rng.integers(0, V, n).tolist() for n in lens]


def test_unequal_prompts_in_one_step_then_one_token_each():
    be = FakeBackend()
    ps = prompts([5, 11, 3])
    res = generate(be, [Request(p, 6) for p in ps])
    assert [r.tokens for r in res] == [alone(p, 6) for p in ps]
    assert all(r.finish_reason == "length" for r in res)
    assert sorted(n for _, n in be.steps[0]) == [3, 5, 11]                 # whole prompts, one step
    assert all(n == 1 for st in be.steps[1:] for _, n in st) and len(be.steps) == 6
    assert not be.seqs and be.cache.slots.live == set()                    # every slot came back


def test_stop_token_ends_only_its_own_sequence_and_is_kept():
    be = FakeBackend()
    ps = prompts([4, 9, 6], seed=1)
    free_run = [alone(p, 12) for p in ps]
    stop = free_run[1][3]                                # request 1 meets it at its 4th token (or earlier)
    res = generate(be, [Request(p, 12, stop_ids=frozenset([stop])) for p in ps])
    for r, p in zip(res, ps):
        want = alone(p, 12, stops=(stop,))
        assert r.tokens == want
        assert r.finish_reason == ("stop" if want[-1] == stop else "length")
    assert res[1].tokens[-1] == stop and len(res[1].tokens) <= 4
    # a stop token inside a prompt stops nothing
    res2 = generate(FakeBackend(), [Request([stop, stop] + ps[0], 3)])
    assert len(res2[0].tokens) >= 1 and res2[0].tokens == alone([stop, stop] + ps[0], 3)


def test_finished_sequences_leave_the_batch_at_once():
    be = FakeBackend()
    ps = prompts([4, 4, 4], seed=2)
    res = generate(be, [Request(ps[0], 2), Request(ps[1], 7), Request(ps[2], 4)])
    assert [len(r.tokens) for r in res] == [2, 7, 4]
    assert [len(st) for st in be.steps] == [3, 3, 2, 2, 1, 1, 1]


def test_batches_follow_one_another_and_slots_are_used_again():
    be = FakeBackend(n_slots=2)
    ps = prompts([3, 8, 5, 2, 7], seed=3)
    res = generate(be, [Request(p, 4) for p in ps])
    assert [r.tokens for r in res] == [alone(p, 4, index=i) for i, p in enumerate(ps)]   # request order kept
    assert len(be.taken) == 5 and set(be.taken) == {0, 1}                  # five requests over two slots
    assert [len(st) for st in be.steps if st[0][1] > 1 or len(st) > 0][0] == 2
    firsts = [st for st in be.steps if any(n > 1 for _, n in st)]
    assert [len(st) for st in firsts] == [2, 2, 1]                         # nobody joins a running batch


def test_batch_is_cut_by_the_cache_size():
    reqs = [Request([1] * 20, 13), Request([1] * 20, 13), Request([1] * 5, 4)]
    assert plan_batch(reqs, 0, 8, capacity=64, page_size=16, max_context=64) == 2     # 32 + 32 tokens
    assert plan_batch(reqs, 0, 1, capacity=640, page_size=16, max_context=64) == 1
    assert plan_batch(reqs, 2, 8, capacity=16, page_size=16, max_context=64) == 1
    with pytest.raises(ValueError, match="cache holds"):
        plan_batch(reqs, 0, 8, capacity=16, page_size=16, max_context=64)
    be = FakeBackend(max_tokens=64, n_slots=4)
    res = generate(be, reqs)
    assert [len(r.tokens) for r in res] == [13, 13, 4]


def test_context_bound_and_bad_prompts():
    be = FakeBackend(max_context=16)
    p = prompts([14], seed=4)[0]
    res = generate(be, [Request(p, 10)])
    # 14 held; tokens 1 and 2 are fed back (15, 16 held); the third is sampled but cannot be fed
    assert len(res[0].tokens) == 3 and res[0].finish_reason == "length"
    assert res[0].tokens == alone(p, 10, max_context=16)[:3]
    full = prompts([16], seed=5)[0]
    assert len(generate(FakeBackend(max_context=16), [Request(full, 5)])[0].tokens) == 1
    with pytest.raises(ValueError, match="exceeds the context"):
        generate(be, [Request([1] * 17, 1)])
    with pytest.raises(ValueError, match="empty"):
        generate(be, [Request([], 1)])
    assert generate(be, [Request(p, 0)])[0].tokens == []
    assert be.cache.slots.live == set()


def test_sampled_tokens_do_not_depend_on_batch_mates():
    sp = SamplingParams(0.8, 0.95, seed=7)
    ps = prompts([6, 3, 9], seed=6)
    together = generate(FakeBackend(), [Request(p, 8, sp) for p in ps])
    for i, p in enumerate(ps):
        assert together[i].tokens == alone(p, 8, sp, index=i)
    other = generate(FakeBackend(), [Request(p, 8, SamplingParams(0.8, 0.95, seed=8)) for p in ps])
    assert [r.tokens for r in other] != [r.tokens for r in together]


def test_callback_and_metrics():
    seen = []
    m = RunMetrics()
    ps = prompts([4, 6], seed=8)
    res = generate(FakeBackend(), [Request(p, 3) for p in ps], on_token=lambda i, t: seen.append((i, t)), metrics=m)
    assert [t for i, t in seen if i == 0] == res[0].tokens and [t for i, t in seen if i == 1] == res[1].tokens
    assert m.prompt_tokens == 10 and m.generated_tokens == 6 and m.decode_steps == 2


def test_a_failing_step_gives_the_slots_back():
    be = FakeBackend(max_tokens=32, n_slots=4)
    be.tokens_capacity = lambda: 10**6          # let the plan through so that the step itself fails
    with pytest.raises(CacheFull):
        generate(be, [Request([1] * 30, 2), Request([1] * 30, 2)])
    assert be.cache.slots.live == set() and be.cache.groups[0].pool.n_free == 1      # one page of 32 positions


def test_runs_of_steps_give_the_same_tokens_and_respect_every_budget():
    sp = SamplingParams(0.9, 0.9, seed=3)
    ps = prompts([5, 11, 3, 8], seed=9)
    news = [6, 13, 2, 9]
    free = [alone(p, n, sp, index=i) for i, (p, n) in enumerate(zip(ps, news))]
    stop = free[1][7]
    reqs = [Request(p, n, sp, frozenset([stop])) for p, n in zip(ps, news)]
    plain = generate(FakeBackend(), reqs)
    be = RunBackend()
    got = generate(be, reqs)
    assert [r.tokens for r in got] == [r.tokens for r in plain]
    assert [r.finish_reason for r in got] == [r.finish_reason for r in plain]
    assert max(be.runs) == 4 and be.cache.slots.live == set()
    # no sequence was stepped past its budget: the cache never held more than prompt + new - 1 tokens
    tight = RunBackend(max_context=16)
    p = prompts([10], seed=10)[0]
    out = generate(tight, [Request(p, 50, sp)])[0]
    assert len(out.tokens) == 7 and out.finish_reason == "length"         # 16 - 10 fed back, one more sampled


def test_a_sequence_that_goes_on_keeps_its_slot_and_runs_single_steps():
    """A request that names a slot continues that slot's sequence: the slot is neither taken nor
    given back, its steps are single ones (no token sampled after the sequence's end may reach a
    slot that is kept), and the result is the one of the whole sequence in one request."""
    be = RunBackend()
    prompt = [5, 9, 2, 7]
    whole = generate(RunBackend(), [Request(prompt, 9, SamplingParams())])[0].tokens
    s = be.take_slot()
    first = generate(be, [Request(prompt, 4, SamplingParams(), slot=s, cached=0)])[0].tokens
    assert first == whole[:4] and be.runs == [] and s in be.seqs
    assert be.cache.length(s) == len(prompt) + 3            # the last sampled token has not been fed
    rest = generate(be, [Request([first[-1]], 5, SamplingParams(), slot=s, cached=be.cache.length(s))])[0].tokens
    assert first + rest == whole and be.cache.slots.n_free == be.n_slots - 1
    be.give_back_slot(s)
    # with temperature too: a draw is keyed by the token's position in its sequence, so a sequence that
    # goes on over two calls draws what it would have drawn in one, and no turn repeats another's numbers
    hot = SamplingParams(temperature=1.5, top_p=1.0, seed=4)
    whole = generate(RunBackend(), [Request(prompt, 9, hot)])[0].tokens
    s = be.take_slot()
    first = generate(be, [Request(prompt, 4, hot, slot=s, cached=0)])[0].tokens
    rest = generate(be, [Request([first[-1]], 5, hot, slot=s, cached=be.cache.length(s))])[0].tokens
    assert first + rest == whole
    seen = []
    import sys
    G = sys.modules[generate.__module__]
    real = G.uniform
    try:
        G.uniform = lambda seed, r, step: seen.append(step) or real(seed, r, step)
        generate(be, [Request([rest[-1]], 3, hot, slot=s, cached=be.cache.length(s))])
        generate(be, [Request([7], 3, hot, slot=s, cached=be.cache.length(s))])
    finally:
        G.uniform = real
    assert len(seen) == len(set(seen))                      # two turns on one state: no uniform is drawn twice
    be.give_back_slot(s)
    with pytest.raises(ValueError, match="no slot"):
        generate(be, [Request([1], 2, SamplingParams(), cached=3)])
    with pytest.raises(ValueError, match="slot of their own"):
        generate(be, [Request([1], 2, SamplingParams(), slot=0, cached=0), Request([1], 2, SamplingParams())])

"""Each part alone, the run order as data, and a toy mixer with state of its own that is
registered, built and stepped without a change to the framework's files."""
import json
import math
import os
from dataclasses import dataclass, field
from types import SimpleNamespace

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

import plain_llama as P
from gpu_helpers import close, model, rand_tokens
from tiny import TINY_A

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}


class Harness:
    """What a part needs of an engine: a cache, a workspace, dtype and device."""

    def __init__(self, kv_needs, state_needs, dtype, max_tokens=1024, n_slots=4):
        from gpullama3_java_amd.cache import Cache
        from gpullama3_java_amd.engine.context import Workspace
        self.dtype, self.device = TD[dtype], torch.device(DEV)
        self.cache = Cache(kv_needs, state_needs, max_tokens, 512, n_slots, self.dtype, self.device)
        self.workspace = Workspace(self.device)

    def context(self, entries):
        """entries: [(slot, n new tokens)] -> a step context (no token ids: parts do not need them)."""
        from gpullama3_java_amd.engine.context import StepContext
        slots = [s for s, _ in entries]
        q_lens = [n for _, n in entries]
        before = [self.cache.length(s) for s in slots]
        self.cache.reserve(dict(entries))
        ctx = StepContext(self, sum(q_lens), len(entries), q_lens, before, slots, all(n == 1 for n in q_lens),
                          max(q_lens), max(b + n for b, n in zip(before, q_lens)))
        i32 = lambda a: torch.as_tensor(np.asarray(a, np.int32)).to(DEV)
        ctx.positions = i32(np.concatenate([np.arange(b, b + n) for b, n in zip(before, q_lens)]))
        ctx.seq_of_token = i32(np.concatenate([[i] * n for i, n in enumerate(q_lens)]))
        ctx.cu_seqlens = i32(np.concatenate([[0], np.cumsum(q_lens)]))
        ctx.kv_before, ctx.slot_ids = i32(before), i32(slots)
        # the block tables as the engine passes them: the cache's own, a row per slot, named by slot numbers
        self.cache.flush_tables()
        ctx._tables = [self.cache.device_table(g) for g in range(len(self.cache.groups))]
        ctx.table_rows = i32(np.concatenate([[s] * n for s, n in entries])) if entries else None
        ctx.seq_rows = ctx.slot_ids
        for s, n in entries:
            self.cache.advance(s, n)
        return ctx


def stored(a, dtype):
    return torch.as_tensor(np.asarray(a, np.float32)).to(TD[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_part(dtype):
    from gpullama3_java_amd.config import NormSpec
    from gpullama3_java_amd.parts import build_part
    rng = np.random.default_rng(0)
    part = build_part("norm", NormSpec(dim=100, eps=1e-3, names={"weight": "w"}), dtype=TD[dtype])
    assert {k: v.shape for k, v in part.tensors().items()} == {"w": (100,)}
    w = stored(1 + 0.3 * rng.standard_normal(100), dtype)
    part.load({"w": w.to(DEV)})
    x = rng.standard_normal((7, 100)).astype(np.float32) * 0.01        # small: eps matters
    out = part(Harness([], [], dtype).context([]) if False else _ctx_only(dtype), torch.as_tensor(x).to(DEV))
    ref = P.rmsnorm(x, w.float().numpy(), 1e-3)
    np.testing.assert_allclose(out.float().cpu().numpy(), ref, atol=(1e-6 if dtype == "float32" else 5e-3) * np.abs(ref).max())


def _ctx_only(dtype):
    from gpullama3_java_amd.cache import KVNeed
    h = Harness([KVNeed(1, 16)], [None], dtype)
    return h.context([(h.cache.take_slot(), 7)])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, Kh, hs, d, pairing, window", [(6, 2, 16, 40, "adjacent", None), (3, 1, 48, 72, "half", None),
                                                           (4, 4, 32, 64, "half", 20)])
def test_attention_part_whole_and_in_pieces(dtype, H, Kh, hs, d, pairing, window):
    from gpullama3_java_amd.config import AttentionSpec, RotarySpec
    from gpullama3_java_amd.parts import RunInfo, build_part
    rng = np.random.default_rng(H * d)
    names = {k: k for k in "qkvo"}
    spec = AttentionSpec(hidden=d, n_heads=H, n_kv_heads=Kh, head_dim=hs, window=window, names=names,
                         position=RotarySpec(head_dim=hs, theta=1000.0, pairing=pairing, max_positions=512))
    part = build_part("mixer", spec, dtype=TD[dtype], device=torch.device(DEV))
    assert {k: tuple(v.shape) for k, v in part.tensors().items()} == {
        "q": (H * hs, d), "k": (Kh * hs, d), "v": (Kh * hs, d), "o": (d, H * hs)}
    W = {n: stored(rng.standard_normal(s.shape) * 0.3, dtype) for n, s in part.tensors().items()}
    part.load({n: t.to(DEV) for n, t in W.items()})
    Wn = {n: t.float().numpy() for n, t in W.items()}
    n_tok = [70, 9]
    hs_in = [stored(rng.standard_normal((n, d)), dtype) for n in n_tok]
    cos, sin = P.rope_table(512, hs, 1000.0)

    def plain(h):
        h = h.float().numpy()
        T = len(h)
        pos = np.arange(T)
        q = P.rope_rotate(P.linear(h, Wn["q"]).reshape(T, H, hs), pos, cos, sin, pairing)
        k = P.rope_rotate(P.linear(h, Wn["k"]).reshape(T, Kh, hs), pos, cos, sin, pairing)
        v = P.linear(h, Wn["v"]).reshape(T, Kh, hs)
        return P.linear(P.attention(q, k, v, window=window).reshape(T, H * hs), Wn["o"])

    refs = [plain(h) for h in hs_in]
    harness = Harness([part.kv_need()], [part.state_need()], dtype)
    assert part.kv_need().window == window and part.state_need() is None
    run = RunInfo(entry=0, kv_entry=0, writes_kv=True)
    slots = [harness.cache.take_slot() for _ in n_tok]
    # both sequences whole in one step; the output is added into x
    x = torch.ones(sum(n_tok), d, device=DEV)
    part.forward(harness.context(list(zip(slots, n_tok))), torch.cat(hs_in).to(DEV), x, run)
    ref = np.concatenate(refs)
    t = (2e-5 if dtype == "float32" else 2e-2) * np.abs(ref).max()
    np.testing.assert_allclose(x.cpu().numpy() - 1, ref, atol=t)
    # again in pieces: 60 + 1 + ... for the first, the second one token at a time
    for s in slots:
        harness.cache.give_back_slot(s)
    s0 = harness.cache.take_slot()
    outs = []
    for lo, hi in [(0, 60)] + [(i, i + 1) for i in range(60, 70)]:
        x = torch.zeros(hi - lo, d, device=DEV)
        part.forward(harness.context([(s0, hi - lo)]), hs_in[0][lo:hi].to(DEV), x, run)
        outs.append(x.cpu().numpy())
    np.testing.assert_allclose(np.concatenate(outs), refs[0], atol=t)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_with_a_window_after_its_first_pages_were_given_back(dtype):
    """A group with a window gives back the pages that lie behind it; the attention of later tokens,
    in chunks and one by one, is that of the plain implementation over the whole sequence, and the
    sequence holds two or three pages however long it grows."""
    from gpullama3_java_amd.config import AttentionSpec, RotarySpec
    from gpullama3_java_amd.parts import RunInfo, build_part
    rng = np.random.default_rng(4)
    H, Kh, hs, d, window, n = 4, 2, 32, 64, 50, 420
    spec = AttentionSpec(hidden=d, n_heads=H, n_kv_heads=Kh, head_dim=hs, window=window, names={k: k for k in "qkvo"},
                         position=RotarySpec(head_dim=hs, theta=1000.0, pairing="half", max_positions=512))
    part = build_part("mixer", spec, dtype=TD[dtype], device=torch.device(DEV))
    W = {k: stored(rng.standard_normal(s_.shape) * 0.3, dtype) for k, s_ in part.tensors().items()}
    part.load({k: t.to(DEV) for k, t in W.items()})
    Wn = {k: t.float().numpy() for k, t in W.items()}
    h = stored(rng.standard_normal((n, d)), dtype)
    hn = h.float().numpy()
    cos, sin = P.rope_table(512, hs, 1000.0)
    pos = np.arange(n)
    q = P.rope_rotate(P.linear(hn, Wn["q"]).reshape(n, H, hs), pos, cos, sin, "half")
    k = P.rope_rotate(P.linear(hn, Wn["k"]).reshape(n, Kh, hs), pos, cos, sin, "half")
    v = P.linear(hn, Wn["v"]).reshape(n, Kh, hs)
    ref = P.linear(P.attention(q, k, v, window=window).reshape(n, H * hs), Wn["o"])
    harness = Harness([part.kv_need()], [None], dtype, max_tokens=64 * 5)    # five pages for 420 tokens
    slot = harness.cache.take_slot()
    run = RunInfo(entry=0, kv_entry=0, writes_kv=True)
    outs, held = [], []
    cuts = [0, 100, 101, 102, 190, 260, 261, 300, 301, 302, 303, 420]       # chunks, and tokens one by one
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        x = torch.zeros(hi - lo, d, device=DEV)
        part.forward(harness.context([(slot, hi - lo)]), h[lo:hi].to(DEV), x, run)
        outs.append(x.cpu().numpy())
        held.append(sum(1 for p_ in harness.cache.slots.pages[slot][0] if p_))
    assert max(held) <= 3 and harness.cache.slots.pages[slot][0][0] == 0
    np.testing.assert_allclose(np.concatenate(outs), ref, atol=(2e-5 if dtype == "float32" else 2e-2) * np.abs(ref).max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_feed_forward_part(dtype):
    from gpullama3_java_amd.config import GatedFeedForwardSpec
    from gpullama3_java_amd.parts import build_part
    rng = np.random.default_rng(2)
    d, F = 72, 200
    part = build_part("ffn", GatedFeedForwardSpec(hidden=d, intermediate=F, names={"gate": "g", "up": "u", "down": "dn"}),
                      dtype=TD[dtype], device=torch.device(DEV))
    assert {k: tuple(v.shape) for k, v in part.tensors().items()} == {"g": (F, d), "u": (F, d), "dn": (d, F)}
    W = {n: stored(rng.standard_normal(s.shape) * 0.2, dtype) for n, s in part.tensors().items()}
    weights = {n: t.to(DEV) for n, t in W.items()}
    part.load(weights)
    assert torch.equal(weights["u"].cpu(), W["u"])                       # stacked, still addressable by name
    h = stored(rng.standard_normal((11, d)), dtype)
    x = torch.full((11, d), 2.0, device=DEV)
    part.forward(_ctx_only(dtype), h.to(DEV), x)
    ref = P.feed_forward(h.float().numpy(), *(W[n].float().numpy() for n in ("g", "u", "dn")))
    np.testing.assert_allclose(x.cpu().numpy() - 2, ref, atol=(2e-5 if dtype == "float32" else 2e-2) * np.abs(ref).max())
    with pytest.raises(ValueError, match="relu"):
        build_part("ffn", GatedFeedForwardSpec(hidden=d, intermediate=F, activation="relu"), dtype=TD[dtype], device=DEV)
    # the other activation, and biases on all three products: a description's matter, no other part
    names = {"gate": "g", "up": "u", "down": "dn", "gate_bias": "gb", "up_bias": "ub", "down_bias": "db"}
    part = build_part("ffn", GatedFeedForwardSpec(hidden=d, intermediate=F, activation="gelu_tanh", names=names),
                      dtype=TD[dtype], device=DEV)
    assert {k: tuple(v.shape) for k, v in part.tensors().items()} == {"g": (F, d), "u": (F, d), "dn": (d, F), "gb": (F,),
                                                              "ub": (F,), "db": (d,)}
    Wb = dict(W, gb=stored(rng.standard_normal(F), "float32"), ub=stored(rng.standard_normal(F), "float32"),
              db=stored(rng.standard_normal(d), "float32"))
    part.load({k: v.to(DEV) for k, v in Wb.items()})
    for rows in (11, 40, 150):                                                # the kernels for few rows, 33 to 64, many
        h = stored(rng.standard_normal((rows, d)), dtype)
        x = torch.full((rows, d), 2.0, device=DEV)
        part.forward(_ctx_only(dtype), h.to(DEV), x)
        f = lambda n: Wb[n].float().numpy().astype(np.float64)
        g = h.float().numpy() @ f("g").T + f("gb")
        act = 0.5 * g * (1 + np.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3))) * (h.float().numpy() @ f("u").T + f("ub"))
        if dtype == "bfloat16":
            act = torch.as_tensor(act).to(torch.bfloat16).double().numpy()
        ref = act @ f("dn").T + f("db")
        np.testing.assert_allclose(x.cpu().numpy() - 2, ref, atol=(2e-5 if dtype == "float32" else 2e-2) * np.abs(ref).max(),
                                   err_msg=f"{rows} rows")


def test_rotary_part_tables():
    """The position encoding alone: its tables are the plain implementation's, with and without the
    llama3 rule; sizes chosen so that all three branches of the rule are taken."""
    from gpullama3_java_amd.config import Llama3RopeScaling, RotarySpec
    from gpullama3_java_amd.parts import build_part
    for hs, theta, scaling in [(48, 10000.0, None), (64, 500000.0, (32.0, 1.0, 4.0, 8192)), (16, 1000.0, (8.0, 2.0, 3.0, 100))]:
        sc = Llama3RopeScaling(*scaling) if scaling else None
        part = build_part("position", RotarySpec(head_dim=hs, theta=theta, scaling=sc, pairing="adjacent", max_positions=300),
                          device=torch.device(DEV))
        plain_sc = None if not scaling else dict(zip(("factor", "low_freq_factor", "high_freq_factor",
                                                      "original_max_position_embeddings"), scaling))
        cos, sin = P.rope_table(300, hs, theta, plain_sc)
        assert part.rot_dim == hs and part.adjacent and part.cos.shape == (300, hs // 2)
        np.testing.assert_array_equal(part.cos.cpu().numpy(), cos)
        np.testing.assert_array_equal(part.sin.cpu().numpy(), sin)
        if scaling:
            f0, f1 = P.rope_frequencies(hs, theta, None), P.rope_frequencies(hs, theta, plain_sc)
            kinds = {"kept" if b == a else "divided" if b == np.float32(a / np.float32(scaling[0])) else "between"
                     for a, b in zip(f0, f1)}
            assert {"kept", "divided"} <= kinds
    with pytest.raises(ValueError, match="even"):
        build_part("position", RotarySpec(head_dim=15, max_positions=8), device=torch.device(DEV))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_tok", [9, 50, 150])
def test_block_part(dtype, n_tok):
    """The arrangement alone: x += mixer(norm(x)); x += ffn(norm(x)), at step sizes that take the
    folded norms (few rows), the sliced products (33 to 64 rows) and the kernels of their own."""
    from gpullama3_java_amd.config import AttentionSpec, BlockSpec, GatedFeedForwardSpec, NormSpec, RotarySpec
    from gpullama3_java_amd.parts import RunInfo, build_part
    rng = np.random.default_rng(n_tok)
    d, H, Kh, hs, F = 80, 4, 2, 32, 144
    spec = BlockSpec(kind="prenorm",
                     mixer_norm=NormSpec(dim=d, eps=1e-4, names={"weight": "n1"}),
                     mixer=AttentionSpec(hidden=d, n_heads=H, n_kv_heads=Kh, head_dim=hs, names={k: k for k in "qkvo"},
                                         position=RotarySpec(head_dim=hs, theta=300.0, pairing="half", max_positions=512)),
                     ffn_norm=NormSpec(dim=d, eps=1e-4, names={"weight": "n2"}),
                     ffn=GatedFeedForwardSpec(hidden=d, intermediate=F, names={"gate": "g", "up": "u", "down": "dn"}))
    block = build_part("block", spec, dtype=TD[dtype], device=torch.device(DEV))
    shapes = {}
    for p_ in block.parts():
        shapes.update({n: t.shape for n, t in p_.tensors().items()})
    assert set(shapes) == {"n1", "n2", "q", "k", "v", "o", "g", "u", "dn"}
    W = {n: stored(1 + 0.2 * rng.standard_normal(sh) if n in ("n1", "n2") else rng.standard_normal(sh) * 0.15, dtype)
         for n, sh in shapes.items()}
    weights = {n: t.to(DEV) for n, t in W.items()}
    for p_ in block.parts():
        p_.load(weights)
    Wn = {n: t.float().numpy() for n, t in W.items()}
    x0 = rng.standard_normal((n_tok, d)).astype(np.float32)
    cos, sin = P.rope_table(512, hs, 300.0)
    pos = np.arange(n_tok)
    h = P.rmsnorm(x0, Wn["n1"], 1e-4)
    q = P.rope_rotate(P.linear(h, Wn["q"]).reshape(n_tok, H, hs), pos, cos, sin, "half")
    k = P.rope_rotate(P.linear(h, Wn["k"]).reshape(n_tok, Kh, hs), pos, cos, sin, "half")
    v = P.linear(h, Wn["v"]).reshape(n_tok, Kh, hs)
    x1 = x0 + P.linear(P.attention(q, k, v).reshape(n_tok, H * hs), Wn["o"])
    ref = x1 + P.feed_forward(P.rmsnorm(x1, Wn["n2"], 1e-4), Wn["g"], Wn["u"], Wn["dn"])
    for fuse in ([False, True] if dtype == "bfloat16" else [False]):
        harness = Harness([block.mixer.kv_need()], [None], dtype)
        harness.fuse = fuse                                                  # as the engine sets it for known parts
        harness.spec = SimpleNamespace(hidden=d)
        ctx = harness.context([(harness.cache.take_slot(), n_tok)])
        assert ctx.fuse == fuse
        x = torch.as_tensor(x0).to(DEV)
        block.forward(ctx, x, RunInfo(entry=0, kv_entry=0, writes_kv=True))
        from gpullama3_java_amd.parts import ops
        ops.settle_residual(ctx, x)                                          # sums still in slices, if any
        t = (2e-5 if dtype == "float32" else 2e-2) * np.abs(ref).max()
        np.testing.assert_allclose(x.cpu().numpy(), ref, atol=t, err_msg=f"fuse {fuse}")


def test_unknown_part_kind_lists_the_known():
    from gpullama3_java_amd.parts import build_part

    @dataclass
    class Odd:
        kind: str = "odd"
    with pytest.raises(KeyError, match="rmsnorm"):
        build_part("norm", Odd(), dtype=torch.float32)


# ------------------------------------------------------------------ the run order is data
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_run_order_names_a_layer_twice_and_reads_another_entry_s_cache(dtype):
    import gpullama3_java_amd as g
    from gpullama3_java_amd.config import Run
    from gpullama3_java_amd.engine import Engine
    from gpullama3_java_amd.weights import load_weights
    from gpullama3_java_amd.parts import DecoderModel
    folder, cfgd, W = model("A")
    order = [(0, None), (1, None), (1, None), (0, 1)]          # layer 1 twice; the last run reads entry 1's keys

    class Reordered(g.LlamaConfiguration):
        def model_spec(self):
            from dataclasses import replace
            return replace(super().model_spec(), run_order=tuple(Run(layer=l, reads=r) for l, r in order))

    cfg = Reordered(**g.config_from_dict(cfgd).__dict__)
    probe = DecoderModel(cfg.model_spec(), TD[dtype], "cpu")
    eng = Engine(cfg, load_weights(folder, probe.expected(), TD[dtype], torch.device(DEV)), dtype=dtype, max_tokens=512)
    assert len(eng.cache.groups[0].entries) == 3                # three entries store keys, the fourth reads
    toks = rand_tokens("A", 3, 50)
    ref = P.forward(cfgd, W, toks, schedule=order)
    s = eng.take_slot()
    got = np.concatenate([eng.step([(s, toks[:30])], want="all").cpu().numpy()]
                         + [eng.step([(s, [t])]).cpu().numpy() for t in toks[30:]])
    close(got, ref, dtype, "reordered run")
    assert np.abs(ref - P.forward(cfgd, W, toks)).max() > 1e-3   # the order matters

    with pytest.raises(ValueError, match="reads entry"):
        class Bad(g.LlamaConfiguration):
            def model_spec(self):
                from dataclasses import replace
                return replace(super().model_spec(), run_order=(Run(0), Run(1, reads=1)))
        DecoderModel(Bad(**cfg.__dict__).model_spec(), torch.float32, "cpu")


# ------------------------------------------------------------------ a toy mixer with state of its own
@dataclass(frozen=True)
class DecaySpec:
    """y_t = s_t . W with s_t = decay * s_{t-1} + h_t: a running sum per sequence, kept per slot."""
    kind: str = "toy_decay"
    hidden: int = 0
    decay: float = 0.5
    names: dict = field(default_factory=dict)


class DecayMixer:
    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype
        self.w = None

    def tensors(self):
        from gpullama3_java_amd.weights import TensorSpec
        return {self.spec.names["w"]: TensorSpec((self.spec.hidden, self.spec.hidden))}

    def load(self, weights):
        self.w = weights[self.spec.names["w"]]

    def kv_need(self):
        return None                                         # nothing per position

    def state_need(self):
        from gpullama3_java_amd.cache import StateNeed
        return StateNeed(self.spec.hidden, torch.float32)

    def forward(self, ctx, h, x, run):
        state = ctx.slot_state(run.entry)                   # [n_slots, hidden], zero for a fresh slot
        o = 0
        for slot, n in zip(ctx.slots, ctx.q_lens):
            s = state[slot].clone()
            for i in range(n):                              # a chunk advances the state token by token
                s = self.spec.decay * s + h[o + i].float()
                x[o + i] += (s.to(self.dtype).float() @ self.w.float().t())
            state[slot] = s
            o += n


def toy_plain(cfg, W, toks):
    x = W["emb"][toks].astype(np.float32)
    for l in range(cfg["n_layers"]):
        h = P.rmsnorm(x, W[f"l{l}.norm"], cfg["eps"])
        s = np.zeros(cfg["hidden"], np.float32)
        out = np.zeros_like(x)
        for t in range(len(toks)):
            s = np.float32(cfg["decay"]) * s + h[t]
            out[t] = s @ W[f"l{l}.w"].T
        x = x + out
    return P.rmsnorm(x, W["final"], cfg["eps"]) @ W["emb"].T


def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    import gpullama3_java_amd as g
    from gpullama3_java_amd.config import BlockSpec, ModelSpec, NormSpec, Run
    from gpullama3_java_amd.engine import Engine
    from gpullama3_java_amd.parts import register_part

    register_part("mixer", "toy_decay", DecayMixer)

    @dataclass(frozen=True)
    class ToyConfig:
        hidden: int
        n_layers: int
        vocab: int
        decay: float
        eps: float
        max_position_embeddings: int = 512
        stop_ids: tuple = ()

        @classmethod
        def from_dict(cls, d):
            return cls(d["hidden"], d["n_layers"], d["vocab"], d["decay"], d["eps"])

        def with_context_length(self, n):
            return self

        def model_spec(self):
            layers = tuple(BlockSpec(kind="prenorm",
                                     mixer_norm=NormSpec(dim=self.hidden, eps=self.eps, names={"weight": f"l{i}.norm"}),
                                     mixer=DecaySpec(hidden=self.hidden, decay=self.decay, names={"w": f"l{i}.w"}),
                                     ffn_norm=None, ffn=None) for i in range(self.n_layers))
            return ModelSpec(architecture="ToyForCausalLM", vocab_size=self.vocab, hidden=self.hidden, layers=layers,
                             run_order=tuple(Run(i) for i in range(self.n_layers)),
                             final_norm=NormSpec(dim=self.hidden, eps=self.eps, names={"weight": "final"}),
                             max_positions=512, tie_embeddings=True, embedding_name="emb", head_name=None)

    g.register_architecture("ToyForCausalLM", ToyConfig)
    cfg = {"architectures": ["ToyForCausalLM"], "hidden": 24, "n_layers": 2, "vocab": 40, "decay": 0.7, "eps": 1e-5}
    rng = np.random.default_rng(0)
    W = {"emb": rng.standard_normal((40, 24)).astype(np.float32), "final": np.ones(24, np.float32)}
    for l in range(2):
        W[f"l{l}.norm"] = (1 + 0.1 * rng.standard_normal(24)).astype(np.float32)
        W[f"l{l}.w"] = (rng.standard_normal((24, 24)) * 0.2).astype(np.float32)
    folder = str(tmp_path / "toy")
    os.makedirs(folder)
    json.dump(cfg, open(os.path.join(folder, "config.json"), "w"))
    save_file({k: torch.as_tensor(v) for k, v in W.items()}, os.path.join(folder, "model.safetensors"))

    eng = Engine.from_folder(folder, dtype="float32", max_tokens=256, n_slots=2)
    assert not eng.cache.groups and sorted(eng.cache.state) == [0, 1]        # state, no keys and values
    a, b = rng.integers(0, 40, 30).tolist(), rng.integers(0, 40, 12).tolist()
    sa, sb = eng.take_slot(), eng.take_slot()
    out = eng.step([(sa, a[:20]), (sb, b[:5])], want="all").cpu().numpy()
    got_a, got_b = [out[:20]], [out[20:]]
    for i in range(7):                                                        # both go on one token at a time
        o = eng.step([(sa, [a[20 + i]]), (sb, [b[5 + i]])]).cpu().numpy()
        got_a.append(o[:1]); got_b.append(o[1:])
    eng.give_back_slot(sb)                                                    # b ends earlier
    got_a.append(eng.step([(sa, a[27:])], want="all").cpu().numpy())
    np.testing.assert_allclose(np.concatenate(got_a), toy_plain(cfg, W, a), atol=2e-4)
    np.testing.assert_allclose(np.concatenate(got_b), toy_plain(cfg, W, b), atol=2e-4)
    eng.give_back_slot(sa)
    s = eng.take_slot()                                                       # a used slot starts from zero state
    again = eng.step([(s, b)], want="all").cpu().numpy()
    np.testing.assert_allclose(again, toy_plain(cfg, W, b), atol=2e-4)
    res = eng.generate([a[:4], b[:6]], max_new_tokens=5)                      # and the generation loop runs it
    assert [len(r.tokens) for r in res] == [5, 5]


# ------------------------------------------------------------------ a toy feed-forward with routing, a toy position encoding
@dataclass(frozen=True)
class LinearAnglesSpec:
    """Rotation of the first ``rot_dim`` elements of a head by pos * (pair + 1) * step, adjacent pairs."""
    kind: str = "toy_linear_angles"
    head_dim: int = 0
    rot_dim: int = 0
    step: float = 0.01
    max_positions: int = 0


def linear_angle_tables(spec):
    pos = np.arange(spec.max_positions, dtype=np.float32)[:, None]
    ang = (pos * ((np.arange(spec.rot_dim // 2, dtype=np.float32) + 1)[None, :] * np.float32(spec.step))).astype(np.float32)
    return np.cos(ang.astype(np.float64)).astype(np.float32), np.sin(ang.astype(np.float64)).astype(np.float32)


class LinearAngles:
    """What the attention mixer asks of a position encoding: cos, sin [positions, rot_dim/2], rot_dim, adjacent."""

    def __init__(self, spec, device):
        cos, sin = linear_angle_tables(spec)
        self.cos, self.sin = torch.from_numpy(cos).to(device), torch.from_numpy(sin).to(device)
        self.rot_dim, self.adjacent, self.max_positions = spec.rot_dim, True, spec.max_positions


@dataclass(frozen=True)
class RoutedSpec:
    """Each token goes to the one expert with the greatest router logit; the expert's output is
    weighted with that logit's softmax probability."""
    kind: str = "toy_routed"
    hidden: int = 0
    n_experts: int = 0
    names: dict = field(default_factory=dict)


class RoutedFeedForward:
    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype

    def tensors(self):
        from gpullama3_java_amd.weights import TensorSpec
        s = self.spec
        return {s.names["router"]: TensorSpec((s.n_experts, s.hidden)),
                s.names["experts"]: TensorSpec((s.n_experts, s.hidden, s.hidden))}

    def load(self, weights):
        self.router, self.experts = weights[self.spec.names["router"]], weights[self.spec.names["experts"]]

    def forward(self, ctx, h, x):
        hf = h.float()
        p = torch.softmax(hf @ self.router.float().t(), dim=-1)              # router logits in 32-bit
        choice = p.argmax(dim=-1)
        for e in range(self.spec.n_experts):                                  # every token of an expert, no capacity
            idx = (choice == e).nonzero().flatten()
            if idx.numel():
                x[idx] += p[idx, e, None] * (hf[idx] @ self.experts[e].float().t())


def mixed_plain(cfg, W, toks, pos_spec):
    d, H, Kh, hs = cfg["hidden"], cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
    T = len(toks)
    cos, sin = linear_angle_tables(pos_spec)
    x = W["emb"][toks].astype(np.float32)
    # layer 0: attention with the toy position encoding, routed feed-forward
    h = P.rmsnorm(x, W["l0.n1"], cfg["eps"])
    q, k = P.linear(h, W["l0.q"]).reshape(T, H, hs), P.linear(h, W["l0.k"]).reshape(T, Kh, hs)
    r = pos_spec.rot_dim
    q[..., :r] = P.rope_rotate(q[..., :r], np.arange(T), cos, sin, "adjacent")
    k[..., :r] = P.rope_rotate(k[..., :r], np.arange(T), cos, sin, "adjacent")
    v = P.linear(h, W["l0.v"]).reshape(T, Kh, hs)
    x = x + P.linear(P.attention(q, k, v).reshape(T, H * hs), W["l0.o"])
    h = P.rmsnorm(x, W["l0.n2"], cfg["eps"])
    p = P.softmax(h @ W["l0.router"].T)
    out = np.zeros_like(x)
    for t in range(T):
        e = int(np.argmax(p[t]))
        out[t] = p[t, e] * (h[t] @ W["l0.experts"][e].T)
    x = x + out
    # layer 1: the toy mixer with state, the framework's dense feed-forward
    h = P.rmsnorm(x, W["l1.n1"], cfg["eps"])
    s = np.zeros(d, np.float32)
    out = np.zeros_like(x)
    for t in range(T):
        s = np.float32(cfg["decay"]) * s + h[t]
        out[t] = s @ W["l1.w"].T
    x = x + out
    x = x + P.feed_forward(P.rmsnorm(x, W["l1.n2"], cfg["eps"]), W["l1.g"], W["l1.u"], W["l1.dn"])
    return P.rmsnorm(x, W["final"], cfg["eps"]) @ W["head"].T


def test_toy_routing_and_toy_position_in_a_model_with_different_layers(tmp_path):
    """One model whose two layers differ in mixer and feed-forward: attention with a position
    encoding defined here and a routed feed-forward defined here; then a mixer with state and the
    framework's dense feed-forward. Registered, built, stepped in pieces and generated from, with no
    change to the framework's files."""
    import gpullama3_java_amd as g
    from gpullama3_java_amd.config import AttentionSpec, BlockSpec, GatedFeedForwardSpec, ModelSpec, NormSpec, Run
    from gpullama3_java_amd.engine import Engine
    from gpullama3_java_amd.parts import register_part

    register_part("mixer", "toy_decay", DecayMixer)
    register_part("ffn", "toy_routed", RoutedFeedForward)
    register_part("position", "toy_linear_angles", LinearAngles)
    pos_spec = LinearAnglesSpec(head_dim=16, rot_dim=8, step=0.05, max_positions=128)

    @dataclass(frozen=True)
    class MixedConfig:
        c: tuple
        max_position_embeddings: int = 128
        stop_ids: tuple = ()

        @classmethod
        def from_dict(cls, d):
            return cls(tuple(sorted((k, v) for k, v in d.items() if k != "architectures")))

        def with_context_length(self, n):
            return self

        def model_spec(self):
            c = dict(self.c)
            d, eps = c["hidden"], c["eps"]
            norm = lambda name: NormSpec(dim=d, eps=eps, names={"weight": name})
            layer0 = BlockSpec(kind="prenorm", mixer_norm=norm("l0.n1"),
                               mixer=AttentionSpec(hidden=d, n_heads=c["heads"], n_kv_heads=c["kv_heads"],
                                                   head_dim=c["head_dim"], position=pos_spec,
                                                   names={k: f"l0.{k}" for k in "qkvo"}),
                               ffn_norm=norm("l0.n2"),
                               ffn=RoutedSpec(hidden=d, n_experts=c["experts"],
                                              names={"router": "l0.router", "experts": "l0.experts"}))
            layer1 = BlockSpec(kind="prenorm", mixer_norm=norm("l1.n1"),
                               mixer=DecaySpec(hidden=d, decay=c["decay"], names={"w": "l1.w"}),
                               ffn_norm=norm("l1.n2"),
                               ffn=GatedFeedForwardSpec(hidden=d, intermediate=c["intermediate"],
                                                        names={"gate": "l1.g", "up": "l1.u", "down": "l1.dn"}))
            return ModelSpec(architecture="MixedToyForCausalLM", vocab_size=c["vocab"], hidden=d, layers=(layer0, layer1),
                             run_order=(Run(0), Run(1)), final_norm=norm("final"), max_positions=128,
                             tie_embeddings=False, embedding_name="emb", head_name="head")

    g.register_architecture("MixedToyForCausalLM", MixedConfig)
    cfg = {"architectures": ["MixedToyForCausalLM"], "hidden": 24, "heads": 3, "kv_heads": 1, "head_dim": 16,
           "experts": 3, "intermediate": 40, "vocab": 50, "decay": 0.6, "eps": 1e-5}
    rng = np.random.default_rng(5)
    d, E, F, V = 24, 3, 40, 50
    W = {"emb": rng.standard_normal((V, d)), "head": rng.standard_normal((V, d)) * 0.3, "final": np.ones(d),
         "l0.q": rng.standard_normal((48, d)) * 0.3, "l0.k": rng.standard_normal((16, d)) * 0.3,
         "l0.v": rng.standard_normal((16, d)) * 0.3, "l0.o": rng.standard_normal((d, 48)) * 0.2,
         "l0.router": rng.standard_normal((E, d)), "l0.experts": rng.standard_normal((E, d, d)) * 0.2,
         "l1.w": rng.standard_normal((d, d)) * 0.2, "l1.g": rng.standard_normal((F, d)) * 0.3,
         "l1.u": rng.standard_normal((F, d)) * 0.3, "l1.dn": rng.standard_normal((d, F)) * 0.2}
    for n in ("l0.n1", "l0.n2", "l1.n1", "l1.n2"):
        W[n] = 1 + 0.1 * rng.standard_normal(d)
    W = {k: v.astype(np.float32) for k, v in W.items()}
    folder = str(tmp_path / "mixed")
    os.makedirs(folder)
    json.dump(cfg, open(os.path.join(folder, "config.json"), "w"))
    save_file({k: torch.as_tensor(v) for k, v in W.items()}, os.path.join(folder, "model.safetensors"))

    eng = Engine.from_folder(folder, dtype="float32", max_tokens=512, n_slots=3)
    assert len(eng.cache.groups) == 1 and sorted(eng.cache.state) == [1]     # keys and values for layer 0, state for layer 1
    a, b = rng.integers(0, V, 70).tolist(), rng.integers(0, V, 9).tolist()
    ref_a, ref_b = mixed_plain(cfg, W, a, pos_spec), mixed_plain(cfg, W, b, pos_spec)
    choices = {int(np.argmax(P.softmax(P.rmsnorm(W["emb"][a], W["l0.n2"], 1e-5) @ W["l0.router"].T)[t])) for t in range(70)}
    assert len(choices) > 1                                                   # more than one expert is in use
    sa, sb = eng.take_slot(), eng.take_slot()
    out = eng.step([(sa, a[:40]), (sb, b[:3])], want="all").cpu().numpy()
    got_a, got_b = [out[:40]], [out[40:]]
    for i in range(6):
        o = eng.step([(sa, [a[40 + i]]), (sb, [b[3 + i]])]).cpu().numpy()
        got_a.append(o[:1]); got_b.append(o[1:])
    eng.give_back_slot(sb)
    got_a.append(eng.step([(sa, a[46:])], want="all").cpu().numpy())
    scale = np.abs(ref_a).max()
    np.testing.assert_allclose(np.concatenate(got_a), ref_a, atol=1e-4 * scale)
    np.testing.assert_allclose(np.concatenate(got_b), ref_b, atol=1e-4 * scale)
    res = eng.generate([a[:5], b[:4]], max_new_tokens=4)
    assert [len(r.tokens) for r in res] == [4, 4]
    assert res[0].tokens[0] == int(np.argmax(mixed_plain(cfg, W, a[:5], pos_spec)[-1]))


# ------------------------------------------------------------------ a mixer with state under captured graphs
class GraphDecayMixer(DecayMixer):
    """The toy mixer again, its decode steps made of launches on the current stream only (indices
    stay on the device), so that the engine may capture them."""
    graph_safe = True

    def forward(self, ctx, h, x, run):
        if not ctx.decode:
            return super().forward(ctx, h, x, run)
        state = ctx.slot_state(run.entry)
        rows = ctx.slot_ids.long()
        s = self.spec.decay * state.index_select(0, rows) + h.float()
        state.index_copy_(0, rows, s)
        x += s.to(self.dtype).float() @ self.w.float().t()


def test_a_mixer_with_state_decodes_from_captured_graphs(tmp_path):
    """Per-slot state is no obstacle to captured decode steps: the entries that pad a batch to its
    bucket work on the sink row of the state area. Captured and eager steps agree bit for bit,
    and both with the plain recurrence; a batch of 9 is padded to 16."""
    import gpullama3_java_amd as g
    from gpullama3_java_amd.config import BlockSpec, ModelSpec, NormSpec, Run
    from gpullama3_java_amd.engine import Engine
    from gpullama3_java_amd.parts import register_part

    register_part("mixer", "toy_decay_graph", GraphDecayMixer)
    from gpullama3_java_amd.parts.norm import RMSNorm

    @dataclass(frozen=True)
    class ToyGraphConfig:
        hidden: int
        n_layers: int
        vocab: int
        decay: float
        eps: float
        max_position_embeddings: int = 512
        stop_ids: tuple = ()

        @classmethod
        def from_dict(cls, d):
            return cls(d["hidden"], d["n_layers"], d["vocab"], d["decay"], d["eps"])

        def with_context_length(self, n):
            return self

        def model_spec(self):
            layers = tuple(BlockSpec(kind="prenorm",
                                     mixer_norm=NormSpec(dim=self.hidden, eps=self.eps, names={"weight": f"l{i}.norm"}),
                                     mixer=replace_kind(DecaySpec(hidden=self.hidden, decay=self.decay, names={"w": f"l{i}.w"})),
                                     ffn_norm=None, ffn=None) for i in range(self.n_layers))
            return ModelSpec(architecture="ToyGraphForCausalLM", vocab_size=self.vocab, hidden=self.hidden, layers=layers,
                             run_order=tuple(Run(i) for i in range(self.n_layers)),
                             final_norm=NormSpec(dim=self.hidden, eps=self.eps, names={"weight": "final"}),
                             max_positions=512, tie_embeddings=True, embedding_name="emb", head_name=None)

    def replace_kind(spec):
        from dataclasses import replace
        return replace(spec, kind="toy_decay_graph")

    g.register_architecture("ToyGraphForCausalLM", ToyGraphConfig)
    cfg = {"architectures": ["ToyGraphForCausalLM"], "hidden": 24, "n_layers": 2, "vocab": 40, "decay": 0.7, "eps": 1e-5}
    rng = np.random.default_rng(1)
    W = {"emb": rng.standard_normal((40, 24)).astype(np.float32), "final": np.ones(24, np.float32)}
    for l in range(2):
        W[f"l{l}.norm"] = (1 + 0.1 * rng.standard_normal(24)).astype(np.float32)
        W[f"l{l}.w"] = (rng.standard_normal((24, 24)) * 0.2).astype(np.float32)
    folder = str(tmp_path / "toygraph")
    os.makedirs(folder)
    json.dump(cfg, open(os.path.join(folder, "config.json"), "w"))
    save_file({k: torch.as_tensor(v) for k, v in W.items()}, os.path.join(folder, "model.safetensors"))

    seqs = [rng.integers(0, 40, 6 + 2 * i).tolist() for i in range(9)]
    outs = {}
    for graphs in (True, False):
        eng = Engine.from_folder(folder, dtype="float32", max_tokens=2048, n_slots=12, use_graphs=graphs)
        assert eng.use_graphs == graphs and sorted(eng.cache.state) == [0, 1]
        slots = [eng.take_slot() for _ in seqs]
        eng.step([(s, q[:3]) for s, q in zip(slots, seqs)], want="none")
        rows = [eng.step([(s, [q[3 + k]]) for s, q in zip(slots, seqs)]).cpu().numpy() for k in range(3)]
        outs[graphs] = np.stack(rows)                                             # [3, 9, vocab]
        if graphs:
            assert any(key[0] == 16 for key in eng._graphs)                       # the batch of 9 ran in a bucket of 16
    assert np.array_equal(outs[True], outs[False])
    for i, q in enumerate(seqs):
        np.testing.assert_allclose(outs[True][:, i], toy_plain(cfg, W, q)[3:6], atol=2e-4)


# ------------------------------------------------------------------ what other decoders put around and inside the blocks
class HalvingBlock:
    """An arrangement of its own that READS the residual rows (it halves them before the usual
    pre-norm sequence) and offers no ``first_norm``: the decoder makes the rows whole before it
    runs and lets no product leave its sums in slices meanwhile."""

    def __init__(self, spec, dtype, device):
        from gpullama3_java_amd.parts.block import PreNormBlock
        self.inner = PreNormBlock(spec, dtype, device)

    def parts(self):
        return self.inner.parts()

    def forward(self, ctx, x, run):
        x.mul_(0.5)
        self.inner.forward(ctx, x, run)


def other_plain(cfg, W, toks):
    """The toy decoder below in numpy: embedding times a multiplier plus a learned position row, halved
    rows, attention without rotation and with biases, gelu feed-forward with biases, scaled logits."""
    d, H, K, hs, L = cfg["hidden"], cfg["heads"], cfg["kv_heads"], cfg["head_dim"], cfg["layers"]
    T = len(toks)
    x = W["emb"][toks].astype(np.float32) * np.float32(cfg["embedding_scale"]) + W["wpe"][:T]
    for l in range(L):
        p = f"l{l}."
        if l in cfg["halving_layers"]:
            x = x * np.float32(0.5)
        h = P.rmsnorm(x, W[p + "n1"], cfg["eps"])
        q = (P.linear(h, W[p + "q"]) + W[p + "qb"]).reshape(T, H, hs)
        k = (P.linear(h, W[p + "k"]) + W[p + "kb"]).reshape(T, K, hs)
        v = (P.linear(h, W[p + "v"]) + W[p + "vb"]).reshape(T, K, hs)
        x = x + P.linear(P.attention(q, k, v).reshape(T, H * hs), W[p + "o"]) + W[p + "ob"]
        h = P.rmsnorm(x, W[p + "n2"], cfg["eps"])
        g = (P.linear(h, W[p + "g"]) + W[p + "gb"]).astype(np.float64)
        act = 0.5 * g * (1 + np.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3)))
        x = x + P.linear((act * (P.linear(h, W[p + "u"]) + W[p + "ub"])).astype(np.float32), W[p + "dn"])
        if p + "db" in W:
            x = x + W[p + "db"]
    logits = (P.linear(P.rmsnorm(x, W["final"], cfg["eps"]), W["emb"]) + W["head_bias"]) * np.float32(cfg["logit_scale"])
    return np.float32(cfg["softcap"]) * np.tanh(logits / np.float32(cfg["softcap"]))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_decoder_of_another_make_from_descriptions_alone(tmp_path, dtype):
    """Embedding multiplier, learned absolute positions, logit scale, a bias and a soft cap on the logits, biases on every projection,
    the other activation and a block kind defined here: all of it is a description and two
    registrations, no file of the framework changes. 40 tokens in one step take the kernels for 33
    to 64 rows, whose products into the residual rows leave their sums in slices (K = 1024): the
    block that reads the rows must find them whole."""
    import gpullama3_java_amd as g
    from gpullama3_java_amd.config import AttentionSpec, BlockSpec, GatedFeedForwardSpec, ModelSpec, NormSpec, Run
    from gpullama3_java_amd.engine import Engine
    from gpullama3_java_amd.parts import register_part

    register_part("block", "toy_halving", HalvingBlock)

    @dataclass(frozen=True)
    class OtherConfig:
        d: dict
        max_position_embeddings: int = 128
        stop_ids: tuple = ()

        @classmethod
        def from_dict(cls, d):
            return cls(dict(d))

        def with_context_length(self, n):
            return self

        def model_spec(self):
            c = self.d
            layers = []
            for l in range(c["layers"]):
                p = f"l{l}."
                ffn_names = {"gate": p + "g", "up": p + "u", "down": p + "dn", "gate_bias": p + "gb", "up_bias": p + "ub"}
                if l in c["down_bias_layers"]:
                    ffn_names["down_bias"] = p + "db"
                layers.append(BlockSpec(
                    kind="toy_halving" if l in c["halving_layers"] else "prenorm",
                    mixer_norm=NormSpec(dim=c["hidden"], eps=c["eps"], names={"weight": p + "n1"}),
                    mixer=AttentionSpec(hidden=c["hidden"], n_heads=c["heads"], n_kv_heads=c["kv_heads"],
                                        head_dim=c["head_dim"], position=None,
                                        names={"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o", "q_bias": p + "qb",
                                               "k_bias": p + "kb", "v_bias": p + "vb", "o_bias": p + "ob"}),
                    ffn_norm=NormSpec(dim=c["hidden"], eps=c["eps"], names={"weight": p + "n2"}),
                    ffn=GatedFeedForwardSpec(hidden=c["hidden"], intermediate=c["inter"], activation="gelu_tanh",
                                             names=ffn_names)))
            return ModelSpec(architecture="OtherForCausalLM", vocab_size=c["vocab"], hidden=c["hidden"], layers=tuple(layers),
                             run_order=tuple(Run(i) for i in range(c["layers"])),
                             final_norm=NormSpec(dim=c["hidden"], eps=c["eps"], names={"weight": "final"}),
                             max_positions=128, tie_embeddings=True, embedding_name="emb", head_name=None,
                             embedding_scale=c["embedding_scale"], position_table_name="wpe", logit_scale=c["logit_scale"],
                             head_bias_name="head_bias", logit_softcap=c["softcap"])

    g.register_architecture("OtherForCausalLM", OtherConfig)
    # three layers: the usual arrangement whose down projection has no bias (its sums stay in slices
    # behind it), then the halving one, which reads the rows, then the usual one again
    cfg = {"architectures": ["OtherForCausalLM"], "hidden": 128, "inter": 1024, "layers": 3, "heads": 4, "kv_heads": 2,
           "head_dim": 32, "vocab": 300, "eps": 1e-5, "embedding_scale": 3.0, "logit_scale": 0.25, "softcap": 2.0,
           "halving_layers": [1], "down_bias_layers": [1, 2]}
    rng = np.random.default_rng(4)
    r = lambda *s, scale=0.05: (rng.standard_normal(s) * scale).astype(np.float32)
    W = {"emb": r(300, 128, scale=0.3), "wpe": r(128, 128, scale=0.3), "final": 1 + r(128, scale=0.1),
         "head_bias": r(300, scale=2.0)}
    for l in range(3):
        p = f"l{l}."
        W.update({p + "n1": 1 + r(128, scale=0.1), p + "n2": 1 + r(128, scale=0.1), p + "q": r(128, 128), p + "k": r(64, 128),
                  p + "v": r(64, 128), p + "o": r(128, 128), p + "qb": r(128, scale=0.3), p + "kb": r(64, scale=0.3),
                  p + "vb": r(64, scale=0.3), p + "ob": r(128, scale=0.3), p + "g": r(1024, 128), p + "u": r(1024, 128),
                  p + "dn": r(128, 1024), p + "gb": r(1024, scale=0.3), p + "ub": r(1024, scale=0.3), p + "db": r(128, scale=0.3)})
    del W["l0.db"]
    if dtype == "bfloat16":                                   # what the engine will hold: matrices in bfloat16
        W = {k: (torch.as_tensor(v).to(torch.bfloat16).float().numpy() if v.ndim == 2 else v) for k, v in W.items()}
    folder = str(tmp_path / "other")
    os.makedirs(folder)
    json.dump(cfg, open(os.path.join(folder, "config.json"), "w"))
    save_file({k: torch.as_tensor(v).to(TD[dtype] if v.ndim == 2 else torch.float32) for k, v in W.items()},
              os.path.join(folder, "model.safetensors"))
    eng = Engine.from_folder(folder, dtype=dtype, max_tokens=512, n_slots=2)
    toks = rng.integers(0, 300, 45).tolist()
    ref = other_plain(cfg, W, toks)
    s = eng.take_slot()
    got = [eng.step([(s, toks[:40])], want="all").cpu().numpy()]
    got += [eng.step([(s, [t])]).cpu().numpy() for t in toks[40:]]
    close(np.concatenate(got), ref, dtype, "a decoder of another make")
    if dtype == "bfloat16":
        # the case is the one it claims to be: without the decoder's care the halving block would halve
        # rows whose last product still lies in slices
        from gpullama3_java_amd.parts import ops
        seen = []
        real = ops.settle_residual
        ops.settle_residual = lambda ctx, x: seen.append(ctx.pending is not None) or real(ctx, x)
        try:
            s2 = eng.take_slot()
            eng.step([(s2, toks[:40])], want="none")
        finally:
            ops.settle_residual = real
        assert any(seen)


# ------------------------------------------------------------------ no final norm; a norm that knows nothing of slices
class PlainRMS:
    """A norm kind of the test's own that reads the residual rows with no thought for sums that a
    product may have left in slices beside them, as any part written from the interface alone would."""
    graph_safe = True          # one kernel launch on the current stream

    def __init__(self, spec, dtype):
        self.dim, self.eps, self.dtype, self.name = spec.dim, spec.eps, dtype, spec.names["weight"]

    def tensors(self):
        from gpullama3_java_amd.weights.loader import TensorSpec
        return {self.name: TensorSpec((self.dim,), "vector")}

    def load(self, weights):
        self.weight = weights[self.name]

    def __call__(self, ctx, x, rows=None, name="normed"):
        from gpullama3_java_amd.csrc import lib as K
        out = ctx.buffer("toy_" + name, (x.shape[0] if rows is None else rows.numel(), self.dim), self.dtype)
        K.rmsnorm(x, self.weight, out, self.eps, rows)
        return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_decoder_without_a_final_norm_and_with_a_norm_that_knows_nothing_of_slices(tmp_path, dtype):
    """``ModelSpec.final_norm = None``: the head reads the wanted rows as they are. The feed-forward's norm is
    a kind defined here that just reads the rows; in a step of 40 tokens the output projection before it
    (K = 1,024) leaves its sums in slices, so the stock block must make the rows whole for it."""
    import gpullama3_java_amd as g
    from gpullama3_java_amd.config import AttentionSpec, BlockSpec, GatedFeedForwardSpec, ModelSpec, NormSpec, Run
    from gpullama3_java_amd.engine import Engine
    from gpullama3_java_amd.parts import ops, register_part

    register_part("norm", "toy_plain_rms", PlainRMS)
    d, H, Kh, hs, F, V, L, eps = 128, 8, 2, 128, 1024, 300, 2, 1e-5

    @dataclass(frozen=True)
    class BareConfig:
        d: dict
        max_position_embeddings: int = 128
        stop_ids: tuple = ()

        @classmethod
        def from_dict(cls, dd):
            return cls(dict(dd))

        def with_context_length(self, n):
            return self

        def model_spec(self):
            layers = []
            for l in range(L):
                p = f"l{l}."
                layers.append(BlockSpec(
                    mixer_norm=NormSpec(dim=d, eps=eps, names={"weight": p + "n1"}),
                    mixer=AttentionSpec(hidden=d, n_heads=H, n_kv_heads=Kh, head_dim=hs, position=None,
                                        names={"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o"}),
                    ffn_norm=NormSpec(kind="toy_plain_rms", dim=d, eps=eps, names={"weight": p + "n2"}),
                    ffn=GatedFeedForwardSpec(hidden=d, intermediate=F, names={"gate": p + "g", "up": p + "u", "down": p + "dn"})))
            return ModelSpec(architecture="BareForCausalLM", vocab_size=V, hidden=d, layers=tuple(layers),
                             run_order=tuple(Run(i) for i in range(L)), final_norm=None, max_positions=128,
                             tie_embeddings=False, embedding_name="emb", head_name="head")

    g.register_architecture("BareForCausalLM", BareConfig)
    rng = np.random.default_rng(9)
    r = lambda *s, scale=0.05: (rng.standard_normal(s) * scale).astype(np.float32)
    W = {"emb": r(V, d, scale=0.3), "head": r(V, d, scale=0.1)}
    for l in range(L):
        p = f"l{l}."
        W.update({p + "n1": 1 + r(d, scale=0.1), p + "n2": 1 + r(d, scale=0.1), p + "q": r(H * hs, d), p + "k": r(Kh * hs, d),
                  p + "v": r(Kh * hs, d), p + "o": r(d, H * hs), p + "g": r(F, d), p + "u": r(F, d), p + "dn": r(d, F)})
    if dtype == "bfloat16":
        W = {k: (torch.as_tensor(v).to(torch.bfloat16).float().numpy() if v.ndim == 2 else v) for k, v in W.items()}

    def plain(toks):
        T = len(toks)
        x = W["emb"][toks].astype(np.float32)
        for l in range(L):
            p = f"l{l}."
            h = P.rmsnorm(x, W[p + "n1"], eps)
            q, k, v = (P.linear(h, W[p + n]).reshape(T, heads, hs) for n, heads in (("q", H), ("k", Kh), ("v", Kh)))
            x = x + P.linear(P.attention(q, k, v).reshape(T, H * hs), W[p + "o"])
            h = P.rmsnorm(x, W[p + "n2"], eps)
            x = x + P.linear(P.silu(P.linear(h, W[p + "g"])) * P.linear(h, W[p + "u"]), W[p + "dn"])
        return P.linear(x, W["head"])                       # no final norm

    folder = str(tmp_path / "bare")
    os.makedirs(folder)
    json.dump({"architectures": ["BareForCausalLM"]}, open(os.path.join(folder, "config.json"), "w"))
    save_file({k: torch.as_tensor(v).to(TD[dtype] if v.ndim == 2 else torch.float32) for k, v in W.items()},
              os.path.join(folder, "model.safetensors"))
    eng = Engine.from_folder(folder, dtype=dtype, max_tokens=512, n_slots=2)
    assert eng.model.final_norm is None
    toks = rng.integers(0, V, 46).tolist()
    ref = plain(toks)
    seen = []
    real = ops.settle_residual
    ops.settle_residual = lambda ctx, x: seen.append(ctx.pending is not None) or real(ctx, x)
    try:
        s = eng.take_slot()
        got = [eng.step([(s, toks[:40])], want=[[0, 17, 39]]).cpu().numpy()]
    finally:
        ops.settle_residual = real
    got += [eng.step([(s, [t])]).cpu().numpy() for t in toks[40:]]
    close(np.concatenate(got), ref[[0, 17, 39] + list(range(40, 46))], dtype, "no final norm, a norm that only reads")
    if dtype == "bfloat16":
        assert any(seen)           # the case is the one it claims to be: slices lay beside the rows when the toy norm came


def test_two_engines_in_one_process_keep_their_own_switches():
    """The fast paths that an engine does without belong to that engine: another engine of the same process,
    built before or after it, keeps all of them; both give the plain implementation's logits."""
    from gpu_helpers import plain_logits
    from gpullama3_java_amd.engine import Engine
    folder, _, _ = model("D")
    bare = Engine.from_folder(folder, dtype="bfloat16", max_tokens=1024, without="tiled,fused,wide")
    full = Engine.from_folder(folder, dtype="bfloat16", max_tokens=1024)
    lean = Engine.from_folder(folder, dtype="bfloat16", max_tokens=1024, weight_copies=False)
    assert bare.without == {"tiled", "fused", "wide"} and full.without == frozenset() and lean.without == {"tiled"}
    copies = lambda e: [getattr(b.mixer.w_qkv, "tiled", None) is not None for b in e.model.blocks]
    assert copies(full) == [True, True] and copies(bare) == [False, False] and copies(lean) == [False, False]
    toks = rand_tokens("D", 3, 30)
    ref = plain_logits("D", toks)
    for eng in (bare, full, lean, bare):
        s = eng.take_slot()
        got = [eng.step([(s, toks[:20])], want="all").cpu().numpy()]
        got += [eng.step([(s, [t])]).cpu().numpy() for t in toks[20:]]
        eng.give_back_slot(s)
        close(np.concatenate(got), ref, "bfloat16")
    with pytest.raises(ValueError, match="unknown fast path"):
        Engine.from_folder(folder, dtype="bfloat16", max_tokens=1024, without="tiled,quick")

"""The engine: a model on one GPU, its cache, and the one step function.

``step`` takes a batch of sequences, each with the tokens it brings (a whole prompt,
a chunk, or one token), runs exactly those tokens as one packed batch against the
cache that earlier steps left, and returns the logits at the wanted places. The
reference's counterpart is ``forward(state, token, position)`` for one token of one
sequence (J/inference/InferenceCore.java:58, J/model/Model.java:61), which pays the
head on every prompt token (J/inference/InferenceEngine.java:312-322); here the
final norm and the head run on the wanted rows only.
"""
from __future__ import annotations

import os
import tempfile

import torch

from ..cache import Cache, CacheFull
from ..config import config_from_dict, load_config
from ..parts import DecoderModel
from ..sampling import DeviceSampler, SamplingParams
from ..weights import load_weights, write_random_model
from .context import StepContext, Workspace
from .generate import Generated, Request, RunMetrics, generate

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def _dtype(d):
    try:
        return _DTYPES[d]
    except KeyError:
        raise ValueError(f"dtype {d!r} is not one of bfloat16, float32") from None


def _require_gpu(device):
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible: the engine runs on HIP kernels only and has no CPU path")
    return torch.device(device)


class Engine:
    """``config``: a registered architecture's configuration; ``weights``: stored name -> device tensor."""

    def __init__(self, config, weights, dtype="bfloat16", device="cuda:0", max_tokens=None, max_context=None,
                 n_slots=None, page_size=64):
        self.device = _require_gpu(device)
        self.dtype = _dtype(dtype)
        limit = config.max_position_embeddings
        max_context = limit if max_context is None or max_context < 0 else min(max_context, limit)
        self.config = config.with_context_length(max_context)
        self.spec = self.config.model_spec()
        self.max_context = max_context
        max_tokens = max_tokens or max_context
        self.model = DecoderModel(self.spec, self.dtype, self.device)
        self.model.load(weights)
        kv_needs, state_needs = self.model.cache_needs()
        if n_slots is None:
            n_slots = max(1, min(-(-max_tokens // page_size), 256))
        with torch.cuda.device(self.device):
            self.cache = Cache(kv_needs, state_needs, max_tokens, max_context, n_slots, self.dtype, self.device,
                               page_size)
        self.workspace = Workspace(self.device)
        self.sampler = DeviceSampler(self.device)
        self.metrics = RunMetrics()

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_folder(cls, folder, dtype="bfloat16", device="cuda:0", **kw):
        """A model folder: config.json picks the architecture, model.safetensors holds the tensors."""
        dev = _require_gpu(device)
        config = load_config(folder)
        probe = DecoderModel(config.model_spec(), _dtype(dtype), "cpu")
        weights = load_weights(folder, probe.expected(), _dtype(dtype), dev)
        return cls(config, weights, dtype=dtype, device=device, **kw)

    @classmethod
    def random(cls, config, seed, dtype="bfloat16", device="cuda:0", std=0.02, norm_std=0.0, folder=None, **kw):
        """Random-weights mode: writes the model folder, then loads it like any other."""
        if isinstance(config, dict):
            config = config_from_dict(config)
        if folder is not None:
            write_random_model(folder, config, seed, std=std, norm_std=norm_std)
            return cls.from_folder(folder, dtype=dtype, device=device, **kw)
        with tempfile.TemporaryDirectory(prefix="gl3-random-") as tmp:
            write_random_model(tmp, config, seed, std=std, norm_std=norm_std)
            return cls.from_folder(tmp, dtype=dtype, device=device, **kw)

    def weights(self):
        """Stored name -> device tensor (stacked matrices appear as views under their stored names)."""
        return self.model.weights

    # ------------------------------------------------------------------ slots
    def take_slot(self):
        return self.cache.take_slot()

    def give_back_slot(self, slot):
        self.cache.give_back_slot(slot)

    @property
    def n_slots(self):
        return self.cache.slots.n_slots

    @property
    def page_size(self):
        return self.cache.page_size

    def slots_free(self):
        return self.cache.slots.n_free

    def tokens_capacity(self):
        return self.cache.tokens_free()

    # ------------------------------------------------------------------ the step
    def step(self, entries, want="last"):
        """Run the tokens of ``entries = [(slot, tokens), ...]`` and return logits.

        Each sequence's tokens are appended at its own length. ``want``: "last"
        (the last token of every entry), "all", "none", or a list with one list of
        indices into each entry's tokens. Returns ``[rows, vocab]`` float32 on the
        device, rows in the order of the entries and of their wanted indices. If the
        cache has no room, ``CacheFull`` is raised and nothing has changed.
        """
        B = len(entries)
        if B == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        slots = [int(s) for s, _ in entries]
        if len(set(slots)) != B:
            raise ValueError("a slot appears twice in one step")
        V = self.spec.vocab_size
        token_ids, positions, seq_of, cu, kv_before, want_rows = [], [], [], [0], [], []
        q_lens = []
        for b, (slot, toks) in enumerate(entries):
            toks = [int(t) for t in toks]
            if not toks:
                raise ValueError(f"entry {b} brings no token")
            bad = [t for t in toks if not 0 <= t < V]
            if bad:
                raise ValueError(f"entry {b}: token id {bad[0]} is outside the vocabulary of {V}")
            start = self.cache.length(slot)
            n = len(toks)
            if want == "last":
                idx = [n - 1]
            elif want == "all":
                idx = list(range(n))
            elif want == "none" or want is None:
                idx = []
            else:
                idx = [int(i) for i in want[b]]
                if any(not 0 <= i < n for i in idx):
                    raise ValueError(f"entry {b}: a wanted place is outside its {n} tokens")
            want_rows.extend(cu[-1] + i for i in idx)
            token_ids.extend(toks)
            positions.extend(range(start, start + n))
            seq_of.extend([b] * n)
            cu.append(cu[-1] + n)
            kv_before.append(start)
            q_lens.append(n)
        self.cache.reserve({s: n for s, n in zip(slots, q_lens)})      # raises CacheFull, nothing changed
        T = cu[-1]
        max_kv = max(k + n for k, n in zip(kv_before, q_lens))
        ctx = StepContext(self, T, B, q_lens, kv_before, slots, decode=all(n == 1 for n in q_lens),
                          max_q_len=max(q_lens), max_kv_len=max_kv)
        width = max(1, -(-max_kv // self.cache.page_size))
        tables = [self.cache.block_rows(g, slots, width) for g in range(len(self.cache.groups))]
        flat = token_ids + positions + seq_of + cu + kv_before + slots + want_rows
        for t in tables:
            for row in t:
                flat.extend(row)
        with torch.cuda.device(self.device):
            dev = torch.tensor(flat, dtype=torch.int32).to(self.device)
            o = 0

            def cut(n):
                nonlocal o
                t = dev[o:o + n]
                o += n
                return t

            ctx.token_ids, ctx.positions, ctx.seq_of_token = cut(T), cut(T), cut(T)
            ctx.cu_seqlens, ctx.kv_before, ctx.slot_ids = cut(B + 1), cut(B), cut(B)
            rows = cut(len(want_rows))
            ctx._tables = [cut(B * width).view(B, width) for _ in tables]
            logits = self.model.forward(ctx, rows)
        for s, n in zip(slots, q_lens):
            self.cache.advance(s, n)
        return logits

    # ------------------------------------------------------------------ generation
    def sample(self, logits, temperatures, top_ps, uniforms):
        with torch.cuda.device(self.device):
            return self.sampler(logits, temperatures, top_ps, uniforms)

    def generate(self, prompts, max_new_tokens=16, temperature=0.0, top_p=1.0, seed=0, stop_ids=None,
                 on_token=None, max_batch=None):
        """Generate for a list of prompts (lists of token ids); returns a ``Generated`` per prompt.

        ``stop_ids`` default to the configuration's; a stop token ends its own
        sequence only and is kept in the result, as the reference's loop keeps it
        (J/inference/InferenceEngine.java:343-348).
        """
        stops = frozenset(self.config.stop_ids if stop_ids is None else stop_ids)
        sampling = SamplingParams(temperature, top_p, seed)
        reqs = [Request(list(p), max_new_tokens, sampling, stops) for p in prompts]
        self.metrics = RunMetrics()
        return generate(self, reqs, on_token=on_token, max_batch=max_batch, metrics=self.metrics)

    def generate_tokens(self, prompt_tokens, stop_tokens, max_tokens, sampler, echo=False, on_token_generated=None):
        """One sequence, in the reference's own terms (J/model/Model.java:66,
        J/inference/InferenceEngine.java:67-141): ``max_tokens`` bounds the position
        (prompt and generated together; negative: the context length), the returned
        list holds the generated tokens only, a stop token included."""
        limit = self.max_context if max_tokens is None or max_tokens < 0 else min(max_tokens, self.max_context)
        new = limit - len(prompt_tokens) + 1
        req = Request(list(prompt_tokens), new, sampler, frozenset(stop_tokens or ()))

        def seen(_, tok):
            if echo:
                import sys
                print(tok, end=" ", file=sys.stderr, flush=True)
            if on_token_generated is not None:
                on_token_generated(tok)

        self.metrics = RunMetrics()
        return generate(self, [req], on_token=seen, metrics=self.metrics)[0].tokens


__all__ = ["Engine", "CacheFull", "Generated", "Request", "RunMetrics"]

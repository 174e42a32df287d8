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

import array
import contextlib
import tempfile
from collections import OrderedDict

import numpy as np
import torch

from ..cache import Cache, CacheFull, check_layout
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


RUN_LENGTH = 16     # most decode steps that run on the device before the host looks at the tokens
_current_device = getattr(torch._C, "_cuda_getDevice", None)


class _DecodeGraph:
    """A captured decode step for one batch bucket: its input buffer on the device and its logits;
    for runs of steps also the sampling of the next tokens and their feeding back."""
    graph = handle = logits = dev = step = fhost = fdev = None
    B_pad = n_input = off_sampled = off_hist = 0

    def launch(self):
        from ..csrc import lib as K
        if self.handle is not None:
            K.graph_launch(self.handle)
        else:
            self.graph.replay()


GRAPHS_KEPT = 24    # captured decode steps that an engine keeps (each owns its logits and the sampler's scratch)


def _without(without, weight_copies):
    from ..parts import ops
    names = set(ops.switches(without))
    if not weight_copies:
        names.add("tiled")
    elif weight_copies == "both":
        names.add("once")
    return frozenset(names)


class Engine:
    """``config``: a registered architecture's configuration; ``weights``: stored name -> device tensor.

    ``weight_copies``: a bfloat16 engine keeps, beside each matrix that decode steps read (QKV, output and down
    projection, the head, and the gate/up rows of small models), a copy in the order in which the matrix cores
    take it, and lets the stored order of those go (the gate/up rows of large models, which no step reads in
    another order, stay as stored; the output projection may keep two copies, in strips of 16 and of 8): 2.5 ->
    2.6 GB for the 1B shape, for 16% more tokens a second at batch 8. False leaves the copies out; "both" keeps
    the stored order of every matrix too (4.0 GB). ``without``: names of fast paths (``parts.ops.SWITCHES``) this engine does not use, for
    measurements and tests. ``max_graphs``: captured decode steps kept at a time; the least recently used
    one goes first."""

    def __init__(self, config, weights, dtype="bfloat16", device="cuda:0", max_tokens=None, max_context=None,
                 n_slots=None, page_size=64, use_graphs=True, without=(), weight_copies=True, max_graphs=GRAPHS_KEPT):
        self.device = _require_gpu(device)
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        self.dtype = _dtype(dtype)
        self.without = _without(without, weight_copies)
        limit = config.max_position_embeddings
        max_context = limit if max_context is None or max_context < 0 else min(max_context, limit)
        self.config = config.with_context_length(max_context)
        self.spec = self.config.model_spec()
        self.max_context = max_context
        max_tokens = max_tokens or max_context
        self.model = DecoderModel(self.spec, self.dtype, self.device, without=self.without)
        kv_needs, state_needs = self.model.cache_needs()
        check_layout(kv_needs, page_size)                 # before the weights are stacked and copied
        self.model.load(weights)
        if n_slots is None:
            n_slots = max(1, min(-(-max_tokens // page_size), 256))
        with torch.cuda.device(self.device):
            self.cache = Cache(kv_needs, state_needs, max_tokens, max_context, n_slots, self.dtype, self.device,
                               page_size)
        self.workspace = Workspace(self.device)
        self.sampler = DeviceSampler(self.device)
        self.metrics = RunMetrics()
        # Decode steps are replayed from captured graphs when every part's work is made of kernel
        # launches on the current stream alone. (Per-slot state is no obstacle: an entry that pads a
        # bucketed batch works on the cache's sink slot, which no sequence owns.)
        parts = [p for b in self.model.blocks for p in b.parts()]
        safe = all(getattr(p, "graph_safe", False) for p in parts)
        self.use_graphs = bool(use_graphs and safe)
        self.fuse = bool(self.dtype == torch.bfloat16 and safe)
        if max_graphs < 1:
            raise ValueError("max_graphs must be at least 1")
        self.max_graphs = int(max_graphs)
        self._graphs = OrderedDict()                      # (batch bucket, context bucket, kind) -> captured step
        self._graphs_generation = 0
        self._stage_ring = [(None, None)] * 4             # (pinned buffer, event after the copy out of it)
        self._stage_next = 0

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_folder(cls, folder, dtype="bfloat16", device="cuda:0", **kw):
        """A model folder: config.json picks the architecture, model.safetensors holds the tensors."""
        dev = _require_gpu(device)
        config = load_config(folder)
        probe = DecoderModel(config.model_spec(), _dtype(dtype), "cpu")
        check_layout(probe.cache_needs()[0], kw.get("page_size", 64))       # before the weights are read
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
        """Stored name -> device tensor (stacked matrices appear as views under their stored names). A matrix that
        the engine keeps in the matrix cores' order alone is put back into the stored order for the caller: a
        tensor of the caller's own, made at each call."""
        from ..parts import ops
        return {name: ops.stored(w) for name, w in self.model.weights.items()}

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

        Each sequence's tokens (a list, a tuple or an array of integers) are appended at its own
        length. ``want``: "last" (the last token of every entry), "all", "none", or a list with one
        list of indices into each entry's tokens. Returns ``[rows, vocab]`` float32 on the
        device, rows in the order of the entries and of their wanted indices: a tensor
        of its own, which later steps do not touch. If the cache has no room,
        ``CacheFull`` is raised and nothing has changed.
        """
        B = len(entries)
        V = self.spec.vocab_size
        if B == 0:
            return torch.empty((0, V), dtype=torch.float32, device=self.device)
        slots, arrays, ints = self._entries(entries)          # (ints: every entry is a list of one int, kept as ints)
        counts = [1] * B if ints else [a.size for a in arrays]
        single = ints or max(counts) == 1
        if single and want != "last" and isinstance(want, (list, tuple)) and len(want) == B \
                and all(len(w) == 1 and w[0] == 0 for w in want):
            want = "last"                         # the only token of every entry: the same step
        if single and want == "last" and self.use_graphs:
            return self._step_decode(slots, arrays if ints else [int(a[0]) for a in arrays])
        if ints:
            arrays = [np.array([t], dtype=np.int32) for t in arrays]
        starts = [self.cache.length(s) for s in slots]
        T = sum(counts)
        tokens = arrays[0] if B == 1 else np.concatenate(arrays)
        if want == "last":
            rows = np.cumsum(counts, dtype=np.int32) - 1
        elif want == "all":
            rows = np.arange(T, dtype=np.int32)
        elif want == "none" or want is None:
            rows = np.empty(0, dtype=np.int32)
        else:
            if len(want) != B:
                raise ValueError(f"{len(want)} lists of wanted places for {B} entries")
            rows, first = [], 0
            for b, n in enumerate(counts):
                idx = [int(i) for i in want[b]]
                if any(not 0 <= i < n for i in idx):
                    raise ValueError(f"entry {b}: a wanted place is outside its {n} tokens")
                rows.extend(first + i for i in idx)
                first += n
            rows = np.asarray(rows, dtype=np.int32)
        self.cache.reserve(dict(zip(slots, counts)))                   # raises CacheFull, nothing changed
        W = int(rows.size)
        max_kv = max(k + n for k, n in zip(starts, counts))
        from ..csrc import lib as K
        with self._on_device():
            self.cache.flush_tables()
            ctx = StepContext(self, T, B, counts, starts, slots, decode=single, max_q_len=max(counts), max_kv_len=max_kv)
            dev = torch.empty(K.stage_step_ints(T, B, W), dtype=torch.int32, device=self.device)
            K.stage_step(dev, self._staging(T + 3 * B + 1 + W), tokens, slots, starts, counts, rows, V)
            self._staged()
            o = 0

            def cut(n):
                nonlocal o
                t = dev[o:o + n]
                o += n
                return t

            ctx.token_ids, ctx.cu_seqlens, ctx.kv_before, ctx.slot_ids = cut(T), cut(B + 1), cut(B), cut(B)
            want_rows = cut(W)
            ctx.positions, ctx.seq_of_token, ctx.table_rows = cut(T), cut(T), cut(T)
            ctx.seq_rows = ctx.slot_ids
            ctx._tables = [self.cache.device_table(g) for g in range(len(self.cache.groups))]
            logits = self.model.forward(ctx, want_rows)
        for s, n in zip(slots, counts):
            self.cache.advance(s, n)
        return logits

    def _entries(self, entries):
        """What every step checks before anything changes: ``(slots, tokens per entry, all_single)``. Slots are
        integers that appear once; tokens are integers inside the vocabulary, at least one an entry. When every
        entry brings a list of one int (the usual decode step) the tokens come back as those ints and
        ``all_single`` is true; else as one int32 array per entry."""
        V = self.spec.vocab_size
        slots, arrays, all_single = [], [], True
        for b, (slot, toks) in enumerate(entries):
            if type(toks) is list and len(toks) == 1 and type(toks[0]) is int:
                a = toks[0]
                lo = hi = a
            else:
                all_single = False
                a = None
                if type(toks) is list:          # (a list of ints, as a tokenizer gives it: half the time of numpy's own walk)
                    try:
                        a = np.frombuffer(array.array("i", toks), dtype=np.int32)
                    except (TypeError, OverflowError):
                        a = None
                if a is None:
                    a = np.asarray(toks.cpu() if isinstance(toks, torch.Tensor) else toks)
                if a.ndim == 0:
                    a = a.reshape(1)
                if a.ndim != 1 or (a.size and a.dtype.kind not in "iu"):
                    raise ValueError(f"entry {b}: tokens must be a flat sequence of integers")
                if a.size == 0:
                    raise ValueError(f"entry {b} brings no token")
                lo, hi = int(a.min()), int(a.max())
                a = a.astype(np.int32, copy=False)
            if lo < 0 or hi >= V:
                raise ValueError(f"entry {b}: token id {lo if lo < 0 else hi} is outside the vocabulary of {V}")
            slots.append(int(slot))
            arrays.append(a)
        if len(set(slots)) != len(slots):
            raise ValueError("a slot appears twice in one step")
        if not all_single:
            arrays = [np.array([a], dtype=np.int32) if type(a) is int else a for a in arrays]
        return slots, arrays, all_single

    def _staging(self, n):
        """Pinned host memory for the next step's input: one of a ring of buffers, free once the copy out of it
        (of the step that used it last) has run."""
        ring = self._stage_ring
        self._stage_next = (self._stage_next + 1) % len(ring)
        buf, event = ring[self._stage_next]
        if event is not None:
            event.synchronize()
        if buf is None or buf.numel() < n:
            buf = torch.empty(max(4096, 2 * n), dtype=torch.int32).pin_memory()
        ring[self._stage_next] = (buf, event)
        return buf

    def _staged(self):
        buf, event = self._stage_ring[self._stage_next]
        if event is None:
            event = torch.cuda.Event()
        event.record()
        self._stage_ring[self._stage_next] = (buf, event)

    # ------------------------------------------------------------------ decode steps from captured graphs
    @property
    def decode_run_length(self):
        return RUN_LENGTH if self.use_graphs else 1


    def _on_device(self):
        """The engine's device as the current one (entering a device context costs as much as a launch)."""
        if _current_device is not None and _current_device() == self.device.index:
            return contextlib.nullcontext()
        return torch.cuda.device(self.device)

    def _step_decode(self, slots, tokens):
        """One token for each of B sequences (checked by ``_entries``): the step's tokens, positions and slot numbers are
        written into the captured step's input buffer by a small kernel that carries them in its
        launch, and the captured launches are replayed. The batch is padded to a bucket; a padded
        entry is a one-token sequence in the cache's sink slot, so it reads and writes nothing
        that a real sequence owns, and its logits are not returned."""
        from ..csrc import lib as K
        starts = [self.cache.length(s) for s in slots]
        B = len(slots)
        cache = self.cache
        cache.reserve_one_each(slots)                                  # raises CacheFull, nothing changed
        with self._on_device():
            dg = self._graph_for(B, max(starts) + 1, run=False)
            cache.flush_tables()
            K.stage_decode(dg.dev, dg.B_pad, tokens, starts, slots, cache.sink_slot)
            dg.launch()
            logits = dg.logits[:B].clone()       # the graph's own buffer is overwritten by the next step
        cache.advance_one_each(slots)
        return logits

    def decode_run(self, entries, n, temperatures, top_ps, uniforms):
        """``n`` decode steps in a row for ``entries = [(slot, token), ...]``: every step samples
        each sequence's next token on the device and feeds it back, the host waits once at the
        end. ``uniforms[k][r]`` is step k's uniform number for entry r. Returns the sampled
        tokens ``[n][len(entries)]``. The cache has all n positions reserved before the first
        step, or ``CacheFull`` is raised and nothing has changed."""
        if not self.use_graphs or not 1 <= n <= RUN_LENGTH:
            raise ValueError(f"a run takes 1..{RUN_LENGTH} steps on an engine that replays graphs")
        from ..csrc import lib as K
        slots, arrays, ints = self._entries([(s, [t] if isinstance(t, int) else t) for s, t in entries])
        if not ints and any(a.size != 1 for a in arrays):
            raise ValueError("a run of decode steps starts from one token per sequence")
        tokens = arrays if ints else [int(a[0]) for a in arrays]
        starts = [self.cache.length(s) for s in slots]
        B = len(slots)
        self.cache.reserve({s: n for s in slots})
        with self._on_device():
            greedy = all(t == 0 for t in temperatures)
            dg = self._graph_for(B, max(starts) + n, run="greedy" if greedy else "sampled")
            self.cache.flush_tables()
            B_pad = dg.B_pad
            f = dg.fhost                          # (free again: the last run ended with a wait for its tokens)
            f.zero_()
            f[0:B] = torch.tensor(list(temperatures), dtype=torch.float32)
            f[B_pad:B_pad + B] = torch.tensor(list(top_ps), dtype=torch.float32)
            u = torch.tensor([list(row) for row in uniforms], dtype=torch.float32)        # [n, B]
            f[2 * B_pad:2 * B_pad + RUN_LENGTH * B_pad].view(RUN_LENGTH, B_pad)[:n, :B] = u
            dg.fdev.copy_(f, non_blocking=True)
            K.stage_decode(dg.dev, B_pad, tokens, starts, slots, self.cache.sink_slot, counter=dg.step)
            for _ in range(n):
                dg.launch()
            hist = dg.dev[dg.off_hist:dg.off_hist + RUN_LENGTH * B_pad].view(RUN_LENGTH, B_pad)[:n, :B].cpu()
        for s in slots:
            self.cache.advance(s, n)
        return hist.tolist()

    def _graph_for(self, B, max_kv, run):
        if self._graphs_generation != self.workspace.generation:
            self._graphs.clear()                 # a scratch buffer moved: the captured addresses are stale
            self._graphs_generation = self.workspace.generation
        B_pad = B if B <= 8 else -(-B // 8) * 8
        kv_bucket = 256
        while kv_bucket < max_kv:
            kv_bucket *= 2
        key = (B_pad, kv_bucket, run)
        dg = self._graphs.get(key)
        if dg is None:
            if len(self._graphs) >= self.max_graphs:
                torch.cuda.synchronize(self.device)                      # no replay of it is still running
            while len(self._graphs) >= self.max_graphs:                  # the least recently used one goes
                self._graphs.popitem(last=False)
            dg = self._capture(B_pad, kv_bucket, run)
            if self._graphs_generation != self.workspace.generation:    # the warm-up grew a buffer
                self._graphs.clear()
                self._graphs_generation = self.workspace.generation
                dg = self._capture(B_pad, kv_bucket, run)
            self._graphs[key] = dg
        else:
            self._graphs.move_to_end(key)
        return dg

    def _capture(self, B_pad, kv_bucket, run=False):
        from ..csrc import lib as K
        G = len(self.cache.groups)
        dg = _DecodeGraph()
        dg.B_pad = B_pad
        # the part that every step brings: tokens | positions | kv_before | slots | step counter;
        # after it what never changes (sequence of each token, sequence bounds, wanted rows) and, for
        # runs, the sampled tokens and their history
        dg.n_input = 4 * B_pad + 1
        off_seq = dg.n_input
        off_cu = off_seq + B_pad
        off_rows = off_cu + B_pad + 1
        dg.off_sampled = off_rows + B_pad
        dg.off_hist = dg.off_sampled + B_pad
        n = dg.off_hist + RUN_LENGTH * B_pad if run else dg.off_sampled
        fixed = torch.zeros(n, dtype=torch.int32)
        fixed[3 * B_pad:4 * B_pad] = self.cache.sink_slot          # padded entries live in the sink slot
        ar = torch.arange(B_pad + 1, dtype=torch.int32)
        fixed[off_seq:off_seq + B_pad] = ar[:B_pad]                # seq_of_token
        fixed[off_cu:off_cu + B_pad + 1] = ar                      # cu_seqlens
        fixed[off_rows:off_rows + B_pad] = ar[:B_pad]              # wanted rows: every entry's only token
        dg.dev = fixed.to(self.device)
        ctx = StepContext(self, B_pad, B_pad, [1] * B_pad, [0] * B_pad, [self.cache.sink_slot] * B_pad, decode=True,
                          max_q_len=1, max_kv_len=kv_bucket)
        ctx.kv_len_hint = kv_bucket
        ctx.replayed = True
        d = dg.dev
        ctx.token_ids, ctx.positions, ctx.kv_before = d[0:B_pad], d[B_pad:2 * B_pad], d[2 * B_pad:3 * B_pad]
        ctx.slot_ids = d[3 * B_pad:4 * B_pad]
        ctx.table_rows = ctx.seq_rows = ctx.slot_ids               # one token per sequence: its slot is its table row
        step = dg.step = d[4 * B_pad:4 * B_pad + 1]
        ctx.seq_of_token = d[off_seq:off_seq + B_pad]
        ctx.cu_seqlens = d[off_cu:off_cu + B_pad + 1]
        rows = d[off_rows:off_rows + B_pad]
        ctx._tables = [self.cache.device_table(g) for g in range(G)]
        if run:
            dg.fhost = torch.zeros((2 + RUN_LENGTH) * B_pad, dtype=torch.float32).pin_memory()
            dg.fdev = torch.zeros((2 + RUN_LENGTH) * B_pad, dtype=torch.float32, device=self.device)
            work = torch.empty(K.sample_work_size(B_pad, self.spec.vocab_size), dtype=torch.float32, device=self.device)
            sampled = d[dg.off_sampled:dg.off_sampled + B_pad]
            hist = d[dg.off_hist:dg.off_hist + RUN_LENGTH * B_pad].view(RUN_LENGTH, B_pad)
            temps, tops = dg.fdev[0:B_pad], dg.fdev[B_pad:2 * B_pad]
            us = dg.fdev[2 * B_pad:]

        def body():
            logits = self.model.forward(ctx, rows)
            if run == "greedy":
                K.argmax_advance(logits, work, sampled, ctx.token_ids, ctx.positions, ctx.kv_before, hist, step)
            elif run:
                K.sample(logits, work, temps, tops, us, sampled, step=step, uniform_stride=B_pad)
                K.decode_advance(ctx.token_ids, ctx.positions, ctx.kv_before, sampled, hist, step)
            return logits

        # once outside a capture: scratch buffers get their sizes, the library is loaded
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            body()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.workspace.frozen = True
        try:
            dg.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(dg.graph):
                dg.logits = body()
        finally:
            self.workspace.frozen = False
        try:
            dg.handle = int(dg.graph.raw_cuda_graph_exec())    # launched without the wrapper's bookkeeping
        except Exception:
            dg.handle = None
        return dg

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

    def create_new_state(self):
        """A sequence that outlives a call of ``generate_tokens``: it holds a slot of the cache
        until ``close`` (the reference's ``createNewState``, J/model/Model.java:78; there the state
        is the cache itself)."""
        return SequenceState(self, self.take_slot())

    def generate_tokens(self, prompt_tokens, stop_tokens, max_tokens, sampler, echo=False, on_token_generated=None,
                        state=None, start_position=0):
        """One sequence, in the reference's own terms (J/model/Model.java:66,
        J/inference/InferenceEngine.java:67-141): ``max_tokens`` bounds the position
        (prompt and generated together; negative: the context length), the returned
        list holds the generated tokens only, a stop token included.

        With a ``state`` the sequence goes on in that state's slot: ``prompt_tokens`` follow the
        ``start_position`` tokens that the slot holds already (the reference's chat loop,
        Model.java:136). The token sampled last is not in the cache when the call returns, as in
        the reference; ``state.length`` says how many are, and the next call's tokens start there."""
        limit = self.max_context if max_tokens is None or max_tokens < 0 else min(max_tokens, self.max_context)
        if state is None:
            if start_position:
                raise ValueError("a start position needs the state that holds the tokens before it")
            slot = None
        else:
            if state.closed:
                raise ValueError("the state has been closed")
            if start_position != state.length:
                raise ValueError(f"the state holds {state.length} tokens; the next tokens start there, "
                                 f"not at {start_position}")
            slot = state.slot
        new = limit - start_position - len(prompt_tokens) + 1
        req = Request(list(prompt_tokens), new, sampler, frozenset(stop_tokens or ()), slot=slot, cached=start_position)

        def seen(_, tok):
            if echo:
                import sys
                print(tok, end=" ", file=sys.stderr, flush=True)
            if on_token_generated is not None:
                on_token_generated(tok)

        self.metrics = RunMetrics()
        return generate(self, [req], on_token=seen, metrics=self.metrics)[0].tokens


class SequenceState:
    """The slot of a sequence that goes on over several calls."""

    def __init__(self, engine, slot):
        self.engine, self.slot, self.closed = engine, slot, False

    @property
    def length(self):
        """Tokens of the sequence that the cache holds."""
        return self.engine.cache.length(self.slot)

    def close(self):
        if not self.closed:
            self.engine.give_back_slot(self.slot)
            self.closed = True

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


__all__ = ["Engine", "SequenceState", "CacheFull", "Generated", "Request", "RunMetrics"]

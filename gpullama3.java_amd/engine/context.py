"""What a step looks like to the parts: the packed tokens of a batch and where each
belongs.

All index arrays are int32 on the device: ``token_ids[T]``, ``positions[T]`` (a
token's place in its own sequence), ``seq_of_token[T]`` (which row of the batch),
``cu_seqlens[B+1]``, ``kv_before[B]`` (tokens a sequence held before this step),
``slot_ids[B]`` (the cache slot of each sequence), and one block table per cache group
with ``table_rows[T]`` / ``seq_rows[B]`` naming the table's row of each token / sequence
(the engine passes the cache's own table, a row per slot, so these are slot numbers; a
context built by hand may bring a table with a row per sequence and leave both unset).
Host copies of the lengths are kept for launch decisions.
"""
from __future__ import annotations

import torch


class Workspace:
    """Named scratch buffers that keep their address from step to step."""

    def __init__(self, device):
        self.device = device
        self._flat = {}
        self.frozen = False
        self.generation = 0        # counts reallocations: captured graphs hold the old addresses

    def get(self, name, shape, dtype):
        n = 1
        for s in shape:
            n *= s
        key = (name, dtype)
        flat = self._flat.get(key)
        if flat is None or flat.numel() < n:
            if self.frozen:
                raise RuntimeError(f"workspace buffer {name!r} would grow while its address is fixed")
            if flat is not None:
                self.generation += 1
            flat = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._flat[key] = flat
        return flat[:n].view(shape)


class StepContext:
    def __init__(self, engine, n_tokens, n_seqs, q_lens, kv_before_host, slots, decode, max_q_len, max_kv_len):
        self.engine = engine
        self.cache = engine.cache
        self.dtype = engine.dtype
        self.device = engine.device
        self.n_tokens, self.n_seqs = n_tokens, n_seqs
        self.q_lens, self.kv_before_host, self.slots = q_lens, kv_before_host, slots
        self.decode = decode
        self.replayed = False              # whether the step's launches are being captured into a graph
        self.max_q_len, self.max_kv_len = max_q_len, max_kv_len
        self.fuse = getattr(engine, "fuse", False)   # few-token steps fold norms and rotation into the products
        self.disabled = getattr(engine, "without", frozenset())   # fast paths that the engine does without
        self.ssq = None                    # (address of the residual stream, its partial sums of squares, how many)
        self.pending = None                # (address of the residual stream, slices of a product still to be added to it)
        self.kv_len_hint = max_kv_len      # what launch shapes are sized for; a replayed graph keeps its own
        self.token_ids = self.positions = self.seq_of_token = self.cu_seqlens = self.kv_before = None
        self.slot_ids = None
        self._tables = []
        self._table_rows = self._seq_rows = None

    def block_table(self, group):
        return self._tables[group]

    @property
    def table_rows(self):
        """[T] the row of the block table that holds each token's sequence."""
        return self._table_rows if self._table_rows is not None else self.seq_of_token

    @table_rows.setter
    def table_rows(self, v):
        self._table_rows = v

    @property
    def seq_rows(self):
        """[B] the row of the block table of each sequence; None: sequence b has row b."""
        return self._seq_rows

    @seq_rows.setter
    def seq_rows(self, v):
        self._seq_rows = v

    def buffer(self, name, shape, dtype):
        return self.engine.workspace.get(name, shape, dtype)

    def ssq_buffer(self, n_partials):
        """[n_partials, 64] partial sums of squares; one buffer, as large as the widest writer needs."""
        most = max(n_partials, -(-self.engine.spec.hidden // 8))
        return self.buffer("ssq", (most, 64), torch.float32)[:n_partials]

    def logits_buffer(self, n_rows, vocab):
        return torch.empty((n_rows, vocab), dtype=torch.float32, device=self.device)

    def slot_state(self, entry):
        """``[n_slots + 1, elements]`` state of one run-order entry; index with ``slot_ids`` (the last
        row belongs to the entries that pad a batch: no sequence's)."""
        return self.cache.slot_state(entry)

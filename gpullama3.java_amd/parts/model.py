"""The decoder: embedding, blocks in their run order, final norm, head.

Built from a ``ModelSpec`` alone. The run order is data: an entry names a layer
(possibly one already named) and, optionally, an earlier entry whose keys and
values it reads instead of making its own.
"""
from __future__ import annotations

import torch

from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import RunInfo, build_part


def expected_tensors(spec, dtype=torch.float32, device="cpu"):
    """Stored name -> TensorSpec of every tensor the model needs (no memory is used)."""
    out = {spec.embedding_name: TensorSpec((spec.vocab_size, spec.hidden))}
    if spec.head_name is not None:
        out[spec.head_name] = TensorSpec((spec.vocab_size, spec.hidden))
    if spec.position_table_name is not None:
        out[spec.position_table_name] = TensorSpec((spec.max_positions, spec.hidden))
    if spec.head_bias_name is not None:
        out[spec.head_bias_name] = TensorSpec((spec.vocab_size,), "vector")
    if spec.final_norm is not None:
        out.update(_norm_tensors(spec.final_norm))
    for b in spec.layers:
        block = build_part("block", b, dtype=dtype, device=device)
        for p in block.parts():
            out.update(p.tensors())
    return out


def _block_needs(block):
    """(KVNeed or None, StateNeed or None) of one run of a block: what the block says itself
    (``cache_needs()``), else what the one of its parts that keeps something per position or per
    sequence says."""
    if hasattr(block, "cache_needs"):
        return block.cache_needs()
    keepers = [p for p in block.parts() if hasattr(p, "kv_need")]
    if len(keepers) > 1:
        raise ValueError("a block with several parts that keep keys, values or state must say what it needs itself "
                         "(cache_needs)")
    return (keepers[0].kv_need(), keepers[0].state_need()) if keepers else (None, None)


def _norm_tensors(spec):
    return build_part("norm", spec, dtype=torch.float32).tensors()


class DecoderModel:
    """``without``: names of fast paths (``ops.SWITCHES``) that this model's engine does without; every part
    finds them as its attribute ``without`` when it loads its weights."""

    def __init__(self, spec, dtype, device, without=frozenset()):
        self.spec, self.dtype, self.device = spec, dtype, device
        self.without = ops.switches(without)
        self.blocks = [build_part("block", b, dtype=dtype, device=device) for b in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, dtype=dtype) if spec.final_norm is not None else None
        # (a layer whose queries read another entry's keys and values needs the q rows alone: then stacked rows keep
        # their stored order)
        may_hold_once = not any(r.reads is not None for r in spec.run_order)
        for part in [p for b in self.blocks for p in b.parts()] + [self.final_norm]:
            if part is not None:
                part.without = self.without
                part.may_hold_once = may_hold_once
        self.runs = []
        for e, r in enumerate(spec.run_order):
            if not 0 <= r.layer < len(self.blocks):
                raise ValueError(f"run order entry {e} names layer {r.layer} of {len(self.blocks)}")
            if r.reads is not None and not (0 <= r.reads < e and spec.run_order[r.reads].reads is None):
                raise ValueError(f"run order entry {e} reads entry {r.reads}, which is not an earlier entry "
                                 "with keys and values of its own")
            self.runs.append(RunInfo(entry=e, kv_entry=e if r.reads is None else r.reads,
                                     writes_kv=r.reads is None))
        self.embedding = self.head = self.position_table = self.head_bias = None
        self.weights = {}

    def expected(self):
        out = {self.spec.embedding_name: TensorSpec((self.spec.vocab_size, self.spec.hidden))}
        if self.spec.head_name is not None:
            out[self.spec.head_name] = TensorSpec((self.spec.vocab_size, self.spec.hidden))
        if self.spec.position_table_name is not None:
            out[self.spec.position_table_name] = TensorSpec((self.spec.max_positions, self.spec.hidden))
        if self.spec.head_bias_name is not None:
            out[self.spec.head_bias_name] = TensorSpec((self.spec.vocab_size,), "vector")
        if self.final_norm is not None:
            out.update(self.final_norm.tensors())
        for b in self.blocks:
            for p in b.parts():
                out.update(p.tensors())
        return out

    def load(self, weights):
        self.weights = weights
        self.embedding = weights[self.spec.embedding_name]
        self.head = self.embedding if self.spec.head_name is None else weights[self.spec.head_name]
        ops.for_few_rows(self.head, without=self.without)
        if ops.can_hold_once(self.head, self.without):
            # every reader of the head (and of a tied embedding) takes the matrix operands' order: the stored
            # order is let go, the copy stands for the matrix under its stored name
            name = self.spec.embedding_name if self.spec.head_name is None else self.spec.head_name
            self.head = weights[name] = K.hold_once(self.head)
            if self.spec.head_name is None:
                self.embedding = self.head
        if self.spec.position_table_name is not None:
            self.position_table = weights[self.spec.position_table_name].to(self.embedding.dtype)
        if self.spec.head_bias_name is not None:     # the epilogues read biases as float
            self.head_bias = weights[self.spec.head_bias_name].float().contiguous()
        if self.final_norm is not None:
            self.final_norm.load(weights)
        for b in self.blocks:
            for p in b.parts():
                p.load(weights)

    def cache_needs(self):
        kv, state = [], []
        for run, r in zip(self.runs, self.spec.run_order):
            kv_need, state_need = _block_needs(self.blocks[r.layer])
            kv.append(kv_need if run.writes_kv else None)
            state.append(state_need)
        return kv, state

    def forward(self, ctx, want_rows):
        """Logits ``[len(want_rows), vocab]`` float32 at the wanted packed rows."""
        x = ctx.buffer("residual", (ctx.n_tokens, self.spec.hidden), torch.float32)
        ctx.ssq = ctx.pending = ctx.next_norm = None   # a context may run more than one forward pass: nothing is left over
        ctx.token_facts, ctx.token_tables = {}, {}
        order = [self.blocks[r.layer] for r in self.spec.run_order]
        # the norm that reads the residual rows after entry i of the run order, where the block says which
        firsts = [getattr(b, "first_norm", lambda: None)() for b in order] + [self.final_norm]
        around = {}
        if self.spec.embedding_scale is not None:
            around["scale"] = self.spec.embedding_scale
        if self.position_table is not None:
            around.update(pos_table=self.position_table, positions=ctx.positions)
        if getattr(ctx, "fuse", False) and ctx.n_tokens <= ops.FUSE_ROWS and getattr(firsts[0], "folds", False):
            # the first norm's sums of squares, and its rows times its weight, come with the embedding
            ssq = ctx.ssq_buffer(1)
            xg = ctx.buffer("rows_times_norm_weight", (ctx.n_tokens, self.spec.hidden), torch.bfloat16)
            K.embed(self.embedding, ctx.token_ids, x, ssq, firsts[0].weight_f32, xg, **around)
            ops.residual_written(ctx, x, ssq, 1, xg, firsts[0])
        else:
            K.embed(self.embedding, ctx.token_ids, x, **around)
            ops.residual_written(ctx, x)
        for i, (run, block) in enumerate(zip(self.runs, order)):
            if hasattr(block, "first_norm"):
                block.forward(ctx, x, run, norm_after=firsts[i + 1])
            else:
                # an arrangement of its own may read the rows as they are: they are made whole first, and
                # nothing is left in slices or prepared for a folded norm while it runs
                ops.settle_residual(ctx, x)
                fuse, ctx.fuse = ctx.fuse, False
                try:
                    block.forward(ctx, x, run)
                finally:
                    ctx.fuse = fuse
                if ctx.pending is not None:
                    raise RuntimeError("a block left sums of a product in slices behind it")
                ops.residual_written(ctx, x)
        n = want_rows.numel()
        logits = ctx.logits_buffer(n, self.spec.vocab_size)
        if n:
            if self.final_norm is not None:
                h = self.final_norm(ctx, x, rows=want_rows, name="final_normed")
            else:
                # a decoder without a final norm: the head reads the wanted rows as they are
                ops.settle_residual(ctx, x)
                h = ctx.buffer("head_rows", (n, self.spec.hidden), self.dtype)
                K.gather_rows(x, want_rows, h)
            ops.linear(h, self.head, logits, ops.EPI_STORE, ctx, bias=self.head_bias)
            if self.spec.logit_scale is not None:
                K.scale_(logits, self.spec.logit_scale)
            if self.spec.logit_softcap is not None:
                K.softcap_(logits, self.spec.logit_softcap)
        return logits

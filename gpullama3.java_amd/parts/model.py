"""The decoder: embedding, blocks in their run order, final norm, head.

Built from a ``ModelSpec`` alone. The run order is data: an entry names a layer
(possibly one already named) and, optionally, an earlier entry whose keys and
values it reads instead of making its own.
"""
from __future__ import annotations

import torch

from ..csrc import lib as K
from ..cache import StateNeed
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
    out.update(_inject_tensors(spec))
    out.update(_around_tensors(spec))
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


def _around_tensors(spec):
    """What stands around the blocks beside embedding, head and final norm: the table of token pairs, and the matrices
    that mix the residual rows with the embedding's output in front of a run-order entry."""
    out = {}
    pair = getattr(spec, "pair_embedding", None)
    if pair is not None:
        out[pair.table_name] = TensorSpec((pair.buckets + 1, spec.hidden))
    for r in spec.run_order:
        b = getattr(r, "before", None)
        if b is not None and hasattr(b, "weight_name"):
            out[b.weight_name] = TensorSpec((spec.hidden, 2 * spec.hidden))
    return out


def _inject_tensors(spec):
    """The tables of vectors that entries of the run order add to the residual rows before they run."""
    out = {}
    for r in spec.run_order:
        b = getattr(r, "before", None)
        if b is not None and getattr(b, "vector_name", None) is not None:
            if not 0 <= b.row < b.vector_rows:
                raise ValueError(f"a run-order entry adds row {b.row} of {b.vector_name!r}, which has {b.vector_rows}")
            out[b.vector_name] = TensorSpec((b.vector_rows, spec.hidden), "matrix")
    return out


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
        out.update(_inject_tensors(self.spec))
        out.update(_around_tensors(self.spec))
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
        # what entries of the run order add to the residual rows, which are 32-bit: the vectors in 32-bit
        self.inject_vectors = {name: weights[name].float().contiguous() for name in _inject_tensors(self.spec)}
        self.keeps_embedding = any(getattr(r, "before", None) is not None
                                   and (getattr(r.before, "embedding", False) or hasattr(r.before, "weight_name"))
                                   for r in self.spec.run_order)
        pair = getattr(self.spec, "pair_embedding", None)
        self.pair_table = weights[pair.table_name].to(self.embedding.dtype) if pair is not None else None
        self.remix = {}
        for r in self.spec.run_order:
            b = getattr(r, "before", None)
            if b is not None and hasattr(b, "weight_name") and b.weight_name not in self.remix:
                self.remix[b.weight_name] = ops.for_few_rows(weights[b.weight_name], without=self.without)
        for b in self.blocks:
            for p in b.parts():
                p.load(weights)

    def cache_needs(self):
        kv, state = [], []
        for run, r in zip(self.runs, self.spec.run_order):
            kv_need, state_need = _block_needs(self.blocks[r.layer])
            kv.append(kv_need if run.writes_kv else None)
            state.append(state_need)
        if getattr(self.spec, "pair_embedding", None) is not None:
            # one more state area behind the run order's: every sequence's last token, for the table of token pairs
            kv.append(None)
            state.append(StateNeed(1, torch.int32))
        return kv, state

    def forward(self, ctx, want_rows):
        """Logits ``[len(want_rows), vocab]`` float32 at the wanted packed rows."""
        S = int(getattr(self.spec, "streams", 1) or 1)      # copies of the residual row per token
        x = ctx.buffer("residual", (ctx.n_tokens, self.spec.hidden), torch.float32)
        ctx.ssq = ctx.pending = ctx.next_norm = None   # a context may run more than one forward pass: nothing is left over
        ctx.token_facts, ctx.token_tables = {}, {}
        ctx.rows_as_input = None        # (the address of rows whose copy in the activations' type a block has left)
        order = [self.blocks[r.layer] for r in self.spec.run_order]
        # the norm that reads the residual rows after entry i of the run order, where the block says which
        firsts = [getattr(b, "first_norm", lambda: None)() for b in order] + [self.final_norm]
        around = {}
        if self.spec.embedding_scale is not None:
            around["scale"] = self.spec.embedding_scale
        if self.position_table is not None:
            around.update(pos_table=self.position_table, positions=ctx.positions)
        pair = getattr(self.spec, "pair_embedding", None)
        if pair is not None:
            # the row of the pair table per token (the embedding kernel adds a row of a second table by index: here the
            # index is the pair's hash, not the position); the sequences' last tokens move on in their slots
            if self.position_table is not None:
                raise ValueError("a decoder has learned positions or a table of token pairs, not both")
            pair_rows = ctx.buffer("pair_rows", (ctx.n_tokens,), torch.int32)
            K.pair_rows(ctx.token_ids, ctx.positions, ctx.seq_of_token, ctx.cu_seqlens, ctx.slot_ids,
                        ctx.cache.slot_state(len(self.runs)), pair.mul_prev, pair.mul_cur, pair.buckets, pair_rows)
            around.update(pos_table=self.pair_table, positions=pair_rows)
        if getattr(ctx, "fuse", False) and ctx.n_tokens <= ops.FUSE_ROWS and getattr(firsts[0], "folds", False):
            # the first norm's sums of squares, and its rows times its weight, come with the embedding
            ssq = ctx.ssq_buffer(1)
            xg = ctx.buffer("rows_times_norm_weight", (ctx.n_tokens, self.spec.hidden), torch.bfloat16)
            K.embed(self.embedding, ctx.token_ids, x, ssq, firsts[0].weight_f32, xg, **around)
            ops.residual_written(ctx, x, ssq, 1, xg, firsts[0])
        else:
            K.embed(self.embedding, ctx.token_ids, x, **around)
            ops.residual_written(ctx, x)
        if S > 1:
            # every copy starts as the embedding's output; the blocks work on all of them, [T, S d]
            one, x = x, ctx.buffer("residual_copies", (ctx.n_tokens, S * self.spec.hidden), torch.float32)
            K.streams_fill(one, x, S)
            ops.residual_written(ctx, x)
        embedded = None
        if getattr(self, "keeps_embedding", False):
            # a later entry of the run order adds the embedding's output back: looked up once more, into rows of its own
            embedded = ctx.buffer("embedding_output", (ctx.n_tokens, self.spec.hidden), torch.float32)
            K.embed(self.embedding, ctx.token_ids, embedded, **around)
        for i, (run, block) in enumerate(zip(self.runs, order)):
            before = getattr(self.spec.run_order[i], "before", None)
            if before is not None or not getattr(block, "keeps_rows_copy", False):
                ctx.rows_as_input = None
            if before is not None and hasattr(before, "weight_name"):
                # x <- W [x; x0]: the rows and the embedding's output side by side as the product's input
                ops.settle_residual(ctx, x)
                both = ctx.buffer("rows_and_embedding", (ctx.n_tokens, 2 * self.spec.hidden), self.dtype)
                K.concat_rows(x, embedded, both)
                ops.linear(both, self.remix[before.weight_name], x, ops.EPI_STORE, ctx)
                ops.residual_written(ctx, x)
            elif before is not None:
                ops.settle_residual(ctx, x)
                vec = self.inject_vectors[before.vector_name][before.row] if before.vector_name is not None else None
                K.residual_inject(x, embedded if before.embedding else None, vec)
                ops.residual_written(ctx, x)
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
            watch = getattr(ctx.engine, "after_block", None)
            if watch is not None:          # a caller that looks at the residual rows after every entry of the run order
                ops.settle_residual(ctx, x)
                watch(i, x)
        n = want_rows.numel()
        logits = ctx.logits_buffer(n, self.spec.vocab_size)
        if n:
            if S > 1:
                # the copies' sum at the wanted rows is what the final norm and the head read
                ops.settle_residual(ctx, x)
                copies, x = x, ctx.buffer("residual_wanted", (n, self.spec.hidden), torch.float32)
                K.streams_sum(copies, S, x, which=want_rows)
                want_rows = None                       # (every row of x, in order)
                ops.residual_written(ctx, x)
            if self.final_norm is not None:
                h = self.final_norm(ctx, x, rows=want_rows, name="final_normed")
            else:
                # a decoder without a final norm: the head reads the wanted rows as they are
                ops.settle_residual(ctx, x)
                h = ctx.buffer("head_rows", (n, self.spec.hidden), self.dtype)
                if want_rows is None:
                    K.cast_rows(x, h)
                else:
                    K.gather_rows(x, want_rows, h)
            ops.linear(h, self.head, logits, ops.EPI_STORE, ctx, bias=self.head_bias)
            if self.spec.logit_scale is not None:
                K.scale_(logits, self.spec.logit_scale)
            if self.spec.logit_softcap is not None:
                K.softcap_(logits, self.spec.logit_softcap)
        return logits

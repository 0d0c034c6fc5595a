"""Causal attention whose keys and values are expanded from one small latent per position.

    c_q = RMSnorm(W_dq h);  q = W_uq c_q            per head [head_dim unrotated | rot_dim rotated]
    W_dkv h = [c' | r'];    c = RMSnorm(c'),  r = the rot_dim part turned by the position: ONE for all heads
    key_h = [W_uk,h c | r],  value_h = W_uv,h c;   softmax((q_h . key_h) scale) over the positions so far
    output = W_o ((the heads' outputs) * sigmoid(W_g h))

The cache keeps per position the row [c | r] alone (padded with zeros to a multiple of 32), for all heads together:
``KVNeed(1 head, values=False)``. The heads' keys and values are never written out. Since
``q_h . (W_uk,h c) = (W_uk,h^T q_h) . c``, the unrotated part of a head's query is taken through ``W_uk,h^T`` into a row
of ``kv_rank`` numbers (the grouped product of ``csrc/routed.hip``, with the heads in the experts' place), the rotated
part is put behind it, and the attention runs over the cached rows as they are: one key head shared by all query
heads, whose values are the keys' first ``kv_rank`` elements (``lib.latent_attention`` on the matrix cores, which
stages a chunk of cached rows in shared memory once for all heads of a tile; ``lib.attention_generic`` with
``values_in_keys`` in 32-bit and for sizes that kernel is not built for). Its
output, the weighted sum of latents per head, goes through ``W_uv,h`` (the grouped product again), the gate and the
output projection.

Norms, angles and the rotation are 32-bit: the stacked product of the mixer's input (query latent, key/value latent and
shared key part, gate) leaves its sums in 32-bit, and ``lib.latent_prep`` norms, turns and writes the cache from there.
"""
from __future__ import annotations

import torch

from ..cache import KVNeed
from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import build_part, register_part


class LatentAttention:
    graph_safe = True      # kernel launches on the current stream only, sizes fixed by the step's tokens
    adds_only = True       # never reads the residual rows

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype, self.device = spec, dtype, device
        self.d, self.H, self.D, self.R, self.vd = spec.hidden, spec.n_heads, spec.head_dim, spec.rot_dim, spec.v_head_dim
        self.q_rank, self.rank = spec.q_rank, spec.kv_rank
        if self.R % 2:
            raise ValueError(f"a rotated key part of {self.R} elements: pairs need an even count")
        self.position = build_part("position", spec.position, device=device) if spec.position is not None and self.R else None
        if self.position is not None and (self.position.rot_dim != self.R or not self.position.adjacent):
            raise ValueError("the rotated key part is turned as a whole, in adjacent pairs")
        if self.R and self.position is None:
            raise ValueError("a rotated key part needs a rotation")
        self.dk = -(-(self.rank + self.R) // 32) * 32        # a cached row: whole steps of the matrix cores' first product
        self.names = spec.names
        self.out_mult = float(getattr(spec, "out_mult", 1.0))
        self.off_q, self.off_kv = 0, self.q_rank
        self.off_g = self.q_rank + self.rank + self.R
        self.n_in = self.off_g + self.H * self.vd
        self.n_pad = -(-self.n_in // 16) * 16
        self.w_in = self.w_uq = self.w_uk_t = self.w_uv = self.w_o = self.q_norm = self.kv_norm = self.out_scale = None

    def tensors(self):
        n, d, H = self.names, self.d, self.H
        return {n["dq"]: TensorSpec((self.q_rank, d)), n["dq_norm"]: TensorSpec((self.q_rank,), "vector"),
                n["uq"]: TensorSpec((H * (self.D + self.R), self.q_rank)),
                n["dkv"]: TensorSpec((self.rank + self.R, d)), n["dkv_norm"]: TensorSpec((self.rank,), "vector"),
                n["uk"]: TensorSpec((H * self.D, self.rank)), n["uv"]: TensorSpec((H * self.vd, self.rank)),
                n["g"]: TensorSpec((H * self.vd, d)), n["o"]: TensorSpec((d, H * self.vd))}

    def load(self, weights):
        n = self.names
        parts = [weights[n[k]] for k in ("dq", "dkv", "g")]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        pad = torch.zeros((self.n_pad - self.n_in, self.d), dtype=dt, device=parts[0].device)
        self.w_in = torch.cat([p.to(dt) for p in parts] + [pad], dim=0).contiguous()
        lo = 0
        for k, p in zip(("dq", "dkv", "g"), parts):      # the stored names stay addressable as views
            weights[n[k]] = self.w_in[lo:lo + p.shape[0]]
            lo += p.shape[0]
        without = getattr(self, "without", frozenset())
        ops.for_few_rows(self.w_in, without=without)
        self.w_uq = ops.for_few_rows(weights[n["uq"]], without=without)
        self.w_o = ops.for_eight_rows(weights[n["o"]], without=without)
        # per head: W_uk,h^T as [kv_rank, head_dim] (a copy; the stored matrix stays under its name), W_uv,h as stored
        self.w_uk_t = weights[n["uk"]].reshape(self.H, self.D, self.rank).transpose(1, 2).contiguous()
        self.w_uv = weights[n["uv"]].reshape(self.H, self.vd, self.rank)
        self.q_norm = weights[n["dq_norm"]].float().contiguous()
        self.kv_norm = weights[n["dkv_norm"]].float().contiguous()
        if self.out_mult != 1.0:      # the constant rides in the output projection's epilogue as a factor per column
            self.out_scale = torch.full((self.d,), self.out_mult, dtype=torch.float32, device=self.w_in.device)

    def kv_need(self):
        return KVNeed(1, self.dk, None, values=False)

    def state_need(self):
        return None

    def forward(self, ctx, h, x, run, epilogue=ops.EPI_ADD):
        """``epilogue``: EPI_ADD adds the output into the residual rows ``x``; EPI_STORE writes it to ``x``, a float32
        buffer of the caller's."""
        if not run.writes_kv:
            raise ValueError("an attention over cached latents keeps latents of its own")
        if isinstance(h, ops.Normed):
            h = h.materialize()
        T, H, D, R, vd, rank, dk = h.shape[0], self.H, self.D, self.R, self.vd, self.rank, self.dk
        k_cache, _ = ctx.cache.layer_kv(run.kv_entry)
        table = ctx.block_table(ctx.cache.group_index(run.kv_entry))
        page = k_cache.shape[2]
        pos = self.position
        cos, sin = (pos.cos, pos.sin) if pos is not None else (None, None)
        mfma = "mfma" not in ops._off(ctx)
        # query latent, key/value latent with the shared key part, and the gate: one product, sums in 32-bit
        proj = ctx.buffer("latent_proj", (T, self.n_pad), torch.float32)
        ops.linear(h, self.w_in, proj, ops.EPI_STORE, ctx)
        cq = ctx.buffer("latent_cq", (T, self.q_rank), self.dtype)
        runs = ctx.buffer("latent_head_runs", (H + 1,), torch.int32)
        rows = ctx.buffer("latent_head_rows", (T * H,), torch.int32)
        K.latent_prep(proj, self.off_q, self.q_rank, self.off_kv, rank, R, self.q_norm, self.kv_norm, self.spec.norm_eps,
                      ctx.positions, ops._table_rows(ctx), table, cos, sin, cq, k_cache, page, H, runs, rows)
        q = ctx.buffer("latent_q", (T, H * (D + R)), self.dtype)
        ops.linear(cq, self.w_uq, q, ops.EPI_STORE, ctx)
        # every head's query as the cached rows take it: [W_uk^T q_unrotated | q_rotated turned | zeros]
        qa = ctx.buffer("latent_q_absorbed", (T, H * dk), self.dtype)
        K.expert_gemm(q.view(T * H, D + R)[:, :D], self.w_uk_t, qa.view(T * H, dk)[:, :rank], offsets=runs, pairs=rows,
                      mfma=mfma)
        K.latent_query(q, H, D, R, ctx.positions, cos, sin, qa, rank)
        att = ctx.buffer("latent_att", (T, H * rank), self.dtype)
        if (self.dtype == torch.bfloat16 and not ops._off(ctx) & {"attn_prefill", "attn_decode"}
                and K.latent_attention_fits(dk, rank, page)):
            splits = K.latent_splits(ctx.n_seqs, ctx.max_q_len, H, ctx.kv_len_hint)
            part_o = part_ml = None
            if splits > 1:
                part_o = ctx.buffer("latent_part_o", (T, H, splits, rank), torch.float32)
                part_ml = ctx.buffer("latent_part_ml", (T, H, splits, 2), torch.float32)
            K.latent_attention(qa, k_cache, ctx.cu_seqlens, ctx.kv_before, table, att, ctx.max_q_len, H, rank, self.spec.scale,
                               seq_rows=getattr(ctx, "seq_rows", None), n_splits=splits, part_o=part_o, part_ml=part_ml)
        else:       # (32-bit, or sizes that the matrix-core kernel is not built for)
            K.attention_generic(qa, k_cache, None, ctx.positions, ops._table_rows(ctx), table, att, H, 1, dk, page, None,
                                self.spec.scale, v_head_dim=rank, values_in_keys=0)
        o = ctx.buffer("latent_out", (T, H * vd), self.dtype)
        K.expert_gemm(att.view(T * H, rank), self.w_uv, o.view(T * H, vd), offsets=runs, pairs=rows, mfma=mfma)
        K.sigmoid_gate(o, proj, self.off_g)
        ops.linear(o, self.w_o, x, epilogue, ctx, col_scale=self.out_scale)


register_part("mixer", "latent_attention", LatentAttention)

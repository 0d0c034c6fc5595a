"""Causal grouped-query attention over the paged cache.

Order as the reference's layer (J/inference/InferenceCore.java:78-151): q, k, v
projections (one product over the three matrices stacked by rows), rotation of q
and k, cache write at the token's position, attention over positions lo..p of the
token's own sequence, output projection added into the residual stream. The reference's
projections have no biases; a description that names ``q_bias``, ``k_bias``, ``v_bias``
(together) or ``o_bias`` among its tensors gets them added in the products' epilogues.

What other decoders' descriptions may ask for besides: no rotation (``position`` None), values of another size than
the keys (``v_head_dim``), a bias on the scores that grows with the distance (``distance_bias``: a slope per head), a
sink in the softmax (``sink``), and a learned factor per channel on the output (``out_scale_name``), applied by the
output projection's epilogue; a window that keeps a sequence's first positions visible (``keep_first``); values that
are rotated by their own position before they are cached, with every head's output turned back by the query's
position (``value_position``); a gate per head (``head_gate`` among the names: sigmoid of one more row per head of the
stacked projection, multiplied into the head's output); a constant factor on the output (``out_mult``). The last three
run on kernels that take any head sizes: one product, one kernel that turns q, k and v in place, the cache write, the
attention, one kernel that turns the output back and applies the gate. On the same path: a norm on queries and keys per
head in front of the rotation (``qk_norm_eps``, in the kernel that turns them), a chunked mask (``chunk``), differential
attention (``differential``: two score maps per head over the same values; queries and keys then have twice the heads,
stored head by head as [map 1, map 2], and the cache keeps twice the key heads beside the value heads), and a mixer
without keys and values of its own (no ``k`` among its names) that only ever reads another entry's; a learned sink per
query head (a stored [n_heads] vector named ``sink``, on every kernel that knows a sink); and values that are the keys
as projected (``values_are_keys``: no value projection; the key rows stand twice in the stacked product, once to be
normed and turned, once to be cached as they are).
"""
from __future__ import annotations

import math

import torch

from ..cache import KVNeed
from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import build_part, register_part


class GQAAttention:
    graph_safe = True      # kernel launches on the current stream only, sizes fixed by (T, B)
    adds_only = True       # never reads the residual rows: sums of the product before it may still lie in slices

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype
        self.d, self.H, self.Kh, self.hs = spec.hidden, spec.n_heads, spec.n_kv_heads, spec.head_dim
        if self.H % self.Kh:
            raise ValueError(f"{self.H} heads are not a multiple of {self.Kh} kv heads")
        self.vd = spec.v_head_dim if getattr(spec, "v_head_dim", None) else self.hs
        # The cache keeps heads in tiles of 16 elements. Without a rotation a head of any other size is stored with
        # zero rows (q, k, v) and zero columns (o) up to the next multiple of 16: scores and outputs are the same
        # numbers, and every kernel sees the padded sizes.
        self.hs_stored, self.vd_stored = self.hs, self.vd
        self.value_position_spec = getattr(spec, "value_position", None)
        self.gated = "head_gate" in spec.names
        self.diff = getattr(spec, "differential", None)
        self.maps = 2 if self.diff is not None else 1
        self.Hq, self.Kq = self.H * self.maps, self.Kh * self.maps      # query and key heads as the kernels count them
        self.qk_norm_eps = getattr(spec, "qk_norm_eps", None)
        self.chunk = int(getattr(spec, "chunk", None) or 0) or None
        self.reads_only = "k" not in spec.names
        self.values_are_keys = bool(getattr(spec, "values_are_keys", False))
        if self.values_are_keys and (self.reads_only or self.vd != self.hs or "v" in spec.names):
            raise ValueError("an attention whose values are its keys has keys of its own, values of their size and no "
                             "value projection")
        if self.chunk and spec.window:
            raise ValueError("an attention has a window or a chunked mask, not both")
        # (rotated values, a gate per head, a rotation with values of another size, a norm on queries and keys, several
        # score maps and a mixer that only reads run on the kernels for any sizes)
        self.general = bool(self.value_position_spec is not None or self.gated
                            or (spec.position is not None and self.vd != self.hs) or self.qk_norm_eps is not None
                            or self.diff is not None or self.reads_only or self.values_are_keys)
        if spec.position is None or self.general:
            # (a rotation touches a head's first elements only: zeros behind them stay zeros)
            self.hs, self.vd = -(-self.hs // 16) * 16, -(-self.vd // 16) * 16
        self.window = spec.window
        self.keep_first = int(getattr(spec, "keep_first", 0) or 0) if spec.window else 0
        self.out_mult = float(getattr(spec, "out_mult", 1.0))
        self.sink = getattr(spec, "sink", None)
        self.sink_name = spec.names.get("sink")       # a stored sink per head takes the place of the constant
        bias = getattr(spec, "distance_bias", None)
        self._slopes_host = bias.slopes(self.H) if bias is not None else None
        self.slopes = None
        self.device = device
        self.out_scale_name = getattr(spec, "out_scale_name", None)
        self.out_scale = None
        self.scale = spec.scale if spec.scale is not None else 1.0 / math.sqrt(self.hs)
        self.position = build_part("position", spec.position, device=device) if spec.position is not None else None
        self.value_position = (build_part("position", self.value_position_spec, device=device)
                               if self.value_position_spec is not None else None)
        if self.value_position is not None and self.value_position.rot_dim > self.vd_stored:
            raise ValueError(f"values of {self.vd_stored} elements cannot be rotated over {self.value_position.rot_dim}")
        self.names = spec.names
        self.biased = "q_bias" in self.names
        if self.biased and not ("k_bias" in self.names and "v_bias" in self.names):
            raise ValueError("an attention names the biases of q, k and v together or none of them")
        self.w_qkv = self.w_q = self.w_o = self.b_qkv = self.b_o = None

    def tensors(self):
        n, d, hs, vd = self.names, self.d, self.hs_stored, self.vd_stored
        out = {n["q"]: TensorSpec((self.Hq * hs, d)), n["o"]: TensorSpec((d, self.H * vd))}
        if not self.reads_only:
            out[n["k"]] = TensorSpec((self.Kq * hs, d))
            if not self.values_are_keys:
                out[n["v"]] = TensorSpec((self.Kh * vd, d))
        if self.sink_name:
            out[self.sink_name] = TensorSpec((self.H,), "vector", 0.0, 1.0)
        if self.qk_norm_eps is not None:
            out[n["q_norm"]] = TensorSpec((hs,), "vector")
            if not self.reads_only:
                out[n["k_norm"]] = TensorSpec((hs,), "vector")
        if self.diff is not None:
            for k in ("lambda_q1", "lambda_k1", "lambda_q2", "lambda_k2"):
                out[n[k]] = TensorSpec((hs,), "vector", 0.0, 0.3)
        if self.biased:
            out.update({n["q_bias"]: TensorSpec((self.H * hs,), "vector", 0.0, 0.1),
                        n["k_bias"]: TensorSpec((self.Kh * hs,), "vector", 0.0, 0.1),
                        n["v_bias"]: TensorSpec((self.Kh * vd,), "vector", 0.0, 0.1)})
        if "o_bias" in n:
            out[n["o_bias"]] = TensorSpec((d,), "vector", 0.0, 0.1)
        if self.out_scale_name:
            out[self.out_scale_name] = TensorSpec((d,), "vector", 1.0, 0.1)
        if self.gated:
            out[n["head_gate"]] = TensorSpec((self.H, d))
        return out

    def load(self, weights):
        n = self.names
        if (self.hs, self.vd) != (self.hs_stored, self.vd_stored):
            weights = _PaddedHeads(weights, self)
        if self.general:
            return self._load_general(weights)
        parts = [weights[n["q"]], weights[n["k"]], weights[n["v"]]]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        self.w_qkv = torch.cat([p.to(dt) for p in parts], dim=0).contiguous()
        qn, kn, vn = self.H * self.hs, self.Kh * self.hs, self.Kh * self.vd
        # the stored names stay addressable as views of the stacked matrix
        weights[n["q"]], weights[n["k"]], weights[n["v"]] = (
            self.w_qkv[:qn], self.w_qkv[qn:qn + kn], self.w_qkv[qn + kn:])
        self.w_q = self.w_qkv[:qn]
        without = getattr(self, "without", frozenset())      # the fast paths that the engine does without
        # (the copy as the product that rotates and writes the cache in its epilogue reads it; biased projections
        # without a rotation, and values of another size, never take that product: a plain copy, which every product
        # of few rows reads)
        ops.for_few_rows(self.w_qkv, (self.H, self.Kh, self.hs, self.position is not None,
                                      bool(self.position is not None and self.position.adjacent))
                         if self.vd == self.hs and (self.position is not None or not self.biased) else None, without=without)
        self.w_o = ops.for_eight_rows(weights[n["o"]], without=without)
        if getattr(self, "may_hold_once", False):
            # the stored order is let go where a copy in the matrix cores' order can stand for the matrix; the stored
            # names then name rows that are put together on request
            if ops.can_hold_once(self.w_qkv, without):
                self.w_qkv, self.w_q = K.hold_once(self.w_qkv), None
                weights[n["q"]], weights[n["k"]], weights[n["v"]] = (
                    ops.StoredRows(self, "w_qkv", 0, qn), ops.StoredRows(self, "w_qkv", qn, qn + kn),
                    ops.StoredRows(self, "w_qkv", qn + kn, qn + kn + vn))
            if ops.can_hold_once(self.w_o, without):
                self.w_o = weights[n["o"]] = K.hold_once(self.w_o)
        if self.biased:     # the epilogues read biases as float
            self.b_qkv = torch.cat([weights[n[k]].float() for k in ("q_bias", "k_bias", "v_bias")]).contiguous()
        if "o_bias" in n:
            self.b_o = weights[n["o_bias"]].float().contiguous()
        self._load_scales(weights)
        if self._slopes_host is not None:
            self.slopes = torch.tensor(self._slopes_host, dtype=torch.float64).to(torch.float32).to(self.w_qkv.device)

    def _load_scales(self, weights):
        if self.sink_name:
            self.sink = weights[self.sink_name].float().contiguous()
        if self.out_scale_name:
            self.out_scale = weights[self.out_scale_name].float().contiguous()
        if self.out_mult != 1.0:      # the constant rides in the output projection's epilogue with the factor per channel
            dev = weights[self.names["o"]].device
            self.out_scale = (self.out_scale * self.out_mult if self.out_scale is not None
                              else torch.full((self.d,), self.out_mult, dtype=torch.float32, device=dev))

    def _load_general(self, weights):
        """q, k, v and the heads' gates stacked for one product (zero rows up to a multiple of 16), stored order."""
        n = self.names
        if self.biased or "o_bias" in n:
            raise ValueError("an attention with rotated values or a gate per head is built without biases")
        if self.reads_only and self.gated:
            raise ValueError("an attention without keys and values of its own is built without a gate per head")
        kinds = ("q",) if self.reads_only else ("q", "k", "k") if self.values_are_keys else ("q", "k", "v")
        parts = [weights[n[k]] for k in kinds] + ([weights[n["head_gate"]]] if self.gated else [])
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        rows = sum(p.shape[0] for p in parts)
        pad = torch.zeros((-(-rows // 16) * 16 - rows, self.d), dtype=dt, device=parts[0].device)
        self.w_qkv = torch.cat([p.to(dt) for p in parts] + [pad], dim=0).contiguous()
        lo = 0
        named = set()
        for k, p in zip(kinds + ("head_gate",), parts):      # the stored names stay addressable as views
            if k not in named:                                # (key rows that stand twice: the first ones)
                weights[n[k]] = self.w_qkv[lo:lo + p.shape[0]]
                named.add(k)
            lo += p.shape[0]
        without = getattr(self, "without", frozenset())
        ops.for_few_rows(self.w_qkv, without=without)
        self.w_q_rows = self.w_qkv[:self.Hq * self.hs]       # what an entry that reads another's keys and values multiplies
        self.w_o = ops.for_eight_rows(weights[n["o"]], without=without)
        self.q_norm_w = self.k_norm_w = None
        if self.qk_norm_eps is not None:      # (padded like the heads; the kernel reads them as float)
            def padded(w):
                out = torch.zeros(self.hs, dtype=torch.float32, device=w.device)
                out[:self.hs_stored] = w.float()
                return out
            self.q_norm_w = padded(weights[n["q_norm"]])
            self.k_norm_w = padded(weights[n["k_norm"]]) if not self.reads_only else None
        if self.diff is not None:
            lq1, lk1, lq2, lk2 = (weights[n[k]].float() for k in ("lambda_q1", "lambda_k1", "lambda_q2", "lambda_k2"))
            self.diff_lambda = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum())) + float(self.diff.offset)
        self._load_scales(weights)
        if self._slopes_host is not None:
            self.slopes = torch.tensor(self._slopes_host, dtype=torch.float64).to(torch.float32).to(self.w_qkv.device)

    def kv_need(self):
        return KVNeed(self.Kq, self.hs, self.window, v_head_dim=None if self.vd == self.hs else self.vd,
                      keep_first=self.keep_first, v_heads=None if self.maps == 1 else self.Kh, chunk=self.chunk)

    def state_need(self):
        return None

    def forward(self, ctx, h, x, run, epilogue=ops.EPI_ADD):
        """``epilogue``: EPI_ADD adds the output into the residual rows ``x``; EPI_STORE writes it to ``x``, a float32
        buffer of the caller's (a mixer that stands beside another)."""
        T, H, Kh, hs, vd = h.shape[0], self.H, self.Kh, self.hs, self.vd
        k_cache, v_cache = ctx.cache.layer_kv(run.kv_entry)
        table = ctx.block_table(ctx.cache.group_index(run.kv_entry))
        if self.general:
            return self._forward_general(ctx, h, x, run, epilogue, k_cache, v_cache, table)
        if vd == hs:
            q = ops.qkv_project(ctx, h, self.w_qkv, self.w_q, self.position, k_cache, v_cache, table, H, Kh, hs,
                                self.dtype, run.writes_kv, bias=self.b_qkv)
        else:
            q = self._project_unequal(ctx, h, k_cache, v_cache, table, run)
        att = ctx.buffer("attn_out", (T, H * vd), self.dtype)
        ops.attention(ctx, q, k_cache, v_cache, table, att, H, Kh, hs, self.window, self.scale, v_head_dim=vd,
                      slopes=self.slopes, sink=self.sink, keep_first=self.keep_first, chunk=self.chunk)
        ops.linear(att, self.w_o, x, epilogue, ctx, bias=self.b_o, col_scale=self.out_scale)

    def _forward_general(self, ctx, h, x, run, epilogue, k_cache, v_cache, table):
        writes = run.writes_kv
        if not writes and (self.value_position is not None or self.gated):
            raise ValueError("an attention with rotated values or a gate per head keeps keys and values of its own")
        if writes and self.reads_only:
            raise ValueError("an attention without keys and values of its own must read another entry's")
        T, H, Hq, Kq, Kh, hs, vd = h.shape[0], self.H, self.Hq, self.Kq, self.Kh, self.hs, self.vd
        qn, kn, vn = Hq * hs, Kq * hs, Kh * vd
        w = self.w_qkv if writes else self.w_q_rows
        qkv = ctx.buffer("qkvg", (T, w.shape[0]), self.dtype)
        ops.linear(h, w, qkv, ops.EPI_STORE, ctx)
        pos, vpos = self.position, self.value_position
        # q, k and v normed and turned in place, k and v into the cache as they come out: one kernel
        qk = (pos.rot_dim, pos.cos, pos.sin) if pos is not None else (0, None, None)
        vr = (vpos.rot_dim, vpos.cos, vpos.sin) if vpos is not None else (0, None, None)
        normed = self.qk_norm_eps is not None
        if writes:
            K.rotate_heads(qkv, ctx.positions, [(0, Hq, hs) + qk, (qn, Kq, hs) + qk, (qn + kn, Kh, vd) + vr],
                           adjacent=bool(pos.adjacent if pos is not None else vpos is not None and vpos.adjacent),
                           cache=(k_cache, v_cache, ops._table_rows(ctx), table, k_cache.shape[2]),
                           norms=[(self.q_norm_w, self.hs_stored), (self.k_norm_w, self.hs_stored), None] if normed else None,
                           norm_eps=self.qk_norm_eps or 0.0)
        elif pos is not None or normed:
            K.rotate_heads(qkv, ctx.positions, [(0, Hq, hs) + qk], adjacent=bool(pos is not None and pos.adjacent),
                           norms=[(self.q_norm_w, self.hs_stored)] if normed else None, norm_eps=self.qk_norm_eps or 0.0)
        att_dtype = self.dtype
        if self.diff is not None and ops.attention_kernel(ctx, self.dtype, k_cache.shape[2], Hq, Kq, hs, self.scale, vd) == "generic":
            att_dtype = torch.float32      # the maps' outputs stay in 32-bit up to their difference, where the kernel can write them so
        att = ctx.buffer("attn_out", (T, Hq * vd), att_dtype)
        ops.attention(ctx, qkv, k_cache, v_cache, table, att, Hq, Kq, hs, self.window, self.scale, v_head_dim=vd,
                      slopes=self.slopes, sink=self.sink, keep_first=self.keep_first, chunk=self.chunk,
                      n_v_heads=Kh if self.maps > 1 else None)
        if self.diff is not None:
            # the two maps' outputs of every head into one: a1 - lambda a2, a unit norm per head, the factor 1 - offset
            both, att = att, ctx.buffer("attn_maps_joined", (T, H * vd), self.dtype)      # (the activations' type again)
            K.diff_combine(both, att, H, vd, self.vd_stored, self.diff_lambda, self.diff.norm_eps, 1.0 - self.diff.offset)
        if vpos is not None or self.gated:
            # every head's output turned back by the query's position, then times the head's gate
            K.rotate_heads(att, ctx.positions,
                           [(0, H, vd, vpos.rot_dim if vpos is not None else 0, vpos.cos if vpos is not None else None,
                             vpos.sin if vpos is not None else None)],
                           adjacent=bool(vpos is not None and vpos.adjacent), back=True,
                           gate=qkv if self.gated else None, gate_col=qn + kn + vn)
        ops.linear(att, self.w_o, x, epilogue, ctx, col_scale=self.out_scale)

    def _project_unequal(self, ctx, h, k_cache, v_cache, table, run):
        """Values of another size than the keys: one product over the stacked rows, then keys and values into the
        cache as they are (such a description has no rotation)."""
        if self.position is not None or not run.writes_kv:
            raise ValueError("an attention whose values have another size than its keys is built without a rotation "
                             "and with keys and values of its own")
        T, qn, kn, vn = h.shape[0], self.H * self.hs, self.Kh * self.hs, self.Kh * self.vd
        qkv = ctx.buffer("qkv", (T, qn + kn + vn), self.dtype)
        ops.linear(h, self.w_qkv, qkv, bias=self.b_qkv)
        K.kv_write(qkv, qn, qn + kn, ctx.positions, ops._table_rows(ctx), table, k_cache, v_cache, self.Kh, self.hs,
                   self.vd, k_cache.shape[2])
        return qkv


class _PaddedHeads:
    """The weights of an attention whose heads are stored in other sizes than the cache's tiles take, as the part
    reads them: every head of q, k (rows), v (rows), their biases and o (columns) padded with zeros. What the part
    writes back (the stacked rows under the stored names) goes to the model's weights as it is: padded."""

    def __init__(self, weights, part):
        self.weights, self.part = weights, part

    def __getitem__(self, name):
        p, n, w = self.part, self.part.names, self.weights[name]
        heads = {n["q"]: (p.Hq, p.hs_stored, p.hs), n.get("k"): (p.Kq, p.hs_stored, p.hs), n.get("v"): (p.Kh, p.vd_stored, p.vd),
                 n.get("q_bias"): (p.Hq, p.hs_stored, p.hs), n.get("k_bias"): (p.Kq, p.hs_stored, p.hs),
                 n.get("v_bias"): (p.Kh, p.vd_stored, p.vd)}
        if name in heads and w.shape[0] == heads[name][0] * heads[name][1]:
            H, d_in, d_out = heads[name]
            out = torch.zeros((H, d_out) + tuple(w.shape[1:]), dtype=w.dtype, device=w.device)
            out[:, :d_in] = w.reshape((H, d_in) + tuple(w.shape[1:]))
            return out.reshape((H * d_out,) + tuple(w.shape[1:])).contiguous()
        if name == n["o"] and w.shape[1] == p.H * p.vd_stored:
            out = torch.zeros((w.shape[0], p.H, p.vd), dtype=w.dtype, device=w.device)
            out[:, :, :p.vd_stored] = w.reshape(w.shape[0], p.H, p.vd_stored)
            return out.reshape(w.shape[0], p.H * p.vd).contiguous()
        return w

    def __setitem__(self, name, value):
        self.weights[name] = value


register_part("mixer", "attention", GQAAttention)

"""Retention as a mixer: linear attention with a fixed decay per head, a matrix per head in place of keys and values.

Per head the sequence's state is a matrix S [key_dim, value_dim] in 32-bit::

    S <- decay_h S + (k key_dim^-1/2) v^T;   o = S^T q

q and k are projections of the input, rotated by the token's position like an attention's (before the factor on k);
there is no softmax and no denominator. Each head's read-out is divided by its root mean square, the heads together
are multiplied by silu of a gate projection, and the output projection follows.

One product makes q, k, v and the gate (rows stacked, padded with zero rows to a multiple of 16); its sums stay in
32-bit, and so does everything up to the output projection's input. The recurrence is ``lib.decay_scan``
(``csrc/scan.hip``), which the state space shares: it walks a step's tokens in order from the slot's state (a long
step as pieces side by side, joined through their start states), so every cut of a sequence into steps gives the same
result up to 32-bit rounding.

What other linear attentions of this form change, all from the description: the factor on k (``key_scale``), silu on q,
k and v behind their projections (``input_activation``, applied in 32-bit as the recurrence reads them), no rotation
(``position`` None), the unit norm over all heads' read-outs together with a stored weight (``norm_over = "all"``), and
the sigmoid of the gate projection in place of its silu (``gate_activation``).
"""
from __future__ import annotations

import torch

from ..cache import StateNeed
from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import build_part, register_part


class Retention:
    graph_safe = True      # kernel launches on the current stream only; the state is indexed with the step's slot numbers on the device
    adds_only = True       # never reads the residual rows

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype
        self.d, self.H, self.D, self.Dv = spec.hidden, spec.n_heads, spec.key_dim, spec.value_dim
        if len(spec.decay) != self.H:
            raise ValueError(f"{len(spec.decay)} decays for {self.H} heads")
        self.names = spec.names
        HD, HV = self.H * self.D, self.H * self.Dv
        self.off_q, self.off_k, self.off_v, self.off_g = 0, HD, 2 * HD, 2 * HD + HV
        self.n_in = 2 * HD + 2 * HV
        self.n_pad = -(-self.n_in // 16) * 16
        self.position = build_part("position", spec.position, device=device) if spec.position is not None else None
        self.out_mult = float(getattr(spec, "out_mult", 1.0))
        self.device = device
        key_scale = getattr(spec, "key_scale", None)
        self.key_scale = float(self.D) ** -0.5 if key_scale is None else float(key_scale)
        self.input_activation = getattr(spec, "input_activation", None)
        self.norm_over = getattr(spec, "norm_over", "head")
        self.gate_activation = getattr(spec, "gate_activation", "silu")
        if self.input_activation not in (None, "silu") or self.norm_over not in ("head", "all") \
                or self.gate_activation not in ("silu", "sigmoid"):
            raise ValueError(f"a retention with input activation {self.input_activation!r}, a norm over {self.norm_over!r} "
                             f"and a gate's {self.gate_activation!r} is not built")
        self.w_in = self.w_o = self.decay = self.out_scale = self.norm_weight = None

    def tensors(self):
        n, d, HD, HV = self.names, self.d, self.H * self.D, self.H * self.Dv
        out = {n["q"]: TensorSpec((HD, d)), n["k"]: TensorSpec((HD, d)), n["v"]: TensorSpec((HV, d)),
               n["g"]: TensorSpec((HV, d)), n["o"]: TensorSpec((d, HV))}
        if self.norm_over == "all":
            out[n["norm"]] = TensorSpec((HV,), "vector")
        return out

    def load(self, weights):
        n = self.names
        parts = [weights[n[k]] for k in ("q", "k", "v", "g")]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        pad = torch.zeros((self.n_pad - self.n_in, self.d), dtype=dt, device=parts[0].device)
        self.w_in = torch.cat([p.to(dt) for p in parts] + [pad], dim=0).contiguous()
        lo = 0
        for k, p in zip(("q", "k", "v", "g"), parts):      # the stored names stay addressable as views
            weights[n[k]] = self.w_in[lo:lo + p.shape[0]]
            lo += p.shape[0]
        without = getattr(self, "without", frozenset())
        ops.for_few_rows(self.w_in, without=without)
        self.w_o = ops.for_eight_rows(weights[n["o"]], without=without)
        dev = self.w_in.device
        self.decay = torch.tensor(self.spec.decay, dtype=torch.float64).to(torch.float32).to(dev)
        if self.out_mult != 1.0:      # the constant rides in the output projection's epilogue as a factor per column
            self.out_scale = torch.full((self.d,), self.out_mult, dtype=torch.float32, device=dev)
        if self.norm_over == "all":
            self.norm_weight = weights[n["norm"]].float().contiguous()

    def kv_need(self):
        return None

    def state_need(self):
        return StateNeed(self.H * self.D * self.Dv, torch.float32)

    def forward(self, ctx, h, x, run, epilogue=ops.EPI_ADD):
        if isinstance(h, ops.Normed):
            h = h.materialize()
        T, H, D, Dv = h.shape[0], self.H, self.D, self.Dv
        proj = ctx.buffer("retention_proj", (T, self.n_pad), torch.float32)
        ops.linear(h, self.w_in, proj, ops.EPI_STORE, ctx)
        pos = self.position
        if pos is not None:
            rot = (pos.rot_dim, pos.cos, pos.sin)
            K.rotate_heads(proj, ctx.positions, [(self.off_q, H, D) + rot, (self.off_k, H, D) + rot], adjacent=pos.adjacent)
        o = ctx.buffer("retention_readout", (T, H * Dv), torch.float32)
        K.decay_scan(proj, self.off_q, proj, self.off_k, proj, self.off_v, ctx.slot_state(run.entry), 0, ctx.cu_seqlens,
                     ctx.slot_ids, o, H, 1, D, Dv, a_head=self.decay, b_const=self.key_scale,
                     silu_inputs=self.input_activation == "silu", **ops.scan_pieces(ctx, H, D, Dv))
        y = ctx.buffer("retention_out", (T, H * Dv), self.dtype)
        K.group_norm_gate(o, proj, self.off_g, y, Dv if self.norm_over == "head" else H * Dv, self.spec.norm_eps,
                          weight=self.norm_weight, gate_act=self.gate_activation)
        ops.linear(y, self.w_o, x, epilogue, ctx, col_scale=self.out_scale)


register_part("mixer", "retention", Retention)

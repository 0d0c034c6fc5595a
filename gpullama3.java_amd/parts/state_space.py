"""A selective state space with a scalar decay per head and token (the Mamba-2 form) as a mixer.

One projection of the input gives ``[z | x | B | C | dt]``. x, B and C pass a causal convolution of a few taps per
channel (the sequence's last ``taps - 1`` inputs are part of its state) and silu. Per head h (group g of B and C)::

    dt = softplus(dt + dt_bias_h);   S <- exp(-exp(A_log_h) dt) S + dt B_g x_h^T;   y_h = S^T C_g + D_h x_h

with S [state_dim, head_dim] in 32-bit. y times silu(z) is divided by its root mean square in ``norm_groups`` equal
parts (the gate comes first), multiplied by a weight, and projected out.

The projection's sums stay in 32-bit, and so does everything behind it up to the output projection's input:
convolution, silu, softplus, both exponentials, the recurrence (``lib.decay_scan``, shared with the retention), the
gate and the norm. Every kernel walks a step's tokens in order from what the slot holds.
"""
from __future__ import annotations

import torch

from ..cache import StateNeed
from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import register_part


class StateSpace:
    graph_safe = True      # kernel launches on the current stream only; the state is indexed with the step's slot numbers on the device
    adds_only = True       # never reads the residual rows

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype
        self.d, self.H, self.P, self.G, self.N = spec.hidden, spec.n_heads, spec.head_dim, spec.n_groups, spec.state_dim
        self.taps, self.norm_groups = spec.conv_taps, spec.norm_groups
        if self.H % self.G:
            raise ValueError(f"{self.H} heads are not a multiple of {self.G} groups")
        self.inner = self.H * self.P
        if self.inner % self.norm_groups:
            raise ValueError(f"{self.norm_groups} parts do not divide the {self.inner} channels of the read-outs' norm")
        self.channels = self.inner + 2 * self.G * self.N
        # columns of the projection
        self.off_z, self.off_x = 0, self.inner
        self.off_dt = self.inner + self.channels
        self.n_in = self.off_dt + self.H
        self.n_pad = -(-self.n_in // 16) * 16
        self.conv_floats = (self.taps - 1) * self.channels
        self.conv_area = -(-self.conv_floats // 4) * 4          # the matrices behind it start at a multiple of 16 bytes
        self.names = spec.names
        self.out_mult = float(getattr(spec, "out_mult", 1.0))
        self.w_in = self.w_o = self.conv_w = self.conv_b = self.A_log = self.dt_bias = self.D = self.norm_w = self.out_scale = None

    def tensors(self):
        n, d, H = self.names, self.d, self.H
        return {n["in"]: TensorSpec((self.n_in, d)), n["conv"]: TensorSpec((self.channels, self.taps), "matrix", 0.0, 0.3),
                n["conv_bias"]: TensorSpec((self.channels,), "vector", 0.0, 0.1),
                n["dt_bias"]: TensorSpec((H,), "vector", 0.0, 0.5), n["A_log"]: TensorSpec((H,), "vector", 0.0, 0.5),
                n["D"]: TensorSpec((H,), "vector", 1.0, 0.2), n["norm"]: TensorSpec((self.inner,), "vector"),
                n["o"]: TensorSpec((d, self.inner))}

    def load(self, weights):
        n = self.names
        w = weights[n["in"]]
        if self.n_pad != self.n_in:      # zero rows up to a multiple of 16: the stored name stays a view
            pad = torch.zeros((self.n_pad - self.n_in, self.d), dtype=w.dtype, device=w.device)
            w = torch.cat([w, pad], dim=0).contiguous()
            weights[n["in"]] = w[:self.n_in]
        without = getattr(self, "without", frozenset())
        self.w_in = ops.for_few_rows(w, without=without)
        self.w_o = ops.for_eight_rows(weights[n["o"]], without=without)
        # what the recurrence's kernels read is kept in 32-bit
        self.conv_w = weights[n["conv"]].float().contiguous()
        self.conv_b = weights[n["conv_bias"]].float().contiguous()
        self.A_log = weights[n["A_log"]].float().contiguous()
        self.dt_bias = weights[n["dt_bias"]].float().contiguous()
        self.D = weights[n["D"]].float().contiguous()
        self.norm_w = weights[n["norm"]].float().contiguous()
        if self.out_mult != 1.0:
            self.out_scale = torch.full((self.d,), self.out_mult, dtype=torch.float32, device=self.w_o.device)

    def kv_need(self):
        return None

    def state_need(self):
        return StateNeed(self.conv_area + self.H * self.N * self.P, torch.float32)

    def forward(self, ctx, h, x, run, epilogue=ops.EPI_ADD):
        if isinstance(h, ops.Normed):
            h = h.materialize()
        T, H, P, G, N, inner = h.shape[0], self.H, self.P, self.G, self.N, self.inner
        state = ctx.slot_state(run.entry)
        proj = ctx.buffer("ssm_proj", (T, self.n_pad), torch.float32)
        ops.linear(h, self.w_in, proj, ops.EPI_STORE, ctx)
        act = ctx.buffer("ssm_act", (T, self.channels), torch.float32)          # [x | B | C] behind convolution and silu
        ab = ctx.buffer("ssm_decay_step", (T, 2 * H), torch.float32)
        K.ssm_prep(proj, self.off_x, self.channels, self.off_dt, H, self.conv_w, self.conv_b, self.A_log, self.dt_bias,
                   state, 0, ctx.cu_seqlens, ctx.seq_of_token, ctx.slot_ids, act, ab)
        o = ctx.buffer("ssm_readout", (T, inner), torch.float32)
        K.decay_scan(act, inner + G * N, act, inner, act, 0, state, self.conv_area, ctx.cu_seqlens, ctx.slot_ids, o,
                     H, H // G, N, P, a_tok=ab[:, :H], b_tok=ab[:, H:], **ops.scan_pieces(ctx, H, N, P))
        y = ctx.buffer("ssm_out", (T, inner), self.dtype)
        K.group_norm_gate(o, proj, self.off_z, y, inner // self.norm_groups, self.spec.norm_eps, weight=self.norm_w,
                          gate_first=True, skip=(act, 0, self.D, P))
        ops.linear(y, self.w_o, x, epilogue, ctx, col_scale=self.out_scale)


register_part("mixer", "state_space", StateSpace)

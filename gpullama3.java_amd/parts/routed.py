"""A mixture of experts as a feed-forward: ``sum over a token's experts of weight * down_e(act(up_e h))``, plus an
expert that every token passes.

The router's logits are a product with 32-bit sums kept in 32-bit; the ``top`` largest choose a token's experts (the
lower number wins a tie) and their weights are the softmax over the chosen logits alone (``lib.route``). The (token,
choice) pairs are ordered by expert on the device, and two grouped products (``lib.expert_gemm``: every tile of rows
belongs to one expert) make the experts' hidden rows and their outputs; the weighted sum runs over a token's pairs
in the order of its choices. A pair's numbers depend on its token and expert alone, so a token's output does not
depend on its batch-mates; no expert has a capacity, no token is dropped. Nothing waits for the host: the launches'
shapes follow from the step's number of tokens, so decode steps can be captured. A shared expert with the experts' own
sizes and activation is stacked behind them as expert number E, and every token gets one more pair for it with weight
1: its products and its part of the sum ride in the experts' launches. One of another form has two products of its own.
"""
from __future__ import annotations

import torch

from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import register_part


class RoutedFeedForward:
    graph_safe = True      # kernel launches on the current stream only, sizes fixed by the step's tokens
    adds_only = True       # never reads the residual rows

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype
        self.d, self.E, self.top, self.names = spec.hidden, spec.n_experts, spec.top, spec.names
        self.F, self.act = spec.expert.intermediate, spec.expert.activation
        self.shared = spec.shared
        if not 1 <= self.top <= self.E:
            raise ValueError(f"the {self.top} largest of {self.E} experts")
        for e in (spec.expert, spec.shared):
            if e is not None and e.activation not in K.EXPERT_ACTIVATIONS:
                raise ValueError(f"activation {e.activation!r} is not built ({sorted(k for k in K.EXPERT_ACTIVATIONS if k)})")
        self.out_mult = float(getattr(spec, "out_mult", 1.0))
        self.w_router = self.w_up = self.w_down = self.s_up = self.s_down = None
        self.merged = False

    def _expert_names(self, e):
        return self.names["expert_up"].format(e=e), self.names["expert_down"].format(e=e)

    def tensors(self):
        out = {self.names["router"]: TensorSpec((self.E, self.d), "matrix", 0.0, 1.0)}
        for e in range(self.E):
            up, down = self._expert_names(e)
            out[up], out[down] = TensorSpec((self.F, self.d)), TensorSpec((self.d, self.F))
        if self.shared is not None:
            out[self.names["shared_up"]] = TensorSpec((self.shared.intermediate, self.d))
            out[self.names["shared_down"]] = TensorSpec((self.d, self.shared.intermediate))
        return out

    def load(self, weights):
        ups, downs = zip(*[[weights[n] for n in self._expert_names(e)] for e in range(self.E)])
        ups, downs = list(ups), list(downs)
        # a shared expert of the experts' own form rides with them as expert number E that every token passes: its
        # products are part of the experts' launches
        self.merged = (self.shared is not None and self.shared.intermediate == self.F and self.shared.activation == self.act
                       and self.top < K.ROUTE_MAX_TOP and self.E < K.ROUTE_MAX_EXPERTS)
        if self.merged:
            ups.append(weights[self.names["shared_up"]])
            downs.append(weights[self.names["shared_down"]])
        # one array per kind, expert after expert; the stored names stay addressable as views
        self.w_up = torch.stack(ups).contiguous()
        self.w_down = torch.stack(downs).contiguous()
        for e in range(self.E):
            up, down = self._expert_names(e)
            weights[up], weights[down] = self.w_up[e], self.w_down[e]
        self.w_router = weights[self.names["router"]]
        if self.merged:
            weights[self.names["shared_up"]], weights[self.names["shared_down"]] = self.w_up[self.E], self.w_down[self.E]
        elif self.shared is not None:
            self.s_up = weights[self.names["shared_up"]].contiguous().unsqueeze(0)
            self.s_down = weights[self.names["shared_down"]].contiguous().unsqueeze(0)

    def forward(self, ctx, h, x, epilogue=ops.EPI_ADD):
        """``epilogue``: EPI_ADD adds the output into the residual rows ``x``; EPI_STORE writes it to ``x``, a float32
        buffer of the caller's."""
        if isinstance(h, ops.Normed):
            h = h.materialize()
        T, d, E, top, F = h.shape[0], self.d, self.E, self.top, self.F
        more = 1 if self.merged else 0            # pairs a token beyond its choices
        per = top + more
        mfma = "mfma" not in ops._off(ctx)
        logits = ctx.buffer("router_logits", (T, E), torch.float32)
        ops.linear(h, self.w_router, logits, ops.EPI_STORE, ctx)
        idx = ctx.buffer("router_choice", (T, per), torch.int32)
        wts = ctx.buffer("router_weights", (T, per), torch.float32)
        offsets = ctx.buffer("router_runs", (E + more + 1,), torch.int32)
        pairs = ctx.buffer("router_pairs", (T * per,), torch.int32)
        K.route(logits, top, idx, wts, offsets, pairs, always=self.merged)
        hidden = ctx.buffer("experts_hidden", (T * per, F), self.dtype)
        K.expert_gemm(h, self.w_up, hidden, act=self.act, offsets=offsets, pairs=pairs, a_div=per, mfma=mfma)
        outs = ctx.buffer("experts_out", (T * per, d), torch.float32)
        K.expert_gemm(hidden, self.w_down, outs, offsets=offsets, pairs=pairs, mfma=mfma)
        if epilogue == ops.EPI_ADD:
            ops.settle_residual(ctx, x)
        first = epilogue == ops.EPI_STORE          # whether x still has to be written rather than added to
        if self.shared is not None and not self.merged:
            s_hidden = ctx.buffer("shared_hidden", (T, self.shared.intermediate), self.dtype)
            K.expert_gemm(h, self.s_up, s_hidden, act=self.shared.activation, mfma=mfma)
            if first:
                K.expert_gemm(s_hidden, self.s_down, x, mfma=mfma)
                first = False
            else:
                ops.linear(s_hidden, self.s_down[0], x, ops.EPI_ADD, ctx)
                ops.settle_residual(ctx, x)
        if self.out_mult != 1.0:
            raise NotImplementedError("a factor on a routed feed-forward's output is not built")
        K.route_combine(outs, wts, x, accumulate=not first)
        ops.residual_written(ctx, x)


register_part("ffn", "routed", RoutedFeedForward)

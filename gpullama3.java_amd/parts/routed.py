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

What a description may change: gated experts (``ExpertSpec.gated``: gate and up rows are stacked in turns, so the
grouped product's epilogue finds a gate value and its up value in neighbouring lanes and writes
``act(min(gate, limit)) * (clamp(up) + shift)`` directly); the other rule for choice and weights (``weights =
"scores"``: a softmax over all router outputs, the choice by score plus a stored correction, the weights from the
chosen scores over their sum); and identity experts (``n_identity``: the router's last outputs; such a pair has no
product, and the weighted sum takes the token's input row for it).
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
        self.I = int(getattr(spec, "n_identity", 0) or 0)       # identity experts: the router's last outputs
        self.scores = getattr(spec, "weights", "chosen_softmax") == "scores"
        if getattr(spec, "weights", "chosen_softmax") not in ("chosen_softmax", "scores"):
            raise ValueError(f"the rule {spec.weights!r} for an expert's weight is not built (chosen_softmax, scores)")
        self.sum_eps = float(getattr(spec, "sum_eps", 0.0))
        if not 1 <= self.top <= self.E + self.I:
            raise ValueError(f"the {self.top} largest of {self.E + self.I} experts")
        for e in (spec.expert, spec.shared):
            known = K.ACTIVATIONS if e is not None and getattr(e, "gated", False) else K.EXPERT_ACTIVATIONS
            if e is not None and e.activation not in known:
                raise ValueError(f"activation {e.activation!r} is not built ({sorted(k for k in known if k)})")
        self.out_mult = float(getattr(spec, "out_mult", 1.0))
        self.w_router = self.w_up = self.w_down = self.s_up = self.s_down = self.correction = None
        self.merged = False

    @staticmethod
    def _rule(e):
        """How ``lib.expert_gemm`` is told an expert's form: ``(act, gated)``."""
        if getattr(e, "gated", False):
            return None, (e.activation, e.limit, float(e.up_shift))
        return e.activation, None

    def _expert_names(self, e):
        return self.names["expert_up"].format(e=e), self.names["expert_down"].format(e=e)

    def tensors(self):
        out = {self.names["router"]: TensorSpec((self.E + self.I, self.d), "matrix", 0.0, 1.0)}
        if "correction" in self.names:
            out[self.names["correction"]] = TensorSpec((self.E + self.I,), "vector", 0.0, 0.02)
        for e in range(self.E):
            up, down = self._expert_names(e)
            out[up], out[down] = TensorSpec((self.F, self.d)), TensorSpec((self.d, self.F))
            if self.spec.expert.gated:
                out[self.names["expert_gate"].format(e=e)] = TensorSpec((self.F, self.d))
        if self.shared is not None:
            out[self.names["shared_up"]] = TensorSpec((self.shared.intermediate, self.d))
            out[self.names["shared_down"]] = TensorSpec((self.d, self.shared.intermediate))
            if self.shared.gated:
                out[self.names["shared_gate"]] = TensorSpec((self.shared.intermediate, self.d))
        return out

    @staticmethod
    def _in_turns(gate, up):
        """Gate and up rows stacked in turns: row 2n the gate's row n, row 2n + 1 the up's."""
        return torch.stack([gate, up], dim=1).reshape(2 * gate.shape[0], gate.shape[1])

    def load(self, weights):
        ups, downs = zip(*[[weights[n] for n in self._expert_names(e)] for e in range(self.E)])
        ups, downs = list(ups), list(downs)
        gated = bool(self.spec.expert.gated)
        if gated:
            ups = [self._in_turns(weights[self.names["expert_gate"].format(e=e)], ups[e]) for e in range(self.E)]
        # a shared expert of the experts' own form rides with them as expert number E that every token passes: its
        # products are part of the experts' launches
        self.merged = (self.shared is not None and self.shared == self.spec.expert and self.I == 0
                       and self.top < K.ROUTE_MAX_TOP and self.E < K.ROUTE_MAX_EXPERTS)
        if self.merged:
            s_up = weights[self.names["shared_up"]]
            ups.append(self._in_turns(weights[self.names["shared_gate"]], s_up) if gated else s_up)
            downs.append(weights[self.names["shared_down"]])
        # one array per kind, expert after expert; the stored names stay addressable as views
        self.w_up = torch.stack(ups).contiguous()
        self.w_down = torch.stack(downs).contiguous()

        def name_up(e, up_name, gate_name):
            if gated:
                weights[gate_name], weights[up_name] = self.w_up[e, 0::2], self.w_up[e, 1::2]
            else:
                weights[up_name] = self.w_up[e]

        for e in range(self.E):
            up, down = self._expert_names(e)
            name_up(e, up, self.names["expert_gate"].format(e=e) if gated else None)
            weights[down] = self.w_down[e]
        self.w_router = weights[self.names["router"]]
        if "correction" in self.names:
            self.correction = weights[self.names["correction"]].float().contiguous()
        if self.merged:
            name_up(self.E, self.names["shared_up"], self.names.get("shared_gate"))
            weights[self.names["shared_down"]] = self.w_down[self.E]
        elif self.shared is not None:
            s_up = weights[self.names["shared_up"]]
            if self.shared.gated:
                self.s_up = self._in_turns(weights[self.names["shared_gate"]], s_up).contiguous().unsqueeze(0)
                weights[self.names["shared_gate"]], weights[self.names["shared_up"]] = self.s_up[0, 0::2], self.s_up[0, 1::2]
            else:
                self.s_up = s_up.contiguous().unsqueeze(0)
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
        routed = E + self.I                       # the router's outputs: the experts, then the identity experts
        logits = ctx.buffer("router_logits", (T, routed), torch.float32)
        ops.linear(h, self.w_router, logits, ops.EPI_STORE, ctx)
        idx = ctx.buffer("router_choice", (T, per), torch.int32)
        wts = ctx.buffer("router_weights", (T, per), torch.float32)
        offsets = ctx.buffer("router_runs", (routed + more + 1,), torch.int32)
        pairs = ctx.buffer("router_pairs", (T * per,), torch.int32)
        K.route(logits, top, idx, wts, offsets, pairs, always=self.merged, scores=self.scores,
                correction=self.correction, sum_eps=self.sum_eps)
        act, gated = self._rule(self.spec.expert)
        hidden = ctx.buffer("experts_hidden", (T * per, F), self.dtype)
        # (the runs of identity experts lie behind the experts': the products leave their pairs alone)
        K.expert_gemm(h, self.w_up, hidden, act=act, gated=gated, offsets=offsets, pairs=pairs, a_div=per, mfma=mfma)
        outs = ctx.buffer("experts_out", (T * per, d), torch.float32)
        K.expert_gemm(hidden, self.w_down, outs, offsets=offsets, pairs=pairs, mfma=mfma)
        if epilogue == ops.EPI_ADD:
            ops.settle_residual(ctx, x)
        first = epilogue == ops.EPI_STORE          # whether x still has to be written rather than added to
        if self.shared is not None and not self.merged:
            s_hidden = ctx.buffer("shared_hidden", (T, self.shared.intermediate), self.dtype)
            s_act, s_gated = self._rule(self.shared)
            K.expert_gemm(h, self.s_up, s_hidden, act=s_act, gated=s_gated, mfma=mfma)
            if first:
                K.expert_gemm(s_hidden, self.s_down, x, mfma=mfma)
                first = False
            else:
                ops.linear(s_hidden, self.s_down[0], x, ops.EPI_ADD, ctx)
                ops.settle_residual(ctx, x)
        if self.out_mult != 1.0:
            raise NotImplementedError("a factor on a routed feed-forward's output is not built")
        K.route_combine(outs, wts, x, accumulate=not first, identity=(idx, E, h) if self.I else None)
        ops.residual_written(ctx, x)


register_part("ffn", "routed", RoutedFeedForward)

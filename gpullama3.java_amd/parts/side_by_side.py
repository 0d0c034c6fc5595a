"""Two mixers side by side: both read the same normalised input, each one's output is normalised over the model width
with a weight of its own, and ``weight`` times the sum of the two (1/2: their average) is the mixer's output.

Either side is any registered mixer whose ``forward`` takes ``epilogue=ops.EPI_STORE`` (its output then goes to a
float32 buffer instead of into the residual rows). A description with ``normalised=False`` asks for the plain sum of
the two outputs instead (each side carries its own factor as its ``out_mult``): no norms, no weights; the second
side's output projection then adds to what the first one's wrote. Keys and values are the one side's that asks for them; states of
both sides share the run-order entry's state area, the left side's first.
"""
from __future__ import annotations

import torch

from ..cache import StateNeed
from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import build_part, register_part


class _Shifted:
    """A step context whose per-slot state is a side's own columns of the entry's state area."""

    def __init__(self, ctx, lo, hi):
        self.__dict__["_ctx"], self.__dict__["_lo"], self.__dict__["_hi"] = ctx, lo, hi

    def __getattr__(self, name):
        return getattr(self._ctx, name)

    def __setattr__(self, name, value):
        setattr(self._ctx, name, value)

    def slot_state(self, entry):
        return self._ctx.slot_state(entry)[:, self._lo:self._hi]


class SideBySide:
    adds_only = True       # never reads the residual rows

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype
        self.d, self.names = spec.hidden, spec.names
        self.left = build_part("mixer", spec.left, dtype=dtype, device=device)
        self.right = build_part("mixer", spec.right, dtype=dtype, device=device)
        self.factor = float(spec.weight) * float(getattr(spec, "out_mult", 1.0))
        self.normalised = bool(getattr(spec, "normalised", True))
        if not self.normalised and self.factor != 1.0:
            raise ValueError("two mixers side by side without norms carry their factors themselves (out_mult of each side)")
        self.w_left = self.w_right = None
        needs = [s.state_need() for s in (self.left, self.right)]
        if any(n is not None and n.dtype != torch.float32 for n in needs):
            raise ValueError("mixers side by side keep their states in 32-bit floats")
        self.state_sizes = [0 if n is None else -(-n.elements // 4) * 4 for n in needs]
        if sum(1 for s in (self.left, self.right) if s.kv_need() is not None) > 1:
            raise ValueError("of two mixers side by side at most one keeps keys and values")

    @property
    def graph_safe(self):
        return bool(getattr(self.left, "graph_safe", False) and getattr(self.right, "graph_safe", False))

    def tensors(self):
        out = ({self.names["left_norm"]: TensorSpec((self.d,), "vector"), self.names["right_norm"]: TensorSpec((self.d,), "vector")}
               if self.normalised else {})
        out.update(self.left.tensors())
        out.update(self.right.tensors())
        return out

    def load(self, weights):
        for side in (self.left, self.right):
            side.without = getattr(self, "without", frozenset())
            side.may_hold_once = getattr(self, "may_hold_once", False)
            side.load(weights)
        if self.normalised:
            self.w_left = weights[self.names["left_norm"]].float().contiguous()
            self.w_right = weights[self.names["right_norm"]].float().contiguous()

    def kv_need(self):
        return self.left.kv_need() or self.right.kv_need()

    def state_need(self):
        n = sum(self.state_sizes)
        return StateNeed(n, torch.float32) if n else None

    def _forward_sum(self, ctx, h, x, run, epilogue):
        """The plain sum: the left side's output projection writes (or adds into) ``x``, the right side's adds to it.
        No product leaves its sums in slices meanwhile: ``x`` may be a buffer that no norm adds them up for."""
        next_norm, ctx.next_norm = ctx.next_norm, None
        fuse, ctx.fuse = getattr(ctx, "fuse", False), False
        try:
            lo = 0
            for side, size, epi in ((self.left, self.state_sizes[0], epilogue), (self.right, self.state_sizes[1], ops.EPI_ADD)):
                side.forward(_Shifted(ctx, lo, lo + size) if size else ctx, h, x, run, epilogue=epi)
                lo += size
        finally:
            ctx.fuse, ctx.next_norm = fuse, next_norm
        ops.residual_written(ctx, x)

    def forward(self, ctx, h, x, run, epilogue=ops.EPI_ADD):
        if isinstance(h, ops.Normed):
            h = h.materialize()
        if not self.normalised:
            if epilogue == ops.EPI_ADD:
                ops.settle_residual(ctx, x)
            return self._forward_sum(ctx, h, x, run, epilogue)
        if epilogue != ops.EPI_ADD:
            raise ValueError("two normalised mixers side by side add into the residual rows")
        T = h.shape[0]
        next_norm, ctx.next_norm = ctx.next_norm, None      # neither side completes the residual rows
        outs, lo = [], 0
        for name, side, size in (("left", self.left, self.state_sizes[0]), ("right", self.right, self.state_sizes[1])):
            out = ctx.buffer(f"side_{name}", (T, self.d), torch.float32)
            side.forward(_Shifted(ctx, lo, lo + size) if size else ctx, h, out, run, epilogue=ops.EPI_STORE)
            outs.append(out)
            lo += size
        ctx.next_norm = next_norm
        ops.settle_residual(ctx, x)
        if (getattr(ctx, "fuse", False) and T == ctx.n_tokens <= ops.FUSE_ROWS and "fused" not in ops._off(ctx)
                and self.d % 16 == 0):
            # the rows are complete after this kernel: it leaves what the norm that follows would use (the rows' sums of
            # squares, and the rows times that norm's weight), so that the next product can take the norm over
            norm, xg = ops._next_norm(ctx, self.d)
            if norm is not None:
                ssq = ctx.ssq_buffer(1)
                K.sides_norm_add(x, outs[0], outs[1], self.w_left, self.w_right, self.spec.norm_eps, self.factor,
                                 ssq, norm.weight_f32, xg)
                return ops.residual_written(ctx, x, ssq, 1, xg, norm)
        K.sides_norm_add(x, outs[0], outs[1], self.w_left, self.w_right, self.spec.norm_eps, self.factor)
        ops.residual_written(ctx, x)


register_part("mixer", "side_by_side", SideBySide)

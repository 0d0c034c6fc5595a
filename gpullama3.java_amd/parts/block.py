"""A layer: the arrangement of norm, mixer and feed-forward.

``prenorm`` is the reference's: the normalised copy feeds the mixer, the residual
stream keeps the sum (J/inference/InferenceCore.java:74, :151, :154, :172).
"""
from __future__ import annotations

from ..csrc import lib as K
from . import ops
from .base import build_part, register_part


class PreNormBlock:
    def __init__(self, spec, dtype, device):
        self.mixer_norm = build_part("norm", spec.mixer_norm, dtype=dtype)
        self.mixer = build_part("mixer", spec.mixer, dtype=dtype, device=device)
        self.ffn_norm = build_part("norm", spec.ffn_norm, dtype=dtype) if spec.ffn is not None else None
        self.ffn = build_part("ffn", spec.ffn, dtype=dtype, device=device) if spec.ffn is not None else None

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def cache_needs(self):
        return self.mixer.kv_need(), self.mixer.state_need()

    def first_norm(self):
        """The norm that reads the residual rows first: the block before this one may prepare its rows."""
        return self.mixer_norm

    def forward(self, ctx, x, run, norm_after=None):
        """``norm_after``: the norm that reads the residual rows after this block, if known."""
        h = self._whole_rows_for(self.mixer_norm, "takes_slices", ctx, x)(ctx, x)
        ctx.next_norm = self.ffn_norm if self.ffn is not None else norm_after
        self._whole_rows_for(self.mixer, "adds_only", ctx, x).forward(ctx, h, x, run)
        if self.ffn is not None:
            h = self._whole_rows_for(self.ffn_norm, "takes_slices", ctx, x)(ctx, x)
            ctx.next_norm = norm_after
            self._whole_rows_for(self.ffn, "adds_only", ctx, x).forward(ctx, h, x)
        ctx.next_norm = None

    @staticmethod
    def _whole_rows_for(part, declares, ctx, x):
        """A product of 17 or more rows may have left its sums in slices beside the residual rows. A norm
        that adds them up itself says so (``takes_slices``), a mixer or feed-forward that only adds to the rows
        says that (``adds_only``); for any other part the rows are made whole before it runs, so a part that
        knows nothing of slices reads what it expects."""
        if not getattr(part, declares, False):
            ops.settle_residual(ctx, x)
        return part


class ParallelBlock:
    """One norm whose output feeds both the mixer and the feed-forward; both add into the residual rows:
    ``h = norm(x); x += mixer(h) + ffn(h)``. The rows are complete after the later of the two, so only that one may
    leave what the norm that reads them next would use."""

    def __init__(self, spec, dtype, device):
        if spec.ffn_norm is not None:
            raise ValueError("a parallel block has one norm: its description names no norm for the feed-forward")
        self.norm = build_part("norm", spec.mixer_norm, dtype=dtype)
        self.mixer = build_part("mixer", spec.mixer, dtype=dtype, device=device)
        self.ffn = build_part("ffn", spec.ffn, dtype=dtype, device=device) if spec.ffn is not None else None

    def parts(self):
        return [p for p in (self.norm, self.mixer, self.ffn) if p is not None]

    def cache_needs(self):
        return self.mixer.kv_need(), self.mixer.state_need()

    def first_norm(self):
        return self.norm

    def forward(self, ctx, x, run, norm_after=None):
        h = PreNormBlock._whole_rows_for(self.norm, "takes_slices", ctx, x)(ctx, x)
        if self.ffn is not None and isinstance(h, ops.Normed) and not getattr(self.ffn, "folds_norm", lambda h: False)(h):
            # a norm that a product was to take over is worked out from the rows when somebody asks for it; a
            # feed-forward whose first product does not take it over would ask after the mixer has added to them,
            # so it is worked out now
            h = h.materialize()
        # (both sublayers read h, and a product of the first must not prepare rows that are not whole yet)
        ctx.next_norm = None if self.ffn is not None else norm_after
        PreNormBlock._whole_rows_for(self.mixer, "adds_only", ctx, x).forward(ctx, h, x, run)
        if self.ffn is not None:
            ctx.next_norm = norm_after
            PreNormBlock._whole_rows_for(self.ffn, "adds_only", ctx, x).forward(ctx, h, x)
        ctx.next_norm = None


class OutNormBlock:
    """The norms stand behind the sublayers: ``x += norm1(mixer(x)); x += norm2(ffn(x))``. Mixer and feed-forward
    read the residual rows themselves (in a bfloat16 engine their rounding to bfloat16, which the kernel that last
    wrote the rows leaves beside them) and write their output to a 32-bit buffer (``epilogue=EPI_STORE``); the norm's
    kernel adds the normalised output into the rows. The block has no ``first_norm``: the decoder hands it whole
    rows and folds no norm into a product while it runs. The copy that the last norm kernel left stays valid for the
    next block of this kind (``keeps_rows_copy``: the decoder forgets it before anything else touches the rows)."""
    keeps_rows_copy = True

    def __init__(self, spec, dtype, device):
        self.dtype = dtype
        self.mixer_norm = build_part("norm", spec.mixer_norm, dtype=dtype)
        self.mixer = build_part("mixer", spec.mixer, dtype=dtype, device=device)
        self.ffn_norm = build_part("norm", spec.ffn_norm, dtype=dtype) if spec.ffn is not None else None
        self.ffn = build_part("ffn", spec.ffn, dtype=dtype, device=device) if spec.ffn is not None else None
        for n in (self.mixer_norm, self.ffn_norm):
            if n is not None and not hasattr(n, "add_into"):
                raise ValueError(f"a norm behind a sublayer must offer add_into; {type(n).__name__} does not")

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def cache_needs(self):
        return self.mixer.kv_need(), self.mixer.state_need()

    def _input(self, ctx, x):
        """What a sublayer reads: the rows themselves in a 32-bit engine, else their copy in the activations' type
        (left by the norm kernel that last wrote the rows, or made here)."""
        if self.dtype == x.dtype:
            return x
        h = ctx.buffer("rows_as_input", tuple(x.shape), self.dtype)
        made = getattr(ctx, "rows_as_input", None)
        if made != x.data_ptr():
            K.cast_rows(x, h)
        return h

    def forward(self, ctx, x, run):
        T, d = x.shape
        cast = ctx.buffer("rows_as_input", (T, d), self.dtype) if self.dtype != x.dtype else None
        y = ctx.buffer("sublayer_out", (T, d), x.dtype)
        self.mixer.forward(ctx, self._input(ctx, x), y, run, epilogue=ops.EPI_STORE)
        watch = getattr(ctx.engine, "after_sublayer", None)      # a caller that looks at a sublayer's output and at the rows behind it
        if watch is not None:
            watch(run.entry, "mixer", y)
        self.mixer_norm.add_into(ctx, x, y, cast)
        if watch is not None:
            watch(run.entry, "mixer_added", x)
        ctx.rows_as_input = x.data_ptr() if cast is not None else None
        if self.ffn is not None:
            self.ffn.forward(ctx, self._input(ctx, x), y, epilogue=ops.EPI_STORE)
            if watch is not None:
                watch(run.entry, "ffn", y)
            self.ffn_norm.add_into(ctx, x, y, cast)


register_part("block", "prenorm", PreNormBlock)
register_part("block", "outnorm", OutNormBlock)
register_part("block", "parallel", ParallelBlock)

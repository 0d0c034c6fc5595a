"""A layer: the arrangement of norm, mixer and feed-forward.

``prenorm`` is the reference's: the normalised copy feeds the mixer, the residual
stream keeps the sum (J/inference/InferenceCore.java:74, :151, :154, :172).
"""
from __future__ import annotations

import torch

from ..csrc import lib as K
from ..weights.loader import TensorSpec
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


class _StreamNumbers:
    """The numbers that mix the copies of the residual row around one block's sublayers: per sublayer ``in`` [S],
    ``mix`` [S, S] (from, to) and ``out`` [S], kept in 32-bit."""
    graph_safe = True

    def __init__(self, S, names):
        self.S, self.names = S, names
        self.values = {}

    def tensors(self):
        shapes = {"in": (self.S,), "mix": (self.S, self.S), "out": (self.S,)}
        # (random weights: around 1 / S for what is read, around the identity for what is kept)
        out = {}
        for key, name in self.names.items():
            kind = key.split("_")[1]
            out[name] = TensorSpec(shapes[kind], "vector", {"in": 1.0 / self.S, "mix": 1.0 / self.S, "out": 1.0}[kind], 0.2)
        return out

    def load(self, weights):
        self.values = {key: weights[name].float().contiguous() for key, name in self.names.items()}

    def of(self, sublayer):
        return tuple(self.values[f"{sublayer}_{k}"] for k in ("in", "mix", "out"))


class StreamsBlock:
    """Every token has S copies of its residual row, ``x`` [T, S d]. A sublayer reads ``norm(sum_s in[s] x_s)`` and
    its output y goes back as ``x_r <- sum_s mix[s, r] x_s + out[r] y``. One kernel (``lib.streams_step``) does the
    write-back of one sublayer and the read of the next; the block's first read is its own launch (the block before
    ends with its write-back: a block may be run more than once, or in another order, so nothing is carried across
    blocks). Mixer and feed-forward write their output to a 32-bit buffer (``epilogue=EPI_STORE``). The block has no
    ``first_norm``: the decoder hands it whole rows and folds no norm into a product while it runs."""

    def __init__(self, spec, dtype, device):
        self.dtype, self.S = dtype, int(spec.streams)
        self.mixer_norm = build_part("norm", spec.mixer_norm, dtype=dtype)
        self.mixer = build_part("mixer", spec.mixer, dtype=dtype, device=device)
        self.ffn_norm = build_part("norm", spec.ffn_norm, dtype=dtype) if spec.ffn is not None else None
        self.ffn = build_part("ffn", spec.ffn, dtype=dtype, device=device) if spec.ffn is not None else None
        for n in (self.mixer_norm, self.ffn_norm):
            if n is not None and not getattr(n, "folds", False):
                raise ValueError(f"the norm in front of a sublayer that reads several copies is weight * x / rms; "
                                 f"{type(n).__name__} is not")
        self.numbers = _StreamNumbers(self.S, spec.stream_names)

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, self.numbers) if p is not None]

    def cache_needs(self):
        return self.mixer.kv_need(), self.mixer.state_need()

    def forward(self, ctx, x, run):
        T, d = x.shape[0], x.shape[1] // self.S
        h = ctx.buffer("streams_input", (T, d), self.dtype)
        y = ctx.buffer("sublayer_out", (T, d), torch.float32)
        watch = getattr(ctx.engine, "after_sublayer", None)      # a caller that looks at a sublayer's output and at the rows behind it
        m_in, m_mix, m_out = self.numbers.of("mixer")
        K.streams_step(x, self.S, in_w=m_in, norm_w=self.mixer_norm.weight_f32, eps=self.mixer_norm.eps, h=h)
        self.mixer.forward(ctx, h, y, run, epilogue=ops.EPI_STORE)
        if watch is not None:
            watch(run.entry, "mixer", y)
        if self.ffn is None:
            K.streams_step(x, self.S, y=y, mix=m_mix, out_w=m_out)
        else:
            f_in, f_mix, f_out = self.numbers.of("ffn")
            K.streams_step(x, self.S, y=y, mix=m_mix, out_w=m_out, in_w=f_in, norm_w=self.ffn_norm.weight_f32,
                           eps=self.ffn_norm.eps, h=h)
            if watch is not None:
                watch(run.entry, "mixer_added", x)
            self.ffn.forward(ctx, h, y, epilogue=ops.EPI_STORE)
            if watch is not None:
                watch(run.entry, "ffn", y)
            K.streams_step(x, self.S, y=y, mix=f_mix, out_w=f_out)
        ops.residual_written(ctx, x)


register_part("block", "prenorm", PreNormBlock)
register_part("block", "streams", StreamsBlock)
register_part("block", "outnorm", OutNormBlock)
register_part("block", "parallel", ParallelBlock)

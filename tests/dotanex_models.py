"""Small Dotanex configurations for the tests, and model folders made from them (never the product's own)."""
from __future__ import annotations

import atexit
import functools
import json
import os
import shutil
import tempfile

import numpy as np

import plain_dotanex as P


def _moe(experts, identity, top, ff, limit, shared=None):
    return {"kind": "moe", "router": {"experts": experts, "identity": identity, "top": top},
            "expert": {"ff": ff, "limit": limit},
            "shared": None if shared is None else {"ff": shared[0], "limit": shared[1]}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _lightning(heads, dim, vdim, decay, mlp, weights_of=None):
    lay = {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}, "mlp": mlp}
    return lay if weights_of is None else dict(lay, weights_of=weights_of)


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, scaling, mlp, weights_of=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    lay = {"type": "latent_attention", "mlp": mlp,
           "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                     "scale": scale, "rot": rot}}
    return lay if weights_of is None else dict(lay, weights_of=weights_of)


def _window(heads, kv, dim, scale, base, dims, scaling, size, mlp, weights_of=None):
    rot = {"base": base, "dims": dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale, "rot": rot}
    if size is not None:
        m["mask"] = {"size": size}
    lay = {"type": "attention", "mixer": m, "mlp": mlp}
    return lay if weights_of is None else dict(lay, weights_of=weights_of)


# every kind of layer; three copies of the residual row; sizes that no tile divides (heads of 24 and 40, a latent of
# 40, a width of 96); a window that is no multiple of anything; identity experts; a shared expert of another size and
# bound than the experts; two layers that run another layer's weights with a state and a cache of their own
MIXED = {
    "architecture": "Dotanex", "vocab": 300, "width": 96, "norm": {"eps": 1e-5}, "streams": 3,
    "layers": [_lightning(3, 24, 40, [0.5, 0.93, 0.999], _dense(72)),
               _window(4, 2, 24, 0.2, 10000.0, 8, (4.0, 1.0, 4.0, 64), 37, _moe(5, 2, 3, 40, 1.5, (24, 0.7))),
               _latent(3, 24, 8, 40, 48, 40, 0.17, 5000.0, (4.0, 64, 16.0, 1.0), _moe(4, 1, 2, 32, 2.0, (32, 2.0))),
               _lightning(3, 24, 40, [0.5, 0.93, 0.999], _dense(72), weights_of=0),
               _latent(3, 24, 8, 40, 48, 40, 0.17, 5000.0, (4.0, 64, 16.0, 1.0), _moe(4, 1, 2, 32, 2.0, (32, 2.0)), weights_of=2)],
}
# a windowed attention first; ONE copy of the residual row (the numbers around the sublayers still act); as many kv
# heads as heads; a window of exactly a page and a layer without a mask; rotations without scaling; no identity experts;
# every expert chosen; no shared expert; a layer without feed-forward; one head; a layer that runs a LATER layer's
# weights; unbounded experts
REORDERED = {
    "architecture": "Dotanex", "vocab": 211, "width": 80, "norm": {"eps": 1e-6}, "streams": 1,
    "layers": [_window(2, 2, 16, 0.25, 300.0, 16, None, 64, _moe(3, 0, 3, 24, 1.0)),
               _latent(2, 16, 4, 16, 16, 32, 0.2, 100.0, None, None, weights_of=4),
               _lightning(1, 16, 16, [0.96], _moe(6, 3, 2, 24, None, (16, None))),
               _window(3, 1, 40, 0.15, 1e6, 40, (8.0, 1.0, 4.0, 32), None, _dense(40)),
               _latent(2, 16, 4, 16, 16, 32, 0.2, 100.0, None, None),
               _lightning(4, 8, 56, [0.99, 0.9, 0.8, 0.3], None)],
}
# no copies at all: the plain residual sum around the same sublayers
PLAIN = {
    "architecture": "Dotanex", "vocab": 150, "width": 64, "norm": {"eps": 1e-5},
    "layers": [_latent(2, 16, 8, 24, 24, 24, 0.2, 1000.0, (2.0, 32, 8.0, 1.0), _dense(48)),
               _lightning(2, 16, 24, [0.9, 0.99], _moe(3, 1, 2, 24, 1.0, (24, 1.0))),
               _window(2, 1, 32, 0.18, 1000.0, 16, None, 20, None)],
}
# head sizes that the matrix cores' kernels are built for, widths in whole tiles: what a bfloat16 engine runs on its
# fast paths (windowed attention with heads of 64 and 128, experts' products on the matrix cores); four copies
TILED = {
    "architecture": "Dotanex", "vocab": 704, "width": 128, "norm": {"eps": 1e-5}, "streams": 4,
    "layers": [_window(4, 2, 64, 0.125, 10000.0, 32, (8.0, 1.0, 4.0, 128), 100, _moe(8, 2, 2, 64, 2.0, (128, 1.0))),
               _lightning(4, 32, 64, [0.7, 0.9, 0.97, 0.995], _dense(256)),
               _latent(4, 64, 32, 64, 96, 64, 0.1, 40000.0, (8.0, 128, 32.0, 1.0), _moe(4, 4, 2, 64, 2.0, (64, 2.0))),
               _window(2, 1, 128, 0.09, 50000.0, 64, None, 130, None),
               _latent(4, 64, 32, 64, 96, 64, 0.1, 40000.0, (8.0, 128, 32.0, 1.0), _moe(4, 4, 2, 64, 2.0, (64, 2.0)), weights_of=2)],
}
CONFIGS = {"mixed": MIXED, "reordered": REORDERED, "plain": PLAIN, "tiled": TILED}

_root = tempfile.mkdtemp(prefix="dotanex-tests-")
atexit.register(shutil.rmtree, _root, ignore_errors=True)


def write_model(folder, cfg, W):
    import torch
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    save_file({k: torch.tensor(v).to(torch.bfloat16).contiguous() for k, v in W.items()},
              os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)


@functools.lru_cache(maxsize=None)
def model(name, seed=3):
    """(folder, config dict, float32 numpy weights as the folder stores them in bfloat16)."""
    cfg = CONFIGS[name]
    W = P.make_weights(cfg, seed)
    folder = os.path.join(_root, f"{name}-{seed}")
    write_model(folder, cfg, W)
    return folder, cfg, W


@functools.lru_cache(maxsize=None)
def tokens(name, seed, n):
    """Token ids at which no router of the model makes a close call (``plain_dotanex.tokens_with_clear_choices``)."""
    _, cfg, W = model(name)
    return P.tokens_with_clear_choices(cfg, W, seed, n)


# Largest allowed difference of a row of logits (its mean taken off, root mean square over the vocabulary) as a
# fraction of the root mean square of the plain logits. float32: sums in another order. bfloat16: activations between
# the parts are rounded to 8 bits of mantissa.
TOL = {"float32": 8e-5, "bfloat16": 3e-2}
# The model with latents of 16 and 32 elements, heads of 16 and experts without a bound averages a row's rounding over
# the fewest elements: twice the bound in bfloat16.
LOOSER = {"reordered": 2.0, "seed": 2.0}      # ("seed": the models drawn from seeds, which are as narrow or narrower)


def row_errors(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all()
    d = got - ref
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / np.sqrt(((ref - ref.mean(-1, keepdims=True)) ** 2).mean())


def close(got, ref, dtype, what="", few_far=0):
    """float32: every row within the bound. bfloat16: rounding has a tail (these models are narrow: a row's error is
    the mean of few elements'), so one row in twenty-five may lie over the bound, and none over two and a half times it
    (``few_far``: but for so many rows); a wrong key, state or expert moves a row by tens of times the bound."""
    e = row_errors(got, ref)
    tol = TOL[dtype] * (LOOSER.get(what.split()[0] if what else "", 1.0) if dtype == "bfloat16" else 1.0)
    bad = np.flatnonzero(e > tol)
    allowed = 0 if dtype == "float32" else max(2, len(e) // 25)
    worst = np.flatnonzero(e > (tol if dtype == "float32" else 2.5 * tol))
    if dtype == "bfloat16" and few_far and len(worst) <= few_far:
        # (a model drawn from a seed may leave a token whose clearest choice of experts is still close: such a row,
        # with another expert in a 16-bit engine, is far off, and the rows around it are not)
        worst, bad = worst[:0], np.setdiff1d(bad, worst)
    assert len(bad) <= allowed and not len(worst), \
        f"{what}: row {int(bad[0])} is the first of {len(bad)} over {tol}: {e[bad[0]]:.3e}; the worst has {e.max():.3e}"
    return float(e.max())


def near(got, ref, dtype, what=""):
    """Elements of residual rows or of a sublayer's output against the plain ones, on the scale of the largest:
    float32 8e-5 (2e-4 for a sublayer alone is the caller's), bfloat16 4e-2 with one element in fifty up to five
    times that (a sublayer deep in a model reads rows that carry the rounding of everything before it)."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert got.shape == ref.shape and np.isfinite(got).all(), what
    d = np.abs(got - ref) / max(np.abs(ref).max(), 1e-3)
    if dtype == "float32":
        assert d.max() < 2e-4, f"{what}: {d.max():.3e}"
    else:
        assert (d > 4e-2).mean() <= 2e-2 and d.max() < 0.2, f"{what}: {(d > 4e-2).mean():.2e} of the elements over, the worst {d.max():.3e}"

"""Small Nolatar configurations for the tests, and model folders made from them (never the product's own)."""
from __future__ import annotations

import atexit
import functools
import json
import os
import shutil
import tempfile

import numpy as np

import plain_nolatar as P


def _moe(experts, top, ff, shared):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff},
            "shared": None if shared is None else {"ff": shared}}


def _mamba(heads, vdim, state, groups, conv, norm_groups, mlp):
    return {"type": "mamba2", "mlp": mlp,
            "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}}


def _left(heads, kv, dim, vdim, scale, base, dims, size=None):
    c = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"base": base, "dims": dims}}
    if size is not None:
        c["mask"] = {"size": size}
    return c


def _right(heads, dim, vdim, decay, base, dims):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay, "rot": {"base": base, "dims": dims}}


def _parallel(left, right, ls, rs, mlp):
    return {"type": "parallel", "mlp": mlp, "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs}}


def _diff(heads, kv, dim, vdim, scale, diff, base, dims, mlp, kv_from=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff, "rot": {"base": base, "dims": dims}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


# every kind of layer; sizes that no tile divides (heads of 24 and 40, a state of 20, a width of 96); rotations over a
# part of the head in both pairings; a chunk that is no multiple of anything; three heads in three groups; a reader
# two layers behind its keys' owner; a layer without feed-forward; experts of another size than the shared one
MIXED = {
    "architecture": "Nolatar", "vocab": 300, "width": 96, "norm": {"eps": 1e-5},
    "layers": [_mamba(3, 24, 20, 3, 3, 1, _moe(5, 2, 40, 72)),
               _diff(4, 1, 24, 40, 0.2, 0.35, 10000.0, 8, _moe(4, 1, 64, None)),
               _parallel(_left(4, 2, 32, 48, 0.18, 5000.0, 16, 37), _right(3, 24, 40, [0.9, 0.97, 0.995], 800.0, 12), 0.7, 1.3, None),
               _diff(4, 1, 24, 40, 0.3, 0.8, 10000.0, 8, _moe(3, 3, 32, 32), kv_from=1)],
}
# an attention first; a reader right behind its owner and a second owner after it; as many kv heads as heads; a chunk
# smaller than a page and one of one page exactly; no mask at all (every earlier key); one group, taps of 2 and 5;
# one expert of which one is chosen; norms in four parts
REORDERED = {
    "architecture": "Nolatar", "vocab": 211, "width": 80, "norm": {"eps": 1e-6},
    "layers": [_diff(2, 2, 16, 16, 0.25, 0.5, 300.0, 16, _moe(1, 1, 48, 24)),
               _diff(2, 2, 16, 16, 0.4, 0.2, 300.0, 16, None, kv_from=0),
               _parallel(_left(2, 2, 16, 32, 0.25, 100.0, 8, 9), _right(1, 16, 16, [0.96], 100.0, 16), 1.0, 0.5, _moe(6, 2, 24, 24)),
               _mamba(4, 16, 8, 1, 2, 4, None),
               _diff(6, 3, 8, 24, 0.35, 0.1, 1000.0, 4, _moe(8, 3, 16, None)),
               _parallel(_left(3, 1, 40, 24, 0.15, 10000.0, 40, 64), _right(2, 40, 8, [0.5, 0.999], 10000.0, 2), -0.8, 0.9, None),
               _parallel(_left(1, 1, 48, 48, 0.14, 1e6, 24, None), _right(4, 8, 56, [0.99, 0.9, 0.8, 0.7], 50.0, 8), 0.5, 0.5, None),
               _mamba(2, 40, 33, 2, 5, 2, _moe(2, 2, 20, 20))],
}
# head sizes that the matrix cores' kernels are built for, widths in whole tiles: what a bfloat16 engine runs on its
# fast paths (experts' products on the matrix cores, heads of 64 and 128 with values of the keys' size). The offset of
# the differential layers keeps their lambda (0.39 and 1.28 with these weights) away from 1, where the two maps cancel
# and a bfloat16 engine's rounding of the maps' outputs is all that is left of a head
TILED = {
    "architecture": "Nolatar", "vocab": 640, "width": 128, "norm": {"eps": 1e-5},
    "layers": [_parallel(_left(4, 2, 64, 64, 0.125, 10000.0, 64, 100), _right(2, 64, 64, [0.97, 0.99], 10000.0, 64), 0.75, 1.2, _moe(4, 2, 64, 128)),
               _mamba(4, 32, 64, 2, 4, 2, _moe(8, 2, 32, 32)),
               _diff(2, 1, 64, 64, 0.125, 0.7, 40000.0, 64, _moe(4, 2, 64, 64)),
               _diff(2, 1, 64, 64, 0.125, 0.7, 40000.0, 64, None, kv_from=2),
               _parallel(_left(2, 1, 128, 128, 0.09, 50000.0, 64, 130), _right(1, 128, 128, [0.98], 50000.0, 32), 1.0, 1.0, None)],
}
CONFIGS = {"mixed": MIXED, "reordered": REORDERED, "tiled": TILED}

_root = tempfile.mkdtemp(prefix="nolatar-tests-")
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
    """Token ids at which no router of the model makes a close call (see ``plain_nolatar.tokens_with_clear_choices``)."""
    _, cfg, W = model(name)
    return P.tokens_with_clear_choices(cfg, W, seed, n)


# Largest allowed difference of a row of logits (its mean taken off, root mean square over the vocabulary) as a
# fraction of the root mean square of the plain logits. float32: sums in another order, through up to eight layers
# whose norms stand behind the sublayers (a sublayer's rounding is scaled up with its output). bfloat16: activations
# between the parts are rounded to 8 bits of mantissa.
TOL = {"float32": 8e-5, "bfloat16": 3e-2}
# The model of eight layers turns rounding into three times the difference that the others do (a twin of the plain
# implementation whose layers read disturbed inputs says so: ``plain_nolatar.Sequence(noise=...)``): its bfloat16 bound.
LOOSER = {"reordered": 2.5}


def bound(dtype, what=""):
    """The bound for rows of the model whose name ``what`` begins with."""
    return TOL[dtype] * (LOOSER.get(what.split()[0] if what else "", 1.0) if dtype == "bfloat16" else 1.0)


def row_errors(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all()
    d = got - ref
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / np.sqrt(((ref - ref.mean(-1, keepdims=True)) ** 2).mean())


def close(got, ref, dtype, what=""):
    e = row_errors(got, ref)
    tol = bound(dtype, what)
    bad = np.flatnonzero(e > tol)
    assert not len(bad), f"{what}: row {int(bad[0])} is the first of {len(bad)} over {tol}: {e[bad[0]]:.3e}"
    return float(e.max())

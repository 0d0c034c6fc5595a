"""The Nolatar configuration on the CPU: reader, run order, descriptions, expected tensors, cache needs, errors, and
the plain implementation's own consistency (a sequence fed whole and in pieces)."""
import copy

import numpy as np
import pytest
import torch

import plain_nolatar as P
from nolatar_models import CONFIGS, MIXED, REORDERED, model

from gpullama3_java_amd.config import ConfigError, config_from_dict
from gpullama3_java_amd.parts import DecoderModel, expected_tensors


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_expected_tensors_are_the_design_s(name):
    cfg = config_from_dict(CONFIGS[name])
    exp = expected_tensors(cfg.model_spec())
    shapes = P.tensor_shapes(CONFIGS[name])
    assert set(exp) == set(shapes)
    for k, s in shapes.items():
        assert tuple(exp[k].shape) == tuple(s), k
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()


def test_run_order_and_descriptions():
    cfg = config_from_dict(MIXED)
    spec = cfg.model_spec()
    assert [r.layer for r in spec.run_order] == [0, 1, 2, 3] and [r.reads for r in spec.run_order] == [None, None, None, 1]
    assert all(b.kind == "outnorm" for b in spec.layers)
    ssm, d1, par, d2 = (b.mixer for b in spec.layers)
    assert (ssm.kind, ssm.n_heads, ssm.head_dim, ssm.state_dim, ssm.n_groups, ssm.conv_taps, ssm.norm_groups) == ("state_space", 3, 24, 20, 3, 3, 1)
    assert d1.differential.offset == 0.35 and d1.position.pairing == "adjacent" and d1.position.head_dim == 8 and "k" in d1.names
    assert "k" not in d2.names and "k_norm" not in d2.names and d2.differential.offset == 0.8
    assert par.normalised is False and par.left.chunk == 37 and par.left.out_mult == 0.7 and par.right.out_mult == 1.3
    assert par.left.position.pairing == "half" and par.right.decay == (0.9, 0.97, 0.995) and par.right.position.head_dim == 12
    assert spec.layers[2].ffn is None and spec.layers[1].ffn.shared is None and spec.layers[0].ffn.shared.intermediate == 72
    assert spec.final_norm.kind == "layernorm" and spec.final_norm.names == {"weight": "final.norm", "bias": "final.norm.b"}
    assert "l2.norm2" in spec.unused_tensor_names


def test_cache_needs():
    m = DecoderModel(config_from_dict(MIXED).model_spec(), torch.float32, "cpu")
    kv, state = m.cache_needs()
    assert kv[0] is None and kv[3] is None                       # a state space; a reader
    assert (kv[1].n_kv_heads, kv[1].v_heads, kv[1].head_dim, kv[1].value_dim, kv[1].chunk) == (2, 1, 32, 48, None)   # (heads padded to 16s)
    assert (kv[2].n_kv_heads, kv[2].v_heads, kv[2].chunk) == (2, None, 37)
    assert state[0].elements == -(-2 * (3 * 24 + 2 * 3 * 20) // 4) * 4 + 3 * 20 * 24
    assert state[2].elements == 3 * 24 * 40 and state[1] is None and state[3] is None


@pytest.mark.parametrize("change, says", [
    (lambda c: c["layers"][0].update(type="gru"), "'type'"),
    (lambda c: c["layers"][0]["mixer"].update(groups=2), "groups"),
    (lambda c: c["layers"][0]["mixer"].update(norm_groups=5), "norm_groups"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "rot"),
    (lambda c: c["layers"][2]["mixer"]["right"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].update(vdim=24), "reads"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "largest"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "'mlp'"),
    (lambda c: c.pop("width"), "'width'"),
])
def test_errors_name_the_key(change, says):
    c = copy.deepcopy(MIXED)
    change(c)
    with pytest.raises(ConfigError, match=says):
        config_from_dict(c)


def test_the_plain_implementation_in_pieces():
    """Fed whole, token by token and in uneven pieces, a sequence gives the same rows: the chunked mask counts from
    position 0, the states and the convolution's inputs carry over."""
    _, cfg, W = model("reordered")
    rng = np.random.default_rng(5)
    toks = rng.integers(0, cfg["vocab"], 90).tolist()
    whole = P.forward(cfg, W, toks)
    s, rows, lo = P.Sequence(cfg, W), [], 0
    for hi in (1, 2, 9, 10, 63, 64, 65, 90):
        rows.append(s.feed(toks[lo:hi])[0])
        lo = hi
    np.testing.assert_allclose(np.concatenate(rows), whole, atol=1e-9)


def test_mechanisms_of_the_plain_implementation():
    # the chunked mask: the first key of a chunk is seen by the chunk's queries alone
    assert P.sees(36, 0, 37) and not P.sees(37, 36, 37) and P.sees(37, 37, 37) and P.sees(73, 37, 37) and not P.sees(74, 73, 37)
    assert P.sees(500, 0, None) and not P.sees(3, 4, None)
    # rotation: position 0 changes nothing, pairs are (i, i + dims/2) or (2i, 2i + 1), the rest passes
    x = np.arange(1.0, 9.0).reshape(1, 1, 8)
    np.testing.assert_allclose(P.turn(x, [0], 100.0, 4, "half"), x)
    a = P.turn(x, [3], 100.0, 4, "half")[0, 0]
    np.testing.assert_allclose([a[0], a[2]], [1 * np.cos(3) - 3 * np.sin(3), 3 * np.cos(3) + 1 * np.sin(3)])
    np.testing.assert_allclose(a[4:], x[0, 0, 4:])
    b = P.turn(x, [3], 100.0, 4, "adjacent")[0, 0]
    np.testing.assert_allclose([b[0], b[1]], [1 * np.cos(3) - 2 * np.sin(3), 2 * np.cos(3) + 1 * np.sin(3)])
    np.testing.assert_allclose([b[2], b[3]], [3 * np.cos(0.3) - 4 * np.sin(0.3), 4 * np.cos(0.3) + 3 * np.sin(0.3)])
    # the router: the largest logits, the lower number first on a tie, weights over the chosen alone
    W = {"r.router": np.eye(3), "r.e0.up": np.eye(3), "r.e0.down": np.eye(3), "r.e1.up": 2 * np.eye(3), "r.e1.down": np.eye(3),
         "r.e2.up": 3 * np.eye(3), "r.e2.down": np.eye(3)}
    c = {"router": {"experts": 3, "top": 2}, "expert": {"ff": 3}, "shared": None}
    h = np.array([[1.0, 1.0, 0.0]])
    y = P.routed_feed_forward(W, "r.", c, h)
    np.testing.assert_allclose(y, 0.5 * P.gelu_erf(h) + 0.5 * P.gelu_erf(2 * h))
    np.testing.assert_allclose(P.gelu_erf(np.array([1.0])), [0.8413447460685429])
    np.testing.assert_allclose(P.layer_norm(np.array([[1.0, 3.0]]), [2.0, 2.0], [0.5, 0.5], 0.0), [[-1.5, 2.5]])

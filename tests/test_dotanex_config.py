"""The Dotanex configuration on the CPU: reader, run order, descriptions, expected tensors, cache needs, errors, the
rotations' frequencies, and the plain implementation's own consistency (a sequence fed whole and in pieces)."""
import copy

import numpy as np
import pytest
import torch

import plain_dotanex as P
from dotanex_models import CONFIGS, MIXED, PLAIN, REORDERED, model

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
    spec = config_from_dict(MIXED).model_spec()
    # five layers of which two run another layer's weights: three blocks, five entries with storage of their own
    assert len(spec.layers) == 3 and [r.layer for r in spec.run_order] == [0, 1, 2, 0, 2] and spec.streams == 3
    assert all(b.kind == "streams" and b.streams == 3 for b in spec.layers)
    light, window, latent = (b.mixer for b in spec.layers)
    assert (light.kind, light.key_scale, light.input_activation, light.norm_over, light.gate_activation, light.position) == \
        ("retention", 1.0, "silu", "all", "sigmoid", None)
    assert light.decay == (0.5, 0.93, 0.999) and light.names["norm"] == "l0.mix.norm"
    assert window.values_are_keys and "v" not in window.names and window.names["sink"] == "l1.mix.sink"
    assert (window.window, window.qk_norm_eps, window.position.pairing, window.position.head_dim) == (37, 1e-5, "half", 8)
    assert window.position.scaling.low_freq_factor == 1.0 and window.position.scaling.original_max_position == 64
    assert (latent.kind, latent.q_rank, latent.kv_rank, latent.rot_dim, latent.position.pairing) == ("latent_attention", 48, 40, 8, "adjacent")
    assert latent.position.scaling.fast == 16.0 and latent.position.scaling.original_max_position == 64
    moe = spec.layers[1].ffn
    assert (moe.n_experts, moe.n_identity, moe.top, moe.weights, moe.sum_eps) == (5, 2, 3, "scores", 1e-20)
    assert moe.expert.gated and (moe.expert.limit, moe.expert.up_shift, moe.expert.activation) == (1.5, 1.0, "quick_gelu")
    assert (moe.shared.intermediate, moe.shared.limit) == (24, 0.7)
    assert spec.layers[0].ffn.kind == "gated" and spec.layers[0].ffn.activation == "silu"
    assert spec.layers[0].stream_names["ffn_mix"] == "l0.hc2.mix"
    # a folder without copies is a pre-norm decoder; a layer may run a LATER layer's weights
    assert all(b.kind == "prenorm" for b in config_from_dict(PLAIN).model_spec().layers)
    spec = config_from_dict(REORDERED).model_spec()
    assert [r.layer for r in spec.run_order] == [0, 3, 1, 2, 3, 4] and spec.layers[4].ffn is None and spec.layers[0].ffn.shared is None


def test_cache_needs():
    m = DecoderModel(config_from_dict(MIXED).model_spec(), torch.float32, "cpu")
    kv, state = m.cache_needs()
    assert kv[0] is None and kv[3] is None and state[0].elements == state[3].elements == 3 * 24 * 40
    assert (kv[1].n_kv_heads, kv[1].head_dim, kv[1].window, kv[1].values) == (2, 32, 37, True)       # (heads padded to 16s)
    assert (kv[2].n_kv_heads, kv[2].head_dim, kv[2].values) == (1, 64, False) and kv[4] == kv[2]     # a latent of 40 + 8 in rows of 64, one array
    assert state[1] is None and state[2] is None


@pytest.mark.parametrize("change, says", [
    (lambda c: c["layers"][0].update(type="gru"), "'type'"),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"].update(vdim=32), "values are the keys"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "rot"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("low"), "low"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=6), "rot"),
    (lambda c: c["layers"][2]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][3].update(weights_of=3), "weights_of"),
    (lambda c: c["layers"][3].update(weights_of=4), "weights_of"),
    (lambda c: c["layers"][3].update(weights_of=1), "type, mixer and mlp"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "largest"),
    (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "'mlp'"),
    (lambda c: c.update(streams=0), "'streams'"),
    (lambda c: c.pop("width"), "'width'"),
])
def test_errors_name_the_key(change, says):
    c = copy.deepcopy(MIXED)
    change(c)
    with pytest.raises(ConfigError, match=says):
        config_from_dict(c)


def test_frequencies_of_both_rotations():
    from gpullama3_java_amd.config.specs import Llama3RopeScaling, YarnRopeScaling
    from gpullama3_java_amd.parts.rotary import frequencies, magnitude
    for base, dims, sc in ((5000.0, 8, (4.0, 64, 16.0, 1.0)), (40000.0, 32, (8.0, 128, 32.0, 1.0)), (1e6, 64, (40.0, 4096, 32.0, 1.0)),
                           (100.0, 4, (2.0, 16, 1.0, 1.0))):
        want, mag = P.yarn_frequencies(base, dims, dict(zip(("factor", "original", "fast", "slow"), sc)))
        np.testing.assert_allclose(frequencies(dims, base, YarnRopeScaling(sc[0], sc[1], sc[2], sc[3])), want, rtol=3e-7)
        assert magnitude(YarnRopeScaling(*sc)) == pytest.approx(mag) and mag == pytest.approx(0.1 * np.log(sc[0]) + 1)
    # by hand: 4 pairs, base 16: f = 1, 1/2, 1/4, 1/8; the ramp runs from pair floor(8 ln(64 / 32 pi) / 2 ln 16) -> 0 (below
    # zero) to pair ceil(8 ln(64 / 2 pi) / (2 ln 16)) = ceil(3.35) = 4: a quarter of the way per pair
    got = frequencies(8, 16.0, YarnRopeScaling(4.0, 64, 16.0, 1.0))
    np.testing.assert_allclose(got, [1.0, 0.5 * (0.25 / 4 + 0.75), 0.25 * (0.5 / 4 + 0.5), 0.125 * (0.75 / 4 + 0.25)], rtol=1e-6)
    for base, dims, sc in ((10000.0, 8, (4.0, 1.0, 4.0, 64)), (1e6, 40, (8.0, 1.0, 4.0, 32)), (500000.0, 64, (8.0, 1.0, 4.0, 8192))):
        want = P.wavelength_frequencies(base, dims, dict(zip(("factor", "low", "high", "original"), sc)))
        np.testing.assert_allclose(frequencies(dims, base, Llama3RopeScaling(*sc)), want, rtol=3e-7)


def test_the_plain_implementation_in_pieces():
    """Fed whole, token by token and in uneven pieces, a sequence gives the same rows: windows count from the query,
    latents and keys accumulate, the recurrent states carry over."""
    for name in ("mixed", "reordered"):
        _, cfg, W = model(name)
        rng = np.random.default_rng(5)
        toks = rng.integers(0, cfg["vocab"], 90).tolist()
        whole = P.forward(cfg, W, toks)
        s, rows, lo = P.Sequence(cfg, W), [], 0
        for hi in (1, 2, 9, 10, 36, 37, 38, 63, 64, 65, 90):
            rows.append(s.feed(toks[lo:hi]))
            lo = hi
        np.testing.assert_allclose(np.concatenate(rows), whole, atol=1e-9)


def test_mechanisms_of_the_plain_implementation():
    # rotation: position 0 changes nothing but the magnitude, pairs are (i, i + n) or (2i, 2i + 1), the rest passes
    x = np.arange(1.0, 9.0).reshape(1, 1, 8)
    np.testing.assert_allclose(P.turn(x, [0], [1.0, 0.1], "half"), x)
    a = P.turn(x, [3], [1.0, 0.1], "half")[0, 0]
    np.testing.assert_allclose([a[0], a[2]], [1 * np.cos(3) - 3 * np.sin(3), 3 * np.cos(3) + 1 * np.sin(3)])
    np.testing.assert_allclose(a[4:], x[0, 0, 4:])
    b = P.turn(x, [3], [1.0, 0.1], "adjacent", 2.0)[0, 0]
    np.testing.assert_allclose([b[0], b[1]], [2 * (1 * np.cos(3) - 2 * np.sin(3)), 2 * (2 * np.cos(3) + 1 * np.sin(3))])
    np.testing.assert_allclose([b[2], b[3]], [2 * (3 * np.cos(0.3) - 4 * np.sin(0.3)), 2 * (4 * np.cos(0.3) + 3 * np.sin(0.3))])
    # the router: the choice by score + correction, the weights by the scores alone; identity experts hand h on
    eye = np.eye(3)
    W = {"r.router": np.array([[1.0, 0, 0], [0, 1.0, 0], [0, 0, 1.0], [0, 0, 0]]), "r.correction": np.array([0.0, 0.0, 0.0, 1.0]),
         **{f"r.e{e}.{k}": (e + 1) * eye for e in range(3) for k in ("gate", "up", "down")}}
    mlp = {"kind": "moe", "router": {"experts": 3, "identity": 1, "top": 2}, "expert": {"ff": 3, "limit": 1.5}, "shared": None}
    h = np.array([[2.0, 1.0, 0.0]])
    idx, w, _ = P.route(h, W, "r.", mlp)
    z = np.exp([2.0, 1.0, 0.0, 0.0])
    assert list(idx[0]) == [3, 0]                         # the correction lifts the identity expert to the top
    np.testing.assert_allclose(w[0], [z[3] / (z[3] + z[0]), z[0] / (z[3] + z[0])])
    g, u = np.minimum(h[0], 1.5), np.clip(h[0], -1.5, 1.5)
    np.testing.assert_allclose(P.mixture(h, W, "r.", mlp)[0], w[0, 0] * h[0] + w[0, 1] * (g / (1 + np.exp(-1.702 * g)) * (u + 1)))
    # the sink takes its share of the weights and adds nothing: one key, sink as large as its score -> half the value
    Wa = {"a.q": eye[:2], "a.k": eye[:2], "a.o": np.eye(2), "a.q.norm": np.ones(2), "a.k.norm": np.ones(2), "a.sink": np.array([0.0])}
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 0.0, "rot": {"base": 10.0, "dims": 2}}
    y = P.window_attention(np.array([[3.0, 4.0, 0.0]]), np.array([0]), Wa, "a.", m, 0.0, {})
    np.testing.assert_allclose(y[0], [1.5, 2.0])          # the value is the key as projected: (3, 4), not its normed form

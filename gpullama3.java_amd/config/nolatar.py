"""Typed configuration of the Nolatar decoder, read from its config.json.

Nolatar is a decoder whose norms stand behind the sublayers: ``x += LN1(mixer(x))``, then, where the layer has a
feed-forward, ``x += LN2(ffn(x))``; the sublayers read the residual rows themselves, and the norms are layer norms
with weight and bias. Its layers differ in kind:

  mamba2:    a selective state space (one projection to [z | x | B | C | dt], a short causal convolution with silu
             over x, B, C, a matrix per head with a scalar decay per token, the gate ``silu(z)`` in front of a unit
             norm in equal parts);
  parallel:  two mixers side by side, ``left_scale * left + right_scale * right``: an attention with a norm on
             queries and keys per head, a rotation in halves over the head's first elements and a chunked mask (a
             query sees the earlier keys of its own chunk), and a retention (linear attention with a fixed decay per
             head, its read-outs divided by their root mean square per head and gated);
  attention: differential attention (two score maps per head over the same values, ``a1 - lambda a2``, a unit norm
             per head, the factor ``1 - diff``), queries and keys normed per head and map and rotated in adjacent
             pairs, causal; a layer with ``kv_from`` reads an earlier layer's keys and values and has none of its own.

The feed-forward is a mixture of experts (``down(gelu(up h))`` each, the erf form of gelu) with a softmax over the
chosen logits, plus an expert that every token passes.

config.json: ``architecture`` "Nolatar", ``vocab``, ``width``, ``norm.eps`` and ``layers``, a list of
``{"type", "mixer": {...}, "mlp": {"kind": "moe", "router": {"experts", "top"}, "expert": {"ff"}, "shared": {"ff"} | null}
| null}`` with
  mamba2:    ``heads``, ``vdim``, ``state``, ``groups``, ``conv``, ``norm_groups``;
  parallel:  ``left`` (``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``rot``: ``base``, ``dims``; ``mask``: ``size``),
             ``right`` (``heads``, ``dim``, ``vdim``, ``decay`` (a list, one per head), ``rot``), ``left_scale``, ``right_scale``;
  attention: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``diff``, ``rot``, ``kv_from`` (optional).
The folder names no longest sequence: ``max_positions`` (ours, optional) bounds it, else ``DEFAULT_MAX_POSITIONS``.
Tensor names: ``embed``, ``final.norm`` (+ ``.b``), ``head``, and per layer i ``l<i>.norm1``, ``l<i>.norm2`` (+ ``.b``),
``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, replace
from typing import Optional

from .registry import ConfigError, _as_ids, register_architecture
from .specs import (AttentionSpec, BlockSpec, Differential, ExpertSpec, LayerNormSpec, ModelSpec, RetentionSpec,
                    RotarySpec, RoutedFeedForwardSpec, Run, SideBySideSpec, StateSpaceSpec)

# what the design fixes
EXPERT_ACTIVATION = "gelu"        # the erf form
LEFT_PAIRING = "half"             # the side-by-side attention and the retention turn element i with i + dims / 2
DIFFERENTIAL_PAIRING = "adjacent" # the differential attention turns element 2i with 2i + 1
DEFAULT_MAX_POSITIONS = 1 << 17   # a folder sets no bound on a sequence's length; the engine's caches need one
TYPES = ("mamba2", "parallel", "attention")


def _int(d, key, where, least=1):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, int) or v < least:
        raise ConfigError(f"config.json: {where}'{key}' must be an integer of at least {least}, found {v!r}")
    return v


def _positive(d, key, where):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not v > 0:
        raise ConfigError(f"config.json: {where}'{key}' must be a positive number, found {v!r}")
    return float(v)


def _number(d, key, where):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {where}'{key}' must be a number, found {v!r}")
    return float(v)


def _rot(c, dim, where):
    rot = c.get("rot") if isinstance(c, dict) else None
    if not isinstance(rot, dict):
        raise ConfigError(f"config.json: {where}'rot' must be an object with 'base' and 'dims'")
    dims = _int(rot, "dims", where + "rot: ", 2)
    if dims % 2 or dims > dim:
        raise ConfigError(f"config.json: {where}rot: {dims} rotated elements of heads of {dim}: pairs need an even "
                          "count, and the rotated part lies inside the head")
    return _positive(rot, "base", where + "rot: "), dims


def _grouped(c, where):
    heads, kv = _int(c, "heads", where), _int(c, "kv_heads", where)
    if heads % kv:
        raise ConfigError(f"config.json: {where}{heads} heads are not a multiple of {kv} kv_heads")
    return heads, kv


def _check_mixer(kind, m, where, i, layers):
    if not isinstance(m, dict):
        raise ConfigError(f"config.json: {where}'mixer' must be an object")
    if kind == "mamba2":
        heads, groups = _int(m, "heads", where), _int(m, "groups", where)
        if heads % groups:
            raise ConfigError(f"config.json: {where}{heads} heads are not a multiple of {groups} groups")
        inner = heads * _int(m, "vdim", where)
        _int(m, "state", where), _int(m, "conv", where)
        if inner % _int(m, "norm_groups", where):
            raise ConfigError(f"config.json: {where}{m['norm_groups']} norm_groups do not divide {inner} channels")
    elif kind == "parallel":
        L, R = m.get("left"), m.get("right")
        if not isinstance(L, dict) or not isinstance(R, dict):
            raise ConfigError(f"config.json: {where}'left' and 'right' must be objects")
        _grouped(L, where + "left: ")
        _int(L, "vdim", where + "left: "), _positive(L, "scale", where + "left: ")
        _rot(L, _int(L, "dim", where + "left: "), where + "left: ")
        if L.get("mask") is not None:
            _int(L["mask"], "size", where + "left: mask: ")
        heads = _int(R, "heads", where + "right: ")
        _int(R, "vdim", where + "right: ")
        _rot(R, _int(R, "dim", where + "right: "), where + "right: ")
        decay = R.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or any(
                isinstance(v, bool) or not isinstance(v, (int, float)) for v in decay):
            raise ConfigError(f"config.json: {where}right: 'decay' must list one number for each of the {heads} heads")
        _number(m, "left_scale", where), _number(m, "right_scale", where)
    else:
        _grouped(m, where)
        _int(m, "vdim", where), _positive(m, "scale", where), _number(m, "diff", where)
        _rot(m, _int(m, "dim", where), where)
        j = m.get("kv_from")
        if j is not None:
            if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < i or layers[j].get("type") != "attention" \
                    or layers[j]["mixer"].get("kv_from") is not None:
                raise ConfigError(f"config.json: {where}'kv_from' must name an earlier attention layer with keys and "
                                  f"values of its own, found {j!r}")
            o = layers[j]["mixer"]
            if any(o.get(k) != m.get(k) for k in ("kv_heads", "dim", "vdim")) or o.get("rot") != m.get("rot"):
                raise ConfigError(f"config.json: {where}layer {j}, whose keys and values this layer reads, has other "
                                  "head counts, sizes or rotation")


def _check_mlp(mlp, where):
    if mlp is None:
        return
    if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
        raise ConfigError(f"config.json: {where}'mlp' must be null or an object of kind 'moe'")
    experts, top = _int(mlp.get("router"), "experts", where + "router: "), _int(mlp.get("router"), "top", where + "router: ")
    if top > experts:
        raise ConfigError(f"config.json: {where}router: the {top} largest of {experts} experts")
    _int(mlp.get("expert"), "ff", where + "expert: ")
    if mlp.get("shared") is not None:
        _int(mlp["shared"], "ff", where + "shared: ")


@dataclass(frozen=True)
class NolatarConfiguration:
    vocab_size: int
    width: int
    norm_eps: float
    layers: tuple                           # the checked entries of config.json's 'layers', as they stand there
    max_positions: int = DEFAULT_MAX_POSITIONS
    context_length: Optional[int] = None
    stop_ids: tuple = ()
    architecture: str = "Nolatar"

    @property
    def max_position_embeddings(self):
        return self.max_positions if self.context_length is None else min(self.context_length, self.max_positions)

    @property
    def hidden_size(self):
        return self.width

    def __hash__(self):
        return hash((self.vocab_size, self.width, self.norm_eps, repr(self.layers), self.max_positions,
                     self.context_length, self.stop_ids))

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d):
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        for i, lay in enumerate(layers_in):
            where = f"layers[{i}]: "
            if not isinstance(lay, dict) or lay.get("type") not in TYPES:
                raise ConfigError(f"config.json: {where}'type' must be one of {TYPES}")
            _check_mixer(lay["type"], lay.get("mixer"), where, i, layers_in)
            _check_mlp(lay.get("mlp"), where + "mlp: ")
        return cls(vocab_size=_int(d, "vocab", ""), width=_int(d, "width", ""),
                   norm_eps=_positive(d.get("norm"), "eps", "norm: "), layers=tuple(copy.deepcopy(layers_in)),
                   max_positions=_int(d, "max_positions", "") if d.get("max_positions") is not None else DEFAULT_MAX_POSITIONS,
                   stop_ids=_as_ids(d.get("eos_token_id")))

    def to_dict(self):
        d = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.width,
             "norm": {"eps": self.norm_eps}, "layers": copy.deepcopy(list(self.layers))}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        if self.stop_ids:
            d["eos_token_id"] = list(self.stop_ids)
        return d

    # ------------------------------------------------------------------ what the engine asks
    def chat_format(self, tokenizer):
        raise ConfigError("a Nolatar model folder brings no chat format: give the prompt as token ids")

    def with_stop_ids(self, ids):
        return replace(self, stop_ids=tuple(ids))

    def with_context_length(self, n):
        if n is None or n < 0:
            return self
        return replace(self, context_length=min(n, self.max_positions))

    def run_order(self):
        """Every layer once; a layer with ``kv_from`` reads the named layer's keys and values."""
        return tuple(Run(layer=i, reads=lay["mixer"].get("kv_from") if lay["type"] == "attention" else None)
                     for i, lay in enumerate(self.layers))

    def _rotary(self, c, pairing):
        base, dims = _rot(c, c["dim"], "")
        return RotarySpec(head_dim=dims, theta=base, pairing=pairing, max_positions=self.max_position_embeddings)

    def _mixer(self, i, lay):
        d, eps, p, m = self.width, self.norm_eps, f"l{i}.mix.", lay["mixer"]
        if lay["type"] == "mamba2":
            return StateSpaceSpec(
                hidden=d, n_heads=m["heads"], head_dim=m["vdim"], n_groups=m["groups"], state_dim=m["state"],
                conv_taps=m["conv"], norm_groups=m["norm_groups"], norm_eps=eps,
                names={"in": p + "in", "conv": p + "conv", "conv_bias": p + "conv.b", "dt_bias": p + "dt_bias",
                       "A_log": p + "A_log", "D": p + "D", "norm": p + "norm", "o": p + "o"})
        if lay["type"] == "parallel":
            L, R = m["left"], m["right"]
            q = p + "left."
            left = AttentionSpec(
                hidden=d, n_heads=L["heads"], n_kv_heads=L["kv_heads"], head_dim=L["dim"], v_head_dim=L["vdim"],
                position=self._rotary(L, LEFT_PAIRING), scale=float(L["scale"]), qk_norm_eps=eps,
                chunk=L["mask"]["size"] if L.get("mask") is not None else None, out_mult=float(m["left_scale"]),
                names={"q": q + "q", "k": q + "k", "v": q + "v", "o": q + "o", "q_norm": q + "q.norm", "k_norm": q + "k.norm"})
            r = p + "right."
            right = RetentionSpec(
                hidden=d, n_heads=R["heads"], key_dim=R["dim"], value_dim=R["vdim"], decay=tuple(float(v) for v in R["decay"]),
                position=self._rotary(R, LEFT_PAIRING), norm_eps=eps, out_mult=float(m["right_scale"]),
                names={"q": r + "q", "k": r + "k", "v": r + "v", "g": r + "g", "o": r + "o"})
            return SideBySideSpec(hidden=d, left=left, right=right, normalised=False, weight=1.0, names={})
        names = {"q": p + "q", "o": p + "o", "q_norm": p + "q.norm", "lambda_q1": p + "lq1", "lambda_k1": p + "lk1",
                 "lambda_q2": p + "lq2", "lambda_k2": p + "lk2"}
        if m.get("kv_from") is None:
            names.update({"k": p + "k", "v": p + "v", "k_norm": p + "k.norm"})
        return AttentionSpec(
            hidden=d, n_heads=m["heads"], n_kv_heads=m["kv_heads"], head_dim=m["dim"], v_head_dim=m["vdim"],
            position=self._rotary(m, DIFFERENTIAL_PAIRING), scale=float(m["scale"]), qk_norm_eps=eps,
            differential=Differential(offset=float(m["diff"]), norm_eps=eps), names=names)

    def model_spec(self):
        d, eps = self.width, self.norm_eps

        def norm(name):
            return LayerNormSpec(dim=d, eps=eps, names={"weight": name, "bias": name + ".b"})

        blocks, unused = [], []
        for i, lay in enumerate(self.layers):
            p = f"l{i}."
            ffn = ffn_norm = None
            mlp = lay.get("mlp")
            if mlp is not None:
                q = p + "mlp."
                shared = mlp.get("shared")
                names = {"router": q + "router", "expert_up": q + "e{e}.up", "expert_down": q + "e{e}.down"}
                if shared is not None:
                    names.update({"shared_up": q + "shared.up", "shared_down": q + "shared.down"})
                ffn = RoutedFeedForwardSpec(
                    hidden=d, n_experts=mlp["router"]["experts"], top=mlp["router"]["top"],
                    expert=ExpertSpec(mlp["expert"]["ff"], EXPERT_ACTIVATION),
                    shared=ExpertSpec(shared["ff"], EXPERT_ACTIVATION) if shared is not None else None, names=names)
                ffn_norm = norm(p + "norm2")
            else:       # (a folder may hold the second norm of a layer without a feed-forward: nothing reads it)
                unused += [p + "norm2", p + "norm2.b"]
            blocks.append(BlockSpec(kind="outnorm", mixer_norm=norm(p + "norm1"), mixer=self._mixer(i, lay),
                                    ffn_norm=ffn_norm, ffn=ffn))
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden=d, layers=tuple(blocks),
            run_order=self.run_order(), final_norm=norm("final.norm"), max_positions=self.max_position_embeddings,
            tie_embeddings=False, embedding_name="embed", head_name="head", stop_ids=self.stop_ids,
            unused_tensor_names=tuple(unused))


register_architecture("Nolatar", NolatarConfiguration)

"""Typed configuration of the Dotanex decoder, read from its config.json.

Dotanex keeps ``streams`` copies of every token's residual row. A sublayer reads a learned mixture of the copies
through an RMS norm; its output goes back into every copy with a factor of its own while the copies are mixed among
themselves (``hc1.*`` around the mixer, ``hc2.*`` around the feed-forward: ``in`` [S], ``mix`` [S, S] indexed
[from, to], ``out`` [S]). All copies start as the embedding's output; their sum goes to the final norm. A folder
without ``streams`` is an ordinary pre-norm decoder. Its layers differ in kind:

  lightning:         linear attention with a fixed decay per head: q, k and v pass silu behind their projections,
                     ``S <- decay_h S + k v^T``, ``o = S^T q``; the heads' read-outs together are divided by their root
                     mean square, times a weight, times sigmoid of a gate projection; output projection;
  latent_attention:  queries through a normed latent; one normed latent per position from which every head's
                     unrotated keys and its values are expanded, and one rotated key part that the heads share
                     (adjacent pairs, frequencies on a ramp over the pair numbers with a factor on cos and sin);
                     causal, ordinary softmax; the heads' outputs times sigmoid of a gate projection;
  attention:         grouped heads, a norm on queries and keys per head, a rotation in halves over the head's first
                     elements with the long waves stretched, a sliding window, a learned sink per head in the softmax;
                     the values are the keys as projected.

A layer with ``weights_of: j`` has no tensors: it runs layer j's with a cache or state of its own. The feed-forward is
``down(silu(gate h) * up h)`` (``kind`` "dense") or a mixture (``kind`` "moe") of experts
``down(g sigmoid(1.702 g) (u + 1))`` with ``g = min(gate h, limit)``, ``u = clamp(up h, -limit, limit)``: the scores are a
softmax over all router outputs, of which the last ``identity`` stand for experts that hand their input on; the
``top`` largest of score + ``correction`` are chosen and weighted with their scores over the chosen scores' sum; a
shared expert of the same form runs for every token.

config.json: ``architecture`` "Dotanex", ``vocab``, ``width``, ``norm.eps``, ``streams`` and ``layers``, a list of
``{"type", "mixer": {...}, "mlp": {...} | null, "weights_of": j (optional)}`` with
  lightning:         ``heads``, ``dim``, ``vdim``, ``decay`` (a list, one per head);
  latent_attention:  ``heads``, ``dim``, ``rot_dim``, ``vdim``, ``q_rank``, ``kv_rank``, ``scale``,
                     ``rot``: ``base``, ``dims``, ``scaling``: ``factor``, ``original``, ``fast``, ``slow``;
  attention:         ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``mask``: ``size``,
                     ``rot``: ``base``, ``dims``, ``scaling``: ``factor``, ``low``, ``high``, ``original``;
  mlp:               ``{"kind": "dense", "ff"}`` or ``{"kind": "moe", "router": {"experts", "identity", "top"},
                     "expert": {"ff", "limit"}, "shared": {"ff", "limit"} | null}``.
The folder names no longest sequence: ``max_positions`` (ours, optional) bounds it, else ``DEFAULT_MAX_POSITIONS``.
Tensor names: ``embed``, ``final.norm``, ``head``, and per layer i ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.hc1.*``,
``l<i>.hc2.*``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, replace
from typing import Optional

from .registry import ConfigError, _as_ids, register_architecture
from .specs import (AttentionSpec, BlockSpec, ExpertSpec, GatedFeedForwardSpec, LatentAttentionSpec, Llama3RopeScaling,
                    ModelSpec, NormSpec, RetentionSpec, RotarySpec, RoutedFeedForwardSpec, Run, YarnRopeScaling)

# what the design fixes
EXPERT_ACTIVATION = "quick_gelu"      # g * sigmoid(1.702 g)
EXPERT_UP_SHIFT = 1.0                 # ... * (u + 1)
DENSE_ACTIVATION = "silu"
WEIGHT_SUM_EPS = 1e-20                # beside the chosen scores' sum
LATENT_PAIRING = "adjacent"           # the latent attention turns element 2i with 2i + 1
WINDOW_PAIRING = "half"               # the windowed attention turns element i with i + dims / 2
LIGHTNING_KEY_SCALE = 1.0             # no factor on k
DEFAULT_MAX_POSITIONS = 1 << 17       # a folder sets no bound on a sequence's length; the engine's caches need one
TYPES = ("lightning", "latent_attention", "attention")


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


def _rot(c, within, where, scaling_keys):
    """(base, dims, scaling dict or None) of a mixer's ``rot``; ``within``: the size of the part that is rotated."""
    rot = c.get("rot") if isinstance(c, dict) else None
    if not isinstance(rot, dict):
        raise ConfigError(f"config.json: {where}'rot' must be an object with 'base' and 'dims'")
    dims = _int(rot, "dims", where + "rot: ", 2)
    if dims % 2 or dims > within:
        raise ConfigError(f"config.json: {where}rot: {dims} rotated elements of {within}: pairs need an even count, and "
                          "the rotated part lies inside the head")
    sc = rot.get("scaling")
    if sc is not None:
        if not isinstance(sc, dict):
            raise ConfigError(f"config.json: {where}rot: 'scaling' must be an object or null")
        for k in scaling_keys:
            _positive(sc, k, where + "rot: scaling: ")
    return _positive(rot, "base", where + "rot: "), dims, sc


def _check_mixer(kind, m, where):
    if not isinstance(m, dict):
        raise ConfigError(f"config.json: {where}'mixer' must be an object")
    heads = _int(m, "heads", where)
    _int(m, "dim", where)
    if kind != "attention" or m.get("vdim") is not None:      # (the windowed attention's values are its keys: their size is the keys')
        _int(m, "vdim", where)
    if kind == "lightning":
        decay = m.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or any(
                isinstance(v, bool) or not isinstance(v, (int, float)) for v in decay):
            raise ConfigError(f"config.json: {where}'decay' must list one number for each of the {heads} heads")
    elif kind == "latent_attention":
        _int(m, "q_rank", where), _int(m, "kv_rank", where), _positive(m, "scale", where)
        rot_dim = _int(m, "rot_dim", where, 2)
        _, dims, _ = _rot(m, rot_dim, where, ("factor", "original", "fast", "slow"))
        if dims != rot_dim:
            raise ConfigError(f"config.json: {where}the rotated key part has {rot_dim} elements, 'rot.dims' says {dims}")
    else:
        kv = _int(m, "kv_heads", where)
        if heads % kv:
            raise ConfigError(f"config.json: {where}{heads} heads are not a multiple of {kv} kv_heads")
        if m.get("vdim") is not None and m["vdim"] != m["dim"]:
            raise ConfigError(f"config.json: {where}the values are the keys: 'vdim' {m['vdim']} must equal 'dim' {m['dim']}")
        _positive(m, "scale", where)
        _rot(m, m["dim"], where, ("factor", "low", "high", "original"))
        if m.get("mask") is not None:
            _int(m["mask"], "size", where + "mask: ")


def _check_expert(e, where):
    _int(e, "ff", where)
    if e.get("limit") is not None:
        _positive(e, "limit", where)


def _check_mlp(mlp, where):
    if mlp is None:
        return
    if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
        raise ConfigError(f"config.json: {where}'mlp' must be null or an object of kind 'dense' or 'moe'")
    if mlp["kind"] == "dense":
        _int(mlp, "ff", where)
        return
    r = mlp.get("router")
    experts, top = _int(r, "experts", where + "router: "), _int(r, "top", where + "router: ")
    identity = _int(r, "identity", where + "router: ", 0) if isinstance(r, dict) and r.get("identity") is not None else 0
    if top > experts + identity:
        raise ConfigError(f"config.json: {where}router: the {top} largest of {experts + identity} experts")
    _check_expert(mlp.get("expert"), where + "expert: ")
    if mlp.get("shared") is not None:
        _check_expert(mlp["shared"], where + "shared: ")


@dataclass(frozen=True)
class DotanexConfiguration:
    vocab_size: int
    width: int
    norm_eps: float
    layers: tuple                           # the checked entries of config.json's 'layers', as they stand there
    streams: Optional[int] = None           # None: one residual row per token and the plain residual sum
    max_positions: int = DEFAULT_MAX_POSITIONS
    context_length: Optional[int] = None
    stop_ids: tuple = ()
    architecture: str = "Dotanex"

    @property
    def max_position_embeddings(self):
        return self.max_positions if self.context_length is None else min(self.context_length, self.max_positions)

    @property
    def hidden_size(self):
        return self.width

    def __hash__(self):
        return hash((self.vocab_size, self.width, self.norm_eps, repr(self.layers), self.streams, self.max_positions,
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
            _check_mixer(lay["type"], lay.get("mixer"), where)
            _check_mlp(lay.get("mlp"), where + "mlp: ")
        for i, lay in enumerate(layers_in):
            j = lay.get("weights_of")
            if j is None:
                continue
            if (isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < len(layers_in) or j == i
                    or layers_in[j].get("weights_of") is not None):
                raise ConfigError(f"config.json: layers[{i}]: 'weights_of' must name another layer with tensors of its "
                                  f"own, found {j!r}")
            if any(layers_in[j].get(k) != lay.get(k) for k in ("type", "mixer", "mlp")):
                raise ConfigError(f"config.json: layers[{i}]: a layer that runs layer {j}'s weights has layer {j}'s "
                                  "type, mixer and mlp")
        streams = d.get("streams")
        if streams is not None:
            streams = _int(d, "streams", "")
        return cls(vocab_size=_int(d, "vocab", ""), width=_int(d, "width", ""),
                   norm_eps=_positive(d.get("norm"), "eps", "norm: "), layers=tuple(copy.deepcopy(layers_in)),
                   streams=streams,
                   max_positions=_int(d, "max_positions", "") if d.get("max_positions") is not None else DEFAULT_MAX_POSITIONS,
                   stop_ids=_as_ids(d.get("eos_token_id")))

    def to_dict(self):
        d = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.width,
             "norm": {"eps": self.norm_eps}, "layers": copy.deepcopy(list(self.layers))}
        if self.streams is not None:
            d["streams"] = self.streams
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        if self.stop_ids:
            d["eos_token_id"] = list(self.stop_ids)
        return d

    # ------------------------------------------------------------------ what the engine asks
    def chat_format(self, tokenizer):
        raise ConfigError("a Dotanex model folder brings no chat format: give the prompt as token ids")

    def with_stop_ids(self, ids):
        return replace(self, stop_ids=tuple(ids))

    def with_context_length(self, n):
        if n is None or n < 0:
            return self
        return replace(self, context_length=min(n, self.max_positions))

    def owners(self):
        """The layers with tensors of their own, in order."""
        return [i for i, lay in enumerate(self.layers) if lay.get("weights_of") is None]

    def run_order(self):
        """Every layer once, in order; a layer with ``weights_of`` runs the named layer's block (each entry of the
        run order has a cache or state of its own)."""
        block_of = {i: n for n, i in enumerate(self.owners())}
        return tuple(Run(layer=block_of[i if lay.get("weights_of") is None else lay["weights_of"]])
                     for i, lay in enumerate(self.layers))

    def _mixer(self, i, lay):
        d, eps, p, m = self.width, self.norm_eps, f"l{i}.mix.", lay["mixer"]
        top = self.max_position_embeddings
        if lay["type"] == "lightning":
            return RetentionSpec(
                hidden=d, n_heads=m["heads"], key_dim=m["dim"], value_dim=m["vdim"], decay=tuple(float(v) for v in m["decay"]),
                position=None, norm_eps=eps, key_scale=LIGHTNING_KEY_SCALE, input_activation="silu", norm_over="all",
                gate_activation="sigmoid",
                names={"q": p + "q", "k": p + "k", "v": p + "v", "g": p + "g", "o": p + "o", "norm": p + "norm"})
        if lay["type"] == "latent_attention":
            base, dims, sc = _rot(m, m["rot_dim"], "", ())
            scaling = (YarnRopeScaling(float(sc["factor"]), int(sc["original"]), float(sc["fast"]), float(sc["slow"]))
                       if sc is not None else None)
            return LatentAttentionSpec(
                hidden=d, n_heads=m["heads"], head_dim=m["dim"], rot_dim=m["rot_dim"], v_head_dim=m["vdim"],
                q_rank=m["q_rank"], kv_rank=m["kv_rank"], scale=float(m["scale"]), norm_eps=eps,
                position=RotarySpec(head_dim=dims, theta=base, scaling=scaling, pairing=LATENT_PAIRING, max_positions=top),
                names={"dq": p + "dq", "dq_norm": p + "dq.norm", "uq": p + "uq", "dkv": p + "dkv", "dkv_norm": p + "dkv.norm",
                       "uk": p + "uk", "uv": p + "uv", "g": p + "g", "o": p + "o"})
        base, dims, sc = _rot(m, m["dim"], "", ())
        scaling = (Llama3RopeScaling(float(sc["factor"]), float(sc["low"]), float(sc["high"]), int(sc["original"]))
                   if sc is not None else None)
        return AttentionSpec(
            hidden=d, n_heads=m["heads"], n_kv_heads=m["kv_heads"], head_dim=m["dim"],
            position=RotarySpec(head_dim=dims, theta=base, scaling=scaling, pairing=WINDOW_PAIRING, max_positions=top),
            window=m["mask"]["size"] if m.get("mask") is not None else None, scale=float(m["scale"]), qk_norm_eps=eps,
            values_are_keys=True,
            names={"q": p + "q", "k": p + "k", "o": p + "o", "q_norm": p + "q.norm", "k_norm": p + "k.norm", "sink": p + "sink"})

    def _ffn(self, i, mlp):
        d, q = self.width, f"l{i}.mlp."
        if mlp["kind"] == "dense":
            return GatedFeedForwardSpec(hidden=d, intermediate=mlp["ff"], activation=DENSE_ACTIVATION,
                                        names={"gate": q + "gate", "up": q + "up", "down": q + "down"})

        def expert(e):
            return ExpertSpec(e["ff"], EXPERT_ACTIVATION, gated=True,
                              limit=float(e["limit"]) if e.get("limit") is not None else None, up_shift=EXPERT_UP_SHIFT)

        names = {"router": q + "router", "correction": q + "correction", "expert_gate": q + "e{e}.gate",
                 "expert_up": q + "e{e}.up", "expert_down": q + "e{e}.down"}
        shared = mlp.get("shared")
        if shared is not None:
            names.update({"shared_gate": q + "shared.gate", "shared_up": q + "shared.up", "shared_down": q + "shared.down"})
        r = mlp["router"]
        return RoutedFeedForwardSpec(
            hidden=d, n_experts=r["experts"], top=r["top"], expert=expert(mlp["expert"]),
            shared=expert(shared) if shared is not None else None, names=names, weights="scores",
            sum_eps=WEIGHT_SUM_EPS, n_identity=int(r.get("identity") or 0))

    def model_spec(self):
        d, eps = self.width, self.norm_eps
        streams = self.streams

        def norm(name):
            return NormSpec(dim=d, eps=eps, names={"weight": name})

        blocks, unused = [], []
        for i in self.owners():
            lay, p = self.layers[i], f"l{i}."
            mlp = lay.get("mlp")
            stream_names = {}
            if streams is not None:
                stream_names = {f"mixer_{k}": f"{p}hc1.{k}" for k in ("in", "mix", "out")}
                if mlp is not None:
                    stream_names.update({f"ffn_{k}": f"{p}hc2.{k}" for k in ("in", "mix", "out")})
                else:       # (a folder may hold the numbers of a feed-forward that the layer does not have)
                    unused += [f"{p}hc2.{k}" for k in ("in", "mix", "out")]
            if mlp is None:
                unused.append(p + "norm2")
            blocks.append(BlockSpec(
                kind="streams" if streams is not None else "prenorm", mixer_norm=norm(p + "norm1"),
                mixer=self._mixer(i, lay), ffn_norm=norm(p + "norm2") if mlp is not None else None,
                ffn=self._ffn(i, mlp) if mlp is not None else None, streams=streams or 1, stream_names=stream_names))
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden=d, layers=tuple(blocks),
            run_order=self.run_order(), final_norm=norm("final.norm"), max_positions=self.max_position_embeddings,
            tie_embeddings=False, embedding_name="embed", head_name="head", stop_ids=self.stop_ids,
            unused_tensor_names=tuple(unused), streams=streams or 1)


register_architecture("Dotanex", DotanexConfiguration)

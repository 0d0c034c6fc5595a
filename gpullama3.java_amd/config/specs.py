"""Descriptions of model parts as plain data.

A model is described without any tensor: a list of block descriptions (each
naming its norm, mixer and feed-forward with every size and constant), the order
in which the blocks run, and the names under which each part's tensors are
stored. The parts of ``parts/`` are built from these and from nothing else, so
no part knows which architecture it serves.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional


@dataclass(frozen=True)
class Llama3RopeScaling:
    """Frequency scaling of long wavelengths (the reference fixes the four numbers in
    code, J/model/loader/ModelLoader.java:235-239; here they come from config.json)."""
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position: int


@dataclass(frozen=True)
class LinearRopeScaling:
    """Every frequency divided by ``factor`` (positions read as ``factor`` times closer together)."""
    factor: float


@dataclass(frozen=True)
class YarnRopeScaling:
    """Pairs that turn fast keep their frequency, pairs that turn slowly have it divided by ``factor``, with a linear
    ramp over the pair's number in between: from the (fractional, rounded down) number of the pair whose wave makes
    ``fast`` turns over ``original_max_position`` positions to the (rounded up) one that makes ``slow`` turns. cos and
    sin are multiplied by ``0.1 ln(factor) + 1``."""
    factor: float
    original_max_position: int
    fast: float
    slow: float


@dataclass(frozen=True)
class RotarySpec:
    """Rotary position encoding of queries and keys."""
    kind: str = "rotary"
    head_dim: int = 0
    theta: float = 10000.0
    scaling: object = None       # None, a Llama3RopeScaling, a LinearRopeScaling or a YarnRopeScaling
    pairing: str = "half"        # "half": (j, j + hs/2); "adjacent": (2j, 2j+1)
    max_positions: int = 0


@dataclass(frozen=True)
class NormSpec:
    """``x / sqrt(mean(x^2) + eps) * (weight_offset + w)``: a weight stored around zero has ``weight_offset`` 1."""
    kind: str = "rmsnorm"
    dim: int = 0
    eps: float = 1e-5
    names: dict = field(default_factory=dict)     # local tensor name -> stored name
    weight_offset: float = 0.0


@dataclass(frozen=True)
class LayerNormSpec:
    """``(x - mean(x)) / sqrt(var(x) + eps) * w + b`` with the variance as the mean of the squared deviations."""
    kind: str = "layernorm"
    dim: int = 0
    eps: float = 1e-5
    names: dict = field(default_factory=dict)     # "weight", "bias" -> stored names


@dataclass(frozen=True)
class Differential:
    """Differential attention: every head has two score maps (queries and keys of their own, the same values); the
    head's output is ``a1 - lambda * a2`` divided by its root mean square (``norm_eps`` inside the root) times
    ``1 - offset``, with ``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + offset`` from four stored vectors of the keys'
    size (names ``lambda_q1``, ``lambda_k1``, ``lambda_q2``, ``lambda_k2`` of the attention). The stored rows of q and
    k lie head by head as [map 1, map 2]."""
    offset: float = 0.0
    norm_eps: float = 1e-5


@dataclass(frozen=True)
class DistanceBias:
    """A bias on the attention scores that grows with the distance: head h of H takes
    ``slope_h * (i - j)`` off the score of query i and key j, ``slope_h = base ** (-exponent * (h + 1) / H)``."""
    base: float = 2.0
    exponent: float = 8.0

    def slopes(self, n_heads):
        return [self.base ** (-self.exponent * (h + 1) / n_heads) for h in range(n_heads)]


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a cache of keys and values. Names ``q_bias``, ``k_bias``,
    ``v_bias`` (together) and ``o_bias`` among ``names`` add biases to the projections."""
    kind: str = "attention"
    hidden: int = 0
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0
    position: Optional[RotarySpec] = None
    window: Optional[int] = None      # None: every earlier key; n: the last n keys
    scale: Optional[float] = None     # None: 1/sqrt(head_dim)
    names: dict = field(default_factory=dict)
    v_head_dim: Optional[int] = None  # the values' size; None: the keys'
    distance_bias: Optional[DistanceBias] = None
    sink: Optional[float] = None      # the score of a key without a value that every query sees (it takes its share
                                      # of the softmax's weights and adds nothing); None: no such key
    out_scale_name: Optional[str] = None   # a stored [hidden] vector that the mixer's output is multiplied by
    keep_first: int = 0               # with a window: the first n positions of a sequence stay visible to every later query
    value_position: Optional[RotarySpec] = None   # values are rotated by their own position before they are cached (over the
                                      # whole value head), and each head's output is turned back by the query's position
    out_mult: float = 1.0             # a constant that the mixer's output is multiplied by
    qk_norm_eps: Optional[float] = None   # queries and keys are divided by their root mean square per head (this eps
                                      # inside the root) and multiplied by the stored [head_dim] weights ``q_norm`` /
                                      # ``k_norm`` (shared by the heads) before the rotation; None: no such norm
    chunk: Optional[int] = None       # n: query i sees key j <= i only if i // n == j // n (chunks count from position 0)
    differential: Optional[Differential] = None
    values_are_keys: bool = False     # no value projection: a position's values are its keys as projected (before the
                                      # norm on keys and the rotation); ``names`` then has no ``v``
    # (a name ``sink`` among ``names``: a stored [n_heads] vector, a learned sink per query head in place of ``sink``)
    # (no ``k`` among ``names``: the mixer has no keys and values of its own and only ever reads another entry's)
    # (a name ``head_gate`` among ``names``: a stored [n_heads, hidden] matrix; head h's output is multiplied by
    # sigmoid of its row's product with the mixer's input, before the output projection)


@dataclass(frozen=True)
class MinGRUSpec:
    """A gated recurrence per channel whose gates read the current token alone (``parts/mingru.py``):
    ``S <- (1 - z) S + z c`` with z = sigmoid(W_z h + b_z), c = g(W_x h + b_x), g(u) = u + 1/2 for u >= 0 and
    sigmoid(u) below; the output projection reads ``S * silu(W_g h)``."""
    kind: str = "mingru"
    hidden: int = 0
    width: int = 0
    names: dict = field(default_factory=dict)
    out_mult: float = 1.0


@dataclass(frozen=True)
class TimeMixSpec:
    """A matrix per head [head_dim, head_dim] in 32-bit that every token decays per key channel and adds its
    key-value product to; the read-out sees the current token's product times a learned bonus per channel
    (``parts/time_mix.py``). Every projection reads its own blend of the token's input and the previous token's."""
    kind: str = "time_mix"
    hidden: int = 0
    n_heads: int = 0
    head_dim: int = 0
    decay_rank: int = 0               # the inner size of the decay's two-step projection
    norm_eps: float = 1e-5            # the read-out's norm per head
    names: dict = field(default_factory=dict)
    out_mult: float = 1.0


@dataclass(frozen=True)
class SideBySideSpec:
    """Two mixers that read the same input; each one's output is normalised over the model width with a weight of its
    own, and ``weight`` times their sum is the mixer's output (``parts/side_by_side.py``)."""
    kind: str = "side_by_side"
    hidden: int = 0
    left: object = None
    right: object = None
    norm_eps: float = 1e-5
    weight: float = 0.5
    names: dict = field(default_factory=dict)     # "left_norm", "right_norm": the stored [hidden] weights
    out_mult: float = 1.0
    normalised: bool = True           # False: the mixer's output is the plain sum of the sides' outputs (each side
                                      # carries its own factor as its ``out_mult``); no norms, no weights


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Causal attention whose keys and values are expanded from one latent per position (``parts/latent_attention.py``).
    Queries: ``c_q = RMSnorm(W_dq h)`` (``q_rank`` elements), ``q = W_uq c_q``, per head [``head_dim`` unrotated |
    ``rot_dim`` rotated]. ``W_dkv h`` gives the latent c (``kv_rank``, RMS-normed) and ``rot_dim`` more elements, one
    rotated key part for all heads. Per head the unrotated key is ``W_uk c`` and the value ``W_uv c``
    (``v_head_dim``); score = (q . k over both parts) * ``scale``; an ordinary softmax; the heads' outputs times
    sigmoid of a gate projection of the mixer's input; output projection. Only c and the rotated part are cached."""
    kind: str = "latent_attention"
    hidden: int = 0
    n_heads: int = 0
    head_dim: int = 0
    rot_dim: int = 0
    v_head_dim: int = 0
    q_rank: int = 0
    kv_rank: int = 0
    scale: float = 1.0
    position: Optional[RotarySpec] = None      # over the rot_dim part
    norm_eps: float = 1e-5
    names: dict = field(default_factory=dict)  # "dq", "dq_norm", "uq", "dkv", "dkv_norm", "uk", "uv", "g", "o"
    out_mult: float = 1.0


@dataclass(frozen=True)
class RetentionSpec:
    """Linear attention with a fixed decay per head and no softmax (``parts/retention.py``): per head a matrix
    S [key_dim, value_dim] in 32-bit, ``S <- decay_h S + k v^T`` with k times ``key_dim ** -0.5``, ``o = S^T q``; q and
    k are rotated like an attention's. Each head's read-out is divided by its root mean square, the heads together are
    multiplied by silu of a gate projection, then the output projection."""
    kind: str = "retention"
    hidden: int = 0
    n_heads: int = 0
    key_dim: int = 0
    value_dim: int = 0
    decay: tuple = ()                 # one factor per head
    position: Optional[RotarySpec] = None
    norm_eps: float = 1e-5
    names: dict = field(default_factory=dict)     # "q", "k", "v", "g", "o" (and "norm", see ``norm_over``)
    out_mult: float = 1.0
    # what other linear attentions of this form change:
    key_scale: Optional[float] = None     # the factor on k; None: key_dim ** -0.5
    input_activation: Optional[str] = None    # "silu": q, k and v pass silu behind their projections
    norm_over: str = "head"               # "head": each head's read-out divided by its root mean square; "all": the heads'
                                          # read-outs together, times the stored weight ``norm`` [n_heads value_dim]
    gate_activation: str = "silu"         # "silu" or "sigmoid" of the gate projection


@dataclass(frozen=True)
class StateSpaceSpec:
    """A selective state space with a scalar decay per head and token (``parts/state_space.py``): one projection gives
    [z | x | B | C | dt]; x, B and C pass a causal convolution of ``conv_taps`` taps per channel and silu; per head
    (``n_heads`` heads of ``head_dim`` share ``n_groups`` B and C of ``state_dim``) ``S <- exp(-exp(A_log) dt) S + dt B
    x^T``, ``y = S^T C + D x`` with ``dt = softplus(dt + dt_bias)``; y times silu(z), divided by its root mean square in
    ``norm_groups`` equal parts, times a weight, then the output projection."""
    kind: str = "state_space"
    hidden: int = 0
    n_heads: int = 0
    head_dim: int = 0
    n_groups: int = 1
    state_dim: int = 0
    conv_taps: int = 4
    norm_groups: int = 1
    norm_eps: float = 1e-5
    names: dict = field(default_factory=dict)     # "in", "conv", "conv_bias", "dt_bias", "A_log", "D", "norm", "o"
    out_mult: float = 1.0


@dataclass(frozen=True)
class GatedDeltaSpec:
    """The gated delta rule: per value head a matrix [key_dim, value_dim] in 32-bit that every token decays,
    corrects towards its value along its key, and reads with its query (``parts/delta.py``). ``n_heads`` value
    heads share ``n_kv_heads`` query/key heads; q, k and v pass a causal convolution of ``conv_taps`` taps."""
    kind: str = "gated_delta"
    hidden: int = 0
    n_heads: int = 0
    n_kv_heads: int = 0
    key_dim: int = 0
    value_dim: int = 0
    conv_taps: int = 1
    unit_eps: float = 1e-6            # inside the root when q and k are scaled to unit length
    norm_eps: float = 1e-5            # the read-out's norm
    names: dict = field(default_factory=dict)
    out_scale_name: Optional[str] = None


@dataclass(frozen=True)
class GatedFeedForwardSpec:
    """down(act(gate(x)) * (up(x) + up_shift)); ``activation``: "silu", "gelu_tanh" or "quick_gelu"
    (z * sigmoid(1.702 z)). A ``limit`` bounds the gate from above and the up value on both sides before
    that. Names ``gate_bias`` and ``up_bias`` (together) and ``down_bias`` among ``names`` add biases to the products."""
    kind: str = "gated"
    hidden: int = 0
    intermediate: int = 0
    activation: str = "silu"
    names: dict = field(default_factory=dict)
    limit: Optional[float] = None
    up_shift: float = 0.0
    out_scale_name: Optional[str] = None   # a stored [hidden] vector that the output is multiplied by
    out_mult: float = 1.0                  # a constant that the output is multiplied by


@dataclass(frozen=True)
class ExpertSpec:
    """One small feed-forward. Without a gate: ``down(act(up h))``; ``activation`` "gelu" (the erf form), "gelu_tanh"
    or "silu". ``gated``: ``down(act(min(gate h, limit)) * (clamp(up h, -limit, limit) + up_shift))`` with
    ``activation`` one of the gated feed-forward's ("silu", "gelu_tanh", "quick_gelu"); ``limit`` None: unbounded."""
    intermediate: int = 0
    activation: str = "gelu"
    gated: bool = False
    limit: Optional[float] = None
    up_shift: float = 0.0


@dataclass(frozen=True)
class RoutedFeedForwardSpec:
    """A mixture of experts (``parts/routed.py``): router logits in 32-bit, the ``top`` largest choose a token's
    experts, their weights are the softmax over the chosen logits alone; ``shared`` (an ``ExpertSpec`` or None) runs
    for every token and is added. Stored names: ``router`` [experts, hidden]; ``expert_up`` / ``expert_down`` are
    patterns with ``{e}`` for the expert's number; ``shared_up`` / ``shared_down``."""
    kind: str = "routed"
    hidden: int = 0
    n_experts: int = 0
    top: int = 1
    expert: ExpertSpec = None
    shared: Optional[ExpertSpec] = None
    names: dict = field(default_factory=dict)
    out_mult: float = 1.0
    # Another rule for the choice (``weights = "scores"``): s = softmax of the router's outputs over ALL experts; the
    # ``top`` largest of s + the stored ``correction`` are chosen; their weights are their s divided by the chosen s'
    # sum plus ``sum_eps``. "chosen_softmax": the softmax over the chosen logits alone.
    weights: str = "chosen_softmax"
    sum_eps: float = 0.0
    n_identity: int = 0               # the router's last outputs stand for experts whose output is their input (no tensors);
                                      # the router has n_experts + n_identity rows
    # (names: ``expert_gate`` beside ``expert_up`` / ``expert_down`` for gated experts, ``shared_gate``; ``correction``)


@dataclass(frozen=True)
class BlockSpec:
    """One layer: how norm, mixer and feed-forward are arranged is ``kind``. "prenorm": x += mixer(norm(x));
    x += ffn(norm(x)). "parallel": h = mixer_norm(x); x += mixer(h) + ffn(h) (one norm, ``ffn_norm`` is None).
    "outnorm": x += mixer_norm(mixer(x)); x += ffn_norm(ffn(x)): the sublayers read the rows themselves, the norms
    stand behind them. "streams": every token has ``ModelSpec.streams`` copies x_1 .. x_S of its row; a sublayer reads
    norm(sum_s in[s] x_s) and its output y goes back as x_r <- sum_s mix[s, r] x_s + out[r] y (all r at once); the
    numbers are stored per sublayer under ``stream_names`` ("mixer_in" [S], "mixer_mix" [S, S], "mixer_out" [S], and
    the same with "ffn_")."""
    kind: str = "prenorm"
    mixer_norm: object = None
    mixer: object = None
    ffn_norm: object = None
    ffn: object = None
    streams: int = 1
    stream_names: dict = field(default_factory=dict)


@dataclass(frozen=True)
class Run:
    """One entry of the run order.

    ``layer`` indexes ``ModelSpec.layers``. A layer may be named by several
    entries; each entry then has storage of its own in the cache, unless
    ``reads`` names an earlier entry of the run order, whose keys and values this
    entry reads instead of making its own.
    """
    layer: int
    reads: Optional[int] = None
    before: object = None                 # an Inject or a Remix: what happens to the residual rows right before this entry runs


@dataclass(frozen=True)
class Inject:
    """Added to every token's residual row: the embedding's output (the rows as they were before the first
    block) when ``embedding``, then row ``row`` of the stored table ``vector_name`` ([rows, hidden]) if named."""
    embedding: bool = False
    vector_name: Optional[str] = None
    vector_rows: int = 0
    row: int = 0


@dataclass(frozen=True)
class Remix:
    """The residual rows are replaced by a learned mixture of themselves and the embedding's output:
    ``x <- W [x; x0]`` with the stored matrix ``weight_name`` ([hidden, 2 hidden], the columns for x first)."""
    weight_name: str = ""


@dataclass(frozen=True)
class PairEmbedding:
    """A second embedding row per token, looked up by a hash of (previous token, token):
    row ``(previous * mul_prev + token * mul_cur) mod buckets`` of the stored table ``table_name``
    ([buckets + 1, hidden]); a sequence's first token takes the last row. The previous token is kept per sequence."""
    table_name: str = ""
    buckets: int = 0
    mul_prev: int = 0
    mul_cur: int = 0


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden: int
    layers: tuple
    run_order: tuple
    final_norm: object                # the norm in front of the head; None: the head reads the rows as they are
    max_positions: int
    tie_embeddings: bool
    embedding_name: str
    head_name: Optional[str]          # None when tied
    stop_ids: tuple = ()
    # what other decoders put around the blocks; the reference's model has none of them
    # (J/inference/InferenceCore.java:69, :175-177):
    embedding_scale: Optional[float] = None       # the embedding row times this
    position_table_name: Optional[str] = None     # a stored [max_positions, hidden] table whose row at the token's position is added to it
    logit_scale: Optional[float] = None           # the logits times this
    head_bias_name: Optional[str] = None          # a stored [vocab] vector added to the logits (before the scale)
    logit_softcap: Optional[float] = None         # the logits become cap * tanh(logits / cap) (after the scale)
    unused_tensor_names: tuple = ()               # stored names that a folder may hold although nothing reads them
    pair_embedding: Optional[PairEmbedding] = None   # a row per (previous token, token) added to the embedding's output
    streams: int = 1                              # copies of the residual row per token (blocks of kind "streams"); all
                                                  # start as the embedding's output, and their sum goes to the final norm

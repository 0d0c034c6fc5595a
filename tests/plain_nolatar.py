"""A plain, slow implementation of the Nolatar decoder in numpy float64, one function per mechanism, written from
the design's equations and sharing nothing with the package: what the GPU tests compare the engine with.

Notation: T tokens of ONE sequence; W maps a stored tensor name to a float array; linear weights are [out, in].
A ``Sequence`` keeps what the design carries from token to token (keys and values, recurrent states, the short
convolution's last inputs) and can be fed in pieces.

The decoder: ``x = E[token]``; every layer is ``x += LN1(mixer(x))`` then ``x += LN2(ffn(x))`` (the sublayers read
x itself, the layer norms with weight and bias stand behind them); final layer norm, head.
"""
from __future__ import annotations

import math

import numpy as np


# ----------------------------------------------------------------- small functions
def layer_norm(x, w, b, eps):
    x = np.asarray(x, np.float64)
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * np.asarray(w, np.float64) + np.asarray(b, np.float64)


def rms_unit(x, eps):
    x = np.asarray(x, np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_erf(z):
    z = np.asarray(z, np.float64)
    return 0.5 * z * (1.0 + np.vectorize(math.erf)(z / math.sqrt(2.0)))


def linear(x, w):
    return np.asarray(x, np.float64) @ np.asarray(w, np.float64).T


def softmax(s):
    e = np.exp(s - s.max())
    return e / e.sum()


# ----------------------------------------------------------------- rotation
def turn(x, positions, base, dims, pairing):
    """x [T, heads, D]: the first ``dims`` elements of every head in pairs, (i, i + dims/2) for "half" and
    (2i, 2i + 1) for "adjacent"; pair i of the token at position p turns by p * base^(-2i/dims). The rest passes."""
    x = np.array(x, np.float64)
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)])
    a = np.asarray(positions, np.float64)[:, None] * f[None, :]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    if pairing == "half":
        i0, i1 = np.arange(half), np.arange(half) + half
    else:
        i0, i1 = 2 * np.arange(half), 2 * np.arange(half) + 1
    u, v = x[..., i0].copy(), x[..., i1].copy()
    x[..., i0] = u * c - v * s
    x[..., i1] = v * c + u * s
    return x


# ----------------------------------------------------------------- attention
def sees(i, j, chunk):
    """Causal; with a chunk size, only keys of the query's own chunk (chunks are counted from position 0)."""
    return j <= i and (chunk is None or i // chunk == j // chunk)


def softmax_attention(q, keys, values, first, scale, chunk):
    """q [T, H, D] for positions first .. first+T-1; keys [n, G, D], values [n, G, Dv] of positions 0 .. n-1.
    Query head h reads key/value head h // (H / G). Returns [T, H, Dv]."""
    T, H, _ = q.shape
    G = keys.shape[1]
    out = np.zeros((T, H, values.shape[2]))
    for t in range(T):
        i = first + t
        js = [j for j in range(i + 1) if sees(i, j, chunk)]
        for h in range(H):
            g = h // (H // G)
            out[t, h] = softmax(keys[js, g] @ q[t, h] * scale) @ values[js, g]
    return out


def head_norm_rows(x, w, eps):
    """RMS norm over the last axis with a weight shared by all heads."""
    return rms_unit(x, eps) * np.asarray(w, np.float64)


class SoftmaxSide:
    """Grouped attention with a norm on queries and keys per head (before the rotation), a rotation over the first
    elements of a head, and a mask that is causal or chunked. ``maps`` 2: differential attention: two score maps over
    the same values, ``a1 - lambda a2``, a unit norm per head and the factor ``1 - diff``."""

    def __init__(self, c, prefix, eps, pairing, maps=1, shared=None):
        self.c, self.p, self.eps, self.pairing, self.maps = c, prefix, eps, pairing, maps
        self.shared = shared                  # the side whose keys and values this one reads, or None
        self.keys, self.values = None, None

    def forward(self, W, h, first):
        c, p, m = self.c, self.p, self.maps
        T = h.shape[0]
        H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        pos = np.arange(first, first + T)
        rot = c["rot"]
        q = linear(h, W[p + "q"]).reshape(T, H * m, D)
        q = turn(head_norm_rows(q, W[p + "q.norm"], self.eps), pos, rot["base"], rot["dims"], self.pairing)
        if self.shared is None:
            k = linear(h, W[p + "k"]).reshape(T, G * m, D)
            k = turn(head_norm_rows(k, W[p + "k.norm"], self.eps), pos, rot["base"], rot["dims"], self.pairing)
            v = linear(h, W[p + "v"]).reshape(T, G, Dv)
            self.keys = k if self.keys is None else np.concatenate([self.keys, k])
            self.values = v if self.values is None else np.concatenate([self.values, v])
            keys, values = self.keys, self.values
        else:
            keys, values = self.shared.keys, self.shared.values
        chunk = (c.get("mask") or {}).get("size")
        if m == 1:
            o = softmax_attention(q, keys, values, first, c["scale"], chunk)
        else:
            # rows lie head by head as [map 1, map 2]
            q, keys = q.reshape(T, H, 2, D), keys.reshape(-1, G, 2, D)
            a1 = softmax_attention(q[:, :, 0], keys[:, :, 0], values, first, c["scale"], chunk)
            a2 = softmax_attention(q[:, :, 1], keys[:, :, 1], values, first, c["scale"], chunk)
            lam = (math.exp(float(W[p + "lq1"] @ W[p + "lk1"])) - math.exp(float(W[p + "lq2"] @ W[p + "lk2"])) + c["diff"])
            o = rms_unit(a1 - lam * a2, self.eps) * (1.0 - c["diff"])
        return linear(o.reshape(T, H * Dv), W[p + "o"])


# ----------------------------------------------------------------- retention
class RetentionSide:
    """Linear attention with a fixed decay per head: S <- decay S + k v^T, o = S^T q; no softmax, no denominator."""

    def __init__(self, c, prefix, eps):
        self.c, self.p, self.eps = c, prefix, eps
        self.S = np.zeros((c["heads"], c["dim"], c["vdim"]))
        self.conditioning = np.inf            # the smallest |o| / (|S| |q|) of the last call: how much of a read-out survives its sum

    def forward(self, W, h, first):
        c, p = self.c, self.p
        T, H, D, Dv = h.shape[0], c["heads"], c["dim"], c["vdim"]
        self.conditioning = np.inf
        pos = np.arange(first, first + T)
        rot = c["rot"]
        q = turn(linear(h, W[p + "q"]).reshape(T, H, D), pos, rot["base"], rot["dims"], "half")
        k = turn(linear(h, W[p + "k"]).reshape(T, H, D), pos, rot["base"], rot["dims"], "half") * D ** -0.5
        v = linear(h, W[p + "v"]).reshape(T, H, Dv)
        o = np.zeros((T, H, Dv))
        for t in range(T):
            for hd in range(H):
                self.S[hd] = c["decay"][hd] * self.S[hd] + np.outer(k[t, hd], v[t, hd])
                o[t, hd] = self.S[hd].T @ q[t, hd]
                self.conditioning = min(self.conditioning, np.linalg.norm(o[t, hd])
                                        / (np.linalg.norm(self.S[hd]) * np.linalg.norm(q[t, hd]) + 1e-300))
        o = rms_unit(o, self.eps).reshape(T, H * Dv) * silu(linear(h, W[p + "g"]))
        return linear(o, W[p + "o"])


class SideBySide:
    def __init__(self, c, prefix, eps):
        self.c = c
        self.left = SoftmaxSide(c["left"], prefix + "left.", eps, "half")
        self.right = RetentionSide(c["right"], prefix + "right.", eps)

    def forward(self, W, h, first):
        return self.c["left_scale"] * self.left.forward(W, h, first) + self.c["right_scale"] * self.right.forward(W, h, first)


# ----------------------------------------------------------------- state-space mixer
class StateSpace:
    """Mamba-2: one projection gives [z | x | B | C | dt]; x, B, C pass a short causal convolution and silu; per head
    S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x; y * silu(z), a unit norm in equal parts with a weight,
    output projection."""

    def __init__(self, c, prefix, eps):
        self.c, self.p, self.eps = c, prefix, eps
        self.inner = c["heads"] * c["vdim"]
        self.channels = self.inner + 2 * c["groups"] * c["state"]
        self.held = np.zeros((c["conv"] - 1, self.channels))
        self.S = np.zeros((c["heads"], c["state"], c["vdim"]))

    def forward(self, W, h, first):
        c, p = self.c, self.p
        T, H, P, N, G = h.shape[0], c["heads"], c["vdim"], c["state"], c["groups"]
        inner = self.inner
        proj = linear(h, W[p + "in"])
        z, xbc, dt = proj[:, :inner], proj[:, inner:inner + self.channels], proj[:, inner + self.channels:]
        taps = c["conv"]
        rows = np.concatenate([self.held, xbc])                  # the inputs of the last taps - 1 tokens in front
        cw, cb = np.asarray(W[p + "conv"], np.float64), np.asarray(W[p + "conv.b"], np.float64)
        conv = np.stack([(rows[t:t + taps] * cw.T).sum(0) + cb for t in range(T)])
        self.held = rows[T:]
        xbc = silu(conv)
        x = xbc[:, :inner].reshape(T, H, P)
        B = xbc[:, inner:inner + G * N].reshape(T, G, N)
        C = xbc[:, inner + G * N:].reshape(T, G, N)
        dt = softplus(dt + np.asarray(W[p + "dt_bias"], np.float64))
        A = np.exp(np.asarray(W[p + "A_log"], np.float64))
        Dk = np.asarray(W[p + "D"], np.float64)
        y = np.zeros((T, H, P))
        for t in range(T):
            for hd in range(H):
                g = hd // (H // G)
                self.S[hd] = math.exp(-A[hd] * dt[t, hd]) * self.S[hd] + dt[t, hd] * np.outer(B[t, g], x[t, hd])
                y[t, hd] = self.S[hd].T @ C[t, g] + Dk[hd] * x[t, hd]
        y = y.reshape(T, inner) * silu(z)
        parts = c["norm_groups"]
        y = rms_unit(y.reshape(T, parts, inner // parts), self.eps).reshape(T, inner) * np.asarray(W[p + "norm"], np.float64)
        return linear(y, W[p + "o"])


# ----------------------------------------------------------------- feed-forward
def expert(W, prefix, h):
    return linear(gelu_erf(linear(h, W[prefix + "up"])), W[prefix + "down"])


def routed_feed_forward(W, prefix, c, h, margins=None):
    """The ``top`` experts with the largest router logits, weighted with the softmax over the chosen logits alone,
    plus an expert that every token passes. ``margins`` (a list) receives, per token, how far the last chosen logit
    lies from the first one left out, in units of the size that a logit of this router has (the root mean squares
    of h's elements and of the router's rows' lengths multiplied)."""
    logits = linear(h, W[prefix + "router"])
    top = c["router"]["top"]
    rows = []
    for t in range(h.shape[0]):
        order = np.argsort(-logits[t], kind="stable")
        chosen = order[:top]
        if margins is not None and top < len(order):
            size = np.sqrt((h[t] ** 2).mean()) * np.sqrt((np.asarray(W[prefix + "router"], np.float64) ** 2).sum(-1).mean())
            margins.append((logits[t, order[top - 1]] - logits[t, order[top]]) / (size + 1e-300))
        w = softmax(logits[t, chosen])
        rows.append(sum(w[i] * expert(W, f"{prefix}e{e}.", h[t:t + 1])[0] for i, e in enumerate(chosen)))
    y = np.stack(rows)
    if c.get("shared"):
        y = y + expert(W, prefix + "shared.", h)
    return y


# ----------------------------------------------------------------- the decoder
class Sequence:
    """``noise``: every layer's input is multiplied by 1 + noise * N(0, 1) per element, as a 16-bit engine's rounding
    would disturb it: the twin of a sequence that tells how far rounding alone moves its logits."""

    def __init__(self, config, W, noise=0.0, seed=0):
        self.c, self.W = config, {k: np.asarray(v, np.float64) for k, v in W.items()}
        self.noise, self.rng = noise, np.random.default_rng([seed, 123])
        self.eps = config["norm"]["eps"]
        self.n = 0
        self.margin = np.inf                  # the closest call of any router in the last feed
        self.mixers = []
        for i, lay in enumerate(config["layers"]):
            p, m = f"l{i}.mix.", lay["mixer"]
            if lay["type"] == "mamba2":
                self.mixers.append(StateSpace(m, p, self.eps))
            elif lay["type"] == "parallel":
                self.mixers.append(SideBySide(m, p, self.eps))
            elif lay["type"] == "attention":
                shared = self.mixers[m["kv_from"]] if m.get("kv_from") is not None else None
                self.mixers.append(SoftmaxSide(m, p, self.eps, "adjacent", maps=2, shared=shared))
            else:
                raise ValueError(lay["type"])

    def feed(self, tokens):
        """Logits [len(tokens), vocab] and the residual rows after every layer [layers, len(tokens), width]."""
        W, eps = self.W, self.eps
        x = W["embed"][list(tokens)]
        after, margins = [], []
        for i, (lay, mixer) in enumerate(zip(self.c["layers"], self.mixers)):
            p = f"l{i}."
            if self.noise:
                x = x * (1.0 + self.noise * self.rng.standard_normal(x.shape))
            x = x + layer_norm(mixer.forward(W, x, self.n), W[p + "norm1"], W[p + "norm1.b"], eps)
            if lay.get("mlp") is not None:
                x = x + layer_norm(routed_feed_forward(W, p + "mlp.", lay["mlp"], x, margins), W[p + "norm2"], W[p + "norm2.b"], eps)
            after.append(x)
        self.n += len(tokens)
        self.margin = min(margins) if margins else np.inf
        self.conditioning = min([m.right.conditioning for m in self.mixers if isinstance(m, SideBySide)], default=np.inf)
        return linear(layer_norm(x, W["final.norm"], W["final.norm.b"], eps), W["head"]), np.stack(after)


def forward(config, W, tokens):
    """Logits [len(tokens), vocab] of one sequence fed whole."""
    return Sequence(config, W).feed(tokens)[0]


# ----------------------------------------------------------------- weights for the tests
def tensor_shapes(cfg):
    """Stored name -> shape of every tensor a configuration asks for."""
    d = cfg["width"]
    out = {"embed": (cfg["vocab"], d), "head": (cfg["vocab"], d), "final.norm": (d,), "final.norm.b": (d,)}
    for i, lay in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        out[p + "norm1"], out[p + "norm1.b"] = (d,), (d,)
        if lay["type"] == "mamba2":
            inner = m["heads"] * m["vdim"]
            ch = inner + 2 * m["groups"] * m["state"]
            out.update({p + "mix.in": (inner + ch + m["heads"], d), p + "mix.conv": (ch, m["conv"]), p + "mix.conv.b": (ch,),
                        p + "mix.dt_bias": (m["heads"],), p + "mix.A_log": (m["heads"],), p + "mix.D": (m["heads"],),
                        p + "mix.norm": (inner,), p + "mix.o": (d, inner)})
        elif lay["type"] == "parallel":
            L, R = m["left"], m["right"]
            q = p + "mix.left."
            out.update({q + "q": (L["heads"] * L["dim"], d), q + "k": (L["kv_heads"] * L["dim"], d),
                        q + "v": (L["kv_heads"] * L["vdim"], d), q + "q.norm": (L["dim"],), q + "k.norm": (L["dim"],),
                        q + "o": (d, L["heads"] * L["vdim"])})
            r = p + "mix.right."
            out.update({r + "q": (R["heads"] * R["dim"], d), r + "k": (R["heads"] * R["dim"], d),
                        r + "v": (R["heads"] * R["vdim"], d), r + "g": (R["heads"] * R["vdim"], d),
                        r + "o": (d, R["heads"] * R["vdim"])})
        else:
            q = p + "mix."
            out.update({q + "q": (m["heads"] * 2 * m["dim"], d), q + "q.norm": (m["dim"],), q + "o": (d, m["heads"] * m["vdim"])})
            for k in ("lq1", "lk1", "lq2", "lk2"):
                out[q + k] = (m["dim"],)
            if m.get("kv_from") is None:
                out.update({q + "k": (m["kv_heads"] * 2 * m["dim"], d), q + "v": (m["kv_heads"] * m["vdim"], d),
                            q + "k.norm": (m["dim"],)})
        mlp = lay.get("mlp")
        if mlp is not None:
            out[p + "norm2"], out[p + "norm2.b"] = (d,), (d,)
            q = p + "mlp."
            out[q + "router"] = (mlp["router"]["experts"], d)
            for e in range(mlp["router"]["experts"]):
                out[f"{q}e{e}.up"], out[f"{q}e{e}.down"] = (mlp["expert"]["ff"], d), (d, mlp["expert"]["ff"])
            if mlp.get("shared") is not None:
                out[q + "shared.up"], out[q + "shared.down"] = (mlp["shared"]["ff"], d), (d, mlp["shared"]["ff"])
    return out


def make_weights(cfg, seed):
    """float32 weights that bfloat16 holds exactly, sized so that every mechanism moves the logits: matrices
    N(0, 1.5/sqrt(fan-in)), norm weights around one, biases around zero, step sizes and decays spread widely."""
    import zlib
    import torch
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        rng = np.random.default_rng([seed, zlib.crc32(name.encode())])
        last = name.split(".")[-1]
        if last in ("norm1", "norm2", "norm"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif last == "b":
            a = 0.3 * rng.standard_normal(shape)
        elif last == "dt_bias":
            a = rng.uniform(-3.0, 1.0, shape)
        elif last == "A_log":
            a = rng.uniform(-2.0, 1.0, shape)
        elif last == "D":
            a = 1.0 + 0.3 * rng.standard_normal(shape)
        elif last == "conv":
            a = 0.5 * rng.standard_normal(shape)
        elif last in ("lq1", "lk1", "lq2", "lk2"):
            a = 0.25 * rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) * (1.5 / np.sqrt(shape[-1]))
        out[name] = torch.tensor(a, dtype=torch.float32).to(torch.bfloat16).float().numpy()
    return out


def tokens_with_clear_choices(cfg, W, seed, n, margin=0.1, noise=2.0 ** -8, bound=0.02, conditioning=0.03):
    """n token ids drawn from a seed at which a 16-bit engine has no close call to make. No router's choice is one: at
    every token and layer the last chosen logit and the first one left out lie at least ``margin`` (times a logit's
    size) apart. No retention's read-out is the small rest of a sum that cancels (the first token's is (q . k) v, and
    its unit norm keeps nothing of q . k but the sign): |o| is at least ``conditioning`` times |S| |q|. And no other
    place turns rounding into another result: a twin of the sequence whose layers read inputs disturbed by ``noise``
    stays within ``bound`` of its logits. A bfloat16 engine then differs from the plain implementation by
    rounding, not by another expert or sign."""
    import copy
    rng = np.random.default_rng([seed, 11])
    seq, twin, out = Sequence(cfg, W), Sequence(cfg, W, noise=noise, seed=seed), []
    while len(out) < n:
        for _ in range(400):
            t = int(rng.integers(0, cfg["vocab"]))
            trial, trial_twin = copy.deepcopy(seq), copy.deepcopy(twin)
            a, b = trial.feed([t])[0][0], trial_twin.feed([t])[0][0]
            d = (b - b.mean()) - (a - a.mean())
            if trial.margin >= margin and trial.conditioning >= conditioning and np.sqrt((d * d).mean()) < bound * np.sqrt(((a - a.mean()) ** 2).mean()):
                break
        else:
            raise RuntimeError("no token without a close call found")
        seq, twin = trial, trial_twin
        out.append(t)
    return out

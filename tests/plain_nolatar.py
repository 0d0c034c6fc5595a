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

    def forward(self, W, h, first):
        c, p = self.c, self.p
        T, H, D, Dv = h.shape[0], c["heads"], c["dim"], c["vdim"]
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


def routed_feed_forward(W, prefix, c, h):
    """The ``top`` experts with the largest router logits, weighted with the softmax over the chosen logits alone,
    plus an expert that every token passes."""
    out = np.zeros((h.shape[0], np.asarray(W[prefix + "shared.down"]).shape[0])) if c.get("shared") else None
    logits = linear(h, W[prefix + "router"])
    top = c["router"]["top"]
    rows = []
    for t in range(h.shape[0]):
        chosen = np.argsort(-logits[t], kind="stable")[:top]
        w = softmax(logits[t, chosen])
        rows.append(sum(w[i] * expert(W, f"{prefix}e{e}.", h[t:t + 1])[0] for i, e in enumerate(chosen)))
    y = np.stack(rows)
    if c.get("shared"):
        y = y + expert(W, prefix + "shared.", h)
    return y


# ----------------------------------------------------------------- the decoder
class Sequence:
    def __init__(self, config, W):
        self.c, self.W = config, {k: np.asarray(v, np.float64) for k, v in W.items()}
        self.eps = config["norm"]["eps"]
        self.n = 0
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
        after = []
        for i, (lay, mixer) in enumerate(zip(self.c["layers"], self.mixers)):
            p = f"l{i}."
            x = x + layer_norm(mixer.forward(W, x, self.n), W[p + "norm1"], W[p + "norm1.b"], eps)
            if lay.get("mlp") is not None:
                x = x + layer_norm(routed_feed_forward(W, p + "mlp.", lay["mlp"], x), W[p + "norm2"], W[p + "norm2.b"], eps)
            after.append(x)
        self.n += len(tokens)
        return linear(layer_norm(x, W["final.norm"], W["final.norm.b"], eps), W["head"]), np.stack(after)

"""A plain, slow implementation of the Dotanex decoder in numpy float64, one function per mechanism, written from
the design's equations and sharing nothing with the package: what the GPU tests compare the engine with.

Notation: T tokens of ONE sequence; W maps a stored tensor name to a float array; linear weights are [out, in].
A ``Sequence`` keeps what the design carries from token to token (keys and values, latents, recurrent states) and can
be fed in pieces.

The decoder keeps ``streams`` copies of the residual row per token. A sublayer reads a learned mixture of the copies
through an RMS norm, and its output goes back into every copy with a factor of its own while the copies are mixed among
themselves. The mixers: a linear attention with a fixed decay per head ("lightning"), a causal attention whose keys
and values are expanded from one small latent per position ("latent_attention"), and a windowed attention whose values
are its keys and whose softmax has a learned sink per head ("attention"). The feed-forward is a gated one or a mixture
of gated experts with identity experts among them.
"""
from __future__ import annotations

import math

import numpy as np


# ----------------------------------------------------------------- small functions
def rms_unit(x, eps):
    x = np.asarray(x, np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * np.asarray(w, np.float64)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-np.asarray(z, np.float64)))


def silu(z):
    return z * sigmoid(z)


def linear(x, w):
    return np.asarray(x, np.float64) @ np.asarray(w, np.float64).T


# ----------------------------------------------------------------- rotation
def plain_frequencies(base, dims):
    return np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])


def yarn_frequencies(base, dims, sc):
    """Frequencies and the factor on cos and sin. Pairs that turn fast keep their frequency, pairs that turn slowly have
    it divided by ``factor``, with a linear ramp over the pair's number in between; the ramp's ends are the (fractional)
    pair numbers whose wave makes ``fast`` and ``slow`` turns over ``original`` positions."""
    f = plain_frequencies(base, dims)
    if sc is None:
        return f, 1.0

    def pair_of(turns):
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(sc["fast"])), 0)
    hi = min(math.ceil(pair_of(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def wavelength_frequencies(base, dims, sc):
    """Short waves stay, long waves are stretched by ``factor``, and those in between are interpolated by how many
    times they fit into ``original`` positions."""
    f = plain_frequencies(base, dims)
    if sc is None:
        return f
    out = []
    for fi in f:
        wave = 2.0 * math.pi / fi
        if wave < sc["original"] / sc["high"]:
            out.append(fi)
        elif wave > sc["original"] / sc["low"]:
            out.append(fi / sc["factor"])
        else:
            s = (sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])
            out.append((1.0 - s) * fi / sc["factor"] + s * fi)
    return np.array(out)


def turn(x, positions, freqs, pairing, magnitude=1.0):
    """x [T, heads, D]: the first 2 len(freqs) elements of every head in pairs, (i, i + n) for "half" and (2i, 2i + 1)
    for "adjacent"; pair i of the token at position p turns by p * freqs[i]. The rest passes."""
    x = np.array(x, np.float64)
    n = len(freqs)
    a = np.asarray(positions, np.float64)[:, None] * np.asarray(freqs)[None, :]
    c, s = magnitude * np.cos(a)[:, None, :], magnitude * np.sin(a)[:, None, :]
    if pairing == "half":
        i0, i1 = np.arange(n), np.arange(n) + n
    else:
        i0, i1 = 2 * np.arange(n), 2 * np.arange(n) + 1
    u, v = x[..., i0].copy(), x[..., i1].copy()
    x[..., i0] = u * c - v * s
    x[..., i1] = v * c + u * s
    return x


# ----------------------------------------------------------------- mixers
def lightning(h, W, p, m, eps, state):
    """``state``: {"S": [H, D, Dv]} (zeros at a sequence's start), moved on token by token."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(linear(h, W[p + "q"])).reshape(T, H, D)
    k = silu(linear(h, W[p + "k"])).reshape(T, H, D)
    v = silu(linear(h, W[p + "v"])).reshape(T, H, Dv)
    S = state.setdefault("S", np.zeros((H, D, Dv)))
    decay = np.asarray(m["decay"], np.float64)
    o = np.zeros((T, H, Dv))
    for t in range(T):
        S *= decay[:, None, None]
        S += k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    y = rms_norm(o.reshape(T, H * Dv), W[p + "norm"], eps) * sigmoid(linear(h, W[p + "g"]))
    return linear(y, W[p + "o"])


def latent_attention(h, positions, W, p, m, eps, state):
    """``state``: {"c": [n, kv_rank], "r": [n, rot_dim]}: the latents and the shared rotated key parts so far."""
    T = h.shape[0]
    H, D, R, Dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m["rot"]
    freqs, mag = yarn_frequencies(rot["base"], rot["dims"], rot.get("scaling"))
    cq = rms_norm(linear(h, W[p + "dq"]), W[p + "dq.norm"], eps)
    q = linear(cq, W[p + "uq"]).reshape(T, H, D + R)
    q_plain, q_rot = q[..., :D], turn(q[..., D:], positions, freqs, "adjacent", mag)
    down = linear(h, W[p + "dkv"])
    c = rms_norm(down[:, :rank], W[p + "dkv.norm"], eps)
    r = turn(down[:, None, rank:], positions, freqs, "adjacent", mag)[:, 0]
    state["c"] = c if "c" not in state else np.concatenate([state["c"], c])
    state["r"] = r if "r" not in state else np.concatenate([state["r"], r])
    keys = linear(state["c"], W[p + "uk"]).reshape(-1, H, D)
    vals = linear(state["c"], W[p + "uv"]).reshape(-1, H, Dv)
    out = np.zeros((T, H, Dv))
    for t in range(T):
        n = positions[t] + 1
        s = (np.einsum("hd,nhd->hn", q_plain[t], keys[:n]) + q_rot[t] @ state["r"][:n].T) * m["scale"]
        w = np.exp(s - s.max(-1, keepdims=True))
        w /= w.sum(-1, keepdims=True)
        out[t] = np.einsum("hn,nhv->hv", w, vals[:n])
    y = out.reshape(T, H * Dv) * sigmoid(linear(h, W[p + "g"]))
    return linear(y, W[p + "o"])


def window_attention(h, positions, W, p, m, eps, state):
    """``state``: {"k": [n, G, D] normed and turned keys, "v": [n, G, D] the keys as projected}."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    rot = m["rot"]
    freqs = wavelength_frequencies(rot["base"], rot["dims"], rot.get("scaling"))
    q = linear(h, W[p + "q"]).reshape(T, H, D)
    k = linear(h, W[p + "k"]).reshape(T, G, D)
    v = k.copy()
    q = turn(rms_norm(q, W[p + "q.norm"], eps), positions, freqs, "half")
    k = turn(rms_norm(k, W[p + "k.norm"], eps), positions, freqs, "half")
    state["k"] = k if "k" not in state else np.concatenate([state["k"], k])
    state["v"] = v if "v" not in state else np.concatenate([state["v"], v])
    size = (m.get("mask") or {}).get("size")
    sink = np.asarray(W[p + "sink"], np.float64)
    out = np.zeros((T, H, D))
    for t in range(T):
        i = positions[t]
        first = 0 if size is None else max(0, i - size + 1)
        for hh in range(H):
            g = hh // (H // G)
            s = state["k"][first:i + 1, g] @ q[t, hh] * m["scale"]
            top = max(s.max(), sink[hh])
            e = np.exp(s - top)
            out[t, hh] = (e / (e.sum() + math.exp(sink[hh] - top))) @ state["v"][first:i + 1, g]
    return linear(out.reshape(T, H * D), W[p + "o"])


# ----------------------------------------------------------------- feed-forward
def dense(h, W, p):
    return linear(silu(linear(h, W[p + "gate"])) * linear(h, W[p + "up"]), W[p + "down"])


def expert(h, W, p, limit):
    """``limit`` None: unbounded."""
    g, u = linear(h, W[p + "gate"]), linear(h, W[p + "up"])
    if limit is not None:
        g, u = np.minimum(g, limit), np.clip(u, -limit, limit)
    return linear(g * sigmoid(1.702 * g) * (u + 1.0), W[p + "down"])


def route(h, W, p, mlp):
    """Per token the chosen experts and their weights: softmax over all router outputs, the choice by score plus a
    stored correction, the weights from the scores themselves divided by their sum."""
    z = linear(h, W[p + "router"])
    s = np.exp(z - z.max(-1, keepdims=True))
    s /= s.sum(-1, keepdims=True)
    choice = s + np.asarray(W[p + "correction"], np.float64)
    top = mlp["router"]["top"]
    idx = np.argsort(-choice, axis=-1, kind="stable")[:, :top]
    w = np.take_along_axis(s, idx, -1)
    return idx, w / (w.sum(-1, keepdims=True) + 1e-20), choice


def mixture(h, W, p, mlp, note=None):
    """``note`` (a list) receives, per token, how far the last chosen expert's choice score lies above the first one
    left out."""
    n_real = mlp["router"]["experts"]
    idx, w, choice = route(h, W, p, mlp)
    if note is not None and choice.shape[-1] > mlp["router"]["top"]:
        ranked = -np.sort(-choice, axis=-1)
        note.extend((ranked[:, mlp["router"]["top"] - 1] - ranked[:, mlp["router"]["top"]]).tolist())
    out = np.zeros_like(h, dtype=np.float64)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t], w[t]):
            out[t] += a * (h[t] if e >= n_real else expert(h[t:t + 1], W, f"{p}e{e}.", mlp["expert"].get("limit"))[0])
    if mlp.get("shared") is not None:
        out += expert(h, W, p + "shared.", mlp["shared"].get("limit"))
    return out


def feed_forward(h, W, p, mlp, note=None):
    return dense(h, W, p) if mlp["kind"] == "dense" else mixture(h, W, p, mlp, note)


# ----------------------------------------------------------------- the decoder
def owner(cfg, i):
    """The layer whose tensors layer i uses."""
    return cfg["layers"][i].get("weights_of", i)


class Sequence:
    """One sequence that is fed in pieces. ``rows`` collects, per piece, the residual rows (the copies' sum) after
    every layer; ``after`` (optional) is called with (layer, sublayer name, the copies [T, streams, d])."""

    def __init__(self, cfg, W, after=None):
        self.cfg, self.W, self.after = cfg, {k: np.asarray(v, np.float64) for k, v in W.items()}, after
        self.n = 0
        self.states = [dict() for _ in cfg["layers"]]
        self.rows = []
        self.gaps = []          # of every router's choices so far (``mixture``)

    def _sublayer(self, xs, p, q, fn):
        """One sublayer under the copies' mixing: xs [T, streams, d] -> the new copies."""
        W, eps = self.W, self.cfg["norm"]["eps"]
        if "streams" not in self.cfg:
            return xs + fn(rms_norm(xs[:, 0], W[f"{p}norm{q}"], eps))[:, None, :]
        u = np.einsum("s,tsd->td", W[f"{p}hc{q}.in"], xs)
        y = fn(rms_norm(u, W[f"{p}norm{q}"], eps))
        return np.einsum("sr,tsd->trd", W[f"{p}hc{q}.mix"], xs) + W[f"{p}hc{q}.out"][None, :, None] * y[:, None, :]

    def feed(self, tokens):
        cfg, W, eps = self.cfg, self.W, self.cfg["norm"]["eps"]
        T = len(tokens)
        positions = np.arange(self.n, self.n + T)
        self.n += T
        xs = np.repeat(W["embed"][np.asarray(tokens)][:, None, :], cfg.get("streams", 1), axis=1)
        rows = []
        for i, lay in enumerate(cfg["layers"]):
            p, m, st = f"l{owner(cfg, i)}.", lay["mixer"], self.states[i]
            if lay["type"] == "lightning":
                mix = lambda h: lightning(h, W, p + "mix.", m, eps, st)
            elif lay["type"] == "latent_attention":
                mix = lambda h: latent_attention(h, positions, W, p + "mix.", m, eps, st)
            else:
                mix = lambda h: window_attention(h, positions, W, p + "mix.", m, eps, st)
            xs = self._sublayer(xs, p, 1, mix)
            if self.after:
                self.after(i, "mixer", xs)
            if lay.get("mlp") is not None:
                xs = self._sublayer(xs, p, 2, lambda h: feed_forward(h, W, p + "mlp.", lay["mlp"], self.gaps))
                if self.after:
                    self.after(i, "ffn", xs)
            rows.append(xs.sum(1))
        self.rows.append(np.stack(rows))
        x = rms_norm(xs.sum(1), W["final.norm"], eps)
        return linear(x, W["head"])


def forward(cfg, W, tokens):
    """Logits [T, vocab] of one sequence fed whole."""
    return Sequence(cfg, W).feed(tokens)


# ----------------------------------------------------------------- models for tests
def tensor_shapes(cfg):
    """Stored name -> shape of every tensor of a model of this design."""
    d, S = cfg["width"], cfg.get("streams")
    out = {"embed": (cfg["vocab"], d), "final.norm": (d,), "head": (cfg["vocab"], d)}
    for i, lay in enumerate(cfg["layers"]):
        if lay.get("weights_of") is not None:
            continue
        p, m, mlp = f"l{i}.", lay["mixer"], lay.get("mlp")
        out[p + "norm1"] = (d,)
        if S is not None:
            out.update({p + "hc1.in": (S,), p + "hc1.mix": (S, S), p + "hc1.out": (S,)})
        H = m["heads"]
        if lay["type"] == "lightning":
            out.update({p + "mix.q": (H * m["dim"], d), p + "mix.k": (H * m["dim"], d), p + "mix.v": (H * m["vdim"], d),
                        p + "mix.g": (H * m["vdim"], d), p + "mix.o": (d, H * m["vdim"]), p + "mix.norm": (H * m["vdim"],)})
        elif lay["type"] == "latent_attention":
            out.update({p + "mix.dq": (m["q_rank"], d), p + "mix.dq.norm": (m["q_rank"],),
                        p + "mix.uq": (H * (m["dim"] + m["rot_dim"]), m["q_rank"]),
                        p + "mix.dkv": (m["kv_rank"] + m["rot_dim"], d), p + "mix.dkv.norm": (m["kv_rank"],),
                        p + "mix.uk": (H * m["dim"], m["kv_rank"]), p + "mix.uv": (H * m["vdim"], m["kv_rank"]),
                        p + "mix.g": (H * m["vdim"], d), p + "mix.o": (d, H * m["vdim"])})
        else:
            out.update({p + "mix.q": (H * m["dim"], d), p + "mix.k": (m["kv_heads"] * m["dim"], d),
                        p + "mix.q.norm": (m["dim"],), p + "mix.k.norm": (m["dim"],), p + "mix.sink": (H,),
                        p + "mix.o": (d, H * m["dim"])})
        if mlp is None:
            continue
        out[p + "norm2"] = (d,)
        if S is not None:
            out.update({p + "hc2.in": (S,), p + "hc2.mix": (S, S), p + "hc2.out": (S,)})
        q = p + "mlp."
        if mlp["kind"] == "dense":
            out.update({q + "gate": (mlp["ff"], d), q + "up": (mlp["ff"], d), q + "down": (d, mlp["ff"])})
            continue
        r = mlp["router"]
        n_all = r["experts"] + r.get("identity", 0)
        out.update({q + "router": (n_all, d), q + "correction": (n_all,)})
        forms = [(f"{q}e{e}.", mlp["expert"]["ff"]) for e in range(r["experts"])]
        if mlp.get("shared") is not None:
            forms.append((q + "shared.", mlp["shared"]["ff"]))
        for pre, ff in forms:
            out.update({pre + "gate": (ff, d), pre + "up": (ff, d), pre + "down": (d, ff)})
    return out


def make_weights(cfg, seed):
    """float32 weights that bfloat16 holds exactly, sized so that every mechanism moves the logits: matrices
    N(0, 1.5/sqrt(fan-in)), norm weights around one, the copies' numbers around an even read and a kept row, sinks
    and corrections of the size of what they stand beside."""
    import zlib
    import torch
    out = {}
    S = cfg.get("streams") or 1
    for name, shape in tensor_shapes(cfg).items():
        rng = np.random.default_rng([seed, zlib.crc32(name.encode())])
        last = name.split(".")[-1]
        if last in ("norm1", "norm2", "norm"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif last == "in":
            a = 1.0 / S + 0.3 * rng.standard_normal(shape)
        elif last == "mix":
            a = np.eye(S) + 0.3 * rng.standard_normal(shape)
        elif last == "out":
            a = 1.0 + 0.3 * rng.standard_normal(shape)
        elif last == "sink":
            a = rng.standard_normal(shape)
        elif last == "correction":
            a = 0.05 * rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) * (1.5 / np.sqrt(shape[-1]))
        out[name] = torch.tensor(a, dtype=torch.float32).to(torch.bfloat16).float().numpy()
    return out


def tokens_with_clear_choices(cfg, W, seed, n, gap=0.05):
    """n token ids drawn from a seed at which no router makes a close call: at every token and layer the last chosen
    expert's choice score lies at least ``gap`` above the first one left out, so an engine that rounds to 16 bits
    chooses the same experts."""
    import copy
    rng = np.random.default_rng([seed, 11])
    seq, out = Sequence(cfg, W), []
    while len(out) < n:
        best = None
        for _ in range(150):
            t = int(rng.integers(0, cfg["vocab"]))
            trial = copy.deepcopy(seq)
            trial.gaps, trial.rows = [], []
            trial.feed([t])
            least = min(trial.gaps) if trial.gaps else math.inf
            if best is None or least > best[0]:
                best = (least, t, trial)
            if least >= gap:
                break
        # (many experts with flat scores leave no token with the full gap: the clearest one found, if it is clear at all)
        if best[0] < gap / 5:
            raise RuntimeError("no token without a close call found")
        seq = best[2]
        out.append(best[1])
    return out

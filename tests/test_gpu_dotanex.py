"""The Dotanex decoder on the GPU against the plain implementation (``plain_dotanex.py``): each mechanism's kernels
alone, with inputs made so that a fault shows, then whole models through the engine's step function, its cache and
state, its batching and its generation loop."""
import numpy as np
import pytest
import torch

import plain_dotanex as P
from dotanex_models import CONFIGS, TOL, close, model, near, row_errors, tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a)).to(dtype).to(DEV)


def i32(a):
    return torch.as_tensor(np.asarray(a, np.int32)).to(DEV)


def host(t):
    return t.float().cpu().numpy().astype(np.float64)


def engine(name, dtype, **kw):
    from gpullama3_java_amd.engine import Engine
    folder, cfg, W = model(name)
    kw.setdefault("max_tokens", 2048)
    kw.setdefault("n_slots", 6)
    return Engine.from_folder(folder, dtype=dtype, **kw), cfg, W


def bf16_exact(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32).to(torch.bfloat16).float().numpy()


# ----------------------------------------------------------------- the copies of the residual row
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("S, d, T", [(1, 40, 3), (2, 96, 7), (3, 256, 70), (4, 1500, 5), (8, 64, 2), (16, 130, 3)])
def test_copies_mixed_around_a_sublayer(S, d, T, dtype):
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([S, d])
    x0 = rng.standard_normal((T, d)).astype(np.float32)
    rows = torch.zeros(T, S * d, device=DEV)
    K.streams_fill(dev(x0), rows, S)
    np.testing.assert_array_equal(host(rows).reshape(T, S, d), np.repeat(x0[:, None], S, 1))
    xs = rng.standard_normal((T, S, d)).astype(np.float32) * 3          # copies that differ
    y = rng.standard_normal((T, d)).astype(np.float32)
    w_in, mix, w_out = (rng.standard_normal(s).astype(np.float32) for s in ((S,), (S, S), (S,)))
    w = (1 + 0.2 * rng.standard_normal(d)).astype(np.float32)
    new = np.einsum("sr,tsd->trd", mix.astype(np.float64), xs) + w_out[None, :, None] * y[:, None, :]
    tol = 2e-5 if dtype == "float32" else 0.05
    # the read alone
    rows, h = dev(xs.reshape(T, S * d)), torch.zeros(T, d, dtype=TD[dtype], device=DEV)
    K.streams_step(rows, S, in_w=dev(w_in), norm_w=dev(w), eps=1e-5, h=h)
    np.testing.assert_allclose(host(h), P.rms_norm(np.einsum("s,tsd->td", w_in, xs), w, 1e-5), atol=tol)
    np.testing.assert_array_equal(host(rows), xs.reshape(T, S * d))
    # the write-back alone: every copy from the OLD copies
    K.streams_step(rows, S, y=dev(y), mix=dev(mix), out_w=dev(w_out))
    np.testing.assert_allclose(host(rows).reshape(T, S, d), new, atol=2e-5)
    # both ends in one launch: the next sublayer reads the NEW copies
    rows = dev(xs.reshape(T, S * d))
    K.streams_step(rows, S, y=dev(y), mix=dev(mix), out_w=dev(w_out), in_w=dev(w_in), norm_w=dev(w), eps=1e-5, h=h)
    np.testing.assert_allclose(host(rows).reshape(T, S, d), new, atol=2e-5)
    np.testing.assert_allclose(host(h), P.rms_norm(np.einsum("s,tsd->td", w_in, new), w, 1e-5), atol=tol)
    # the copies' sum at chosen rows
    which = [T - 1, 0, T - 1]
    out = torch.zeros(3, d, device=DEV)
    K.streams_sum(rows, S, out, which=i32(which))
    np.testing.assert_allclose(host(out), new.sum(1)[which], atol=2e-5)


@pytest.mark.parametrize("d", [300, 1500, 2048, 4100])
def test_a_row_s_bits_do_not_depend_on_the_size_of_its_step(d):
    """A step of few tokens runs on larger blocks than one of many: the same row comes out with the same bits."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(d)
    S, T = 3, 200
    xs, y = rng.standard_normal((T, S * d)).astype(np.float32), rng.standard_normal((T, d)).astype(np.float32)
    w_in, mix, w_out = (dev(rng.standard_normal(s).astype(np.float32)) for s in ((S,), (S, S), (S,)))
    w = dev((1 + 0.2 * rng.standard_normal(d)).astype(np.float32))
    got = []
    for n in (T, 5):
        rows, h = dev(xs[:n]), torch.zeros(n, d, device=DEV)
        K.streams_step(rows, S, y=dev(y[:n]), mix=mix, out_w=w_out, in_w=w_in, norm_w=w, eps=1e-6, h=h)
        got.append((host(rows)[:5], host(h)[:5]))
    np.testing.assert_array_equal(got[0][0], got[1][0])
    np.testing.assert_array_equal(got[0][1], got[1][1])


# ----------------------------------------------------------------- attention kernels: sinks per head, window edges
def paged(k, v, page, dtype):
    """One sequence's keys [S, G, D] and values [S, G, Dv] (None: no value array) as a paged cache in the kernels'
    order; its pages are 1, 2, ... Returns (k_cache, v_cache, block table [1, pages])."""
    from gpullama3_java_amd.cache.layout import tile_keys, tile_values
    S, G, D = k.shape
    n = -(-S // page)
    kc = np.zeros((n + 1, G, page, D), np.float32)
    for j in range(S):
        kc[1 + j // page, :, j % page] = k[j]
    vc = None
    if v is not None:
        vc = np.zeros((n + 1, G, v.shape[2], page), np.float32)
        for j in range(S):
            vc[1 + j // page, :, :, j % page] = v[j]
        vc = dev(tile_values(vc), TD[dtype])
    return dev(tile_keys(kc), TD[dtype]), vc, i32(np.arange(1, n + 1)[None])


def plain_heads(q, k, v, positions, scale, window=None, sinks=None):
    """q [T, H, D], k [S, G, D], v [S, G, Dv]: causal softmax attention per head, a window and a sink per head."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for t, p in enumerate(positions):
        lo = 0 if window is None else max(0, p - window + 1)
        for h in range(H):
            g = h // (H // G)
            s = k[lo:p + 1, g] @ q[t, h] * scale
            top = s.max() if sinks is None else max(s.max(), sinks[h])
            e = np.exp(s - top)
            out[t, h] = (e / (e.sum() + (0.0 if sinks is None else np.exp(sinks[h] - top)))) @ v[lo:p + 1, g]
    return out


def marked(rng, S, G, D, at, by=16.0):
    """Keys and values of which key ``at`` stands out: every query finds it if it may see it."""
    k = bf16_exact(rng.standard_normal((S, G, D)) * 0.3)
    v = bf16_exact(rng.standard_normal((S, G, D)))
    k[at] = bf16_exact(by * np.ones((G, D)) / np.sqrt(D))
    v[at] = 7.0
    return k, v


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, D, window", [(4, 2, 32, 37), (3, 3, 16, 64), (2, 1, 48, 9), (2, 2, 64, 136), (4, 1, 80, None)])
def test_sinks_per_head_and_window_edges_with_a_marked_key(H, G, D, window, dtype):
    """A key that every query would pick lies just inside the window of one query and just outside the next one's; the
    sinks differ from head to head, one of them so large that its head's output nearly vanishes."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([H, D])
    S, at = 300, 150
    k, v = marked(rng, S, G, D, at)
    w = window or 10 ** 6
    positions = [0, 1, at - 1, at, at + 1, at + w - 2, at + w - 1, at + w, at + w + 1, 255, 256, S - 1]
    positions = [p for p in positions if p < S]
    T = len(positions)
    q = bf16_exact(rng.standard_normal((T, H, D)) * 0.3 + 1.0 / np.sqrt(D))
    sinks = np.linspace(-2.0, 1.0, H).astype(np.float32)
    sinks[-1] = 9.0
    kc, vc, table = paged(k, v, 64, dtype)
    out = torch.zeros(T, H * D, dtype=TD[dtype], device=DEV)
    K.attention_generic(dev(q.reshape(T, H * D), TD[dtype]), kc, vc, i32(positions), i32([0] * T), table, out, H, G, D, 64,
                        window, 0.5, sink=dev(sinks))
    ref = plain_heads(q, k, v, positions, 0.5, window, sinks)
    np.testing.assert_allclose(host(out).reshape(T, H, D), ref, atol=2e-5 if dtype == "float32" else 0.04)
    seen = [abs(ref[positions.index(p), 0]).max() for p in (at, at + 1)]
    assert min(seen) > 2.0                                  # the marked key carries its value into what sees it
    if window is not None and at + w < S:
        assert abs(ref[positions.index(at + w - 1), 0]).max() > 2.0 > 1.5 > abs(ref[positions.index(at + w), 0]).max()


@pytest.mark.parametrize("kernel", [("decode", 1), ("decode", 3), ("prompt", 1), ("prompt", 10 ** 6)])
@pytest.mark.parametrize("H, G, D, window", [(8, 1, 64, 37), (4, 2, 32, 64), (2, 2, 96, 9), (3, 1, 128, 136), (4, 4, 64, None)])
def test_sinks_per_head_and_window_edges_on_the_matrix_cores(H, G, D, window, kernel):
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([H, D, 1])
    S, at = 330, 150
    k, v = marked(rng, S, G, D, at)
    w = window or 10 ** 6
    sinks = np.linspace(-2.0, 1.0, H).astype(np.float32)
    sinks[-1] = 9.0
    kc, vc, table = paged(k, v, 64, "bfloat16")
    if kernel[0] == "decode":
        positions = [p for p in (0, 1, at, at + 1, at + w - 1, at + w, 255, 256, S - 1) if p < S]
    else:
        first = max(0, at + w - 40) if window is not None and at + w + 20 < S else at - 30       # a portion that passes the edge
        positions = list(range(first, min(S, first + 90)))
    T = len(positions)
    q = bf16_exact(rng.standard_normal((T, H, D)) * 0.3 + 1.0 / np.sqrt(D))
    qd, out = dev(q.reshape(T, H * D), torch.bfloat16), torch.zeros(T, H * D, dtype=torch.bfloat16, device=DEV)
    if kernel[0] == "decode":
        n = kernel[1]
        part_o = torch.zeros((T, H, n, D), dtype=torch.float32, device=DEV) if n > 1 else None
        part_ml = torch.zeros((T, H, n, 2), dtype=torch.float32, device=DEV) if n > 1 else None
        K.attention_decode(qd, kc, vc, i32(positions), i32([0] * T), table, out, H, G, D, 64, window, 0.5, n, part_o, part_ml,
                           sink=dev(sinks))
    else:
        K.attention_prefill(qd, kc, vc, i32([0, T]), i32([positions[0]]), table, out, T, H, G, D, 64, window, 0.5,
                            wide_from=kernel[1], sink=dev(sinks))
    ref = plain_heads(q, k, v, positions, 0.5, window, sinks)
    np.testing.assert_allclose(host(out).reshape(T, H, D), ref, atol=0.05)


# ----------------------------------------------------------------- attention over cached latents
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, rank, rot", [(3, 40, 8), (8, 64, 16), (2, 16, 4), (4, 512, 64), (16, 96, 32)])
def test_values_inside_the_keys_and_a_far_marked_latent(H, rank, rot, dtype):
    """The cached rows [latent | shared rotated part | zeros] are keys and, in their first ``rank`` elements, values,
    for all heads alike; one latent hundreds of positions back stands out and is found."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([H, rank])
    dk = -(-(rank + rot) // 16) * 16
    S, at = 700, 3
    rows = np.zeros((S, 1, dk))
    rows[:, 0, :rank + rot] = bf16_exact(rng.standard_normal((S, rank + rot)) * 0.3)
    rows[at, 0, :rank] = bf16_exact(40.0 / np.sqrt(rank))
    positions = [0, 2, 3, 4, 63, 64, 65, 127, 128, 640, S - 1]
    T = len(positions)
    q = np.zeros((T, H, dk))
    q[:, :, :rank + rot] = bf16_exact(rng.standard_normal((T, H, rank + rot)) * 0.3)
    q[:, :, :rank] += bf16_exact(1.0 / np.sqrt(rank))
    q = bf16_exact(q)
    kc, _, table = paged(rows, None, 64, dtype)
    out = torch.zeros(T, H * rank, dtype=TD[dtype], device=DEV)
    K.attention_generic(dev(q.reshape(T, H * dk), TD[dtype]), kc, None, i32(positions), i32([0] * T), table, out, H, 1, dk, 64,
                        None, 0.4, v_head_dim=rank, values_in_keys=0)
    ref = plain_heads(q, rows, rows[:, :, :rank], positions, 0.4)
    np.testing.assert_allclose(host(out).reshape(T, H, rank), ref, atol=2e-5 if dtype == "float32" else 0.03)
    far = ref[positions.index(S - 1), :, 0]
    assert np.median(far) > 0.5 * 40.0 / np.sqrt(rank)          # position 3 still carries the far queries' outputs


@pytest.mark.parametrize("kind", ["decode", "decode in 5 parts", "prompt", "portion", "portion in 3 parts"])
@pytest.mark.parametrize("H, rank, rot", [(3, 48, 16), (8, 64, 16), (16, 96, 32), (32, 256, 32), (5, 16, 4), (70, 32, 32), (1, 64, 64)])
def test_cached_latents_on_the_matrix_cores(H, rank, rot, kind):
    """The same attention from the matrix-core kernel: tiles of (token, head) pairs that span several tokens or a part
    of one token's heads, one token a sequence or a portion of a prompt behind 150 cached positions, a marked latent
    far back, keys up to the tokens' own positions and no further."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([H, rank, 2])
    dk = -(-(rank + rot) // 32) * 32
    assert K.latent_attention_fits(dk, rank, 64)
    S, at = 420, 3
    rows = np.zeros((S, 1, dk))
    rows[:, 0, :rank + rot] = bf16_exact(rng.standard_normal((S, rank + rot)) * 0.3)
    rows[at, 0, :rank] = bf16_exact(40.0 / np.sqrt(rank))
    kc, _, table = paged(rows, None, 64, "bfloat16")
    splits = int(kind.split()[2]) if " in " in kind else 1
    kind = kind.split()[0]
    if kind == "decode":
        positions = [0, 2, 3, 4, 31, 32, 63, 64, 65, 127, 128, 300, S - 1]
        cu, before, seq_rows, longest = list(range(len(positions) + 1)), positions, [0] * len(positions), 1
    else:
        first = 0 if kind == "prompt" else 150
        positions = list(range(first, first + 170))
        cu, before, seq_rows, longest = [0, len(positions)], [first], [0], len(positions)
    T = len(positions)
    q = np.zeros((T, H, dk))
    q[:, :, :rank + rot] = rng.standard_normal((T, H, rank + rot)) * 0.3
    q[:, :, :rank] += 1.0 / np.sqrt(rank)
    q = bf16_exact(q)
    out = torch.zeros(T, H * rank, dtype=torch.bfloat16, device=DEV)
    parts = {}
    if splits > 1:       # (a split may find no key of a short sequence: its part counts for nothing)
        parts = dict(n_splits=splits, part_o=torch.zeros(T * H * splits * rank, device=DEV),
                     part_ml=torch.zeros(T * H * splits * 2, device=DEV))
    K.latent_attention(dev(q.reshape(T, H * dk), torch.bfloat16), kc, i32(cu), i32(before), table, out, longest, H, rank, 0.4,
                       seq_rows=i32(seq_rows), **parts)
    ref = plain_heads(q, rows, rows[:, :, :rank], positions, 0.4)
    np.testing.assert_allclose(host(out).reshape(T, H, rank), ref, atol=0.03, rtol=0.01)
    assert np.median(ref[-1, :, 0]) > 0.5 * 40.0 / np.sqrt(rank)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, D, R, q_rank, rank", [(3, 24, 8, 48, 40), (4, 64, 32, 96, 64), (2, 16, 4, 16, 32), (5, 8, 2, 20, 24)])
def test_latents_normed_turned_and_cached(H, D, R, q_rank, rank, dtype):
    from gpullama3_java_amd.cache.layout import untile_keys
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([H, D, R])
    T, page, dk = 9, 32, -(-(rank + R) // 16) * 16
    positions = [0, 1, 31, 32, 33, 70, 5, 95, 64]
    ld = q_rank + rank + R + 5
    proj = rng.standard_normal((T, ld)).astype(np.float32) * 2
    wq, wkv = (1 + 0.2 * rng.standard_normal(q_rank)).astype(np.float32), (1 + 0.2 * rng.standard_normal(rank)).astype(np.float32)
    freqs, mag = P.yarn_frequencies(777.0, R, {"factor": 4.0, "original": 40, "fast": 8.0, "slow": 1.0})
    ang = np.arange(128)[:, None] * freqs[None, :]
    cos, sin = dev(mag * np.cos(ang)), dev(mag * np.sin(ang))
    k_cache = torch.zeros(4, 1, page, dk, dtype=TD[dtype], device=DEV)
    table = i32([[1, 2, 3]])
    cq = torch.zeros(T, q_rank, dtype=TD[dtype], device=DEV)
    runs, pairs = torch.zeros(H + 1, dtype=torch.int32, device=DEV), torch.zeros(T * H, dtype=torch.int32, device=DEV)
    K.latent_prep(dev(proj), 2, q_rank, 2 + q_rank, rank, R, dev(wq), dev(wkv), 1e-5, i32(positions), i32([0] * T), table, cos, sin,
                  cq, k_cache, page, H, runs, pairs)
    tol = 3e-5 if dtype == "float32" else 0.05
    np.testing.assert_allclose(host(cq), P.rms_norm(proj[:, 2:2 + q_rank], wq, 1e-5), atol=tol)
    flat = untile_keys(host(k_cache)).reshape(4 * page, dk)[page:]          # the sequence's positions in order
    c = P.rms_norm(proj[:, 2 + q_rank:2 + q_rank + rank], wkv, 1e-5)
    r = P.turn(proj[:, None, 2 + q_rank + rank:2 + q_rank + rank + R], positions, freqs, "adjacent", mag)[:, 0]
    for t, p in enumerate(positions):
        np.testing.assert_allclose(flat[p, :rank], c[t], atol=tol)
        np.testing.assert_allclose(flat[p, rank:rank + R], r[t], atol=tol)
        assert not flat[p, rank + R:].any()
    assert list(runs.cpu().numpy()) == [h * T for h in range(H + 1)]
    assert list(pairs.cpu().numpy()) == [t * H + h for h in range(H) for t in range(T)]
    # the rotated part of every head's query behind the absorbed part
    q = bf16_exact(rng.standard_normal((T, H, D + R)))
    qa = torch.full((T, H * dk), 3.0, dtype=TD[dtype], device=DEV)
    K.latent_query(dev(q.reshape(T, -1), TD[dtype]), H, D, R, i32(positions), cos, sin, qa, rank)
    got = host(qa).reshape(T, H, dk)
    np.testing.assert_allclose(got[:, :, rank:rank + R], P.turn(q[:, :, D:], positions, freqs, "adjacent", mag), atol=tol)
    assert (got[:, :, :rank] == 3.0).all() and not got[:, :, rank + R:].any()


# ----------------------------------------------------------------- lightning attention
@pytest.mark.parametrize("H, N, P_", [(3, 24, 40), (4, 32, 64), (1, 16, 16), (2, 8, 100)])
def test_decayed_matrix_with_silu_inputs_whole_and_in_steps(H, N, P_):
    """q, k and v pass silu as the recurrence reads them; the state is carried over steps of 1, 2 and many tokens."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([H, N, P_])
    T = 150
    q, k, v = (rng.standard_normal((T, H * n)).astype(np.float32) for n in (N, N, P_))
    decay = np.linspace(0.4, 0.999, H).astype(np.float32)
    S = np.zeros((H, N, P_))
    ref = np.zeros((T, H, P_))
    qs, ks, vs = (P.silu(a.astype(np.float64)).reshape(T, H, -1) for a in (q, k, v))
    for t in range(T):
        S = S * decay[:, None, None] + ks[t][:, :, None] * vs[t][:, None, :]
        ref[t] = np.einsum("hnp,hn->hp", S, qs[t])
    state = torch.zeros(3, H * N * P_, device=DEV)
    rows = []
    lo = 0
    for hi in (1, 2, 4, 70, 71, 150):
        out = torch.zeros(hi - lo, H * P_, device=DEV)
        K.decay_scan(dev(q[lo:hi]), 0, dev(k[lo:hi]), 0, dev(v[lo:hi]), 0, state, 0, i32([0, hi - lo]), i32([1]), out, H, 1, N, P_,
                     a_head=dev(decay), b_const=1.0, silu_inputs=True)
        rows.append(host(out))
        lo = hi
    np.testing.assert_allclose(np.concatenate(rows).reshape(T, H, P_), ref, rtol=2e-4, atol=2e-4 * np.abs(ref).max())
    np.testing.assert_allclose(host(state[1]).reshape(H, N, P_), S, rtol=2e-4, atol=2e-4 * np.abs(S).max())
    assert not host(state[0]).any() and not host(state[2]).any()


@pytest.mark.parametrize("dtype", DTYPES)
def test_unit_norm_over_all_heads_with_a_sigmoid_gate(dtype):
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(8)
    T, C = 6, 3 * 40
    o, g = rng.standard_normal((T, C)).astype(np.float32) * 4, rng.standard_normal((T, C + 7)).astype(np.float32)
    w = (1 + 0.2 * rng.standard_normal(C)).astype(np.float32)
    out = torch.zeros(T, C, dtype=TD[dtype], device=DEV)
    K.group_norm_gate(dev(o), dev(g), 7, out, C, 1e-5, weight=dev(w), gate_act="sigmoid")
    np.testing.assert_allclose(host(out), P.rms_norm(o, w, 1e-5) * P.sigmoid(g[:, 7:]), atol=2e-5 if dtype == "float32" else 0.03)


# ----------------------------------------------------------------- the mixture of experts
def test_router_scores_correction_and_weights():
    """The choice goes by score plus correction, the weights by the scores alone: a correction that lifts an expert
    into the choice leaves its weight small; ties go to the lower number."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(4)
    T, E = 70, 7
    logits = rng.standard_normal((T, E)).astype(np.float32) * 2
    logits[0] = 1.0
    corr = np.zeros(E, np.float32)
    corr[5] = 0.4                                       # expert 5 is chosen nearly always, whatever its score
    for top in (1, 2, 3, 7):
        for c in (None, corr):
            idx, wts = torch.zeros(T, top, dtype=torch.int32, device=DEV), torch.zeros(T, top, device=DEV)
            offsets, pairs = torch.zeros(E + 1, dtype=torch.int32, device=DEV), torch.zeros(T * top, dtype=torch.int32, device=DEV)
            K.route(dev(logits), top, idx, wts, offsets, pairs, scores=True, correction=None if c is None else dev(c), sum_eps=1e-20)
            idx, wts, offsets, pairs = idx.cpu().numpy(), host(wts), offsets.cpu().numpy(), pairs.cpu().numpy()
            z = logits.astype(np.float64)
            s = np.exp(z - z.max(-1, keepdims=True))
            s /= s.sum(-1, keepdims=True)
            for t in range(T):
                order = np.argsort(-(s[t] + (0 if c is None else c)), kind="stable")[:top]
                assert list(idx[t]) == list(order), (top, t)
                np.testing.assert_allclose(wts[t], s[t, order] / s[t, order].sum(), atol=1e-6)
            assert offsets[0] == 0 and offsets[-1] == T * top and sorted(pairs) == list(range(T * top))
            for e in range(E):
                assert all(idx.reshape(-1)[p] == e for p in pairs[offsets[e]:offsets[e + 1]])
    assert (idx == 5).any(1).all()


@pytest.mark.parametrize("dtype, mfma", [("float32", False), ("bfloat16", False), ("bfloat16", True)])
@pytest.mark.parametrize("E, I, top, T, d, F, limit", [(5, 2, 3, 90, 96, 40, 1.5), (3, 0, 3, 7, 64, 72, None), (11, 4, 2, 300, 128, 88, 2.0),
                                                      (4, 1, 1, 1, 80, 48, 1.0), (4, 2, 2, 700, 200, 136, 2.0), (8, 3, 2, 8, 1024, 520, 0.7),
                                                      (2, 6, 2, 64, 320, 24, 1.0), (4, 0, 2, 100, 192, 64, 2.0)])
def test_gated_experts_and_identity_experts(E, I, top, T, d, F, limit, dtype, mfma):
    """Every kernel of the grouped product (by run length) with gate and up rows in turns; pairs of identity experts
    have no product, and the weighted sum takes the input row for them."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([E, T, d])
    h = bf16_exact(rng.standard_normal((T, d)))
    gate, up = (bf16_exact(rng.standard_normal((E, F, d)) * 1.5 / np.sqrt(d)) for _ in range(2))
    down = bf16_exact(rng.standard_normal((E, d, F)) / np.sqrt(F))
    turns = np.stack([gate, up], axis=2).reshape(E, 2 * F, d)
    logits = rng.standard_normal((T, E + I)).astype(np.float32)
    idx, wts = torch.zeros(T, top, dtype=torch.int32, device=DEV), torch.zeros(T, top, device=DEV)
    offsets, pairs = torch.zeros(E + I + 1, dtype=torch.int32, device=DEV), torch.zeros(T * top, dtype=torch.int32, device=DEV)
    K.route(dev(logits), top, idx, wts, offsets, pairs, scores=True, sum_eps=1e-20)
    hidden = torch.zeros(T * top, F, dtype=TD[dtype], device=DEV)
    hd = dev(h, TD[dtype])
    K.expert_gemm(hd, dev(turns, TD[dtype]), hidden, gated=("quick_gelu", limit, 1.0), offsets=offsets, pairs=pairs, a_div=top, mfma=mfma)
    outs = torch.zeros(T * top, d, device=DEV)
    K.expert_gemm(hidden, dev(down, TD[dtype]), outs, offsets=offsets, pairs=pairs, mfma=mfma)
    y = torch.full((T, d), 2.0, device=DEV)
    K.route_combine(outs, wts, y, accumulate=True, identity=(idx, E, hd) if I else None)
    choice, w = idx.cpu().numpy(), host(wts)
    assert not I or T < 8 or (choice >= E).any()
    tol = 3e-5 if dtype == "float32" else 0.04

    def plain_hidden(e, row):
        g, u = gate[e] @ row, up[e] @ row
        if limit is not None:
            g, u = np.minimum(g, limit), np.clip(u, -limit, limit)
        return g * P.sigmoid(1.702 * g) * (u + 1.0)

    got_hidden, got_outs = host(hidden), host(outs)
    ref_y = np.full((T, d), 2.0)
    for t in range(T):
        for j in range(top):
            e, p = choice[t, j], t * top + j
            if e >= E:
                ref_y[t] += w[t, j] * h[t]
                continue
            np.testing.assert_allclose(got_hidden[p], plain_hidden(e, h[t]), atol=tol)
            ref_out = down[e] @ got_hidden[p]
            np.testing.assert_allclose(got_outs[p], ref_out, atol=3 * tol)
            ref_y[t] += w[t, j] * ref_out
    np.testing.assert_allclose(host(y), ref_y, atol=3 * tol)
    # one gated expert over every row in its own order: the expert that every token passes
    dense = torch.zeros(T, F, dtype=TD[dtype], device=DEV)
    K.expert_gemm(hd, dev(turns[:1], TD[dtype]), dense, gated=("quick_gelu", limit, 1.0), mfma=mfma)
    np.testing.assert_allclose(host(dense), np.stack([plain_hidden(0, h[t]) for t in range(T)]), atol=tol)


# ----------------------------------------------------------------- whole models through the engine
def copies_sum(cfg, x):
    S = cfg.get("streams", 1)
    x = x.float().cpu().numpy()
    return x.reshape(x.shape[0], S, -1).sum(1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompt_and_every_layer(name, dtype):
    eng, cfg, W = engine(name, dtype)
    toks = tokens(name, 1, 210)                       # beyond every window, over four pages
    seq = P.Sequence(cfg, W)
    ref = seq.feed(toks)
    seen = []
    eng.after_block = lambda i, x: seen.append(copies_sum(cfg, x))
    s = eng.take_slot()
    got = eng.step([(s, toks)], want="all").cpu().numpy()
    eng.after_block = None
    assert len(seen) == len(seq.rows[0]) == len(cfg["layers"])
    for r, (a, b) in enumerate(zip(seen, seq.rows[0])):     # the first layer that differs names the mechanism
        near(a, b, dtype, f"layer {r}")
    close(got, ref, dtype, name)
    # the first tokens of a sequence, each alone from an empty slot
    for n in (1, 2, 3):
        s2 = eng.take_slot()
        close(eng.step([(s2, toks[:n])], want="all").cpu().numpy(), ref[:n], dtype, f"{name} first {n}")
        eng.give_back_slot(s2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_every_sublayer_alone(name, dtype):
    """Each mixer's and each feed-forward's output against the plain one computed from the plain copies in front of
    it: a fault does not hide behind the layers before it."""
    if "streams" not in CONFIGS[name]:
        pytest.skip("the plain residual sum: sublayers add into the rows themselves, there is nothing to look at apart")
    eng, cfg, W = engine(name, dtype)
    toks = tokens(name, 6, 75)
    want = {}
    seq = P.Sequence(cfg, W)
    inner = seq._sublayer

    def noting(xs, p, q, fn):           # what a sublayer returns, by the order in which the sublayers run
        def fn_noted(h):
            y = fn(h)
            want[len(want)] = y
            return y
        return inner(xs, p, q, fn_noted)

    seq._sublayer = noting
    seq.feed(toks)
    seen = []
    eng.after_sublayer = lambda e, kind, t: seen.append(t.float().cpu().numpy()) if kind in ("mixer", "ffn") else None
    eng.step([(eng.take_slot(), toks)], want="none")
    eng.after_sublayer = None
    assert len(seen) == len(want)
    for n, ref in want.items():
        near(seen[n], ref, dtype, f"sublayer {n}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prompt_then_token_by_token(name, dtype):
    """Decoding passes every window's edge and two page borders; the decoded rows are those of the whole prompt."""
    eng, cfg, W = engine(name, dtype)
    toks = tokens(name, 2, 200)
    ref = P.forward(cfg, W, toks)
    s = eng.take_slot()
    rows = [eng.step([(s, toks[:3])], want="all").cpu().numpy()]
    for t in toks[3:]:
        rows.append(eng.step([(s, [t])]).cpu().numpy())
    close(np.concatenate(rows), ref, dtype, name)
    assert eng.cache.length(s) == 200


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name, cuts", [("mixed", [2, 4, 7, 36, 38, 64, 66, 74, 128, 129, 131, 190]),
                                        ("reordered", [1, 3, 5, 9, 10, 12, 33, 63, 65, 67, 100, 102, 190]),
                                        ("plain", [19, 21, 23, 64, 190]),
                                        ("tiled", [99, 101, 130, 131, 190])])
def test_portions_of_a_prompt(name, cuts, dtype):
    eng, cfg, W = engine(name, dtype)
    toks = tokens(name, 3, 190)
    ref = P.forward(cfg, W, toks)
    s = eng.take_slot()
    rows, lo = [], 0
    for hi in cuts:
        rows.append(eng.step([(s, toks[lo:hi])], want="all").cpu().numpy())
        lo = hi
    close(np.concatenate(rows), ref, dtype, name)
    if dtype == "float32":
        # nothing but rounding hangs on the cut: against the same prompt in one step
        s2 = eng.take_slot()
        whole = eng.step([(s2, toks)], want="all").cpu().numpy()
        assert row_errors(np.concatenate(rows), whole).max() < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_unequal_requests_in_one_batch_and_slots_used_again(name, dtype):
    eng, cfg, W = engine(name, dtype, n_slots=4, max_tokens=1024)
    lens = [1, 70, 131, 9]
    prompts = [tokens(name, 10 + i, n + 12) for i, n in enumerate(lens)]
    refs = [P.forward(cfg, W, p) for p in prompts]
    for time in range(2):                             # the second time takes the slots and pages that the first gave back
        slots = [eng.take_slot() for _ in lens]
        order = list(range(4)) if time == 0 else [2, 0, 3, 1]
        got = eng.step([(slots[i], prompts[i][:lens[i]]) for i in order], want="all").cpu().numpy()
        lo = 0
        for i in order:
            close(got[lo:lo + lens[i]], refs[i][:lens[i]], dtype, f"{name} prompt {i} time {time}")
            lo += lens[i]
        live = list(order)
        for step in range(12):
            if step == 5:                             # one request ends earlier
                eng.give_back_slot(slots[live.pop(0)])
            got = eng.step([(slots[i], [prompts[i][lens[i] + step]]) for i in live]).cpu().numpy()
            for r, i in enumerate(live):
                close(got[r:r + 1], refs[i][lens[i] + step:lens[i] + step + 1], dtype, f"{name} request {i} step {step}")
        for i in live:
            eng.give_back_slot(slots[i])
    assert eng.slots_free() == 4


def test_a_windowed_layer_gives_pages_back_and_a_state_starts_at_zero_again():
    """The cache of a windowed attention holds the window only: pages in front of it go back to the pool as the
    sequence grows and are used again by another sequence; a slot that is used again starts its recurrent states at
    zero; the logits stay those of the plain implementation."""
    eng, cfg, W = engine("mixed", "float32", n_slots=2, max_tokens=700)
    toks, other = tokens("mixed", 40, 330), tokens("mixed", 41, 100)
    ref, ref_other = P.forward(cfg, W, toks), P.forward(cfg, W, other)
    a = eng.take_slot()
    rows = [eng.step([(a, toks[:150])], want="all").cpu().numpy()]
    windowed = [g for g, group in enumerate(eng.cache.groups) if group.need.window]
    assert windowed
    for g in windowed:                               # a window of 37: only the last pages are still held
        assert len([p for p in eng.cache.slots.pages[a][g] if p]) <= 2
    b = eng.take_slot()
    rows_b = [eng.step([(b, other[:60])], want="all").cpu().numpy()]
    for j in range(150, 330):
        entries = [(a, [toks[j]])] + ([(b, [other[60 + j - 150]])] if 60 + j - 150 < 100 else [])
        out = eng.step(entries).cpu().numpy()
        rows.append(out[:1])
        if len(entries) > 1:
            rows_b.append(out[1:])
    close(np.concatenate(rows), ref, "float32", "the long request")
    close(np.concatenate(rows_b), ref_other, "float32", "the one that took its pages")
    eng.give_back_slot(b)
    b = eng.take_slot()                               # the same slot, whose states the last sequence left full
    close(eng.step([(b, other)], want="all").cpu().numpy(), ref_other, "float32", "a slot used again")


def test_long_decoding_in_32_bit():
    eng, cfg, W = engine("mixed", "float32")
    toks = tokens("mixed", 4, 300)
    ref = P.forward(cfg, W, toks)
    s = eng.take_slot()
    rows = [eng.step([(s, toks[:2])], want="all").cpu().numpy()]
    for t in toks[2:]:
        rows.append(eng.step([(s, [t])]).cpu().numpy())
    close(np.concatenate(rows), ref, "float32")


def test_greedy_generation_through_the_scheduler():
    """The engine's own entry point and scheduler: three prompts of unequal lengths, greedy, in 32-bit (a bfloat16
    engine may choose another expert on a close call of a token that it generated itself)."""
    eng, cfg, W = engine("mixed", "float32")
    prompts = [tokens("mixed", 20, 5), tokens("mixed", 21, 45), tokens("mixed", 22, 1)]
    out = eng.generate(prompts, max_new_tokens=20, temperature=0.0)
    for p, r in zip(prompts, out):
        assert len(r.tokens) == 20
        seq = list(p)
        for t in r.tokens:
            logits = P.forward(cfg, W, seq)[-1]
            best = int(np.argmax(logits))
            assert t == best or logits[best] - logits[t] < 1e-4 * np.abs(logits).max(), (len(seq), t, best)
            seq.append(t)
    assert eng.slots_free() == eng.n_slots


def test_generation_in_bfloat16_runs_captured_steps():
    """A bfloat16 engine decodes from captured graphs: the same tokens come out of eager steps, run after run."""
    eng, cfg, W = engine("tiled", "bfloat16")
    assert eng.use_graphs
    prompts = [tokens("tiled", 23, 9), tokens("tiled", 24, 70)]
    first = [r.tokens for r in eng.generate(prompts, max_new_tokens=24, temperature=0.0)]
    again = [r.tokens for r in eng.generate(prompts, max_new_tokens=24, temperature=0.0)]
    plain, _, _ = engine("tiled", "bfloat16", use_graphs=False)
    eager = [r.tokens for r in plain.generate(prompts, max_new_tokens=24, temperature=0.0)]
    assert first == again == eager


def test_the_command_line_takes_the_model(capsys):
    from gpullama3_java_amd import cli
    folder, cfg, W = model("reordered")
    prompt = tokens("reordered", 30, 6)
    rc = cli.main(["--model", folder, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "12", "--temperature", "0",
                   "--dtype", "float32", "--stream", "false"])
    assert not rc
    words = capsys.readouterr().out.split()
    got = [int(w) for w in words if w.lstrip("-").isdigit()]
    seq = list(prompt)
    for t in got[:3]:
        assert t == int(np.argmax(P.forward(cfg, W, seq)[-1]))
        seq.append(t)
    assert len(got) >= 3


def test_the_trace_runner_replays_a_model_of_this_design(tmp_path):
    """bin/trace_run as a user drives it: a request whole, one with its last tokens one by one, two of unequal lengths
    in one batch that end at different times; the model class comes from the folder's config.json."""
    from test_gpu_replay import Replay
    name = "mixed"
    folder, cfg, W = model(name)
    V = cfg["vocab"]
    reqs = {"a": tokens(name, 50, 90), "b": tokens(name, 51, 140), "c": tokens(name, 52, 7)}
    ref = {k: P.forward(cfg, W, t) for k, t in reqs.items()}
    rp = Replay(folder, "float32", tmp_path, max_tokens=400)
    t = reqs["a"]
    close(rp.step([("a", t, list(range(len(t))))], end=["a"]).reshape(-1, V), ref["a"], "float32", "whole")
    t = reqs["b"]
    rows = [rp.step([("b", t[:100], [0, 50, 99])]).reshape(-1, V)]
    for j in range(100, len(t)):
        rows.append(rp.step([("b", [t[j]], [0])], end=["b"] if j == len(t) - 1 else []).reshape(-1, V))
    close(np.concatenate(rows), ref["b"][[0, 50, 99] + list(range(100, len(t)))], "float32", "decoded")
    got = {"a": [], "c": []}
    out = rp.step([("c", reqs["c"][:3], [0, 1, 2]), ("a", reqs["a"][:70], [69])]).reshape(-1, V)
    got["c"].append(out[:3]); got["a"].append(out[3:])
    for j in range(20):
        live = [k for k in ("c", "a") if (3 if k == "c" else 70) + j < len(reqs[k])]
        at = {k: (3 if k == "c" else 70) + j for k in live}
        out = rp.step([(k, [reqs[k][at[k]]], [0]) for k in live], end=[k for k in live if at[k] + 1 == len(reqs[k])]).reshape(-1, V)
        for r, k in enumerate(live):
            got[k].append(out[r:r + 1])
    close(np.concatenate(got["c"]), ref["c"], "float32", "the shorter of a batch")
    close(np.concatenate(got["a"]), ref["a"][69:90], "float32", "the longer of a batch")
    rp.close()


# ----------------------------------------------------------------- seeded random configurations
def random_config(seed):
    """A configuration drawn from a seed: copies, widths, head counts and sizes (multiples of 8 that no tile need
    divide, latents of any even size), layer order, windows, limits, experts and identity experts, scalings on and
    off, layers that run another layer's weights."""
    from dotanex_models import _dense, _latent, _lightning, _moe, _window
    rng = np.random.default_rng([seed, 77])
    pick = lambda *a: a[int(rng.integers(0, len(a)))]
    width = int(pick(48, 64, 72, 104, 128))

    def mlp():
        kind = pick("dense", "moe", "moe", None)
        if kind is None:
            return None
        if kind == "dense":
            return _dense(int(pick(24, 40, 56, 96)))
        experts, identity = int(pick(1, 2, 3, 5, 8)), int(pick(0, 0, 1, 3))
        top = int(rng.integers(1, min(experts + identity, 4) + 1))
        shared = pick(None, (int(pick(16, 24, 40)), pick(None, 0.5, 1.0, 3.0)))
        return _moe(experts, identity, top, int(pick(8, 24, 33, 40)), pick(None, 0.7, 1.0, 2.0), shared)

    def layer():
        kind = pick("lightning", "latent", "window")
        if kind == "lightning":
            H = int(pick(1, 2, 3, 5))
            return _lightning(H, int(pick(8, 16, 20, 32)), int(pick(8, 24, 40, 64)), [float(rng.uniform(0.3, 0.9995)) for _ in range(H)], mlp())
        if kind == "latent":
            rot = int(pick(2, 4, 8, 16))
            scaling = pick(None, (float(pick(2.0, 8.0, 40.0)), int(pick(16, 64, 256)), float(pick(8.0, 32.0)), float(pick(1.0, 2.0))))
            dim = int(pick(8, 16, 24, 40))
            return _latent(int(pick(1, 2, 3, 6)), dim, rot, int(pick(8, 16, 24, 48)), int(pick(12, 16, 40, 64)), int(pick(10, 16, 32, 48, 80)),
                           float((dim + rot) ** -0.5 * rng.uniform(0.7, 1.4)), float(pick(100.0, 1e4, 2.5e5)), scaling, mlp())
        G = int(pick(1, 2, 3))
        dim = int(pick(8, 16, 24, 32, 64))
        dims = int(pick(2, 4, 8, dim))
        dims = min(dims, dim) // 2 * 2
        scaling = pick(None, (float(pick(2.0, 8.0, 32.0)), 1.0, float(pick(2.0, 4.0)), int(pick(16, 64, 512))))
        return _window(G * int(pick(1, 2, 4)), G, dim, float(dim ** -0.5 * rng.uniform(0.7, 1.4)), float(pick(100.0, 1e4, 5e5)), dims, scaling,
                       pick(None, 1, 2, 7, 33, 64, 65, 100), mlp())

    layers = [layer() for _ in range(int(rng.integers(2, 6)))]
    for i in range(len(layers)):                        # some layers run another layer's weights
        j = int(rng.integers(0, len(layers)))
        if rng.random() < 0.3 and j != i and "weights_of" not in layers[j] and "weights_of" not in layers[i] \
                and not any(l.get("weights_of") == i for l in layers):
            layers[i] = dict(layers[j], weights_of=j)
    cfg = {"architecture": "Dotanex", "vocab": int(pick(97, 150, 256, 301)), "width": width, "norm": {"eps": float(pick(1e-6, 1e-5))},
           "layers": layers}
    streams = pick(None, 1, 2, 3, 5)
    if streams is not None:
        cfg["streams"] = int(streams)
    return cfg


@pytest.mark.parametrize("seed", range(12))
def test_seeded_random_configurations(seed, tmp_path):
    """Whole, in portions with the last tokens one by one, and as one of a batch of three: 32-bit against the plain
    implementation to rounding, bfloat16 within its bound."""
    from dotanex_models import write_model
    from gpullama3_java_amd.engine import Engine
    cfg = random_config(seed)
    W = P.make_weights(cfg, seed)
    folder = str(tmp_path / "model")
    write_model(folder, cfg, W)
    toks = P.tokens_with_clear_choices(cfg, W, seed, 150)
    others = [P.tokens_with_clear_choices(cfg, W, seed + 100 + i, n) for i, n in enumerate((40, 9))]
    ref = P.forward(cfg, W, toks)
    refs = [P.forward(cfg, W, t) for t in others]
    for dtype in DTYPES:
        eng = Engine.from_folder(folder, dtype=dtype, max_tokens=1024, n_slots=4)
        s = eng.take_slot()
        what = f"seed {seed} {dtype}"
        close(eng.step([(s, toks)], want="all").cpu().numpy(), ref, dtype, what + " whole", few_far=4)
        eng.give_back_slot(s)
        s = eng.take_slot()
        rows = [eng.step([(s, toks[:70])], want="all").cpu().numpy(), eng.step([(s, toks[70:72])], want="all").cpu().numpy(),
                eng.step([(s, toks[72:140])], want="all").cpu().numpy()]
        rows += [eng.step([(s, [t])]).cpu().numpy() for t in toks[140:]]
        close(np.concatenate(rows), ref, dtype, what + " in portions", few_far=4)
        eng.give_back_slot(s)
        slots = [eng.take_slot() for _ in range(3)]
        got = eng.step([(slots[0], others[0][:30]), (slots[1], toks[:100]), (slots[2], others[1][:3])], want="all").cpu().numpy()
        close(got[:30], refs[0][:30], dtype, what + " batch 0", few_far=2)
        close(got[30:130], ref[:100], dtype, what + " batch 1", few_far=3)
        close(got[130:], refs[1][:3], dtype, what + " batch 2", few_far=1)
        for j in range(6):
            got = eng.step([(slots[0], [others[0][30 + j]]), (slots[1], [toks[100 + j]]), (slots[2], [others[1][3 + j]])]).cpu().numpy()
            close(got[0:1], refs[0][30 + j:31 + j], dtype, what + f" decode 0 step {j}")
            close(got[1:2], ref[100 + j:101 + j], dtype, what + f" decode 1 step {j}")
            close(got[2:3], refs[1][3 + j:4 + j], dtype, what + f" decode 2 step {j}")
        del eng

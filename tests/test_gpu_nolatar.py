"""The Nolatar decoder on the GPU against the plain implementation (``plain_nolatar.py``): each mechanism's kernels
alone, with inputs made so that a fault shows, then whole models through the engine's step function, its cache and
state, its batching and its generation loop."""
import numpy as np
import pytest
import torch

import plain_nolatar as P
from nolatar_models import CONFIGS, LOOSER, TOL, close, model, row_errors, tokens, write_model

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


# ----------------------------------------------------------------- layer norm
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d", [40, 96, 256, 1500])
def test_layer_norm_behind_a_sublayer_and_over_chosen_rows(d, dtype):
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(d)
    x, y = rng.standard_normal((7, d)) * 3, rng.standard_normal((7, d)) * 5 + 2.0       # (a mean far from zero)
    w, b = 1 + 0.2 * rng.standard_normal(d), 0.3 * rng.standard_normal(d)
    xd, cast = dev(x), torch.zeros(7, d, dtype=TD[dtype], device=DEV)
    K.layernorm_add(xd, dev(y), dev(w), dev(b), 1e-5, cast)
    ref = x.astype(np.float32) + P.layer_norm(y.astype(np.float32), w.astype(np.float32), b.astype(np.float32), 1e-5)
    np.testing.assert_allclose(host(xd), ref, atol=2e-5)
    np.testing.assert_allclose(host(cast), ref, atol=2e-5 if dtype == "float32" else 0.06)
    rows = [5, 0, 5]
    out = torch.zeros(3, d, dtype=TD[dtype], device=DEV)
    K.layernorm(dev(y), dev(w), dev(b), out, 1e-5, i32(rows))
    np.testing.assert_allclose(host(out), P.layer_norm(y.astype(np.float32)[rows], w.astype(np.float32), b.astype(np.float32), 1e-5),
                               atol=2e-5 if dtype == "float32" else 0.06)


# ----------------------------------------------------------------- norm on queries and keys, rotation
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pairing, D, Dpad, dims", [("half", 24, 32, 16), ("adjacent", 24, 32, 8), ("half", 48, 48, 48),
                                                    ("adjacent", 96, 96, 96), ("adjacent", 8, 16, 2)])
def test_norm_per_head_in_front_of_the_rotation(pairing, D, Dpad, dims, dtype):
    """Heads padded with zeros to the cache's tiles keep their own size in the norm's mean; the rotation touches the
    first ``dims`` elements in the description's pairing."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([D, dims])
    T, H, G = 5, 3, 2
    positions = [0, 1, 7, 300, 301]
    q, k = bf16_exact(rng.standard_normal((T, H, D))), bf16_exact(rng.standard_normal((T, G, D)) * 4)
    wq, wk = 1 + 0.3 * rng.standard_normal(D), 1 + 0.3 * rng.standard_normal(D)
    rows = np.zeros((T, (H + G) * Dpad), np.float32)
    rows[:, :H * Dpad].reshape(T, H, Dpad)[:, :, :D] = q
    rows[:, H * Dpad:].reshape(T, G, Dpad)[:, :, :D] = k
    half = dims // 2
    f = np.array([1000.0 ** (-2.0 * i / dims) for i in range(half)])
    ang = np.arange(400)[:, None] * f[None]
    cos, sin = dev(np.cos(ang)), dev(np.sin(ang))
    rd = dev(rows, TD[dtype])
    pad = lambda w: dev(np.concatenate([w, np.zeros(Dpad - D)]))
    K.rotate_heads(rd, i32(positions), [(0, H, Dpad, dims, cos, sin), (H * Dpad, G, Dpad, dims, cos, sin)],
                   adjacent=pairing == "adjacent", norms=[(pad(wq), D), (pad(wk), D)], norm_eps=1e-6)
    got = host(rd)
    ref_q = P.turn(P.head_norm_rows(q, wq, 1e-6), positions, 1000.0, dims, pairing)
    ref_k = P.turn(P.head_norm_rows(k, wk, 1e-6), positions, 1000.0, dims, pairing)
    tol = 3e-5 if dtype == "float32" else 0.03
    np.testing.assert_allclose(got[:, :H * Dpad].reshape(T, H, Dpad)[:, :, :D], ref_q, atol=tol)
    np.testing.assert_allclose(got[:, H * Dpad:].reshape(T, G, Dpad)[:, :, :D], ref_k, atol=tol)
    assert not got[:, :H * Dpad].reshape(T, H, Dpad)[:, :, D:].any()


# ----------------------------------------------------------------- the chunked mask and several score maps
def paged(k, v, page, dtype):
    """One sequence's keys [S, Gk, D] and values [S, Gv, Dv] as a paged cache in the kernels' order; its pages are
    1, 2, ... Returns (k_cache, v_cache, block table [1, pages])."""
    from gpullama3_java_amd.cache.layout import tile_keys, tile_values
    S, Gk, D = k.shape
    Gv, Dv = v.shape[1], v.shape[2]
    n = -(-S // page)
    kc = np.zeros((n + 1, Gk, page, D), np.float32)
    vc = np.zeros((n + 1, Gv, Dv, page), np.float32)
    for j in range(S):
        kc[1 + j // page, :, j % page] = k[j]
        vc[1 + j // page, :, :, j % page] = v[j]
    return (dev(tile_keys(kc), TD[dtype]), dev(tile_values(vc), TD[dtype]), i32(np.arange(1, n + 1)[None]))


def attention_on_gpu(q, k, v, positions, dtype, chunk, scale, maps=1, page=64, out_dtype=None):
    """q [T, H * maps, D], k [S, G * maps, D], v [S, G, Dv] -> [T, H * maps, Dv] from the kernel for any sizes."""
    from gpullama3_java_amd.csrc import lib as K
    T, Hq, D = q.shape
    kc, vc, table = paged(k, v, page, dtype)
    out = torch.zeros(T, Hq * v.shape[2], dtype=TD[out_dtype or dtype], device=DEV)
    K.attention_generic(dev(q.reshape(T, Hq * D), TD[dtype]), kc, vc, i32(positions), i32([0] * T), table, out, Hq, k.shape[1],
                        D, page, None, scale, v_head_dim=v.shape[2], chunk=chunk or 0, n_v_heads=v.shape[1] if maps > 1 else None)
    return host(out).reshape(T, Hq, v.shape[2])


def attention_on_matrix_cores(q, k, v, positions, chunk, scale, kernel, maps=1, page=64):
    """The same from the matrix-core kernels (bfloat16, values of the keys' size): ``kernel`` ("decode", splits): one
    token a sequence; ("prompt", wide_from): the tokens of one sequence, the first of them at positions[0]."""
    from gpullama3_java_amd.csrc import lib as K
    T, Hq, D = q.shape
    kc, vc, table = paged(k, v, page, "bfloat16")
    out = torch.zeros(T, Hq * D, dtype=torch.bfloat16, device=DEV)
    qd = dev(q.reshape(T, Hq * D), torch.bfloat16)
    n_v = v.shape[1] if maps > 1 else None
    if kernel[0] == "decode":
        n = kernel[1]
        part_o = torch.zeros((T, Hq, n, D), dtype=torch.float32, device=DEV) if n > 1 else None
        part_ml = torch.zeros((T, Hq, n, 2), dtype=torch.float32, device=DEV) if n > 1 else None
        K.attention_decode(qd, kc, vc, i32(positions), i32([0] * T), table, out, Hq, k.shape[1], D, page, None, scale, n, part_o,
                           part_ml, chunk=chunk or 0, n_v_heads=n_v)
    else:
        K.attention_prefill(qd, kc, vc, i32([0, T]), i32([positions[0]]), table, out, T, Hq, k.shape[1], D, page, None, scale,
                            wide_from=kernel[1], chunk=chunk or 0, n_v_heads=n_v)
    return host(out).reshape(T, Hq, D)


def plain_attention_at(q, k, v, positions, chunk, scale):
    return np.concatenate([P.softmax_attention(q[t:t + 1], k[:p + 1], v[:p + 1], p, scale, chunk) for t, p in enumerate(positions)])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, D, Dv, chunk", [(4, 2, 32, 48, 37), (3, 3, 16, 16, 64), (2, 1, 48, 32, 9), (2, 2, 64, 64, 190),
                                               (2, 1, 16, 32, 1), (1, 1, 32, 32, None)])
def test_chunk_edges_with_a_marked_key(H, G, D, Dv, chunk, dtype):
    """One key answers every query strongly and carries a value far from the others: a query's output shows whether
    it sees that key. The key stands at a chunk's first and last position, queries right at, before and behind the
    next chunk's start, at page borders (64) and far on."""
    rng = np.random.default_rng([H, D, chunk or 0])
    S, c = 330, chunk or 10 ** 6
    for marked in sorted({0, c - 1, c, 2 * c - 1, 63, 64, (200 // c) * c} & set(range(S))):
        q, k = bf16_exact(rng.standard_normal((S, H, D)) * 0.3), bf16_exact(rng.standard_normal((S, G, D)) * 0.3)
        v = bf16_exact(rng.standard_normal((S, G, Dv)))
        k[marked] = 0.0
        k[marked, :, 0] = 6.0
        q[:, :, 0] = 6.0
        v[marked] = 30.0
        edge = (marked // c + 1) * c                      # the first position that no longer sees the marked key
        positions = sorted({p for p in (marked, marked + 1, edge - 1, edge, edge + 1, 63, 64, 65, 127, 128, 329) if marked <= p < S}
                           | {0, 1, max(0, marked - 1)})
        ref = plain_attention_at(q[positions], k, v, positions, chunk, 0.25)
        got = attention_on_gpu(q[positions], k, v, positions, dtype, chunk, 0.25)
        sees = [P.sees(p, marked, chunk) for p in positions]
        assert any(sees) and (marked == 0 and chunk is None or not all(sees))
        np.testing.assert_allclose(got, ref, atol=2e-4 if dtype == "float32" else 0.25, err_msg=f"marked {marked}")
        for t, see in enumerate(sees):      # the marked value dominates exactly where the key is visible
            assert (np.abs(got[t]).mean() > 10.0) == see, (marked, positions[t])


@pytest.mark.parametrize("kernel", [("decode", 1), ("decode", 3), ("prompt", 1), ("prompt", 10 ** 6)])
@pytest.mark.parametrize("H, G, D, chunk", [(8, 1, 64, 37), (4, 2, 32, 64), (2, 2, 96, 9), (3, 1, 128, 190), (4, 4, 64, 100)])
def test_chunk_edges_on_the_matrix_cores(H, G, D, chunk, kernel):
    """The marked key at a chunk's first and last position and at a page border, against the plain attention: decode
    steps (one block and three splits of the keys) at positions right at and around the next chunk's start, and prompt
    steps (both kernels) whose tokens begin in one chunk, behind cached tokens, and end in the next."""
    rng = np.random.default_rng([H, D, chunk])
    S = 330
    for marked in sorted({0, chunk - 1, chunk, 2 * chunk - 1, 64, (200 // chunk) * chunk} & set(range(S))):
        q, k = bf16_exact(rng.standard_normal((S, H, D)) * 0.3), bf16_exact(rng.standard_normal((S, G, D)) * 0.3)
        v = bf16_exact(rng.standard_normal((S, G, D)))
        k[marked] = 0.0
        k[marked, :, 0] = 6.0
        q[:, :, 0] = 6.0
        v[marked] = 30.0
        edge = (marked // chunk + 1) * chunk
        if kernel[0] == "decode":
            positions = sorted({p for p in (marked, marked + 1, edge - 1, edge, edge + 1, 63, 64, 65, 127, 128, 329) if marked <= p < S}
                               | {0, 1, max(0, marked - 1)})
        else:
            first = max(0, marked - 5)
            positions = list(range(first, min(S, max(edge + 40, first + 150))))
        ref = plain_attention_at(q[positions], k, v, positions, chunk, 0.25)
        got = attention_on_matrix_cores(q[positions], k, v, positions, chunk, 0.25, kernel)
        np.testing.assert_allclose(got, ref, atol=0.25, err_msg=f"marked {marked}")
        for t, p in enumerate(positions):
            assert (np.abs(got[t]).mean() > 10.0) == P.sees(p, marked, chunk), (marked, p)


@pytest.mark.parametrize("kernel", [("decode", 1), ("decode", 2), ("prompt", 1), ("prompt", 10 ** 6)])
@pytest.mark.parametrize("H, G, D", [(4, 2, 64), (4, 1, 32), (3, 3, 96), (20, 1, 64), (2, 1, 128)])
def test_two_score_maps_on_the_matrix_cores(H, G, D, kernel):
    rng = np.random.default_rng([H, G, D, 5])
    S = 200
    q, k = bf16_exact(rng.standard_normal((S, H, 2, D))), bf16_exact(rng.standard_normal((S, G, 2, D)))
    k[:, :, 1] *= 4.0
    v = bf16_exact(rng.standard_normal((S, G, D)) + np.arange(G)[None, :, None] * 3.0)
    positions = [0, 1, 63, 64, 65, 199] if kernel[0] == "decode" else list(range(30, 200))
    got = attention_on_matrix_cores(q[positions].reshape(-1, H * 2, D), k.reshape(S, G * 2, D), v, positions, None, 0.2, kernel, maps=2)
    got = got.reshape(len(positions), H, 2, D)
    for m in range(2):
        ref = plain_attention_at(q[positions][:, :, m], k[:, :, m], v, positions, None, 0.2)
        np.testing.assert_allclose(got[:, :, m], ref, atol=0.05, err_msg=f"map {m}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, D, Dv", [(4, 2, 48, 96), (4, 1, 32, 48), (3, 3, 16, 16), (6, 3, 16, 32)])
def test_two_score_maps_over_the_same_values(H, G, D, Dv, dtype):
    """Queries and keys lie head by head as [map 1, map 2]; both maps of a head read the head's group's values. The
    maps' keys differ (one map's keys are scaled so that it looks at one key only), so a kernel that took the other
    map's keys, or another group's values, would show."""
    rng = np.random.default_rng([H, G, D])
    S = 150
    q, k = bf16_exact(rng.standard_normal((S, H, 2, D))), bf16_exact(rng.standard_normal((S, G, 2, D)))
    k[:, :, 1] *= 4.0
    v = bf16_exact(rng.standard_normal((S, G, Dv)) + np.arange(G)[None, :, None] * 3.0)
    positions = [0, 1, 63, 64, 65, 149]
    got = attention_on_gpu(q[positions].reshape(-1, H * 2, D), k.reshape(S, G * 2, D), v, positions, dtype, None, 0.2, maps=2)
    got = got.reshape(len(positions), H, 2, Dv)
    for m in range(2):
        ref = plain_attention_at(q[positions][:, :, m], k[:, :, m], v, positions, None, 0.2)
        np.testing.assert_allclose(got[:, :, m], ref, atol=2e-4 if dtype == "float32" else 0.05, err_msg=f"map {m}")
    if dtype == "bfloat16":
        # the same kernel writes its output in 32-bit beside 16-bit operands: what it rounded before is what differs
        wide = attention_on_gpu(q[positions].reshape(-1, H * 2, D), k.reshape(S, G * 2, D), v, positions, dtype, None, 0.2, maps=2,
                                out_dtype="float32").reshape(got.shape)
        np.testing.assert_array_equal(torch.tensor(wide).to(torch.bfloat16).float().numpy(), got)
        for m in range(2):
            ref = plain_attention_at(q[positions][:, :, m], k[:, :, m], v, positions, None, 0.2)
            np.testing.assert_allclose(wide[:, :, m], ref, atol=2e-4, err_msg=f"map {m} in 32-bit")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_maps_outputs_joined(dtype):
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(8)
    T, H, D, Dpad = 6, 3, 40, 48
    a = np.zeros((T, H, 2, Dpad))
    a[..., :D] = bf16_exact(rng.standard_normal((T, H, 2, D)))
    out = torch.zeros(T, H * Dpad, dtype=TD[dtype], device=DEV)
    K.diff_combine(dev(a.reshape(T, -1), TD[dtype]), out, H, Dpad, D, 0.37, 1e-5, 1 - 0.55)
    ref = P.rms_unit(a[:, :, 0, :D] - 0.37 * a[:, :, 1, :D], 1e-5) * 0.45
    got = host(out).reshape(T, H, Dpad)
    np.testing.assert_allclose(got[..., :D], ref, atol=1e-5 if dtype == "float32" else 0.02)
    assert not got[..., D:].any()
    if dtype == "bfloat16":
        # the maps' outputs in 32-bit, the result in bfloat16; two maps that nearly cancel (lambda close to 1 over
        # nearly equal outputs) keep what 16-bit inputs would lose
        b = a.copy()
        b[:, :, 1, :D] = b[:, :, 0, :D] * (1 + 1e-3 * rng.standard_normal((T, H, D)))
        K.diff_combine(dev(b.reshape(T, -1)), out, H, Dpad, D, 0.999, 1e-5, 0.45)
        ref = P.rms_unit(b[:, :, 0, :D] - 0.999 * b[:, :, 1, :D], 1e-5) * 0.45
        np.testing.assert_allclose(host(out).reshape(T, H, Dpad)[..., :D], ref, atol=0.02)


# ----------------------------------------------------------------- the state space's and the retention's kernels
def scan_reference(q, k, v, a, b, S, heads_per_group):
    """q, k [T, G, N], v [T, H, P], a, b [T, H]; S [H, N, P] is advanced in place. Returns o [T, H, P]."""
    T, H, Pd = v.shape
    o = np.zeros((T, H, Pd))
    for t in range(T):
        for h in range(H):
            g = h // heads_per_group
            S[h] = a[t, h] * S[h] + b[t, h] * np.outer(k[t, g], v[t, h])
            o[t, h] = S[h].T @ q[t, g]
    return o


@pytest.mark.parametrize("H, G, N, P_", [(3, 3, 20, 24), (4, 2, 48, 32), (2, 1, 8, 100), (1, 1, 128, 64), (2, 2, 33, 40),
                                         (1, 1, 200, 16), (2, 1, 16, 300), (6, 6, 32, 64), (1, 1, 1, 1), (1, 1, 256, 64)])
def test_decayed_matrix_whole_and_in_pieces(H, G, N, P_):
    """Three sequences of unequal lengths in one launch, from states that are not zero, whole and cut into pieces down
    to one token; decays and steps per token and head, and per head; the states of slots that no sequence of the step
    owns stay as they are."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([H, N, P_])
    lens, slots, n_slots = [37, 1, 20], [4, 0, 2], 6
    T, off = sum(lens), 12                          # the matrices start behind 12 floats of something else
    q, k = rng.standard_normal((T, G * N + 5)) * 0.5, rng.standard_normal((T, G * N)) * 0.5     # (rows wider than their heads)
    v = rng.standard_normal((T, H * P_))
    a, b = rng.uniform(0.3, 1.0, (T, H)), rng.uniform(0.1, 2.0, (T, H))
    S0 = rng.standard_normal((n_slots, off + H * N * P_))
    cu = np.concatenate([[0], np.cumsum(lens)])
    for per_token in (True, False):
        a_head = rng.uniform(0.5, 0.999, H)
        aa, bb = (a, b) if per_token else (np.broadcast_to(a_head, (T, H)), np.full((T, H), 0.7))
        ref_S, ref_o = S0.copy(), np.zeros((T, H, P_))
        for s, (lo, hi) in enumerate(zip(cu[:-1], cu[1:])):
            Sm = ref_S[slots[s], off:].reshape(H, N, P_)
            ref_o[lo:hi] = scan_reference(q[lo:hi, 5:].reshape(-1, G, N), k[lo:hi].reshape(-1, G, N), v[lo:hi].reshape(-1, H, P_),
                                          aa[lo:hi], bb[lo:hi], Sm, H // G)
        kw = dict(a_tok=dev(aa), b_tok=dev(bb)) if per_token else dict(a_head=dev(a_head), b_const=0.7)
        qd, kd, vd = dev(q), dev(k), dev(v)
        # whole
        state, out = dev(S0), torch.zeros(T, H * P_, device=DEV)
        K.decay_scan(qd, 5, kd, 0, vd, 0, state, off, i32(cu), i32(slots), out, H, H // G, N, P_, **kw)
        scale = max(1.0, np.abs(ref_o).max())
        np.testing.assert_allclose(host(out).reshape(T, H, P_), ref_o, atol=2e-5 * scale)
        np.testing.assert_allclose(host(state), ref_S, atol=2e-5 * max(1.0, np.abs(ref_S).max()))
        # in pieces: the first sequence in steps of 1, 2, 16, 17 and the rest, the third in two
        state, got = dev(S0), np.zeros((T, H * P_))
        for s, cuts in ((0, [1, 3, 19, 36, 37]), (1, [1]), (2, [7, 20])):
            lo = 0
            for hi in cuts:
                rows = slice(int(cu[s]) + lo, int(cu[s]) + hi)
                piece = torch.zeros(hi - lo, H * P_, device=DEV)
                pk = ({"a_tok": kw["a_tok"][rows], "b_tok": kw["b_tok"][rows]} if per_token else kw)
                K.decay_scan(qd[rows], 5, kd[rows], 0, vd[rows], 0, state, off, i32([0, hi - lo]), i32([slots[s]]), piece,
                             H, H // G, N, P_, **pk)
                got[rows] = host(piece)
                lo = hi
        np.testing.assert_allclose(got.reshape(T, H, P_), ref_o, atol=2e-5 * scale)
        np.testing.assert_allclose(host(state), ref_S, atol=2e-5 * max(1.0, np.abs(ref_S).max()))


def test_decayed_matrix_reads_what_was_written_hundreds_of_tokens_ago():
    """One token writes a value under a key of its own; 600 tokens later (other keys in between, a decay close to one)
    a query along that key reads it back, scaled by the decays' product."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(3)
    T, N, P_ = 640, 32, 16
    k = rng.standard_normal((T, N)) * 0.05
    k[:, 0] = 0.0
    k[20] = 0.0
    k[20, 0] = 1.0
    v = rng.standard_normal((T, P_)) * 0.05
    v[20] = 7.0
    q = np.zeros((T, N))
    q[620, 0] = 1.0
    out, state = torch.zeros(T, P_, device=DEV), torch.zeros(2, N * P_, device=DEV)
    K.decay_scan(dev(q), 0, dev(k), 0, dev(v), 0, state, 0, i32([0, T]), i32([1]), out, 1, 1, N, P_, a_head=dev([0.999]),
                 b_const=1.0)
    np.testing.assert_allclose(host(out)[620], 7.0 * 0.999 ** 600 * np.ones(P_), rtol=2e-4)
    assert not host(state)[0].any()


@pytest.mark.parametrize("H, G, N, P_, lens", [(2, 1, 24, 40, [700, 33, 1, 515]), (5, 5, 16, 16, [129]), (1, 1, 128, 64, [97, 640]),
                                               (3, 1, 33, 300, [260, 259])])
def test_decayed_matrix_of_a_long_step_in_pieces_side_by_side(H, G, N, P_, lens):
    """With scratch for the pieces' start states a long step runs as pieces side by side: sequences of unequal
    lengths (one of a single token, one shorter than a piece, some that end inside a piece) from states that are not
    zero give the read-outs and end states of the token-by-token recurrence, with decays per token (some of them
    close to zero, so that a piece's product of decays underflows) and per head; other slots stay as they are."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([H, N, P_, len(lens)])
    n_slots, off = len(lens) + 2, 8
    slots = list(rng.permutation(n_slots)[:len(lens)])
    T = sum(lens)
    piece = K.scan_piece_len(max(lens), len(lens), H)
    assert piece and max(lens) > piece and any(n % piece for n in lens)
    q, k = rng.standard_normal((T, G * N)) * 0.3, rng.standard_normal((T, G * N)) * 0.3
    v = rng.standard_normal((T, H * P_))
    a, b = rng.uniform(0.8, 1.0, (T, H)), rng.uniform(0.1, 1.0, (T, H))
    a[rng.random((T, H)) < 0.02] = 1e-30
    S0 = rng.standard_normal((n_slots, off + H * N * P_))
    cu = np.concatenate([[0], np.cumsum(lens)])
    scratch = torch.full((K.scan_pieces_floats(max(lens), len(lens), H, N, P_),), float("nan"), device=DEV)
    for per_token in (True, False):
        a_head = rng.uniform(0.9, 0.999, H)
        aa, bb = (a, b) if per_token else (np.broadcast_to(a_head, (T, H)), np.full((T, H), 0.4))
        ref_S, ref_o = S0.copy(), np.zeros((T, H, P_))
        for s, (lo, hi) in enumerate(zip(cu[:-1], cu[1:])):
            Sm = ref_S[slots[s], off:].reshape(H, N, P_)
            ref_o[lo:hi] = scan_reference(q[lo:hi].reshape(-1, G, N), k[lo:hi].reshape(-1, G, N), v[lo:hi].reshape(-1, H, P_),
                                          aa[lo:hi], bb[lo:hi], Sm, H // G)
        kw = dict(a_tok=dev(aa), b_tok=dev(bb)) if per_token else dict(a_head=dev(a_head), b_const=0.4)
        state, out = dev(S0), torch.zeros(T, H * P_, device=DEV)
        K.decay_scan(dev(q), 0, dev(k), 0, dev(v), 0, state, off, i32(cu), i32(slots), out, H, H // G, N, P_,
                     pieces=scratch, max_len=max(lens), **kw)
        scale = max(1.0, np.abs(ref_o).max())
        np.testing.assert_allclose(host(out).reshape(T, H, P_), ref_o, atol=3e-5 * scale)
        np.testing.assert_allclose(host(state), ref_S, atol=3e-5 * max(1.0, np.abs(ref_S).max()))


def test_a_marked_key_is_read_across_many_pieces():
    """One token writes a value under a key of its own in the step's second piece; a query in a far later piece reads
    it back scaled by the product of the decays in between, through the pieces' joined start states."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(5)
    T, N, P_ = 1500, 32, 16
    piece = K.scan_piece_len(T, 1, 1)
    w, r = piece + 3, T - piece - 7
    k = rng.standard_normal((T, N)) * 0.05
    k[:, 0] = 0.0
    k[w] = 0.0
    k[w, 0] = 1.0
    v = rng.standard_normal((T, P_)) * 0.05
    v[w] = 7.0
    q = np.zeros((T, N))
    q[r, 0] = 1.0
    out, state = torch.zeros(T, P_, device=DEV), torch.zeros(2, N * P_, device=DEV)
    scratch = torch.zeros(K.scan_pieces_floats(T, 1, 1, N, P_), device=DEV)
    K.decay_scan(dev(q), 0, dev(k), 0, dev(v), 0, state, 0, i32([0, T]), i32([1]), out, 1, 1, N, P_, a_head=dev([0.999]),
                 b_const=1.0, pieces=scratch, max_len=T)
    np.testing.assert_allclose(host(out)[r], 7.0 * 0.999 ** (r - w) * np.ones(P_), rtol=3e-4)
    assert not host(state)[0].any()


@pytest.mark.parametrize("taps", [1, 2, 4, 5])
def test_short_convolution_across_steps(taps):
    """The last taps - 1 inputs of a sequence are part of its state: a prompt in pieces of 1, 2 and more tokens (fewer
    than the taps, and more) gives what the whole prompt gives; before a sequence's start stand zeros; decay and step
    size per head come out of the same launch."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(taps)
    C, H, T, n_slots, off = 300, 3, 23, 4, 8
    ld = 7 + C + H + 3
    proj = rng.standard_normal((T, ld))
    w, bias = rng.standard_normal((C, taps)) * 0.5, rng.standard_normal(C) * 0.2
    A_log, dt_bias = rng.uniform(-2, 1, H), rng.uniform(-3, 30, H)
    x = proj[:, 7:7 + C]
    padded = np.concatenate([np.zeros((taps - 1, C)), x])
    ref = P.silu(np.stack([(padded[t:t + taps] * w.T).sum(0) + bias for t in range(T)]))
    dt = P.softplus(proj[:, 7 + C:7 + C + H] + dt_bias)
    held = (taps - 1) * C
    S0 = rng.standard_normal((n_slots, off + held + 5))
    S0[2, off:off + held] = 0.0                       # a slot as it is handed out
    for cuts in ([T], [1, 2, 3, 5, 6, 10, 11, 23]):
        state, lo = dev(S0), 0
        act, ab = np.zeros((T, C)), np.zeros((T, 2 * H))
        for hi in cuts:
            a_, ab_ = torch.zeros(hi - lo, C, device=DEV), torch.zeros(hi - lo, 2 * H, device=DEV)
            K.ssm_prep(dev(proj[lo:hi]), 7, C, 7 + C, H, dev(w), dev(bias), dev(A_log), dev(dt_bias), state, off,
                       i32([0, hi - lo]), i32([0] * (hi - lo)), i32([2]), a_, ab_)
            act[lo:hi], ab[lo:hi] = host(a_), host(ab_)
            lo = hi
        np.testing.assert_allclose(act, ref, atol=2e-5)
        np.testing.assert_allclose(ab[:, H:], dt, rtol=1e-5, atol=1e-7)
        np.testing.assert_allclose(ab[:, :H], np.exp(-np.exp(A_log) * dt), rtol=1e-4, atol=1e-7)
        after = host(state)
        if taps > 1:
            np.testing.assert_allclose(after[2, off:off + held].reshape(taps - 1, C), padded[T:], atol=1e-6)
        after[2, off:off + held] = S0[2, off:off + held]
        np.testing.assert_allclose(after, S0.astype(np.float32))          # nothing else was touched


@pytest.mark.parametrize("dtype", DTYPES)
def test_gate_and_unit_norm_in_both_orders(dtype):
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(12)
    T, H, Pd, parts = 5, 6, 20, 3
    C = H * Pd
    o, gate_rows, xs = rng.standard_normal((T, C)) * 3, rng.standard_normal((T, C + 9)), rng.standard_normal((T, 4 + C))
    w, D = 1 + 0.2 * rng.standard_normal(C), rng.standard_normal(H)
    out = torch.zeros(T, C, dtype=TD[dtype], device=DEV)
    tol = 2e-5 if dtype == "float32" else 0.05
    # the gate first, then the norm in equal parts, with a weight and the skipped input: the state space's
    K.group_norm_gate(dev(o), dev(gate_rows), 9, out, C // parts, 1e-5, weight=dev(w), gate_first=True, skip=(dev(xs), 4, dev(D), Pd))
    y = (o + np.repeat(D, Pd)[None] * xs[:, 4:]) * P.silu(gate_rows[:, 9:])
    ref = P.rms_unit(y.reshape(T, parts, -1), 1e-5).reshape(T, C) * w
    np.testing.assert_allclose(host(out), ref, atol=tol)
    # the norm per head first, then the gate, no weight: the retention's
    K.group_norm_gate(dev(o), dev(gate_rows), 9, out, Pd, 1e-5)
    ref = P.rms_unit(o.reshape(T, H, Pd), 1e-5).reshape(T, C) * P.silu(gate_rows[:, 9:])
    np.testing.assert_allclose(host(out), ref, atol=tol)


# ----------------------------------------------------------------- the routed feed-forward's kernels
def test_router_choice_ties_weights_and_runs():
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(4)
    T, E = 70, 7
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[0] = 1.0                                  # all equal: the lowest numbers win
    logits[1, [2, 5]] = 3.0                          # a tie between the two largest
    logits[2, [6, 1, 3]] = [2.0, 2.0, 2.0]
    for top in (1, 2, 3, 7):
        idx, wts = torch.zeros(T, top, dtype=torch.int32, device=DEV), torch.zeros(T, top, device=DEV)
        offsets, pairs = torch.zeros(E + 1, dtype=torch.int32, device=DEV), torch.zeros(T * top, dtype=torch.int32, device=DEV)
        K.route(dev(logits), top, idx, wts, offsets, pairs)
        idx, wts, offsets, pairs = idx.cpu().numpy(), host(wts), offsets.cpu().numpy(), pairs.cpu().numpy()
        for t in range(T):
            order = np.argsort(-logits[t], kind="stable")[:top]
            assert list(idx[t]) == list(order), (top, t)
            np.testing.assert_allclose(wts[t], P.softmax(logits[t, order].astype(np.float64)), atol=1e-6)
        assert offsets[0] == 0 and offsets[-1] == T * top and sorted(pairs) == list(range(T * top))
        for e in range(E):
            assert all(idx.reshape(-1)[p] == e for p in pairs[offsets[e]:offsets[e + 1]])
    # one more expert that every token passes, with weight 1, behind a token's choices: in a small step (one launch) and
    # in a larger one
    for n, top in ((70, 2), (9, 3), (1, 1)):
        per = top + 1
        idx, wts = torch.zeros(n, per, dtype=torch.int32, device=DEV), torch.zeros(n, per, device=DEV)
        offsets, pairs = torch.zeros(E + 2, dtype=torch.int32, device=DEV), torch.zeros(n * per, dtype=torch.int32, device=DEV)
        K.route(dev(logits[:n]), top, idx, wts, offsets, pairs, always=True)
        idx, wts, offsets, pairs = idx.cpu().numpy(), host(wts), offsets.cpu().numpy(), pairs.cpu().numpy()
        for t in range(n):
            order = np.argsort(-logits[t], kind="stable")[:top]
            assert list(idx[t]) == list(order) + [E], (top, t)
            np.testing.assert_allclose(wts[t], list(P.softmax(logits[t, order].astype(np.float64))) + [1.0], atol=1e-6)
        assert offsets[0] == 0 and offsets[-1] == n * per and sorted(pairs) == list(range(n * per))
        assert sorted(pairs[offsets[E]:]) == [t * per + top for t in range(n)]
        for e in range(E + 1):
            assert all(idx.reshape(-1)[p] == e for p in pairs[offsets[e]:offsets[e + 1]])


@pytest.mark.parametrize("dtype, mfma", [("float32", False), ("bfloat16", False), ("bfloat16", True)])
@pytest.mark.parametrize("E, top, T, d, F", [(5, 2, 90, 96, 40), (3, 3, 7, 64, 72), (11, 2, 300, 128, 88), (4, 1, 1, 80, 48), (6, 2, 3, 256, 33),
                                             (4, 2, 700, 200, 136), (2, 1, 1000, 72, 264), (8, 2, 8, 1024, 520), (3, 2, 40, 2056, 48),
                                             (2, 2, 64, 320, 24), (4, 2, 50, 256, 136), (4, 2, 100, 192, 64), (2, 1, 24, 136, 72)])
def test_experts_products_over_runs_of_pairs(E, top, T, d, F, dtype, mfma):
    """Runs of unequal lengths, experts that nobody chose, more pairs than a tile holds, one token; each pair's hidden
    row and output against the plain expert of its choice."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([E, T, d])
    h = bf16_exact(rng.standard_normal((T, d)))
    up, down = bf16_exact(rng.standard_normal((E, F, d)) / np.sqrt(d)), bf16_exact(rng.standard_normal((E, d, F)) / np.sqrt(F))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, E - 1] = -50.0 if E > top else logits[:, E - 1]             # the last expert is never chosen
    idx, wts = torch.zeros(T, top, dtype=torch.int32, device=DEV), torch.zeros(T, top, device=DEV)
    offsets, pairs = torch.zeros(E + 1, dtype=torch.int32, device=DEV), torch.zeros(T * top, dtype=torch.int32, device=DEV)
    K.route(dev(logits), top, idx, wts, offsets, pairs)
    hidden = torch.zeros(T * top, F, dtype=TD[dtype], device=DEV)
    K.expert_gemm(dev(h, TD[dtype]), dev(up, TD[dtype]), hidden, act="gelu", offsets=offsets, pairs=pairs, a_div=top, mfma=mfma)
    outs = torch.zeros(T * top, d, device=DEV)
    K.expert_gemm(hidden, dev(down, TD[dtype]), outs, offsets=offsets, pairs=pairs, mfma=mfma)
    y = torch.full((T, d), 2.0, device=DEV)
    K.route_combine(outs, wts, y, accumulate=True)
    choice, w = idx.cpu().numpy(), host(wts)
    ref_hidden = np.stack([P.gelu_erf(up[choice[t, j]] @ h[t]) for t in range(T) for j in range(top)])
    tol = 2e-5 if dtype == "float32" else 0.03
    np.testing.assert_allclose(host(hidden), ref_hidden, atol=tol)
    ref_out = np.stack([down[choice[t, j]] @ host(hidden)[t * top + j] for t in range(T) for j in range(top)])
    np.testing.assert_allclose(host(outs), ref_out, atol=tol * 3)
    ref_y = 2.0 + (w[:, :, None] * ref_out.reshape(T, top, d)).sum(1)
    np.testing.assert_allclose(host(y), ref_y, atol=tol * 3)
    # one expert over every row in its own order: the expert that every token passes
    dense = torch.zeros(T, F, dtype=TD[dtype], device=DEV)
    K.expert_gemm(dev(h, TD[dtype]), dev(up[:1], TD[dtype]), dense, act="gelu", mfma=mfma)
    np.testing.assert_allclose(host(dense), P.gelu_erf(h @ up[0].T), atol=tol)


# ----------------------------------------------------------------- whole models through the engine
def plain_trace(cfg, W, toks):
    return P.Sequence(cfg, W).feed(toks)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompt_and_every_layer(name, dtype):
    eng, cfg, W = engine(name, dtype)
    toks = tokens(name, 1, 210)                       # beyond every chunk, over four pages
    ref, trace = plain_trace(cfg, W, toks)
    seen = []
    eng.after_block = lambda i, x: seen.append(x.float().cpu().numpy())
    s = eng.take_slot()
    got = eng.step([(s, toks)], want="all").cpu().numpy()
    eng.after_block = None
    assert len(seen) == len(trace) == len(cfg["layers"])
    for r, (a, b) in enumerate(zip(seen, trace)):     # the first layer that differs names the mechanism
        np.testing.assert_allclose(a, b, atol=(8e-5 if dtype == "float32" else 4e-2 * LOOSER.get(name, 1.0)) * np.abs(b).max(),
                                   err_msg=f"layer {r}")
    close(got, ref, dtype, name)
    # the first tokens of a sequence, each alone from an empty slot
    for n in (1, 2, 3):
        s2 = eng.take_slot()
        close(eng.step([(s2, toks[:n])], want="all").cpu().numpy(), ref[:n], dtype, f"{name} first {n}")
        eng.give_back_slot(s2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_every_sublayer_alone(name, dtype):
    """Each mixer's and each feed-forward's output against the plain one computed from the plain rows in front of it:
    a fault does not hide behind the layers before it."""
    eng, cfg, W = engine(name, dtype)
    toks = tokens(name, 6, 75)
    seq = P.Sequence(cfg, W)
    x = seq.W["embed"][toks]
    want = {}
    for i, (lay, mixer) in enumerate(zip(cfg["layers"], seq.mixers)):
        p = f"l{i}."
        want[(i, "mixer")] = mixer.forward(seq.W, x, 0)
        x = x + P.layer_norm(want[(i, "mixer")], seq.W[p + "norm1"], seq.W[p + "norm1.b"], seq.eps)
        if lay.get("mlp") is not None:
            want[(i, "ffn")] = P.routed_feed_forward(seq.W, p + "mlp.", lay["mlp"], x)
            x = x + P.layer_norm(want[(i, "ffn")], seq.W[p + "norm2"], seq.W[p + "norm2.b"], seq.eps)
    seen = {}
    eng.after_sublayer = lambda e, kind, t: seen.__setitem__((e, kind), t.float().cpu().numpy())
    eng.step([(eng.take_slot(), toks)], want="none")
    eng.after_sublayer = None
    for key, ref in want.items():
        scale = np.sqrt((ref ** 2).mean())
        np.testing.assert_allclose(seen[key], ref, atol=(2e-4 if dtype == "float32" else 0.12 * LOOSER.get(name, 1.0)) * max(scale, 1e-3),
                                   err_msg=str(key))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prompt_then_token_by_token(name, dtype):
    """Decoding passes every chunk's edge and two page borders; the decoded rows are those of the whole prompt."""
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


def test_a_chunked_layer_gives_pages_back_and_reads_none_of_them():
    """The cache of a chunked attention holds the current chunk only: pages in front of it go back to the pool as the
    sequence grows, are used again by another sequence, and the logits stay those of the plain implementation."""
    eng, cfg, W = engine("reordered", "float32", n_slots=3, max_tokens=640)
    toks, other = tokens("reordered", 40, 400), tokens("reordered", 41, 100)
    ref, ref_other = P.forward(cfg, W, toks), P.forward(cfg, W, other)
    a = eng.take_slot()
    rows = [eng.step([(a, toks[:150])], want="all").cpu().numpy()]
    chunked = [g for g, group in enumerate(eng.cache.groups) if group.need.chunk]
    assert chunked
    for g in chunked:                                # chunks of 9 and of 64: only the last pages are still held
        held = [p for p in eng.cache.slots.pages[a][g] if p]
        assert len(held) <= 2, (g, held)
    b = eng.take_slot()
    rows_b = [eng.step([(b, other[:60])], want="all").cpu().numpy()]
    for j in range(150, 400):
        entries = [(a, [toks[j]])] + ([(b, [other[60 + j - 150]])] if 60 + j - 150 < 100 else [])
        out = eng.step(entries).cpu().numpy()
        rows.append(out[:1])
        if len(entries) > 1:
            rows_b.append(out[1:])
    close(np.concatenate(rows), ref, "float32", "the long request")
    close(np.concatenate(rows_b), ref_other, "float32", "the one that took its pages")


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
    """Sizes, counts, order of layers, chunks and constants drawn from a seed: what no hand-made configuration
    happened to combine."""
    rng = np.random.default_rng([seed, 77])
    pick = lambda xs: xs[int(rng.integers(len(xs)))]
    width = pick([40, 64, 72, 90, 128, 200])
    n_layers = int(rng.integers(2, 7))

    def rot(dim):
        return {"base": pick([100.0, 10000.0, 250000.0, 1e6]), "dims": pick([d for d in (2, 4, 8, 16, 24, 32, 48, 64, 96, 128) if d <= dim])}

    layers, owners = [], []
    for i in range(n_layers):
        mlp = None
        if rng.random() < 0.8:
            experts = pick([1, 2, 3, 5, 8, 12])
            mlp = {"kind": "moe", "router": {"experts": experts, "top": int(rng.integers(1, min(experts, 4) + 1))},
                   "expert": {"ff": pick([16, 24, 40, 64, 96])}, "shared": pick([None, {"ff": 32}, {"ff": 72}])}
        kind = pick(["mamba2", "parallel", "attention", "attention"])
        if kind == "mamba2":
            heads = pick([1, 2, 3, 4, 6])
            vdim = pick([8, 16, 24, 32, 64])
            m = {"heads": heads, "vdim": vdim, "state": pick([4, 16, 20, 48, 64, 128]), "groups": pick([g for g in (1, 2, 3, 6) if heads % g == 0]),
                 "conv": pick([2, 3, 4]), "norm_groups": pick([g for g in (1, 2, 3, 4, 8) if (heads * vdim) % g == 0])}
        elif kind == "parallel":
            heads = pick([1, 2, 3, 4, 6, 8])
            dim, rdim = pick([8, 16, 24, 32, 40, 64, 96]), pick([8, 16, 20, 32, 64])
            left = {"heads": heads, "kv_heads": pick([k for k in (1, 2, 3, 4, 6, 8) if heads % k == 0]), "dim": dim,
                    "vdim": pick([8, 16, 24, 32, 48, 64, 96]), "scale": float(pick([0.1, 0.2, dim ** -0.5])), "rot": rot(dim)}
            if rng.random() < 0.85:
                left["mask"] = {"size": pick([1, 2, 7, 31, 32, 64, 65, 100, 150, 500])}
            rh = pick([1, 2, 3, 4])
            right = {"heads": rh, "dim": rdim, "vdim": pick([8, 16, 24, 40, 64]), "rot": rot(rdim),
                     "decay": [float(1 - 2.0 ** -rng.integers(2, 11)) for _ in range(rh)]}
            m = {"left": left, "right": right, "left_scale": float(pick([0.5, 0.6, 1.0, 1.5])), "right_scale": float(pick([0.4, 1.0, 1.1]))}
        else:
            if owners and rng.random() < 0.45:
                j = pick(owners)
                o = layers[j]["mixer"]
                m = {"heads": o["kv_heads"] * pick([1, 2, 3]), "kv_heads": o["kv_heads"], "dim": o["dim"], "vdim": o["vdim"],
                     "scale": float(pick([0.1, 0.15, 0.3])), "diff": float(pick([0.2, 0.6, 0.8])), "rot": dict(o["rot"]), "kv_from": j}
            else:
                heads = pick([1, 2, 3, 4, 6])
                dim = pick([8, 16, 24, 32, 48, 64])
                m = {"heads": heads, "kv_heads": pick([k for k in (1, 2, 3, 6) if heads % k == 0]), "dim": dim,
                     "vdim": pick([8, 16, 24, 32, 48, 96]), "scale": float(pick([0.1, 0.15, dim ** -0.5])),
                     "diff": float(pick([0.2, 0.5, 0.6, 0.8])), "rot": rot(dim)}
                owners.append(i)
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    return {"architecture": "Nolatar", "vocab": int(rng.integers(50, 700)), "width": width, "norm": {"eps": pick([1e-5, 1e-6])},
            "layers": layers}


def close_mostly(got, ref, dtype, what):
    """32-bit: every row within the bound. bfloat16: a drawn configuration may run six layers over a width of 40, where
    single rows gather more rounding than the hand-made models' bound allows for: at most one row in fifty beyond the
    bound, none beyond twice the bound (a fault moves whole runs of rows by many times that)."""
    if dtype == "float32":
        return close(got, ref, dtype, what)
    e = row_errors(got, ref)
    assert (e > 2 * TOL[dtype]).sum() == 0 and (e > TOL[dtype]).sum() <= max(1, len(e) // 50), \
        f"{what}: {int((e > TOL[dtype]).sum())} of {len(e)} rows over {TOL[dtype]}, the worst {e.max():.3e}"


@pytest.mark.parametrize("seed", range(10))
def test_seeded_random_configurations(seed, tmp_path):
    from gpullama3_java_amd.engine import Engine
    cfg = random_config(seed)
    W = P.make_weights(cfg, seed)
    write_model(str(tmp_path), cfg, W)
    prompts = [P.tokens_with_clear_choices(cfg, W, 100 * seed + i, n) for i, n in enumerate((172, 1, 40))]
    refs = [P.forward(cfg, W, p) for p in prompts]
    for dtype in DTYPES:
        eng = Engine.from_folder(str(tmp_path), dtype=dtype, max_tokens=1024, n_slots=4)
        # whole; the last 40 tokens one by one; three unequal requests in one batch, then together token by token
        s = eng.take_slot()
        close_mostly(eng.step([(s, prompts[0])], want="all").cpu().numpy(), refs[0], dtype, f"seed {seed} whole")
        eng.give_back_slot(s)
        s = eng.take_slot()
        rows = [eng.step([(s, prompts[0][:132])], want="all").cpu().numpy()]
        for t in prompts[0][132:]:
            rows.append(eng.step([(s, [t])]).cpu().numpy())
        close_mostly(np.concatenate(rows), refs[0], dtype, f"seed {seed} decoded")
        eng.give_back_slot(s)
        slots = [eng.take_slot() for _ in prompts]
        cut = [150, 1, 20]
        got = eng.step([(slots[i], prompts[i][:cut[i]]) for i in range(3)], want="all").cpu().numpy()
        lo = 0
        for i in range(3):
            close_mostly(got[lo:lo + cut[i]], refs[i][:cut[i]], dtype, f"seed {seed} batch prompt {i}")
            lo += cut[i]
        for step in range(20):
            live = [i for i in range(3) if cut[i] + step < len(prompts[i])]
            got = eng.step([(slots[i], [prompts[i][cut[i] + step]]) for i in live]).cpu().numpy()
            for r, i in enumerate(live):
                close_mostly(got[r:r + 1], refs[i][cut[i] + step:cut[i] + step + 1], dtype, f"seed {seed} batch step {step} request {i}")
        del eng

"""ctypes bindings of the HIP library, with the host-side checks every launch needs.

Each wrapper checks, before anything reaches the GPU, that its tensors live on the
device, are contiguous where the kernel assumes it, have the dtypes and shapes the
kernel's indexing assumes, and that index tensors are int32. There is no CPU
fallback: without a GPU, or without the library, the call raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_uint32, c_void_p

import torch

from . import build as _build

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}
EPI_STORE, EPI_ADD, EPI_GATED = 0, 1, 2
ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "quick_gelu": 2}     # the gated epilogue's activation
FAST_ACTIVATIONS = ("silu", "gelu_tanh")     # what the matrix-core products' gated epilogues apply

_lib = None


class KernelError(RuntimeError):
    pass


def library():
    """The loaded library; built first if no build matches the sources."""
    global _lib
    if _lib is None:
        path = _build.library_path() or _build.build()
        lib = ctypes.CDLL(path)
        lib.gl3_last_error.restype = ctypes.c_char_p
        _declare(lib)
        _lib = lib
    return _lib


def library_file():
    library()
    return _build.library_path()


def _declare(lib):
    P, I, L, F = c_void_p, c_int, c_long, c_float
    sigs = {
        "gl3_abi_version": [],
        "gl3_fill_u32": [P, c_uint32, L, P],
        "gl3_embed": [P, I, P, P, I, I, P, P, P, F, P, P, I, P],
        "gl3_scale_f32": [P, F, L, P],
        "gl3_softcap_f32": [P, F, L, P],
        "gl3_rmsnorm": [P, P, P, I, P, I, I, I, F, P],
        "gl3_gather_rows": [P, P, P, I, I, I, P],
        "gl3_add_slices_rmsnorm": [P, P, P, I, L, L, P, I, P, I, I, I, F, P],
        "gl3_rope_cache_write": [P, I, P, P, P, I, P, P, P, P, I, I, I, I, I, I, I, I, P],
        "gl3_gemm_generic": [P, I, P, I, P, I, I, I, I, L, L, L, I, P, I, I, P, F, F, P, P],
        "gl3_attention_generic": [P, L, P, P, I, P, P, P, I, P, L, I, I, I, I, I, I, F, I, P, I, F, I, I, I, I, P, I, P],
        "gl3_pair_rows": [P, P, P, P, P, P, L, L, L, L, P, I, P],
        "gl3_concat_rows": [P, P, P, I, I, I, P],
        "gl3_rotate_heads": [P, I, L, P, I, P, P, P, P, P, P, I, I, I, P, L, I, P, P, P, P, I, I, P, P, F, P],
        "gl3_diff_combine": [P, I, L, P, L, I, I, I, I, I, F, F, F, P],
        "gl3_layernorm": [P, P, P, P, P, I, I, I, F, P],
        "gl3_layernorm_add": [P, P, P, P, I, I, F, P, I, P],
        "gl3_cast_rows": [P, P, I, L, P],
        "gl3_ssm_prep": [P, L, I, I, I, I, I, I, P, P, I, P, P, P, L, L, P, P, P, P, P, P],
        "gl3_decay_scan": [P, L, I, P, L, I, P, L, I, P, P, L, P, F, P, L, L, P, P, P, L, I, I, I, I, I, P, L, I, I, I, P],
        "gl3_group_norm_gate": [P, P, L, I, P, I, P, L, I, P, F, I, I, I, I, P, I, I, P],
        "gl3_route": [P, I, I, I, P, P, P, P, I, I, P, F, P],
        "gl3_expert_gemm": [P, I, L, I, P, I, I, I, I, P, P, I, P, I, L, I, I, I, F, F, P],
        "gl3_route_combine": [P, P, I, I, I, P, I, P, I, P, I, P],
        "gl3_streams_step": [P, I, I, I, P, P, P, P, P, F, P, I, P],
        "gl3_streams_fill": [P, P, I, I, I, P],
        "gl3_streams_sum": [P, P, I, I, I, P, P],
        "gl3_latent_prep": [P, L, I, I, I, I, I, I, P, P, F, P, P, P, I, P, P, P, P, I, I, I, I, P, P, P],
        "gl3_latent_query": [P, I, I, I, I, I, P, P, P, P, I, I, P],
        "gl3_sigmoid_gate": [P, I, P, L, I, I, I, P],
        "gl3_latent_attention_supports": [I, I, I],
        "gl3_latent_attention": [P, L, P, P, P, P, P, I, P, L, I, I, I, I, I, I, I, F, I, P, P, L, P],
        "gl3_sides_norm_add": [P, P, P, P, P, F, F, I, I, P, P, P, P],
        "gl3_tanh_rows": [P, L, I, P, I, L, P],
        "gl3_mingru_scan": [P, L, I, P, L, P, P, P, I, I, I, P, P],
        "gl3_shift_mix": [P, I, I, P, I, P, L, P, P, P, P, I, I, I, P],
        "gl3_timemix": [P, P, P, L, P, L, P, P, L, L, P, P, P, I, I, I, P, L, P, F, P, I, I, P],
        "gl3_head_norm_gate": [P, P, P, F, P, I, I, I, I, P],
        "gl3_kv_write": [P, I, L, I, I, P, P, P, I, P, P, I, I, I, I, I, P],
        "gl3_residual_inject": [P, P, P, I, I, P],
        "gl3_delta_state_floats": [I, I, I, I, I],
        "gl3_delta_prep": [P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, I, I, I, I, I, L, F, F, I, P],
        "gl3_delta_recurrence": [P, P, P, P, P, P, P, I, I, P, P, I, F, I, I, I, I, I, I, I, L, P],
        "gl3_sample": [P, L, P, P, P, P, P, I, I, P, I, P],
        "gl3_sample_work_floats": [I, I],
        "gl3_argmax": [P, L, P, P, I, I, P],
        "gl3_argmax_advance": [P, L, P, P, I, I, P, P, P, P, I, P, P],
        "gl3_argmax_static": [P, L, P, I, I, P],
        "gl3_decode_advance": [P, P, P, P, P, I, P, I, P],
        "gl3_gemm_skinny": [P, P, P, I, I, I, I, L, L, L, I, I, P, I, P, P, L, P, I, P, P, I, F, F, P, P],
        "gl3_gemm_skinny_wide": [P, P, P, I, I, I, I, L, L, L, I, I, L, I, P, I, P, I, F, I, I, F, F, P, P],
        "gl3_gemm_skinny_norm": [P, P, P, I, F, P, P, I, I, I, I, L, L, L, I, I, P, I, P, I, F, F, P, P],
        "gl3_qkv_rope_cache": [P, P, I, F, P, P, L, I, I, L, L, P, P, P, I, P, P, P, P, I, I, I, I, I, I, P, P, P, I, P],
        "gl3_token_facts": [P, P, P, I, I, P, P, I, P, P, P, I, P],
        "gl3_gemm_mfma": [P, P, P, I, I, I, I, L, L, L, I, I, P, L, L, P, I, I, I, P, F, F, P, P],
        "gl3_attention_decode_supports": [I, I],
        "gl3_attention_prefill_supports": [I, I],
        "gl3_attention_prefill": [P, L, P, P, P, P, P, P, I, P, L, I, I, I, I, I, I, I, F, I, P, I, F, I, I, I, P, P],
        "gl3_scatter_i32": [P, L, P, P, I, P],
        "gl3_upload": [P, P, L, P],
        "gl3_stage_decode": [P, I, I, P, P, P, I, P, P],
        "gl3_stage_step": [P, P, P, I, P, P, P, I, P, I, I, P],
        "gl3_graph_launch": [P, P],
        "gl3_attention_decode": [P, L, P, P, P, P, P, I, P, P, L, P, L, I, I, I, I, I, I, F, I, P, I, F, I, I, I, P, P],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name, None)
        if fn is None:
            continue
        fn.argtypes = args
        fn.restype = c_int
    lib.gl3_sample_work_floats.restype = ctypes.c_long
    lib.gl3_delta_state_floats.restype = ctypes.c_long
    lib._optional = set()


def has(name):
    return hasattr(library(), name)


def _check(rc, name):
    if rc != 0:
        raise KernelError(f"{name}: {library().gl3_last_error().decode()}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current stream of the current device (asked for at every launch: a graph capture changes it).
    The raw handle where this torch offers it: building a stream object costs as much as a launch."""
    if _raw_stream is not None and _raw_device is not None:
        return c_void_p(_raw_stream(_raw_device()))
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t, name, dtype=None, contiguous=True):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name} must be a tensor on the GPU (the kernels have no CPU path)")
    if dtype is not None and t.dtype not in (dtype if isinstance(dtype, tuple) else (dtype,)):
        raise KernelError(f"{name} has dtype {t.dtype}, expected {dtype}")
    if contiguous and not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    return t


def held_once(w):
    """Whether the matrix is kept in the matrix cores' order ALONE (``hold_once``): its memory is one of its
    copies (``w.tiled``, ``w.tiled8``), and only what reads such an order may touch it."""
    return getattr(w, "operand_order_only", False)


def _w_order(w):
    """How a weight lies, for the kernels that read any order: (0, the stored rows, no table), (1, the copy in
    the operands' order, each row's place in it or nothing), (2, the copy in packed strips of 8 rows, nothing)."""
    if not held_once(w):
        return 0, _ptr(w), c_void_p(0)
    t = getattr(w, "tiled", None)
    if t is not None:
        return 1, _ptr(t), _ptr(getattr(t, "row_pos", None))
    return 2, _ptr(w.tiled8), c_void_p(0)


def _code(t, name):
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"{name} has dtype {t.dtype}; the kernels take float32 and bfloat16") from None


def _ptr(t):
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(0)


def _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, who, v_head_dim=None, n_v=None):
    """Keys [pages, kv heads, page, head_dim]; values transposed [pages, kv heads, head_dim, page]; inside a
    page both lie in the kernels' tiles (``cache/layout.py``), which needs pages of a multiple of 32 positions
    and heads of a multiple of 16 elements. ``v_head_dim``: the values' size where a kernel takes another than the keys'."""
    vd = head_dim if v_head_dim is None else v_head_dim
    if vd % 16:
        raise KernelError(f"{who}: values of {vd} elements are not a multiple of 16")
    if (k_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (n_kv, page_size, head_dim)
            or tuple(v_cache.shape) != (k_cache.shape[0], n_kv if n_v is None else n_v, vd, page_size)):
        raise KernelError(f"{who}: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} for kv {n_kv} "
                          f"page {page_size} hs {head_dim}")
    if page_size % 32 or head_dim % 16:
        raise KernelError(f"{who}: the cache lies in tiles: pages of {page_size} positions must be a multiple of 32, "
                          f"heads of {head_dim} elements a multiple of 16")


# ------------------------------------------------------------------ ops
def fill_u32(t, value):
    _dev(t, "tensor")
    if t.element_size() * t.numel() % 4:
        raise KernelError("fill_u32 needs a multiple of 4 bytes")
    _check(library().gl3_fill_u32(_ptr(t), value, t.element_size() * t.numel() // 4, _stream()), "fill_u32")


def _check_next(next_weight, xg, rows, d, who):
    """The next norm's float weight [d] and the bfloat16 rows [rows, d] that receive weight * x."""
    if (next_weight is None) != (xg is None):
        raise KernelError(f"{who}: the next norm's weight and its rows come together")
    if xg is not None:
        _dev(next_weight, "next_weight", torch.float32); _dev(xg, "xg", torch.bfloat16, contiguous=False)
        if next_weight.shape != (d,) or xg.dim() != 2 or xg.shape != (rows, d) or xg.stride(1) != 1:
            raise KernelError(f"{who}: next weight {tuple(next_weight.shape)}, rows {tuple(xg.shape)} for [{rows}, {d}]")


def _bias(bias, n, who):
    """A bias per output column: float32 [n] on the device, or None."""
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.shape != (n,):
            raise KernelError(f"{who}: bias {tuple(bias.shape)} for {n} columns")
    return _ptr(bias)


def _col_scale(col_scale, n, epilogue, who):
    """A factor per output column (store and add epilogues): float32 [n] on the device, or None."""
    if col_scale is not None:
        _dev(col_scale, "col_scale", torch.float32)
        if col_scale.shape != (n,) or epilogue == EPI_GATED:
            raise KernelError(f"{who}: a factor per column {tuple(col_scale.shape)} for {n} columns, epilogue {epilogue}")
    return _ptr(col_scale)


def _slopes(slopes, n_heads, who):
    """A slope per query head for the bias that grows with the distance: float32 [H] on the device, or None."""
    if slopes is not None:
        _dev(slopes, "slopes", torch.float32)
        if slopes.shape != (n_heads,):
            raise KernelError(f"{who}: {tuple(slopes.shape)} slopes for {n_heads} heads")
    return _ptr(slopes)


def _sink(sink, n_heads, who):
    """A sink as the kernels take it: ``(has one number, that number, pointer to one number per head)``. ``sink`` is
    None, a number, or a float32 tensor [n_heads] on the device."""
    if sink is None:
        return 0, 0.0, None
    if isinstance(sink, torch.Tensor):
        _dev(sink, "sink", torch.float32)
        if sink.shape != (n_heads,):
            raise KernelError(f"{who}: {tuple(sink.shape)} sinks for {n_heads} heads")
        return 0, 0.0, _ptr(sink)
    return 1, float(sink), None


def _act(act, who):
    try:
        return ACTIVATIONS[act]
    except KeyError:
        raise KernelError(f"{who}: activation {act!r} is not built ({sorted(ACTIVATIONS)})") from None


def scale_(t, factor):
    """t *= factor (float32, contiguous)."""
    _dev(t, "tensor", torch.float32)
    _check(library().gl3_scale_f32(_ptr(t), float(factor), t.numel(), _stream()), "scale_f32")


def softcap_(t, cap):
    """t = cap * tanh(t / cap) (float32, contiguous)."""
    _dev(t, "tensor", torch.float32)
    _check(library().gl3_softcap_f32(_ptr(t), float(cap), t.numel(), _stream()), "softcap_f32")


def _table_steps(table):
    """0, or the k-steps of 32 a strip of a table that is held once (in the operands' order, rows in order)."""
    if not held_once(table):
        return 0
    t = getattr(table, "tiled", None)
    if t is None or getattr(t, "row_pos", None) is not None or t.data_ptr() != table.data_ptr():
        raise KernelError("embed: a table that is held once must be its copy in the operands' order, rows in order")
    return -(-table.shape[1] // 32)


def embed(table, ids, out, ssq=None, next_weight=None, xg=None, scale=1.0, pos_table=None, positions=None):
    """out[t] = scale * table[ids[t]] (+ pos_table[positions[t]]) as float32. The caller has checked
    ids < rows and positions < rows of ``pos_table``. ``ssq`` (at least 64 floats, at most 64 tokens)
    receives each row's sum of squares; with it ``xg`` [T, d] bfloat16 may receive ``next_weight *
    out``, the rows as the product after the next norm reads them."""
    _dev(table, "table"); _dev(ids, "ids", torch.int32); _dev(out, "out", torch.float32)
    T, d = out.shape
    if table.dim() != 2 or table.shape[1] != d or ids.numel() != T:
        raise KernelError(f"embed: table {tuple(table.shape)}, ids {tuple(ids.shape)}, out {tuple(out.shape)}")
    if ssq is not None:
        _dev(ssq, "ssq", torch.float32)
        if ssq.numel() < 64 or T > 64:
            raise KernelError("embed: sums of squares need 64 floats and at most 64 tokens")
    _check_next(next_weight, xg, T, d, "embed")
    if xg is not None and (ssq is None or not xg.is_contiguous()):
        raise KernelError("embed: the next norm's rows come with the sums of squares, contiguous")
    if pos_table is not None:
        _dev(pos_table, "pos_table", table.dtype); _dev(positions, "positions", torch.int32)
        if pos_table.dim() != 2 or pos_table.shape[1] != d or positions.numel() != T:
            raise KernelError(f"embed: table of positions {tuple(pos_table.shape)} for rows of {d}")
    _check(library().gl3_embed(_ptr(table), _code(table, "table"), _ptr(ids), _ptr(out), T, d, _ptr(ssq),
                               _ptr(next_weight), _ptr(xg), float(scale), _ptr(pos_table),
                               _ptr(positions) if pos_table is not None else c_void_p(0), _table_steps(table),
                               _stream()), "embed")


def rmsnorm(x, weight, out, eps, rows=None):
    """out[r] = weight * x[rows[r]] / rms (rows None: every row in order)."""
    _dev(x, "x", torch.float32); _dev(weight, "weight"); _dev(out, "out")
    d = x.shape[-1]
    n = out.shape[0]
    if x.dim() != 2 or out.dim() != 2 or out.shape[1] != d or weight.shape != (d,):
        raise KernelError(f"rmsnorm: x {tuple(x.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    if rows is not None:
        _dev(rows, "rows", torch.int32)
        if rows.numel() != n:
            raise KernelError(f"rmsnorm: {rows.numel()} rows for {n} outputs")
    elif x.shape[0] != n:
        raise KernelError(f"rmsnorm: {x.shape[0]} inputs for {n} outputs")
    _check(library().gl3_rmsnorm(_ptr(x), _ptr(rows), _ptr(weight), _code(weight, "weight"), _ptr(out),
                                 _code(out, "out"), n, d, float(eps), _stream()), "rmsnorm")


def gather_rows(x, rows, out):
    """out[r] = x[rows[r]] in ``out``'s dtype (x float32; the caller has checked rows < rows of x)."""
    _dev(x, "x", torch.float32); _dev(rows, "rows", torch.int32); _dev(out, "out")
    if x.dim() != 2 or out.dim() != 2 or out.shape != (rows.numel(), x.shape[1]):
        raise KernelError(f"gather_rows: x {tuple(x.shape)}, {rows.numel()} rows, out {tuple(out.shape)}")
    _check(library().gl3_gather_rows(_ptr(x), _ptr(rows), _ptr(out), _code(out, "out"), out.shape[0], x.shape[1],
                                     _stream()), "gather_rows")


def add_slices_rmsnorm(x, slices, weight=None, out=None, eps=0.0, rows=None):
    """x += slices[0] + slices[1] + ... (in that order; ``slices`` [S, rows of x, d] float32), and
    out[r] = weight * x[r] / rms when ``out`` is given. With ``rows`` the listed rows are normalised
    and x keeps its values."""
    _dev(x, "x", torch.float32); _dev(slices, "slices", torch.float32, contiguous=False)
    d = x.shape[-1]
    if (x.dim() != 2 or slices.dim() != 3 or slices.shape[1:] != x.shape or slices.stride(2) != 1
            or (weight is None) != (out is None)):
        raise KernelError(f"add_slices_rmsnorm: x {tuple(x.shape)}, slices {tuple(slices.shape)}")
    n = x.shape[0]
    if out is not None:
        _dev(weight, "weight"); _dev(out, "out")
        n = out.shape[0]
        if out.dim() != 2 or out.shape[1] != d or weight.shape != (d,):
            raise KernelError(f"add_slices_rmsnorm: weight {tuple(weight.shape)}, out {tuple(out.shape)} for d={d}")
    if rows is not None:
        _dev(rows, "rows", torch.int32)
        if out is None or rows.numel() != n:
            raise KernelError("add_slices_rmsnorm: rows select the rows that are normalised, one per output row")
    elif x.shape[0] != n:
        raise KernelError(f"add_slices_rmsnorm: {x.shape[0]} inputs for {n} outputs")
    _check(library().gl3_add_slices_rmsnorm(
        _ptr(x), _ptr(rows), _ptr(slices), slices.shape[0], slices.stride(0), slices.stride(1), _ptr(weight),
        _code(weight, "weight") if weight is not None else 0, _ptr(out), _code(out, "out") if out is not None else 0,
        n, d, float(eps), _stream()), "add_slices_rmsnorm")


def rope_cache_write(qkv, positions, seq_of_token, block_table, cos, sin, k_cache, v_cache, n_heads, n_kv,
                     head_dim, rot_dim, adjacent, page_size, write_kv=True):
    """Rotate q (in place) and k, and write k and v into one layer's paged cache.

    qkv [T, (H+2K)*hs] (or [T, H*hs] when ``write_kv`` is false); caches
    [pages, K, page_size, hs]; block_table [B, width] int32.
    """
    _dev(qkv, "qkv"); _dev(positions, "positions", torch.int32)
    T = qkv.shape[0]
    width = (n_heads + (2 * n_kv if write_kv else 0)) * head_dim
    if qkv.dim() != 2 or qkv.shape[1] != width or positions.numel() != T:
        raise KernelError(f"rope_cache_write: qkv {tuple(qkv.shape)} for {n_heads}+2*{n_kv} heads of {head_dim}")
    if cos is not None:
        _dev(cos, "cos", torch.float32); _dev(sin, "sin", torch.float32)
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != rot_dim // 2:
            raise KernelError(f"rope_cache_write: table {tuple(cos.shape)} for rot_dim {rot_dim}")
    stride = 0
    if write_kv:
        _dev(seq_of_token, "seq_of_token", torch.int32); _dev(block_table, "block_table", torch.int32)
        _dev(k_cache, "k_cache", qkv.dtype); _dev(v_cache, "v_cache", qkv.dtype)
        if seq_of_token.numel() != T or block_table.dim() != 2:
            raise KernelError("rope_cache_write: seq_of_token / block_table shapes")
        _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, "rope_cache_write")
        stride = block_table.shape[1]
    _check(library().gl3_rope_cache_write(
        _ptr(qkv), _code(qkv, "qkv"), _ptr(positions), _ptr(seq_of_token), _ptr(block_table), stride,
        _ptr(cos), _ptr(sin), _ptr(k_cache), _ptr(v_cache), T, n_heads, n_kv, head_dim, rot_dim, int(adjacent),
        page_size, int(write_kv), _stream()), "rope_cache_write")


def gemm_generic(a, w, out, epilogue=EPI_STORE, bias=None, act="silu", act_limit=0.0, act_shift=0.0, col_scale=None):
    """out = a @ w.T with float multiply-adds; see gemm_generic.hip for the epilogues.
    ``a`` and ``out`` may be row-strided views (last dimension contiguous). ``bias``: float32, one
    per row of ``w``; ``act``: the gated epilogue's activation, with ``act_limit`` (a bound on gate and up
    values, 0: none) and ``act_shift`` (added to the up value); ``col_scale``: float32, a factor per output
    column of the store and add epilogues, applied to the sums (and the bias) before they are stored or added."""
    _dev(a, "a", contiguous=False); _dev(w, "w"); _dev(out, "out", contiguous=False)
    if a.dim() != 2 or w.dim() != 2 or out.dim() != 2 or a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: operands must be 2-d with a contiguous last dimension")
    M, K = a.shape
    N = out.shape[1]
    rows = 2 * N if epilogue == EPI_GATED else N
    if w.shape != (rows, K) or out.shape[0] != M:
        raise KernelError(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}, epilogue {epilogue}")
    order, wp, pos = _w_order(w)
    if col_scale is not None:
        _dev(col_scale, "col_scale", torch.float32)
        if col_scale.shape != (N,) or epilogue == EPI_GATED:
            raise KernelError(f"gemm_generic: a factor per column {tuple(col_scale.shape)} for {N} columns, epilogue {epilogue}")
    _check(library().gl3_gemm_generic(_ptr(a), _code(a, "a"), wp, _code(w, "w"), _ptr(out), _code(out, "out"),
                                      M, N, K, a.stride(0), w.stride(0), out.stride(0), epilogue,
                                      _bias(bias, rows, "gemm_generic"), _act(act, "gemm_generic"), order, pos,
                                      float(act_limit), float(act_shift), _ptr(col_scale), _stream()),
           "gemm_generic")


def attention_generic(q, k_cache, v_cache, positions, seq_of_token, block_table, out, n_heads, n_kv, head_dim,
                      page_size, window, scale, v_head_dim=None, slopes=None, sink=None, keep_first=0, chunk=0, n_v_heads=None,
                      values_in_keys=None):
    """``sink`` may also be a float32 tensor [H]: a sink per query head. ``values_in_keys``: n: the cache has no value
    array (``v_cache`` None); the values are elements n .. n + v_head_dim of the key rows (heads of up to 1024).
    q: a [T, >= H*hs] view whose first H*hs columns of each row are the queries. ``v_head_dim``: the values'
    size where it is not the keys'; ``slopes``: float32 [H], score - slopes[h] * distance; ``sink``: the score of a
    key without a value that every query sees (None: no such key); ``keep_first``: with a window, the sequence's
    first keys that stay visible to every later query; ``chunk``: n > 0: query i sees key j <= i only if
    i // n == j // n (no window then); ``n_v_heads``: value heads where they are fewer than the key heads: several
    score maps over the same values, ``maps = n_kv / n_v_heads``; query and key heads then lie head by head as
    [map 0, map 1, ...], and map m of a head reads key head ``g * maps + m`` and value head g of the head's group."""
    _dev(q, "q", contiguous=False); _dev(out, "out", contiguous=False)
    _dev(k_cache, "k_cache", q.dtype)
    if values_in_keys is None:
        _dev(v_cache, "v_cache", q.dtype)
    elif v_cache is not None or n_v_heads is not None:
        raise KernelError("attention: values inside the keys come without a value array and with as many value heads")
    _dev(positions, "positions", torch.int32); _dev(seq_of_token, "seq_of_token", torch.int32)
    _dev(block_table, "block_table", torch.int32)
    T = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < n_heads * head_dim or out.dtype not in (q.dtype, torch.float32):
        raise KernelError(f"attention: q {tuple(q.shape)} {q.dtype} for {n_heads} heads of {head_dim}, out {out.dtype}")
    vd = head_dim if v_head_dim is None else int(v_head_dim)
    if out.shape != (T, n_heads * vd) or out.stride(1) != 1:
        raise KernelError(f"attention: out {tuple(out.shape)}")
    n_v = n_kv if n_v_heads is None else int(n_v_heads)
    if values_in_keys is None:
        _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, "attention", vd, n_v)
    elif (k_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (n_kv, page_size, head_dim) or values_in_keys < 0
          or values_in_keys + vd > head_dim):
        raise KernelError(f"attention: keys {tuple(k_cache.shape)} for {n_kv} heads of {head_dim} in pages of {page_size}, "
                          f"values of {vd} from element {values_in_keys}")
    if positions.numel() != T or seq_of_token.numel() != T or block_table.dim() != 2:
        raise KernelError("attention: positions / seq_of_token / block_table shapes")
    has_sink, sink_value, sinks = _sink(sink, n_heads, "attention")
    if chunk and window:
        raise KernelError("attention: a chunked mask has no window")
    if slopes is not None:
        _dev(slopes, "slopes", torch.float32)
        if slopes.shape != (n_heads,):
            raise KernelError(f"attention: {tuple(slopes.shape)} slopes for {n_heads} heads")
    _check(library().gl3_attention_generic(
        _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _code(q, "q"), _ptr(positions), _ptr(seq_of_token),
        _ptr(block_table), block_table.shape[1], _ptr(out), out.stride(0), T, n_heads, n_kv, head_dim, page_size,
        int(window or 0), float(scale), vd, _ptr(slopes), has_sink, sink_value,
        int(keep_first or 0) if window else 0, int(chunk or 0), n_v, _code(out, "out"), sinks,
        -1 if values_in_keys is None else int(values_in_keys), _stream()),
        "attention_generic")


def kv_write(rows, k_off, v_off, positions, table_rows, block_table, k_cache, v_cache, n_kv, head_dim, v_head_dim,
             page_size):
    """Keys (columns ``k_off`` .. of ``rows`` [T, ld]) and values (``v_off`` ..) of the step's tokens into one
    layer's paged cache, unrotated; the values may have another size than the keys."""
    _dev(rows, "rows", contiguous=False); _dev(positions, "positions", torch.int32)
    _dev(table_rows, "table_rows", torch.int32); _dev(block_table, "block_table", torch.int32)
    _dev(k_cache, "k_cache", rows.dtype); _dev(v_cache, "v_cache", rows.dtype)
    T = rows.shape[0]
    if rows.dim() != 2 or rows.stride(1) != 1 or positions.numel() != T or table_rows.numel() != T or block_table.dim() != 2:
        raise KernelError(f"kv_write: rows {tuple(rows.shape)}, {positions.numel()} positions")
    _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, "kv_write", v_head_dim)
    if k_off < 0 or v_off < 0 or k_off + n_kv * head_dim > rows.shape[1] or v_off + n_kv * v_head_dim > rows.shape[1]:
        raise KernelError(f"kv_write: columns {k_off} and {v_off} of rows of {rows.shape[1]}")
    _check(library().gl3_kv_write(_ptr(rows), _code(rows, "rows"), rows.stride(0), k_off, v_off, _ptr(positions),
                                  _ptr(table_rows), _ptr(block_table), block_table.shape[1], _ptr(k_cache), _ptr(v_cache),
                                  T, n_kv, head_dim, v_head_dim, page_size, _stream()), "kv_write")


def residual_inject(x, rows=None, vec=None):
    """x += rows (float32, x's shape) + vec (float32 [d]); either may be None."""
    _dev(x, "x", torch.float32)
    if x.dim() != 2:
        raise KernelError(f"residual_inject: x {tuple(x.shape)}")
    if rows is not None:
        _dev(rows, "rows", torch.float32)
        if rows.shape != x.shape:
            raise KernelError(f"residual_inject: rows {tuple(rows.shape)} for x {tuple(x.shape)}")
    if vec is not None:
        _dev(vec, "vec", torch.float32)
        if vec.shape != (x.shape[1],):
            raise KernelError(f"residual_inject: a vector {tuple(vec.shape)} for rows of {x.shape[1]}")
    _check(library().gl3_residual_inject(_ptr(x), _ptr(rows), _ptr(vec), x.shape[0], x.shape[1], _stream()),
           "residual_inject")


# ------------------------------------------------------------------ around and inside mixers with a state per sequence
def pair_rows(token_ids, positions, seq_of_token, cu_seqlens, slot_ids, state, mul_prev, mul_cur, buckets, rows):
    """rows[t] = (previous token * mul_prev + token * mul_cur) mod buckets, ``buckets`` for a sequence's first token;
    ``state`` [slots, >= 1] int32 holds every sequence's last token and is brought up to date."""
    for t, n in ((token_ids, "token_ids"), (positions, "positions"), (seq_of_token, "seq_of_token"),
                 (cu_seqlens, "cu_seqlens"), (slot_ids, "slot_ids"), (state, "state"), (rows, "rows")):
        _dev(t, n, torch.int32)
    T = token_ids.numel()
    if positions.numel() != T or seq_of_token.numel() != T or rows.numel() != T or state.dim() != 2 \
            or cu_seqlens.numel() != slot_ids.numel() + 1:
        raise KernelError(f"pair_rows: {T} tokens, {positions.numel()} positions, state {tuple(state.shape)}")
    _check(library().gl3_pair_rows(_ptr(token_ids), _ptr(positions), _ptr(seq_of_token), _ptr(cu_seqlens), _ptr(slot_ids),
                                   _ptr(state), state.stride(0), int(mul_prev), int(mul_cur), int(buckets), _ptr(rows), T,
                                   _stream()), "pair_rows")


def concat_rows(a, b, out):
    """out[t] = [a[t]; b[t]] in ``out``'s dtype (a, b float32 [T, d]; out [T, 2 d])."""
    _dev(a, "a", torch.float32); _dev(b, "b", torch.float32); _dev(out, "out")
    if a.dim() != 2 or a.shape != b.shape or out.shape != (a.shape[0], 2 * a.shape[1]):
        raise KernelError(f"concat_rows: a {tuple(a.shape)}, b {tuple(b.shape)}, out {tuple(out.shape)}")
    _check(library().gl3_concat_rows(_ptr(a), _ptr(b), _ptr(out), _code(out, "out"), a.shape[0], a.shape[1], _stream()),
           "concat_rows")


def rotate_heads(rows, positions, runs, adjacent=False, back=False, gate=None, gate_col=0, cache=None, norms=None,
                 norm_eps=0.0):
    """Runs of heads inside ``rows`` [T, ld] turned in place by the tokens' positions. ``runs``: up to three of
    ``(first column, heads, head_dim, rot_dim, cos, sin)`` with tables [positions, rot_dim / 2] float32 (None, None: not
    rotated). ``back``: by minus the angle. ``gate`` (one run): rows [T, *] of the same dtype whose column
    ``gate_col + h`` holds head h's gate; every element of the head is multiplied by its sigmoid. ``cache``:
    ``(k_cache, v_cache, table_rows, block_table, page_size)``; the runs are then queries, keys and values, and keys and
    values also go to the tokens' places in one layer's paged cache (the values may have fewer heads than the keys).
    ``norms``: per run None or ``(weight float32 [head_dim], n)``: the run's heads are first divided by their root
    mean square over their first n elements (``norm_eps`` inside the root; what lies behind them must be zeros) and
    multiplied by the weight."""
    _dev(rows, "rows", contiguous=False); _dev(positions, "positions", torch.int32)
    T = rows.shape[0]
    if rows.dim() != 2 or rows.stride(1) != 1 or positions.numel() != T or not 1 <= len(runs) <= 3:
        raise KernelError(f"rotate_heads: rows {tuple(rows.shape)}, {positions.numel()} positions, {len(runs)} runs")
    n = len(runs)
    for col, heads, hd, rd, cos, sin in runs:
        if cos is not None:
            _dev(cos, "cos", torch.float32); _dev(sin, "sin", torch.float32)
            if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != rd // 2:
                raise KernelError(f"rotate_heads: table {tuple(cos.shape)} for {rd} rotated elements")
        if col < 0 or col + heads * hd > rows.shape[1] or rd > hd or rd % 2:
            raise KernelError(f"rotate_heads: {heads} heads of {hd} ({rd} rotated) from column {col} of rows of {rows.shape[1]}")
    ints = [(c_int * n)(*[int(r[i]) for r in runs]) for i in range(4)]
    tabs = [(c_void_p * n)(*[r[i].data_ptr() if r[i] is not None else None for r in runs]) for i in (4, 5)]
    gate_ld = 0
    if gate is not None:
        _dev(gate, "gate", rows.dtype, contiguous=False)
        if gate.dim() != 2 or gate.shape[0] != T or gate.stride(1) != 1 or n != 1 or gate_col < 0 or gate_col + runs[0][1] > gate.shape[1]:
            raise KernelError(f"rotate_heads: gate {tuple(gate.shape)} from column {gate_col}")
        gate_ld = gate.stride(0)
    kc = vc = trows = table = None
    stride = page = 0
    if cache is not None:
        kc, vc, trows, table, page = cache
        _dev(trows, "table_rows", torch.int32); _dev(table, "block_table", torch.int32)
        _dev(kc, "k_cache", rows.dtype); _dev(vc, "v_cache", rows.dtype)
        if n != 3 or trows.numel() != T or table.dim() != 2:
            raise KernelError("rotate_heads: a cache write takes queries, keys and values and a table row per token")
        _check_cache(kc, vc, runs[1][1], page, runs[1][2], "rotate_heads", runs[2][2], runs[2][1])
        stride = table.shape[1]
    norm_ws = norm_dims = None
    if norms is not None and any(x is not None for x in norms):
        if len(norms) != n:
            raise KernelError(f"rotate_heads: {len(norms)} norms for {n} runs")
        for (w, nd), r in zip([x if x is not None else (None, 0) for x in norms], runs):
            if w is not None:
                _dev(w, "norm weight", torch.float32)
                if w.shape != (r[2],) or not 0 < nd <= r[2]:
                    raise KernelError(f"rotate_heads: a norm weight {tuple(w.shape)} over {nd} of a head's {r[2]} elements")
        norm_ws = (c_void_p * n)(*[x[0].data_ptr() if x is not None else None for x in norms])
        norm_dims = (c_int * n)(*[int(x[1]) if x is not None else 0 for x in norms])
    _check(library().gl3_rotate_heads(_ptr(rows), _code(rows, "rows"), rows.stride(0), _ptr(positions), T, *ints, *tabs, n,
                                      int(bool(adjacent)), int(bool(back)), _ptr(gate), gate_ld, int(gate_col), _ptr(kc),
                                      _ptr(vc), _ptr(trows), _ptr(table), stride, int(page), norm_ws, norm_dims,
                                      float(norm_eps), _stream()), "rotate_heads")


def diff_combine(att, out, H, D, dim, lam, eps, mult):
    """``att`` [T, 2 H D]: head by head the output under the first score map and under the second; ``out`` [T, H D] =
    (a1 - lam * a2) / rms over the head's first ``dim`` elements (what lies behind them holds zeros) * mult. ``att`` has
    ``out``'s type or is float32."""
    _dev(att, "att", contiguous=False); _dev(out, "out", contiguous=False)
    if att.dtype not in (out.dtype, torch.float32):
        raise KernelError(f"diff_combine: {att.dtype} -> {out.dtype}")
    T = att.shape[0]
    if att.dim() != 2 or att.stride(1) != 1 or att.shape[1] < 2 * H * D or out.shape != (T, H * D) or out.stride(1) != 1:
        raise KernelError(f"diff_combine: {tuple(att.shape)} -> {tuple(out.shape)} for {H} heads of {D}")
    _check(library().gl3_diff_combine(_ptr(att), _code(att, "att"), att.stride(0), _ptr(out), out.stride(0), _code(out, "out"), T, int(H), int(D),
                                      int(dim), float(lam), float(eps), float(mult), _stream()), "diff_combine")


def layernorm(x, weight, bias, out, eps, rows=None):
    """out[r] = layer norm of x[rows[r]] (of x[r] without ``rows``) with float32 weight and bias."""
    _dev(x, "x", torch.float32); _dev(weight, "weight", torch.float32); _dev(bias, "bias", torch.float32); _dev(out, "out")
    d = x.shape[1]
    n = x.shape[0] if rows is None else rows.numel()
    if rows is not None:
        _dev(rows, "rows", torch.int32)
    if x.dim() != 2 or weight.shape != (d,) or bias.shape != (d,) or out.shape != (n, d):
        raise KernelError(f"layernorm: x {tuple(x.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    _check(library().gl3_layernorm(_ptr(x), _ptr(rows), _ptr(weight), _ptr(bias), _ptr(out), _code(out, "out"), n, d,
                                   float(eps), _stream()), "layernorm")


def layernorm_add(x, y, weight, bias, eps, cast=None):
    """x += layer norm of y, row by row (both float32); ``cast`` (same shape, the activations' type) receives the new
    rows of x."""
    _dev(x, "x", torch.float32); _dev(y, "y", torch.float32)
    _dev(weight, "weight", torch.float32); _dev(bias, "bias", torch.float32)
    T, d = x.shape
    if x.dim() != 2 or y.shape != (T, d) or weight.shape != (d,) or bias.shape != (d,):
        raise KernelError(f"layernorm_add: x {tuple(x.shape)}, y {tuple(y.shape)}, weight {tuple(weight.shape)}")
    if cast is not None:
        _dev(cast, "cast")
        if cast.shape != (T, d):
            raise KernelError(f"layernorm_add: cast {tuple(cast.shape)}")
    _check(library().gl3_layernorm_add(_ptr(x), _ptr(y), _ptr(weight), _ptr(bias), T, d, float(eps), _ptr(cast),
                                       _code(cast, "cast") if cast is not None else F32, _stream()), "layernorm_add")


def cast_rows(x, out):
    """``out`` = the float32 ``x`` in out's type."""
    _dev(x, "x", torch.float32); _dev(out, "out")
    if out.shape != x.shape:
        raise KernelError(f"cast_rows: {tuple(x.shape)} -> {tuple(out.shape)}")
    _check(library().gl3_cast_rows(_ptr(x), _ptr(out), _code(out, "out"), x.numel(), _stream()), "cast_rows")


def _f32_rows(t, name, cols):
    _dev(t, name, torch.float32, contiguous=False)
    if t.dim() != 2 or t.stride(1) != 1 or t.shape[1] < cols:
        raise KernelError(f"{name}: rows {tuple(t.shape)} hold fewer than {cols} columns")
    return t


def _state_area(state, state_off, need, who):
    _dev(state, "state", torch.float32, contiguous=False)
    if state.dim() != 2 or state.stride(1) != 1 or state_off < 0 or state_off + need > state.shape[1]:
        raise KernelError(f"{who}: a state of {tuple(state.shape)} for {need} floats from {state_off}")


def ssm_prep(proj, col_x, channels, col_dt, heads, conv_w, conv_b, A_log, dt_bias, state, state_off, cu_seqlens,
             seq_of_token, slot_ids, act, ab):
    """The state space's short convolution with silu over ``channels`` columns of ``proj`` [T, ld] float32 from
    ``col_x`` on (``conv_w`` [channels, taps], the last tap the current token's; the sequences' last taps - 1 inputs
    live in ``state`` [slots, *] from ``state_off`` on and move on) -> ``act`` [T, channels]; and per head the decay
    and the step size from column ``col_dt`` on -> ``ab`` [T, 2 heads] = (exp(-exp(A_log) dt), dt), dt = softplus(. + dt_bias)."""
    T = proj.shape[0]
    _f32_rows(proj, "proj", max(col_x + channels, col_dt + heads))
    taps = conv_w.shape[1]
    for t, name, shape in ((conv_w, "conv_w", (channels, taps)), (A_log, "A_log", (heads,)), (dt_bias, "dt_bias", (heads,)),
                           (act, "act", (T, channels)), (ab, "ab", (T, 2 * heads))):
        _dev(t, name, torch.float32)
        if tuple(t.shape) != shape:
            raise KernelError(f"ssm_prep: {name} {tuple(t.shape)}, expected {shape}")
    if conv_b is not None:
        _dev(conv_b, "conv_b", torch.float32)
        if conv_b.shape != (channels,):
            raise KernelError(f"ssm_prep: conv_b {tuple(conv_b.shape)}")
    _state_area(state, state_off, (taps - 1) * channels, "ssm_prep")
    _dev(cu_seqlens, "cu_seqlens", torch.int32); _dev(seq_of_token, "seq_of_token", torch.int32); _dev(slot_ids, "slot_ids", torch.int32)
    B = cu_seqlens.numel() - 1
    if seq_of_token.numel() != T or slot_ids.numel() < B:
        raise KernelError("ssm_prep: seq_of_token / slot_ids shapes")
    _check(library().gl3_ssm_prep(_ptr(proj), proj.stride(0), T, B, int(col_x), int(channels), int(col_dt), int(heads),
                                  _ptr(conv_w), _ptr(conv_b), taps, _ptr(A_log), _ptr(dt_bias), _ptr(state), state.stride(0),
                                  int(state_off), _ptr(cu_seqlens), _ptr(seq_of_token), _ptr(slot_ids), _ptr(act), _ptr(ab),
                                  _stream()), "ssm_prep")


SCAN_PIECE_BLOCKS = 1024      # a long step's recurrence is cut until about this many (sequence, piece, head) run side by side
SCAN_PIECE_LEAST = 32         # tokens: shorter pieces cost more in their start states than they gain


def scan_piece_len(max_len, n_seqs, H):
    """The length of the pieces into which ``decay_scan`` cuts a step whose longest sequence has ``max_len`` tokens, or
    0 for a step in one piece. It follows from the step's shape alone."""
    want = max(1, SCAN_PIECE_BLOCKS // max(1, n_seqs * H))
    piece = max(SCAN_PIECE_LEAST, -(-max_len // want))
    piece = -(-piece // 16) * 16
    return piece if max_len > piece else 0


def scan_pieces_floats(max_len, n_seqs, H, N, P):
    """Floats of scratch that ``decay_scan`` needs for such a step (0: none)."""
    piece = scan_piece_len(max_len, n_seqs, H)
    return n_seqs * -(-max_len // piece) * H * (N * P + 1) if piece else 0


def decay_scan(q, col_q, k, col_k, v, col_v, state, state_off, cu_seqlens, slot_ids, out, H, heads_per_group, N, P,
               a_tok=None, b_tok=None, a_head=None, b_const=1.0, pieces=None, max_len=0, silu_inputs=False):
    """Per (sequence, head) ``S <- a S + b k v^T`` and ``o = S^T q`` token by token, S [N, P] float32 in ``state``
    [slots, *] from ``state_off + h N P`` on. q and k: float32 rows whose group g (``heads_per_group`` heads share one)
    starts at column ``col + g N``; v: head h at ``col_v + h P``. a and b: per token and head (``a_tok``, ``b_tok``,
    columns h of rows of the same stride) or per head (``a_head`` [H]) / one number (``b_const``). ``out`` [T, H P].
    With ``pieces`` (float32 scratch of ``scan_pieces_floats`` elements) and ``max_len`` (the longest sequence of the
    step) a long step runs as pieces side by side, joined through their start states. ``silu_inputs``: q, k and v pass
    silu as they are read."""
    groups = H // heads_per_group
    _f32_rows(q, "q", col_q + groups * N); _f32_rows(k, "k", col_k + groups * N); _f32_rows(v, "v", col_v + H * P)
    _dev(out, "out", torch.float32)
    T = q.shape[0]
    if k.shape[0] != T or v.shape[0] != T or out.shape != (T, H * P):
        raise KernelError(f"decay_scan: rows {q.shape[0]}, {k.shape[0]}, {v.shape[0]}; out {tuple(out.shape)}")
    ld_ab = 0
    for t, name in ((a_tok, "a_tok"), (b_tok, "b_tok")):
        if t is not None:
            _f32_rows(t, name, H)
            if t.shape[0] != T or (ld_ab and t.stride(0) != ld_ab):
                raise KernelError(f"decay_scan: {name} {tuple(t.shape)}")
            ld_ab = t.stride(0)
    if a_tok is None:
        _dev(a_head, "a_head", torch.float32)
        if a_head.shape != (H,):
            raise KernelError(f"decay_scan: a_head {tuple(a_head.shape)}")
    _state_area(state, state_off, H * N * P, "decay_scan")
    _dev(cu_seqlens, "cu_seqlens", torch.int32); _dev(slot_ids, "slot_ids", torch.int32)
    B = cu_seqlens.numel() - 1
    piece_len = 0
    if pieces is not None:
        _dev(pieces, "pieces", torch.float32)
        if not pieces.is_contiguous() or max_len < 1 or max_len > T:
            raise KernelError(f"decay_scan: pieces {tuple(pieces.shape)}, the longest of {T} tokens' sequences has {max_len}")
        piece_len = scan_piece_len(max_len, B, H)
    _check(library().gl3_decay_scan(_ptr(q), q.stride(0), int(col_q), _ptr(k), k.stride(0), int(col_k), _ptr(v), v.stride(0),
                                    int(col_v), _ptr(a_tok), _ptr(b_tok), ld_ab, _ptr(a_head), float(b_const), _ptr(state),
                                    state.stride(0), int(state_off), _ptr(cu_seqlens), _ptr(slot_ids), _ptr(out),
                                    out.stride(0), B, int(H), int(heads_per_group), int(N), int(P),
                                    _ptr(pieces) if piece_len else None, pieces.numel() if piece_len else 0, int(max_len),
                                    int(piece_len), int(bool(silu_inputs)), _stream()), "decay_scan")


def group_norm_gate(o, gate, col_g, out, gsize, eps, weight=None, gate_first=False, skip=None, gate_act="silu"):
    """``o`` [T, C] float32 (+ ``skip = (rows, col, d [heads], head_dim)``: d[h] times the rows' columns), times silu of
    the gate columns (``gate`` rows float32 from ``col_g``) before (``gate_first``) or after being divided by its root
    mean square over every ``gsize`` channels; times ``weight`` [C]. ``out`` [T, C] in the activations' type.
    ``gate_act``: "silu" or "sigmoid" of the gate columns."""
    if gate_act not in ("silu", "sigmoid"):
        raise KernelError(f"group_norm_gate: a gate's {gate_act!r} is not built (silu, sigmoid)")
    _dev(o, "o", torch.float32); _dev(out, "out")
    T, C = o.shape
    _f32_rows(gate, "gate", col_g + C)
    if out.shape != (T, C) or gate.shape[0] != T or C % gsize:
        raise KernelError(f"group_norm_gate: o {tuple(o.shape)}, out {tuple(out.shape)}, groups of {gsize}")
    if weight is not None:
        _dev(weight, "weight", torch.float32)
        if weight.shape != (C,):
            raise KernelError(f"group_norm_gate: weight {tuple(weight.shape)}")
    sx = sd = None
    ld_x = col_x = hd = 0
    if skip is not None:
        sx, col_x, sd, hd = skip
        _f32_rows(sx, "skip rows", col_x + C); _dev(sd, "skip factors", torch.float32)
        if sx.shape[0] != T or C % hd or sd.shape != (C // hd,):
            raise KernelError(f"group_norm_gate: skip rows {tuple(sx.shape)}, factors {tuple(sd.shape)}")
        ld_x = sx.stride(0)
    _check(library().gl3_group_norm_gate(_ptr(o), _ptr(sx), ld_x, int(col_x), _ptr(sd), int(hd), _ptr(gate), gate.stride(0),
                                         int(col_g), _ptr(weight), float(eps), int(bool(gate_first)), T, C, int(gsize),
                                         _ptr(out), _code(out, "out"), int(gate_act == "sigmoid"), _stream()), "group_norm_gate")


EXPERT_ACTIVATIONS = {None: 0, "gelu": 1, "gelu_tanh": 2, "silu": 3}
ROUTE_MAX_TOP, ROUTE_MAX_EXPERTS = 16, 1024      # as csrc/routed.hip has them


def route(logits, top, idx, wts, offsets, pairs, always=False, scores=False, correction=None, sum_eps=0.0):
    """Router logits [T, E] float32 -> the ``top`` largest per token (``idx`` [T, top] int32, the lower number wins a
    tie) with the softmax over them alone (``wts`` [T, top]); and the (token, choice) pairs ordered by expert:
    ``offsets`` [E + 1] int32, ``pairs`` [T top] int32 (pair t * top + j). ``always``: every token has one more pair
    behind its choices, with expert number E and weight 1 (``idx`` and ``wts`` [T, top + 1], ``offsets`` [E + 2],
    ``pairs`` [T (top + 1)]). ``scores``: the other rule: s = softmax over all E logits, the choice goes by
    s + ``correction`` (float32 [E], optional), the weights are the chosen s divided by their sum plus ``sum_eps``."""
    _dev(logits, "logits", torch.float32)
    T, E = logits.shape
    if correction is not None:
        _dev(correction, "correction", torch.float32)
        if not scores or correction.shape != (E,):
            raise KernelError(f"route: a correction {tuple(correction.shape)} for {E} scores")
    more = 1 if always else 0
    for t, name, shape, dt in ((idx, "idx", (T, top + more), torch.int32), (wts, "wts", (T, top + more), torch.float32),
                               (offsets, "offsets", (E + more + 1,), torch.int32),
                               (pairs, "pairs", (T * (top + more),), torch.int32)):
        _dev(t, name, dt)
        if tuple(t.shape) != shape:
            raise KernelError(f"route: {name} {tuple(t.shape)}, expected {shape}")
    _check(library().gl3_route(_ptr(logits), T, E, int(top), _ptr(idx), _ptr(wts), _ptr(offsets), _ptr(pairs),
                               E if always else -1, int(bool(scores)), _ptr(correction), float(sum_eps), _stream()), "route")


def expert_gemm(a, w, out, act=None, offsets=None, pairs=None, a_div=1, mfma=True, gated=None):
    """``out[p] = act(w[e] @ a[p // a_div])`` for every pair p of expert e's run (``offsets``, ``pairs`` of ``route``);
    without them ``w`` is one expert [1, N, K] that takes every row of ``a`` in its own order. ``w`` [E, N, K];
    ``out`` [pairs, N] in bfloat16 or float32. ``gated = (activation, limit, shift)``: the rows of every ``w[e]`` are
    gate and up rows in turns (2n: gate n, 2n + 1: up n) and ``out`` [pairs, N / 2] = act(min(gate, limit)) *
    (clamp(up, -limit, limit) + shift) (``limit`` None or 0: unbounded); ``act`` is then None. ``offsets`` may run on
    behind the E experts of ``w`` (experts without a product of their own): their pairs are left alone."""
    _dev(a, "a", contiguous=False); _dev(w, "w", a.dtype); _dev(out, "out", contiguous=False)
    n_out = w.shape[1] // 2 if gated is not None and w.dim() == 3 else (w.shape[1] if w.dim() == 3 else -1)
    if w.dim() != 3 or a.dim() != 2 or a.stride(1) != 1 or out.stride(1) != 1 or a.shape[1] != w.shape[2] or out.shape[1] != n_out:
        raise KernelError(f"expert_gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    E, N, K = w.shape
    n_rows = out.shape[0]
    gate_act, limit, shift = -1, 0.0, 0.0
    if gated is not None:
        if act is not None or gated[0] not in ACTIVATIONS or N % 2:
            raise KernelError(f"expert_gemm: a gated product of {N} rows with {gated[0]!r} ({sorted(ACTIVATIONS)}), act {act!r}")
        gate_act, limit, shift = ACTIVATIONS[gated[0]], float(gated[1] or 0.0), float(gated[2])
    if offsets is not None:
        _dev(offsets, "offsets", torch.int32); _dev(pairs, "pairs", torch.int32)
        if offsets.numel() < E + 1 or pairs.numel() != n_rows or a.shape[0] * a_div < n_rows:
            raise KernelError(f"expert_gemm: {offsets.numel()} offsets, {pairs.numel()} pairs, {a.shape[0]} rows x {a_div}")
    elif E != 1 or a.shape[0] != n_rows or a_div != 1:
        raise KernelError("expert_gemm: without runs one expert takes every row")
    if act not in EXPERT_ACTIVATIONS:
        raise KernelError(f"expert_gemm: activation {act!r} is not built ({sorted(k for k in EXPERT_ACTIVATIONS if k)})")
    _check(library().gl3_expert_gemm(_ptr(a), _code(a, "a"), a.stride(0), int(a_div), _ptr(w), _code(w, "w"), E, N, K,
                                     _ptr(offsets), _ptr(pairs), n_rows, _ptr(out), _code(out, "out"), out.stride(0),
                                     EXPERT_ACTIVATIONS[act], int(bool(mfma)), gate_act, limit, shift, _stream()), "expert_gemm")


def route_combine(y, wts, out, accumulate=False, identity=None):
    """``out[t]`` (+)= sum over j of ``wts[t, j] * y[t * top + j]``; y [T top, d] float32, out [T, d] float32.
    ``identity = (idx [T, top] int32, n_real, h [T, d])``: a pair whose expert number is ``n_real`` or more stands for
    the token's input row ``h[t]`` itself."""
    _dev(y, "y", torch.float32); _dev(wts, "wts", torch.float32); _dev(out, "out", torch.float32)
    T, top = wts.shape
    if y.dim() != 2 or y.shape[0] != T * top or out.shape != (T, y.shape[1]):
        raise KernelError(f"route_combine: y {tuple(y.shape)}, wts {tuple(wts.shape)}, out {tuple(out.shape)}")
    idx = h = None
    n_real = 0
    if identity is not None:
        idx, n_real, h = identity
        _dev(idx, "idx", torch.int32); _dev(h, "h")
        if idx.shape != wts.shape or h.shape != out.shape:
            raise KernelError(f"route_combine: choices {tuple(idx.shape)}, input rows {tuple(h.shape)}")
    _check(library().gl3_route_combine(_ptr(y), _ptr(wts), T, top, y.shape[1], _ptr(out), int(bool(accumulate)), _ptr(idx),
                                       int(n_real), _ptr(h), _code(h, "h") if h is not None else 0, _stream()),
           "route_combine")


def streams_step(rows, S, y=None, mix=None, out_w=None, in_w=None, norm_w=None, eps=0.0, h=None):
    """``rows`` [T, S d] float32: S copies of every token's residual row. With ``y`` [T, d] (a sublayer's output) the
    copies become ``x_r <- sum_s mix[s, r] x_s + out_w[r] y``; with ``in_w`` [S] the next sublayer's input
    ``h = RMSnorm(sum_s in_w[s] x_s) * norm_w`` is made from the (new) copies. All numbers float32 on the device."""
    _dev(rows, "rows", torch.float32)
    T, d = rows.shape[0], rows.shape[1] // S
    if rows.dim() != 2 or rows.shape[1] != S * d:
        raise KernelError(f"streams_step: rows {tuple(rows.shape)} for {S} copies")
    if y is not None:
        _dev(y, "y", torch.float32); _dev(mix, "mix", torch.float32); _dev(out_w, "out_w", torch.float32)
        if y.shape != (T, d) or mix.shape != (S, S) or out_w.shape != (S,):
            raise KernelError(f"streams_step: y {tuple(y.shape)}, mix {tuple(mix.shape)}, out {tuple(out_w.shape)}")
    if in_w is not None:
        _dev(in_w, "in_w", torch.float32); _dev(norm_w, "norm_w", torch.float32); _dev(h, "h")
        if in_w.shape != (S,) or norm_w.shape != (d,) or h.shape != (T, d):
            raise KernelError(f"streams_step: in {tuple(in_w.shape)}, norm {tuple(norm_w.shape)}, h {tuple(h.shape)}")
    _check(library().gl3_streams_step(_ptr(rows), T, int(S), d, _ptr(y), _ptr(mix), _ptr(out_w), _ptr(in_w), _ptr(norm_w),
                                      float(eps), _ptr(h), _code(h, "h") if h is not None else 0, _stream()), "streams_step")


def streams_fill(src, rows, S):
    """Every one of the S copies in ``rows`` [T, S d] takes ``src`` [T, d] (float32)."""
    _dev(src, "src", torch.float32); _dev(rows, "rows", torch.float32)
    T, d = src.shape
    if rows.shape != (T, S * d):
        raise KernelError(f"streams_fill: {tuple(src.shape)} into {tuple(rows.shape)} as {S} copies")
    _check(library().gl3_streams_fill(_ptr(src), _ptr(rows), T, int(S), d, _stream()), "streams_fill")


def streams_sum(rows, S, out, which=None):
    """``out[r]`` = the sum of the S copies of token ``which[r]`` (None: token r); float32."""
    _dev(rows, "rows", torch.float32); _dev(out, "out", torch.float32)
    n, d = out.shape
    if rows.dim() != 2 or rows.shape[1] != S * d:
        raise KernelError(f"streams_sum: rows {tuple(rows.shape)} as {S} copies of {d}")
    if which is not None:
        _dev(which, "which", torch.int32)
        if which.numel() != n:
            raise KernelError(f"streams_sum: {which.numel()} rows for {n} outputs")
    elif rows.shape[0] != n:
        raise KernelError(f"streams_sum: {rows.shape[0]} tokens for {n} outputs")
    _check(library().gl3_streams_sum(_ptr(rows), _ptr(which), n, int(S), d, _ptr(out), _stream()), "streams_sum")


def latent_prep(proj, col_q, q_rank, col_kv, rank, rot, wq, wkv, eps, positions, table_rows, block_table, cos, sin, cq,
                k_cache, page_size, H, offsets, pairs):
    """``proj`` [T, ld] float32 holds the sums of a query latent (``q_rank`` from ``col_q``) and of a key/value latent
    (``rank`` from ``col_kv``, then ``rot`` elements of a key part that all heads share). ``cq`` [T, q_rank] = the
    first divided by its root mean square times ``wq``; the token's row of ``k_cache`` [page, 1, page_size, dk] takes
    [the second the same way with ``wkv`` | the shared part turned in adjacent pairs by the position | zeros].
    ``offsets`` [H + 1] and ``pairs`` [T H] receive the runs with which ``expert_gemm`` works head by head on rows
    [T H, *] (row t H + h is head h of token t)."""
    _f32_rows(proj, "proj", max(col_q + q_rank, col_kv + rank + rot))
    T = proj.shape[0]
    _dev(wq, "wq", torch.float32); _dev(wkv, "wkv", torch.float32); _dev(cq, "cq"); _dev(k_cache, "k_cache", cq.dtype)
    _dev(positions, "positions", torch.int32); _dev(table_rows, "table_rows", torch.int32)
    _dev(block_table, "block_table", torch.int32); _dev(offsets, "offsets", torch.int32); _dev(pairs, "pairs", torch.int32)
    if rot:
        _dev(cos, "cos", torch.float32); _dev(sin, "sin", torch.float32)
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != rot // 2:
            raise KernelError(f"latent_prep: table {tuple(cos.shape)} for {rot} rotated elements")
    if (wq.shape != (q_rank,) or wkv.shape != (rank,) or cq.shape != (T, q_rank) or k_cache.dim() != 4 or k_cache.shape[1] != 1
            or k_cache.shape[2] != page_size or positions.numel() != T or table_rows.numel() != T or block_table.dim() != 2
            or offsets.numel() != H + 1 or pairs.numel() != T * H):
        raise KernelError(f"latent_prep: weights {tuple(wq.shape)}, {tuple(wkv.shape)}; cq {tuple(cq.shape)}; cache "
                          f"{tuple(k_cache.shape)}; {offsets.numel()} offsets, {pairs.numel()} pairs for {T} tokens of {H} heads")
    _check(library().gl3_latent_prep(_ptr(proj), proj.stride(0), T, int(col_q), int(q_rank), int(col_kv), int(rank), int(rot),
                                     _ptr(wq), _ptr(wkv), float(eps), _ptr(positions), _ptr(table_rows), _ptr(block_table),
                                     block_table.shape[1], _ptr(cos), _ptr(sin), _ptr(cq), _ptr(k_cache), _code(cq, "cq"),
                                     int(page_size), k_cache.shape[3], int(H), _ptr(offsets), _ptr(pairs), _stream()),
           "latent_prep")


def latent_query(q, H, dim, rot, positions, cos, sin, qa, rank):
    """``q`` [T, H (dim + rot)]: every head's last ``rot`` elements, turned in adjacent pairs by the token's position,
    go to columns ``rank .. rank + rot`` of the head's row in ``qa`` [T, H dk], zeros behind them."""
    _dev(q, "q"); _dev(qa, "qa", q.dtype); _dev(positions, "positions", torch.int32)
    T = q.shape[0]
    dk = qa.shape[1] // H
    if q.shape != (T, H * (dim + rot)) or qa.shape != (T, H * dk) or dk < rank + rot or positions.numel() != T:
        raise KernelError(f"latent_query: q {tuple(q.shape)}, qa {tuple(qa.shape)} for {H} heads of {dim} + {rot}, latents of {rank}")
    if rot:
        _dev(cos, "cos", torch.float32); _dev(sin, "sin", torch.float32)
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != rot // 2:
            raise KernelError(f"latent_query: table {tuple(cos.shape)} for {rot} rotated elements")
    _check(library().gl3_latent_query(_ptr(q), _code(q, "q"), T, int(H), int(dim), int(rot), _ptr(positions), _ptr(cos),
                                      _ptr(sin), _ptr(qa), int(rank), dk, _stream()), "latent_query")


def latent_attention_fits(dk, rank, page_size):
    """Whether the matrix-core attention over cached latents is built for rows of ``dk`` with values of ``rank``."""
    return bool(library().gl3_latent_attention_supports(int(dk), int(rank), int(page_size)))


def latent_splits(n_seqs, max_q_len, H, kv_len):
    """Blocks that share a sequence's cached rows in ``latent_attention``: a step of few (token, head) tiles over
    many keys is cut until the chip has blocks, each with at least four chunks of 32 keys."""
    rows = max_q_len * H
    blocks = n_seqs * -(-rows // (64 if rows <= 64 else 128))      # (as the kernel's launch cuts the pairs into tiles)
    return int(max(1, min(256 // max(blocks, 1), kv_len // 128, 32)))


def latent_attention(q, k_cache, cu_seqlens, kv_before, block_table, out, max_q_len, H, rank, scale, seq_rows=None,
                     n_splits=1, part_o=None, part_ml=None):
    """Causal attention of ``q`` [T, H dk] (bfloat16) over a cache of one array, ``k_cache`` [page, 1, page_size, dk],
    whose rows are keys and, in their first ``rank`` elements, values, for all H heads alike; ``out`` [T, H rank].
    ``cu_seqlens`` [B + 1] and ``kv_before`` [B] say which tokens of the packed ``q`` belong to which sequence and
    where they sit in it; ``seq_rows`` [B] (optional) names each sequence's row of ``block_table``. With ``n_splits``
    > 1 (``latent_splits``) the keys are shared out over blocks whose parts go through ``part_o`` (T H n_splits rank
    floats) and ``part_ml`` (T H n_splits 2 floats)."""
    _dev(q, "q", torch.bfloat16, contiguous=False); _dev(out, "out", torch.bfloat16, contiguous=False)
    _dev(k_cache, "k_cache", torch.bfloat16)
    _dev(cu_seqlens, "cu_seqlens", torch.int32); _dev(kv_before, "kv_before", torch.int32)
    _dev(block_table, "block_table", torch.int32)
    T, B = q.shape[0], kv_before.numel()
    if k_cache.dim() != 4 or k_cache.shape[1] != 1:
        raise KernelError(f"latent_attention: a cache of {tuple(k_cache.shape)}")
    page, dk = k_cache.shape[2], k_cache.shape[3]
    if (q.dim() != 2 or q.stride(1) != 1 or q.shape[1] != H * dk or out.shape != (T, H * rank) or out.stride(1) != 1
            or cu_seqlens.numel() != B + 1 or block_table.dim() != 2 or max_q_len < 1):
        raise KernelError(f"latent_attention: q {tuple(q.shape)}, out {tuple(out.shape)} for {H} heads of {dk} / {rank}")
    if seq_rows is not None:
        _dev(seq_rows, "seq_rows", torch.int32)
        if seq_rows.numel() != B:
            raise KernelError("latent_attention: one table row per sequence")
    elif block_table.shape[0] < B:
        raise KernelError("latent_attention: the block table has fewer rows than there are sequences")
    floats = 0
    if n_splits > 1:
        _dev(part_o, "part_o", torch.float32); _dev(part_ml, "part_ml", torch.float32)
        if part_o.numel() < T * H * n_splits * rank or part_ml.numel() < T * H * n_splits * 2:
            raise KernelError("latent_attention: the workspace of the splits is too small")
        floats = T * H * n_splits * (rank + 2)
    _check(library().gl3_latent_attention(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(cu_seqlens), _ptr(kv_before),
                                          _ptr(block_table), _ptr(seq_rows), block_table.shape[1], _ptr(out), out.stride(0), T, B,
                                          int(max_q_len), int(H), dk, int(rank), page, float(scale), int(n_splits),
                                          _ptr(part_o), _ptr(part_ml), floats, _stream()),
           "latent_attention")


def sigmoid_gate(a, gate, col_g):
    """``a`` [T, C] *= sigmoid(gate[:, col_g : col_g + C]); the gate's rows are float32."""
    _dev(a, "a")
    T, C = a.shape
    _f32_rows(gate, "gate", col_g + C)
    if gate.shape[0] != T:
        raise KernelError(f"sigmoid_gate: {gate.shape[0]} gate rows for {T}")
    _check(library().gl3_sigmoid_gate(_ptr(a), _code(a, "a"), _ptr(gate), gate.stride(0), int(col_g), T, C, _stream()),
           "sigmoid_gate")


def sides_norm_add(x, a, b, wa, wb, eps, factor, ssq=None, next_weight=None, xg=None):
    """x += factor * (a / rms(a) * wa + b / rms(b) * wb); all float32, a and b [T, d] like x (b may be None).
    ``ssq`` (at least 64 floats, at most 64 tokens) receives each completed row's sum of squares; with it ``xg`` [T, d]
    bfloat16 may receive ``next_weight * row``, the rows as the product after the next norm reads them."""
    _dev(x, "x", torch.float32); _dev(a, "a", torch.float32); _dev(wa, "wa", torch.float32)
    if x.dim() != 2 or a.shape != x.shape or wa.shape != (x.shape[1],):
        raise KernelError(f"sides_norm_add: x {tuple(x.shape)}, a {tuple(a.shape)}, weight {tuple(wa.shape)}")
    if b is not None:
        _dev(b, "b", torch.float32); _dev(wb, "wb", torch.float32)
        if b.shape != x.shape or wb.shape != wa.shape:
            raise KernelError(f"sides_norm_add: b {tuple(b.shape)}, weight {tuple(wb.shape)}")
    if ssq is not None:
        _dev(ssq, "ssq", torch.float32)
        if ssq.numel() < 64 or x.shape[0] > 64:
            raise KernelError("sides_norm_add: sums of squares need 64 floats and at most 64 tokens")
    _check_next(next_weight, xg, x.shape[0], x.shape[1], "sides_norm_add")
    if xg is not None and (ssq is None or not xg.is_contiguous()):
        raise KernelError("sides_norm_add: the next norm's rows come with the sums of squares, contiguous")
    _check(library().gl3_sides_norm_add(_ptr(x), _ptr(a), _ptr(b), _ptr(wa), _ptr(wb) if b is not None else c_void_p(0),
                                        float(eps), float(factor), x.shape[0], x.shape[1], _ptr(ssq), _ptr(next_weight),
                                        _ptr(xg), _stream()), "sides_norm_add")


def tanh_rows(src, out):
    """out = tanh(src) in ``out``'s dtype: src float32 [T, n] (rows may be strided), out [T, n] contiguous."""
    _dev(src, "src", torch.float32, contiguous=False); _dev(out, "out")
    if src.dim() != 2 or src.stride(1) != 1 or out.shape != src.shape:
        raise KernelError(f"tanh_rows: src {tuple(src.shape)}, out {tuple(out.shape)}")
    _check(library().gl3_tanh_rows(_ptr(src), src.stride(0), src.shape[1], _ptr(out), _code(out, "out"), src.numel(),
                                   _stream()), "tanh_rows")


MINGRU_RUN = 32      # tokens of a run of the three-pass scan (MG_RUN in mixers.hip)


def mingru_scan(proj, width, state, cu_seqlens, slot_ids, out, max_q_len=1, runs=None):
    """The minGRU recurrence over the step's tokens from the state in each sequence's slot: ``proj`` [T, >= 3 width]
    float32 holds the update gate's, the candidate's and the output gate's sums; ``out`` [T, width] receives
    S_t * silu(gate); ``state`` [slots, >= width] float32 is advanced. With ``runs`` (float32, at least
    2 * sequences * ceil(max_q_len / 32) * width elements) and a longest sequence of ``max_q_len`` > 32 tokens the scan
    runs in three passes over runs of 32 tokens."""
    _dev(proj, "proj", torch.float32, contiguous=False); _dev(state, "state", torch.float32, contiguous=False); _dev(out, "out")
    _dev(cu_seqlens, "cu_seqlens", torch.int32); _dev(slot_ids, "slot_ids", torch.int32)
    T, B = proj.shape[0], slot_ids.numel()
    if (state.dim() != 2 or state.stride(1) != 1 or proj.dim() != 2 or proj.stride(1) != 1 or proj.shape[1] < 3 * width or out.shape != (T, width) or state.dim() != 2
            or state.shape[1] < width or cu_seqlens.numel() != B + 1):
        raise KernelError(f"mingru_scan: proj {tuple(proj.shape)}, out {tuple(out.shape)}, state {tuple(state.shape)}")
    if runs is not None:
        _dev(runs, "runs", torch.float32)
        if runs.numel() < 2 * B * -(-int(max_q_len) // MINGRU_RUN) * width:
            raise KernelError(f"mingru_scan: scratch of {runs.numel()} floats for {B} sequences of up to {max_q_len} tokens")
    _check(library().gl3_mingru_scan(_ptr(proj), proj.stride(0), int(width), _ptr(state), state.stride(0), _ptr(cu_seqlens),
                                     _ptr(slot_ids), _ptr(out), _code(out, "out"), B, int(max_q_len), _ptr(runs), _stream()),
           "mingru_scan")


def shift_mix(h, mu, state, cu_seqlens, seq_of_token, slot_ids, out, one_token_each=False):
    """out[s, t] = h[t] + (row of the token before t - h[t]) * mu[s]; a step's first token of a sequence reads the row
    that ``state`` [slots, >= d] float32 holds for it, and the step's last row is left there. ``mu`` [n, d] float32;
    ``out`` [n, T, d] of h's dtype."""
    _dev(h, "h"); _dev(mu, "mu", torch.float32); _dev(state, "state", torch.float32, contiguous=False); _dev(out, "out", h.dtype)
    _dev(cu_seqlens, "cu_seqlens", torch.int32); _dev(seq_of_token, "seq_of_token", torch.int32)
    _dev(slot_ids, "slot_ids", torch.int32)
    T, d = h.shape
    B = slot_ids.numel()
    if (mu.dim() != 2 or mu.shape[1] != d or out.shape != (mu.shape[0], T, d) or state.dim() != 2 or state.shape[1] < d
            or state.stride(1) != 1
            or cu_seqlens.numel() != B + 1 or seq_of_token.numel() != T):
        raise KernelError(f"shift_mix: h {tuple(h.shape)}, mu {tuple(mu.shape)}, out {tuple(out.shape)}, state {tuple(state.shape)}")
    _check(library().gl3_shift_mix(_ptr(h), _code(h, "h"), d, _ptr(mu), mu.shape[0], _ptr(state), state.stride(0),
                                   _ptr(cu_seqlens), _ptr(seq_of_token), _ptr(slot_ids), _ptr(out), T, B,
                                   int(bool(one_token_each)), _stream()), "shift_mix")


def timemix(r, k, v, w_log, bonus, state, state_off, cu_seqlens, slot_ids, out, H, D, gate=None, norm_w=None, eps=0.0,
            normed=None, max_q_len=0):
    """The decayed matrix per head, token by token from the state in each sequence's slot (``mixers.hip``): r, k, v
    [T, H D] float32 (rows of one common stride), w_log [T, H D] float32 (the decay is exp(-exp(w_log))), bonus [H, D];
    ``state`` [slots, >= state_off + H D D] float32. ``out`` [T, H D] float32 (may be None) receives the raw read-outs;
    ``normed`` [T, H D] (may be None; then ``gate`` [T, H D] float32, ``norm_w`` [H D] float32 and ``eps``) receives
    read-out / rms per head * norm_w * silu(gate). ``max_q_len`` (0: unknown): the most tokens a sequence brings; the
    kernel's rounds, and with them a block's shared memory, are no longer than that."""
    for t, n in ((r, "r"), (k, "k"), (v, "v"), (w_log, "w_log")):
        _dev(t, n, torch.float32, contiguous=False)
    _dev(bonus, "bonus", torch.float32)
    _dev(state, "state", torch.float32, contiguous=False)
    _dev(cu_seqlens, "cu_seqlens", torch.int32); _dev(slot_ids, "slot_ids", torch.int32)
    T, B = r.shape[0], slot_ids.numel()
    if (any(t.shape != (T, H * D) or t.stride(1) != 1 for t in (r, k, v, w_log)) or not r.stride(0) == k.stride(0) == v.stride(0)
            or bonus.numel() != H * D or state.dim() != 2
            or state.shape[1] < state_off + H * D * D or state.stride(1) != 1 or cu_seqlens.numel() != B + 1):
        raise KernelError(f"timemix: r {tuple(r.shape)} for {H} heads of {D}, state {tuple(state.shape)}")
    if out is None and normed is None:
        raise KernelError("timemix: nothing to write to")
    if out is not None:
        _dev(out, "out", torch.float32)
        if out.shape != (T, H * D):
            raise KernelError(f"timemix: out {tuple(out.shape)}")
    ld_g = 0
    if normed is not None:
        _dev(normed, "normed"); _dev(gate, "gate", torch.float32, contiguous=False); _dev(norm_w, "norm_w", torch.float32)
        if normed.shape != (T, H * D) or gate.shape != (T, H * D) or gate.stride(1) != 1 or norm_w.numel() != H * D:
            raise KernelError(f"timemix: normed {tuple(normed.shape)}, gate {tuple(gate.shape)}, weight {tuple(norm_w.shape)}")
        ld_g = gate.stride(0)
    _check(library().gl3_timemix(_ptr(r), _ptr(k), _ptr(v), r.stride(0), _ptr(w_log), w_log.stride(0), _ptr(bonus),
                                 _ptr(state), state.stride(0), int(state_off), _ptr(cu_seqlens), _ptr(slot_ids), _ptr(out),
                                 B, H, D, _ptr(gate), ld_g, _ptr(norm_w), float(eps), _ptr(normed),
                                 _code(normed, "normed") if normed is not None else F32, int(max_q_len), _stream()), "timemix")


def head_norm_gate(o, weight, gate, eps, out, H, D):
    """out[t, h] = o[t, h] / rms(o[t, h]) * weight[h] * silu(gate[t, h]) per head of D elements; o, gate [T, H D] float32,
    weight [H D] float32, out [T, H D]."""
    _dev(o, "o", torch.float32); _dev(weight, "weight", torch.float32); _dev(gate, "gate", torch.float32); _dev(out, "out")
    T = o.shape[0]
    if o.shape != (T, H * D) or gate.shape != o.shape or out.shape != o.shape or weight.numel() != H * D:
        raise KernelError(f"head_norm_gate: o {tuple(o.shape)}, gate {tuple(gate.shape)}, out {tuple(out.shape)}")
    _check(library().gl3_head_norm_gate(_ptr(o), _ptr(weight), _ptr(gate), float(eps), _ptr(out), _code(out, "out"), T, H, D,
                                        _stream()), "head_norm_gate")


# ------------------------------------------------------------------ the gated delta rule
def delta_state_floats(H, G, D, Dv, taps):
    """Floats of one sequence's state: the heads' matrices in tiles of 16 value columns, then the convolution's
    held inputs (``delta_rule.hip``). No GPU is needed to ask."""
    return H * (-(-Dv // 16)) * D * 16 + (2 * G * D + H * Dv) * (taps - 1)


def _delta_common(state, cu_seqlens, slot_ids, H, G, D, Dv, taps, who):
    _dev(state, "state", torch.float32); _dev(cu_seqlens, "cu_seqlens", torch.int32); _dev(slot_ids, "slot_ids", torch.int32)
    B = slot_ids.numel()
    if state.dim() != 2 or state.shape[1] < delta_state_floats(H, G, D, Dv, taps) or cu_seqlens.numel() != B + 1:
        raise KernelError(f"{who}: state {tuple(state.shape)}, {cu_seqlens.numel()} bounds for {B} sequences")
    return B


def delta_prep(proj, offsets, conv_w, A_log, dt_bias, state, cu_seqlens, seq_of_token, slot_ids, act, gates,
               H, G, D, Dv, taps, unit_eps, q_scale, one_token_each=False):
    """The step's q, k, v after the short convolution, silu and (q, k) the scaling to unit length into ``act``
    [T, 2 G D + H Dv], the heads' decays and write strengths into ``gates`` [T, 2 H]; then each sequence's held
    inputs move on. ``proj`` [T, ld] float32; ``offsets``: the first columns of q, k, v, b and a in it.
    ``one_token_each``: the caller vouches that every sequence brings exactly one token (one launch less)."""
    _dev(proj, "proj", torch.float32, contiguous=False)
    for t, n in ((conv_w, "conv_w"), (A_log, "A_log"), (dt_bias, "dt_bias"), (act, "act"), (gates, "gates")):
        _dev(t, n, torch.float32)
    _dev(seq_of_token, "seq_of_token", torch.int32)
    T = proj.shape[0]
    C = 2 * G * D + H * Dv
    B = _delta_common(state, cu_seqlens, slot_ids, H, G, D, Dv, taps, "delta_prep")
    if (proj.dim() != 2 or proj.stride(1) != 1 or conv_w.shape != (C, taps) or A_log.shape != (H,) or dt_bias.shape != (H,)
            or act.shape != (T, C) or gates.shape != (T, 2 * H) or seq_of_token.numel() != T or len(offsets) != 5):
        raise KernelError(f"delta_prep: proj {tuple(proj.shape)}, conv {tuple(conv_w.shape)}, act {tuple(act.shape)}")
    ends = (G * D, G * D, H * Dv, H, H)
    if any(o < 0 or o + e > proj.shape[1] for o, e in zip(offsets, ends)):
        raise KernelError(f"delta_prep: columns {tuple(offsets)} of rows of {proj.shape[1]}")
    _check(library().gl3_delta_prep(_ptr(proj), _ptr(conv_w), _ptr(A_log), _ptr(dt_bias), _ptr(state), _ptr(cu_seqlens),
                                    _ptr(seq_of_token), _ptr(slot_ids), _ptr(act), _ptr(gates), T, B, H, G, D, Dv, taps,
                                    proj.stride(0), *[int(o) for o in offsets], state.stride(0), float(unit_eps),
                                    float(q_scale), int(bool(one_token_each) and T == B), _stream()), "delta_prep")


def delta_recurrence(act, gates, state, cu_seqlens, slot_ids, readout, proj, off_gate, norm_w, out, H, G, D, Dv, taps, eps):
    """The rule itself, token by token for every sequence of the step from the state it holds, then the read-outs'
    norm: ``out[t, h] = o[t, h] / rms * norm_w * silu(gate[t, h])`` (``out`` [T, H Dv] float32 or bfloat16), the gate in
    columns ``off_gate`` .. of ``proj``; ``readout`` [T, H Dv] float32 is scratch for the raw read-outs."""
    _dev(act, "act", torch.float32); _dev(gates, "gates", torch.float32); _dev(readout, "readout", torch.float32)
    _dev(proj, "proj", torch.float32, contiguous=False); _dev(norm_w, "norm_w", torch.float32); _dev(out, "out")
    T = act.shape[0]
    B = _delta_common(state, cu_seqlens, slot_ids, H, G, D, Dv, taps, "delta_recurrence")
    if (act.shape != (T, 2 * G * D + H * Dv) or gates.shape != (T, 2 * H) or readout.shape != (T, H * Dv)
            or out.shape != (T, H * Dv) or norm_w.shape != (Dv,) or proj.dim() != 2 or proj.stride(1) != 1
            or proj.shape[0] != T or off_gate < 0 or off_gate + H * Dv > proj.shape[1]):
        raise KernelError(f"delta_recurrence: act {tuple(act.shape)}, gates {tuple(gates.shape)}, out {tuple(out.shape)}, "
                          f"proj {tuple(proj.shape)}")
    _check(library().gl3_delta_recurrence(_ptr(act), _ptr(gates), _ptr(state), _ptr(cu_seqlens), _ptr(slot_ids),
                                          _ptr(readout), _ptr(proj), proj.stride(0), off_gate, _ptr(norm_w), _ptr(out),
                                          _code(out, "out"), float(eps), T, B, H, G, D, Dv, taps, state.stride(0), _stream()),
           "delta_recurrence")


def decode_advance(token_ids, positions, kv_before, sampled, history, step):
    """Feed the sampled tokens back, move every sequence on by one, log the tokens in row step[0]
    of ``history`` [rows, n], count the step."""
    n = token_ids.numel()
    for t, name in ((token_ids, "token_ids"), (positions, "positions"), (kv_before, "kv_before"),
                    (sampled, "sampled"), (history, "history"), (step, "step")):
        _dev(t, name, torch.int32)
    if positions.numel() != n or kv_before.numel() != n or sampled.numel() < n or history.dim() != 2 or history.shape[1] < n:
        raise KernelError("decode_advance: sizes")
    _check(library().gl3_decode_advance(_ptr(token_ids), _ptr(positions), _ptr(kv_before), _ptr(sampled),
                                        _ptr(history), history.stride(0), _ptr(step), n, _stream()), "decode_advance")


def argmax(logits, work, out):
    """Every row's first greatest logit; ``work``: at least 128 floats per row."""
    _dev(logits, "logits", torch.float32, contiguous=False); _dev(work, "work", torch.float32)
    _dev(out, "out", torch.int32)
    R, V = logits.shape
    if logits.stride(1) != 1 or work.numel() < 128 * R or out.numel() < R:
        raise KernelError("argmax: argument sizes")
    _check(library().gl3_argmax(_ptr(logits), logits.stride(0), _ptr(work), _ptr(out), R, V, _stream()), "argmax")


def argmax_advance(logits, work, out, token_ids, positions, kv_before, history, step):
    """``argmax`` into ``out`` and ``decode_advance`` with its result, in two launches instead of three."""
    _dev(logits, "logits", torch.float32, contiguous=False); _dev(work, "work", torch.float32)
    R, V = logits.shape
    for t, name in ((out, "out"), (token_ids, "token_ids"), (positions, "positions"), (kv_before, "kv_before"),
                    (history, "history"), (step, "step")):
        _dev(t, name, torch.int32)
    if (logits.stride(1) != 1 or work.numel() < 128 * R or out.numel() < R or token_ids.numel() != R
            or positions.numel() != R or kv_before.numel() != R or history.dim() != 2 or history.shape[1] < R or R > 1024):
        raise KernelError("argmax_advance: argument sizes")
    _check(library().gl3_argmax_advance(_ptr(logits), logits.stride(0), _ptr(work), _ptr(out), R, V, _ptr(token_ids),
                                        _ptr(positions), _ptr(kv_before), _ptr(history), history.stride(0), _ptr(step),
                                        _stream()), "argmax_advance")


def sample_work_size(rows, vocab):
    """Floats of scratch that `sample` and `argmax` need for `rows` rows."""
    return max(int(library().gl3_sample_work_floats(int(rows), int(vocab))), 128 * rows)


def sample(logits, work, temperature, top_p, uniform, out, step=None, uniform_stride=0):
    _dev(logits, "logits", torch.float32, contiguous=False); _dev(work, "work", torch.float32)
    for t, n in ((temperature, "temperature"), (top_p, "top_p"), (uniform, "uniform")):
        _dev(t, n, torch.float32)
    _dev(out, "out", torch.int32)
    R, V = logits.shape
    if logits.stride(1) != 1 or work.numel() < sample_work_size(R, V) or min(temperature.numel(), top_p.numel(), uniform.numel(),
                                                              out.numel()) < R:
        raise KernelError("sample: argument sizes")
    if step is not None:
        _dev(step, "step", torch.int32)
    _check(library().gl3_sample(_ptr(logits), logits.stride(0), _ptr(work), _ptr(temperature), _ptr(top_p),
                                _ptr(uniform), _ptr(out), R, V, _ptr(step), int(uniform_stride), _stream()), "sample")


# ------------------------------------------------------------------ bfloat16 product for few rows
def gemm_skinny_fits(a, w, out, epilogue):
    M, K = a.shape
    return (M <= 64 and K % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and (out.dtype == torch.float32 or (out.dtype == torch.bfloat16 and epilogue != EPI_ADD)))


def skinny_strip_rows(M, N, K, epilogue):
    """Rows of w that a block of the skinny kernel takes: 8 where strips of 16 would leave more than a
    third of the CUs without a block. With at most 8 rows of ``a`` the half-empty tile of such a strip
    takes the next 32 k instead (N=2048, 8 rows: K=8192 12.4 -> 9.7 us, K=2048 6.1 -> 4.3 us); with 9
    to 16 rows half the tile idles, which pays only where K is too long for the kernel that keeps its
    rows of ``a`` in registers (17.0 -> 15.8 us at N=2048, K=8192). Else 16."""
    if epilogue == EPI_GATED or -(-N // 16) > 160:
        return 16
    return 8 if M <= 8 or (M <= 16 and K > 4096) else 16


def skinny_keeps_operands(M, K):
    """Whether the skinny product (store epilogue, no folded norm) of ``M`` rows over ``K`` columns runs on
    the kernel whose waves keep their operands of ``a`` in registers: with 17 to 64 rows that is K up to
    2,048, with fewer rows up to 4,096. Beyond it the kernel that streams the rows of ``a`` for every strip
    runs, which a product of very many strips should leave to the tiled kernel."""
    return K <= (2048 if M > 16 else 4096)


def packed_rows(n_columns, dtype, device):
    """A buffer for at most 8 rows of ``n_columns`` elements in the order in which the products of strips of
    8 weight rows read them: [step of 64 columns][lane 16 q + r][8 elements], lane (r, q) holding row r % 8 at
    column 32 (r // 8) + 8 q. A product with ``pack_out`` writes it, one with ``a_packed`` reads it."""
    return torch.empty((-(-n_columns // 64), 64, 8), dtype=dtype, device=device)


def gemm_skinny(a, w, out, epilogue=EPI_STORE, waves=0, ssq_out=None, strip_rows=16, next_weight=None, xg=None,
                bias=None, act="silu", a_packed=False, act_limit=0.0, act_shift=0.0, col_scale=None):
    """out (=, +=, gated) a @ w.T on the matrix cores for at most 64 rows of ``a``. ``ssq_out``
    [N/strip_rows, 64] float32 (add epilogue): partial sums of squares of the completed rows; with it
    ``xg`` [M, N] bfloat16 may receive ``next_weight * out``, the rows as the product after the next
    norm reads them. ``a_packed`` (strips of 8 rows, at most 8 rows): ``a`` is a ``packed_rows`` buffer."""
    _dev(a, "a", torch.bfloat16, contiguous=False); _dev(w, "w", torch.bfloat16); _dev(out, "out", contiguous=False)
    if a_packed:
        if (w.dim() != 2 or out.dim() != 2 or out.stride(1) != 1 or not a.is_contiguous()
                or a.numel() < -(-w.shape[1] // 64) * 512 or out.shape[0] > 8 or strip_rows != 8 or waves):
            raise KernelError("gemm_skinny: rows in the packed order go with strips of 8 weight rows and at most 8 rows")
        a = a.view(-1)[:8 * w.shape[1]].view(8, w.shape[1])[:out.shape[0]]     # (the shape only: the kernel knows the order)
    if a.dim() != 2 or w.dim() != 2 or out.dim() != 2 or a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: operands must be 2-d with a contiguous last dimension")
    M, K = a.shape
    N = out.shape[1]
    rows = 2 * N if epilogue == EPI_GATED else N
    if w.shape != (rows, K) or out.shape[0] != M:
        raise KernelError(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}, epilogue {epilogue}")
    if ssq_out is not None:
        _dev(ssq_out, "ssq_out", torch.float32)
        if epilogue != EPI_ADD or N % 16 or ssq_out.numel() < N // strip_rows * 64:
            raise KernelError("gemm_skinny: sums of squares need the add epilogue, N % 16 == 0 and 64 floats a strip")
    _check_next(next_weight, xg, M, N, "gemm_skinny")
    if xg is not None and ssq_out is None:
        raise KernelError("gemm_skinny: the next norm's rows come with the sums of squares")
    if held_once(w) and not (skinny_takes(w, M, strip_rows) and (strip_rows == 8 or _tiled(w, rows, K, n_out=N).value)
                             and a.stride(0) < 2 ** 24 and K < 2 ** 24):
        raise KernelError("gemm_skinny: a weight kept in the matrix cores' order alone is read through the copy whose strips "
                          f"the call names (strips of {strip_rows} rows, {M} rows of a)")
    _check(library().gl3_gemm_skinny(_ptr(a), _ptr(w), _ptr(out), _code(out, "out"), M, N, K, a.stride(0), w.stride(0),
                                     out.stride(0), epilogue, waves, _ptr(ssq_out), strip_rows, _ptr(next_weight),
                                     _ptr(xg), xg.stride(0) if xg is not None else 0, _bias(bias, rows, "gemm_skinny"),
                                     _act(act, "gemm_skinny"), _tiled(w, rows, K, n_out=N), _tiled8(w, rows, K), int(bool(a_packed)),
                                     float(act_limit), float(act_shift), _col_scale(col_scale, N, epilogue, "gemm_skinny"),
                                     _stream()), "gemm_skinny")


def strip_rows_of(n_rows, qkv=None):
    """Which row of W is row r of strip t of 16, as the kernels' ``sk_strip_row`` names them: rows
    16 t + r (the last strip repeats the last row), and for the stacked q, k, v rows with half-split
    pairing (``qkv`` = (n_heads, n_kv, head_dim, rotated, adjacent)) 8 rows of a rotated head and the
    8 half a head further, so that both elements of a pair lie in one tile."""
    n_strips = -(-n_rows // 16)
    rows = torch.arange(n_strips * 16).clamp(max=n_rows - 1).view(n_strips, 16)
    if qkv is not None:
        n_heads, n_kv, hs, rotated, adjacent = qkv
        if rotated and not adjacent:
            per_head = hs // 16
            t = torch.arange(n_strips).view(-1, 1)
            r = torch.arange(16).view(1, -1)
            hd, sub = t // per_head, t % per_head
            paired = hd * hs + 8 * sub + torch.where(r < 8, r, hs // 2 + r - 8)
            rows = torch.where(hd < n_heads + n_kv, paired, rows)
    return rows.reshape(-1)


def tile_weight(w, qkv=None):
    """A copy of ``w`` [N, K] (bfloat16, N % 16 == 0) in the order in which the matrix cores take it as an
    operand: [strip of 16 rows][k-step of 32][lane = 16 * (k block of 8) + row][8 elements], k padded with
    zeros to whole steps. The products of few rows whose kernels keep their rows of A in registers read
    it where a weight carries one (``w.tiled``): a load is then 1 KB of consecutive memory."""
    N, K = w.shape
    if N % 16 or w.dtype != torch.bfloat16:
        raise KernelError(f"tile_weight: {tuple(w.shape)} {w.dtype}")
    steps = -(-K // 32)
    rows = strip_rows_of(N, qkv).to(w.device)
    wp = torch.zeros(N, steps * 32, dtype=w.dtype, device=w.device)
    wp[:, :K] = w[rows]
    t = wp.view(N // 16, 16, steps, 4, 8).permute(0, 2, 3, 1, 4).contiguous()
    t.tiled_for = qkv
    if not torch.equal(rows, torch.arange(N, device=rows.device)):
        # the place of each stored row in the copy, for the kernels that read the copy row by row
        t.row_pos = torch.empty(N, dtype=torch.int32, device=w.device)
        t.row_pos[rows] = torch.arange(N, dtype=torch.int32, device=w.device)
    return t


def tile_weight8(w):
    """A copy of ``w`` [N, K] (bfloat16, N % 8 == 0) in the order of the packed tiles that the products of
    at most 8 rows use for strips of 8 weight rows: [strip of 8 rows][step of 64 k][lane][8 elements], lane
    16 q + r holding row r % 8 at k = 32 (r // 8) + 8 q, k padded with zeros to whole steps."""
    N, K = w.shape
    if N % 8 or w.dtype != torch.bfloat16:
        raise KernelError(f"tile_weight8: {tuple(w.shape)} {w.dtype}")
    steps = -(-K // 64)
    wp = torch.zeros(N, steps * 64, dtype=w.dtype, device=w.device)
    wp[:, :K] = w
    # [strip, row, step, half, q, element] -> [strip, step, q, half, row, element]
    return wp.view(N // 8, 8, steps, 2, 4, 8).permute(0, 2, 4, 3, 1, 5).contiguous()


def untile_weight(t, n_rows, K):
    """The rows of a matrix out of its copy in the matrix operands' order (``tile_weight``): a new tensor
    [n_rows, K] in the stored order."""
    steps = -(-K // 32)
    rows = t.view(n_rows // 16, steps, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(n_rows, steps * 32)[:, :K]
    pos = getattr(t, "row_pos", None)
    return (rows[pos.long()] if pos is not None else rows).contiguous()


def untile_weight8(t, n_rows, K):
    """The same out of the copy in packed strips of 8 rows (``tile_weight8``)."""
    steps = -(-K // 64)
    # [strip, step, q, half, row, element] -> [strip, row, step, half, q, element]
    return t.view(n_rows // 8, steps, 4, 2, 8, 8).permute(0, 4, 1, 3, 2, 5).reshape(n_rows, steps * 64)[:, :K].contiguous()


def stored_order(w):
    """``w`` as the rows lie in the model's file: ``w`` itself, or (held once) rebuilt from a copy, a new tensor."""
    if not held_once(w):
        return w
    t = getattr(w, "tiled", None)
    return untile_weight(t, *w.shape) if t is not None else untile_weight8(w.tiled8, *w.shape)


def can_hold_once(w):
    """Whether one of the copies that ``w`` carries has exactly the matrix's elements, over whole steps of 64 k
    (the tiled product's step), so that it can stand for the matrix."""
    N, K = w.shape
    t, t8 = getattr(w, "tiled", None), getattr(w, "tiled8", None)
    return K % 64 == 0 and ((t is not None and N % 16 == 0 and t.numel() == N * K)
                            or (t8 is not None and N % 8 == 0 and t8.numel() == N * K))


def hold_once(w):
    """``w`` (which carries ``w.tiled`` and/or ``w.tiled8``, over whole steps of k) as a matrix that is kept in
    the matrix cores' order alone: a tensor of the same shape and dtype whose memory IS a copy. Whoever drops
    ``w`` then frees the stored order. The kernels that read any order (the embedding, the generic and the tiled
    product, the kernel of whole lines, and those of few rows that take the copies anyway) are told by
    ``held_once``; the others refuse it."""
    if not can_hold_once(w):
        raise KernelError(f"hold_once: {tuple(w.shape)} has no copy in the matrix cores' order that could stand for it")
    N, K = w.shape
    t, t8 = getattr(w, "tiled", None), getattr(w, "tiled8", None)
    base = t if (t is not None and N % 16 == 0 and t.numel() == N * K) else t8
    alias = base.view(N, K)
    alias.operand_order_only = True
    if t is not None:
        alias.tiled = t
    if t8 is not None:
        alias.tiled8 = t8
    return alias


def skinny_takes(w, M, strip_rows, qkv=None):
    """Whether the products of few rows can read ``w`` in strips of ``strip_rows``: always when the stored order
    is there; a weight that is held once through the copy whose strips those are (rows in order, or for ``qkv``)."""
    if not held_once(w):
        return True
    N, K = w.shape
    if strip_rows == 8:
        return M <= 8 and bool(_tiled8(w, N, K).value)
    return bool(_tiled(w, N, K, qkv=qkv).value)


def _tiled8(w, n_rows, K):
    t = getattr(w, "tiled8", None)
    if t is None or n_rows % 8 or t.numel() != n_rows * -(-K // 64) * 64:
        return c_void_p(0)
    return _ptr(t)


def _tiled(w, n_rows, K, qkv=None, n_out=None):
    """The pointer to ``w.tiled`` if the weight carries a copy in the operands' order that fits this call
    (``n_out``: the output columns, where the gate rows and the up rows must each fill whole strips)."""
    t = getattr(w, "tiled", None)
    if (t is None or n_rows % 16 or (n_out is not None and n_out % 16) or t.numel() != n_rows * -(-K // 32) * 32
            or getattr(t, "tiled_for", None) != qkv):
        return c_void_p(0)
    return _ptr(t)


def gemm_skinny_wide_fits(a, w, out, epilogue):
    return (8 < a.shape[0] <= 64 and gemm_skinny_fits(a, w, out, epilogue)
            and not (held_once(w) and getattr(getattr(w, "tiled", None), "row_pos", None) is not None))


def wide_slices(N, K):
    """Into how many slices of K the wide kernel's product [*, K] x [N, K] is cut: enough blocks for
    the chip (a block takes 32 columns where they are few), at least one pair of k-steps (64 k) for
    each of a block's 8 waves."""
    return max(1, min(8, 256 // -(-N // 32), K // 512))


def gemm_skinny_wide(a, w, out, epilogue=EPI_STORE, strips=0, bias=None, act="silu", act_limit=0.0, act_shift=0.0,
                     col_scale=None):
    """out (=, +=, gated) a @ w.T for 17 to 64 rows of ``a``. ``out`` with three axes [slices, M, N]
    (float32, store epilogue) takes the sums of one slice of K each: the caller adds them up; that form
    also takes 9 to 16 rows."""
    _dev(a, "a", torch.bfloat16, contiguous=False); _dev(w, "w", torch.bfloat16); _dev(out, "out", contiguous=False)
    M, K = a.shape
    slices, slice_stride = 1, 0
    rows = out
    if out.dim() == 3:
        slices, slice_stride, rows = out.shape[0], out.stride(0), out[0]
    N = rows.shape[1]
    wrows = 2 * N if epilogue == EPI_GATED else N
    if (w.shape != (wrows, K) or rows.shape[0] != M or rows.stride(1) != 1 or a.stride(1) != 1
            or not (16 < M <= 64 or (8 < M <= 16 and epilogue == EPI_STORE and out.dtype == torch.float32))):
        raise KernelError(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}, epilogue {epilogue}")
    order, wp, pos = _w_order(w)
    if pos.value:
        raise KernelError("gemm_skinny_wide: a copy whose strips hold the rows in another order is not read row by row")
    _check(library().gl3_gemm_skinny_wide(_ptr(a), wp, _ptr(out), _code(out, "out"), M, N, K, a.stride(0),
                                          w.stride(0), rows.stride(0), epilogue, slices, slice_stride, strips,
                                          _bias(bias, wrows, "gemm_skinny_wide"), _act(act, "gemm_skinny_wide"),
                                          None, 0, 0.0, 0, order, float(act_limit), float(act_shift),
                                          _col_scale(col_scale, N, epilogue, "gemm_skinny_wide"), _stream()), "gemm_skinny_wide")


def _check_norm_args(xg, ssq, n_partials, K):
    _dev(xg, "xg", torch.bfloat16, contiguous=False); _dev(ssq, "ssq", torch.float32)
    if xg.dim() != 2 or xg.stride(1) != 1 or xg.shape[1] != K:
        raise KernelError(f"folded norm: rows {tuple(xg.shape)} for K={K}")
    if xg.shape[0] > 64 or n_partials < 1 or ssq.numel() < n_partials * 64:
        raise KernelError("folded norm: at most 64 rows, and n_partials * 64 partial sums")


def gemm_skinny_norm_fits(xg, w, out, epilogue):
    K = xg.shape[1]
    return (xg.shape[0] <= 64 and K % 8 == 0 and xg.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and xg.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and w.dtype == torch.bfloat16
            and ((epilogue == EPI_STORE and out.dtype in (torch.float32, torch.bfloat16))
                 or (epilogue == EPI_GATED and out.dtype == torch.bfloat16)))


def gemm_skinny_norm(xg, ssq, n_partials, eps, w, out, epilogue=EPI_STORE, rows=None, waves=0, bias=None, act="silu",
                     pack_out=False, whole_lines=False, act_limit=0.0, act_shift=0.0):
    """out (=, gated) RMSNorm(x)[rows] @ w.T, where ``xg`` = bfloat16(norm weight * x) was left by the
    kernel that completed the rows of x, together with their sums of squares as partial sums.
    ``pack_out`` (at most 8 rows, bfloat16): ``out`` is a ``packed_rows`` buffer. ``whole_lines`` (gated
    epilogue, at most 16 rows, all rows): the kernel that loads both operands as whole lines and takes
    several strips a block (``gemm_skinny_wide``'s) does the work."""
    _dev(w, "w", torch.bfloat16); _dev(out, "out", contiguous=False)
    K = w.shape[1]
    _check_norm_args(xg, ssq, n_partials, K)
    M = xg.shape[0]
    if rows is not None:
        _dev(rows, "rows", torch.int32)
        M = rows.numel()
    if pack_out:
        n_out = w.shape[0] // 2 if epilogue == EPI_GATED else w.shape[0]
        if M > 8 or out.dtype != torch.bfloat16 or not out.is_contiguous() or out.numel() < -(-n_out // 64) * 512:
            raise KernelError("gemm_skinny_norm: the packed order holds at most 8 rows of bfloat16")
        out = out.view(-1)[:8 * n_out].view(8, n_out)[:M]                      # (the shape only: the kernel knows the order)
    N = out.shape[1]
    wrows = 2 * N if epilogue == EPI_GATED else N
    if w.shape != (wrows, K) or out.shape[0] != M or out.stride(1) != 1 or M > 64:
        raise KernelError(f"gemm: rows {tuple(xg.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}, epilogue {epilogue}")
    if held_once(w) and not whole_lines and not _tiled(w, wrows, K, n_out=N).value:
        raise KernelError("gemm_skinny_norm: a weight kept in the matrix cores' order alone is read through its copy")
    if whole_lines:
        if epilogue != EPI_GATED or rows is not None or M > 16 or waves:
            raise KernelError("gemm_skinny_norm: whole lines go with the gated epilogue, at most 16 rows, all of them")
        order, wp, pos = _w_order(w)
        if pos.value or order == 2:
            raise KernelError("gemm_skinny_norm: the gated product of whole lines reads stored rows or the operands' order")
        return _check(library().gl3_gemm_skinny_wide(
            _ptr(xg), wp, _ptr(out), _code(out, "out"), M, N, K, xg.stride(0), w.stride(0), out.stride(0), epilogue,
            1, 0, 0, _bias(bias, wrows, "gemm_skinny_norm"), _act(act, "gemm_skinny_norm"), _ptr(ssq), n_partials,
            float(eps), int(bool(pack_out)), order, float(act_limit), float(act_shift), None, _stream()), "gemm_skinny_wide")
    _check(library().gl3_gemm_skinny_norm(
        _ptr(xg), _ptr(rows), _ptr(ssq), n_partials, float(eps), _ptr(w), _ptr(out), _code(out, "out"), M, N, K,
        xg.stride(0), w.stride(0), out.stride(0), epilogue, waves, _bias(bias, wrows, "gemm_skinny_norm"),
        _act(act, "gemm_skinny_norm"), _tiled(w, wrows, K, n_out=N), int(bool(pack_out)), float(act_limit), float(act_shift),
        None, _stream()), "gemm_skinny_norm")


def qkv_rope_cache_fits(a, w_qkv, head_dim, rot_dim):
    """a: normalised bfloat16 rows, or bfloat16(norm weight * x) with the sums of squares."""
    K = a.shape[1]
    return (a.shape[0] <= 64 and a.stride(1) == 1 and a.dtype == torch.bfloat16 and K % 8 == 0
            and a.stride(0) % 8 == 0 and w_qkv.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and w_qkv.data_ptr() % 16 == 0 and w_qkv.dtype == torch.bfloat16
            and head_dim % 16 == 0 and rot_dim in (0, head_dim))


def token_facts(positions, table_rows, block_table, page_size, cos, sin, pages, rot, tables=None):
    """What hangs on each token's position, looked up once for all layers of a step: ``pages`` [T] int32
    receives the page of the token's position (``block_table[table_rows[t]][positions[t] // page_size]``) and
    ``rot`` [T, 2 * half] float32 its rows of ``cos`` and ``sin`` one after the other (``cos``, ``sin``, ``rot``
    all None: no rotation, the pages alone). ``qkv_rope_cache`` takes both in place of its own look-ups.
    ``tables`` [T, width of ``block_table``] int32 (optional) receives each token's row of the block table up to
    its position's page: ``attention_decode`` reads it with ``seq_of_token=None``."""
    _dev(positions, "positions", torch.int32); _dev(table_rows, "table_rows", torch.int32)
    _dev(block_table, "block_table", torch.int32); _dev(pages, "pages", torch.int32)
    T = positions.numel()
    if table_rows.numel() != T or pages.numel() != T or block_table.dim() != 2:
        raise KernelError("token_facts: one row of the table and one page per token")
    half = 0
    if cos is not None:
        _dev(cos, "cos", torch.float32); _dev(sin, "sin", torch.float32); _dev(rot, "rot", torch.float32)
        half = cos.shape[1]
        if cos.shape != sin.shape or cos.dim() != 2 or rot.shape != (T, 2 * half):
            raise KernelError(f"token_facts: tables {tuple(cos.shape)}, rows {tuple(rot.shape)} for {T} tokens")
    elif sin is not None or rot is not None:
        raise KernelError("token_facts: the tables and the rows for them come together")
    if tables is not None:
        _dev(tables, "tables", torch.int32)
        if tables.shape != (T, block_table.shape[1]):
            raise KernelError(f"token_facts: the tokens' rows {tuple(tables.shape)} of a table {tuple(block_table.shape)}")
    _check(library().gl3_token_facts(_ptr(positions), _ptr(table_rows), _ptr(block_table), block_table.shape[1], int(page_size),
                                     _ptr(cos), _ptr(sin), half, _ptr(pages), _ptr(rot), _ptr(tables), T, _stream()),
           "token_facts")


def qkv_rope_cache(a, ssq, n_partials, eps, w_qkv, q_out, positions, seq_of_token, block_table, cos, sin,
                   k_cache, v_cache, n_heads, n_kv, head_dim, adjacent, page_size, waves=0, token_pages=None, token_rot=None):
    """a @ w_qkv.T, rotation, q into ``q_out`` [T, H*hs] bfloat16, k and v into the cache. ``ssq`` None:
    ``a`` holds the rows as they are; else ``a`` = bfloat16(norm weight * x) and the product is that
    of RMSNorm(x), the rows' sums of squares coming as partial sums. ``token_pages``, ``token_rot``: what
    ``token_facts`` made of the same positions, table and rotation (then the kernel does not look them up)."""
    _dev(w_qkv, "w_qkv", torch.bfloat16); _dev(q_out, "q_out", torch.bfloat16, contiguous=False)
    K = w_qkv.shape[1]
    if ssq is None:
        _dev(a, "a", torch.bfloat16, contiguous=False)
        if a.dim() != 2 or a.stride(1) != 1 or a.shape[1] != K or a.shape[0] > 64:
            raise KernelError(f"qkv_rope_cache: rows {tuple(a.shape)} for K={K}")
        n_partials = 0
    else:
        _check_norm_args(a, ssq, n_partials, K)
    T = a.shape[0]
    _dev(positions, "positions", torch.int32); _dev(seq_of_token, "seq_of_token", torch.int32)
    _dev(block_table, "block_table", torch.int32)
    _dev(k_cache, "k_cache", torch.bfloat16); _dev(v_cache, "v_cache", torch.bfloat16)
    _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, "qkv_rope_cache")
    if (w_qkv.shape[0] != (n_heads + 2 * n_kv) * head_dim or q_out.shape[0] != T or q_out.stride(1) != 1
            or q_out.shape[1] < n_heads * head_dim or positions.numel() != T or seq_of_token.numel() != T
            or block_table.dim() != 2):
        raise KernelError("qkv_rope_cache: shapes")
    if cos is not None:
        _dev(cos, "cos", torch.float32); _dev(sin, "sin", torch.float32)
        if cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != head_dim // 2:
            raise KernelError(f"qkv_rope_cache: table {tuple(cos.shape)} for head_dim {head_dim}")
    # (the kernel reads the tables through 32-bit byte offsets)
    if block_table.numel() >= 2 ** 29 or (cos is not None and cos.numel() >= 2 ** 29):
        raise KernelError("qkv_rope_cache: a block table or rotation table of 2 GiB or more")
    if token_pages is not None:
        _dev(token_pages, "token_pages", torch.int32)
        if token_pages.numel() != T or (cos is not None and (token_rot is None or token_rot.dtype != torch.float32
                                                             or token_rot.shape != (T, head_dim) or not token_rot.is_cuda
                                                             or not token_rot.is_contiguous())):
            raise KernelError("qkv_rope_cache: a page per token, and with a rotation a row [head_dim] of cos and sin per token")
    copy = _tiled(w_qkv, w_qkv.shape[0], K, qkv=(n_heads, n_kv, head_dim, cos is not None, bool(adjacent)))
    if held_once(w_qkv) and not copy.value:
        raise KernelError("qkv_rope_cache: weights kept in the operands' order alone need the copy made for this rotation")
    _check(library().gl3_qkv_rope_cache(
        _ptr(a), _ptr(ssq), n_partials, float(eps), _ptr(w_qkv), _ptr(q_out), q_out.stride(0), T, K, a.stride(0),
        w_qkv.stride(0), _ptr(positions), _ptr(seq_of_token), _ptr(block_table), block_table.shape[1], _ptr(cos),
        _ptr(sin), _ptr(k_cache), _ptr(v_cache), n_heads, n_kv, head_dim, int(adjacent), page_size, waves,
        copy, _ptr(token_pages), _ptr(token_rot if token_pages is not None and cos is not None else None),
        int(held_once(w_qkv)), _stream()),
        "qkv_rope_cache")


# ------------------------------------------------------------------ bfloat16 attention of a decode step
def attention_decode_fits(head_dim, n_heads, n_kv, page_size):
    return bool(library().gl3_attention_decode_supports(head_dim, page_size)) and n_heads % n_kv == 0


def decode_splits(n_tokens, n_heads, n_kv, kv_len, head_dim=64):
    """Blocks that share a sequence's keys. A split costs a second kernel that merges the parts, which
    is worth its few microseconds only when a block would otherwise walk hundreds of KB of keys (more
    than 128 K elements, or 256 K and more where the step has more than 16 blocks anyway; ``kv_len`` is
    what the launch is sized for, in a replayed step the next power of two, so 4,096 stands for 2,049
    to 4,096 keys), then one split per 64 K elements (per 32 K where the step has at most 16 blocks: one
    sequence of the 1B layers at 4,000 keys, 0.865 -> 0.822 ms a step; the same within 1% at 8,000 to 32,768 keys),
    and only until every CU has a block: more splits than that were slower at every batch and context
    measured (heads of 64, 16 sequences at 8,200 keys: 54 us with 2 splits, 63 us with 8)."""
    blocks = n_tokens * n_kv * -(-(n_heads // n_kv) // 16)
    elements = kv_len * head_dim
    if elements <= 131072 or (blocks > 16 and elements < 262144):
        return 1
    return int(max(1, min(elements // (32768 if blocks <= 16 else 65536), 256 // blocks, 32)))


def attention_decode(q, k_cache, v_cache, positions, seq_of_token, block_table, out, n_heads, n_kv, head_dim,
                     page_size, window, scale, n_splits, part_o=None, part_ml=None, slopes=None, sink=None, keep_first=0,
                     chunk=0, n_v_heads=None):
    """``slopes`` (float32 [H]): score - slopes[h] * distance; ``sink``: the score of a key without a value that every
    query sees (None: none); ``keep_first``: with a window, the sequence's first keys that stay visible; ``chunk`` and
    ``n_v_heads`` as in ``attention_generic``. One token per sequence. ``part_o`` [T, H, splits, hs] and ``part_ml`` [T, H, splits, 2] float32
    are needed when ``n_splits`` > 1 (contiguous, adjacent is not required). ``seq_of_token`` None: token t's
    pages are row t of ``block_table`` (a table of the step's own, as ``token_facts`` makes it)."""
    _dev(q, "q", torch.bfloat16, contiguous=False); _dev(out, "out", torch.bfloat16, contiguous=False)
    _dev(k_cache, "k_cache", torch.bfloat16); _dev(v_cache, "v_cache", torch.bfloat16)
    _dev(positions, "positions", torch.int32); _dev(block_table, "block_table", torch.int32)
    if seq_of_token is not None:
        _dev(seq_of_token, "seq_of_token", torch.int32)
    T = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < n_heads * head_dim:
        raise KernelError(f"attention: q {tuple(q.shape)} for {n_heads} heads of {head_dim}")
    if out.shape != (T, n_heads * head_dim) or out.stride(1) != 1:
        raise KernelError(f"attention: out {tuple(out.shape)}")
    n_v = n_kv if n_v_heads is None else int(n_v_heads)
    if n_kv % n_v or n_heads % (n_kv // n_v) or (chunk and window):
        raise KernelError(f"attention: {n_heads} heads, {n_kv} key heads, {n_v} value heads, chunk {chunk}, window {window}")
    _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, "attention", None, n_v)
    if (positions.numel() != T or block_table.dim() != 2
            or (seq_of_token.numel() != T if seq_of_token is not None else block_table.shape[0] < T)):
        raise KernelError("attention: positions / seq_of_token / block_table shapes")
    floats = 0
    if n_splits > 1:
        _dev(part_o, "part_o", torch.float32); _dev(part_ml, "part_ml", torch.float32)
        if part_o.numel() < T * n_heads * n_splits * head_dim or part_ml.numel() < T * n_heads * n_splits * 2:
            raise KernelError("attention: the workspace of the splits is too small")
        floats = T * n_heads * n_splits * (head_dim + 2)
    has_sink, sink_value, sinks = _sink(sink, n_heads, "attention_decode")
    _check(library().gl3_attention_decode(
        _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(positions), _ptr(seq_of_token), _ptr(block_table),
        block_table.shape[1], _ptr(part_o), _ptr(part_ml), floats, _ptr(out), out.stride(0), T, n_heads, n_kv,
        head_dim, page_size, int(window or 0), float(scale), n_splits, _slopes(slopes, n_heads, "attention_decode"),
        has_sink, sink_value, int(keep_first or 0) if window else 0, int(chunk or 0), n_kv // n_v, sinks,
        _stream()), "attention_decode")


# ------------------------------------------------------------------ bfloat16 product for many rows
def gemm_mfma_fits(a, w, out, epilogue):
    M, K = a.shape
    return (K % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and (out.dtype == torch.float32 or (out.dtype == torch.bfloat16 and epilogue != EPI_ADD)))


def gemm_mfma(a, w, out, epilogue=EPI_STORE, more_slices=None, bias=None, act="silu", shape=0, act_limit=0.0,
              act_shift=0.0, col_scale=None):
    """out (=, +=, gated) a @ w.T on the matrix cores, tiled for many rows of ``a``. With
    ``more_slices`` [S, M, N] float32 K is cut into S + 1 slices: the first goes into ``out``, the
    others' sums are stored there, for the caller to add to ``out`` in that order."""
    _dev(a, "a", torch.bfloat16, contiguous=False); _dev(w, "w", torch.bfloat16); _dev(out, "out", contiguous=False)
    slices, p_stride, ldp = 1, 0, 0
    if more_slices is not None:
        _dev(more_slices, "more_slices", torch.float32, contiguous=False)
        if (more_slices.dim() != 3 or more_slices.shape[1:] != out.shape or more_slices.stride(2) != 1
                or epilogue == EPI_GATED):
            raise KernelError(f"gemm: slices {tuple(more_slices.shape)} for out {tuple(out.shape)}, epilogue {epilogue}")
        slices, p_stride, ldp = more_slices.shape[0] + 1, more_slices.stride(0), more_slices.stride(1)
    if a.dim() != 2 or w.dim() != 2 or out.dim() != 2 or a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: operands must be 2-d with a contiguous last dimension")
    M, K = a.shape
    N = out.shape[1]
    rows = 2 * N if epilogue == EPI_GATED else N
    if w.shape != (rows, K) or out.shape[0] != M:
        raise KernelError(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}, epilogue {epilogue}")
    order, wp, pos = _w_order(w)
    _check(library().gl3_gemm_mfma(_ptr(a), wp, _ptr(out), _code(out, "out"), M, N, K, a.stride(0), w.stride(0),
                                   out.stride(0), epilogue, slices, _ptr(more_slices), p_stride, ldp,
                                   _bias(bias, rows, "gemm_mfma"), _act(act, "gemm_mfma"), int(shape), order, pos,
                                   float(act_limit), float(act_shift), _col_scale(col_scale, N, epilogue, "gemm_mfma"),
                                   _stream()), "gemm_mfma")


def mfma_slices(M, N, K):
    """Into how many slices of K the tiled product [M, K] x [N, K] into the residual stream is cut
    where the tiles of 128 x 128 are at most one for each of the chip's 512 places (two blocks a CU).
    A block's time is its walk along K (half a microsecond per 64 columns, whatever else runs), so few
    tiles over a long K are better cut, down to slices of 512 columns; the norm that follows adds the
    slices up."""
    tiles = -(-M // 128) * -(-N // 128)
    return max(1, min(8, 512 // tiles, K // 512))


def mfma_plan(M, N, K):
    """(tile shape, slices of K) for the tiled product [M, K] x [N, K] into the residual stream, whose
    slices the norm that follows adds up. Few tiles: tiles of 128 x 128 and ``mfma_slices``. More tiles
    than places: the plan with the least estimated time among tiles of 128 (512 places) or 256 (256
    places) with one to four slices and tiles of 128 rows x 256 (256 places) with one, the estimate being (rounds the blocks need on their places) x
    (steps of 64 columns a block walks) x (time of such a step with the chip full: 1.05 us and 1.7 us)
    + what the norm pays per slice (0.35 us per MB). What decides is the last, partly empty round:
    276 tiles of 256 take two rounds for the work of 1.08, and two slices of them 2.16 of 3. Fitted to
    60 sizes (300 to 8,192 rows, the output and down projections of three models) times ten plans: the
    plan chosen is on average 1.4% slower than the best one measured, 13% at worst; one slice and the
    tile by the number of tiles alone was 4.1% and 36%."""
    if -(-M // 128) * -(-N // 128) <= 256:
        return 1, mfma_slices(M, N, K)
    best = None
    # (tile rows, tile columns, places on the chip, time of a step of 64 columns with the chip full); the tile of 128
    # rows x 256, one block a CU, whole K only: 0.95 us a step. It is the plan where its tiles are one round and the
    # others need two rounds or slices: the output projection of 2,048 rows of the 3B layers 81 -> 68 us with its norm,
    # of the 8B layers 110 -> 97 us, of 5,886 rows 307 -> 280 us, of 4,096 rows of the 1B layers 64 -> 60 us.
    for shape, rows, cols, places, step_us in ((1, 128, 128, 512, 1.05), (2, 256, 256, 256, 1.7), (5, 128, 256, 256, 0.95)):
        for slices in ((1,) if shape == 5 else (1, 2, 3, 4)):
            if slices > 1 and K // slices < 512:
                continue
            blocks = -(-M // rows) * -(-N // cols) * slices
            estimate = -(-blocks // places) * -(-K // (64 * slices)) * step_us + 0.35e-6 * (slices + 1.5) * M * N * 4
            if best is None or estimate < best[0]:
                best = (estimate, shape, slices)
    return best[1], best[2]


# ------------------------------------------------------------------ bfloat16 attention of a prefill step
def attention_prefill_fits(head_dim, n_heads, n_kv, page_size):
    return bool(library().gl3_attention_prefill_supports(head_dim, page_size)) and n_heads % n_kv == 0


def attention_prefill(q, k_cache, v_cache, cu_seqlens, kv_before, block_table, out, max_q_len, n_heads, n_kv,
                      head_dim, page_size, window, scale, seq_rows=None, wide_from=0, slopes=None, sink=None, keep_first=0,
                      chunk=0, n_v_heads=None):
    """``slopes`` (float32 [H]): score - slopes[h] * distance; ``sink``: the score of a key without a value that every
    query sees (None: none); ``chunk`` and ``n_v_heads`` as in ``attention_generic``. Any number of tokens per sequence; ``cu_seqlens`` [B+1] and ``kv_before`` [B] say which tokens
    of the packed ``q`` belong to which sequence and where they sit in it. ``seq_rows`` [B] (optional)
    names each sequence's row of ``block_table``; without it sequence b reads row b. ``wide_from``: from
    how many tokens of the step's longest sequence on the kernel with 128 queries a block runs
    (0: the library's choice; tests run both kernels on the same inputs)."""
    _dev(q, "q", torch.bfloat16, contiguous=False); _dev(out, "out", torch.bfloat16, contiguous=False)
    _dev(k_cache, "k_cache", torch.bfloat16); _dev(v_cache, "v_cache", torch.bfloat16)
    _dev(cu_seqlens, "cu_seqlens", torch.int32); _dev(kv_before, "kv_before", torch.int32)
    _dev(block_table, "block_table", torch.int32)
    T = q.shape[0]
    B = kv_before.numel()
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < n_heads * head_dim:
        raise KernelError(f"attention: q {tuple(q.shape)} for {n_heads} heads of {head_dim}")
    if out.shape != (T, n_heads * head_dim) or out.stride(1) != 1:
        raise KernelError(f"attention: out {tuple(out.shape)}")
    n_v = n_kv if n_v_heads is None else int(n_v_heads)
    if n_kv % n_v or n_heads % (n_kv // n_v) or (chunk and window):
        raise KernelError(f"attention: {n_heads} heads, {n_kv} key heads, {n_v} value heads, chunk {chunk}, window {window}")
    _check_cache(k_cache, v_cache, n_kv, page_size, head_dim, "attention", None, n_v)
    if cu_seqlens.numel() != B + 1 or block_table.dim() != 2 or max_q_len < 1:
        raise KernelError("attention: cu_seqlens / kv_before / block_table shapes")
    if seq_rows is not None:
        _dev(seq_rows, "seq_rows", torch.int32)
        if seq_rows.numel() != B:
            raise KernelError("attention: one table row per sequence")
    elif block_table.shape[0] < B:
        raise KernelError("attention: the block table has fewer rows than there are sequences")
    has_sink, sink_value, sinks = _sink(sink, n_heads, "attention_prefill")
    _check(library().gl3_attention_prefill(
        _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(cu_seqlens), _ptr(kv_before), _ptr(block_table),
        _ptr(seq_rows), block_table.shape[1], _ptr(out), out.stride(0), B, int(max_q_len), n_heads, n_kv, head_dim,
        page_size, int(window or 0), float(scale), int(wide_from), _slopes(slopes, n_heads, "attention_prefill"),
        has_sink, sink_value, int(keep_first or 0) if window else 0, int(chunk or 0), n_kv // n_v, sinks,
        _stream()), "attention_prefill")


# ------------------------------------------------------------------ host to device without tensor objects
def scatter_i32(dst, places, values):
    """dst.view(-1)[places[i]] = values[i]: the places and values travel in the launch itself."""
    _dev(dst, "dst", torch.int32)
    n = len(places)
    if n != len(values):
        raise KernelError("scatter_i32: as many places as values")
    if n == 0:
        return
    arr = (c_int * n)
    _check(library().gl3_scatter_i32(_ptr(dst), dst.numel(), arr(*places), arr(*values), n, _stream()), "scatter_i32")


def stage_decode(dst, n_pad, tokens, positions, slots, pad_slot, counter=None):
    """The input of a captured decode step into its device buffer ``dst`` (int32, 4 * n_pad at least):
    tokens | positions | tokens held before | slots of ``len(tokens)`` sequences, padded to ``n_pad``
    with one-token sequences in ``pad_slot``. The numbers travel inside the launch."""
    n = len(tokens)
    if len(positions) != n or len(slots) != n or n > n_pad or dst.numel() < 4 * n_pad:
        raise KernelError("stage_decode: sizes")
    arr = c_int * n
    _check(library().gl3_stage_decode(_ptr(dst), n_pad, n, arr(*tokens), arr(*positions), arr(*slots), pad_slot,
                                      _ptr(counter), _stream()), "stage_decode")


def stage_step_ints(T, B, W):
    """Elements of the device buffer that ``stage_step`` fills."""
    return 4 * T + 3 * B + 1 + W


def stage_step(dev, pinned, tokens, slots, starts, counts, want, vocab):
    """The input of a step of any shape into its device buffer ``dev`` (int32):
    tokens[T] | cu_seqlens[B+1] | kv_before[B] | slots[B] | wanted rows[W] | positions[T] | seq_of_token[T] | table_rows[T].
    ``tokens`` [T], ``want`` [W]: contiguous int32 numpy arrays (the entries' tokens one after another, packed
    rows); ``slots``, ``starts``, ``counts``: one int per entry. The host's part travels as one copy out of
    ``pinned`` (pinned int32 host tensor, free again once that copy has run), the per-token arrays are expanded
    on the device. Token ids are checked against ``vocab``, counts against ``tokens``, rows against T."""
    _dev(dev, "dev", torch.int32)
    T, B, W = int(tokens.size), len(slots), int(want.size)
    if len(starts) != B or len(counts) != B or B == 0 or T == 0:
        raise KernelError("stage_step: one slot, start and count per entry, and at least one token")
    if (tokens.dtype != "int32" or want.dtype != "int32" or not tokens.flags.c_contiguous or not want.flags.c_contiguous
            or tokens.ndim != 1 or want.ndim != 1):
        raise KernelError("stage_step: tokens and wanted rows are contiguous int32 arrays")
    if pinned.is_cuda or not pinned.is_pinned() or pinned.dtype != torch.int32 or pinned.numel() < T + 3 * B + 1 + W:
        raise KernelError("stage_step: the staging buffer must be pinned int32 host memory of T + 3 B + 1 + W elements")
    if dev.numel() < 4 * T + 3 * B + 1 + W:
        raise KernelError("stage_step: the device buffer is too small")
    arr = c_int * B
    _check(library().gl3_stage_step(_ptr(dev), c_void_p(pinned.data_ptr()), c_void_p(tokens.ctypes.data), T, arr(*slots),
                                    arr(*starts), arr(*counts), B, c_void_p(want.ctypes.data if W else 0), W, int(vocab),
                                    _stream()), "stage_step")


def graph_launch(graph_exec):
    """Launch an instantiated graph (its raw handle) on the current stream."""
    _check(library().gl3_graph_launch(c_void_p(graph_exec), _stream()), "graph_launch")


def upload(dst, src_pinned, n_bytes=None):
    """Copy from pinned host memory to the device on the current stream."""
    _dev(dst, "dst")
    if src_pinned.is_cuda or not src_pinned.is_pinned():
        raise KernelError("upload: the source must be pinned host memory")
    n = src_pinned.numel() * src_pinned.element_size() if n_bytes is None else int(n_bytes)
    if n > dst.numel() * dst.element_size() or n > src_pinned.numel() * src_pinned.element_size():
        raise KernelError("upload: more bytes than the tensors hold")
    _check(library().gl3_upload(_ptr(dst), c_void_p(src_pinned.data_ptr()), n, _stream()), "upload")

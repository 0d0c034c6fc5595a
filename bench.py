"""Decode and prefill throughput of the Llama-3.2-1B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--shape 1b|3b|8b]
                    [--prompt-len P] [--prefill-len T] [--workload decode|unequal8]

A step is one decode step of the generation loop: the engine's step for B sequences (one
token each, from the cache left by 512-token prompts) and the greedy pick of the next
token on the device. ``value`` is decoded tokens a second at the default batch of 8.
The same line carries the prefill of one 2,048-token prompt, the decode step's share of
the memory roofline, and decode at batch 1 and 64. Peaks are the published ones of the
MI355X: 8 TB/s HBM3E, 2.5 PFLOP/s dense bf16 matrix throughput. Other layer sizes (--shape) and
lengths are for looking further; the default run is the one that is reported.

Two further workloads with lines of the same form:
  * ``--workload unequal8`` (with the layers of Llama-3.2-3B unless --shape says otherwise): 8 requests
    whose prompt lengths are drawn uniformly from [64, 2048] with the seed, their prompts in ONE packed
    step (timed as the prefill), then --steps decode steps (default 128); the bytes of a step are the
    weights once and the cache at the lengths the sequences really have at that step.
  * the Llama-3.1-8B pair: ``--shape 8b --batch 64 --prompt-len 1024 --prefill-len 8192 --points ""``.

``--arch melizen`` measures another decoder of the library instead, beside Llama layers of equal size on the same
machine: a Melizen model (windowed attention with a distance bias and a sink in every other layer, a gated delta
rule in the others, one norm a layer, a bounded gated feed-forward) with the width, feed-forward size, head sizes,
vocabulary and layer count of ``--shape`` (``--layers`` for fewer), random weights. Its line carries prefill and
decode throughput of both and their ratio; the default run and its line are not touched by it.
``--arch nodupel`` does the same for a Nodupel model (every fourth layer a minGRU, the others an attention with
rotated values, a gate per head and a window that keeps the first keys beside a time mixing with heads of 64; the
shape's gated feed-forward in every layer; a hashed table of token pairs beside the embedding; no loop).
``--arch nolatar`` does the same for a Nolatar model (layers in turns of four: a state space with heads of 64 and a
state of 128, a chunked attention beside a retention, a differential attention, and one more that reads the third's
keys and values; layer norms behind the sublayers; in every layer a routed feed-forward of 8 experts of a quarter of
the shape's feed-forward size, two a token, beside a shared expert of that size: the shape's multiply-adds a token
in three quarters of its feed-forward, 2.25 times its feed-forward weights).
``--arch dotanex`` does the same for a Dotanex model (two copies of the residual row mixed around every sublayer;
layers in turns of four: a lightning attention, an attention over cached latents, a lightning attention, a windowed
attention with learned sinks whose values are its keys; the first layer's feed-forward is the shape's own, every other
layer has 8 gated experts of a quarter of that size and 2 identity experts, two a token, beside a shared expert).
``--beside nolatar`` puts a Nolatar model of the same sizes beside it instead of the Llama layers.
"""
import argparse
import json
import os
import shutil
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

# every size as the model's own config.json gives it; "1b" is the shape that the default run measures
_COMMON = {"architectures": ["LlamaForCausalLM"], "vocab_size": 128256, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
           "hidden_act": "silu"}


def _scaling(factor):
    return {"rope_type": "llama3", "factor": factor, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
            "original_max_position_embeddings": 8192}


SHAPES = {
    "1b": ("Llama-3.2-1B shape", {**_COMMON, "hidden_size": 2048, "intermediate_size": 8192, "num_hidden_layers": 16,
                                  "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
                                  "max_position_embeddings": 4096, "rope_scaling": _scaling(32.0),
                                  "tie_word_embeddings": True}),
    "3b": ("Llama-3.2-3B shape", {**_COMMON, "hidden_size": 3072, "intermediate_size": 8192, "num_hidden_layers": 28,
                                  "num_attention_heads": 24, "num_key_value_heads": 8, "head_dim": 128,
                                  "max_position_embeddings": 4096, "rope_scaling": _scaling(32.0),
                                  "tie_word_embeddings": True}),
    "8b": ("Llama-3.1-8B shape", {**_COMMON, "hidden_size": 4096, "intermediate_size": 14336, "num_hidden_layers": 32,
                                  "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
                                  "max_position_embeddings": 8192, "rope_scaling": _scaling(8.0),
                                  "tie_word_embeddings": False}),
}
SHAPE = SHAPES["1b"][1]
CONTEXT = 4096
PROMPT = 512
PREFILL = 2048


def weight_bytes(c, esize):
    per_layer = c.hidden_size * (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim \
        + c.num_attention_heads * c.head_dim * c.hidden_size + 3 * c.hidden_size * c.intermediate_size \
        + 2 * c.hidden_size
    return esize * (c.num_hidden_layers * per_layer + c.vocab_size * c.hidden_size + c.hidden_size)


def decode_bytes(c, esize, kv_lens):
    """Every weight once (the head too; of the embedding only the rows used) and the cache
    of the live requests."""
    cache = sum(kv_lens) * 2 * c.num_hidden_layers * c.num_key_value_heads * c.head_dim * esize
    return weight_bytes(c, esize) + len(kv_lens) * c.hidden_size * esize + cache


def prefill_flops(c, T, rows=1):
    linear = 2 * T * c.num_hidden_layers * (
        c.hidden_size * (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim
        + c.num_attention_heads * c.head_dim * c.hidden_size + 3 * c.hidden_size * c.intermediate_size)
    attention = c.num_hidden_layers * 4 * c.num_attention_heads * c.head_dim * T * (T + 1) // 2
    return linear + attention + 2 * rows * c.hidden_size * c.vocab_size


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed decode steps (default 64; 128 for unequal8)")
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--shape", default="1b", choices=sorted(SHAPES), help="layer sizes; the default is what is reported")
    ap.add_argument("--layers", type=int, default=None,
                    help="fewer layers than the shape has (reported as such); never smaller layers")
    ap.add_argument("--prompt-len", type=int, default=PROMPT, help="tokens every sequence holds before the decode steps")
    ap.add_argument("--prefill-len", type=int, default=PREFILL, help="tokens of the prompt whose prefill is timed")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=None,
                    help="the longest sequence (max_position_embeddings) instead of the shape's; reported as seq_len")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,64", help="further decode batch sizes, comma-separated")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--workload", default="decode", choices=["decode", "unequal8"])
    ap.add_argument("--arch", default="llama", choices=["llama", "melizen", "nodupel", "nolatar", "dotanex"],
                    help="melizen, nodupel, nolatar, dotanex: a model of that design with the shape's sizes beside Llama layers of "
                         "equal size (a line of its own form)")
    ap.add_argument("--beside", default="llama", choices=["llama", "melizen", "nodupel", "nolatar"],
                    help="with --arch: the model of equal size that is measured beside it")
    ap.add_argument("--without", default="", help="names of fast paths to switch off for a comparison on the same machine, "
                    "comma-separated (parts/ops.py: tiled, packed, fused, wide, ...); the line then says so in `config`")
    args = ap.parse_args()
    if args.workload == "unequal8" and "--shape" not in " ".join(sys.argv):
        args.shape = "3b"
    if args.steps is None:
        args.steps = 128 if args.workload == "unequal8" else 64
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU library")
        return 2

    if args.arch in ("melizen", "nodupel", "nolatar", "dotanex"):
        return other_beside_llama(args)

    import numpy as np
    import torch
    import gpullama3_java_amd as g
    from gpullama3_java_amd.engine import Engine

    shape_name, shape = SHAPES[args.shape]
    if args.context is not None:
        shape = {**shape, "max_position_embeddings": args.context}
    context = shape["max_position_embeddings"]
    prompt_len, prefill_len = args.prompt_len, args.prefill_len
    if args.layers is None:
        args.layers = shape["num_hidden_layers"]
    cfg = g.config_from_dict({**shape, "num_hidden_layers": args.layers})
    esize = 2 if args.dtype == "bfloat16" else 4
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    K, W = args.steps, args.warmup
    points = [int(b) for b in args.points.split(",") if b]
    biggest = max([args.batch] + points)
    per_seq = -(-(prompt_len + K + W + 1) // 64) * 64
    if args.workload == "unequal8":
        args.batch, points, biggest = 8, [], 8
        per_seq = -(-(2048 + K + W + 1) // 64) * 64
        prefill_len = 0
    tmp = tempfile.mkdtemp(prefix="gl3-bench-")
    try:
        t0 = time.time()
        g.write_random_model(tmp, cfg, args.seed)
        print(f"[bench] random {args.layers}-layer model written in {time.time() - t0:.0f} s", file=sys.stderr, flush=True)
        eng = Engine.from_folder(tmp, dtype=args.dtype, max_context=context,
                                 max_tokens=max(biggest * per_seq, prefill_len + 64), n_slots=biggest,
                                 without=args.without)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    rng = np.random.default_rng(args.seed)
    V = cfg.vocab_size

    def sync():
        torch.cuda.synchronize()

    if args.workload == "unequal8":
        return unequal8(args, eng, cfg, rng, shape_name, shape, esize, short, sync)

    # ---- prefill: one prompt (2,048 tokens unless told otherwise), logits at its last token
    def prefill_once():
        s = eng.take_slot()
        toks = rng.integers(0, V, prefill_len).tolist()
        sync(); t = time.perf_counter()
        eng.step([(s, toks)])
        sync(); dt = time.perf_counter() - t
        eng.give_back_slot(s)
        return dt
    prefill_once()
    prefill_s = min(prefill_once() for _ in range(3))
    print(f"[bench] prefill {prefill_len} tokens: {prefill_s * 1e3:.2f} ms", file=sys.stderr, flush=True)

    # ---- decode at batch B after prompts of prompt_len tokens
    def decode(B):
        slots = [eng.take_slot() for _ in range(B)]
        for lo in range(0, B, 8):                              # prompts in groups of 8 to bound the step's memory
            eng.step([(s, rng.integers(0, V, prompt_len).tolist()) for s in slots[lo:lo + 8]], want="none")
        temps, tops = [0.0] * B, [1.0] * B
        toks = rng.integers(0, V, B).tolist()
        run = eng.decode_run_length

        def steps(toks, n):
            """n decode steps: runs of steps on the device, the tokens fed back there, as the
            generation loop does it."""
            while n > 0:
                m = min(run, n)
                if m > 1:
                    toks = eng.decode_run(list(zip(slots, toks)), m, temps, tops, [[0.0] * B] * m)[-1]
                else:
                    toks = eng.sample(eng.step([(s, [t]) for s, t in zip(slots, toks)]), temps, tops, [0.0] * B)
                n -= m
            return toks
        toks = steps(toks, W)
        kv = [eng.cache.length(s) for s in slots]
        sync(); t = time.perf_counter()
        toks = steps(toks, K)
        sync(); dt = time.perf_counter() - t
        for s in slots:
            eng.give_back_slot(s)
        mean_kv = [n + (K + 1) / 2 for n in kv]               # the cache read grows by one token a step
        return dt, decode_bytes(cfg, esize, mean_kv)

    results = {}
    for B in [args.batch] + [b for b in points if b != args.batch]:
        dt, nbytes = decode(B)
        results[B] = (dt, nbytes)
        print(f"[bench] decode B={B}: {dt / K * 1e3:.3f} ms/step, {B * K / dt:.0f} tok/s, "
              f"{nbytes / (dt / K) / 1e9:.0f} GB/s", file=sys.stderr, flush=True)

    dt, nbytes = results[args.batch]
    ms = dt / K * 1e3
    achieved = nbytes / (dt / K) / 1e9
    flops = prefill_flops(cfg, prefill_len)
    line = {
        "metric": f"decode tok/s at batch {args.batch} ({shape_name}, {prompt_len}-token prompts)",
        "value": round(args.batch * K / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic: random N(0,0.02) weights, uniform random token ids",
        "config": {
            "model": shape_name, "layers": args.layers, "layers_of_shape": shape["num_hidden_layers"],
            "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
            "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "vocab_size": cfg.vocab_size, "tied_head": cfg.tie_word_embeddings, "rope_theta": cfg.rope_theta,
            "rope_scaling_factor": cfg.rope_scaling.factor, "rms_norm_eps": cfg.rms_norm_eps,
            "global_batch": args.batch, "seq_len": context, "prompt_len": prompt_len, "prefill_len": prefill_len,
            "parallelism": "single GPU", "sampling": "greedy on device", **({"without": args.without} if args.without else {}),
        },
        "prefill": {"value": round(prefill_len / prefill_s, 1), "tokens": prefill_len, "ms": round(prefill_s * 1e3, 3),
                    "frac": round(flops / prefill_s / (PEAK_TFLOPS[short] * 1e12), 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
        "points": {f"decode_b{B}": round(B * K / results[B][0], 1) for B in results if B != args.batch},
    }
    print(json.dumps(line))
    return 0


def unequal8(args, eng, cfg, rng, shape_name, shape, esize, short, sync):
    """8 requests with prompts of unequal lengths that start together: the prompts in one packed step,
    then one token each per step (runs of steps on the device, as the generation loop drives them)."""
    import torch
    K, W, V = args.steps, args.warmup, cfg.vocab_size
    lens = rng.integers(64, 2049, 8).tolist()
    prompts = [rng.integers(0, V, n).tolist() for n in lens]
    best = None
    for _ in range(2):                                   # the first pass sizes the buffers
        slots = [eng.take_slot() for _ in range(8)]
        sync(); t = time.perf_counter()
        eng.step(list(zip(slots, prompts)))
        sync(); dt = time.perf_counter() - t
        best = dt if best is None else min(best, dt)
        if _ == 0:
            for s in slots:
                eng.give_back_slot(s)
    prefill_s = best
    T = sum(lens)
    print(f"[bench] packed prefill of {lens} = {T} tokens: {prefill_s * 1e3:.2f} ms", file=sys.stderr, flush=True)
    temps, tops = [0.0] * 8, [1.0] * 8
    toks = rng.integers(0, V, 8).tolist()
    run = eng.decode_run_length

    def steps(toks, n):
        while n > 0:
            m = min(run, n)
            if m > 1:
                toks = eng.decode_run(list(zip(slots, toks)), m, temps, tops, [[0.0] * 8] * m)[-1]
            else:
                toks = eng.sample(eng.step([(s, [t]) for s, t in zip(slots, toks)]), temps, tops, [0.0] * 8)
            n -= m
        return toks
    toks = steps(toks, W)
    kv = [eng.cache.length(s) for s in slots]
    sync(); t = time.perf_counter()
    steps(toks, K)
    sync(); dt = time.perf_counter() - t
    nbytes = decode_bytes(cfg, esize, [n + (K + 1) / 2 for n in kv])      # the mean over the K steps
    ms = dt / K * 1e3
    achieved = nbytes / (dt / K) / 1e9
    # the flops of the packed prompts: the products of T tokens, each prompt's own causal attention, 8 head rows
    flops = prefill_flops(cfg, T, rows=8) - cfg.num_hidden_layers * 4 * cfg.num_attention_heads * cfg.head_dim * (
        T * (T + 1) // 2 - sum(n * (n + 1) // 2 for n in lens))
    line = {
        "metric": f"decode tok/s, 8 requests with prompts of {min(lens)}..{max(lens)} tokens ({shape_name})",
        "value": round(8 * K / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic: random N(0,0.02) weights, uniform random token ids",
        "config": {
            "model": shape_name, "layers": args.layers, "layers_of_shape": shape["num_hidden_layers"],
            "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
            "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "vocab_size": cfg.vocab_size, "tied_head": cfg.tie_word_embeddings, "global_batch": 8,
            "seq_len": shape["max_position_embeddings"], "prompt_len_min": min(lens), "prompt_len_max": max(lens),
            "prompt_tokens": T, "mean_context": round(sum(kv) / 8 + (K + 1) / 2, 1), "new_tokens": K,
            "parallelism": "single GPU", "sampling": "greedy on device", **({"without": args.without} if args.without else {}),
        },
        "prefill": {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
                    "frac": round(flops / prefill_s / (PEAK_TFLOPS[short] * 1e12), 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
        "points": {},
    }
    print(json.dumps(line))
    return 0


def melizen_config(shape, layers, window=1024):
    """A Melizen model with the sizes of a Llama shape: attention layers with the shape's heads (values of the keys'
    size) and a window, delta layers with as many value heads of the same size over the shape's kv heads, the
    shape's feed-forward in every layer."""
    d, F = shape["hidden_size"], shape["intermediate_size"]
    H, G, hs = shape["num_attention_heads"], shape["num_key_value_heads"], shape["head_dim"]
    mlp = {"kind": "dense", "ff": F, "limit": 7.0}
    attn = {"type": "attention", "mlp": mlp,
            "mixer": {"heads": H, "kv_heads": G, "dim": hs, "vdim": hs, "scale": hs ** -0.5, "mask": {"size": window}}}
    delta = {"type": "delta", "mlp": mlp, "mixer": {"heads": H, "kv_heads": G, "dim": hs, "vdim": hs, "conv": 4}}
    return {"architecture": "Melizen", "vocab": shape["vocab_size"], "width": d, "max_positions": shape["max_position_embeddings"],
            "norm": {"eps": 1e-5}, "layers": [attn if i % 2 == 0 else delta for i in range(layers)]}


def nodupel_config(shape, layers, window=1024, keep_first=4):
    """A Nodupel model with the sizes of a Llama shape: every fourth layer a minGRU of the model's width, the others an
    attention with the shape's heads (rotated values, a gate per head, a window that keeps the first keys) beside a
    time mixing with heads of 64 over the model's width; the shape's feed-forward in every layer; no loop."""
    d, F = shape["hidden_size"], shape["intermediate_size"]
    H, G, hs = shape["num_attention_heads"], shape["num_key_value_heads"], shape["head_dim"]
    mlp = {"kind": "dense", "ff": F}
    left = {"heads": H, "kv_heads": G, "dim": hs, "vdim": hs, "scale": hs ** -0.5,
            "rot": {"base": shape.get("rope_theta", 500000.0), "dims": hs}, "mask": {"size": window, "keep_first": keep_first}}
    side = {"type": "parallel", "mlp": mlp, "mixer": {"left": left, "right": {"heads": d // 64, "dim": 64}}}
    gru = {"type": "mingru", "mlp": mlp, "mixer": {"width": d}}
    return {"architecture": "Nodupel", "vocab": shape["vocab_size"], "width": d, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
            "logit_softcap": 30.0, "max_positions": shape["max_position_embeddings"], "decay_rank": [64] * layers,
            "embedding": {"scale": 1.0, "bigram": {"buckets": 65521, "mul_prev": 31, "mul_cur": 17}},
            "layers": [gru if i % 4 == 0 else side for i in range(layers)]}


def nolatar_config(shape, layers, chunk=1024):
    """A Nolatar model with the sizes of a Llama shape, layers in turns of four: a state space (heads of 64 over the
    model's width, a state of 128, 8 groups), a chunked attention with the shape's heads beside a retention (half as
    many heads, values of twice the keys' size), a differential attention with half the shape's heads (two score
    maps each, values of the keys' size), and one more that reads the third's keys and values. Every layer has 8
    experts of a quarter of the shape's feed-forward size, two a token, and a shared expert of that size."""
    d, F = shape["hidden_size"], shape["intermediate_size"]
    H, G, hs = shape["num_attention_heads"], shape["num_key_value_heads"], shape["head_dim"]
    base = shape.get("rope_theta", 500000.0)
    mlp = {"kind": "moe", "router": {"experts": 8, "top": 2}, "expert": {"ff": F // 4}, "shared": {"ff": F // 4}}
    rot = {"base": base, "dims": hs}
    ssm = {"type": "mamba2", "mlp": mlp,
           "mixer": {"heads": d // 64, "vdim": 64, "state": 128, "groups": 8, "conv": 4, "norm_groups": 8}}
    left = {"heads": H, "kv_heads": G, "dim": hs, "vdim": hs, "scale": hs ** -0.5, "rot": rot, "mask": {"size": chunk}}
    right = {"heads": H // 2, "dim": hs, "vdim": 2 * hs, "rot": rot, "decay": [1.0 - 2.0 ** (-5 - (i % 8)) for i in range(H // 2)]}
    side = {"type": "parallel", "mlp": mlp, "mixer": {"left": left, "right": right, "left_scale": 0.75, "right_scale": 1.25}}
    diff = {"heads": H // 2, "kv_heads": max(1, G // 2), "dim": hs, "vdim": hs, "scale": hs ** -0.5, "diff": 0.5, "rot": rot}
    out = []
    for i in range(layers):
        kind = i % 4
        if kind == 3:
            out.append({"type": "attention", "mlp": mlp, "mixer": {**diff, "kv_from": i - 1}})
        else:
            out.append([ssm, side, {"type": "attention", "mlp": mlp, "mixer": diff}][kind])
    return {"architecture": "Nolatar", "vocab": shape["vocab_size"], "width": d, "norm": {"eps": 1e-5},
            "max_positions": shape["max_position_embeddings"], "layers": out}


def dotanex_config(shape, layers, window=1024, streams=2):
    """A Dotanex model with the sizes of a Llama shape, layers in turns of four: a lightning attention (half the
    shape's heads, values of twice the keys' size), an attention over cached latents (the shape's heads, latents of half
    the width for queries), a
    lightning attention, and a windowed attention with the shape's heads and a sink per head (the latents: 256 elements
    for keys and values, or four heads' size where that is less, beside a rotated part of 32). The first layer has the
    shape's feed-forward; every other layer 8 gated experts of a quarter of its size and 2 identity experts, two a
    token, and a shared expert of that size."""
    d, F = shape["hidden_size"], shape["intermediate_size"]
    H, G, hs = shape["num_attention_heads"], shape["num_key_value_heads"], shape["head_dim"]
    base = shape.get("rope_theta", 500000.0)
    top = shape["max_position_embeddings"]
    moe = {"kind": "moe", "router": {"experts": 8, "identity": 2, "top": 2}, "expert": {"ff": F // 4, "limit": 7.0},
           "shared": {"ff": F // 4, "limit": 7.0}}
    light = {"heads": H // 2, "dim": hs, "vdim": 2 * hs, "decay": [1.0 - 2.0 ** (-5 - (i % 8)) for i in range(H // 2)]}
    rot_dim, kv_rank = min(hs // 2, 32), min(4 * hs, 256)      # (cached rows of 288: what the matrix-core kernel takes)
    latent = {"heads": H, "dim": hs, "rot_dim": rot_dim, "vdim": hs, "q_rank": d // 2, "kv_rank": kv_rank,
              "scale": (hs + rot_dim) ** -0.5,
              "rot": {"base": base, "dims": rot_dim, "scaling": {"factor": 8.0, "original": top // 8, "fast": 32.0, "slow": 1.0}}}
    win = {"heads": H, "kv_heads": G, "dim": hs, "vdim": hs, "scale": hs ** -0.5, "mask": {"size": window},
           "rot": {"base": base, "dims": hs, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": top // 8}}}
    kinds = [("lightning", light), ("latent_attention", latent), ("lightning", light), ("attention", win)]
    out = [{"type": kinds[i % 4][0], "mixer": kinds[i % 4][1], "mlp": {"kind": "dense", "ff": F} if i == 0 else moe}
           for i in range(layers)]
    return {"architecture": "Dotanex", "vocab": shape["vocab_size"], "width": d, "norm": {"eps": 1e-5}, "streams": streams,
            "max_positions": top, "layers": out}


def other_beside_llama(args):
    """Prefill of one prompt and decode steps at --batch for a model of another design (--arch) and for Llama layers
    of equal size, one after the other on the same machine."""
    import numpy as np
    import torch
    import gpullama3_java_amd as g
    from gpullama3_java_amd.engine import Engine

    shape_name, shape = SHAPES[args.shape]
    layers = args.layers or shape["num_hidden_layers"]
    K, W, B = args.steps, args.warmup, args.batch
    prompt_len, prefill_len = args.prompt_len, args.prefill_len
    per_seq = -(-(prompt_len + K + W + 1) // 64) * 64
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    arch = args.arch
    makers = {"melizen": melizen_config, "nodupel": nodupel_config, "nolatar": nolatar_config, "dotanex": dotanex_config}
    beside = "llama" if args.beside == arch else args.beside
    configs = {arch: g.config_from_dict(makers[arch](shape, layers)),
               beside: g.config_from_dict({**shape, "num_hidden_layers": layers} if beside == "llama"
                                          else makers[beside](shape, layers))}
    results = {}
    for name, cfg in configs.items():
        tmp = tempfile.mkdtemp(prefix="gl3-bench-")
        try:
            g.write_random_model(tmp, cfg, args.seed, norm_std=0.02)
            eng = Engine.from_folder(tmp, dtype=args.dtype, max_tokens=max(B * per_seq, prefill_len + 64), n_slots=B,
                                     without=args.without)
        finally:
            shutil.rmtree(tmp, ignore_errors=True)
        rng = np.random.default_rng(args.seed)
        V = eng.spec.vocab_size

        def prefill_once():
            s = eng.take_slot()
            toks = rng.integers(0, V, prefill_len).tolist()
            torch.cuda.synchronize(); t = time.perf_counter()
            eng.step([(s, toks)])
            torch.cuda.synchronize(); dt = time.perf_counter() - t
            eng.give_back_slot(s)
            return dt
        prefill_once()
        prefill_s = min(prefill_once() for _ in range(3))
        slots = [eng.take_slot() for _ in range(B)]
        for lo in range(0, B, 8):
            eng.step([(s, rng.integers(0, V, prompt_len).tolist()) for s in slots[lo:lo + 8]], want="none")
        temps, tops = [0.0] * B, [1.0] * B
        toks = rng.integers(0, V, B).tolist()
        run = eng.decode_run_length

        def steps(toks, n):
            while n > 0:
                m = min(run, n)
                if m > 1:
                    toks = eng.decode_run(list(zip(slots, toks)), m, temps, tops, [[0.0] * B] * m)[-1]
                else:
                    toks = eng.sample(eng.step([(s, [t]) for s, t in zip(slots, toks)]), temps, tops, [0.0] * B)
                n -= m
            return toks
        toks = steps(toks, W)
        torch.cuda.synchronize(); t = time.perf_counter()
        steps(toks, K)
        torch.cuda.synchronize(); dt = time.perf_counter() - t
        results[name] = {"prefill_ms": round(prefill_s * 1e3, 3), "prefill_tok_s": round(prefill_len / prefill_s, 1),
                         "decode_ms_per_step": round(dt / K * 1e3, 4), "decode_tok_s": round(B * K / dt, 1)}
        print(f"[bench] {name}: prefill {prefill_len} tokens {prefill_s * 1e3:.2f} ms, decode B={B} {dt / K * 1e3:.3f} ms/step",
              file=sys.stderr, flush=True)
        del eng
        torch.cuda.empty_cache()
    m, l = results[arch], results[beside]
    title = arch.capitalize()
    line = {
        "metric": f"decode tok/s at batch {B}, {title} model of the {shape_name}'s sizes ({prompt_len}-token prompts)",
        "value": m["decode_tok_s"], "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": m["decode_ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic: random N(0,0.02) weights, uniform random token ids",
        "config": {"model": f"{title}, sizes of the {shape_name}", "layers": layers, "global_batch": B,
                   "seq_len": shape["max_position_embeddings"], "prompt_len": prompt_len, "prefill_len": prefill_len,
                   "attention_window": 1024, "parallelism": "single GPU", "sampling": "greedy on device",
                   **({"without": args.without} if args.without else {})},
        arch: m, f"{beside}_of_equal_size": l,
        f"{arch}_over_{beside}": {"prefill_time": round(m["prefill_ms"] / l["prefill_ms"], 3),
                               "decode_step_time": round(m["decode_ms_per_step"] / l["decode_ms_per_step"], 3)},
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

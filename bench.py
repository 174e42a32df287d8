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


if __name__ == "__main__":
    sys.exit(main())

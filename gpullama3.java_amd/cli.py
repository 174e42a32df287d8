"""Command line in the manner of the reference's ``llama-tornado`` launcher and its
Java options (R/llama-tornado:330-398, J/Options.java:31-48, :84-117): the same
option names with the same meanings where the reference has them.

  --model, -m <path>       model folder (config.json + model.safetensors); the reference takes a .gguf file
  --prompt, -p <string>    input prompt; needs tokenizer.json in the model folder
  --prompt-ids <ids>       input prompt as comma-separated token ids (the library's contract starts at ids)
  --temperature, --temp    sampling temperature, 0 = greedy (default 0.1)
  --top-p                  nucleus mass in [0,1]; 0 or 1 disables (default 0.95)
  --seed, -s               random seed (default: the clock)
  --max-tokens, -n         upper bound on positions, prompt and generated together;
                           < 0: the model's context length (default 512)
  --stream <bool>          print tokens as they are generated (default true)
  --echo <bool>            print all tokens, the prompt's too, to stderr (default false)
  --dtype                  bfloat16 | float32 (not in the reference, whose GPU path is fp16 weights only)
  --write-random-model <config.json>   write a random-weights model folder into --model and exit
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time


def _bool(v):
    return str(v).lower() in ("1", "true", "yes", "on")


def create_parser():
    p = argparse.ArgumentParser(prog="llama-hip", description="Llama 3 generation on one MI355X",
                                formatter_class=argparse.ArgumentDefaultsHelpFormatter)
    p.add_argument("--model", "-m", dest="model_path", required=True, help="model folder")
    p.add_argument("--prompt", "-p", help="input prompt (needs tokenizer.json in the model folder)")
    p.add_argument("--prompt-ids", help="input prompt as comma-separated token ids")
    p.add_argument("--temperature", "--temp", type=float, default=0.1, help="sampling temperature, 0 = greedy")
    p.add_argument("--top-p", type=float, default=0.95, help="top-p (nucleus) mass in [0,1]")
    p.add_argument("--seed", "-s", type=int, default=None, help="random seed (default: the clock)")
    p.add_argument("--max-tokens", "-n", type=int, default=512,
                   help="bound on positions, prompt and generated together; < 0 = the context length")
    p.add_argument("--stream", type=_bool, default=True, help="print tokens as they are generated")
    p.add_argument("--echo", type=_bool, default=False, help="print all tokens to stderr")
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--write-random-model", metavar="CONFIG_JSON",
                   help="write a random-weights model folder into --model from this config.json and exit")
    return p


def main(argv=None):
    args = create_parser().parse_args(argv)
    if not 0 <= args.temperature:
        print("ERROR Invalid argument: --temperature must be non-negative", file=sys.stderr)
        return 2
    if not 0 <= args.top_p <= 1:
        print("ERROR Invalid argument: --top-p must be within [0, 1]", file=sys.stderr)
        return 2
    seed = args.seed if args.seed is not None else time.time_ns()
    import gpullama3_java_amd as g
    if args.write_random_model:
        with open(args.write_random_model) as f:
            cfg = g.config_from_dict(json.load(f))
        g.write_random_model(args.model_path, cfg, seed)
        print(f"wrote {args.model_path}")
        return 0
    tokenizer = None
    tok_path = os.path.join(args.model_path, "tokenizer.json")
    if os.path.isfile(tok_path):
        from tokenizers import Tokenizer
        tokenizer = Tokenizer.from_file(tok_path)
    if args.prompt_ids:
        prompt = [int(t) for t in args.prompt_ids.replace(" ", "").split(",") if t]
    elif args.prompt is not None:
        if tokenizer is None:
            print(f"ERROR --prompt needs {tok_path}; without a tokenizer give --prompt-ids", file=sys.stderr)
            return 2
        prompt = tokenizer.encode(args.prompt).ids
    else:
        print('ERROR Missing argument: --prompt is required e.g. --prompt "Why is the sky blue?"', file=sys.stderr)
        return 2
    engine = g.load_model(args.model_path, context_length=args.max_tokens, dtype=args.dtype,
                          max_tokens=None)
    sampler = g.select_sampler(engine.config.vocab_size, args.temperature, args.top_p, seed)
    if args.echo:
        print(" ".join(str(t) for t in prompt), end=" ", file=sys.stderr, flush=True)

    def show(tok):
        if args.stream:
            text = tokenizer.decode([tok]) if tokenizer is not None else f"{tok} "
            print(text, end="", flush=True)

    out = engine.generate_tokens(prompt, engine.config.stop_ids, args.max_tokens, sampler, echo=args.echo,
                                 on_token_generated=show)
    if out and out[-1] in engine.config.stop_ids:
        out = out[:-1]                                # callers drop the stop token (J/model/Model.java:242-244)
    if not args.stream:
        print(tokenizer.decode(out) if tokenizer is not None else " ".join(str(t) for t in out))
    else:
        print()
    m = engine.metrics
    total = m.prompt_tokens + m.generated_tokens
    secs = m.prefill_seconds + m.decode_seconds
    # the reference's line (J/auxiliary/LastRunMetrics.java:27-31), then prompt and decode apart
    print(f"\nachieved tok/s: {total / secs if secs else 0:.2f}. Tokens: {total}, seconds: {secs:.2f}", file=sys.stderr)
    print(f"prefill: {m.prompt_tokens} tokens in {m.prefill_seconds:.3f} s; decode: {m.decode_steps} steps in "
          f"{m.decode_seconds:.3f} s", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())

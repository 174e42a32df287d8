"""Command line in the manner of the reference's ``llama-tornado`` launcher and its
Java options (R/llama-tornado:330-398, J/Options.java:31-48, :84-117): the same
option names with the same meanings where the reference has them.

  --model, -m <path>            model folder (config.json + model.safetensors); the reference takes a .gguf file
  --interactive, --chat, -i     chat mode: a prompt per line of standard input, "quit" or "exit" ends it
  --instruct                    one prompt, one answer (the default mode)
  --prompt, -p <string>         input prompt; needs tokenizer.json in the model folder
  --system-prompt, -sp <string> system prompt, put in front of the dialogue
  --suffix <string>             accepted as in the reference, where only fill-in-the-middle models use it
  --prompt-ids <ids>            the prompt as comma-separated token ids, fed as they are
                                (not in the reference; the library's contract starts at ids)
  --temperature, --temp         sampling temperature, 0 = greedy (default 0.1)
  --top-p                       nucleus mass in [0,1]; 0 or 1 disables (default 0.95)
  --seed, -s                    random seed (default: the clock)
  --max-tokens, -n              upper bound on positions, prompt and generated together;
                                < 0: the model's context length (default 1024)
  --stream <bool>               print tokens as they are generated (default true)
  --echo <bool>                 print all tokens, the prompt's too, to stderr (default false)
  --dtype                       bfloat16 | float32 (not in the reference, whose GPU path is fp16 weights only)
  --write-random-model <config.json>   write a random-weights model folder into --model and exit

With a text prompt the tokens are those of the reference's chat format
(J/model/Model.java:76-260): begin-of-text, the system message if one is given, the user's
message, and the header of the assistant's answer.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

from .chat import ASSISTANT, SYSTEM, USER, HFTokenizer, Message

DEFAULT_MAX_TOKENS = 1024      # J/Options.java:10


def _bool(v):
    return str(v).lower() in ("1", "true", "yes", "on")


def create_parser():
    p = argparse.ArgumentParser(prog="llama-hip", description="Llama 3 generation on one MI355X",
                                formatter_class=argparse.ArgumentDefaultsHelpFormatter)
    p.add_argument("--model", "-m", dest="model_path", required=True, help="model folder")
    p.add_argument("--interactive", "--chat", "-i", dest="interactive", action="store_true", help="run in chat mode")
    p.add_argument("--instruct", dest="interactive", action="store_false",
                   help="run in instruct (once) mode, the default mode")
    p.add_argument("--prompt", "-p", help="input prompt (needs tokenizer.json in the model folder)")
    p.add_argument("--system-prompt", "-sp", dest="system_prompt", help="(optional) system prompt")
    p.add_argument("--suffix", help="suffix for fill-in-the-middle requests (no Llama model takes one)")
    p.add_argument("--prompt-ids", help="input prompt as comma-separated token ids, fed as they are")
    p.add_argument("--temperature", "--temp", type=float, default=0.1, help="sampling temperature, 0 = greedy")
    p.add_argument("--top-p", type=float, default=0.95, help="top-p (nucleus) mass in [0,1]")
    p.add_argument("--seed", "-s", type=int, default=None, help="random seed (default: the clock)")
    p.add_argument("--max-tokens", "-n", type=int, default=DEFAULT_MAX_TOKENS,
                   help="bound on positions, prompt and generated together; < 0 = the context length")
    p.add_argument("--stream", type=_bool, default=True, help="print tokens as they are generated")
    p.add_argument("--echo", type=_bool, default=False, help="print all tokens to stderr")
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--write-random-model", metavar="CONFIG_JSON",
                   help="write a random-weights model folder into --model from this config.json and exit")
    p.set_defaults(interactive=False)
    return p


def _print_metrics(engine):
    m = engine.metrics
    total = m.prompt_tokens + m.generated_tokens
    secs = m.prefill_seconds + m.decode_seconds
    # the reference's line (J/auxiliary/LastRunMetrics.java:27-31), then prompt and decode apart
    print(f"\nachieved tok/s: {total / secs if secs else 0:.2f}. Tokens: {total}, seconds: {secs:.2f}", file=sys.stderr)
    print(f"prefill: {m.prompt_tokens} tokens in {m.prefill_seconds:.3f} s; decode: {m.decode_steps} steps in "
          f"{m.decode_seconds:.3f} s", file=sys.stderr)


def run_interactive(engine, chat, tokenizer, sampler, args, lines=None, out=None):
    """The reference's chat loop (J/model/Model.java:76-181): the dialogue's tokens stay in one
    slot of the cache, every turn feeds what has come since. ``lines`` (an iterable of user
    lines; default: standard input) and ``out`` are for tests.

    The reference counts the stop token of an answer as held although it never ran it through the
    model (Model.java:145-146); here it is fed at the head of the next turn, so the cache holds
    every token of the dialogue."""
    out = out or sys.stdout
    conversation = [chat.begin_of_text]
    if args.system_prompt is not None:
        conversation += chat.encode_message(Message(SYSTEM, args.system_prompt))
    lines = iter(lines) if lines is not None else iter(sys.stdin.readline, "")
    with engine.create_new_state() as state:
        while True:
            print("> ", end="", file=out, flush=True)
            line = next(lines, None)
            if line is None:
                break
            user_text = line.rstrip("\n")
            if user_text in ("quit", "exit"):
                break
            conversation += chat.encode_message(Message(USER, user_text))
            conversation += chat.encode_header(Message(ASSISTANT, ""))

            def show(tok):
                if args.stream and tok not in chat.stop_tokens:
                    print(tokenizer.decode([tok]), end="", file=out, flush=True)

            start = state.length
            response = engine.generate_tokens(conversation[start:], chat.stop_tokens, args.max_tokens, sampler,
                                              echo=args.echo, on_token_generated=show, state=state,
                                              start_position=start)
            conversation += response          # the stop token stays in the history, not in what is shown
            stopped = bool(response) and response[-1] in chat.stop_tokens
            if stopped:
                response = response[:-1]
            if not args.stream:
                print(tokenizer.decode(response), file=out)
            if not stopped:
                print("\nThe context is full. A larger --max-tokens gives the conversation more room.", file=sys.stderr)
                break
            print(file=out)
            _print_metrics(engine)
    return conversation


def main(argv=None):
    args = create_parser().parse_args(argv)
    if not 0 <= args.temperature:
        print("error: --temperature takes 0 (greedy) or a positive number", file=sys.stderr)
        return 2
    if not 0 <= args.top_p <= 1:
        print("error: --top-p takes a mass between 0 and 1", file=sys.stderr)
        return 2
    seed = args.seed if args.seed is not None else time.time_ns()
    import gpullama3_java_amd as g
    if args.write_random_model:
        with open(args.write_random_model) as f:
            cfg = g.config_from_dict(json.load(f))
        g.write_random_model(args.model_path, cfg, seed)
        print(f"wrote {args.model_path}")
        return 0
    tokenizer = chat = None
    tok_path = os.path.join(args.model_path, "tokenizer.json")
    if os.path.isfile(tok_path):
        tokenizer = HFTokenizer(tok_path)
        # the dialogue's token protocol belongs to the architecture: its configuration class says which
        make_format = getattr(g.load_config(args.model_path), "chat_format", None)
        chat = make_format(tokenizer) if make_format is not None else None
    if args.suffix is not None:
        print("note: --suffix is for fill-in-the-middle models; a Llama model takes none, it is ignored", file=sys.stderr)
    if args.interactive:
        if chat is None:
            print(f"error: chat mode needs {tok_path} and an architecture with a chat format", file=sys.stderr)
            return 2
        prompt = None
    elif args.prompt_ids:
        prompt = [int(t) for t in args.prompt_ids.replace(" ", "").split(",") if t]
        stop_ids = None
    elif args.prompt is not None:
        if chat is None:
            print(f"error: a text prompt needs {tok_path} and an architecture with a chat format; "
                  "--prompt-ids takes token ids as they are", file=sys.stderr)
            return 2
        dialog = [Message(SYSTEM, args.system_prompt)] if args.system_prompt is not None else []
        prompt = chat.encode_dialog_prompt(True, dialog + [Message(USER, args.prompt)])
        stop_ids = chat.stop_tokens
    else:
        print("error: give --prompt (or --prompt-ids), or --interactive for a dialogue", file=sys.stderr)
        return 2
    engine = g.load_model(args.model_path, context_length=args.max_tokens, dtype=args.dtype,
                          max_tokens=None)
    sampler = g.select_sampler(engine.spec.vocab_size, args.temperature, args.top_p, seed)
    if args.interactive:
        run_interactive(engine, chat, tokenizer, sampler, args)
        return 0
    stop_ids = stop_ids if stop_ids is not None else engine.config.stop_ids
    if args.echo:
        print(" ".join(str(t) for t in prompt), end=" ", file=sys.stderr, flush=True)

    def show(tok):
        if args.stream and tok not in stop_ids:       # special tokens are not shown (LlamaTokenizer.java:55-57)
            text = tokenizer.decode([tok]) if tokenizer is not None else f"{tok} "
            print(text, end="", flush=True)

    out = engine.generate_tokens(prompt, stop_ids, args.max_tokens, sampler, echo=args.echo,
                                 on_token_generated=show)
    if out and out[-1] in stop_ids:
        out = out[:-1]                                # callers drop the stop token (J/model/Model.java:242-244)
    if not args.stream:
        print(tokenizer.decode(out) if tokenizer is not None else " ".join(str(t) for t in out))
    else:
        print()
    _print_metrics(engine)
    return 0


if __name__ == "__main__":
    sys.exit(main())

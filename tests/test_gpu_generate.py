"""Greedy generation through the entry point and the command line, against the plain
implementation; sampled generation against the replayed logits."""
import os
import subprocess
import sys

import numpy as np
import pytest

import plain_llama as P
from gpu_helpers import DTYPES, model, plain_logits, rand_tokens
from gpullama3_java_amd.sampling import uniform

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def plain_greedy(name, prompt, n, tie=0.0):
    seq, out = list(prompt), []
    for _ in range(n):
        out.append(int(np.argmax(plain_logits(name, seq)[-1])))
        seq.append(out[-1])
    return out


def agrees_with_plain(name, prompt, got, dtype):
    """Token by token: the plain argmax, or a logit within rounding of it (then follow the engine)."""
    seq = list(prompt)
    for t in got:
        l = plain_logits(name, seq)[-1]
        best = int(np.argmax(l))
        margin = {"float32": 1e-5, "bfloat16": 2e-2}[dtype] * np.abs(l).max()
        assert t == best or l[best] - l[t] <= margin, (seq, t, best, l[best] - l[t])
        seq.append(t)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_entry_point_greedy(name, dtype):
    import gpullama3_java_amd as g
    folder, cfgd, _ = model(name)
    eng = g.load_model(folder, context_length=-1, dtype=dtype)
    sampler = g.select_sampler(cfgd["vocab_size"], 0.0, 0.95, seed=1)
    prompt = rand_tokens(name, 3, 11)
    seen = []
    out = eng.generate_tokens(prompt, stop_tokens=set(), max_tokens=11 + 8 - 1, sampler=sampler,
                              on_token_generated=seen.append)
    assert len(out) == 8 and seen == out                  # max_tokens bounds the position, as in the reference
    agrees_with_plain(name, prompt, out, dtype)
    if dtype == "float32":
        assert out == plain_greedy(name, prompt, 8)
    # a stop token ends the sequence and is kept
    out2 = eng.generate_tokens(prompt, stop_tokens={out[2]}, max_tokens=-1, sampler=sampler)
    assert out2 == out[:out.index(out[2]) + 1]
    assert eng.cache.slots.live == set()
    assert eng.metrics.prompt_tokens == 11 and eng.metrics.generated_tokens == len(out2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_batched_generation_equals_each_alone(dtype):
    from gpullama3_java_amd.engine import Engine
    name = "B"
    folder, _, _ = model(name)
    eng = Engine.from_folder(folder, dtype=dtype, max_tokens=1024, n_slots=2)     # 5 requests over 2 slots
    prompts = [rand_tokens(name, 20 + i, n) for i, n in enumerate((3, 17, 40, 9, 64))]
    res = eng.generate(prompts, max_new_tokens=12)
    for p, r in zip(prompts, res):
        assert len(r.tokens) == 12 and r.finish_reason == "length"
        agrees_with_plain(name, p, r.tokens, dtype)
    alone = [eng.generate([p], max_new_tokens=12)[0].tokens for p in prompts]
    if dtype == "float32":
        assert alone == [r.tokens for r in res]
    stop = res[1].tokens[4]
    res2 = eng.generate(prompts, max_new_tokens=12, stop_ids=[stop])
    for r, r0 in zip(res2, res):
        cut = r0.tokens.index(stop) + 1 if stop in r0.tokens else 12
        assert r.tokens == r0.tokens[:cut] and r.finish_reason == ("stop" if stop in r0.tokens else "length")


def test_sampled_generation_follows_the_logits():
    """With temperature and top-p every drawn token is what the plain rule draws from the
    plain logits of the sequence so far, with the draw's own uniform number."""
    from gpullama3_java_amd.engine import Engine
    name = "B"
    folder, _, _ = model(name)
    eng = Engine.from_folder(folder, dtype="float32", max_tokens=1024)
    prompts = [rand_tokens(name, 30 + i, n) for i, n in enumerate((3, 17, 40))]
    res = eng.generate(prompts, max_new_tokens=12, temperature=0.8, top_p=0.95, seed=9)
    for i, (p, r) in enumerate(zip(prompts, res)):
        seq = list(p)
        for k, t in enumerate(r.tokens):
            u = uniform(9, i, len(p) + k)
            l = plain_logits(name, seq)[-1]
            want = P.sample(l, 0.8, 0.95, u)
            if t != want:                                   # allowed only at an edge of the running sum
                assert any(P.sample(l, 0.8, 0.95, min(max(u + d, 0), 0.9999999)) == t for d in (-2e-5, 2e-5)), (i, k)
            seq.append(t)
    again = eng.generate(prompts[::-1], max_new_tokens=12, temperature=0.8, top_p=0.95, seed=9)
    assert [r.tokens for r in again] != [r.tokens for r in res[::-1]]      # the request index is part of the draw
    same = eng.generate(prompts, max_new_tokens=12, temperature=0.8, top_p=0.95, seed=9)
    assert [r.tokens for r in same] == [r.tokens for r in res]


def test_command_line(tmp_path):
    folder, cfgd, _ = model("A")
    prompt = rand_tokens("A", 4, 6)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "llama-hip"), "--model", folder, "--prompt-ids",
           ",".join(map(str, prompt)), "--temperature=0", "-n", "13", "--stream", "false", "--dtype", "float32"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [int(t) for t in r.stdout.split()] == plain_greedy("A", prompt, 8)
    assert "achieved tok/s" in r.stderr and "Tokens: 14" in r.stderr
    bad = subprocess.run(cmd[:4] + ["--top-p", "1.5", "--prompt-ids", "1"], capture_output=True, text=True, timeout=300)
    assert bad.returncode != 0 and "--top-p takes a mass between 0 and 1" in bad.stderr
    noprompt = subprocess.run(cmd[:4] + ["--prompt", "hello"], capture_output=True, text=True, timeout=300)
    assert noprompt.returncode != 0 and "tokenizer.json" in noprompt.stderr


def test_a_sequence_goes_on_in_its_state():
    """Two calls on one state give what one sequence gives: the second call's tokens follow those
    that the slot holds (the reference's chat loop, J/model/Model.java:136), the slot is kept
    between the calls and given back at the end."""
    import gpullama3_java_amd as g
    from gpullama3_java_amd.sampling import SamplingParams
    folder, _, _ = model("B")
    eng = g.load_model(folder, dtype="float32", max_tokens=1024)
    free = eng.slots_free()
    first = rand_tokens("B", 60, 9)
    with eng.create_new_state() as state:
        assert eng.slots_free() == free - 1 and state.length == 0
        a = eng.generate_tokens(first, (), len(first) + 5, SamplingParams(), state=state, start_position=0)
        assert a == plain_greedy("B", first, len(a)) and len(a) == 6
        assert state.length == len(first) + len(a) - 1            # the token sampled last has not been fed
        with pytest.raises(ValueError, match="start there"):
            eng.generate_tokens([1], (), 64, SamplingParams(), state=state, start_position=3)
        more = rand_tokens("B", 61, 4)
        seq = first + a + more
        start = state.length
        b = eng.generate_tokens(seq[start:], (), len(seq) + 4, SamplingParams(), state=state, start_position=start)
        assert b == plain_greedy("B", seq, len(b)) and len(b) == 5
        assert eng.slots_free() == free - 1
    assert eng.slots_free() == free
    with pytest.raises(ValueError, match="closed"):
        eng.generate_tokens([1], (), 64, SamplingParams(), state=state, start_position=0)


def test_chat_loop_keeps_the_dialogue_in_the_cache():
    """The interactive loop with a toy tokenizer over a tiny model: every turn's answer is the plain
    implementation's greedy continuation of the whole dialogue so far. A random model never emits the
    end-of-turn id on purpose, so the toy format stops at a class of ordinary ids as well, chosen so
    that both turns end by it."""
    import argparse
    import io
    import gpullama3_java_amd as g
    from gpullama3_java_amd import cli
    from gpullama3_java_amd.chat import ASSISTANT, USER, SYSTEM, LlamaChatFormat, Message
    from test_chat_format import ToyTokenizer
    folder, cfgd, _ = model("B")       # its head is its own: a tied one repeats the last token
    limit = 100
    lines = ["hi", "more", "quit", "never read"]
    tok = ToyTokenizer()
    chosen = None
    for modulus, rest in ((2, 0), (2, 1), (3, 0), (3, 1), (3, 2)):
        chat = LlamaChatFormat(tok)
        chat.stop_tokens = frozenset(chat.stop_tokens) | frozenset(t for t in range(200) if t % modulus == rest)
        conv = [chat.begin_of_text] + chat.encode_message(Message(SYSTEM, "s"))
        ok = True
        for line in lines[:2]:
            conv += chat.encode_message(Message(USER, line)) + chat.encode_header(Message(ASSISTANT, ""))
            gen = plain_greedy("B", conv, 12)
            ends = [k for k, t in enumerate(gen) if t in chat.stop_tokens]
            if not ends or ends[0] == 0:          # an answer of at least one token before the stop
                ok = False
                break
            conv += gen[:ends[0] + 1]
        if ok and len(conv) < limit:
            chosen = (chat, conv)
            break
    assert chosen is not None, "no class of ids ends both turns; change the lines"
    chat, want = chosen
    eng = g.load_model(folder, dtype="float32", max_tokens=1024)
    args = argparse.Namespace(system_prompt="s", stream=True, echo=False, max_tokens=limit)
    out = io.StringIO()
    free = eng.slots_free()
    got = cli.run_interactive(eng, chat, tok, g.select_sampler(cfgd["vocab_size"], 0.0, 1.0, 1), args, lines=lines, out=out)
    assert got == want
    assert out.getvalue().count("> ") == 3 and eng.slots_free() == free


def test_command_line_with_a_text_prompt(tmp_path):
    """--prompt through a tokenizer.json in the model folder: the tokens that the model sees are the
    chat format's (begin of text, system and user message, the assistant's header), the answer is the
    plain implementation's greedy continuation, printed as text."""
    import shutil
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers
    from gpullama3_java_amd.chat import SYSTEM, USER, HFTokenizer, LlamaChatFormat, Message
    folder, cfgd, _ = model("B")
    mine = str(tmp_path / "model")
    shutil.copytree(folder, mine)
    alphabet = sorted(pre_tokenizers.ByteLevel.alphabet())
    tok = Tokenizer(models.BPE(vocab={ch: i for i, ch in enumerate(alphabet)}, merges=[]))
    tok.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False)
    tok.decoder = decoders.ByteLevel()
    tok.add_special_tokens(["<|begin_of_text|>", "<|start_header_id|>", "<|end_header_id|>", "<|eot_id|>",
                            "<|end_of_text|>"])
    assert tok.get_vocab_size() <= cfgd["vocab_size"]
    tok.save(os.path.join(mine, "tokenizer.json"))
    hf = HFTokenizer(os.path.join(mine, "tokenizer.json"))
    chat = LlamaChatFormat(hf)
    assert hf.encode("hi") == [alphabet.index("h"), alphabet.index("i")] and hf.decode(hf.encode("a b")) == "a b"
    prompt = chat.encode_dialog_prompt(True, [Message(SYSTEM, "s"), Message(USER, "hi there")])
    limit = len(prompt) + 10
    want = plain_greedy("B", prompt, 11)
    if any(t in chat.stop_tokens for t in want):
        want = want[:[t in chat.stop_tokens for t in want].index(True)]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "llama-hip"), "-m", mine, "-p", " hi there ", "-sp", "s",
           "--temperature=0", "-n", str(limit), "--stream", "false", "--dtype", "float32"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert r.stdout.rstrip("\n") == hf.decode(want).rstrip("\n")
    assert f"Tokens: {len(prompt) + len(want)}" in r.stderr
    chatty = subprocess.run(cmd[:4] + ["--chat", "--temperature=0", "-n", str(limit), "--dtype", "float32"],
                            input="hi there\nquit\n", capture_output=True, text=True, timeout=300)
    assert chatty.returncode == 0, chatty.stderr
    assert chatty.stdout.startswith("> ")

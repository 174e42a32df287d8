"""bin/trace_run, driven as a user drives it: the same requests whole, with the last 32
tokens one by one, and in batches of unequal lengths over a cache that holds one batch,
compared with the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from gpu_helpers import CONFIGS, DTYPES, first_bad_row, model, plain_logits, rand_tokens

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class Replay:
    def __init__(self, folder, dtype, out, max_tokens):
        self.out = str(out)
        self.p = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder,
                                   "--dtype", dtype, "--out", self.out, "--max-tokens", str(max_tokens)],
                                  stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
        self.n = 0

    def step(self, entries, end=()):
        """entries: [(id, tokens, want)] -> logits [wanted, vocab] or None."""
        rec = {"step": self.n, "entries": [{"id": i, "tokens": t, "want": w} for i, t, w in entries], "end": list(end)}
        self.p.stdin.write(json.dumps(rec) + "\n")
        self.p.stdin.flush()
        line = self.p.stdout.readline().strip()
        assert line == f"done {self.n}", f"trace_run said {line!r} (exit {self.p.poll()})"
        path = os.path.join(self.out, f"{self.n}.f32")
        self.n += 1
        if not any(w for _, _, w in entries):
            assert not os.path.exists(path)
            return None
        return np.fromfile(path, dtype="<f4")

    def close(self):
        self.p.stdin.close()
        assert self.p.wait(timeout=60) == 0


@pytest.mark.parametrize("name", ["A", "B", "D"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_replay_cuts(name, dtype, tmp_path):
    folder, cfgd, _ = model(name)
    V = cfgd["vocab_size"]
    limit = cfgd["max_position_embeddings"]
    lens = [n for n in (5, 40, 100, 129, 190) if n <= limit]
    reqs = {f"r{i}": rand_tokens(name, 40 + i, n) for i, n in enumerate(lens)}
    ref = {k: plain_logits(name, t) for k, t in reqs.items()}
    # the cache holds 3 requests of up to 192 tokens: batches of three must reuse what earlier ones held
    rp = Replay(folder, dtype, tmp_path, max_tokens=3 * 192)

    def check(got, want, what):
        got = got.reshape(-1, V)
        bad = first_bad_row(got, want, dtype)
        assert bad is None, f"{name} {dtype} {what}: first wrong row {bad} of {len(want)}"

    for k, t in reqs.items():                                   # 1. alone and whole
        check(rp.step([(k, t, list(range(len(t))))], end=[k]), ref[k], f"{k} whole")
    for k, t in reqs.items():                                   # 2. the last 32 one by one
        if len(t) <= 32:
            continue
        cut = len(t) - 32
        rows = [rp.step([(k, t[:cut], list(range(cut)))]).reshape(-1, V)]
        for j in range(cut, len(t)):
            rows.append(rp.step([(k, [t[j]], [0])], end=[k] if j == len(t) - 1 else []).reshape(-1, V))
        check(np.concatenate(rows), ref[k], f"{k} last 32 one by one")
    keys = list(reqs)                                           # 3. unequal batches, shorter requests end earlier
    for b in range(0, len(keys), 3):
        batch = keys[b:b + 3]
        prompt = {k: max(1, len(reqs[k]) // 3) for k in batch}
        got = {k: [] for k in batch}
        out = rp.step([(k, reqs[k][:prompt[k]], list(range(prompt[k]))) for k in batch]).reshape(-1, V)
        o = 0
        for k in batch:
            got[k].append(out[o:o + prompt[k]]); o += prompt[k]
        pos = dict(prompt)
        live = [k for k in batch if pos[k] < len(reqs[k])]
        done_after_prompt = [k for k in batch if k not in live]
        if done_after_prompt:
            rp.step([], end=done_after_prompt)
        while live:
            ending = [k for k in live if pos[k] + 1 == len(reqs[k])]
            out = rp.step([(k, [reqs[k][pos[k]]], [0]) for k in live], end=ending).reshape(-1, V)
            for r, k in enumerate(live):
                got[k].append(out[r:r + 1]); pos[k] += 1
            live = [k for k in live if k not in ending]
        for k in batch:
            check(np.concatenate(got[k]), ref[k], f"{k} in batch {batch}")
    assert rp.step([("x", [1, 2, 3], [])]) is None              # nothing wanted: no file
    rp.close()


def test_replay_refuses_more_than_the_cache_holds(tmp_path):
    folder, _, _ = model("A")
    rp = Replay(folder, "float32", tmp_path, max_tokens=64)
    rp.step([("a", [1] * 60, [59])])
    rp.p.stdin.write(json.dumps({"step": 1, "entries": [{"id": "b", "tokens": [1], "want": [0]}], "end": []}) + "\n")
    rp.p.stdin.close()
    assert rp.p.wait(timeout=60) != 0                           # a second request needs a second page

"""Shared by the GPU tests: model folders in a temporary place, the plain logits of a
token list, and the tolerances (fixed here once; a failing test is a fault, not a
reason to touch them)."""
from __future__ import annotations

import atexit
import functools
import os
import shutil
import tempfile

import numpy as np
from safetensors.torch import load_file

import gpullama3_java_amd as g
import plain_llama as P
from tiny import TINY_A, TINY_B, TINY_C, TINY_D

CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}
DTYPES = ["float32", "bfloat16"]

# Largest allowed |engine - plain| as a fraction of the largest |plain| logit of the
# compared rows. float32: sums of a few hundred products in another order. bfloat16:
# activations are rounded to 8 bits of mantissa (2^-9 relative) at every part's
# output; measured over the three configurations with matrices N(0, 0.05) the largest
# difference is 5e-3 to 7e-3 of the logit scale on every row alike (it grows with the
# weights' scale: 1.8e-2 at N(0, 0.1)), so 2e-2 leaves a factor of three. Faults that
# move a logit by less (one key among hundreds under near-uniform weights) are caught
# by the float32 runs of the same tests, whose bound is a thousand times tighter, and
# by the kernel tests whose inputs make one score stand out.
TOL = {"float32": 2e-5, "bfloat16": 2e-2}

_root = tempfile.mkdtemp(prefix="gl3-tests-")
atexit.register(shutil.rmtree, _root, ignore_errors=True)


@functools.lru_cache(maxsize=None)
def model(name, seed=1, std=0.05, norm_std=0.1):
    """(folder, config dict, float32 numpy weights as the folder stores them)."""
    cfgd = CONFIGS[name]
    folder = os.path.join(_root, f"{name}-{seed}-{std}-{norm_std}")
    g.write_random_model(folder, g.config_from_dict(cfgd), seed, std=std, norm_std=norm_std)
    W = {k: v.float().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return folder, cfgd, W


@functools.lru_cache(maxsize=None)
def _plain(name, toks, seed, std, norm_std):
    _, cfgd, W = model(name, seed, std, norm_std)
    return P.forward(cfgd, W, list(toks))


def plain_logits(name, toks, seed=1, std=0.05, norm_std=0.1):
    return _plain(name, tuple(int(t) for t in toks), seed, std, norm_std)


def close(got, ref, dtype, what=""):
    got, ref = np.asarray(got), np.asarray(ref)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    scale = max(float(np.abs(ref).max()), 1e-3)
    err = float(np.abs(got - ref).max())
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    assert err <= TOL[dtype] * scale, f"{what}: max |diff| {err:.3e} > {TOL[dtype]} * {scale:.3f}"
    return err / scale


def first_bad_row(got, ref, dtype):
    scale = max(float(np.abs(ref).max()), 1e-3)
    bad = np.flatnonzero(np.abs(got - ref).max(axis=-1) > TOL[dtype] * scale)
    return int(bad[0]) if len(bad) else None


def rand_tokens(name, seed, n):
    rng = np.random.default_rng([seed, 31])
    return rng.integers(0, CONFIGS[name]["vocab_size"], size=n).tolist()

"""Small Melizen configurations for the tests, and model folders made from them (never the product's own)."""
from __future__ import annotations

import atexit
import functools
import json
import os
import shutil
import tempfile

import numpy as np

import plain_melizen as P


def _attn(heads, kv, dim, vdim, window, scale, mlp):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def _delta(heads, kv, dim, vdim, conv, mlp):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def _mlp(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


# a loop from the first layer on, three passes; values larger than keys, grouped heads, windows that are no
# multiple of anything, a layer without a feed-forward, key sizes that no tile divides
LOOPED = {
    "architecture": "Melizen", "vocab": 300, "width": 96, "max_positions": 600, "norm": {"eps": 1e-5},
    "layers": [_delta(4, 2, 32, 48, 3, _mlp(160, 1.5)), _attn(6, 2, 32, 48, 40, 0.2, _mlp(128, 3.0)),
               _delta(2, 2, 24, 16, 2, None), _attn(4, 4, 16, 16, 17, 0.25, _mlp(72, 0.75))],
    "loop": {"start": 0, "stop": 2, "times": 3},
}
# no loop; an attention that sees every earlier key; one head; values smaller than keys; a convolution of one tap
# and one of five; another eps; an odd width and vocabulary
STRAIGHT = {
    "architecture": "Melizen", "vocab": 203, "width": 72, "max_positions": 400, "norm": {"eps": 1e-6},
    "layers": [_attn(3, 1, 48, 32, None, 0.15, _mlp(100, 2.5)), _delta(1, 1, 40, 20, 1, _mlp(64, 1.0)),
               _delta(6, 3, 16, 32, 5, None), _attn(2, 2, 64, 16, 70, 0.11, None)],
}
# the loop in the middle and at the end of the list
LOOP_AT_END = {
    "architecture": "Melizen", "vocab": 128, "width": 64, "max_positions": 320, "norm": {"eps": 1e-5},
    # (the first attention's heads are no multiples of the cache's tiles: they are padded when the weights load)
    "layers": [_attn(2, 1, 24, 40, 9, 0.3, _mlp(96, 2.0)), _delta(2, 1, 16, 16, 4, _mlp(96, 2.0)),
               _attn(4, 2, 32, 16, 33, 0.2, None)],
    "loop": {"start": 1, "stop": 3, "times": 2},
}
# head sizes that the matrix-core attention kernels are built for (values of the keys' size), two kv heads for
# eight query heads, widths in whole tiles: what a bfloat16 engine runs on its fast paths
TILED = {
    "architecture": "Melizen", "vocab": 640, "width": 128, "max_positions": 512, "norm": {"eps": 1e-5},
    "layers": [_attn(8, 2, 64, 64, 100, 0.125, _mlp(256, 4.0)), _delta(4, 2, 64, 64, 3, _mlp(256, 1.5)),
               _attn(4, 4, 32, 32, None, 0.18, _mlp(128, 1.0)), _attn(2, 1, 96, 96, 70, 0.1, None),
               _attn(2, 2, 128, 128, 130, 0.09, _mlp(128, 3.0))],
    "loop": {"start": 1, "stop": 2, "times": 2},
}
CONFIGS = {"looped": LOOPED, "straight": STRAIGHT, "loop_at_end": LOOP_AT_END, "tiled": TILED}

_root = tempfile.mkdtemp(prefix="melizen-tests-")
atexit.register(shutil.rmtree, _root, ignore_errors=True)


@functools.lru_cache(maxsize=None)
def model(name, seed=3):
    """(folder, config dict, float32 numpy weights as the folder stores them in bfloat16)."""
    import torch
    from safetensors.torch import save_file
    cfg = CONFIGS[name]
    W = P.make_weights(cfg, seed)
    folder = os.path.join(_root, f"{name}-{seed}")
    os.makedirs(folder, exist_ok=True)
    save_file({k: torch.tensor(v).to(torch.bfloat16).contiguous() for k, v in W.items()},
              os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    return folder, cfg, W


def tokens(name, seed, n):
    rng = np.random.default_rng([seed, 5])
    return rng.integers(0, CONFIGS[name]["vocab"], size=n).tolist()


# Largest allowed difference of a row of logits (its mean taken off, root mean square over the vocabulary) as a
# fraction of the root mean square of the plain logits. float32: sums in another order. bfloat16: activations
# between the parts are rounded to 8 bits of mantissa; measured 4e-3 to 9e-3 with these models.
TOL = {"float32": 3e-5, "bfloat16": 3e-2}


def row_errors(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all()
    d = got - ref
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / np.sqrt(((ref - ref.mean(-1, keepdims=True)) ** 2).mean())


def close(got, ref, dtype, what=""):
    e = row_errors(got, ref)
    bad = np.flatnonzero(e > TOL[dtype])
    assert not len(bad), f"{what}: row {int(bad[0])} is the first of {len(bad)} over {TOL[dtype]}: {e[bad[0]]:.3e}"
    return float(e.max())

"""Small Nodupel configurations for the tests, and model folders made from them (never the product's own)."""
from __future__ import annotations

import atexit
import functools
import json
import os
import shutil
import tempfile

import numpy as np

import plain_nodupel as P


def _left(heads, kv, dim, vdim, scale, base, dims, factor=None, size=None, keep=None):
    rot = {"base": base, "dims": dims}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    c = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if size is not None:
        c["mask"] = {"size": size} if keep is None else {"size": size, "keep_first": keep}
    return c


def _parallel(left, heads, dim, ff):
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": heads, "dim": dim}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _mingru(width, ff):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _emb(scale, buckets, mul_prev, mul_cur):
    return {"scale": scale, "bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}


# a loop from the first layer on, three passes; a rotation over a part of the head, values larger than keys, two kv
# heads, a window and kept keys that are multiples of nothing, heads that no tile divides, a layer without feed-forward
LOOPED = {
    "architecture": "Nodupel", "vocab": 300, "width": 96, "norm": {"eps": 1e-5}, "residual_mult": 0.7,
    "logit_softcap": 20.0, "embedding": _emb(9.5, 211, 7, 13),
    "layers": [_parallel(_left(4, 2, 32, 48, 0.2, 10000.0, 16, 4.0, 37, 5), 3, 24, 160),
               _mingru(72, 128),
               _parallel(_left(2, 2, 24, 40, 0.25, 500.0, 24, None, 17, 0), 2, 40, None)],
    "loop": {"start": 0, "stop": 2, "times": 3},
}
# no loop and no soft cap; a minGRU first; an attention that sees every earlier key; one kv head for six heads;
# a residual factor of one; multipliers so large that their products need 64 bits; a width that no tile divides
STRAIGHT = {
    "architecture": "Nodupel", "vocab": 203, "width": 100, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
    "embedding": _emb(1.0, 97, 2000000011, 1999999973),
    "layers": [_mingru(40, 100), _parallel(_left(6, 1, 16, 32, 0.3, 20000.0, 8, 1.5), 1, 64, 64),
               _mingru(100, None), _parallel(_left(3, 3, 48, 16, 0.12, 10000.0, 48, None, 70, 3), 4, 16, 96)],
}
# the loop at the end of the list, one pass only (its mixture still runs); more kept keys than a page holds, kept
# keys beyond the window's size
LOOP_AT_END = {
    "architecture": "Nodupel", "vocab": 128, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.45,
    "logit_softcap": 8.0, "embedding": _emb(4.0, 64, 5, 3),
    "layers": [_parallel(_left(2, 1, 32, 32, 0.2, 1000.0, 32, 8.0, 9, 70), 2, 32, 96), _mingru(50, 96),
               _parallel(_left(4, 2, 16, 16, 0.3, 10000.0, 4, None, 33, 12), 3, 20, None)],
    "loop": {"start": 1, "stop": 3, "times": 1},
}
# head sizes that the matrix-core attention kernels are built for, widths in whole tiles: what a bfloat16 engine
# runs on its fast paths
TILED = {
    "architecture": "Nodupel", "vocab": 640, "width": 128, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
    "logit_softcap": 30.0, "embedding": _emb(11.3, 1021, 31, 17),
    "layers": [_parallel(_left(8, 2, 64, 64, 0.125, 10000.0, 64, 2.0, 100, 4), 2, 64, 256), _mingru(128, 256),
               _parallel(_left(4, 4, 32, 32, 0.18, 10000.0, 32, None), 4, 32, 128),
               _parallel(_left(2, 1, 128, 128, 0.09, 50000.0, 64, None, 130, 40), 1, 128, None)],
    "loop": {"start": 1, "stop": 3, "times": 2},
}
CONFIGS = {"looped": LOOPED, "straight": STRAIGHT, "loop_at_end": LOOP_AT_END, "tiled": TILED}
RANKS = {"looped": 8, "straight": 5, "loop_at_end": 12, "tiled": 32}

_root = tempfile.mkdtemp(prefix="nodupel-tests-")
atexit.register(shutil.rmtree, _root, ignore_errors=True)


@functools.lru_cache(maxsize=None)
def model(name, seed=3):
    """(folder, config dict, float32 numpy weights as the folder stores them in bfloat16)."""
    import torch
    from safetensors.torch import save_file
    cfg = CONFIGS[name]
    W = P.make_weights(cfg, seed, RANKS[name])
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
# between the parts are rounded to 8 bits of mantissa.
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

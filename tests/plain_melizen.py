"""A plain, slow implementation of the Melizen decoder in numpy float64, one function per mechanism, written
from the design's equations and sharing nothing with the package: what the GPU tests compare the engine with.

Notation: T tokens of ONE sequence, positions 0 .. T-1; W maps a stored tensor name to a float array; linear
weights are [out, in].
"""
from __future__ import annotations

import zlib

import numpy as np


# ----------------------------------------------------------------- mechanisms
def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = np.asarray(x, np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def norm_around_zero(x, w, eps):
    """RMS norm whose stored weight lies around zero: the factor is 1 + w."""
    return rms_unit(x, eps) * (1.0 + np.asarray(w, np.float64))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def head_slopes(n_heads):
    return np.array([2.0 ** (-8.0 * (h + 1) / n_heads) for h in range(n_heads)])


def sink_attention(q, k, v, scale, window=None, slopes=None, sink=0.0, first=0):
    """q [T, H, D], k [S, G, D], v [S, G, Dv]; query t sits at position first + t, key j at position j.
    score = q.k * scale - slope_h * (i - j) over the keys with 0 <= i - j < window; the weights are
    exp(s_j) / (exp(sink) + sum exp(s)), sink None: an ordinary softmax. Returns [T, H, Dv]."""
    q, k, v = (np.asarray(a, np.float64) for a in (q, k, v))
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        i = first + t
        lo = 0 if window is None else max(0, i - window + 1)
        js = np.arange(lo, i + 1)
        for h in range(H):
            g = h // (H // G)
            s = (k[js, g] @ q[t, h]) * scale
            if slopes is not None:
                s = s - slopes[h] * (i - js)
            m = max(s.max(), sink) if sink is not None else s.max()
            e = np.exp(s - m)
            den = e.sum() + (np.exp(sink - m) if sink is not None else 0.0)
            out[t, h] = (e / den) @ v[js, g]
    return out


def short_conv_silu(x, w, held=None):
    """x [T, C] over time, w [C, taps] (the last column is the current token's). ``held``: the taps - 1 inputs
    before x[0] ([taps - 1, C], oldest first; None: zeros). Returns (silu(conv) [T, C], the new held inputs)."""
    x, w = np.asarray(x, np.float64), np.asarray(w, np.float64)
    T, C = x.shape
    taps = w.shape[1]
    held = np.zeros((taps - 1, C)) if held is None else np.asarray(held, np.float64)
    xp = np.concatenate([held, x], 0)
    y = np.zeros((T, C))
    for r in range(taps):
        y += xp[r:r + T] * w[:, r]
    return silu(y), xp[len(xp) - (taps - 1):] if taps > 1 else np.zeros((0, C))


def unit_length(x, eps=1e-6):
    x = np.asarray(x, np.float64)
    return x / np.sqrt((x * x).sum(-1, keepdims=True) + eps)


def delta_rule(q, k, v, g, beta, S=None):
    """One head: q, k [T, D], v [T, Dv], g, beta [T]. S [D, Dv] (None: zeros). Returns (o [T, Dv], S)."""
    q, k, v = (np.asarray(a, np.float64) for a in (q, k, v))
    T, D = q.shape
    S = np.zeros((D, v.shape[1])) if S is None else np.array(S, np.float64)
    o = np.zeros((T, v.shape[1]))
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o, S


def bounded_gated_ffn(h, w_gate, w_up, w_down, limit):
    g = np.minimum(h @ w_gate.T, limit)
    u = np.clip(h @ w_up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w_down.T


# ----------------------------------------------------------------- mixers
def attention_mixer(h, W, m, p, first=0, past=None):
    """``past``: (k, v) of the positions before ``first`` or None. Returns (output [T, width], (k, v) so far)."""
    T = len(h)
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).reshape(T, H, D)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).reshape(T, G, D)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).reshape(T, G, Dv)
    if past is not None:
        k, v = np.concatenate([past[0], k]), np.concatenate([past[1], v])
    window = m["mask"]["size"] if m.get("mask") else None
    o = sink_attention(q, k, v, m["scale"], window, head_slopes(H), 0.0, first)
    return o.reshape(T, H * Dv) @ W[p + "o"].T, (k, v)


def delta_mixer(h, W, m, p, eps, state=None):
    """``state``: (S [H, D, Dv], held inputs of q, k, v) or None. Returns (output, state)."""
    T = len(h)
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    S, held = state if state is not None else (np.zeros((H, D, Dv)), [None, None, None])
    q, hq = short_conv_silu(h @ W[p + "q"].T, W[p + "q.conv"], held[0])
    k, hk = short_conv_silu(h @ W[p + "k"].T, W[p + "k.conv"], held[1])
    v, hv = short_conv_silu(h @ W[p + "v"].T, W[p + "v.conv"], held[2])
    q = unit_length(q.reshape(T, G, D)) * D ** -0.5
    k = unit_length(k.reshape(T, G, D))
    v = v.reshape(T, H, Dv)
    beta = sigmoid(h @ W[p + "b"].T)
    g = np.exp(-np.exp(W[p + "A_log"]) * softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    gate = (h @ W[p + "g"].T).reshape(T, H, Dv)
    o = np.zeros((T, H, Dv))
    S = np.array(S)
    for hh in range(H):
        c = hh // (H // G)
        o[:, hh], S[hh] = delta_rule(q[:, c], k[:, c], v[:, hh], g[:, hh], beta[:, hh], S[hh])
    y = rms_unit(o, eps) * W[p + "norm"] * silu(gate)
    return y.reshape(T, H * Dv) @ W[p + "o"].T, (S, [hq, hk, hv])


# ----------------------------------------------------------------- the decoder
def run_order(cfg):
    """[(layer, pass number if the entry starts a pass of the loop else None)]."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp or lp["stop"] <= lp["start"]:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(lp["start"])]
    for t in range(lp["times"]):
        order += [(i, t if i == lp["start"] else None) for i in range(lp["start"], lp["stop"])]
    return order + [(i, None) for i in range(lp["stop"], n)]


class Sequence:
    """A sequence that is fed in pieces: keeps every run-order entry's keys and values or state."""

    def __init__(self, cfg, W):
        self.cfg, self.W = cfg, {k: np.asarray(v, np.float64) for k, v in W.items()}
        self.order = run_order(cfg)
        self.kept = [None] * len(self.order)
        self.n = 0

    def feed(self, tokens, trace=None):
        """Logits [len(tokens), vocab] of the next tokens."""
        cfg, W = self.cfg, self.W
        eps = cfg["norm"]["eps"]
        T = len(tokens)
        x = W["embed"][np.asarray(tokens)] + W["pos"][self.n:self.n + T]
        embedded = x.copy()
        for e, (i, t) in enumerate(self.order):
            if t is not None:
                if t > 0:
                    x = x + embedded
                x = x + W["loop.step"][t]
            lay, p = cfg["layers"][i], f"l{i}."
            h = norm_around_zero(x, W[p + "norm1"], eps)
            if lay["type"] == "attention":
                y, self.kept[e] = attention_mixer(h, W, lay["mixer"], p + "mix.", self.n, self.kept[e])
            else:
                y, self.kept[e] = delta_mixer(h, W, lay["mixer"], p + "mix.", eps, self.kept[e])
            y = y * W[p + "ls1"]
            if lay.get("mlp") is not None:
                f = lay["mlp"]
                y = y + bounded_gated_ffn(h, W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"], f["limit"]) * W[p + "ls2"]
            x = x + y
            if trace is not None:
                trace.append(x.copy())
        self.n += T
        return norm_around_zero(x, W["final.norm"], eps) @ W["head"].T


def forward(cfg, W, tokens):
    return Sequence(cfg, W).feed(tokens)


# ----------------------------------------------------------------- test models
def tensor_shapes(cfg):
    d, V = cfg["width"], cfg["vocab"]
    shapes = {"embed": (V, d), "pos": (cfg["max_positions"], d), "final.norm": (d,), "head": (V, d)}
    lp = cfg.get("loop")
    if lp and lp["stop"] > lp["start"]:
        shapes["loop.step"] = (lp["times"], d)
    for i, lay in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        shapes.update({p + "norm1": (d,), p + "ls1": (d,)})
        if lay["type"] == "attention":
            shapes.update({p + "mix.q": (H * D, d), p + "mix.q.b": (H * D,), p + "mix.k": (G * D, d), p + "mix.k.b": (G * D,),
                           p + "mix.v": (G * Dv, d), p + "mix.v.b": (G * Dv,), p + "mix.o": (d, H * Dv)})
        else:
            c = m["conv"]
            shapes.update({p + "mix.q": (G * D, d), p + "mix.q.conv": (G * D, c), p + "mix.k": (G * D, d),
                           p + "mix.k.conv": (G * D, c), p + "mix.v": (H * Dv, d), p + "mix.v.conv": (H * Dv, c),
                           p + "mix.b": (H, d), p + "mix.a": (H, d), p + "mix.A_log": (H,), p + "mix.dt_bias": (H,),
                           p + "mix.norm": (Dv,), p + "mix.g": (H * Dv, d), p + "mix.o": (d, H * Dv)})
        if lay.get("mlp") is not None:
            F = lay["mlp"]["ff"]
            shapes.update({p + "mlp.gate": (F, d), p + "mlp.up": (F, d), p + "mlp.down": (d, F), p + "ls2": (d,)})
    return shapes


def make_weights(cfg, seed):
    """float32 weights that bfloat16 holds exactly, sized so that every mechanism moves the logits: matrices
    N(0, 1/sqrt(fan-in)), norm weights around zero, layer scales around one, a wide spread of decays."""
    import torch
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        rng = np.random.default_rng([seed, zlib.crc32(name.encode())])
        last = name.split(".")[-1]
        if last in ("norm1",) or name == "final.norm":
            a = 0.2 * rng.standard_normal(shape)
        elif last in ("ls1", "ls2"):
            a = 0.6 + 0.2 * rng.standard_normal(shape)
        elif last == "norm":
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif last == "b" and len(shape) == 1:
            a = 0.3 * rng.standard_normal(shape)
        elif last == "A_log":
            a = rng.uniform(-4.0, 0.5, shape)
        elif last == "dt_bias":
            a = rng.uniform(-3.0, 1.0, shape)
        elif last == "conv":
            a = 0.6 * rng.standard_normal(shape)
        elif name in ("embed", "pos", "loop.step"):
            a = 0.7 * rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) * (1.5 / np.sqrt(shape[-1]))
        out[name] = torch.tensor(a, dtype=torch.float32).to(torch.bfloat16).float().numpy()
    return out

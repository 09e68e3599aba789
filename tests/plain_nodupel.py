"""A plain, slow implementation of the Nodupel decoder in numpy float64, one function per mechanism, written from
the design's equations and sharing nothing with the package: what the GPU tests compare the engine with.

Notation: T tokens of ONE sequence; W maps a stored tensor name to a float array; linear weights are [out, in].
A ``Sequence`` keeps what the design carries from token to token (the previous token, every pass's keys and values,
the recurrent states) and can be fed in pieces.
"""
from __future__ import annotations

import math

import numpy as np


# ----------------------------------------------------------------- small functions
def rms_unit(x, eps):
    x = np.asarray(x, np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * np.asarray(w, np.float64)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def linear(x, w, b=None):
    y = np.asarray(x, np.float64) @ np.asarray(w, np.float64).T
    return y if b is None else y + np.asarray(b, np.float64)


# ----------------------------------------------------------------- embedding
def bigram_rows(tokens, before, buckets, mul_prev, mul_cur):
    """The row of the pair table for every token: hashed from (previous token, token); a sequence's first token
    (``before`` None and index 0) takes the row behind the hashed ones."""
    rows, prev = [], before
    for t in tokens:
        rows.append(buckets if prev is None else (int(prev) * mul_prev + int(t) * mul_cur) % buckets)
        prev = t
    return rows


def embed(tokens, before, table, pair_table, scale, buckets, mul_prev, mul_cur):
    table, pair_table = np.asarray(table, np.float64), np.asarray(pair_table, np.float64)
    return table[list(tokens)] * scale + pair_table[bigram_rows(tokens, before, buckets, mul_prev, mul_cur)]


# ----------------------------------------------------------------- rotation
def turn_halves(x, positions, base, dims, divide=1.0, back=False):
    """x [T, heads, D]: the first ``dims`` elements of every head as pairs (i, i + dims/2); pair i of the token at
    position p turns by p * base^(-2i/dims) / divide (``back``: by minus that). The rest passes."""
    x = np.array(x, np.float64)
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)]) / divide
    a = np.asarray(positions, np.float64)[:, None] * f[None, :]
    if back:
        a = -a
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    u, v = x[..., :half].copy(), x[..., half:dims].copy()
    x[..., :half] = u * c - v * s
    x[..., half:dims] = v * c + u * s
    return x


# ----------------------------------------------------------------- attention
def visible(i, j, size, keep_first):
    return j <= i and (size is None or i - j < size or j < keep_first)


def masked_attention(q, k, v, scale, size, keep_first, first=0):
    """q [T, H, D] at positions first .. first + T - 1; k [S, G, D], v [S, G, Dv] at positions 0 .. S - 1.
    Ordinary softmax over the keys that ``visible`` allows. Returns [T, H, Dv]."""
    q, k, v = (np.asarray(a, np.float64) for a in (q, k, v))
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        i = first + t
        js = np.array([j for j in range(i + 1) if visible(i, j, size, keep_first)])
        for h in range(H):
            g = h // (H // G)
            s = (k[js, g] @ q[t, h]) * scale
            e = np.exp(s - s.max())
            out[t, h] = (e / e.sum()) @ v[js, g]
    return out


# ----------------------------------------------------------------- recurrences
def mingru_scan(z, u, state):
    """z, u [T, C]; state [C]. Candidate: u + 1/2 where u >= 0, sigmoid(u) below. Returns (S_t [T, C], last S)."""
    z, u = np.asarray(z, np.float64), np.asarray(u, np.float64)
    cand = np.where(u >= 0, u + 0.5, sigmoid(u))
    out = np.zeros_like(z)
    S = np.array(state, np.float64)
    for t in range(z.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        out[t] = S
    return out, S


def shifted(h, before):
    """The previous token's row for every token: ``before`` ([d] or None: zeros) in front of h[:-1]."""
    h = np.asarray(h, np.float64)
    first = np.zeros((1, h.shape[1])) if before is None else np.asarray(before, np.float64)[None]
    return np.concatenate([first, h[:-1]], 0)


def decayed_outer_scan(r, k, v, w, bonus, state):
    """r, k, w [T, H, D], v [T, H, Dv], bonus [H, D], state [H, D, Dv]. Per head
    o_t = (S + diag(bonus) k_t v_t^T)^T r_t, then S <- diag(w_t) S + k_t v_t^T. Returns (o [T, H, Dv], S)."""
    r, k, v, w = (np.asarray(a, np.float64) for a in (r, k, v, w))
    bonus = np.asarray(bonus, np.float64)
    S = np.array(state, np.float64)
    T, H, _ = r.shape
    out = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        for h in range(H):
            kv = np.outer(k[t, h], v[t, h])
            out[t, h] = (S[h] + bonus[h][:, None] * kv).T @ r[t, h]
            S[h] = w[t, h][:, None] * S[h] + kv
    return out, S


# ----------------------------------------------------------------- the model
class Sequence:
    def __init__(self, cfg, W):
        self.cfg, self.W = cfg, {k: np.asarray(v, np.float64) for k, v in W.items()}
        self.n = 0
        self.prev_token = None
        self.order = self.run_order(cfg)
        self.state = [dict() for _ in self.order]        # one per entry of the run order
        self.layers = []                                  # the residual rows after every layer run, per call of feed

    @staticmethod
    def run_order(cfg):
        """[(layer, starts a pass)]"""
        n = len(cfg["layers"])
        loop = cfg.get("loop")
        if not loop:
            return [(i, False) for i in range(n)]
        out = [(i, False) for i in range(loop["start"])]
        for _ in range(loop["times"]):
            out += [(i, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
        return out + [(i, False) for i in range(loop["stop"], n)]

    def feed(self, tokens):
        """Logits [T, vocab] of the tokens, which follow what the sequence has seen."""
        cfg, W = self.cfg, self.W
        T = len(tokens)
        pos = np.arange(self.n, self.n + T)
        e = cfg["embedding"]
        b = e["bigram"]
        x0 = embed(tokens, self.prev_token, W["embed"], W["bigram"], e["scale"], b["buckets"], b["mul_prev"], b["mul_cur"])
        x = x0.copy()
        m, eps = cfg["residual_mult"], cfg["norm"]["eps"]
        self.layers = []
        for entry, (i, starts) in enumerate(self.order):
            lay, p, st = cfg["layers"][i], f"l{i}.", self.state[entry]
            if starts:
                x = linear(np.concatenate([x, x0], 1), W["loop.in"])
            h = rms_norm(x, W[p + "norm1"], eps)
            if lay["type"] == "mingru":
                y = self.mingru(lay["mixer"], p + "mix.", h, st)
            elif lay["type"] == "parallel":
                y = self.parallel(lay["mixer"], p + "mix.", h, st, pos, eps)
            else:
                raise ValueError(lay["type"])
            x = x + m * y
            if lay.get("mlp") is not None:
                h = rms_norm(x, W[p + "norm2"], eps)
                x = x + m * linear(gelu_tanh(linear(h, W[p + "mlp.gate"])) * linear(h, W[p + "mlp.up"]), W[p + "mlp.down"])
            self.layers.append(x.copy())
        self.n += T
        self.prev_token = tokens[-1]
        cap = cfg.get("logit_softcap")
        logits = linear(rms_norm(x, W["final.norm"], eps), W["head"])
        return logits if cap is None else cap * np.tanh(logits / cap)

    def mingru(self, mc, p, h, st):
        W = self.W
        z = sigmoid(linear(h, W[p + "z"], W[p + "z.b"]))
        u = linear(h, W[p + "x"], W[p + "x.b"])
        S, st["S"] = mingru_scan(z, u, st.get("S", np.zeros(mc["width"])))
        return linear(S * silu(linear(h, W[p + "g"])), W[p + "o"])

    def left(self, c, p, h, st, pos):
        W = self.W
        T = h.shape[0]
        H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        rot = c["rot"]
        divide = (rot.get("scaling") or {}).get("factor", 1.0)
        q = turn_halves(linear(h, W[p + "q"]).reshape(T, H, D), pos, rot["base"], rot["dims"], divide)
        k = turn_halves(linear(h, W[p + "k"]).reshape(T, G, D), pos, rot["base"], rot["dims"], divide)
        v = turn_halves(linear(h, W[p + "v"]).reshape(T, G, Dv), pos, rot["base"], Dv)
        st["k"] = k if "k" not in st else np.concatenate([st["k"], k], 0)
        st["v"] = v if "v" not in st else np.concatenate([st["v"], v], 0)
        mask = c.get("mask") or {}
        o = masked_attention(q, st["k"], st["v"], c["scale"], mask.get("size"), mask.get("keep_first", 0), first=int(pos[0]))
        o = turn_halves(o, pos, rot["base"], Dv, back=True)
        o = o * sigmoid(linear(h, W[p + "g"]))[:, :, None]
        return linear(o.reshape(T, H * Dv), W[p + "o"])

    def right(self, c, p, h, st, eps):
        W = self.W
        T, d = h.shape
        H, D = c["heads"], c["dim"]
        before = shifted(h, st.get("h"))
        st["h"] = h[-1].copy()
        mix = {s: h + (before - h) * W[p + "mu." + s] for s in "rkvgw"}
        r, k, v = (linear(mix[s], W[p + s]).reshape(T, H, D) for s in "rkv")
        gate = silu(linear(mix["g"], W[p + "g"]))
        w = np.exp(-np.exp(linear(np.tanh(linear(mix["w"], W[p + "w1"])), W[p + "w2"]) + W[p + "w0"])).reshape(T, H, D)
        o, st["S"] = decayed_outer_scan(r, k, v, w, W[p + "u"], st.get("S", np.zeros((H, D, D))))
        o = rms_unit(o, eps).reshape(T, H * D) * W[p + "norm"] * gate
        return linear(o, W[p + "o"])

    def parallel(self, mc, p, h, st, pos, eps):
        W = self.W
        a = self.left(mc["left"], p + "left.", h, st.setdefault("left", {}), pos)
        b = self.right(mc["right"], p + "right.", h, st.setdefault("right", {}), eps)
        return 0.5 * (rms_norm(a, W[p + "left.out"], eps) + rms_norm(b, W[p + "right.out"], eps))


def forward(cfg, W, tokens):
    """Logits [T, vocab] of one sequence from its start."""
    return Sequence(cfg, W).feed(list(tokens))


# ----------------------------------------------------------------- weights for tests
def tensor_shapes(cfg, decay_rank=8):
    d = cfg["width"]
    out = {"embed": (cfg["vocab"], d), "bigram": (cfg["embedding"]["bigram"]["buckets"] + 1, d),
           "final.norm": (d,), "head": (cfg["vocab"], d)}
    if cfg.get("loop"):
        out["loop.in"] = (d, 2 * d)
    for i, lay in enumerate(cfg["layers"]):
        p = f"l{i}."
        out[p + "norm1"] = (d,)
        m = lay["mixer"]
        if lay["type"] == "mingru":
            w = m["width"]
            out.update({p + "mix.z": (w, d), p + "mix.z.b": (w,), p + "mix.x": (w, d), p + "mix.x.b": (w,),
                        p + "mix.g": (w, d), p + "mix.o": (d, w)})
        else:
            L, R = m["left"], m["right"]
            q = p + "mix.left."
            out.update({q + "q": (L["heads"] * L["dim"], d), q + "k": (L["kv_heads"] * L["dim"], d),
                        q + "v": (L["kv_heads"] * L["vdim"], d), q + "g": (L["heads"], d),
                        q + "o": (d, L["heads"] * L["vdim"]), q + "out": (d,)})
            r = p + "mix.right."
            hd = R["heads"] * R["dim"]
            out.update({r + "mu." + s: (d,) for s in "rkvgw"})
            out.update({r + s: (hd, d) for s in "rkvg"})
            out.update({r + "w1": (decay_rank, d), r + "w2": (hd, decay_rank), r + "w0": (hd,), r + "u": (R["heads"], R["dim"]),
                        r + "norm": (hd,), r + "o": (d, hd), r + "out": (d,)})
        if lay.get("mlp") is not None:
            ff = lay["mlp"]["ff"]
            out.update({p + "norm2": (d,), p + "mlp.gate": (ff, d), p + "mlp.up": (ff, d), p + "mlp.down": (d, ff)})
    return out


def make_weights(cfg, seed, decay_rank=8):
    """float32 weights that bfloat16 holds exactly, sized so that every mechanism moves the logits: matrices
    N(0, 1.5/sqrt(fan-in)), norm weights around one, blends anywhere between the two tokens, a wide spread of decays."""
    import zlib
    import torch
    out = {}
    for name, shape in tensor_shapes(cfg, decay_rank).items():
        rng = np.random.default_rng([seed, zlib.crc32(name.encode())])
        last = name.split(".")[-1]
        if last in ("norm1", "norm2", "norm", "out"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif ".mu." in name:
            a = rng.uniform(0.0, 1.0, shape)
        elif last == "w0":
            a = rng.uniform(-5.0, 0.5, shape)
        elif last == "u" and ".right." in name:
            a = 0.5 * rng.standard_normal(shape)
        elif last == "b" and len(shape) == 1:
            a = 0.5 * rng.standard_normal(shape)
        elif name == "embed":
            a = rng.standard_normal(shape) / cfg["embedding"]["scale"]
        elif name == "bigram":
            a = 0.7 * rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) * (1.5 / np.sqrt(shape[-1]))
        out[name] = torch.tensor(a, dtype=torch.float32).to(torch.bfloat16).float().numpy()
    return out

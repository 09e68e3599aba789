"""Typed configuration of the Nodupel decoder, read from its config.json.

Nodupel is a pre-norm decoder whose layers differ in kind. The embedding row (times a constant) is joined by a row
of a second table that a hash of (previous token, token) picks. A layer is ``x += m * mixer(norm1(x))`` and, where it
has a feed-forward, ``x += m * ffn(norm2(x))`` with one constant ``m`` for the model. Its mixer is either a minGRU (a
gated recurrence per channel) or two mixers side by side whose normalised outputs are averaged: an attention with a
rotation of queries and keys over a part of the head, values that are rotated by their own position and turned back
at the output, a window that also keeps a sequence's first positions, and a gate per head; and an RWKV-style time
mixing, a decayed matrix per head. A run of the layers, ``loop.start .. loop.stop - 1``, is entered ``loop.times``
times in a row with the same weights and cache and state of its own per pass; every pass begins with
``x <- W_in [x; x0]``, x0 being the embedding's output. The feed-forward is gated with the tanh form of gelu; the
logits pass a soft cap.

config.json: ``architecture`` "Nodupel", ``vocab``, ``width``, ``norm.eps``, ``residual_mult``, ``logit_softcap``,
``embedding`` (``scale``, ``bigram``: ``buckets``, ``mul_prev``, ``mul_cur``), ``loop`` (``start``, ``stop``, ``times``) and
``layers``, a list of ``{"type": "mingru" | "parallel", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}`` with
  mingru:   ``width``;
  parallel: ``left`` (``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``rot``: ``base``, ``dims``, ``scaling.factor``;
            ``mask``: ``size``, ``keep_first``) and ``right`` (``heads``, ``dim``).
The folder names no longest sequence: ``max_positions`` (ours, optional) bounds it, else ``DEFAULT_MAX_POSITIONS``.
Tensor names: ``embed``, ``bigram``, ``loop.in``, ``final.norm``, ``head``, and per layer i ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Optional

from .registry import ConfigError, _as_ids, register_architecture
from .specs import (AttentionSpec, BlockSpec, GatedFeedForwardSpec, LinearRopeScaling, MinGRUSpec, ModelSpec, NormSpec,
                    PairEmbedding, Remix, RotarySpec, Run, SideBySideSpec, TimeMixSpec)

# what the design fixes
ACTIVATION = "gelu_tanh"          # the feed-forward's gate
SIDE_WEIGHT = 0.5                 # the two sides' normalised outputs are averaged
ROTARY_PAIRING = "half"           # element i of the rotated part turns with element i + dims / 2
DEFAULT_MAX_POSITIONS = 1 << 17   # a folder sets no bound on a sequence's length; the engine's caches need one


def _int(d, key, where, least=1):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, int) or v < least:
        raise ConfigError(f"config.json: {where}'{key}' must be an integer of at least {least}, found {v!r}")
    return v


def _positive(d, key, where):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not v > 0:
        raise ConfigError(f"config.json: {where}'{key}' must be a positive number, found {v!r}")
    return float(v)


def _number(d, key, where):
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {where}'{key}' must be a number, found {v!r}")
    return float(v)


@dataclass(frozen=True)
class NodupelLeft:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int
    rot_factor: Optional[float] = None      # linear scaling: frequencies divided by this
    window: Optional[int] = None            # mask.size; None: every earlier key
    keep_first: int = 0


@dataclass(frozen=True)
class NodupelRight:
    heads: int
    dim: int


@dataclass(frozen=True)
class NodupelLayer:
    type: str                               # "mingru" | "parallel"
    width: Optional[int] = None             # mingru
    left: Optional[NodupelLeft] = None
    right: Optional[NodupelRight] = None
    ff: Optional[int] = None                # None: no feed-forward


@dataclass(frozen=True)
class NodupelConfiguration:
    vocab_size: int
    width: int
    norm_eps: float
    residual_mult: float
    embedding_scale: float
    bigram_buckets: int
    bigram_mul_prev: int
    bigram_mul_cur: int
    layers: tuple
    logit_softcap: Optional[float] = None
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    has_loop: bool = False                  # whether config.json carries 'loop' (its W_in then runs, also for one pass)
    decay_rank: tuple = ()                  # per layer: the inner size of a time mixing's decay projection (from the weights)
    max_positions: int = DEFAULT_MAX_POSITIONS
    context_length: Optional[int] = None
    stop_ids: tuple = ()
    architecture: str = "Nodupel"

    @property
    def max_position_embeddings(self):
        return self.max_positions if self.context_length is None else min(self.context_length, self.max_positions)

    @property
    def hidden_size(self):
        return self.width

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d):
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, lay in enumerate(layers_in):
            where = f"layers[{i}]: "
            if not isinstance(lay, dict) or lay.get("type") not in ("mingru", "parallel"):
                raise ConfigError(f"config.json: {where}'type' must be 'mingru' or 'parallel'")
            m = lay.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"config.json: {where}'mixer' must be an object")
            kw = dict(type=lay["type"])
            if lay["type"] == "mingru":
                kw["width"] = _int(m, "width", where)
            else:
                kw["left"] = cls._left(m.get("left"), where + "left: ")
                r = m.get("right")
                kw["right"] = NodupelRight(heads=_int(r, "heads", where + "right: "), dim=_int(r, "dim", where + "right: "))
            mlp = lay.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json: {where}'mlp' must be null or an object of kind 'dense'")
                kw["ff"] = _int(mlp, "ff", where + "mlp: ")
            layers.append(NodupelLayer(**kw))
        loop = d.get("loop")
        start = stop = 0
        times = 1
        if loop is not None:
            if not isinstance(loop, dict):
                raise ConfigError("config.json: 'loop' must be null or an object with 'start', 'stop' and 'times'")
            start, stop, times = _int(loop, "start", "loop: ", 0), _int(loop, "stop", "loop: ", 0), _int(loop, "times", "loop: ")
            if not start <= stop <= len(layers):
                raise ConfigError(f"config.json: loop: layers {start} .. {stop} of {len(layers)}")
        emb = d.get("embedding")
        if not isinstance(emb, dict) or not isinstance(emb.get("bigram"), dict):
            raise ConfigError("config.json: 'embedding' must be an object with 'scale' and 'bigram'")
        big = emb["bigram"]
        cap = d.get("logit_softcap")
        ranks = d.get("decay_rank")
        return cls(vocab_size=_int(d, "vocab", ""), width=_int(d, "width", ""),
                   norm_eps=_positive(d.get("norm"), "eps", "norm: "), residual_mult=_number(d, "residual_mult", ""),
                   embedding_scale=_number(emb, "scale", "embedding: "),
                   bigram_buckets=_int(big, "buckets", "embedding: bigram: "),
                   bigram_mul_prev=_int(big, "mul_prev", "embedding: bigram: ", 0),
                   bigram_mul_cur=_int(big, "mul_cur", "embedding: bigram: ", 0), layers=tuple(layers),
                   logit_softcap=None if cap is None else _positive(d, "logit_softcap", ""),
                   loop_start=start, loop_stop=stop, loop_times=times, has_loop=loop is not None and stop > start,
                   decay_rank=tuple(ranks) if isinstance(ranks, (list, tuple)) else (),
                   max_positions=_int(d, "max_positions", "") if d.get("max_positions") is not None else DEFAULT_MAX_POSITIONS,
                   stop_ids=_as_ids(d.get("eos_token_id")))

    @staticmethod
    def _left(c, where):
        if not isinstance(c, dict):
            raise ConfigError(f"config.json: {where}must be an object")
        heads, kv = _int(c, "heads", where), _int(c, "kv_heads", where)
        if heads % kv:
            raise ConfigError(f"config.json: {where}{heads} heads are not a multiple of {kv} kv_heads")
        dim, vdim = _int(c, "dim", where), _int(c, "vdim", where)
        rot = c.get("rot")
        dims = _int(rot, "dims", where + "rot: ", 2)
        if dims % 2 or dims > dim or vdim % 2:
            raise ConfigError(f"config.json: {where}rot: {dims} rotated elements of heads of {dim}, values of {vdim}: "
                              "pairs need even sizes, and the rotated part lies inside the head")
        scaling = rot.get("scaling")
        factor = None if scaling is None else _positive(scaling, "factor", where + "rot: scaling: ")
        mask = c.get("mask")
        window, keep = None, 0
        if mask is not None:
            window = _int(mask, "size", where + "mask: ")
            keep = _int(mask, "keep_first", where + "mask: ", 0) if mask.get("keep_first") is not None else 0
        return NodupelLeft(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=_positive(c, "scale", where),
                           rot_base=_positive(rot, "base", where + "rot: "), rot_dims=dims, rot_factor=factor,
                           window=window, keep_first=keep)

    def to_dict(self):
        layers = []
        for lay in self.layers:
            if lay.type == "mingru":
                m = {"width": lay.width}
            else:
                L = lay.left
                rot = {"base": L.rot_base, "dims": L.rot_dims}
                if L.rot_factor is not None:
                    rot["scaling"] = {"factor": L.rot_factor}
                left = {"heads": L.heads, "kv_heads": L.kv_heads, "dim": L.dim, "vdim": L.vdim, "scale": L.scale, "rot": rot}
                if L.window is not None:
                    left["mask"] = {"size": L.window, "keep_first": L.keep_first}
                m = {"left": left, "right": {"heads": lay.right.heads, "dim": lay.right.dim}}
            layers.append({"type": lay.type, "mixer": m, "mlp": None if lay.ff is None else {"kind": "dense", "ff": lay.ff}})
        d = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.width,
             "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
             "embedding": {"scale": self.embedding_scale,
                           "bigram": {"buckets": self.bigram_buckets, "mul_prev": self.bigram_mul_prev,
                                      "mul_cur": self.bigram_mul_cur}},
             "layers": layers}
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        if self.has_loop:
            d["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.decay_rank:
            d["decay_rank"] = list(self.decay_rank)
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        if self.stop_ids:
            d["eos_token_id"] = list(self.stop_ids)
        return d

    # ------------------------------------------------------------------ what the engine asks
    def chat_format(self, tokenizer):
        raise ConfigError("a Nodupel model folder brings no chat format: give the prompt as token ids")

    def with_stop_ids(self, ids):
        return replace(self, stop_ids=tuple(ids))

    def with_context_length(self, n):
        if n is None or n < 0:
            return self
        return replace(self, context_length=min(n, self.max_positions))

    def with_tensor_shapes(self, shapes):
        """Sizes that only the weights give: the inner size of every time mixing's decay projection
        (``l<i>.mix.right.w1`` is [rank, width]). ``shapes``: stored name -> shape."""
        ranks = []
        for i, lay in enumerate(self.layers):
            s = shapes.get(f"l{i}.mix.right.w1") if lay.type == "parallel" else None
            ranks.append(int(s[0]) if s is not None and len(s) == 2 else 0)
        return replace(self, decay_rank=tuple(ranks)) if any(ranks) else self

    def _rank(self, i):
        r = self.decay_rank[i] if i < len(self.decay_rank) else 0
        return r if r else max(8, self.width // 16)

    def run_order(self):
        """Layers before the loop once, the loop's layers ``times`` times in a row, the rest once; the first entry of
        every pass is preceded by the mixture with the embedding's output."""
        if not self.has_loop:
            return tuple(Run(layer=i) for i in range(len(self.layers)))
        runs = [Run(layer=i) for i in range(self.loop_start)]
        for _ in range(self.loop_times):
            for i in range(self.loop_start, self.loop_stop):
                runs.append(Run(layer=i, before=Remix("loop.in") if i == self.loop_start else None))
        runs += [Run(layer=i) for i in range(self.loop_stop, len(self.layers))]
        return tuple(runs)

    def model_spec(self):
        d, eps, m = self.width, self.norm_eps, self.residual_mult
        n_max = self.max_position_embeddings
        blocks = []
        for i, lay in enumerate(self.layers):
            p = f"l{i}."
            if lay.type == "mingru":
                mixer = MinGRUSpec(hidden=d, width=lay.width, out_mult=m,
                                   names={k: p + "mix." + v for k, v in {
                                       "z": "z", "z_bias": "z.b", "x": "x", "x_bias": "x.b", "g": "g", "o": "o"}.items()})
            else:
                L, R = lay.left, lay.right
                q = p + "mix.left."
                left = AttentionSpec(
                    hidden=d, n_heads=L.heads, n_kv_heads=L.kv_heads, head_dim=L.dim, v_head_dim=L.vdim,
                    position=RotarySpec(head_dim=L.rot_dims, theta=L.rot_base, pairing=ROTARY_PAIRING, max_positions=n_max,
                                        scaling=None if L.rot_factor is None else LinearRopeScaling(L.rot_factor)),
                    value_position=RotarySpec(head_dim=L.vdim, theta=L.rot_base, pairing=ROTARY_PAIRING, max_positions=n_max),
                    window=L.window, keep_first=L.keep_first if L.window is not None else 0, scale=L.scale,
                    names={"q": q + "q", "k": q + "k", "v": q + "v", "o": q + "o", "head_gate": q + "g"})
                r = p + "mix.right."
                right = TimeMixSpec(
                    hidden=d, n_heads=R.heads, head_dim=R.dim, decay_rank=self._rank(i), norm_eps=eps,
                    names={k: r + v for k, v in {
                        "mu_r": "mu.r", "mu_k": "mu.k", "mu_v": "mu.v", "mu_g": "mu.g", "mu_w": "mu.w", "r": "r", "k": "k",
                        "v": "v", "g": "g", "w1": "w1", "w2": "w2", "w0": "w0", "u": "u", "norm": "norm", "o": "o"}.items()})
                mixer = SideBySideSpec(hidden=d, left=left, right=right, norm_eps=eps, weight=SIDE_WEIGHT, out_mult=m,
                                       names={"left_norm": q + "out", "right_norm": r + "out"})
            ffn = ffn_norm = None
            if lay.ff is not None:
                ffn = GatedFeedForwardSpec(hidden=d, intermediate=lay.ff, activation=ACTIVATION, out_mult=m,
                                           names={"gate": p + "mlp.gate", "up": p + "mlp.up", "down": p + "mlp.down"})
                ffn_norm = NormSpec(dim=d, eps=eps, names={"weight": p + "norm2"})
            blocks.append(BlockSpec(kind="prenorm", mixer_norm=NormSpec(dim=d, eps=eps, names={"weight": p + "norm1"}),
                                    mixer=mixer, ffn_norm=ffn_norm, ffn=ffn))
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden=d, layers=tuple(blocks),
            run_order=self.run_order(), final_norm=NormSpec(dim=d, eps=eps, names={"weight": "final.norm"}),
            max_positions=n_max, tie_embeddings=False, embedding_name="embed", head_name="head",
            stop_ids=self.stop_ids, embedding_scale=self.embedding_scale, logit_softcap=self.logit_softcap,
            pair_embedding=PairEmbedding("bigram", self.bigram_buckets, self.bigram_mul_prev, self.bigram_mul_cur),
            # (a folder may hold the second norm of a layer without a feed-forward, and the mixture of a loop over no
            # layer: nothing reads them)
            unused_tensor_names=tuple(f"l{i}.norm2" for i, lay in enumerate(self.layers) if lay.ff is None)
            + (() if self.has_loop else ("loop.in",)))


register_architecture("Nodupel", NodupelConfiguration)

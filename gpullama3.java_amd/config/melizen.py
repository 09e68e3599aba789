"""Typed configuration of the Melizen decoder, read from its config.json.

Melizen is a decoder with learned absolute positions and a list of layers that differ in kind: each layer has
ONE norm whose output feeds both its mixer and its feed-forward (their outputs, each times a learned vector per
channel, are added to the residual stream together), and its mixer is either a windowed attention without a
rotation (a bias that grows with the distance, and a softmax with a sink) or a gated delta rule. A run of the
layers, ``loop.start .. loop.stop - 1``, is entered ``loop.times`` times in a row with the same weights; every pass
has cache and state of its own, is preceded by a learned vector per pass added to the residual rows, and every pass
but the first also by the embedding's output added back.

config.json: ``architecture`` "Melizen", ``vocab``, ``width``, ``max_positions``, ``norm.eps``, ``loop``
(``start``, ``stop``, ``times``; absent: every layer once) and ``layers``, a list of
``{"type": "attention" | "delta", "mixer": {...}, "mlp": {"kind": "dense", "ff", "limit"} | null}`` with
  attention: ``heads``, ``kv_heads``, ``dim`` (queries and keys), ``vdim`` (values), ``scale``, ``mask.size`` (the window);
  delta:     ``heads`` (value heads), ``kv_heads`` (query/key heads), ``dim``, ``vdim``, ``conv`` (taps).
Tensor names: ``embed``, ``pos``, ``loop.step``, ``final.norm``, ``head``, and per layer i ``l<i>.norm1``, ``l<i>.ls1``,
``l<i>.ls2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Optional

from .registry import ConfigError, _as_ids, register_architecture
from .specs import (AttentionSpec, BlockSpec, DistanceBias, GatedDeltaSpec, GatedFeedForwardSpec, Inject, ModelSpec,
                    NormSpec, Run)

# what the design fixes
SLOPE_BASE, SLOPE_EXPONENT = 2.0, 8.0     # slope of head h of H: 2 ** (-8 (h + 1) / H)
SINK_SCORE = 0.0                          # one is added to the softmax's denominator: a key with the score 0
UNIT_EPS = 1e-6                           # inside the root when q and k of the delta rule are scaled to unit length
GATE_SLOPE_ACTIVATION = "quick_gelu"      # the feed-forward's gate: z * sigmoid(1.702 z)
UP_SHIFT = 1.0                            # ... times (up + 1)


def _int(d, key, where, least=1):
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, int) or v < least:
        raise ConfigError(f"config.json: {where}'{key}' must be an integer of at least {least}, found {v!r}")
    return v


def _positive(d, key, where):
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not v > 0:
        raise ConfigError(f"config.json: {where}'{key}' must be a positive number, found {v!r}")
    return float(v)


@dataclass(frozen=True)
class MelizenFeedForward:
    ff: int
    limit: float


@dataclass(frozen=True)
class MelizenLayer:
    type: str                     # "attention" | "delta"
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: Optional[float] = None     # attention
    window: Optional[int] = None      # attention: mask.size
    conv: Optional[int] = None        # delta: taps
    mlp: Optional[MelizenFeedForward] = None


@dataclass(frozen=True)
class MelizenConfiguration:
    vocab_size: int
    width: int
    max_positions: int            # rows of the learned position table
    norm_eps: float
    layers: tuple
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    context_length: Optional[int] = None     # a shorter context for a run; None: max_positions
    stop_ids: tuple = ()
    architecture: str = "Melizen"

    @property
    def max_position_embeddings(self):
        return self.max_positions if self.context_length is None else min(self.context_length, self.max_positions)

    @property
    def hidden_size(self):
        return self.width

    @classmethod
    def from_dict(cls, d):
        width = _int(d, "width", "")
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        norm = d.get("norm")
        if not isinstance(norm, dict):
            raise ConfigError("config.json: 'norm' must be an object with 'eps'")
        layers = []
        for i, lay in enumerate(layers_in):
            where = f"layers[{i}]: "
            if not isinstance(lay, dict) or lay.get("type") not in ("attention", "delta"):
                raise ConfigError(f"config.json: {where}'type' must be 'attention' or 'delta'")
            m = lay.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"config.json: {where}'mixer' must be an object")
            heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
            if heads % kv:
                raise ConfigError(f"config.json: {where}{heads} heads are not a multiple of {kv} kv_heads")
            kw = dict(type=lay["type"], heads=heads, kv_heads=kv, dim=_int(m, "dim", where), vdim=_int(m, "vdim", where))
            if lay["type"] == "attention":
                kw["scale"] = _positive(m, "scale", where)
                mask = m.get("mask")
                if mask is not None:
                    if not isinstance(mask, dict):
                        raise ConfigError(f"config.json: {where}'mask' must be an object with 'size'")
                    kw["window"] = _int(mask, "size", where + "mask: ")
            else:
                kw["conv"] = _int(m, "conv", where)
            mlp = lay.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}'mlp' must be null or an object of kind 'dense'")
                kw["mlp"] = MelizenFeedForward(ff=_int(mlp, "ff", where + "mlp: "), limit=_positive(mlp, "limit", where + "mlp: "))
            layers.append(MelizenLayer(**kw))
        loop = d.get("loop")
        start = stop = 0
        times = 1
        if loop is not None:
            if not isinstance(loop, dict):
                raise ConfigError("config.json: 'loop' must be null or an object with 'start', 'stop' and 'times'")
            start, stop, times = _int(loop, "start", "loop: ", 0), _int(loop, "stop", "loop: ", 0), _int(loop, "times", "loop: ")
            if not start <= stop <= len(layers):
                raise ConfigError(f"config.json: loop: layers {start} .. {stop} of {len(layers)}")
        return cls(vocab_size=_int(d, "vocab", ""), width=width, max_positions=_int(d, "max_positions", ""),
                   norm_eps=_positive(norm, "eps", "norm: "), layers=tuple(layers), loop_start=start, loop_stop=stop,
                   loop_times=times, stop_ids=_as_ids(d.get("eos_token_id")))

    def to_dict(self):
        layers = []
        for lay in self.layers:
            m = {"heads": lay.heads, "kv_heads": lay.kv_heads, "dim": lay.dim, "vdim": lay.vdim}
            if lay.type == "attention":
                m["scale"] = lay.scale
                if lay.window is not None:
                    m["mask"] = {"size": lay.window}
            else:
                m["conv"] = lay.conv
            layers.append({"type": lay.type, "mixer": m,
                           "mlp": None if lay.mlp is None else {"kind": "dense", "ff": lay.mlp.ff, "limit": lay.mlp.limit}})
        d = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.width,
             "max_positions": self.max_positions, "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.looped:
            d["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.stop_ids:
            d["eos_token_id"] = list(self.stop_ids)
        return d

    @property
    def looped(self):
        return self.loop_stop > self.loop_start

    def chat_format(self, tokenizer):
        raise ConfigError("a Melizen model folder brings no chat format: give the prompt as token ids")

    def with_stop_ids(self, ids):
        return replace(self, stop_ids=tuple(ids))

    def with_context_length(self, n):
        if n is None or n < 0:
            return self
        return replace(self, context_length=min(n, self.max_positions))

    def run_order(self):
        """Layers before the loop once, the loop's layers ``times`` times in a row, the rest once. The first entry
        of every pass is preceded by the pass's vector and, from the second pass on, by the embedding's output."""
        if not self.looped:
            return tuple(Run(layer=i) for i in range(len(self.layers)))
        runs = [Run(layer=i) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            for i in range(self.loop_start, self.loop_stop):
                before = None
                if i == self.loop_start:
                    before = Inject(embedding=t > 0, vector_name="loop.step", vector_rows=self.loop_times, row=t)
                runs.append(Run(layer=i, before=before))
        runs += [Run(layer=i) for i in range(self.loop_stop, len(self.layers))]
        return tuple(runs)

    def model_spec(self):
        d, eps = self.width, self.norm_eps
        blocks = []
        for i, lay in enumerate(self.layers):
            p = f"l{i}."
            if lay.type == "attention":
                mixer = AttentionSpec(
                    hidden=d, n_heads=lay.heads, n_kv_heads=lay.kv_heads, head_dim=lay.dim, v_head_dim=lay.vdim,
                    position=None, window=lay.window, scale=lay.scale,
                    distance_bias=DistanceBias(SLOPE_BASE, SLOPE_EXPONENT), sink=SINK_SCORE, out_scale_name=p + "ls1",
                    names={"q": p + "mix.q", "k": p + "mix.k", "v": p + "mix.v", "o": p + "mix.o",
                           "q_bias": p + "mix.q.b", "k_bias": p + "mix.k.b", "v_bias": p + "mix.v.b"})
            else:
                mixer = GatedDeltaSpec(
                    hidden=d, n_heads=lay.heads, n_kv_heads=lay.kv_heads, key_dim=lay.dim, value_dim=lay.vdim,
                    conv_taps=lay.conv, unit_eps=UNIT_EPS, norm_eps=eps, out_scale_name=p + "ls1",
                    names={k: p + "mix." + v for k, v in {
                        "q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv",
                        "b": "b", "a": "a", "A_log": "A_log", "dt_bias": "dt_bias", "g": "g", "norm": "norm", "o": "o"}.items()})
            ffn = None
            if lay.mlp is not None:
                ffn = GatedFeedForwardSpec(hidden=d, intermediate=lay.mlp.ff, activation=GATE_SLOPE_ACTIVATION,
                                           limit=lay.mlp.limit, up_shift=UP_SHIFT, out_scale_name=p + "ls2",
                                           names={"gate": p + "mlp.gate", "up": p + "mlp.up", "down": p + "mlp.down"})
            blocks.append(BlockSpec(kind="parallel",
                                    mixer_norm=NormSpec(dim=d, eps=eps, names={"weight": p + "norm1"}, weight_offset=1.0),
                                    mixer=mixer, ffn_norm=None, ffn=ffn))
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden=d, layers=tuple(blocks),
            run_order=self.run_order(),
            final_norm=NormSpec(dim=d, eps=eps, names={"weight": "final.norm"}, weight_offset=1.0),
            max_positions=self.max_positions, tie_embeddings=False, embedding_name="embed", head_name="head",
            stop_ids=self.stop_ids, position_table_name="pos",
            # (a folder may hold the scale of a feed-forward that a layer does not have, and the passes' vectors of a
            # loop over no layer: nothing reads them)
            unused_tensor_names=tuple(f"l{i}.ls2" for i, lay in enumerate(self.layers) if lay.mlp is None)
            + (() if self.looped else ("loop.step",)))


register_architecture("Melizen", MelizenConfiguration)

"""RWKV-style time mixing as a mixer: a decayed matrix per head in place of a cache of keys and values.

With h the normalised input and h' the previous token's (zeros at a sequence's start), each of r, k, v, g, w reads a
blend of its own, ``h + (h' - h) * mu_s``. r, k, v are projections of theirs into ``n_heads`` heads of ``head_dim``;
the gate is silu of one more; the decay per head and key channel is ``exp(-exp(W_w2 tanh(W_w1 blend_w) + w0))``. Per
head, with S [head_dim, head_dim] in 32-bit::

    o = (S + diag(u) k v^T)^T r;    S <- diag(decay) S + k v^T

(the bonus u counts for the current token only). Each head's o is divided by its root mean square, multiplied by a
weight per channel and by the gate, and goes through the output projection. The projections' sums stay in 32-bit,
and so does everything behind them. The rows of W_r, W_k, W_v, W_g and W_w1 are stacked: a step of few tokens makes
all five projections with ONE product over the five blends stacked by rows (every blend meets every matrix; the
kernels read the five blocks on the diagonal; the weights, which are what such a step waits for, are read once), a
prompt makes five products over the stored matrices. A sequence's state (its last h, then the heads' matrices) lives in the cache's
per-slot state, zeroed when the slot is handed out; the kernels (``csrc/mixers.hip``) walk a step's tokens in order
from it, so every cut of a sequence into steps gives the same result.
"""
from __future__ import annotations

import torch

from ..cache import StateNeed
from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import register_part

_BLENDS = ("r", "k", "v", "g", "w")


class TimeMix:
    graph_safe = True      # kernel launches on the current stream only; the state is indexed with the step's slot numbers on the device
    adds_only = True       # never reads the residual rows

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype
        self.d, self.H, self.D, self.rank = spec.hidden, spec.n_heads, spec.head_dim, spec.decay_rank
        if not 1 <= self.D <= 256:
            raise ValueError(f"heads of {self.D} elements: the time mixing's kernel holds up to 256")
        self.names = spec.names
        self.out_mult = float(getattr(spec, "out_mult", 1.0))
        self.state_off = -(-self.d // 4) * 4          # the matrices follow the held row
        self.mu = self.w = self.w0 = self.bonus = self.norm_w = self.w_o = self.out_scale = None

    def tensors(self):
        n, d, HD = self.names, self.d, self.H * self.D
        out = {n["mu_" + s]: TensorSpec((d,), "vector", 0.5, 0.25) for s in _BLENDS}
        out.update({n[s]: TensorSpec((HD, d)) for s in ("r", "k", "v", "g")})
        out.update({n["w1"]: TensorSpec((self.rank, d)), n["w2"]: TensorSpec((HD, self.rank)),
                    n["w0"]: TensorSpec((HD,), "vector", -1.0, 0.5), n["u"]: TensorSpec((self.H, self.D), "vector", 0.0, 0.5),
                    n["norm"]: TensorSpec((HD,), "vector"), n["o"]: TensorSpec((d, HD))})
        return out

    def load(self, weights):
        n = self.names
        without = getattr(self, "without", frozenset())
        parts = [weights[n[s]] for s in ("r", "k", "v", "g", "w1")]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        rows = sum(p.shape[0] for p in parts)
        pad = torch.zeros((-(-rows // 16) * 16 - rows, self.d), dtype=dt, device=parts[0].device)
        self.w_all = ops.for_few_rows(torch.cat([p.to(dt) for p in parts] + [pad], dim=0).contiguous(), without=without)
        lo = 0
        self.w = {}
        for s, p in zip(("r", "k", "v", "g", "w1"), parts):      # the stored names stay addressable as views
            self.w[s] = weights[n[s]] = self.w_all[lo:lo + p.shape[0]]
            lo += p.shape[0]
        self.w["w2"] = ops.for_few_rows(weights[n["w2"]], without=without)
        self.w_o = ops.for_eight_rows(weights[n["o"]], without=without)
        # what the kernels behind the projections read is kept in 32-bit
        self.mu = torch.stack([weights[n["mu_" + s]].float() for s in _BLENDS]).contiguous()
        self.w0 = weights[n["w0"]].float().contiguous()
        self.bonus = weights[n["u"]].float().contiguous()
        self.norm_w = weights[n["norm"]].float().contiguous()
        if self.out_mult != 1.0:
            self.out_scale = torch.full((self.d,), self.out_mult, dtype=torch.float32, device=self.mu.device)

    def kv_need(self):
        return None

    def state_need(self):
        return StateNeed(self.state_off + self.H * self.D * self.D, torch.float32)

    def forward(self, ctx, h, x, run, epilogue=ops.EPI_ADD):
        if isinstance(h, ops.Normed):
            h = h.materialize()
        T, d, H, D = h.shape[0], self.d, self.H, self.D
        state = ctx.slot_state(run.entry)
        blends = ctx.buffer("timemix_blends", (len(_BLENDS), T, d), self.dtype)
        K.shift_mix(h, self.mu, state, ctx.cu_seqlens, ctx.seq_of_token, ctx.slot_ids, blends,
                    one_token_each=bool(ctx.decode and ctx.max_q_len == 1))
        HD = H * D
        if 5 * T <= ops.CHUNK_ROWS and self.dtype == torch.bfloat16:
            # few tokens: one product of all five blends with all five matrices; block (s, s) is projection s
            both = ctx.buffer("timemix_all", (5 * T, self.w_all.shape[0]), torch.float32)
            ops.linear(blends.view(5 * T, d), self.w_all, both, ops.EPI_STORE, ctx)
            r, k, v, g = (both[i * T:(i + 1) * T, i * HD:(i + 1) * HD] for i in range(4))
            inner = both[4 * T:5 * T, 4 * HD:4 * HD + self.rank]
        else:
            proj = ctx.buffer("timemix_proj", (4, T, HD), torch.float32)        # r, k, v, gate
            for i, s in enumerate(("r", "k", "v", "g")):
                ops.linear(blends[i], self.w[s], proj[i], ops.EPI_STORE, ctx)
            r, k, v, g = proj[0], proj[1], proj[2], proj[3]
            inner = ctx.buffer("timemix_decay_inner", (T, self.rank), torch.float32)
            ops.linear(blends[4], self.w["w1"], inner, ops.EPI_STORE, ctx)
        squashed = ctx.buffer("timemix_decay_tanh", (T, self.rank), self.dtype)
        K.tanh_rows(inner, squashed)
        w_log = ctx.buffer("timemix_decay_log", (T, HD), torch.float32)
        ops.linear(squashed, self.w["w2"], w_log, ops.EPI_STORE, ctx, bias=self.w0)
        y = ctx.buffer("timemix_out", (T, HD), self.dtype)
        if ctx.max_q_len <= 16 or not g.is_contiguous():
            # the recurrence, and at the end of its round the read-outs' norm per head with weight and gate: one launch
            K.timemix(r, k, v, w_log, self.bonus, state, self.state_off, ctx.cu_seqlens, ctx.slot_ids, None, H, D,
                      gate=g, norm_w=self.norm_w, eps=self.spec.norm_eps, normed=y, max_q_len=ctx.max_q_len)
        else:
            # a prompt: a second barrier in every round of the chain costs more than a kernel that does all norms at once
            # (2,048 tokens, 32 heads of 64: 8 layers 10.8 against 12.5 ms)
            o = ctx.buffer("timemix_readout", (T, HD), torch.float32)
            K.timemix(r, k, v, w_log, self.bonus, state, self.state_off, ctx.cu_seqlens, ctx.slot_ids, o, H, D,
                      max_q_len=ctx.max_q_len)
            K.head_norm_gate(o, self.norm_w, g, self.spec.norm_eps, y, H, D)
        ops.linear(y, self.w_o, x, epilogue, ctx, col_scale=self.out_scale)


register_part("mixer", "time_mix", TimeMix)

"""minGRU as a mixer: a gated recurrence per channel whose gates read the current token alone.

With h the normalised input, per channel c of ``width``::

    z = sigmoid(W_z h + b_z);   u = W_x h + b_x;   cand = u + 1/2 (u >= 0), sigmoid(u) (u < 0)
    S <- (1 - z) S + z cand;    out = W_o (S * silu(W_g h))

The rows of W_z, W_x and W_g are stacked for one product (zero rows up to a multiple of 16) whose sums stay in
32-bit; gates, candidate and state are 32-bit. A sequence's state ([width] floats) lives in the cache's per-slot
state, zeroed when the slot is handed out; the kernel (``csrc/mixers.hip``) walks a step's tokens in order from it, so
every cut of a sequence into steps gives the same result.
"""
from __future__ import annotations

import torch

from ..cache import StateNeed
from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import register_part


class MinGRU:
    graph_safe = True      # kernel launches on the current stream only; the state is indexed with the step's slot numbers on the device
    adds_only = True       # never reads the residual rows

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype
        self.d, self.W, self.names = spec.hidden, spec.width, spec.names
        self.n_pad = -(-3 * self.W // 16) * 16
        self.out_mult = float(getattr(spec, "out_mult", 1.0))
        self.w_in = self.w_o = self.bias = self.out_scale = None

    def tensors(self):
        n, d, W = self.names, self.d, self.W
        return {n["z"]: TensorSpec((W, d)), n["x"]: TensorSpec((W, d)), n["g"]: TensorSpec((W, d)),
                n["o"]: TensorSpec((d, W)), n["z_bias"]: TensorSpec((W,), "vector", 0.0, 0.5),
                n["x_bias"]: TensorSpec((W,), "vector", 0.0, 0.5)}

    def load(self, weights):
        n = self.names
        parts = [weights[n[k]] for k in ("z", "x", "g")]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        pad = torch.zeros((self.n_pad - 3 * self.W, self.d), dtype=dt, device=parts[0].device)
        self.w_in = torch.cat([p.to(dt) for p in parts] + [pad], dim=0).contiguous()
        for i, k in enumerate(("z", "x", "g")):      # the stored names stay addressable as views
            weights[n[k]] = self.w_in[i * self.W:(i + 1) * self.W]
        without = getattr(self, "without", frozenset())
        ops.for_few_rows(self.w_in, without=without)
        self.w_o = ops.for_eight_rows(weights[n["o"]], without=without)
        self.bias = torch.zeros(self.n_pad, dtype=torch.float32, device=self.w_in.device)
        self.bias[:self.W] = weights[n["z_bias"]].float()
        self.bias[self.W:2 * self.W] = weights[n["x_bias"]].float()
        if self.out_mult != 1.0:
            self.out_scale = torch.full((self.d,), self.out_mult, dtype=torch.float32, device=self.w_in.device)

    def kv_need(self):
        return None

    def state_need(self):
        return StateNeed(self.W, torch.float32)

    def forward(self, ctx, h, x, run, epilogue=ops.EPI_ADD):
        T = h.shape[0]
        proj = ctx.buffer("mingru_proj", (T, self.n_pad), torch.float32)
        ops.linear(h, self.w_in, proj, ops.EPI_STORE, ctx, bias=self.bias)
        y = ctx.buffer("mingru_out", (T, self.W), self.dtype)
        runs = None
        if ctx.max_q_len > 2 * K.MINGRU_RUN:      # a long prompt: the scan in three passes over runs of tokens
            runs = ctx.buffer("mingru_runs", (2, ctx.n_seqs, -(-ctx.max_q_len // K.MINGRU_RUN), self.W), torch.float32)
        K.mingru_scan(proj, self.W, ctx.slot_state(run.entry), ctx.cu_seqlens, ctx.slot_ids, y, ctx.max_q_len, runs)
        ops.linear(y, self.w_o, x, epilogue, ctx, col_scale=self.out_scale)


register_part("mixer", "mingru", MinGRU)

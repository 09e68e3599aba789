"""The gated delta rule as a mixer: a matrix per head in place of a cache of keys and values.

Per value head (``n_heads`` of them share ``n_kv_heads`` query/key heads) the sequence's state is a matrix
S [key_dim, value_dim] in 32-bit. A token decays it, corrects what S holds under its key towards its value, and
reads it with its query::

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

q, k and v are projections of the normalised input that pass a short causal convolution over time per channel
and silu; q and k are then scaled to unit length per head (q also by key_dim ** -0.5). g = exp(-exp(A_log) *
softplus(a + dt_bias)) and beta = sigmoid(b) come from two more columns per head of the same projection. Each
head's read-out is divided by its root mean square, multiplied by a weight shared by the heads and by silu of a
gate (one more projection), and goes through the output projection into the residual stream.

One product makes all of it: the rows of q, k, v, the gate, b and a are stacked (and padded with zero rows to a
multiple of 16), its sums stay in 32-bit. The state of a sequence (the matrices, and the last ``conv_taps - 1``
inputs of the convolution) lives in the cache's per-slot state, zeroed when the slot is handed out; the kernels
(``csrc/delta_rule.hip``) walk a step's tokens one by one from it, so every cut of a sequence into steps gives the
same result.
"""
from __future__ import annotations

import torch

from ..cache import StateNeed
from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import register_part


class GatedDeltaRule:
    graph_safe = True      # kernel launches on the current stream only; the state is indexed with the step's slot numbers on the device
    adds_only = True       # never reads the residual rows

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype
        self.d, self.H, self.G = spec.hidden, spec.n_heads, spec.n_kv_heads
        self.D, self.Dv, self.taps = spec.key_dim, spec.value_dim, spec.conv_taps
        if self.H % self.G:
            raise ValueError(f"{self.H} value heads are not a multiple of {self.G} query/key heads")
        if not 1 <= self.D <= 256:
            raise ValueError(f"keys of {self.D} elements: the delta rule's kernels hold up to 256")
        self.names = spec.names
        GD, HV = self.G * self.D, self.H * self.Dv
        # columns of the stacked projection
        self.off_q, self.off_k, self.off_v, self.off_g = 0, GD, 2 * GD, 2 * GD + HV
        self.off_b, self.off_a = 2 * GD + 2 * HV, 2 * GD + 2 * HV + self.H
        self.n_in = 2 * GD + 2 * HV + 2 * self.H
        self.n_pad = -(-self.n_in // 16) * 16
        self.channels = 2 * GD + HV
        self.out_scale_name = getattr(spec, "out_scale_name", None)
        self.w_in = self.w_o = self.conv_w = self.A_log = self.dt_bias = self.norm_w = self.out_scale = None

    def tensors(self):
        n, d, GD, HV, H = self.names, self.d, self.G * self.D, self.H * self.Dv, self.H
        out = {n["q"]: TensorSpec((GD, d)), n["k"]: TensorSpec((GD, d)), n["v"]: TensorSpec((HV, d)),
               n["g"]: TensorSpec((HV, d)), n["b"]: TensorSpec((H, d)), n["a"]: TensorSpec((H, d)),
               n["o"]: TensorSpec((d, HV)),
               n["q_conv"]: TensorSpec((GD, self.taps)), n["k_conv"]: TensorSpec((GD, self.taps)),
               n["v_conv"]: TensorSpec((HV, self.taps)),
               n["A_log"]: TensorSpec((H,), "vector", 0.0, 0.5), n["dt_bias"]: TensorSpec((H,), "vector", 0.0, 0.5),
               n["norm"]: TensorSpec((self.Dv,), "vector")}
        if self.out_scale_name:
            out[self.out_scale_name] = TensorSpec((d,), "vector", 1.0, 0.1)
        return out

    def load(self, weights):
        n = self.names
        parts = [weights[n[k]] for k in ("q", "k", "v", "g", "b", "a")]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        pad = torch.zeros((self.n_pad - self.n_in, self.d), dtype=dt, device=parts[0].device)
        self.w_in = torch.cat([p.to(dt) for p in parts] + [pad], dim=0).contiguous()
        lo = 0
        for k, p in zip(("q", "k", "v", "g", "b", "a"), parts):      # the stored names stay addressable as views
            weights[n[k]] = self.w_in[lo:lo + p.shape[0]]
            lo += p.shape[0]
        without = getattr(self, "without", frozenset())
        ops.for_few_rows(self.w_in, without=without)
        self.w_o = ops.for_eight_rows(weights[n["o"]], without=without)
        # what the recurrence's kernels read is kept in 32-bit
        self.conv_w = torch.cat([weights[n[k]].float() for k in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.A_log = weights[n["A_log"]].float().contiguous()
        self.dt_bias = weights[n["dt_bias"]].float().contiguous()
        self.norm_w = weights[n["norm"]].float().contiguous()
        if self.out_scale_name:
            self.out_scale = weights[self.out_scale_name].float().contiguous()

    def kv_need(self):
        return None

    def state_need(self):
        return StateNeed(K.delta_state_floats(self.H, self.G, self.D, self.Dv, self.taps), torch.float32)

    def forward(self, ctx, h, x, run):
        T, H, G, D, Dv, taps = h.shape[0], self.H, self.G, self.D, self.Dv, self.taps
        state = ctx.slot_state(run.entry)
        proj = ctx.buffer("delta_proj", (T, self.n_pad), torch.float32)
        ops.linear(h, self.w_in, proj, ops.EPI_STORE, ctx)
        act = ctx.buffer("delta_act", (T, self.channels), torch.float32)
        gates = ctx.buffer("delta_gates", (T, 2 * H), torch.float32)
        K.delta_prep(proj, (self.off_q, self.off_k, self.off_v, self.off_b, self.off_a), self.conv_w, self.A_log,
                     self.dt_bias, state, ctx.cu_seqlens, ctx.seq_of_token, ctx.slot_ids, act, gates, H, G, D, Dv, taps,
                     self.spec.unit_eps, float(D) ** -0.5, one_token_each=bool(ctx.decode and ctx.max_q_len == 1))
        o = ctx.buffer("delta_readout", (T, H * Dv), torch.float32)
        y = ctx.buffer("delta_out", (T, H * Dv), self.dtype)
        K.delta_recurrence(act, gates, state, ctx.cu_seqlens, ctx.slot_ids, o, proj, self.off_g, self.norm_w, y,
                           H, G, D, Dv, taps, self.spec.norm_eps)
        ops.linear(y, self.w_o, x, ops.EPI_ADD, ctx, col_scale=self.out_scale)


register_part("mixer", "gated_delta", GatedDeltaRule)

"""A state-space mixer with a selective scan (the first Mamba form), without a cache of keys.

h -> [x | z] (``inner`` each) by one product; x passes a short causal convolution over time per channel (with a bias)
and SiLU; x -> [dt_in (dt_rank) | B (state) | C (state)] by a second product; the step size is
dt = softplus(W_dt dt_in + dt_bias), one per channel; A = -exp(A_log) [inner, state].  Per channel c and state n, with
the state S carried from token to token in float:

    S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;    y_c = sum_n S[c, n] C_n + D_c x_c

then y * silu(z) and the output projection.  State per request: the convolution's last taps - 1 inputs and S.
Step sizes (their product's result included), softplus, exponentials and S are float in every mode."""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import Mixer, StateNeed, register_part
from .delta import _rows


class SelectiveScan(Mixer):
    graph_safe = True      # its kernels walk the requests from the step's device tensors

    def __init__(self, prefix: str, position, hidden_size: int, inner: int, state: int, dt_rank: int, taps: int):
        if not 1 <= taps <= ops.MAX_CONV_TAPS:
            raise ValueError(f"a short convolution has 1 to {ops.MAX_CONV_TAPS} taps, got {taps}")
        if not 0 < state <= ops.SCAN_MAX_STATES:
            raise ValueError(f"{state} states per channel are not supported: the scan kernel holds a channel's states in "
                             f"the registers of up to 16 lanes, {ops.SCAN_MAX_STATES} at most")
        self.prefix, self.hidden_size = prefix, hidden_size
        self.inner, self.state, self.dt_rank, self.taps = inner, state, dt_rank, taps

    # ---- weights
    def tensor_specs(self):
        p, W, I, S, R = self.prefix, self.hidden_size, self.inner, self.state, self.dt_rank
        return [TensorSpec(p + "in", (2 * I, W)), TensorSpec(p + "conv", (I, self.taps), "bias"),
                TensorSpec(p + "conv.b", (I,), "bias"), TensorSpec(p + "x", (R + 2 * S, I)),
                TensorSpec(p + "dt", (I, R)), TensorSpec(p + "dt.b", (I,), "bias"),
                TensorSpec(p + "A_log", (I, S), "bias"), TensorSpec(p + "D", (I,), "norm"),
                TensorSpec(p + "o", (W, I))]

    def load(self, get, rt):
        self.rt = rt
        t = {s.name[len(self.prefix):]: get(s) for s in self.tensor_specs()}
        self.w_in, self.w_x, self.w_dt, self.w_o = (linear.prepare_weight(t[n]) for n in ("in", "x", "dt", "o"))
        self.conv_w, self.conv_b, self.dt_bias, self.D = t["conv"], t["conv.b"], t["dt.b"], t["D"]
        self.A = (-torch.exp(t["A_log"].float())).contiguous()

    # ---- state
    def state_need(self):
        return (StateNeed((max(1, self.taps - 1), self.inner), None),
                StateNeed((self.inner, self.state), torch.float32))

    # ---- step
    def forward(self, h, ctx, kv, state):
        conv_state, S = state.slots
        N, I, R, n = ctx.num_tokens, self.inner, self.dt_rank, self.state
        xz = linear.linear(h, self.w_in)
        x = ops.short_conv(xz[:, :I], self.conv_w, conv_state, ctx, self.rt.empty(N, I), ops.CONV_SILU, bias=self.conv_b)
        proj = linear.linear(x, self.w_x)
        dt_in = linear.linear(_rows(proj, 0, R), self.w_dt, out_dtype=torch.float32)
        y = ops.selective_scan(x, dt_in, self.dt_bias, self.A, proj[:, R:R + n], proj[:, R + n:], self.D, xz[:, I:], S, ctx,
                               self.rt.empty(N, I))
        return linear.linear(y, self.w_o)


register_part("mixer", "selective_scan", SelectiveScan)

"""The gated delta rule as a mixer without a cache of keys.

h -> q, k (kv_heads x dim), v (heads x vdim), each through a short causal convolution over time and SiLU; q and k
made unit vectors per head (q also times dim^-1/2); beta = sigmoid(W_b h); the decay
g = exp(-exp(A_log) * softplus(a + dt_bias)) with, by ``decay``, "channel": a = W_a2 W_a1 h, one number per head and
key channel, or "head": a = W_a h, one number per head.  Per head, with the state S [dim, vdim] carried from token to
token in float:

    S <- g * S (row i by g_i);  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q

so the read-out sees the token's own write.  o is divided by its root mean square per head, scaled by a weight shared
by the heads and gated, by ``gate``, with "low_rank_sigmoid": sigmoid(W_g2 W_g1 h) or "silu": silu(W_g h); then the
output projection.  Head i reads q/k head i // (heads // kv_heads).  State per request: the convolution's last
taps - 1 inputs and S."""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import Mixer, StateNeed, register_part


def _rows(t: torch.Tensor, lo: int, hi: int) -> torch.Tensor:
    """Columns lo..hi of ``t`` as the input of a product: the slice itself where a kernel takes it as it lies."""
    s = t[:, lo:hi]
    # the float kernel takes any row slice; the few-rows matrix-core kernels take rows that start 16-byte aligned
    if t.dtype == torch.float32 or (t.shape[0] <= ops.SKINNY_MAX_ROWS and s.shape[1] % 8 == 0
                                    and (t.shape[0] == 1 or s.stride(0) % 8 == 0) and s.data_ptr() % 16 == 0):
        return s
    return s.contiguous()


class GatedDelta(Mixer):
    graph_safe = True      # its kernels walk the requests from the step's device tensors

    def __init__(self, prefix: str, position, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int,
                 eps: float, decay_rank: int = 0, gate_rank: int = 0, decay: str = "channel",
                 gate: str = "low_rank_sigmoid"):
        if decay not in ("channel", "head") or gate not in ("low_rank_sigmoid", "silu"):
            raise ValueError(f"decay is 'channel' or 'head' and gate 'low_rank_sigmoid' or 'silu', got {decay!r}, {gate!r}")
        if (decay == "channel" and decay_rank <= 0) or (gate == "low_rank_sigmoid" and gate_rank <= 0):
            raise ValueError("a low-rank map needs its rank")
        if heads % kv_heads:
            raise ValueError(f"{heads} heads cannot share {kv_heads} query/key heads")
        if not 1 <= taps <= ops.MAX_CONV_TAPS:
            raise ValueError(f"a short convolution has 1 to {ops.MAX_CONV_TAPS} taps, got {taps}")
        if dim > 512:
            raise ValueError(f"key size {dim} is not supported: the kernel holds a column of the state in registers, up to 512 rows")
        self.prefix, self.hidden_size = prefix, hidden_size
        self.heads, self.kv_heads, self.dim, self.vdim, self.taps = heads, kv_heads, dim, vdim, taps
        self.decay, self.gate = decay, gate
        self.decay_rank = decay_rank if decay == "channel" else 0
        self.gate_rank = gate_rank if gate == "low_rank_sigmoid" else 0
        self.eps = float(eps)
        self.qk, self.vw = kv_heads * dim, heads * vdim

    # ---- weights
    def tensor_specs(self):
        p, W = self.prefix, self.hidden_size
        H, D = self.heads, self.dim
        specs = []
        for name, rows in (("q", self.qk), ("k", self.qk), ("v", self.vw)):
            specs += [TensorSpec(p + name, (rows, W)), TensorSpec(p + name + ".conv", (rows, self.taps), "bias")]
        specs += [TensorSpec(p + "b", (H, W)), TensorSpec(p + "A_log", (H,), "bias"),
                  TensorSpec(p + "norm", (self.vdim,), "norm")]
        if self.decay == "channel":
            specs += [TensorSpec(p + "a1", (self.decay_rank, W)), TensorSpec(p + "a2", (H * D, self.decay_rank)),
                      TensorSpec(p + "dt_bias", (H * D,), "bias")]
        else:
            specs += [TensorSpec(p + "a", (H, W)), TensorSpec(p + "dt_bias", (H,), "bias")]
        if self.gate == "low_rank_sigmoid":
            specs += [TensorSpec(p + "g1", (self.gate_rank, W)), TensorSpec(p + "g2", (self.vw, self.gate_rank))]
        else:
            specs += [TensorSpec(p + "g", (self.vw, W))]
        specs.append(TensorSpec(p + "o", (W, self.vw)))
        return specs

    def load(self, get, rt):
        self.rt = rt
        t = {s.name[len(self.prefix):]: get(s) for s in self.tensor_specs()}
        # one product for everything that reads h and is used in the activations' type:
        # q | k | v | a1 (if the decay is low-rank) | g1 or g | b
        packed = [t["q"], t["k"], t["v"]] + ([t["a1"]] if self.decay == "channel" else [])
        packed += [t["g1"] if self.gate == "low_rank_sigmoid" else t["g"], t["b"]]
        self.w_in = linear.prepare_weight(torch.cat(packed, dim=0))
        self.conv_w = torch.cat([t["q.conv"], t["k.conv"], t["v.conv"]], dim=0).contiguous()
        # the decay's input leaves its product as float: a2 after a1, or a straight from h
        self.w_a = linear.prepare_weight(t["a2"] if self.decay == "channel" else t["a"])
        self.w_g2 = linear.prepare_weight(t["g2"]) if self.gate == "low_rank_sigmoid" else None
        self.w_o = linear.prepare_weight(t["o"])
        self.A_log, self.dt_bias, self.norm_w = t["A_log"], t["dt_bias"], t["norm"]

    # ---- state
    def state_need(self):
        return (StateNeed((max(1, self.taps - 1), 2 * self.qk + self.vw), None),
                StateNeed((self.heads, self.dim, self.vdim), torch.float32))

    # ---- step
    def forward(self, h, ctx, kv, state):
        return self.forward_residual(h, ctx, kv, state, None)

    def forward_residual(self, h, ctx, kv, state, x):
        conv_state, S = state.slots
        N = ctx.num_tokens
        cw = 2 * self.qk + self.vw
        a_at, g_at = cw, cw + self.decay_rank
        b_at = g_at + (self.gate_rank if self.gate == "low_rank_sigmoid" else self.vw)
        proj = linear.linear(h, self.w_in)
        qkv = ops.short_conv(proj[:, :cw], self.conv_w, conv_state, ctx, self.rt.empty(N, cw), ops.CONV_SILU)
        if self.decay == "channel":
            a = linear.linear(_rows(proj, a_at, g_at), self.w_a, out_dtype=torch.float32)
        else:
            a = linear.linear(h, self.w_a, out_dtype=torch.float32)
        gate = proj[:, g_at:b_at] if self.w_g2 is None else linear.linear(_rows(proj, g_at, b_at), self.w_g2)
        o = self.rt.empty(N, self.vw, dtype=torch.float32)
        ops.gated_delta(qkv[:, :self.qk], qkv[:, self.qk:2 * self.qk], qkv[:, 2 * self.qk:], a, proj[:, b_at:],
                        self.A_log, self.dt_bias, S, ctx, o, self.heads, self.kv_heads, self.dim, self.vdim,
                        decay_per_channel=self.decay == "channel")
        y = ops.gated_head_norm(o, self.norm_w, gate, self.rt.empty(N, self.vw), self.heads, self.vdim, self.eps,
                                "sigmoid" if self.gate == "low_rank_sigmoid" else "silu")
        return linear.linear_residual(y, self.w_o, None, x)


register_part("mixer", "gated_delta", GatedDelta)

"""Attention through a low-rank latent.

Queries: c_q = norm(W_dq h), q = W_uq c_q, head by head [dim flat | rot_dim rotated].  Keys and values: W_dkv h gives
kv_rank + rot_dim numbers; the first kv_rank, normalised, are the latent c, the rest, rotated by the position, are one
key part kr shared by all heads.  A head's flat key is W_uk c and its value W_uv c, so only c and kr are cached and

    score(n, j) = scale (q_flat . W_uk c_j + q_rot . kr_j) = scale ([W_uk^T q_flat ; q_rot] . [c_j ; kr_j])
    out(n)     = W_uv sum_j p_j c_j

: the two per-head maps act on the query and on the attention's result, and the attention itself reads the pages of
latents as they lie, one "head" for all query heads.  The softmax may have a window (the last ``window`` keys up to
the token itself) and a sink (a learned number per head that joins the denominator, unscaled, with no value).  The
heads' outputs are gated by sigmoid(W_g h) before the output projection."""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import CacheNeed, Mixer, PageTensor, register_part


class LatentAttention(Mixer):
    def __init__(self, prefix: str, position, hidden_size: int, heads: int, dim: int, rot_dim: int, vdim: int,
                 q_rank: int, kv_rank: int, scale: float, eps: float, window: Optional[int] = None, sink: bool = True,
                 output_gate: bool = True):
        if position is None or not hasattr(position, "rotate"):
            raise ValueError("latent attention needs a position encoding that can turn a slice of a vector (rotary_pairs)")
        if window is not None and window <= 0:
            raise ValueError("window must be positive")
        if kv_rank > 1024:
            raise ValueError(f"latent size {kv_rank} is not supported: the attention kernel takes up to 1,024")
        self.prefix, self.position, self.hidden_size = prefix, position, hidden_size
        self.heads, self.dim, self.rot_dim, self.vdim = heads, dim, rot_dim, vdim
        self.q_rank, self.kv_rank, self.scale, self.eps = q_rank, kv_rank, float(scale), float(eps)
        self.window, self.sink, self.output_gate = window, sink, output_gate

    # ---- weights
    def tensor_specs(self):
        p, W, H = self.prefix, self.hidden_size, self.heads
        specs = [TensorSpec(p + "dq", (self.q_rank, W)), TensorSpec(p + "dq.norm", (self.q_rank,), "norm"),
                 TensorSpec(p + "uq", (H * (self.dim + self.rot_dim), self.q_rank)),
                 TensorSpec(p + "dkv", (self.kv_rank + self.rot_dim, W)),
                 TensorSpec(p + "dkv.norm", (self.kv_rank,), "norm"),
                 TensorSpec(p + "uk", (H * self.dim, self.kv_rank)), TensorSpec(p + "uv", (H * self.vdim, self.kv_rank))]
        if self.sink:
            specs.append(TensorSpec(p + "sink", (H,), "bias"))
        if self.output_gate:
            specs.append(TensorSpec(p + "g", (H * self.vdim, W)))
        specs.append(TensorSpec(p + "o", (W, H * self.vdim)))
        return specs + self.position.tensor_specs()

    def load(self, get, rt):
        self.rt = rt
        t = {s.name[len(self.prefix):]: get(s) for s in LatentAttention.tensor_specs(self) if s.name.startswith(self.prefix)}
        H = self.heads
        # one product for everything that reads h: dq | dkv | g
        self.w_in = linear.prepare_weight(torch.cat([t["dq"], t["dkv"]] + ([t["g"]] if self.output_gate else []), dim=0))
        self.w_uq, self.w_o = linear.prepare_weight(t["uq"]), linear.prepare_weight(t["o"])
        self.q_norm, self.kv_norm = t["dq.norm"], t["dkv.norm"]
        self.m_uk = t["uk"].view(H, self.dim, self.kv_rank).contiguous()                     # q_flat @ m_uk[h] = W_uk^T q_flat
        self.m_uv = t["uv"].view(H, self.vdim, self.kv_rank).transpose(1, 2).contiguous()    # o_latent @ m_uv[h] = W_uv o_latent
        self.sink_w = t["sink"] if self.sink else None
        self.position.load(get, rt)

    # ---- cache: the latent and the shared rotated key part
    def cache_need(self):
        tensors = [PageTensor("c", 1, self.kv_rank), PageTensor("kr", 1, self.rot_dim)]
        if ops.latent_mfma_sizes(self.kv_rank, self.rot_dim):
            # the matrix-core attention weighs the latents with the keys along a row: a transposed copy, kept only in
            # bfloat16 with pages of a multiple of 16 tokens
            tensors.append(PageTensor("ct", 1, self.kv_rank, transpose_at=16, transpose_in=torch.bfloat16,
                                      only_transposed=True))
        return CacheNeed(tuple(tensors), self.window)

    # ---- step
    def forward(self, h, ctx, kv, state):
        return self.forward_residual(h, ctx, kv, state, None)

    def forward_residual(self, h, ctx, kv, state, x):
        if kv is None:
            raise RuntimeError("latent attention needs a cache view")
        N, H, D, R, C, E = ctx.num_tokens, self.heads, self.dim, self.rot_dim, self.kv_rank, self.vdim
        proj = linear.linear(h, self.w_in)
        kv_at, g_at = self.q_rank, self.q_rank + C + R
        cq = ops.rms_norm_rows(proj[:, :kv_at], self.q_norm, self.eps, self.rt.empty(N, self.q_rank))
        q = linear.linear(cq, self.w_uq).view(N, H, D + R)
        if kv.store:
            ops.latent_kv_store(proj[:, kv_at:g_at], self.kv_norm, self.eps, ctx.positions, self.position.inv_freq,
                                kv.slot_mapping, kv.pages["c"], kv.pages["kr"], kv.pages.get("ct"))
        q_lat = self.rt.empty(N, H, C + R)
        ops.head_matmul(q[:, :, :D], self.m_uk, q_lat[:, :, :C])
        self.position.rotate(q[:, :, D:], q_lat[:, :, C:], ctx)
        o_lat = ops.latent_attention(q_lat, kv, ctx, self.rt.empty(N, H, C), self.scale, self.window, self.sink_w)
        y = ops.head_matmul(o_lat, self.m_uv, self.rt.empty(N, H, E), gate=proj[:, g_at:] if self.output_gate else None)
        return linear.linear_residual(y.view(N, H * E), self.w_o, None, x)


register_part("mixer", "latent_attention", LatentAttention)

"""Plain, slow, whole-sequence Gemadra decoder used only as the test oracle.

One function per mechanism, written from the design's equations in this file's own notation; no cache, no
batching, token-by-token loops where the design is a recurrence, and no import from the product package.
Everything runs in one floating type chosen by the caller (float64 by default).

Notation: a sequence is T tokens at positions 0..T-1; W is the model's width; every linear map is stored
[out, in] and applied as y = x @ W.T.

The design
* residual stream x; every layer:  x <- x + mixer(h) + ff(norm2(x)),  h = n + shortconv(n),  n = norm1(x)
* norm(x) = x / sqrt(mean(x^2) + eps) * (1 + w)
* shortconv(n)_t = sum_j w[:, j] * n_(t - taps + 1 + j)   (zeros before the start)
* mixers: ``channel_delta`` (a gated delta rule with one decay per head and key channel) and
  ``latent_attention`` (attention through a low-rank latent with a shared rotated key part, a sliding window,
  a per-head sink in the softmax's denominator and an output gate)
* feed-forward: down(xielu(up(h)))
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch
import torch.nn.functional as F
from safetensors import safe_open


# --------------------------------------------------------------------------- files
def read_config(model_dir) -> dict:
    return json.loads((Path(model_dir) / "config.json").read_text())


def read_weights(model_dir, dtype=torch.float64) -> dict:
    out = {}
    for f in sorted(Path(model_dir).glob("*.safetensors")):
        with safe_open(str(f), framework="pt") as fh:
            for name in fh.keys():
                out[name] = fh.get_tensor(name).to(dtype)
    return out


# --------------------------------------------------------------------------- small pieces
def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square over the last dimension, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """The layers' and the model's norm: the stored weight lies around zero."""
    return rms(x, eps) * (1.0 + w)


def plain_norm(x, w, eps):
    """The norms inside the mixers: the stored weight is the scale itself."""
    return rms(x, eps) * w


def causal_conv(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x [T, C], w [C, taps]: y_t = sum_j w[:, j] * x_(t - taps + 1 + j); the last column meets the current token."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return y


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def xielu(z: torch.Tensor, p, q) -> torch.Tensor:
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2."""
    ap = F.softplus(p)
    an = 0.5 + F.softplus(q)
    pos = ap * z * z + 0.5 * z
    neg = an * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, ..., >= dims]: the first ``dims`` entries turn, entry 2i with entry 2i+1, by positions * base^(-2i/dims)."""
    T = x.shape[0]
    i = torch.arange(dims // 2, dtype=x.dtype)
    f = base ** (-2.0 * i / dims)
    a = positions.to(x.dtype)[:, None] * f[None, :]            # [T, dims/2]
    shape = [T] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = a.cos().reshape(shape), a.sin().reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# --------------------------------------------------------------------------- feed-forward
def same(x):
    return x


def rounder(act_dtype):
    """x as an engine that stores activations in ``act_dtype`` would hold it (None: exact).  Used only to measure
    how far a faithful reduced-precision computation strays from the exact one."""
    return same if act_dtype is None else (lambda x: x.to(act_dtype).to(x.dtype))


def dense_ff(h, w, prefix, rd=same):
    act = w[prefix + "act"]
    return rd(rd(xielu(rd(h @ w[prefix + "up"].T), act[0], act[1])) @ w[prefix + "down"].T)


# --------------------------------------------------------------------------- the delta-rule mixer
def delta_rule(q, k, v, g, beta):
    """One head.  q, k, g [T, D]; v [T, E]; beta [T].  S [D, E] starts at zero.  Per token:
    S <- g * S (row i by g_i);  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, D = q.shape
    E = v.shape[1]
    S = torch.zeros(D, E, dtype=q.dtype)
    out = torch.zeros(T, E, dtype=q.dtype)
    for t in range(T):
        S = g[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def channel_delta(h, w, prefix, m, eps, rd=same):
    """h [T, W]; ``m`` the mixer's sizes (heads, kv_heads, dim, vdim).  ``rd`` rounds what an engine would store in
    its activations' type (the recurrence itself and what enters it beside q, k, v stay exact)."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]

    def branch(name):
        return rd(F.silu(causal_conv(rd(h @ w[prefix + name].T), w[prefix + name + ".conv"])))

    q = branch("q").reshape(T, G, D)
    k = branch("k").reshape(T, G, D)
    v = branch("v").reshape(T, H, E)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(rd(h @ w[prefix + "b"].T))                               # [T, H]
    a = rd(h @ w[prefix + "a1"].T) @ w[prefix + "a2"].T + w[prefix + "dt_bias"]     # [T, H*D]
    rate = torch.exp(w[prefix + "A_log"])                                          # [H]
    g = torch.exp(-rate[None, :, None] * F.softplus(a.reshape(T, H, D)))
    gate = torch.sigmoid(rd(rd(h @ w[prefix + "g1"].T) @ w[prefix + "g2"].T)).reshape(T, H, E)
    heads = []
    for i in range(H):
        j = i // (H // G)
        o = delta_rule(q[:, j], k[:, j], v[:, i], g[:, i], beta[:, i])
        heads.append(plain_norm(o, w[prefix + "norm"], eps) * gate[:, i])
    return rd(rd(torch.cat(heads, dim=-1)) @ w[prefix + "o"].T)


# --------------------------------------------------------------------------- latent attention
def latent_attention(h, w, prefix, m, eps, rd=same):
    """h [T, W]; ``m``: heads, dim (unrotated), rot_dim, vdim, kv_rank, rot {base, dims}, mask {size}, scale."""
    T = h.shape[0]
    H, D, R, E, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = rd(plain_norm(rd(h @ w[prefix + "dq"].T), w[prefix + "dq.norm"], eps))
    q = rd(cq @ w[prefix + "uq"].T).reshape(T, H, D + R)
    q_flat, q_rot = q[..., :D], rotate_interleaved(q[..., D:], pos, m["rot"]["dims"], m["rot"]["base"])
    kv = rd(h @ w[prefix + "dkv"].T)
    c = rd(plain_norm(kv[:, :C], w[prefix + "dkv.norm"], eps))
    k_rot = rd(rotate_interleaved(kv[:, C:], pos, m["rot"]["dims"], m["rot"]["base"]))    # [T, R], shared by heads
    k_flat = (c @ w[prefix + "uk"].T).reshape(T, H, D)
    v = (c @ w[prefix + "uv"].T).reshape(T, H, E)
    window = (m.get("mask") or {}).get("size")
    out = torch.zeros(T, H, E, dtype=h.dtype)
    for t in range(T):
        lo = 0 if window is None else max(0, t - window + 1)
        for i in range(H):
            s = (k_flat[lo:t + 1, i] @ q_flat[t, i] + k_rot[lo:t + 1] @ q_rot[t, i]) * m["scale"]
            sink = w[prefix + "sink"][i]
            top = torch.maximum(s.max(), sink)
            e = torch.exp(s - top)
            out[t, i] = (e[:, None] * v[lo:t + 1, i]).sum(0) / (e.sum() + torch.exp(sink - top))
    gate = torch.sigmoid(rd(h @ w[prefix + "g"].T))
    return rd(rd(out.reshape(T, H * E) * gate) @ w[prefix + "o"].T)


MIXERS = {"channel_delta": channel_delta, "latent_attention": latent_attention}


# --------------------------------------------------------------------------- the model
def forward(cfg: dict, w: dict, tokens, dtype=torch.float64, layers_out=None, act_dtype=None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  ``layers_out``: a list that receives the residual stream after every layer.
    ``act_dtype``: round the activations between the products as an engine of that type would (the residual stream,
    the norms' and recurrences' own arithmetic stay exact)."""
    rd = rounder(act_dtype)
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        n = rd(offset_norm(x, w[p + "norm1"], eps))
        h = rd(n + causal_conv(n, w[p + "canon1"]))
        y = MIXERS[layer["type"]](h, w, p + "mix.", layer["mixer"], eps, rd)
        if layer.get("mlp") is not None:
            y = y + dense_ff(rd(offset_norm(x, w[p + "norm2"], eps)), w, p + "mlp.", rd)
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    return rd(offset_norm(x, w["final.norm"], eps)) @ w["head"].T

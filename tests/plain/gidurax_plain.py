"""Plain, slow, whole-sequence Gidurax decoder used only as the test oracle.

One function per mechanism, written from the design's equations in this file's own notation; no cache, no
batching, token-by-token loops where the design is a recurrence, and no import from the product package.
Everything runs in one floating type chosen by the caller (float64 by default).

Notation: a sequence is T tokens at positions 0..T-1; W is the model's width; every linear map is stored
[out, in] and applied as y = x @ M.T.

The design
* x = embed[token] * embedding.scale =: e (kept)
* a stretch of layers [start, stop) is walked ``times`` times with the same weights; before pass t > 0 the kept e
  is added to x, and before every pass t the row t of ``loop.step`` is added to x
* a layer:  x <- x + m * norm1b(mixer(norm1(x)));  x <- x + m * norm2b(ff(norm2(x)))   (m = residual_mult)
* norm(x) = x / sqrt(mean(x^2) + eps) * w
* mixers: ``delta`` (gated delta rule, one decay per head), ``attention`` (grouped heads, q/k norm, a query
  temperature that grows with the logarithm of the position, a sink in the softmax's denominator) and ``mamba1``
  (selective scan)
* feed-forward: down(gelu(up(h))) with the exact gelu, alone or as routed experts (some of them identities) with an
  always-on shared expert behind a sigmoid gate
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
def same(x):
    return x


def rounder(act_dtype):
    """x as an engine that stores activations in ``act_dtype`` would hold it (None: exact).  Used only to measure how far
    a faithful reduced-precision computation strays from the exact one; ``rd`` below is such a function, applied to
    what the products and the convolutions leave (never to the residual stream, norms, decays or states)."""
    return same if act_dtype is None else (lambda x: x.to(act_dtype).to(x.dtype))


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square over the last dimension, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms(x, eps) * w


def silu(z):
    return z / (1.0 + torch.exp(-z))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def causal_conv(x: torch.Tensor, w: torch.Tensor, bias=None) -> torch.Tensor:
    """x [T, C], w [C, taps]: y_t = sum_j w[:, j] * x_(t - taps + 1 + j) (+ bias); the last column meets the token."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    if bias is not None:
        y = y + bias
    return y


def unit(x: torch.Tensor) -> torch.Tensor:
    """x / sqrt(sum(x^2) + 1e-6) over the last dimension."""
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + 1e-6)


# --------------------------------------------------------------------------- mixer: gated delta rule
def delta_decay(h, w_a, A_log, dt_bias):
    """g [T, heads] = exp(-exp(A_log) * softplus(h W_a^T + dt_bias))."""
    return torch.exp(-torch.exp(A_log) * softplus(h @ w_a.T + dt_bias))


def delta_recurrence(q, k, v, g, beta, S0=None):
    """q, k [T, heads, D] (already unit vectors, q scaled), v [T, heads, E], g, beta [T, heads].
    Per head:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.  Returns o [T, heads, E] and S."""
    T, H, D = q.shape
    E = v.shape[2]
    S = torch.zeros(H, D, E, dtype=q.dtype) if S0 is None else S0.clone()
    o = torch.zeros(T, H, E, dtype=q.dtype)
    for t in range(T):
        for h in range(H):
            Sh = S[h] * g[t, h]
            u = beta[t, h] * (v[t, h] - Sh.T @ k[t, h])
            Sh = Sh + torch.outer(k[t, h], u)
            S[h] = Sh
            o[t, h] = Sh.T @ q[t, h]
    return o, S


def delta_mixer(h, w, p, m, eps, rd=same):
    """h [T, W]; w: the tensors; p: the layer's prefix ('l3.mix.'); m: the mixer's sizes."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rd(silu(causal_conv(rd(h @ w[p + "q"].T), w[p + "q.conv"]))).reshape(T, G, D)
    k = rd(silu(causal_conv(rd(h @ w[p + "k"].T), w[p + "k.conv"]))).reshape(T, G, D)
    v = rd(silu(causal_conv(rd(h @ w[p + "v"].T), w[p + "v.conv"]))).reshape(T, H, E)
    q = unit(q) * D ** -0.5
    k = unit(k)
    rep = H // G
    q = q.repeat_interleave(rep, dim=1)
    k = k.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(rd(h @ w[p + "b"].T))
    g = delta_decay(h, w[p + "a"], w[p + "A_log"], w[p + "dt_bias"])
    o, _ = delta_recurrence(q, k, v, g, beta)
    o = rms(o, eps) * w[p + "norm"]
    o = rd(o * silu(rd(h @ w[p + "g"].T)).reshape(T, H, E))
    return rd(o.reshape(T, H * E) @ w[p + "o"].T)


# --------------------------------------------------------------------------- mixer: attention
def query_temperature(T: int, coef: float, every: int, dtype) -> torch.Tensor:
    """[T]: 1 + coef * ln(floor((p + 1) / every) + 1)."""
    pos = torch.arange(T)
    return (1.0 + coef * torch.log((torch.div(pos + 1, every, rounding_mode="floor") + 1).to(dtype))).to(dtype)


def sink_softmax_attention(q, k, v, scale, sink):
    """q [T, H, D], k [T, H, D], v [T, H, E], sink [H]: causal attention whose softmax denominator also holds
    exp(sink_h).  Written position by position."""
    T, H, _ = q.shape
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        for i in range(T):
            s = (k[: i + 1, h] @ q[i, h]) * scale
            top = torch.maximum(s.max(), sink[h])
            e = torch.exp(s - top)
            den = e.sum() + torch.exp(sink[h] - top)
            out[i, h] = (e / den) @ v[: i + 1, h]
    return out


def attention_mixer(h, w, p, m, eps, rd=same):
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rd(h @ w[p + "q"].T).reshape(T, H, D)
    k = rd(h @ w[p + "k"].T).reshape(T, G, D)
    v = rd(h @ w[p + "v"].T).reshape(T, G, E)
    q = norm(q, w[p + "q.norm"], eps)
    k = rd(norm(k, w[p + "k.norm"], eps))
    temp = m.get("q_temp")
    if temp is not None:
        q = q * query_temperature(T, temp["coef"], temp["every"], h.dtype)[:, None, None]
    q = rd(q)
    rep = H // G
    k = k.repeat_interleave(rep, dim=1)
    v = v.repeat_interleave(rep, dim=1)
    o = rd(sink_softmax_attention(q, k, v, m["scale"], w[p + "sink"]))
    return rd(o.reshape(T, H * E) @ w[p + "o"].T)


# --------------------------------------------------------------------------- mixer: selective scan
def selective_scan(x, dt, A, B, C, Dskip, S0=None):
    """x, dt [T, I]; A [I, N]; B, C [T, N]; Dskip [I].  S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;
    y_c = sum_n S[c, n] C_n + Dskip_c x_c."""
    T, I = x.shape
    S = torch.zeros(I, A.shape[1], dtype=x.dtype) if S0 is None else S0.clone()
    y = torch.zeros(T, I, dtype=x.dtype)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + Dskip * x[t]
    return y, S


def mamba_mixer(h, w, p, m, rd=same):
    I, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = rd(h @ w[p + "in"].T)
    x, z = xz[:, :I], xz[:, I:]
    x = rd(silu(causal_conv(x, w[p + "conv"], w[p + "conv.b"])))
    proj = rd(x @ w[p + "x"].T)
    dt, B, C = proj[:, :R], proj[:, R:R + N], proj[:, R + N:]
    dt = softplus(dt @ w[p + "dt"].T + w[p + "dt.b"])
    A = -torch.exp(w[p + "A_log"])
    y, _ = selective_scan(x, dt, A, B, C, w[p + "D"])
    return rd(rd(y * silu(z)) @ w[p + "o"].T)


# --------------------------------------------------------------------------- feed-forward
def dense_ff(h, up, down, rd=same):
    return rd(rd(gelu_erf(rd(h @ up.T))) @ down.T)


def route(h, w_router, correction, top: int):
    """Scores s = softmax(h W_router^T) over all outputs; the ``top`` largest of s + correction are chosen; their
    weights are their s, as they are.  Returns (chosen [T, top], weights [T, top])."""
    s = torch.softmax(h @ w_router.T, dim=-1)
    chosen = torch.topk(s + correction, top, dim=-1).indices
    return chosen, torch.gather(s, 1, chosen)


def moe_ff(h, w, p, mlp, rd=same):
    r = mlp["router"]
    n_real, n_id, top = r["experts"], r.get("identity", 0), r["top"]
    chosen, weights = route(h, w[p + "router"], w[p + "correction"], top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(chosen[t, j])
            if e >= n_real:          # the last outputs of the router are identities
                assert e < n_real + n_id
                y = h[t]
            else:
                y = dense_ff(h[t:t + 1], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"], rd)[0]
            out[t] += weights[t, j] * y
    if mlp.get("shared") is not None:
        gate = torch.sigmoid(h @ w[p + "shared.sg"].T)          # [T, 1]
        out = out + gate * dense_ff(h, w[p + "shared.up"], w[p + "shared.down"], rd)
    return out


def feed_forward(h, w, p, mlp, rd=same):
    if mlp["kind"] == "dense":
        return dense_ff(h, w[p + "up"], w[p + "down"], rd)
    if mlp["kind"] == "moe":
        return moe_ff(h, w, p, mlp, rd)
    raise ValueError(mlp["kind"])


# --------------------------------------------------------------------------- the model
def layer_order(cfg: dict):
    """[(layer index, pass number or None when the run does not open a pass)], in running order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None) for i in range(start)]
    for t in range(times):
        for i in range(start, stop):
            order.append((i, t if i == start else None))
    order += [(i, None) for i in range(stop, n)]
    return order


def run_layer(x, i, entry, w, cfg, rd=same):
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    p = f"l{i}."
    h = rd(norm(x, w[p + "norm1"], eps))
    kind = entry["type"]
    if kind == "delta":
        y = delta_mixer(h, w, p + "mix.", entry["mixer"], eps, rd)
    elif kind == "attention":
        y = attention_mixer(h, w, p + "mix.", entry["mixer"], eps, rd)
    elif kind == "mamba1":
        y = mamba_mixer(h, w, p + "mix.", entry["mixer"], rd)
    else:
        raise ValueError(kind)
    x = x + m * norm(y, w[p + "norm1b"], eps)
    if entry.get("mlp") is not None:
        y = feed_forward(rd(norm(x, w[p + "norm2"], eps)), w, p + "mlp.", entry["mlp"], rd)
        x = x + m * norm(y, w[p + "norm2b"], eps)
    return x


def forward(cfg: dict, w: dict, tokens, dtype=torch.float64, layers_out=None, act_dtype=None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  ``layers_out``: a list that receives x after every layer run.  ``act_dtype``:
    round what lies between the products as an engine of that type would (see ``rounder``)."""
    rd = rounder(act_dtype)
    w = {k: v.to(dtype) for k, v in w.items()}
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = w["embed"][ids] * (cfg.get("embedding") or {}).get("scale", 1.0)
    e = x.clone()
    for i, t in layer_order(cfg):
        if t is not None:
            if t > 0:
                x = x + e
            x = x + w["loop.step"][t]
        x = run_layer(x, i, cfg["layers"][i], w, cfg, rd)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rd(norm(x, w["final.norm"], cfg["norm"]["eps"])) @ w["head"].T


def greedy(cfg, w, prompt, n_new, dtype=torch.float64):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(cfg, w, tokens, dtype)[-1].argmax()))
    return tokens[len(prompt):]

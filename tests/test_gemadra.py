"""The Gemadra design against the plain implementation in ``tests/plain/gemadra_plain.py``: every mechanism alone,
then whole models of several small shapes replayed whole, token by token, in portions and in mixed batches (32-bit
and bfloat16 through graphs), and greedy generation through the engine's own entry point."""
import copy
import io
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tests import traces
from tests.plain import gemadra_plain as P


# ================================================================================================ configurations
def delta_layer(heads, kv_heads, dim, vdim, conv, ff, decay_rank=None, gate_rank=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}
    if decay_rank is not None:
        m["decay_rank"], m["gate_rank"] = decay_rank, gate_rank
    return {"type": "channel_delta", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, q_rank, window, ff, base=10000.0, dims=None, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "rot": {"base": base, "dims": rot_dim if dims is None else dims},
         "scale": (dim + rot_dim) ** -0.5 if scale is None else scale}
    if window is not None:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def config(vocab, width, eps, taps, layers):
    return {"architecture": "Gemadra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps},
            "layers": layers}


# Shapes that differ in every size: which mixer comes first, heads that share query/key heads or not, one head, key
# and value sizes that differ, windows that are no multiple of a page, a window of one page, no window, rotation of a
# part of the rotated vector, a layer without a feed-forward, two to five taps.
SHAPES = {
    "P": config(211, 96, 1e-5, 3, [
        latent_layer(3, 16, 8, 24, 40, 28, window=21, ff=160),
        delta_layer(4, 2, 16, 24, conv=2, ff=128),
        latent_layer(2, 24, 12, 16, 48, 20, window=16, ff=None, base=500.0, dims=8),
        delta_layer(1, 1, 40, 12, conv=5, ff=96)]),
    "Q": config(330, 128, 3e-6, 4, [
        delta_layer(6, 3, 24, 40, conv=4, ff=192),
        delta_layer(2, 2, 72, 64, conv=3, ff=None),
        latent_layer(5, 32, 16, 32, 64, 48, window=37, ff=256, base=100000.0),
        latent_layer(4, 16, 32, 48, 96, 32, window=None, ff=128)]),
    "R": config(150, 64, 1e-6, 2, [
        latent_layer(1, 32, 4, 8, 24, 16, window=5, ff=64),
        delta_layer(3, 1, 8, 136, conv=3, ff=72)]),
}
# latents of 128 and 256 entries with rotated parts of 32 and 64: in bfloat16 with pages of 16 these layers' attention
# runs on the matrix cores (seven and three heads: tiles holding several tokens' heads, windows across page borders)
SHAPES["S"] = config(257, 160, 1e-5, 3, [
    latent_layer(7, 16, 32, 24, 128, 40, window=45, ff=192),
    delta_layer(2, 1, 64, 32, conv=4, ff=160),
    latent_layer(3, 32, 64, 16, 256, 24, window=None, ff=128, base=1000.0, dims=48)])
RANKS = {"P": (12, 20), "Q": (16, 8), "R": (5, 7), "S": (8, 8)}      # (decay_rank, gate_rank): config.json leaves them to the shapes


def tensor_shapes(cfg, ranks):
    """Names and shapes, stated here from the design (not asked of the product)."""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (W,)
        out[p + "canon1"] = (W, cfg["canon"]["taps"])
        if layer["type"] == "channel_delta":
            H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            ra, rg = m.get("decay_rank") or ranks[0], m.get("gate_rank") or ranks[1]
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * E)):
                out[p + "mix." + n] = (rows, W)
                out[p + "mix." + n + ".conv"] = (rows, m["conv"])
            out.update({p + "mix.b": (H, W), p + "mix.A_log": (H,), p + "mix.norm": (E,), p + "mix.a1": (ra, W),
                        p + "mix.a2": (H * D, ra), p + "mix.dt_bias": (H * D,), p + "mix.g1": (rg, W),
                        p + "mix.g2": (H * E, rg), p + "mix.o": (W, H * E)})
        else:
            H, D, R, E, C, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out.update({p + "mix.dq": (Q, W), p + "mix.dq.norm": (Q,), p + "mix.uq": (H * (D + R), Q),
                        p + "mix.dkv": (C + R, W), p + "mix.dkv.norm": (C,), p + "mix.uk": (H * D, C),
                        p + "mix.uv": (H * E, C), p + "mix.sink": (H,), p + "mix.g": (H * E, W), p + "mix.o": (W, H * E)})
        if layer["mlp"] is not None:
            F_ = layer["mlp"]["ff"]
            out.update({p + "norm2": (W,), p + "mlp.up": (F_, W), p + "mlp.down": (W, F_), p + "mlp.act": (2,)})
    return out


def random_weights(cfg, ranks, seed, dtype=torch.bfloat16):
    """Weights large enough that every mechanism moves the logits: scores of order one, sinks that take a real
    share, decays between slow and fast, convolution taps of the input's own size."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg, ranks).items():
        leaf = name.split(".")[-1]
        r = torch.randn(shape, generator=g)
        if name in ("embed",):
            t = r
        elif leaf in ("norm1", "norm2") or name == "final.norm":
            t = 0.2 * r                                   # stored around zero
        elif name.endswith("dq.norm") or name.endswith("dkv.norm") or name.endswith("mix.norm"):
            t = 1.0 + 0.2 * r
        elif leaf == "conv" or leaf == "canon1":
            t = 0.5 * r
        elif leaf == "A_log":
            t = -2.0 + r                                  # rates from 0.02 to 1: memories long and short
        elif leaf == "dt_bias":
            t = 0.5 * r
        elif leaf == "sink":
            t = 1.0 + r
        elif leaf == "act":
            t = 0.5 * r
        else:
            t = r * (2.0 / math.sqrt(shape[-1]))
        w[name] = t.to(dtype).contiguous()
    return w


def write_model(folder, cfg, weights):
    import json
    from safetensors.torch import save_file

    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file(weights, str(folder / "model.safetensors"))
    return folder


def requests_for(vocab, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": [int(t) for t in rng.integers(0, vocab, n)] for i, n in enumerate(lengths)}


# ================================================================================================ the oracle's own pins
def test_plain_pieces_against_library_routines():
    torch.manual_seed(0)
    x = torch.randn(9, 6, dtype=torch.float64)
    w = torch.randn(6, 4, dtype=torch.float64)
    # the convolution: torch's, on the sequence padded with taps - 1 zeros at its start
    ref = F.conv1d(F.pad(x.T[None], (3, 0)), w[:, None, :], groups=6)[0].T
    assert torch.allclose(P.causal_conv(x, w), ref, atol=1e-12)
    # the rotation: complex multiplication of neighbouring pairs
    v = torch.randn(5, 3, 8, dtype=torch.float64)
    pos = torch.tensor([0, 1, 7, 30, 1000])
    f = 10000.0 ** (-torch.arange(0, 6, 2, dtype=torch.float64) / 6)
    z = torch.view_as_complex(v[..., :6].reshape(5, 3, 3, 2).contiguous()) * torch.polar(torch.ones(5, 3, dtype=torch.float64),
                                                                                        pos[:, None] * f)[:, None, :]
    got = P.rotate_interleaved(v, pos, 6, 10000.0)
    assert torch.allclose(got[..., :6], torch.view_as_real(z).reshape(5, 3, 6), atol=1e-12)
    assert torch.equal(got[..., 6:], v[..., 6:])
    # xIELU: continuous with slope 1/2 at zero, quadratic on the right
    p, q = torch.tensor(0.3, dtype=torch.float64), torch.tensor(-0.2, dtype=torch.float64)
    e = torch.tensor([1e-7], dtype=torch.float64)
    assert abs(float(P.xielu(e, p, q) - P.xielu(-e, p, q)) / 2e-7 - 0.5) < 1e-5
    assert torch.allclose(P.xielu(torch.tensor([2.0], dtype=torch.float64), p, q), F.softplus(p) * 4 + 1.0)
    # gelu_tanh is torch's
    assert torch.allclose(P.gelu_tanh(x), F.gelu(x, approximate="tanh"), atol=1e-12)


def test_plain_delta_rule_properties():
    """With g = 1 and beta = 1 the rule stores v under a unit key and reads it back exactly; decay halves it."""
    D, E = 5, 3
    k = torch.zeros(2, D, dtype=torch.float64)
    k[0, 1] = k[1, 1] = 1.0
    v = torch.tensor([[1.0, 2.0, 3.0], [0.0, 0.0, 0.0]], dtype=torch.float64)
    q = k.clone()
    one = torch.ones(2, D, dtype=torch.float64)
    out = P.delta_rule(q, k, v, one, torch.tensor([1.0, 0.0], dtype=torch.float64))
    assert torch.allclose(out[0], v[0]) and torch.allclose(out[1], v[0])       # written, then still there
    out = P.delta_rule(q, k, v, one, torch.tensor([1.0, 1.0], dtype=torch.float64))
    assert torch.allclose(out[1], v[1])                                        # overwritten by the second write
    out = P.delta_rule(q, k, v, 0.5 * one, torch.tensor([1.0, 0.0], dtype=torch.float64))
    assert torch.allclose(out[1], 0.5 * v[0])                                  # decayed once before the second read


def test_plain_latent_attention_window_and_sink():
    """One head, keys made so that token t's score against token j is known: the window cuts exactly at
    t - size + 1 and the sink takes its share of the denominator."""
    T, W, C = 6, 4, 4
    m = {"heads": 1, "dim": 2, "rot_dim": 2, "vdim": C, "kv_rank": C, "q_rank": 2, "rot": {"base": 10.0, "dims": 2},
         "mask": {"size": 3}, "scale": 1.0}
    z = lambda *s: torch.zeros(*s, dtype=torch.float64)
    w = {"dq": z(2, W), "dq.norm": torch.ones(2, dtype=torch.float64), "uq": z(4, 2), "dkv": z(C + 2, W),
         "dkv.norm": torch.ones(C, dtype=torch.float64), "uk": z(2, C), "uv": torch.eye(C, dtype=torch.float64),
         "sink": torch.tensor([0.0], dtype=torch.float64), "g": z(C, W), "o": torch.eye(W, C, dtype=torch.float64)}
    w["dkv"][:C, :] = torch.eye(C, W)
    h = torch.eye(T, W, dtype=torch.float64)[:, :W] * 3.0
    h[4:] = torch.tensor([[3.0, 0, 0, 0], [0, 3.0, 0, 0]])
    out = P.latent_attention(h, {"x." + k: v for k, v in w.items()}, "x.", m, 1e-6)
    # all scores are zero: each visible key and the sink weigh the same; the gate is sigmoid(0) = 1/2
    c = P.plain_norm(h @ w["dkv"][:C].T, w["dkv.norm"], 1e-6)
    for t in range(T):
        lo = max(0, t - 2)
        want = c[lo:t + 1].sum(0) / (t + 1 - lo + 1) * 0.5
        assert torch.allclose(out[t], want, atol=1e-12), t


def test_config_reads_every_size_and_refuses_what_it_does_not_know():
    from llm_infrence_engine_amd.config import ConfigError, config_from_dict

    for name, cfg in SHAPES.items():
        c = config_from_dict(copy.deepcopy(cfg))
        assert type(c).__name__ == "GemadraConfig" and c.to_dict() == cfg
        with pytest.raises(ConfigError):          # the low ranks are in no key: the tensors' shapes have them
            c.to_spec()
        shapes = tensor_shapes(cfg, RANKS[name])
        full = c.with_tensor_shapes(lambda n: shapes.get(n))
        from llm_infrence_engine_amd.parts.model import Model

        model = Model(full.to_spec())
        assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == shapes
        needs = model.run_needs()
        for layer, (kv, state, _) in zip(cfg["layers"], needs):
            m = layer["mixer"]
            if layer["type"] == "latent_attention":
                assert [(t.name, t.heads, t.width) for t in kv.tensors[:2]] == [("c", 1, m["kv_rank"]), ("kr", 1, m["rot_dim"])]
                # a transposed copy of the latents only at the sizes the matrix-core kernel has, and only where kept so
                assert [t.name for t in kv.tensors[2:]] == (["ct"] if name == "S" else [])
                assert all(t.only_transposed for t in kv.tensors[2:])
                assert kv.window == (m.get("mask") or {}).get("size")
                assert state.shape == (max(1, cfg["canon"]["taps"] - 1), cfg["width"])
            else:
                assert kv is None and len(state) == 3
                assert state[2].shape == (m["heads"], m["dim"], m["vdim"]) and state[2].dtype == torch.float32
                assert state[1].shape == (m["conv"] - 1, 2 * m["kv_heads"] * m["dim"] + m["heads"] * m["vdim"])
    bad = copy.deepcopy(SHAPES["P"])
    bad["layers"][0]["type"] = "something_else"
    with pytest.raises(ConfigError):
        config_from_dict(bad)
    bad = copy.deepcopy(SHAPES["P"])
    del bad["layers"][1]["mixer"]["vdim"]
    with pytest.raises(ConfigError):
        config_from_dict(bad)
    bad = copy.deepcopy(SHAPES["P"])
    bad["layers"][0]["mlp"]["kind"] = "routed"
    with pytest.raises(ConfigError):
        config_from_dict(bad)


def test_plain_model_prefix_property():
    """The plain model is causal: the logits of a prefix do not change when tokens follow."""
    cfg = SHAPES["R"]
    w = {k: v.double() for k, v in random_weights(cfg, RANKS["R"], 5).items()}
    toks = requests_for(cfg["vocab"], [14], 1)["r0"]
    full = P.forward(cfg, w, toks)
    assert torch.allclose(P.forward(cfg, w, toks[:9]), full[:9], atol=1e-9)


# ================================================================================================ kernels alone (GPU)
gpu = pytest.mark.gpu


class _Ctx:
    """The fields of a step that the kernels of this file read, for requests with the given portion lengths."""

    def __init__(self, q_lens, slots, starts=None, dev="cuda"):
        starts = starts or [0] * len(q_lens)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
        self.num_requests, self.num_tokens = len(q_lens), sum(q_lens)
        self.q_start = i32([0] + list(np.cumsum(q_lens)))
        self.token_req = i32([r for r, n in enumerate(q_lens) for _ in range(n)])
        self.positions = i32([s + t for s, n in zip(starts, q_lens) for t in range(n)])
        self.state_slots = i32(slots)
        self.context_lens = i32([s + n for s, n in zip(starts, q_lens)])
        self.max_q_len = max(q_lens)
        self.n_live_tokens = None


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,mode", [(4, 1), (2, 2), (5, 0), (1, 1)])
def test_short_conv_in_portions_and_batches(dtype, taps, mode):
    """Three sequences fed in portions of unequal sizes, batched together, from slots that are not in order:
    the same as each sequence convolved whole."""
    from llm_infrence_engine_amd.kernels import ops

    torch.manual_seed(taps)
    C, lens = 70, [23, 9, 14]
    xs = [torch.randn(n, C).to(dtype) for n in lens]
    w = torch.randn(C, taps)
    want = []
    for x in xs:
        y = P.causal_conv(x.double(), w.double())
        want.append({0: y, 1: x.double() + y, 2: F.silu(y)}[mode])
    state = torch.full((6, max(1, taps - 1), C), 7.0, dtype=dtype, device="cuda")   # stale values of earlier users
    slots = [4, 1, 3]
    state[slots] = 0                                                             # a request's slot starts at zero
    cuts = [[2, 5, 1, 15], [9], [1, 1, 1, 11]]
    got = [[] for _ in lens]
    at = [0, 0, 0]
    for step in range(4):
        live = [r for r in range(3) if step < len(cuts[r])]
        q_lens = [cuts[r][step] for r in live]
        ctx = _Ctx(q_lens, [slots[r] for r in live])
        x = torch.cat([xs[r][at[r]:at[r] + cuts[r][step]] for r in live]).cuda()
        wide = torch.zeros(x.shape[0], C + 6, dtype=dtype, device="cuda")           # rows as slices of wider rows
        wide[:, 3:3 + C] = x
        out = ops.short_conv(wide[:, 3:3 + C], w.cuda(), state, ctx, torch.empty(x.shape[0], C, dtype=dtype, device="cuda"), mode)
        o = 0
        for r in live:
            got[r].append(out[o:o + cuts[r][step]].cpu())
            o += cuts[r][step]
            at[r] += cuts[r][step]
    tol = 1e-5 if dtype == torch.float32 else 6e-2
    for r in range(3):
        assert (torch.cat(got[r]).double() - want[r]).abs().max() < tol
    assert (state[[0, 2, 5]] == 7.0).all()                                        # nobody else's slot was touched


def _delta_inputs(T, H, G, D, E, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g)
    return dict(q=r(T, G * D), k=r(T, G * D), v=r(T, H * E), a=r(T, H * D), b=r(T, H), A_log=-1.5 + r(H), dt_bias=0.5 * r(H * D))


def _plain_delta(x, H, G, D, E):
    T = x["q"].shape[0]
    d = {k: v.double() for k, v in x.items()}
    q, k = d["q"].reshape(T, G, D), d["k"].reshape(T, G, D)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    gdec = torch.exp(-torch.exp(d["A_log"])[None, :, None] * F.softplus(d["a"].reshape(T, H, D) + d["dt_bias"].reshape(H, D)))
    beta = torch.sigmoid(d["b"])
    v = d["v"].reshape(T, H, E)
    return torch.stack([P.delta_rule(q[:, i // (H // G)], k[:, i // (H // G)], v[:, i], gdec[:, i], beta[:, i])
                        for i in range(H)], dim=1).reshape(T, H * E)


@gpu
@pytest.mark.parametrize("H,G,D,E", [(4, 2, 16, 24), (1, 1, 40, 12), (3, 1, 8, 136), (2, 2, 128, 128), (2, 1, 72, 64),
                                     (1, 1, 200, 70), (2, 2, 1, 1)])
def test_gated_delta_against_the_plain_recurrence(H, G, D, E):
    """A sequence in one portion, and the same sequence in portions beside another request: same outputs, same state."""
    from llm_infrence_engine_amd.kernels import ops

    T = 45
    x = _delta_inputs(T, H, G, D, E, seed=H * 100 + D)
    want = _plain_delta(x, H, G, D, E)
    dev = {k: v.cuda() for k, v in x.items()}
    qkv = torch.cat([dev["q"], dev["k"], dev["v"]], dim=1)
    qk = G * D

    def run(state, ctx, rows):
        out = torch.empty(len(rows), H * E, device="cuda")
        sub = qkv[rows].contiguous()
        ops.gated_delta(sub[:, :qk], sub[:, qk:2 * qk], sub[:, 2 * qk:], dev["a"][rows].contiguous(),
                        dev["b"][rows].contiguous(), dev["A_log"], dev["dt_bias"], state, ctx, out, H, G, D, E)
        return out

    state = torch.zeros(5, H, D, E, device="cuda")
    whole = run(state, _Ctx([T], [2]), list(range(T)))
    assert (whole.cpu().double() - want).abs().max() < 2e-5
    # portions 1, 17, 2, 25 in slot 3, beside the same sequence fed 20 + 25 in slot 0: both must equal the whole run
    state2 = torch.zeros(5, H, D, E, device="cuda")
    got_a, got_b = [], []
    a_cuts, b_cuts = [1, 17, 2, 25], [20, 25, 0, 0]
    pa = pb = 0
    for ca, cb in zip(a_cuts, b_cuts):
        rows = list(range(pa, pa + ca)) + list(range(pb, pb + cb))
        lens, slots = ([ca, cb], [3, 0]) if cb else ([ca], [3])
        out = run(state2, _Ctx(lens, slots), rows)
        got_a.append(out[:ca])
        got_b.append(out[ca:])
        pa, pb = pa + ca, pb + cb
    assert (torch.cat(got_a) - whole).abs().max() < 1e-5 and (torch.cat(got_b) - whole).abs().max() < 1e-5
    assert (state2[3] - state[2]).abs().max() < 1e-5 and (state2[0] - state[2]).abs().max() < 1e-5
    assert (state2[[1, 2, 4]] == 0).all()


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_head_norm_activation_rotation_and_head_products(dtype):
    from llm_infrence_engine_amd.kernels import ops

    torch.manual_seed(3)
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    N, H, E = 11, 3, 20
    o, wn, gate = torch.randn(N, H * E), 1 + 0.2 * torch.randn(E), torch.randn(N, H * E).to(dtype)
    want = (P.plain_norm(o.double().reshape(N, H, E), wn.double(), 1e-5) * torch.sigmoid(gate.double().reshape(N, H, E))).reshape(N, -1)
    got = ops.gated_head_norm(o.cuda(), wn.cuda(), gate.cuda(), torch.empty(N, H * E, dtype=dtype, device="cuda"), H, E, 1e-5)
    assert (got.cpu().double() - want).abs().max() < tol
    # xIELU on both sides of zero
    z = (3 * torch.randn(7, 33)).to(dtype)
    pq = torch.tensor([0.4, -0.3])
    got = ops.xielu(z.cuda(), pq.cuda(), torch.empty_like(z, device="cuda"))
    want = P.xielu(z.double(), pq[0].double(), pq[1].double())
    assert ((got.cpu().double() - want).abs() / (1 + want.abs())).max() < tol
    # rotation of neighbouring pairs inside a slice of wider heads, part of the slice left alone
    x = torch.randn(N, H, 30).to(dtype)
    pos = torch.tensor([0, 1, 2, 3, 50, 51, 400, 1000, 1001, 5000, 7], dtype=torch.int32)
    inv = (100.0 ** (-torch.arange(0, 6, 2, dtype=torch.float64) / 6)).float()
    dst = torch.zeros(N, H, 12, dtype=dtype, device="cuda")
    ops.rotary_pairs(x.cuda()[:, :, 20:30], dst[:, :, 1:11], pos.cuda(), inv.cuda())
    want = P.rotate_interleaved(x[:, :, 20:30].double(), pos, 6, 100.0)
    assert (dst[:, :, 1:11].cpu().double() - want).abs().max() < (2e-4 if dtype == torch.float32 else tol)
    assert (dst[:, :, 0] == 0).all() and (dst[:, :, 11] == 0).all()
    # per-head products with and without a gate, into a slice of a wider output
    I, J = 18, 37
    a, m, g = torch.randn(N, H, I).to(dtype), torch.randn(H, I, J).to(dtype), torch.randn(N, H * J).to(dtype)
    out = torch.zeros(N, H, J + 5, dtype=dtype, device="cuda")
    ops.head_matmul(a.cuda(), m.cuda(), out[:, :, :J], gate=g.cuda())
    want = torch.einsum("nhi,hij->nhj", a.double(), m.double()) * torch.sigmoid(g.double().reshape(N, H, J))
    assert ((out[:, :, :J].cpu().double() - want).abs() / (1 + want.abs())).max() < tol and (out[:, :, J:] == 0).all()


def _latent_setup(dtype, page, C, R, lens, n_pages=64, transposed_copy=False):
    """Pages and a table for requests of the given lengths, filled by the store kernel from random rows."""
    from llm_infrence_engine_amd.kernels import ops
    from llm_infrence_engine_amd.parts.base import KVView

    g = torch.Generator().manual_seed(11)
    c_pages = torch.full((n_pages, 1, page, C), 9.0, dtype=dtype, device="cuda")     # what earlier users left
    r_pages = torch.full((n_pages, 1, page, R), 9.0, dtype=dtype, device="cuda")
    width = max(-(-n // page) for n in lens)
    table = torch.zeros(len(lens) + 1, width, dtype=torch.int32)
    order = list(torch.randperm(n_pages - 1, generator=g).numpy() + 1)             # pages in no order
    rows = []
    for r, n in enumerate(lens):
        for p in range(-(-n // page)):
            table[r, p] = int(order.pop())
        rows.append(torch.randn(n, C + R, generator=g).to(dtype))
    kv = KVView({"c": c_pages, "kr": r_pages}, {"c": False, "kr": False}, table.cuda(), None, True, None, None)
    if transposed_copy:      # what the pool keeps beside the latents for the matrix-core kernel
        kv.pages["ct"] = torch.full((n_pages, 1, C, page), 9.0, dtype=dtype, device="cuda")
        kv.transposed["ct"] = True
    return kv, rows, ops


@gpu
@pytest.mark.parametrize("dtype,C,R", [(torch.float32, 24, 6), (torch.bfloat16, 24, 6), (torch.bfloat16, 128, 32),
                                       (torch.bfloat16, 256, 64)])
@pytest.mark.parametrize("page,window", [(16, 21), (8, 16), (4, None), (16, 1), (32, None), (16, 33)])
def test_latent_attention_window_edges_sink_and_pages(dtype, C, R, page, window):
    """Keys are made so that exactly one key has a large score with a query: the key just inside the window must
    carry the output, the key just outside must not be seen at all, in a prompt's portion and for a single token,
    also where the edge falls on a page's border; without such a key the sink takes its share."""
    H = 3 if C < 128 else 7          # the larger sizes run on the matrix cores where the pages allow (7 heads: tiles
    lens = [70, 33]                  # that hold the heads of several tokens, and a last tile filled in part)
    matrix_cores = C >= 128 and page % 16 == 0
    kv, rows, ops = _latent_setup(dtype, page, C, R, lens, transposed_copy=matrix_cores)
    w_norm = torch.ones(C)
    inv = (1000.0 ** (-torch.arange(0, R, 2, dtype=torch.float64) / R)).float()
    # a loud feature in column 0 of the latent of chosen tokens of request 0
    loud = {}
    for t in (5, 20, 31, 48, 49, 63):
        rows[0][t] = 0.05 * rows[0][t]
        rows[0][t, 0] = 40.0
        loud[t] = True
    for r, x in enumerate(rows):
        n = x.shape[0]
        slot = torch.tensor([int(kv.block_table[r, t // page]) * page + t % page for t in range(n)], dtype=torch.int32)
        ops.latent_kv_store(x.cuda(), w_norm.cuda(), 1e-6, torch.arange(n, dtype=torch.int32).cuda(), inv.cuda(), slot.cuda(),
                            kv.pages["c"], kv.pages["kr"], kv.pages.get("ct"))
    if matrix_cores:
        for r, n in enumerate(lens):                      # the transposed copy holds what the latents' pages hold
            for t in (0, n // 2, n - 1):
                pg, off = int(kv.block_table[r, t // page]), t % page
                assert torch.equal(kv.pages["ct"][pg, 0, :, off], kv.pages["c"][pg, 0, off, :])
    c = [P.plain_norm(x[:, :C].double(), w_norm.double(), 1e-6) for x in rows]
    kr = [P.rotate_interleaved(x[:, C:].double(), torch.arange(x.shape[0]), R, 1000.0) for x in rows]
    sink = torch.tensor([0.5, -1.0, 2.0, 0.0, 1.0, -3.0, 4.0])[:H]
    scale = 0.3 if C < 128 else 0.3 * (30 / (C + R)) ** 0.5

    def plain(r, t, q):
        lo = 0 if window is None else max(0, t - window + 1)
        keys = torch.cat([c[r][lo:t + 1], kr[r][lo:t + 1]], dim=1)
        s = keys @ q.double().T * scale                                  # [keys, H]
        top = torch.maximum(s.max(0).values, sink.double())
        e = torch.exp(s - top)
        return (e.T @ c[r][lo:t + 1]) / (e.sum(0) + torch.exp(sink.double() - top))[:, None]

    tol = 3e-5 if dtype == torch.float32 else 5e-2
    # one step: a portion of request 0 (tokens 40..69) beside the last token of request 1
    before = ops.launches.get("latent_attention_mfma", 0)
    toks = [(0, t) for t in range(40, 70)] + [(1, 32)]
    q = (0.5 * torch.randn(len(toks), H, C + R)).to(dtype)
    q[:, 0, 0] = 8.0 * 0.3 / scale                                       # head 0 listens for the loud feature
    ctx = _Ctx([30, 1], [0, 1], starts=[40, 32])
    out = ops.latent_attention(q.cuda(), kv, ctx, torch.empty(len(toks), H, C, dtype=dtype, device="cuda"), scale, window, sink.cuda())
    for i, (r, t) in enumerate(toks):
        assert (out[i].cpu().double() - plain(r, t, q[i])).abs().max() < tol, (r, t)
    if window is not None and window > 1:
        # token 48 + window - 1 still sees the loud key 48 (and 49); the next one has lost 48
        t_in = 48 + window - 1
        if 40 <= t_in < 69:
            seen = out[t_in - 40, 0, 0].item()
            assert seen > 0.85 * float(c[0][48, 0])
    # single tokens at every place around the edges, each alone (a decoded token)
    for t in sorted({0, 1, 5, 6, 20, 31, 32, 47, 48, 49, 63, 64, 69} | ({5 + window - 1, 5 + window} if window else set())):
        if t >= 70:
            continue
        q1 = (0.5 * torch.randn(1, H, C + R)).to(dtype)
        q1[:, 0, 0] = 8.0 * 0.3 / scale
        o = ops.latent_attention(q1.cuda(), kv, _Ctx([1], [0], starts=[t]), torch.empty(1, H, C, dtype=dtype, device="cuda"),
                                 scale, window, sink.cuda())
        assert (o[0].cpu().double() - plain(0, t, q1[0])).abs().max() < tol, t
    assert (ops.launches.get("latent_attention_mfma", 0) > before) == (matrix_cores and dtype == torch.bfloat16)
    # without a sink the weights sum to one
    ones = ops.latent_attention(q.cuda(), kv, ctx, torch.empty(len(toks), H, C, dtype=dtype, device="cuda"), scale, window, None)
    assert torch.isfinite(ones).all()


# ================================================================================================ whole models (GPU)
F32_ATOL = 2e-3
BF16_NOISE = 3.0
PAGES = {"P": 16, "Q": 8, "R": 4, "S": 16}


def rounded_forward(cfg, w, toks):
    """(exact logits, how far the plain model strays from them when its activations are rounded to bfloat16): a
    faithful reduced-precision computation's own error, of which the bfloat16 path's bound is a multiple."""
    exact = P.forward(cfg, w, toks)
    return exact, float((P.forward(cfg, w, toks, act_dtype=torch.bfloat16) - exact).abs().max())


@pytest.fixture(scope="module", params=list(SHAPES))
def shape(request, tmp_path_factory):
    name = request.param
    cfg = SHAPES[name]
    weights = random_weights(cfg, RANKS[name], seed=ord(name))
    folder = write_model(tmp_path_factory.mktemp("gemadra" + name), cfg, weights)
    lengths = {"P": [5, 61, 2, 130, 33, 48], "Q": [1, 9, 90, 47, 150, 64], "R": [3, 26, 70, 17, 2, 41, 60, 33],
               "S": [70, 3, 140, 50, 97, 33]}[name]
    reqs = requests_for(cfg["vocab"], lengths, seed=ord(name))
    w64 = {k: v.double() for k, v in weights.items()}
    want, noise = {}, {}
    for rid, toks in reqs.items():
        want[rid], noise[rid] = rounded_forward(cfg, w64, toks)
        want[rid] = want[rid].numpy()
    return name, cfg, folder, reqs, want, noise


def _replay(folder, dtype, steps, out, max_tokens, page):
    from llm_infrence_engine_amd.engine.trace import replay

    log = io.StringIO()
    runner = replay(folder, dtype, out, max_tokens, traces.to_lines(steps), log=log, page_size=page)
    assert log.getvalue().split() == [x for st in steps for x in ("done", str(st["step"]))]
    runner.manager.check_invariants()
    assert all(g.allocator.num_in_use() == 0 for g in runner.manager.groups), "a finished request kept pages"
    assert runner.manager.num_requests() == 0
    if dtype == "bfloat16":
        assert runner.graphs is not None and runner.graphs.launches > 0      # the serving path: steps replay from graphs
    return runner


def _compare(got, want, noise, dtype):
    assert got
    for (rid, pos), row in got.items():
        err = np.abs(row.astype(np.float64) - want[rid][pos]).max()
        bound = F32_ATOL if dtype == "float32" else BF16_NOISE * max(noise[rid], 0.02)
        assert err < bound, f"request {rid} position {pos}: max |dlogit| {err:.3e} >= {bound:.3e}"


@gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "bulk_then_single", "changing_portions", "mixed"])
def test_replay_against_plain(shape, tmp_path, dtype, mode):
    name, cfg, folder, reqs, want, noise = shape
    page = PAGES[name]
    up = lambda n: -(-n // 64) * 64
    if mode == "mixed":
        # room for the two longest requests only: pages and state slots are handed out again and again
        max_tokens = sum(sorted(up(len(t)) for t in reqs.values())[-2:])
        steps = traces.mixed(reqs, max_tokens, seed=3, max_live=4, tail=20)
    else:
        max_tokens = max(up(len(t)) for t in reqs.values())
        steps = {"whole": traces.whole, "bulk_then_single": lambda r: traces.bulk_then_single(r, tail=45),
                 "changing_portions": traces.changing_portions}[mode](reqs)
    from llm_infrence_engine_amd.kernels import ops

    before = ops.launches.get("latent_attention_mfma", 0)
    runner = _replay(folder, dtype, steps, tmp_path / "out", max_tokens, page)
    if mode == "whole":      # launched kernel by kernel or captured, the shape S's attention is the matrix cores' in bfloat16
        assert (ops.launches.get("latent_attention_mfma", 0) > before) == (name == "S" and dtype == "bfloat16")
    _compare(traces.collect(steps, tmp_path / "out", cfg["vocab"]), want, noise, dtype)
    if mode == "mixed":
        for g in runner.manager.groups:
            assert g.allocator.pages_granted_again() > 0


@gpu
def test_portions_and_batches_change_nothing_in_32_bit(shape, tmp_path):
    """The logits at a position do not depend on how the prompt was cut or on what else was in the batch, beyond
    rounding: whole against portions against mixed, directly (not through the oracle)."""
    name, cfg, folder, reqs, want, noise = shape
    page = PAGES[name]
    up = lambda n: -(-n // 64) * 64
    outs = {}
    for mode, steps in (("whole", traces.whole(reqs)), ("portions", traces.changing_portions(reqs, sizes=(2, 3, 2, 31, 5, 2))),
                        ("mixed", traces.mixed(reqs, sum(up(len(t)) for t in reqs.values()), seed=9, tail=10))):
        _replay(folder, "float32", steps, tmp_path / mode, sum(up(len(t)) for t in reqs.values()), page)
        outs[mode] = traces.collect(steps, tmp_path / mode, cfg["vocab"])
    for mode in ("portions", "mixed"):
        for key, row in outs[mode].items():
            assert np.abs(row - outs["whole"][key]).max() < 2e-4, (mode, key)


@gpu
def test_one_row_and_few_pages_serve_every_request_in_turn(shape):
    """An engine with a single request row and pages for one request: every request gets the state slot and the pages
    its predecessor left, in portions, and must start from zero state and see none of the old keys."""
    from llm_infrence_engine_amd.engine.batch import StepEntry
    from llm_infrence_engine_amd.engine.runner import load_runner

    name, cfg, folder, reqs, want, noise = shape
    page = PAGES[name]
    longest = max(len(t) for t in reqs.values())
    runner = load_runner(folder, dtype="float32", page_size=page, num_pages=-(-longest // page) + 1, max_requests=1,
                         max_len=-(-longest // page) * page)
    for rid, toks in reqs.items():
        cut = max(1, len(toks) // 2)
        first = runner.step([StepEntry(rid, toks[:cut], list(range(cut)))])
        assert runner.manager.row(rid) == 0
        got = [first.cpu().numpy()]
        if cut < len(toks):
            got.append(runner.step([StepEntry(rid, toks[cut:], list(range(len(toks) - cut)))]).cpu().numpy())
        runner.free_request(rid)
        assert np.abs(np.concatenate(got) - want[rid]).max() < F32_ATOL, rid
    runner.manager.check_invariants()
    assert all(g.allocator.pages_granted_again() > 0 for g in runner.manager.groups)


@gpu
def test_far_token_reaches_the_end_through_the_state(tmp_path):
    """A token 400 places back, far outside every window, still moves the last logits (the delta rule's state
    carries it), in the plain model and equally in the engine, whole and decoded token by token."""
    cfg = config(97, 64, 1e-5, 2, [delta_layer(2, 1, 128, 16, conv=2, ff=64), latent_layer(2, 16, 8, 16, 32, 16, window=9, ff=64)])
    ranks = (6, 6)
    weights = random_weights(cfg, ranks, seed=1)
    for k in weights:
        if k.endswith("A_log"):
            weights[k] = torch.full_like(weights[k], -7.0)          # a memory of about a thousand tokens
    folder = write_model(tmp_path / "m", cfg, weights)
    w64 = {k: v.double() for k, v in weights.items()}
    rng = np.random.default_rng(5)
    a = [int(t) for t in rng.integers(0, 97, 420)]
    b = list(a)
    b[7] = (b[7] + 50) % 97
    la, lb = P.forward(cfg, w64, a)[-1].numpy(), P.forward(cfg, w64, b)[-1].numpy()
    assert np.abs(la - lb).max() > 0.01, "the test's weights forget too fast to show anything"
    reqs = {"a": a, "b": b}
    for mode, steps in (("whole", traces.whole(reqs)), ("single", traces.bulk_then_single(reqs, tail=380))):
        _replay(folder, "float32", steps, tmp_path / mode, 2 * 448, 16)
        got = traces.collect(steps, tmp_path / mode, 97)
        assert np.abs(got[("a", 419)] - la).max() < 5e-4 and np.abs(got[("b", 419)] - lb).max() < 5e-4


@gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(shape, dtype):
    """``LLM.generate``: scheduler, prompt portions, continuous batching, graphs in bfloat16.  Every emitted token is
    the plain model's choice at its place, or within rounding of it."""
    import llm_infrence_engine_amd as eng

    name, cfg, folder, reqs, want, noise = shape
    weights = {k: v.double() for k, v in random_weights(cfg, RANKS[name], seed=ord(name)).items()}
    prompts = [toks[:max(1, len(toks) // 3)] for toks in list(reqs.values())[:4]]
    llm = eng.LLM(str(folder), dtype=dtype, block_size=PAGES[name], max_len=128, max_seqs=3,
                  max_prefill_chunk=7)
    outs = llm.generate(prompts, eng.SamplingParams(max_new_tokens=12))
    slack = 2 * F32_ATOL if dtype == "float32" else None
    for p, o in zip(prompts, outs):
        assert len(o.token_ids) == 12 and o.finish_reason == "length"
        logits = P.forward(cfg, weights, p + o.token_ids)[len(p) - 1:-1]
        for t, row in zip(o.token_ids, logits):
            gap = float(row.max() - row[t])
            assert gap <= (slack if slack is not None else BF16_NOISE * max(max(noise.values()), 0.02)), (name, dtype, gap)
    m = llm.engine.runner.manager
    m.check_invariants()
    assert all(g.allocator.num_in_use() == 0 for g in m.groups) and m.num_requests() == 0
    if dtype == "bfloat16":
        # four decode steps to a graph launch, each fed the token the one before chose on the device: the same tokens
        del llm
        several = eng.LLM(str(folder), dtype=dtype, block_size=PAGES[name], max_len=128, max_seqs=3, max_prefill_chunk=7,
                          decode_steps_per_launch=4)
        again = several.generate(prompts, eng.SamplingParams(max_new_tokens=12))
        assert [o.token_ids for o in again] == [o.token_ids for o in outs]


@gpu
def test_command_line_generates(shape):
    import subprocess
    import sys

    from tests.conftest import ROOT

    name, cfg, folder, reqs, want, noise = shape
    r = subprocess.run([sys.executable, "-m", "llm_infrence_engine_amd", "--model", str(folder), "--dtype", "float32",
                        "--prompt-ids", "5,17,3", "--max-new-tokens", "4"], cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]

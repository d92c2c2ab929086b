"""The Gidurax design against the plain implementation in ``tests/plain/gidurax_plain.py``: every mechanism alone,
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
from tests.plain import gidurax_plain as P


# ================================================================================================ configurations
def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, identity=None, shared=None):
    r = {"experts": experts, "top": top}
    if identity is not None:
        r["identity"] = identity
    return {"kind": "moe", "expert": {"ff": ff}, "router": r, "shared": None if shared is None else {"ff": shared}}


def delta_layer(heads, kv_heads, dim, vdim, conv, mlp):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def attention_layer(heads, kv_heads, dim, vdim, scale, mlp, temp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if temp is not None:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def mamba_layer(inner, state, dt_rank, conv, mlp):
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}, "mlp": mlp}


def config(vocab, width, eps, mult, scale, layers, loop=None):
    c = {"architecture": "Gidurax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
         "embedding": {"scale": scale}, "layers": layers}
    if loop is not None:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


# Shapes that differ in every size and in the order of their layers: a looped stretch at the start, in the middle
# (behind a layer that runs once) and none; attention inside the loop (a cache per pass); key and value sizes that
# differ; one key/value head, as many as query heads, groups of three; temperatures with short periods so that several
# steps of the logarithm fall into a prompt; 2 to 5 taps; state sizes that are no power of two; experts with and without
# identities and a shared expert, a top of one; a layer without a feed-forward.
SHAPES = {
    "P": config(211, 96, 1e-5, 0.6, 4.0, [
        mamba_layer(64, 8, 5, 3, dense(128)),
        attention_layer(6, 2, 16, 24, 0.3, moe(40, 5, 2, identity=2, shared=56), temp=(0.4, 16)),
        delta_layer(4, 2, 16, 24, 2, None),
        attention_layer(3, 3, 32, 32, 0.2, dense(72))], loop=(0, 2, 2)),
    "Q": config(330, 128, 3e-6, 1.0, 11.3, [
        delta_layer(6, 3, 24, 40, 4, moe(64, 7, 1)),
        mamba_layer(80, 20, 7, 5, moe(48, 4, 3, identity=1, shared=None)),
        delta_layer(2, 2, 72, 64, 3, dense(192)),
        attention_layer(4, 1, 64, 64, 0.125, dense(200), temp=(0.25, 7)),
        mamba_layer(96, 33, 4, 2, dense(96))], loop=(1, 4, 3)),
    "R": config(150, 64, 1e-6, 0.85, 1.0, [
        attention_layer(2, 1, 8, 40, 0.4, moe(24, 3, 2, identity=0, shared=32)),
        delta_layer(3, 1, 8, 136, 3, dense(72)),
        mamba_layer(40, 130, 3, 4, None)]),
}
# heads of 64 with pages of 16: in bfloat16 this attention runs on the matrix cores
SHAPES["S"] = config(257, 160, 1e-5, 0.75, 12.6, [
    attention_layer(6, 2, 64, 64, 0.11, moe(64, 6, 2, identity=1, shared=64), temp=(0.35, 32)),
    mamba_layer(192, 16, 6, 4, dense(192)),
    attention_layer(4, 4, 32, 32, 0.18, dense(128))], loop=(0, 1, 2))
PAGES = {"P": 16, "Q": 8, "R": 4, "S": 16}
# seeds of the shapes' weights.  A router's choice is a comparison of floats: with some weights a token's last chosen and
# first unchosen expert lie closer together than bfloat16 activations can tell apart, and the two precisions then run
# different experts for that token, which no bound on rounding covers; these seeds have no such token in the tests' requests
SEEDS = {"P": ord("P"), "Q": ord("Q"), "R": ord("R"), "S": 1001}


def tensor_shapes(cfg):
    """Names and shapes, stated here from the design (not asked of the product)."""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    if cfg.get("loop"):
        out["loop.step"] = (cfg["loop"]["times"], W)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (W,)
        if layer["type"] == "delta":
            H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * E)):
                out[p + "mix." + n] = (rows, W)
                out[p + "mix." + n + ".conv"] = (rows, m["conv"])
            out.update({p + "mix.b": (H, W), p + "mix.A_log": (H,), p + "mix.norm": (E,), p + "mix.a": (H, W),
                        p + "mix.dt_bias": (H,), p + "mix.g": (H * E, W), p + "mix.o": (W, H * E)})
        elif layer["type"] == "attention":
            H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * D, W), p + "mix.k": (G * D, W), p + "mix.v": (G * E, W), p + "mix.q.norm": (D,),
                        p + "mix.k.norm": (D,), p + "mix.sink": (H,), p + "mix.o": (W, H * E)})
        else:
            I, N, R = m["inner"], m["state"], m["dt_rank"]
            out.update({p + "mix.in": (2 * I, W), p + "mix.conv": (I, m["conv"]), p + "mix.conv.b": (I,),
                        p + "mix.x": (R + 2 * N, I), p + "mix.dt": (I, R), p + "mix.dt.b": (I,), p + "mix.A_log": (I, N),
                        p + "mix.D": (I,), p + "mix.o": (W, I)})
        mlp = layer["mlp"]
        if mlp is None:
            continue
        out[p + "norm2"] = out[p + "norm2b"] = (W,)
        if mlp["kind"] == "dense":
            out.update({p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
        else:
            r, F_ = mlp["router"], mlp["expert"]["ff"]
            for e in range(r["experts"]):
                out.update({f"{p}mlp.e{e}.up": (F_, W), f"{p}mlp.e{e}.down": (W, F_)})
            n_out = r["experts"] + (r.get("identity") or 0)
            out.update({p + "mlp.router": (n_out, W), p + "mlp.correction": (n_out,)})
            if mlp.get("shared"):
                S_ = mlp["shared"]["ff"]
                out.update({p + "mlp.shared.up": (S_, W), p + "mlp.shared.down": (W, S_), p + "mlp.shared.sg": (1, W)})
    return out


def random_weights(cfg, seed, dtype=torch.bfloat16):
    """Weights large enough that every mechanism moves the logits: scores of order one, sinks that take a real share,
    decays between slow and fast, routers that spread their choices, corrections that change them."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        r = torch.randn(shape, generator=g)
        if name == "embed":
            t = r / max(1.0, cfg["embedding"]["scale"])
        elif name == "loop.step":
            t = 0.5 * r
        elif leaf in ("norm1", "norm2", "norm1b", "norm2b", "norm") or name == "final.norm":
            t = 1.0 + 0.2 * r
        elif leaf in ("conv",):
            t = 0.5 * r
        elif leaf == "A_log":
            t = (-2.0 + r) if len(shape) == 1 else (-1.0 + 0.7 * r)
        elif name.endswith("conv.b") or leaf in ("dt_bias", "correction"):
            t = 0.3 * r
        elif name.endswith("dt.b"):
            t = -1.5 + 0.5 * r
        elif leaf == "D":
            t = 1.0 + 0.3 * r
        elif leaf == "sink":
            t = 1.0 + r
        elif leaf == "router":
            t = r * (3.0 / math.sqrt(shape[-1]))
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
    b = torch.randn(6, dtype=torch.float64)
    ref = F.conv1d(F.pad(x.T[None], (3, 0)), w[:, None, :], bias=b, groups=6)[0].T
    assert torch.allclose(P.causal_conv(x, w, b), ref, atol=1e-12)
    assert torch.allclose(P.gelu_erf(x), F.gelu(x), atol=1e-12)
    assert torch.allclose(P.silu(x), F.silu(x), atol=1e-12)
    assert torch.allclose(P.softplus(5 * x), F.softplus(5 * x), atol=1e-12)
    assert torch.allclose(P.norm(x, b, 1e-5), F.rms_norm(x, (6,), b, 1e-5), atol=1e-12)
    # with a sink far below every score the attention is the library's causal attention
    q, k, v = (torch.randn(7, 2, 5, dtype=torch.float64) for _ in range(3))
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True, scale=0.3)
    got = P.sink_softmax_attention(q, k, v, 0.3, torch.full((2,), -200.0, dtype=torch.float64))
    assert torch.allclose(got, ref.transpose(0, 1), atol=1e-12)
    # a sink equal to the only score takes half of the first token's weight
    got = P.sink_softmax_attention(torch.zeros(1, 1, 5, dtype=torch.float64), k[:1, :1], v[:1, :1], 1.0,
                                   torch.zeros(1, dtype=torch.float64))
    assert torch.allclose(got[0, 0], 0.5 * v[0, 0])
    # the temperature steps up where floor((p + 1) / every) does
    t = P.query_temperature(10, 0.5, 4, torch.float64)
    assert torch.allclose(t[:3], torch.ones(3, dtype=torch.float64)) and abs(float(t[3]) - (1 + 0.5 * math.log(2))) < 1e-12
    assert abs(float(t[7]) - (1 + 0.5 * math.log(3))) < 1e-12 and float(t[6]) == float(t[3])


def test_plain_recurrences_have_their_closed_forms():
    # the scan with constant inputs is a geometric series
    T, I, N = 6, 2, 3
    dt = torch.full((T, I), 0.5, dtype=torch.float64)
    x = torch.ones(T, I, dtype=torch.float64)
    A = -torch.tensor([[1.0, 2.0, 3.0], [0.5, 0.1, 4.0]], dtype=torch.float64)
    Bm = torch.ones(T, N, dtype=torch.float64) * 2.0
    Cm = torch.ones(T, N, dtype=torch.float64)
    y, S = P.selective_scan(x, dt, A, Bm, Cm, torch.tensor([0.0, 3.0], dtype=torch.float64))
    a = torch.exp(0.5 * A)
    want = (1.0 - a ** T) / (1.0 - a)          # sum of a^j, j < T, times dt x B = 1
    assert torch.allclose(S, want, atol=1e-12)
    assert torch.allclose(y[-1], want.sum(1) + torch.tensor([0.0, 3.0], dtype=torch.float64), atol=1e-12)
    # the delta rule stores v under a unit key and reads it back; a second write under the same key replaces it
    D, E = 5, 3
    k = torch.zeros(2, 1, D, dtype=torch.float64)
    k[:, 0, 1] = 1.0
    v = torch.tensor([[[1.0, 2.0, 3.0]], [[0.0, 0.0, 0.0]]], dtype=torch.float64)
    one = torch.ones(2, 1, dtype=torch.float64)
    out, _ = P.delta_recurrence(k, k, v, one, torch.tensor([[1.0], [0.0]], dtype=torch.float64))
    assert torch.allclose(out[0, 0], v[0, 0]) and torch.allclose(out[1, 0], v[0, 0])
    out, _ = P.delta_recurrence(k, k, v, one, one)
    assert torch.allclose(out[1, 0], v[1, 0])
    out, _ = P.delta_recurrence(k, k, v, 0.5 * one, torch.tensor([[1.0], [0.0]], dtype=torch.float64))
    assert torch.allclose(out[1, 0], 0.5 * v[0, 0])


def test_plain_router_and_loop_order():
    h = torch.eye(3, dtype=torch.float64)
    wr = torch.tensor([[2.0, 0, 0], [1.0, 0, 0], [0.0, 0, 0], [-1.0, 0, 0]], dtype=torch.float64)
    corr = torch.tensor([0.0, 0.0, 0.0, 5.0], dtype=torch.float64)
    chosen, weights = P.route(h[:1], wr, corr, 2)
    s = torch.softmax(torch.tensor([2.0, 1.0, 0.0, -1.0], dtype=torch.float64), 0)
    # the correction brings output 3 in; the weights are the plain scores, not renormalised and without the correction
    assert set(chosen[0].tolist()) == {3, 0}
    assert torch.allclose(weights[0].sort().values, torch.stack([s[3], s[0]]).sort().values)
    # an identity expert returns its input times its weight
    w = {"m.router": wr, "m.correction": corr, "m.e0.up": torch.zeros(2, 3, dtype=torch.float64),
         "m.e0.down": torch.zeros(3, 2, dtype=torch.float64)}
    mlp = {"router": {"experts": 1, "identity": 3, "top": 1}, "shared": None}
    assert torch.allclose(P.moe_ff(h[:1], w, "m.", mlp), s[3] * h[:1])
    cfg = {"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}}
    assert P.layer_order(cfg) == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None), (4, None)]
    assert P.layer_order({"layers": [0, 0]}) == [(0, None), (1, None)]


def test_config_reads_every_size_and_refuses_what_it_does_not_know():
    from llm_infrence_engine_amd.config import ConfigError, config_from_dict
    from llm_infrence_engine_amd.parts.model import Model

    for name, cfg in SHAPES.items():
        c = config_from_dict(copy.deepcopy(cfg))
        assert type(c).__name__ == "GiduraxConfig" and c.to_dict() == cfg
        model = Model(c.to_spec())
        assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == tensor_shapes(cfg)
        order = P.layer_order(cfg)
        assert [(r.layer, r.opens_pass) for r in model.spec.order] == order
        for (i, _), (kv, state, _) in zip(order, model.run_needs()):
            layer = cfg["layers"][i]
            m = layer["mixer"]
            if layer["type"] == "attention":
                assert state is None and kv.window is None
                assert [(t.name, t.heads, t.width) for t in kv.tensors] == [("k", m["kv_heads"], m["dim"]), ("v", m["kv_heads"], m["vdim"])]
            elif layer["type"] == "delta":
                assert kv is None and state[1].shape == (m["heads"], m["dim"], m["vdim"]) and state[1].dtype == torch.float32
                assert state[0].shape == (m["conv"] - 1, 2 * m["kv_heads"] * m["dim"] + m["heads"] * m["vdim"])
            else:
                assert kv is None and state[1].shape == (m["inner"], m["state"]) and state[1].dtype == torch.float32
                assert state[0].shape == (m["conv"] - 1, m["inner"])
        assert model.graph_safe() is True
    for change in (lambda c: c["layers"][0].__setitem__("type", "something_else"),
                   lambda c: c["layers"][1]["mixer"].pop("vdim"),
                   lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"),
                   lambda c: c.__setitem__("loop", {"start": 2, "stop": 2, "times": 2}),
                   lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 99)):
        bad = copy.deepcopy(SHAPES["P"])
        change(bad)
        with pytest.raises(ConfigError):
            config_from_dict(bad)


def test_plain_model_prefix_property():
    """The plain model is causal: the logits of a prefix do not change when tokens follow."""
    cfg = SHAPES["R"]
    w = {k: v.double() for k, v in random_weights(cfg, 5).items()}
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
        self.max_context_len = max(s + n for s, n in zip(starts, q_lens))
        self.n_live_tokens = None


def _in_portions(lens, cuts, slots, run):
    """Feeds three sequences in portions of unequal sizes, batched together: ``run(live, at, q_lens, ctx)`` returns the
    step's rows; returns every sequence's rows put together again."""
    got = [[] for _ in lens]
    at = [0] * len(lens)
    for step in range(max(len(c) for c in cuts)):
        live = [r for r in range(len(lens)) if step < len(cuts[r])]
        q_lens = [cuts[r][step] for r in live]
        out = run(live, list(at), q_lens, _Ctx(q_lens, [slots[r] for r in live], [at[r] for r in live]))
        o = 0
        for r, n in zip(live, q_lens):
            got[r].append(out[o:o + n].cpu())
            o += n
            at[r] += n
    return [torch.cat(g) for g in got]


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_short_conv_with_a_bias(dtype):
    from llm_infrence_engine_amd.kernels import ops

    torch.manual_seed(3)
    C, lens, taps = 70, [23, 9, 14], 4
    xs = [torch.randn(n, C).to(dtype) for n in lens]
    w, b = torch.randn(C, taps), torch.randn(C)
    want = [F.silu(P.causal_conv(x.double(), w.double(), b.double())) for x in xs]
    state = torch.full((6, taps - 1, C), 7.0, dtype=dtype, device="cuda")
    slots = [4, 1, 3]
    state[slots] = 0

    def run(live, at, q_lens, ctx):
        x = torch.cat([xs[r][at[r]:at[r] + n] for r, n in zip(live, q_lens)]).cuda()
        return ops.short_conv(x, w.cuda(), state, ctx, torch.empty_like(x), ops.CONV_SILU, bias=b.cuda())

    got = _in_portions(lens, [[2, 5, 1, 15], [9], [1, 1, 1, 11]], slots, run)
    for g, x in zip(got, want):
        assert (g.double() - x).abs().max() < (1e-5 if dtype == torch.float32 else 6e-2)
    assert (state[[0, 2, 5]] == 7.0).all()


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("I,N", [(70, 8), (33, 3), (64, 16), (40, 24), (20, 64), (18, 130)])
def test_selective_scan_in_portions_and_batches(dtype, I, N):
    """Three sequences in portions down to one token, batched, from slots in no order and with stale values around:
    the same as each scanned whole; a chunk's edge (16 tokens) falls inside the portions."""
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(I * N)
    lens = [45, 9, 23]
    r = lambda *s: torch.randn(*s, generator=g)
    seqs = [dict(x=r(n, I).to(dtype), z=r(n, I).to(dtype), B=r(n, N).to(dtype), C=r(n, N).to(dtype), dt=r(n, I) - 1.0) for n in lens]
    A, D, bias = -torch.exp(-1.0 + 0.7 * r(I, N)), 1.0 + 0.3 * r(I), 0.3 * r(I)
    want = []
    for s in seqs:
        d = {k: v.double() for k, v in s.items()}
        y, _ = P.selective_scan(d["x"], P.softplus(d["dt"] + bias.double()), A.double(), d["B"], d["C"], D.double())
        want.append(y * P.silu(d["z"]))
    state = torch.full((6, I, N), 7.0, device="cuda")
    slots = [4, 1, 3]
    state[slots] = 0

    def run(live, at, q_lens, ctx):
        cat = lambda key: torch.cat([seqs[r_][key][at[r_]:at[r_] + n] for r_, n in zip(live, q_lens)]).cuda()
        bc = torch.cat([cat("B"), cat("C")], dim=1)          # B and C as slices of one row, as the mixer has them
        x = cat("x")
        return ops.selective_scan(x, cat("dt"), bias.cuda(), A.cuda(), bc[:, :N], bc[:, N:], D.cuda(), cat("z"), state, ctx,
                                  torch.empty_like(x))

    got = _in_portions(lens, [[2, 17, 1, 25], [9], [1, 1, 20, 1]], slots, run)
    for gt, wt in zip(got, want):
        scale = float(wt.abs().max())
        assert (gt.double() - wt).abs().max() < (2e-5 if dtype == torch.float32 else 2e-2) * max(1.0, scale)
    assert (state[[0, 2, 5]] == 7.0).all()


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E", [(4, 2, 16, 24), (3, 1, 8, 136), (2, 2, 72, 64), (1, 1, 128, 32)])
def test_delta_rule_with_a_decay_per_head(dtype, H, G, D, E):
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(H * D + E)
    r = lambda *s: torch.randn(*s, generator=g)
    lens = [37, 5, 20]
    seqs = [dict(q=r(n, G * D).to(dtype), k=r(n, G * D).to(dtype), v=r(n, H * E).to(dtype), b=r(n, H).to(dtype), a=r(n, H)) for n in lens]
    A_log, dt_bias = -1.5 + r(H), 0.5 * r(H)
    want = []
    for s in seqs:
        d = {k: v.double() for k, v in s.items()}
        n = d["q"].shape[0]
        q = (P.unit(d["q"].reshape(n, G, D)) * D ** -0.5).repeat_interleave(H // G, dim=1)
        k = P.unit(d["k"].reshape(n, G, D)).repeat_interleave(H // G, dim=1)
        gd = torch.exp(-torch.exp(A_log.double()) * P.softplus(d["a"] + dt_bias.double()))
        o, _ = P.delta_recurrence(q, k, d["v"].reshape(n, H, E), gd, torch.sigmoid(d["b"]))
        want.append(o.reshape(n, H * E))
    state = torch.full((5, H, D, E), 3.0, device="cuda")
    slots = [2, 0, 3]
    state[slots] = 0

    def run(live, at, q_lens, ctx):
        cat = lambda key: torch.cat([seqs[r_][key][at[r_]:at[r_] + n] for r_, n in zip(live, q_lens)]).cuda()
        qkv = torch.cat([cat("q"), cat("k"), cat("v")], dim=1)
        out = torch.empty(qkv.shape[0], H * E, device="cuda")
        return ops.gated_delta(qkv[:, :G * D], qkv[:, G * D:2 * G * D], qkv[:, 2 * G * D:], cat("a"), cat("b"), A_log.cuda(),
                               dt_bias.cuda(), state, ctx, out, H, G, D, E, decay_per_channel=False)

    got = _in_portions(lens, [[2, 16, 1, 18], [5], [1, 1, 17, 1]], slots, run)
    for gt, wt in zip(got, want):
        assert (gt.double() - wt).abs().max() < (2e-5 if dtype == torch.float32 else 2e-2)
    assert (state[[1, 4]] == 3.0).all()


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norms_that_join_the_residual_stream(dtype):
    from llm_infrence_engine_amd.kernels import ops

    torch.manual_seed(1)
    for N, H in ((5, 96), (3, 330), (2, 13000)):
        x, y = torch.randn(N, H), (3 * torch.randn(N, H)).to(dtype)
        w1, w2 = 1 + 0.2 * torch.randn(H), 1 + 0.2 * torch.randn(H)
        nx = x.double() + P.norm(y.double(), w1.double(), 1e-5)
        xg = x.cuda()
        ops.rms_norm_add(y.cuda(), w1.cuda(), 1e-5, xg)
        assert (xg.cpu().double() - nx).abs().max() < 1e-5
        xg = x.cuda()
        out = ops.rms_norm_add(y.cuda(), w1.cuda(), 1e-5, xg, w2.cuda(), 3e-6, torch.empty(N, H, dtype=dtype, device="cuda"))
        assert (xg.cpu().double() - nx).abs().max() < 1e-5
        assert (out.cpu().double() - P.norm(nx, w2.double(), 3e-6)).abs().max() < (1e-5 if dtype == torch.float32 else 4e-2)
    x, kept, vec = torch.randn(4, 50), torch.randn(4, 50), torch.randn(50)
    assert torch.allclose(ops.add_rows(x.cuda(), kept.cuda(), vec.cuda()).cpu(), x + kept + vec, atol=1e-6)
    assert torch.allclose(ops.add_rows(x.cuda(), None, vec.cuda()).cpu(), x + vec, atol=1e-6)
    o = torch.randn(6, 3 * 20)
    gate = torch.randn(6, 3 * 20).to(dtype)
    wn = 1 + 0.2 * torch.randn(20)
    got = ops.gated_head_norm(o.cuda(), wn.cuda(), gate.cuda(), torch.empty(6, 60, dtype=dtype, device="cuda"), 3, 20, 1e-5, "silu")
    want = (P.norm(o.double().reshape(6, 3, 20), wn.double(), 1e-5) * P.silu(gate.double().reshape(6, 3, 20))).reshape(6, 60)
    assert (got.cpu().double() - want).abs().max() < (1e-5 if dtype == torch.float32 else 4e-2)
    e = ops.embed(torch.tensor([2, 0], dtype=torch.int32, device="cuda"), x.to(dtype).cuda(), torch.empty(2, 50, device="cuda"), 7.5)
    assert torch.allclose(e.cpu(), x.to(dtype).float()[[2, 0]] * 7.5, atol=1e-6)
    z = torch.randn(1000).to(dtype)
    assert (ops.gelu(z.cuda(), torch.empty_like(z.cuda())).cpu().double() - P.gelu_erf(z.double())).abs().max() < \
        (1e-6 if dtype == torch.float32 else 2e-2)


def _paged(keys, vals, page, order, dtype, transposed=False):
    """Pages holding one sequence's keys [T, G, D] and values [T, G, E] in the pages ``order`` names, others full of
    stale large values; returns (k_pages, v_pages, table)."""
    T, G, D = keys.shape
    E = vals.shape[2]
    n = -(-T // page)
    P_ = max(order) + 2
    k_pages = torch.full((P_, G, page, D), 50.0, dtype=dtype)
    v_pages = torch.full((P_, G, E, page) if transposed else (P_, G, page, E), 50.0, dtype=dtype)
    for i in range(n):
        rows = slice(i * page, min(T, (i + 1) * page))
        cnt = rows.stop - rows.start
        k_pages[order[i], :, :cnt] = keys[rows].transpose(0, 1).to(dtype)
        if transposed:
            v_pages[order[i], :, :, :cnt] = vals[rows].permute(1, 2, 0).to(dtype)
        else:
            v_pages[order[i], :, :cnt] = vals[rows].transpose(0, 1).to(dtype)
    table = torch.zeros(2, n + 3, dtype=torch.int32)
    table[1, :n] = torch.tensor(order[:n], dtype=torch.int32)
    return k_pages.cuda(), v_pages.cuda(), table.cuda()


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E,page", [(6, 2, 16, 24, 4), (4, 1, 64, 64, 16), (3, 3, 32, 8, 8), (8, 2, 64, 64, 16), (2, 1, 6, 10, 4),
                                          (6, 2, 64, 64, 16), (3, 1, 128, 128, 16), (5, 1, 32, 32, 16)])
def test_attention_with_a_sink_and_a_loud_far_key(dtype, H, G, D, E, page):
    """One sequence of 300 tokens in pages in no order: the last 40 queries attend over everything.  One key far back
    (at a page's last slot) is made loud for one query, so that leaving it out, or being one token off, shows; sinks of
    both signs take their share.  Values may have another size than keys."""
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(D + E)
    T, Tq = 300, 40
    q = torch.randn(T, H, D, generator=g).to(dtype)
    k = torch.randn(T, G, D, generator=g).to(dtype)
    v = torch.randn(T, G, E, generator=g).to(dtype)
    far = 3 * page - 1
    k[far, 0] = (4.0 * q[T - 5, 0].float() / q[T - 5, 0].float().norm()).to(dtype)
    sink = torch.tensor([5.0, -3.0, 4.0, 6.0, -1.0, 0.0, 5.5, 3.0][:H])
    scale = 0.7 / math.sqrt(D)
    rep = H // G
    want = P.sink_softmax_attention(q.double(), k.double().repeat_interleave(rep, 1), v.double().repeat_interleave(rep, 1),
                                    scale, sink.double())[T - Tq:]
    kk, vv = k.double().repeat_interleave(rep, 1), v.double().repeat_interleave(rep, 1)
    without = P.sink_softmax_attention(q.double(), kk, vv, scale, torch.full((H,), -200.0, dtype=torch.float64))[T - Tq:]
    assert (want - without).abs().max() > 0.05          # the sinks matter in this test
    order = list(np.random.default_rng(1).permutation(np.arange(1, 1 + -(-T // page))))
    for transposed in (False, True):
        k_pages, v_pages, table = _paged(k, v, page, order, dtype, transposed)
        ctx = _Ctx([Tq], [0], [T - Tq])

        class KV:
            pass

        kv = KV()
        kv.k_pages, kv.v_pages, kv.v_transposed, kv.block_table = k_pages, v_pages, transposed, table
        kv.table_rows = torch.tensor([1], dtype=torch.int32, device="cuda")
        out = torch.empty(Tq, H * E, dtype=dtype, device="cuda")
        ops.paged_attention(q[T - Tq:].reshape(Tq, H * D).cuda(), kv, ctx, out, H, scale, None, sink.cuda())
        err = (out.cpu().double().reshape(Tq, H, E) - want).abs().max()
        assert err < (2e-5 if dtype == torch.float32 else 3e-2), (transposed, float(err))


@gpu
@pytest.mark.parametrize("H,G,D", [(8, 2, 64), (4, 4, 32), (14, 2, 128)])
def test_sink_attention_when_single_tokens_are_decoded(H, G, D):
    """A step of single tokens in bfloat16 over contexts short and long (beyond the length from which a small batch's
    keys are split over blocks and combined): the matrix-core kernels with the sink, against the plain attention."""
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(H + D)
    page, lens = 16, [1300, 40, 700]
    sink = torch.tensor([4.0, -3.0, 6.0, 7.0, -1.0, 0.0, 5.5, 3.0, 1.0, 2.0, 8.0, -2.0, 4.5, 6.5][:H])
    scale, rep = 1.1 / math.sqrt(D), H // G
    qs, want, tables, kps, vps, base = [], [], [], [], [], 1
    for T in lens:
        q = torch.randn(1, H, D, generator=g).bfloat16()
        k = torch.randn(T, G, D, generator=g).bfloat16()
        v = torch.randn(T, G, D, generator=g).bfloat16()
        k[5, 0] = (5.0 * q[0, 0].float() / q[0, 0].float().norm()).bfloat16()          # a loud key near the start
        full_q = torch.zeros(T, H, D, dtype=torch.float64)
        full_q[T - 1] = q[0].double()
        want.append(P.sink_softmax_attention(full_q, k.double().repeat_interleave(rep, 1), v.double().repeat_interleave(rep, 1),
                                             scale, sink.double())[T - 1])
        n = -(-T // page)
        order = [base + int(i) for i in np.random.default_rng(T).permutation(n)]
        kp, vp, table = _paged(k, v, page, order, torch.bfloat16, True)
        kps.append(kp), vps.append(vp), tables.append(table[1]), qs.append(q.reshape(1, H * D))
        base += n
    P_ = base + 1
    k_pages = torch.zeros(P_, G, page, D, dtype=torch.bfloat16, device="cuda")
    v_pages = torch.zeros(P_, G, D, page, dtype=torch.bfloat16, device="cuda")
    width = max(t.numel() for t in tables)
    table = torch.zeros(len(lens) + 1, width, dtype=torch.int32, device="cuda")
    for r, (kp, vp, tb) in enumerate(zip(kps, vps, tables)):
        used = tb[tb > 0].long()
        k_pages[used], v_pages[used] = kp[used], vp[used]
        table[r + 1, :tb.numel()] = tb
    ctx = _Ctx([1] * len(lens), [0] * len(lens), [T - 1 for T in lens])

    class KV:
        pass

    kv = KV()
    kv.k_pages, kv.v_pages, kv.v_transposed, kv.block_table = k_pages, v_pages, True, table
    kv.table_rows = torch.tensor([1, 2, 3], dtype=torch.int32, device="cuda")
    out = torch.empty(len(lens), H * D, dtype=torch.bfloat16, device="cuda")
    ops.paged_attention(torch.cat(qs).cuda(), kv, ctx, out, H, scale, None, sink.cuda())
    for r in range(len(lens)):
        assert (out[r].cpu().double().reshape(H, D) - want[r]).abs().max() < 3e-2, r


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E,page", [(6, 2, 16, 24, 4), (2, 1, 40, 8, 8), (4, 4, 64, 64, 16)])
def test_head_norm_temperature_and_cache_store(dtype, H, G, D, E, page):
    from llm_infrence_engine_amd.kernels import ops

    torch.manual_seed(D)
    N, every, coef = 21, 4, 0.35
    width = (H + G) * D + G * E
    qkv = torch.randn(N, width).to(dtype)
    qw, kw = 1 + 0.2 * torch.randn(D), 1 + 0.2 * torch.randn(D)
    pos = torch.arange(N, dtype=torch.int32) + 2          # positions 2..22: the steps at 3, 7, 11, ... fall inside
    temp = 1.0 + coef * torch.log((torch.div(pos + 1, every, rounding_mode="floor") + 1).double())
    wq = P.norm(qkv[:, :H * D].double().reshape(N, H, D), qw.double(), 1e-5) * temp[:, None, None]
    wk = P.norm(qkv[:, H * D:(H + G) * D].double().reshape(N, G, D), kw.double(), 1e-5)
    tol = 1e-5 if dtype == torch.float32 else 4e-2
    slots = torch.tensor([(3 + n // page) * page + n % page if n != 5 else -1 for n in range(N)], dtype=torch.int32)
    for transposed in (False, True):
        k_pages = torch.zeros(12, G, page, D, dtype=dtype, device="cuda")
        v_pages = torch.zeros((12, G, E, page) if transposed else (12, G, page, E), dtype=dtype, device="cuda")
        got = qkv.cuda()
        ops.qk_norm_store(got, H, G, D, E, qw.cuda(), kw.cuda(), 1e-5, pos.cuda(), coef, every, slots.cuda(), k_pages, v_pages, transposed)
        got = got.cpu()
        assert (got[:, :H * D].double().reshape(N, H, D) - wq).abs().max() < tol
        assert (got[:, H * D:(H + G) * D].double().reshape(N, G, D) - wk).abs().max() < tol
        assert torch.equal(got[:, (H + G) * D:], qkv[:, (H + G) * D:])
        for n in range(N):
            pg, off = 3 + n // page, n % page
            kk = k_pages[pg, :, off].cpu()
            vv = (v_pages[pg, :, :, off] if transposed else v_pages[pg, :, off]).cpu()
            if n == 5:        # a token without a slot stores nothing
                assert not kk.any() and not vv.any()
            else:
                assert torch.equal(kk, got[n, H * D:(H + G) * D].reshape(G, D))
                assert torch.equal(vv, qkv[n, (H + G) * D:].reshape(G, E))
        assert not k_pages[:3].any() and not k_pages[3 + -(-N // page):].any()


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,I,top,F_,S_,W,N", [(5, 2, 2, 40, 56, 72, 37), (7, 0, 1, 64, 0, 72, 37), (4, 1, 3, 48, 0, 72, 37),
                                               (70, 3, 6, 24, 32, 72, 37), (6, 2, 3, 96, 0, 64, 40), (4, 1, 2, 64, 32, 96, 300), (3, 0, 2, 288, 0, 160, 400),
                                               (4, 1, 2, 192, 0, 128, 300), (3, 0, 2, 320, 64, 256, 400)])
def test_routed_experts_alone(dtype, E, I, top, F_, S_, W, N):
    """The part against the plain feed-forward: choices (identities among them: the correction pushes them in),
    weights, experts, the shared expert and its gate.  The last two shapes run on the matrix cores in bfloat16, in
    tiles of 16 rows, (the next two) of 128 and (the last two, whose sizes are multiples of 64) of 256 on the tiled
    kernel, with fewer and more features than a block's tile."""
    from llm_infrence_engine_amd.kernels import ops
    from llm_infrence_engine_amd.parts.base import Runtime
    from llm_infrence_engine_amd.parts.experts import RoutedExperts

    g = torch.Generator().manual_seed(E * 10 + top)
    r = lambda *s: torch.randn(*s, generator=g)
    w = {"m.router": (r(E + I, W) * 0.4).to(dtype), "m.correction": torch.cat([0.05 * r(E), 0.3 + 0.05 * r(I)]).to(dtype)}
    for e in range(E):
        w[f"m.e{e}.up"], w[f"m.e{e}.down"] = (r(F_, W) * 0.25).to(dtype), (r(W, F_) * 0.25).to(dtype)
    if S_:
        w.update({"m.shared.up": (r(S_, W) * 0.25).to(dtype), "m.shared.down": (r(W, S_) * 0.25).to(dtype),
                  "m.shared.sg": (r(1, W) * 0.3).to(dtype)})
    h = r(N, W).to(dtype)
    mlp = {"router": {"experts": E, "identity": I, "top": top}, "shared": {"ff": S_} if S_ else None}
    w64 = {k: v.double() for k, v in w.items()}
    want = P.moe_ff(h.double(), w64, "m.", mlp)
    chosen, weights = P.route(h.double(), w64["m.router"], w64["m.correction"], top)
    if I:
        assert (chosen >= E).any(), "the test's correction brings no identity expert in"
    part = RoutedExperts("m.", W, F_, E, top, I, S_)
    part.load(lambda s: (w[s.name].float() if s.role != "matrix" else w[s.name].to(dtype)).cuda(), Runtime(torch.device("cuda"), dtype))
    got = part.forward(h.cuda(), None)
    assert got.dtype == torch.float32
    assert (got.cpu().double() - want).abs().max() < (2e-5 if dtype == torch.float32 else 6e-2) * max(1.0, float(want.abs().max()) / 4)
    # the router alone: the same choices (as sets) and the same weights
    logits = (h.double() @ w64["m.router"].T).float().cuda()
    ids, wts = ops.moe_route(logits, w["m.correction"].float().cuda(), top)
    assert torch.equal(ids.cpu().long().sort(1).values, chosen.sort(1).values)
    assert torch.allclose(wts.cpu().double().sort(1).values, weights.sort(1).values, atol=1e-6)
    # the grouping: every (token, choice) of an expert with tensors sits in exactly one row of a tile of its expert
    flat = ids.cpu().reshape(-1)
    for tile in (ops.moe_tile_rows(), ops.moe_wide_tile_rows(), ops.moe_widest_tile_rows()):
        rows, tile_expert = (t.cpu() for t in ops.moe_align(ids, E, tile))
        assert rows.numel() == tile * tile_expert.numel()
        seen = rows[rows >= 0]
        assert sorted(seen.tolist()) == [i for i in range(N * top) if flat[i] < E]
        for p_, item in enumerate(rows.tolist()):
            if item >= 0:
                assert tile_expert[p_ // tile] == flat[item]


# ================================================================================================ whole models (GPU)
F32_ATOL = 2e-3
BF16_NOISE = 3.0


def rounded_forward(cfg, w, toks):
    """(exact logits, how far the plain model strays from them when its activations are rounded to bfloat16): a
    faithful reduced-precision computation's own error, of which the bfloat16 path's bound is a multiple."""
    exact = P.forward(cfg, w, toks)
    return exact, float((P.forward(cfg, w, toks, act_dtype=torch.bfloat16) - exact).abs().max())


@pytest.fixture(scope="module", params=list(SHAPES))
def shape(request, tmp_path_factory):
    name = request.param
    cfg = SHAPES[name]
    weights = random_weights(cfg, seed=SEEDS[name])
    folder = write_model(tmp_path_factory.mktemp("gidurax" + name), cfg, weights)
    lengths = {"P": [5, 61, 2, 130, 33, 48], "Q": [1, 9, 90, 47, 110, 64], "R": [3, 26, 70, 17, 2, 41, 60, 33],
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
    runner = _replay(folder, dtype, steps, tmp_path / "out", max_tokens, page)
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
    total = sum(up(len(t)) for t in reqs.values())
    for mode, steps in (("whole", traces.whole(reqs)), ("portions", traces.changing_portions(reqs, sizes=(2, 3, 2, 31, 5, 2))),
                        ("mixed", traces.mixed(reqs, total, seed=9, tail=10))):
        _replay(folder, "float32", steps, tmp_path / mode, total, page)
        outs[mode] = traces.collect(steps, tmp_path / mode, cfg["vocab"])
    for mode in ("portions", "mixed"):
        for key, row in outs[mode].items():
            assert np.abs(row - outs["whole"][key]).max() < 2e-4, (mode, key)


@gpu
def test_one_row_and_few_pages_serve_every_request_in_turn(shape):
    """An engine with a single request row and pages for one request: every request gets the state slots and the pages
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
        got = [runner.step([StepEntry(rid, toks[:cut], list(range(cut)))]).cpu().numpy()]
        assert runner.manager.row(rid) == 0
        if cut < len(toks):
            got.append(runner.step([StepEntry(rid, toks[cut:], list(range(len(toks) - cut)))]).cpu().numpy())
        runner.free_request(rid)
        assert np.abs(np.concatenate(got) - want[rid]).max() < F32_ATOL, rid
    runner.manager.check_invariants()
    assert all(g.allocator.pages_granted_again() > 0 for g in runner.manager.groups)


@gpu
@pytest.mark.parametrize("kind", ["mamba1", "delta", "attention"])
def test_far_token_reaches_the_end(tmp_path, kind):
    """A token 400 places back still moves the last logits, through the scan's or the delta rule's state (made slow to
    forget) or through attention's cache, in the plain model and equally in the engine, whole and decoded token by token
    (the decoded stretch passes several steps of the query temperature)."""
    mixer = {"mamba1": mamba_layer(48, 12, 4, 2, dense(64)), "delta": delta_layer(2, 1, 32, 16, 2, dense(64)),
             "attention": attention_layer(2, 1, 16, 24, 0.5, dense(64), temp=(0.5, 50))}[kind]
    cfg = config(97, 64, 1e-5, 0.8, 3.0, [mixer])
    weights = random_weights(cfg, seed=1)
    for k_ in weights:
        if k_.endswith("A_log"):
            weights[k_] = torch.full_like(weights[k_], -7.0)        # a memory of about a thousand tokens
        if k_.endswith("dt.b"):
            weights[k_] = torch.full_like(weights[k_], 0.5)
    folder = write_model(tmp_path / "m", cfg, weights)
    w64 = {k_: v.double() for k_, v in weights.items()}
    rng = np.random.default_rng(5)
    a = [int(t) for t in rng.integers(0, 97, 420)]
    b = list(a)
    b[7] = (b[7] + 50) % 97
    la, lb = P.forward(cfg, w64, a)[-1].numpy(), P.forward(cfg, w64, b)[-1].numpy()
    assert np.abs(la - lb).max() > 0.003, "the test's weights forget too fast to show anything"
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
    weights = {k: v.double() for k, v in random_weights(cfg, seed=SEEDS[name]).items()}
    prompts = [toks[:max(1, len(toks) // 3)] for toks in list(reqs.values())[:4]]
    llm = eng.LLM(str(folder), dtype=dtype, block_size=PAGES[name], max_len=128, max_seqs=3, max_prefill_chunk=7)
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

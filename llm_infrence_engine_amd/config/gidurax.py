"""Typed configuration of the Gidurax decoder and its translation into a ``ModelSpec``.

config.json: ``architecture`` "Gidurax", ``vocab``, ``width``, ``norm.eps``, ``residual_mult``, ``embedding.scale``,
``layers`` (one entry per layer: ``type``, the mixer: "delta", "attention" or "mamba1"; ``mixer``, its sizes and
constants; ``mlp``: {"kind": "dense", "ff"}, {"kind": "moe", "expert": {"ff"}, "router": {"experts", "identity", "top"},
"shared": {"ff"} or null}, or null for a layer without a feed-forward) and optionally ``loop`` {"start", "stop", "times"}:
the layers start .. stop - 1 are walked ``times`` times in a row with the same weights, each walk with caches and states
of its own.

Fixed by the design and therefore constants here: every sublayer lies between two norms and joins the residual sum
weighted by ``residual_mult`` (folded into the second norm's weight); norms store their scale as it is; the delta mixer
has one decay per head and a SiLU gate; attention normalises its query and key heads, has no rotation, a query
temperature from ``q_temp`` {"coef", "every"}, a sink per head and no window; feed-forwards use the exact gelu; before
every walk over the looped stretch row t of ``loop.step`` is added to the residual stream, and before every walk but the
first also the embedding's output; tensors are named ``embed``, ``loop.step``, ``l<i>.norm1``, ``l<i>.norm1b``,
``l<i>.norm2``, ``l<i>.norm2b``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

import copy
import json
from dataclasses import dataclass
from typing import Optional, Tuple

from .registry import ConfigError, register_architecture
from .spec import ModelSpec, PartSpec, Run, layer

MIXERS = ("delta", "attention", "mamba1")


def _need(d, key: str, where: str, kind=int, positive: bool = True):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError(f"config.json: {where} lacks the required key {key!r}")
    v = d[key]
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int) or (v <= 0 if positive else v < 0):
            raise ConfigError(f"config.json: {where}.{key} must be a {'positive' if positive else 'non-negative'} integer, got {v!r}")
    elif kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"config.json: {where}.{key} must be a number, got {v!r}")
        v = float(v)
    return v


@dataclass(frozen=True)
class GiduraxConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    embedding_scale: float
    layers: Tuple[dict, ...]          # as config.json gives them (checked in __post_init__, never changed afterwards)
    loop: Optional[Tuple[int, int, int]] = None     # (start, stop, times)

    architecture = "Gidurax"

    def __hash__(self):
        return hash(json.dumps(self.to_dict(), sort_keys=True))

    def __post_init__(self):
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.norm_eps >= 0:
            raise ConfigError(f"norm.eps must be >= 0, got {self.norm_eps}")
        if not self.layers:
            raise ConfigError("config.json: 'layers' is empty")
        for i, entry in enumerate(self.layers):
            where = f"layers[{i}]"
            kind = entry.get("type") if isinstance(entry, dict) else None
            if kind not in MIXERS:
                raise ConfigError(f"config.json: {where}.type is {kind!r}; this design has {', '.join(MIXERS)}")
            m = entry.get("mixer")
            if kind == "delta":
                for k in ("heads", "kv_heads", "dim", "vdim", "conv"):
                    _need(m, k, where + ".mixer")
            elif kind == "attention":
                for k in ("heads", "kv_heads", "dim", "vdim"):
                    _need(m, k, where + ".mixer")
                _need(m, "scale", where + ".mixer", float)
                if m.get("q_temp") is not None:
                    _need(m["q_temp"], "coef", where + ".mixer.q_temp", float)
                    _need(m["q_temp"], "every", where + ".mixer.q_temp")
            else:
                for k in ("inner", "state", "dt_rank", "conv"):
                    _need(m, k, where + ".mixer")
            if kind != "mamba1" and m["heads"] % m["kv_heads"]:
                raise ConfigError(f"config.json: {where}.mixer: {m['heads']} heads cannot share {m['kv_heads']} kv_heads")
            mlp = entry.get("mlp")
            if mlp is not None:
                if mlp.get("kind") == "dense":
                    _need(mlp, "ff", where + ".mlp")
                elif mlp.get("kind") == "moe":
                    _need(mlp.get("expert"), "ff", where + ".mlp.expert")
                    r = mlp.get("router")
                    _need(r, "experts", where + ".mlp.router")
                    _need(r, "top", where + ".mlp.router")
                    if r.get("identity") is not None:
                        _need(r, "identity", where + ".mlp.router", positive=False)
                    if r["top"] > r["experts"] + (r.get("identity") or 0):
                        raise ConfigError(f"config.json: {where}.mlp.router: top {r['top']} exceeds the experts there are")
                    if mlp.get("shared") is not None:
                        _need(mlp["shared"], "ff", where + ".mlp.shared")
                else:
                    raise ConfigError(f"config.json: {where}.mlp.kind is {mlp.get('kind')!r}; this design has 'dense' and 'moe'")
        if self.loop is not None:
            start, stop, times = self.loop
            if not (0 <= start < stop <= len(self.layers)) or times <= 0:
                raise ConfigError(f"config.json: loop {{start: {start}, stop: {stop}, times: {times}}} does not name a "
                                  f"stretch of the {len(self.layers)} layers walked at least once")

    # ------------------------------------------------------------------ config.json
    @classmethod
    def from_dict(cls, d: dict) -> "GiduraxConfig":
        layers = d.get("layers")
        if not isinstance(layers, list):
            raise ConfigError("config.json lacks the list 'layers'")
        loop = d.get("loop")
        if loop is not None:
            loop = (_need(loop, "start", "loop", positive=False), _need(loop, "stop", "loop"), _need(loop, "times", "loop"))
        return cls(vocab=_need(d, "vocab", "config"), width=_need(d, "width", "config"),
                   norm_eps=_need(d.get("norm"), "eps", "norm", float),
                   residual_mult=_need(d, "residual_mult", "config", float) if d.get("residual_mult") is not None else 1.0,
                   embedding_scale=_need(d["embedding"], "scale", "embedding", float)
                   if isinstance(d.get("embedding"), dict) and d["embedding"].get("scale") is not None else 1.0,
                   layers=tuple(copy.deepcopy(e) for e in layers), loop=loop)

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "residual_mult": self.residual_mult, "embedding": {"scale": self.embedding_scale},
             "layers": [copy.deepcopy(e) for e in self.layers]}
        if self.loop is not None:
            d["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        return d

    # ------------------------------------------------------------------ derived sizes
    @property
    def num_params(self) -> int:
        from ..parts.model import Model

        total = 0
        for s in Model(self.to_spec()).tensor_specs():
            n = 1
            for d in s.shape:
                n *= d
            total += n
        return total

    # ------------------------------------------------------------------ the model as data
    def _mixer(self, i: int, entry: dict):
        """(mixer PartSpec, position PartSpec or None) of layer i."""
        m, p, W = entry["mixer"], f"l{i}.mix.", self.width
        if entry["type"] == "delta":
            return PartSpec("gated_delta", p, {
                "hidden_size": W, "heads": m["heads"], "kv_heads": m["kv_heads"], "dim": m["dim"], "vdim": m["vdim"],
                "taps": m["conv"], "eps": self.norm_eps, "decay": "head", "gate": "silu"}), None
        if entry["type"] == "mamba1":
            return PartSpec("selective_scan", p, {"hidden_size": W, "inner": m["inner"], "state": m["state"],
                                                  "dt_rank": m["dt_rank"], "taps": m["conv"]}), None
        temp = m.get("q_temp") or {}
        position = PartSpec("qk_norm_temperature", p, {"head_dim": m["dim"], "eps": self.norm_eps, "qk_norm": True,
                                                       "coef": float(temp.get("coef", 0.0)), "every": int(temp.get("every", 1))})
        mixer = PartSpec("gqa_attention", p, {
            "hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
            "value_dim": m["vdim"], "scale": float(m["scale"]), "qkv_bias": False, "out_bias": False, "window": None,
            "sink": True, "names": (("k", "k"), ("o", "o"), ("q", "q"), ("sink", "sink"), ("v", "v"))})
        return mixer, position

    def _feed_forward(self, i: int, mlp: dict) -> PartSpec:
        p, W = f"l{i}.mlp.", self.width
        if mlp["kind"] == "dense":
            return PartSpec("dense_act", p, {"hidden_size": W, "intermediate_size": mlp["ff"], "activation": "gelu"})
        r = mlp["router"]
        return PartSpec("routed_experts", p, {
            "hidden_size": W, "expert_ff": mlp["expert"]["ff"], "experts": r["experts"], "identity": r.get("identity") or 0,
            "top": r["top"], "shared_ff": (mlp.get("shared") or {}).get("ff", 0), "activation": "gelu"})

    def order(self) -> Tuple[Run, ...]:
        n = len(self.layers)
        if self.loop is None:
            return tuple(Run(i) for i in range(n))
        start, stop, times = self.loop
        runs = [Run(i) for i in range(start)]
        for t in range(times):
            runs += [Run(i, opens_pass=t if i == start else None) for i in range(start, stop)]
        return tuple(runs + [Run(i) for i in range(stop, n)])

    def to_spec(self) -> ModelSpec:
        W, eps, m = self.width, self.norm_eps, self.residual_mult
        layers = []
        for i, entry in enumerate(self.layers):
            p = f"l{i}."
            mixer, position = self._mixer(i, entry)
            mlp = entry.get("mlp")

            def norm(name, gain=1.0):
                return PartSpec("rms_norm", p, {"size": W, "eps": eps, "name": name, "gain": gain})

            layers.append(layer(
                "sandwich_residual", position=position, mixer_norm=norm("norm1"), mixer=mixer,
                mixer_post_norm=norm("norm1b", m),
                feed_forward_norm=None if mlp is None else norm("norm2"),
                feed_forward=None if mlp is None else self._feed_forward(i, mlp),
                feed_forward_post_norm=None if mlp is None else norm("norm2b", m)))
        return ModelSpec(
            architecture=self.architecture, hidden_size=W, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", "", {"vocab_size": self.vocab, "hidden_size": W, "name": "embed",
                                                       "scale": self.embedding_scale}),
            layers=tuple(layers), order=self.order(),
            final_norm=PartSpec("rms_norm", "final.", {"size": W, "eps": eps, "name": "norm"}),
            head=PartSpec("lm_head", "", {"hidden_size": W, "vocab_size": self.vocab, "tied_to": None, "name": "head"}),
            ignorable=tuple(f"l{i}.{n}" for i, e in enumerate(self.layers) if e.get("mlp") is None for n in ("norm2", "norm2b")),
            pass_entry=None if self.loop is None else
            PartSpec("pass_step", "loop.", {"hidden_size": W, "times": self.loop[2], "name": "step", "readd_embedding": True}),
        )


register_architecture(GiduraxConfig.architecture, GiduraxConfig, model_type="gidurax")

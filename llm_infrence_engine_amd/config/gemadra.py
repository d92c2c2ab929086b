"""Typed configuration of the Gemadra decoder and its translation into a ``ModelSpec``.

config.json: ``architecture`` "Gemadra", ``vocab``, ``width``, ``norm.eps``, ``canon.taps`` and ``layers``, a list
with one entry per layer: ``type`` (the mixer: "channel_delta" or "latent_attention"), ``mixer`` (its sizes and
constants) and ``mlp`` ({"kind": "dense", "ff": n}, or null for a layer without a feed-forward).  Sizes that
config.json leaves out (the ranks of the delta mixer's two low-rank maps) are taken from the shapes of the tensors
(``with_tensor_shapes``), or stated as ``decay_rank`` / ``gate_rank`` in the mixer's entry.

Fixed by the design and therefore constants here: every layer is parallel (both branches read the same x) with
two norms whose scale is stored around zero, as is the model's last norm; a short causal convolution is added to the
mixer's input in every layer; the feed-forward is down(xielu(up(x))); rotation pairs neighbouring entries; the
latent attention has a window, a sink and an output gate; tensors are named ``embed``, ``l<i>.norm1``,
``l<i>.norm2``, ``l<i>.canon1``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Optional, Tuple

from .registry import ConfigError, register_architecture
from .spec import ModelSpec, PartSpec, Run, layer

MIXERS = ("channel_delta", "latent_attention")


def _need(d: dict, key: str, where: str, kind=int):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError(f"config.json: {where} lacks the required key {key!r}")
    v = d[key]
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
            raise ConfigError(f"config.json: {where}.{key} must be a positive integer, got {v!r}")
    elif kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"config.json: {where}.{key} must be a number, got {v!r}")
        v = float(v)
    return v


@dataclass(frozen=True)
class GemadraConfig:
    vocab: int
    width: int
    norm_eps: float
    canon_taps: int
    layers: Tuple[dict, ...]      # as config.json gives them (checked in __post_init__, never changed afterwards)

    architecture = "Gemadra"

    def __hash__(self):
        import json

        return hash(json.dumps(self.to_dict(), sort_keys=True))

    def __post_init__(self):
        if self.vocab <= 0 or self.width <= 0 or self.canon_taps <= 0:
            raise ConfigError("vocab, width and canon.taps must be positive")
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
            if kind == "channel_delta":
                for k in ("heads", "kv_heads", "dim", "vdim", "conv"):
                    _need(m, k, where + ".mixer")
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"config.json: {where}.mixer: {m['heads']} heads cannot share {m['kv_heads']} kv_heads")
            else:
                for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"):
                    _need(m, k, where + ".mixer")
                _need(m, "scale", where + ".mixer", float)
                rot = m.get("rot") or {}
                _need(rot, "base", where + ".mixer.rot", float)
                dims = _need(rot, "dims", where + ".mixer.rot")
                if dims % 2 or dims > m["rot_dim"]:
                    raise ConfigError(f"config.json: {where}.mixer.rot.dims = {dims} must be even and at most rot_dim")
                if m.get("mask") is not None:
                    _need(m["mask"], "size", where + ".mixer.mask")
            mlp = entry.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp.kind is {mlp.get('kind')!r}; this design has 'dense'")
                _need(mlp, "ff", where + ".mlp")

    # ------------------------------------------------------------------ config.json
    @classmethod
    def from_dict(cls, d: dict) -> "GemadraConfig":
        layers = d.get("layers")
        if not isinstance(layers, list):
            raise ConfigError("config.json lacks the list 'layers'")
        return cls(vocab=_need(d, "vocab", "config"), width=_need(d, "width", "config"),
                   norm_eps=_need(d.get("norm"), "eps", "norm", float),
                   canon_taps=_need(d.get("canon"), "taps", "canon"),
                   layers=tuple(copy.deepcopy(e) for e in layers))

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.norm_eps}, "canon": {"taps": self.canon_taps},
                "layers": [copy.deepcopy(e) for e in self.layers]}

    def with_tensor_shapes(self, shape_of) -> "GemadraConfig":
        """The configuration with the sizes that only the tensors' shapes give: ``shape_of(name)`` is a tensor's
        shape, or None if the checkpoint has no such tensor."""
        layers = []
        for i, entry in enumerate(self.layers):
            entry = copy.deepcopy(entry)
            if entry["type"] == "channel_delta":
                for key, tensor in (("decay_rank", f"l{i}.mix.a1"), ("gate_rank", f"l{i}.mix.g1")):
                    shape = shape_of(tensor)
                    if entry["mixer"].get(key) is None and shape is not None and len(shape) == 2:
                        entry["mixer"][key] = int(shape[0])
            layers.append(entry)
        return GemadraConfig(self.vocab, self.width, self.norm_eps, self.canon_taps, tuple(layers))

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
        if entry["type"] == "channel_delta":
            for key in ("decay_rank", "gate_rank"):
                if m.get(key) is None:
                    raise ConfigError(f"layers[{i}].mixer.{key} is not in config.json; it is the first size of the tensor "
                                      f"l{i}.mix.{'a1' if key == 'decay_rank' else 'g1'} (load the configuration with the "
                                      f"checkpoint beside it, or state the key)")
            return PartSpec("gated_delta", p, {
                "hidden_size": W, "heads": m["heads"], "kv_heads": m["kv_heads"], "dim": m["dim"], "vdim": m["vdim"],
                "taps": m["conv"], "decay_rank": m["decay_rank"], "gate_rank": m["gate_rank"], "eps": self.norm_eps}), None
        window: Optional[int] = (m.get("mask") or {}).get("size")
        mixer = PartSpec("latent_attention", p, {
            "hidden_size": W, "heads": m["heads"], "dim": m["dim"], "rot_dim": m["rot_dim"], "vdim": m["vdim"],
            "q_rank": m["q_rank"], "kv_rank": m["kv_rank"], "scale": float(m["scale"]), "eps": self.norm_eps,
            "window": window, "sink": True, "output_gate": True})
        position = PartSpec("rotary_pairs", "", {"width": m["rot_dim"], "dims": m["rot"]["dims"],
                                                 "theta": float(m["rot"]["base"])})
        return mixer, position

    def to_spec(self) -> ModelSpec:
        W = self.width
        layers = []
        for i, entry in enumerate(self.layers):
            p = f"l{i}."
            mixer, position = self._mixer(i, entry)
            mlp = entry.get("mlp")
            layers.append(layer(
                "parallel_residual",
                position=position,
                mixer_norm=PartSpec("rms_norm", p, {"size": W, "eps": self.norm_eps, "offset": 1.0, "name": "norm1"}),
                input_filter=PartSpec("short_conv", p, {"channels": W, "taps": self.canon_taps, "add_input": True,
                                                        "name": "canon1"}),
                mixer=mixer,
                feed_forward_norm=None if mlp is None else
                PartSpec("rms_norm", p, {"size": W, "eps": self.norm_eps, "offset": 1.0, "name": "norm2"}),
                feed_forward=None if mlp is None else
                PartSpec("dense_act", p + "mlp.", {"hidden_size": W, "intermediate_size": mlp["ff"], "activation": "xielu"}),
            ))
        return ModelSpec(
            architecture=self.architecture, hidden_size=W, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", "", {"vocab_size": self.vocab, "hidden_size": W, "name": "embed"}),
            layers=tuple(layers), order=tuple(Run(i) for i in range(len(layers))),
            final_norm=PartSpec("rms_norm", "final.", {"size": W, "eps": self.norm_eps, "offset": 1.0, "name": "norm"}),
            head=PartSpec("lm_head", "", {"hidden_size": W, "vocab_size": self.vocab, "tied_to": None, "name": "head"}),
            # a layer without a feed-forward has no use for a second norm, whether or not the checkpoint carries one
            ignorable=tuple(f"l{i}.norm2" for i, e in enumerate(self.layers) if e.get("mlp") is None),
        )


register_architecture(GemadraConfig.architecture, GemadraConfig, model_type="gemadra")

"""Maps over time that a block lays before a part's input.

``short_conv``: h <- h + conv(h) (or conv(h) alone), a causal convolution over time on every channel with ``taps``
weights per channel, the last of them meeting the token itself; inputs before a sequence's start are zero.  The last
taps - 1 inputs of a request are its state, kept in the type of the activations so that a portion continues with
exactly the values a whole prompt would have read."""
from __future__ import annotations

from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import SequenceFilter, StateNeed, register_part


class ShortConv(SequenceFilter):
    def __init__(self, prefix: str, channels: int, taps: int, add_input: bool = True, name: str = "weight"):
        if not 1 <= taps <= ops.MAX_CONV_TAPS:
            raise ValueError(f"a short convolution has 1 to {ops.MAX_CONV_TAPS} taps, got {taps}")
        self.prefix, self.channels, self.taps, self.add_input, self.name = prefix, channels, taps, add_input, name

    def tensor_specs(self):
        return [TensorSpec(self.prefix + self.name, (self.channels, self.taps), "bias")]

    def load(self, get, rt):
        self.rt = rt
        self.weight = get(self.tensor_specs()[0])

    def state_need(self):
        return StateNeed((max(1, self.taps - 1), self.channels), None)

    def forward(self, h, ctx, state):
        out = self.rt.empty(h.shape[0], self.channels)
        return ops.short_conv(h, self.weight, state.slots, ctx, out,
                              ops.CONV_ADD_INPUT if self.add_input else ops.CONV_SUM)


register_part("filter", "short_conv", ShortConv)

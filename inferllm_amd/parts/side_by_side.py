"""Two mixers that read the same rows; their outputs are added with a scale each."""
from __future__ import annotations

from typing import Dict

from ..kernels import ops
from ..weights.loader import TensorWant
from .base import Mixer, StepContext, build_part, register_part


@register_part("mixer", "side_by_side")
class SideBySide(Mixer):
    """out = left_scale * left(h) + right_scale * right(h).

    `left` and `right` are `PartSpec`s of mixers.  The pair keeps on its cache line what its
    mixers keep: at most one of them keys and values, at most one fixed-size state.  A block that
    adds scaled sums in a kernel of its own sets `takes_scaled_sums` and gets the two outputs as
    `ops.ScaledSum`; any other gets their float32 sum.
    """

    takes_scaled_sums = False

    def __init__(self, left, right, left_scale: float = 1.0, right_scale: float = 1.0, tensors=None):
        super().__init__(tensors)
        self.left, self.right = build_part("mixer", left), build_part("mixer", right)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        both = (self.left, self.right)
        if sum(m.kv_spec() is not None for m in both) > 1 or sum(m.state_spec() is not None for m in both) > 1:
            raise ValueError("side_by_side: a cache line holds one mixer's keys and values and one "
                             "mixer's state; these two both keep the same kind")
        self.graph_safe = all(m.graph_safe for m in both)
        self.graph_safe_prompts = all(m.graph_safe_prompts for m in both)
        self.takes_continuations = all(m.takes_continuations for m in both)

    def wants(self) -> Dict[str, TensorWant]:
        return {**self.left.wants(), **self.right.wants()}

    def kv_spec(self):
        return self.left.kv_spec() or self.right.kv_spec()

    def state_spec(self):
        return self.left.state_spec() or self.right.state_spec()

    def load(self, tensors) -> None:
        for m in (self.left, self.right):
            m.decode_copies, m.position = self.decode_copies, self.position
            m.load(tensors)

    def tunables(self):
        return tuple(self.left.tunables()) + tuple(self.right.tunables())

    def forward(self, h, ctx: StepContext, line, writes_cache, position):
        a = self.left.forward(h, ctx, line, writes_cache, position)
        b = self.right.forward(h, ctx, line, writes_cache, position)
        both = ops.ScaledSum(a, self.left_scale, b, self.right_scale)
        return both if self.takes_scaled_sums else both.tensor()

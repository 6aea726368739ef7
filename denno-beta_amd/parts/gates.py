"""Result gates: what a sublayer returns is multiplied, element by element, by a sigmoid that reads the rows the
sublayer itself read.  A gate only makes the sigmoid's arguments (`logits(h)`, 32-bit rows); the multiplication
happens in the kernel that takes the sublayer's result into the stream (parts.norms.StreamRMSNorm.add_into)."""
from __future__ import annotations

import torch

from .base import GATES, Part
from .linear import Linear


@GATES.register("sigmoid_linear")
class SigmoidLinearGate(Part):
    """sigmoid(W h + b), one number per column of the sublayer's result."""
    graph_safe = True
    absent = False

    def __init__(self, width: int, out_width: int, weight_name: str, bias_name=None):
        self.width, self.out_width = width, out_width
        self.proj = Linear(width, out_width, weight_name, bias_name, init_std=width ** -0.5)

    def param_specs(self):
        return self.proj.param_specs()

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.proj.bind(tensors)

    def logits(self, h):
        return self.proj(h, out_dtype=torch.float32)


@GATES.register("none")
class NoGate(Part):
    """No gate: the sublayer's result goes on as it is."""
    graph_safe = True
    absent = True

    def __init__(self):
        pass

    def logits(self, h):
        return None

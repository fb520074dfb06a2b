"""Dense feed-forward with the xIELU activation: ``W_down act(W_up x)`` without bias, where
``act(z) = softplus(p) z^2 + z/2`` for ``z > 0`` and ``(1/2 + softplus(q)) (exp(z) - 1 - z) + z/2`` otherwise;
``p`` and ``q`` are two learned numbers per layer."""
from __future__ import annotations

import math

import torch

from .base import FeedForward, TensorSpec


def _softplus(z: float) -> float:
    return max(z, 0.0) + math.log1p(math.exp(-abs(z)))


class DenseXielu(FeedForward):
    """params: width, inner.  names: up, down, act (the two numbers p, q)."""
    graph_safe = True

    def tensor_specs(self):
        d, i = self.params["width"], self.params["inner"]
        return {self.names["up"]: TensorSpec((i, d)), self.names["down"]: TensorSpec((d, i)),
                self.names["act"]: TensorSpec((2,))}

    def bind(self, tensors, rt):
        self.rt = rt
        self.w_up = rt.weight(tensors[self.names["up"]])
        self.w_down = rt.weight(tensors[self.names["down"]])
        p, q = (float(v) for v in tensors[self.names["act"]].float().cpu())
        self.a_pos, self.a_neg = _softplus(p), 0.5 + _softplus(q)

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in (self.w_up, self.w_down))

    def step_flops(self, rows):
        return 2 * rows * (self.w_up.w.numel() + self.w_down.w.numel())

    def forward(self, x, step):
        rt = self.rt
        z = rt.linear(x, self.w_up)
        return rt.linear(rt.ops.xielu(z, z, self.a_pos, self.a_neg), self.w_down, partials=True)     # in place

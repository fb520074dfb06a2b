"""HGRN2: a linear recurrence over a matrix state per head with a single gate: what a channel keeps of its old
state is `f`, and what it takes of the new value is `1 - f`.

``q = silu(W_q x)``, ``v = W_v x``, ``f = low + (1 - low) * sigmoid(W_f x + b_f)`` per head and key channel
(``low`` a stored lower bound); per head ``S_t = diag(f_t) S_{t-1} + (1 - f_t) v_t^T`` and ``o_t = S_t^T q_t``
(no key, no other scale); every head's ``o`` is RMS-normed over its value lanes with one shared weight, the heads
are concatenated and projected.  ``S`` starts at zero, is float32 and is carried per sequence as fixed-size state."""
from __future__ import annotations

import torch

from .base import Mixer, StateNeed, TensorSpec


class HGRN2(Mixer):
    """params: width, heads, dim, vdim, eps.  names: q, f, f_bias, lower, v, norm, o."""
    graph_safe = True

    def tensor_specs(self):
        p, n = self.params, self.names
        d, H, dk, dv = p["width"], p["heads"], p["dim"], p["vdim"]
        return {n["q"]: TensorSpec((H * dk, d)), n["f"]: TensorSpec((H * dk, d)), n["f_bias"]: TensorSpec((H * dk,)),
                n["lower"]: TensorSpec((H * dk,)), n["v"]: TensorSpec((H * dv, d)), n["norm"]: TensorSpec((dv,)),
                n["o"]: TensorSpec((d, H * dv))}

    def cache_need(self):
        p = self.params
        return StateNeed((p["heads"], p["dim"], p["vdim"]), torch.float32)

    def bind(self, tensors, rt):
        self.rt = rt
        p, n = self.params, self.names
        self.H, self.dk, self.dv, self.eps = p["heads"], p["dim"], p["vdim"], float(p["eps"])
        ws = [tensors[n[r]] for r in ("q", "f", "v")]
        if len({w.dtype for w in ws}) != 1:
            ws = [w.float() for w in ws]
        self.w_in = rt.weight(torch.cat(ws, dim=0))
        self.f_bias = tensors[n["f_bias"]].float().contiguous()
        self.low = tensors[n["lower"]].float().contiguous()
        self.norm_w = tensors[n["norm"]].float().contiguous()
        self.w_o = rt.weight(tensors[n["o"]])

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in (self.w_in, self.w_o))

    def step_flops(self, rows):
        return 2 * rows * (self.w_in.w.numel() + self.w_o.w.numel())

    def mixing_flops(self, past, new):
        return 4 * self.H * self.dk * self.dv * new

    def forward(self, x, step, view):
        return self.output(self.scan(self.project(x), step, view))

    def project(self, x):
        return self.rt.linear(x, self.w_in)

    def output(self, mixed):
        return self.rt.linear(mixed, self.w_o, partials=True)

    def scan(self, proj, step, view):
        """The recurrence over the step's tokens, each sequence from its own state -> [tokens, heads * vdim]."""
        rt = self.rt
        o_raw = torch.zeros(proj.shape[0], self.H * self.dv, dtype=torch.float32, device=proj.device)
        out = torch.empty(proj.shape[0], self.H * self.dv, dtype=rt.dtype, device=proj.device)
        return rt.ops.hgrn2_scan(proj, self.f_bias, self.low, self.norm_w, self.eps, view.tensor, o_raw, out, step,
                                 self.H, self.dk, self.dv)

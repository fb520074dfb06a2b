"""Gated linear attention: a matrix state per head that decays channel by channel and takes every token's key and
value as an outer product.

``q = W_q x * dim^-1/2``, ``k = W_k x`` (heads x dim), ``v = W_v x`` (heads x vdim); a decay per key channel
``alpha = sigmoid(W_a2 (W_a1 x) + b)^(1/tau)``; per head ``S_t = diag(alpha_t) S_{t-1} + k_t v_t^T`` and
``o_t = S_t^T q_t``.  Every head's ``o`` is RMS-normed over its value lanes with one shared weight, the heads are
concatenated, multiplied by ``silu(W_g x)`` and projected.  ``S`` starts at zero, is float32 and is carried per
sequence as fixed-size state; the decays (through their logarithm), the scaled queries, the recurrence and the
head norm are float32 in every mode."""
from __future__ import annotations

import torch

from .base import Mixer, StateNeed, TensorSpec


class GatedLinearAttention(Mixer):
    """params: width, heads, dim, vdim, tau, eps, decay_rank (inner width of the decay's two projections).
    names: q, k, v, g, a1, a2, a2_bias, norm, o."""
    graph_safe = True

    def tensor_specs(self):
        p, n = self.params, self.names
        d, H, dk, dv, r = p["width"], p["heads"], p["dim"], p["vdim"], p["decay_rank"]
        return {n["q"]: TensorSpec((H * dk, d)), n["k"]: TensorSpec((H * dk, d)), n["v"]: TensorSpec((H * dv, d)),
                n["g"]: TensorSpec((H * dv, d)), n["a1"]: TensorSpec((r, d)), n["a2"]: TensorSpec((H * dk, r)),
                n["a2_bias"]: TensorSpec((H * dk,)), n["norm"]: TensorSpec((dv,)), n["o"]: TensorSpec((d, H * dv))}

    def cache_need(self):
        p = self.params
        return StateNeed((p["heads"], p["dim"], p["vdim"]), torch.float32)

    def bind(self, tensors, rt):
        self.rt = rt
        p, n = self.params, self.names
        self.H, self.dk, self.dv, self.rank = p["heads"], p["dim"], p["vdim"], p["decay_rank"]
        self.tau, self.eps = float(p["tau"]), float(p["eps"])
        ws = [tensors[n[r]] for r in ("q", "k", "v", "g")]
        # the decay's first projection starts at a multiple of 8 columns, so that its rows of the result can feed
        # the second one as they lie
        lead = sum(w.shape[0] for w in ws)
        pad = (-lead) % 8
        if pad:
            ws.append(torch.zeros(pad, ws[0].shape[1], dtype=ws[0].dtype, device=ws[0].device))
        self.a1_at = lead + pad
        ws.append(tensors[n["a1"]])
        tail = (-(self.a1_at + self.rank)) % 8
        if tail:
            ws.append(torch.zeros(tail, ws[0].shape[1], dtype=ws[0].dtype, device=ws[0].device))
        if len({w.dtype for w in ws}) != 1:
            ws = [w.float() for w in ws]
        self.w_in = rt.weight(torch.cat(ws, dim=0))
        self.w_a2 = rt.weight(tensors[n["a2"]])
        self.w_o = rt.weight(tensors[n["o"]])
        self.a2_bias = tensors[n["a2_bias"]].float().contiguous()
        self.norm_w = tensors[n["norm"]].float().contiguous()

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in (self.w_in, self.w_a2, self.w_o))

    def step_flops(self, rows):
        return 2 * rows * sum(w.w.numel() for w in (self.w_in, self.w_a2, self.w_o))

    def mixing_flops(self, past, new):
        return 5 * self.H * self.dk * self.dv * new

    def forward(self, x, step, view):
        return self.output(self.scan(self.project(x), step, view))

    def project(self, x):
        """The stacked projection [q | k | v | g | a1] and the decays' logits (before their bias)."""
        rt = self.rt
        proj = rt.linear(x, self.w_in)
        low = proj[:, self.a1_at:self.a1_at + self.rank]
        if low.data_ptr() % 16 or low.stride(0) % 8 or self.rank % 8:
            low = low.contiguous()
        return proj, rt.linear(low, self.w_a2)

    def scan(self, projected, step, view):
        """The recurrence over the step's tokens, each sequence from its own state -> [tokens, heads * vdim]."""
        rt = self.rt
        proj, decay_in = projected
        T = proj.shape[0]
        o_raw = torch.zeros(T, self.H * self.dv, dtype=torch.float32, device=proj.device)
        out = torch.empty(T, self.H * self.dv, dtype=rt.dtype, device=proj.device)
        return rt.ops.gla_scan(proj, decay_in, self.a2_bias, self.tau, self.norm_w, self.eps, view.tensor, o_raw, out,
                               step, self.H, self.dk, self.dv)

    def output(self, mixed):
        return self.rt.linear(mixed, self.w_o, partials=True)

"""Delta-rule mixer whose state decays channel by channel (a decay for every key channel of every head).

``q = W_q x`` and ``k = W_k x`` (kv_heads x dim), ``v = W_v x`` (heads x vdim); each passes a short causal
convolution per channel and SiLU; q and k become unit vectors per head (q also times dim^-1/2); head h reads
q/k head ``h // (heads / kv_heads)``.  ``beta = sigmoid(W_b x)`` per head; ``g = exp(-exp(A_log_h) *
softplus(W_a2 W_a1 x + dt_bias))`` per head and key channel.  Per head and token, in this order:
``S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``.  ``o`` is divided by its root mean square
over the value lanes, times a shared weight, times ``sigmoid(W_g2 W_g1 x)``, then projected.  ``S`` (float32)
and the last taps-1 inputs of the convolutions are carried per sequence as fixed-size state."""
from __future__ import annotations

import torch

from .base import Mixer, StateNeed, TensorSpec


class ChannelDelta(Mixer):
    """params: width, heads, kv_heads, dim, vdim, conv (taps), decay_rank, gate_rank, eps.
    names: q, k, v, q_conv, k_conv, v_conv, b, A_log, norm, a1, a2, dt_bias, g1, g2, o."""
    graph_safe = True

    def tensor_specs(self):
        p, n = self.params, self.names
        d, H, G, dk, dv, taps = p["width"], p["heads"], p["kv_heads"], p["dim"], p["vdim"], p["conv"]
        ra, rg = p["decay_rank"], p["gate_rank"]
        return {n["q"]: TensorSpec((G * dk, d)), n["k"]: TensorSpec((G * dk, d)), n["v"]: TensorSpec((H * dv, d)),
                n["q_conv"]: TensorSpec((G * dk, taps)), n["k_conv"]: TensorSpec((G * dk, taps)),
                n["v_conv"]: TensorSpec((H * dv, taps)), n["b"]: TensorSpec((H, d)), n["A_log"]: TensorSpec((H,)),
                n["norm"]: TensorSpec((dv,)), n["a1"]: TensorSpec((ra, d)), n["a2"]: TensorSpec((H * dk, ra)),
                n["dt_bias"]: TensorSpec((H * dk,)), n["g1"]: TensorSpec((rg, d)), n["g2"]: TensorSpec((H * dv, rg)),
                n["o"]: TensorSpec((d, H * dv))}

    def _channels(self):
        p = self.params
        return 2 * p["kv_heads"] * p["dim"] + p["heads"] * p["vdim"]

    def cache_need(self):
        p = self.params
        state = StateNeed((p["heads"], p["dim"], p["vdim"]), torch.float32)
        if p["conv"] <= 1:
            return state
        return (state, StateNeed((p["conv"] - 1, self._channels()), torch.float32))

    def bind(self, tensors, rt):
        self.rt = rt
        p, n = self.params, self.names
        self.H, self.G, self.dk, self.dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
        self.taps, self.eps = int(p["conv"]), float(p["eps"])
        self.ra, self.rg = p["decay_rank"], p["gate_rank"]
        if self.H % self.G:
            raise ValueError(f"{self.H} heads are no multiple of {self.G} query/key heads")
        self.C = self._channels()
        ws = [tensors[n[r]] for r in ("q", "k", "v", "a1", "g1", "b")]
        if len({w.dtype for w in ws}) != 1:
            ws = [w.float() for w in ws]
        rows = sum(w.shape[0] for w in ws)
        if rows % 8:     # rows of the stacked product start at multiples of 16 bytes
            ws.append(torch.zeros(8 - rows % 8, ws[0].shape[1], dtype=ws[0].dtype, device=ws[0].device))
        self.w_in = rt.weight(torch.cat(ws, dim=0))
        self.w_a2, self.w_g2, self.w_o = (rt.weight(tensors[n[r]]) for r in ("a2", "g2", "o"))
        f = lambda r: tensors[n[r]].float().contiguous()
        self.taps_w = torch.cat([f("q_conv"), f("k_conv"), f("v_conv")], dim=0).contiguous()
        self.dt_bias, self.a_log, self.norm_w = f("dt_bias"), f("A_log"), f("norm")
        self.no_hist = torch.zeros(1, dtype=torch.float32, device=rt.device)

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in (self.w_in, self.w_a2, self.w_g2, self.w_o))

    def step_flops(self, rows):
        return 2 * rows * sum(w.w.numel() for w in (self.w_in, self.w_a2, self.w_g2, self.w_o))

    def mixing_flops(self, past, new):
        return 7 * self.H * self.dk * self.dv * new

    @staticmethod
    def _aligned(t):
        return t if t.data_ptr() % 16 == 0 and t.stride(0) % 8 == 0 else t.contiguous()

    def forward(self, x, step, view):
        return self.output(self.scan(self.project(x, step, view), step, view))

    def project(self, x, step, view):
        """The stacked projection, the convolutions with their activations and unit norms (which also move the
        sequences' convolution history on), and the two low-rank projections' second halves."""
        rt, C = self.rt, self.C
        hist = view[1].tensor if isinstance(view, tuple) else self.no_hist
        proj = rt.linear(x, self.w_in)           # [T, q | k | v | a1 | g1 | b | padding]
        qkv = torch.empty(x.shape[0], C, dtype=torch.float32, device=x.device)
        rt.ops.conv_prepare(proj, self.taps_w, hist, qkv, step, C, self.G, self.dk)
        decay_in = rt.linear(self._aligned(proj[:, C:C + self.ra]), self.w_a2)
        gate_in = rt.linear(self._aligned(proj[:, C + self.ra:C + self.ra + self.rg]), self.w_g2)
        return proj, qkv, decay_in, gate_in

    def scan(self, projected, step, view):
        """The recurrence over the step's tokens, each sequence from its own state -> [tokens, heads * vdim]."""
        rt = self.rt
        proj, qkv, decay_in, gate_in = projected
        state = view[0].tensor if isinstance(view, tuple) else view.tensor
        T = qkv.shape[0]
        o_raw = torch.zeros(T, self.H * self.dv, dtype=torch.float32, device=qkv.device)
        out = torch.empty(T, self.H * self.dv, dtype=rt.dtype, device=qkv.device)
        return rt.ops.delta_scan(qkv, proj, self.C + self.ra + self.rg, decay_in, self.dt_bias, self.a_log, gate_in,
                                 self.norm_w, self.eps, state, o_raw, out, step, self.H, self.G, self.dk, self.dv)

    def output(self, mixed):
        return self.rt.linear(mixed, self.w_o, partials=True)

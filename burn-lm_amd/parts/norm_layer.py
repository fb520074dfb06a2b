"""Layer norm with weight and bias over a residual kept as several streams.

``y = (u - mean(u)) / sqrt(var(u) + eps) * weight + bias`` with the variance as the mean of the squared
deviations; mean, variance and scaling are float32.  The residual is float32 ``[tokens, streams, width]``
(one stream is the plain residual); ``u`` is read out of the streams with one coefficient per stream, after
the result of the sublayer before has been written into them (`Pending`), all in one kernel."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .base import Norm, TensorSpec


@dataclass
class Pending:
    """A sublayer's result that is not in the streams yet: ``x'_t = sum_s mix[s, t] x_s + write[t] * y * scale``.
    y: [tokens, width] in the activation dtype, or float32 planes [planes, tokens, width] to be summed."""
    y: torch.Tensor
    scale: torch.Tensor   # float32 [width]
    mix: torch.Tensor     # float32 [streams, streams], indexed [from, to]
    write: torch.Tensor   # float32 [streams]

    def as_tuple(self):
        return self.y, self.scale, self.mix, self.write


class LayerNorm(Norm):
    """params: width, eps, streams (default 1), out_scale (default 1: the normalised rows are multiplied by it).
    names: weight, bias."""
    graph_safe = True

    def tensor_specs(self):
        d = self.params["width"]
        return {self.names["weight"]: TensorSpec((d,)), self.names["bias"]: TensorSpec((d,))}

    def bind(self, tensors, rt):
        self.rt = rt
        self.gamma = tensors[self.names["weight"]].float().contiguous()
        self.beta = tensors[self.names["bias"]].float().contiguous()
        self.eps = float(self.params["eps"])
        self.streams = int(self.params.get("streams", 1))
        self.out_scale = float(self.params.get("out_scale", 1.0))
        self._ones = None     # the trivial layer scale, mixing matrix and write coefficient of a plain delta

    def step_bytes(self, rows):
        return 2 * self.gamma.numel() * 4

    def read_streams(self, h, pending, read, out_dtype, rows=None, write_h=True, stash=None):
        """Writes `pending` into the streams h (kept if write_h), reads ``u = sum_t read[t] h_t`` (read None: the
        plain sum) and returns its layer norm in out_dtype for all rows or the listed ones."""
        x = h if h.dim() == 3 else h.unsqueeze(1)
        if x.shape[1] != self.streams:
            raise ValueError(f"the residual has {x.shape[1]} streams, this norm was built for {self.streams}")
        n = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty(n, x.shape[2], dtype=out_dtype, device=x.device)
        return self.rt.ops.streams_norm(x, out, self.gamma, self.beta, self.eps, read=read,
                                        pending=None if pending is None else pending.as_tuple(), rows=rows,
                                        write_x=write_h, out_scale=self.out_scale, stash=stash)

    def add_norm(self, h, delta, rows=None, write_h=True, out_dtype=None):
        """The norm of the sum of the streams, after `delta` (None, a Pending, or with one stream a plain result:
        [tokens, width] or float32 planes) has been written into them; out_dtype: the activation dtype unless given."""
        if delta is not None and not isinstance(delta, Pending):
            if self.streams != 1:
                raise ValueError("a plain delta can only be added to a residual of one stream")
            if self._ones is None or self._ones[0].device != h.device:
                one = torch.ones(1, dtype=torch.float32, device=h.device)
                self._ones = (torch.ones(h.shape[-1], dtype=torch.float32, device=h.device), one.view(1, 1), one)
            delta = Pending(delta, *self._ones)
        return self.read_streams(h, delta, None, out_dtype or self.rt.dtype, rows=rows, write_h=write_h)

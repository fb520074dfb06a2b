"""Residual connections with several streams (hyper-connections), with layer scale and token shift, and
the block that arranges a mixer and a feed-forward around them.

Instead of one residual ``x`` there are ``s`` streams ``x_1 .. x_s`` (equal at the start).  A sublayer reads
``u = sum_s read[s] x_s``, runs on the norm of ``u``, and its result ``y`` (times a per-channel layer scale)
goes back as ``x_t <- sum_s mix[s, t] x_s + write[t] y`` for all t at once.  Token shift: the normalised rows
that a sublayer reads are first blended with those of the token before, ``n_t + (n_{t-1} - n_t) * mu``
(zeros before a sequence's first token); the last token's ``n`` is kept per sequence as fixed-size state.
The write of ``y`` is deferred to the next read, so write, read and norm are one kernel."""
from __future__ import annotations

import torch

from .base import Block, Part, StateNeed, TensorSpec
from .norm_layer import Pending


class HyperConnection(Part):
    """params: width, streams, shift (whether the rows read are blended with the token before).
    names: read [streams], write [streams], mix [streams, streams], scale [width], shift [width] (if shift)."""
    graph_safe = True

    def tensor_specs(self):
        p, n = self.params, self.names
        s, d = p["streams"], p["width"]
        specs = {n["read"]: TensorSpec((s,)), n["write"]: TensorSpec((s,)), n["mix"]: TensorSpec((s, s)),
                 n["scale"]: TensorSpec((d,))}
        if p.get("shift"):
            specs[n["shift"]] = TensorSpec((d,))
        return specs

    def bind(self, tensors, rt):
        self.rt = rt
        f = lambda role: tensors[self.names[role]].float().contiguous()
        self.read_w, self.write_w, self.mix, self.scale = f("read"), f("write"), f("mix"), f("scale")
        self.shift = f("shift") if self.params.get("shift") else None

    def step_bytes(self, rows):
        return 4 * (self.read_w.numel() + self.write_w.numel() + self.mix.numel() + self.scale.numel()
                    + (self.shift.numel() if self.shift is not None else 0))

    def cache_need(self):
        return StateNeed((self.params["width"],), torch.float32) if self.params.get("shift") else None

    def read(self, h, pending, norm, step, view):
        """The sublayer's input rows in the activation dtype: `pending` written into the streams, the read-out,
        the norm, and the shift (view: the StateView of the sequences' last normalised rows)."""
        rt = self.rt
        if self.shift is None:
            return norm.read_streams(h, pending, self.read_w, rt.dtype)
        stash = torch.empty(step.n_seqs, h.shape[-1], dtype=torch.float32, device=h.device)
        n = norm.read_streams(h, pending, self.read_w, torch.float32, stash=(view.tensor, stash, step))
        out = torch.empty(n.shape, dtype=rt.dtype, device=h.device)
        return rt.ops.token_shift(n, self.shift, stash, view.tensor, out, step)

    def pend(self, y):
        return Pending(y, self.scale, self.mix, self.write_w)


def _flat(need):
    return [] if need is None else (list(need) if isinstance(need, (tuple, list)) else [need])


class HyperBlock(Block):
    """Pre-norm layer over several streams: mixer, then feed-forward, each with its connection and norm."""
    roles = {"mixer_link": "connection", "mixer_norm": "norm", "mixer": "mixer",
             "ffn_link": "connection", "ffn_norm": "norm", "feed_forward": "feed_forward"}

    def cache_need(self):
        return tuple(_flat(self.mixer_link.cache_need()) + _flat(self.mixer.cache_need()))

    def _views(self, view):
        views = list(view) if isinstance(view, (tuple, list)) else [view]
        n_link = len(_flat(self.mixer_link.cache_need()))
        link_view = views[0] if n_link else None
        need, rest = self.mixer.cache_need(), views[n_link:]
        mixer_view = tuple(rest) if isinstance(need, (tuple, list)) else (rest[0] if rest else None)
        return link_view, mixer_view

    def forward(self, h, delta, step, view):
        link_view, mixer_view = self._views(view)
        x = self.mixer_link.read(h, delta, self.mixer_norm, step, link_view)
        pending = self.mixer_link.pend(self.mixer.forward(x, step, mixer_view))
        return self._feed_forward(h, pending, step)

    def _feed_forward(self, h, pending, step):
        x = self.ffn_link.read(h, pending, self.ffn_norm, step, None)
        return self.ffn_link.pend(self.feed_forward.forward(x, step))


class HyperMixerBlock(HyperBlock):
    """The same without a feed-forward."""
    roles = {"mixer_link": "connection", "mixer_norm": "norm", "mixer": "mixer"}

    def _feed_forward(self, h, pending, step):
        return pending

"""Attention whose keys and values are expanded from one low-rank latent per token (latent attention).

``q = W_q x`` per head as ``[dim plain lanes | rot_dim lanes turned by position]``; ``W_dkv x`` gives the latent
``c`` (kv_rank lanes, RMS-normed with a weight) and one turned key part shared by all heads (rot_dim lanes).
A head's plain key is ``W_uk c`` and its value ``W_uv c``; score = (q_plain . k_plain + q_rot . k_rot) * scale,
causal softmax, output projection over the concatenated heads.  Only ``[c | k_rot]`` is cached: the scores are
computed as ``(W_uk^T q_plain) . c`` and the values applied as ``W_uv (sum_j p_j c_j)``, which is the same
function, so the cache holds one row of kv_rank + rot_dim lanes per token for all heads and no value pages.
Rotation: lane i of the first ``rot_dims`` turned lanes pairs with lane i + rot_dims/2."""
from __future__ import annotations

import os

import torch

from .base import KVNeed, Mixer, TensorSpec

DECODE_BLOCKS_PER_UNIT = 2     # blocks of four (token, head) wavefronts the split decode aims for per compute unit
MFMA_MAX_PIECES = 64           # most pieces the matrix-core decode cuts a sequence's pages into


class LatentAttention(Mixer):
    """params: width, heads, dim, rot_dim, vdim, kv_rank, scale, rot_dims, eps, position (the rotary table's
    owner, given by the model builder).  names: q, dkv, dkv_norm, uk, uv, o."""
    graph_safe = True

    def tensor_specs(self):
        p, n = self.params, self.names
        d, H, dn, dr, dv, R = p["width"], p["heads"], p["dim"], p["rot_dim"], p["vdim"], p["kv_rank"]
        return {n["q"]: TensorSpec((H * (dn + dr), d)), n["dkv"]: TensorSpec((R + dr, d)),
                n["dkv_norm"]: TensorSpec((R,)), n["uk"]: TensorSpec((H * dn, R)), n["uv"]: TensorSpec((H * dv, R)),
                n["o"]: TensorSpec((d, H * dv))}

    def cache_need(self):
        """One row [latent | turned key part] per token for all heads.  Where the matrix-core attention runs
        (bfloat16, sizes it is built for) the latent is kept a second time, transposed, as the value pages."""
        p = self.params
        if getattr(self, "use_mfma", False):
            return KVNeed(1, p["kv_rank"] + p["rot_dim"], 0, value_dim=p["kv_rank"])
        return KVNeed(1, p["kv_rank"] + p["rot_dim"], 0, no_values=True)

    def bind(self, tensors, rt):
        self.rt = rt
        p, n = self.params, self.names
        self.H, self.dn, self.dr, self.dv, self.R = p["heads"], p["dim"], p["rot_dim"], p["vdim"], p["kv_rank"]
        self.scale, self.eps, self.rot = float(p["scale"]), float(p["eps"]), int(p["rot_dims"])
        if self.rot % 2 or not 0 <= self.rot <= self.dr:
            raise ValueError(f"{self.rot} turning lanes do not fit a turned part of {self.dr} lanes")
        self.position = p["position"]
        ws = [tensors[n["q"]], tensors[n["dkv"]]]
        if ws[0].dtype != ws[1].dtype:
            ws = [w.float() for w in ws]
        self.n_q = ws[0].shape[0]
        self.w_in = rt.weight(torch.cat(ws, dim=0))
        self.norm_w = tensors[n["dkv_norm"]].float().contiguous()
        H, dn, dv, R = self.H, self.dn, self.dv, self.R
        self.w_uk_t = tensors[n["uk"]].view(H, dn, R).transpose(1, 2).contiguous()   # [H, R, dn]: q_plain -> latent lanes
        self.w_uv = tensors[n["uv"]].view(H, dv, R).contiguous()
        self.w_o = rt.weight(tensors[n["o"]])
        rt.ops.latent_attn_init(rt.device)
        self.use_mfma = (os.environ.get("BURN_LM_AMD_LATENT_MFMA") != "0" and self.w_uk_t.dtype == torch.bfloat16
                         and rt.ops.latent_attn_mfma_supported(rt.dtype, R, self.dr))

    def step_bytes(self, rows):
        return sum(w.numel() * w.element_size() for w in (self.w_in.w, self.w_o.w, self.w_uk_t, self.w_uv))

    def step_flops(self, rows):
        return 2 * rows * (self.w_in.w.numel() + self.w_o.w.numel() + self.w_uk_t.numel() + self.w_uv.numel())

    def mixing_flops(self, past, new):
        """Scores over kv_rank + rot_dim lanes and weighted latents over kv_rank lanes, per (query, visible row, head)."""
        pairs = new * past + new * (new + 1) // 2
        return 2 * self.H * (2 * self.R + self.dr) * pairs

    def forward(self, x, step, view):
        return self.output(self.attend(self.project(x, step, view), step, view))

    def project(self, x, step, view):
        """The absorbed queries [tokens, heads, kv_rank + rot_dim] (float32) of the step's tokens; their latents and
        turned key parts are in the cache afterwards."""
        rt, ops = self.rt, self.rt.ops
        H, dn, dr, R = self.H, self.dn, self.dr, self.R
        T = x.shape[0]
        qd = rt.linear(x, self.w_in)                         # [T, H (dn + dr) | R + dr]
        q, down = qd[:, :self.n_q], qd[:, self.n_q:]
        mfma = self.use_mfma and view.v.numel() > 0 and view.page_size == 64
        qabs = torch.empty(T, H, R + dr, dtype=rt.dtype if mfma else torch.float32, device=x.device)
        ops.latent_write(down, q, self.norm_w, self.eps, self.position.table, self.rot, qabs, view.k, step,
                         view.block_table(step), view.page_size, H, dn, R, dr, write_kv=view.store,
                         vcache=view.v if mfma else None)
        ops.head_project(q, dn + dr, self.w_uk_t, qabs.view(T, H * (R + dr)), R + dr)
        return qabs

    def attend(self, qabs, step, view):
        """Every (token, head)'s weighted sum of the latents it sees -> float32 [tokens, heads, kv_rank]."""
        rt, ops = self.rt, self.rt.ops
        H, dr, R = self.H, self.dr, self.R
        T = qabs.shape[0]
        olat = torch.empty(T, H, R, dtype=torch.float32, device=qabs.device)
        n_splits = 1
        if qabs.dtype == torch.bfloat16:        # the matrix-core form: one wavefront per 16 (token, head) pairs
            if step.max_new == 1:
                waves = step.n_seqs * ((H + 15) // 16)
                pages = (step.max_len_after + 63) // 64
                # up to a wavefront for every vector unit of the chip: a wavefront waits out a page's trip from memory
                # with nothing else to do, so short pieces are what shortens the step
                n_splits = max(1, min(pages, (4 * rt.compute_units) // waves, MFMA_MAX_PIECES,
                                      ops.latent_attn_mfma_max_splits(step.n_seqs, 1, H, R)))
            return ops.latent_attn_mfma(qabs, olat, view.k, view.v, step, view.block_table(step), view.page_size, H, R,
                                        dr, self.scale, n_splits)
        if step.max_new == 1:
            chunks = (step.max_len_after + 63) // 64
            blocks = (T * H + 3) // 4
            n_splits = max(1, min(chunks, (DECODE_BLOCKS_PER_UNIT * rt.compute_units) // blocks,
                                  ops.latent_attn_max_splits(T, H, R)))
        return ops.latent_attn(qabs, olat, view.k, step, view.block_table(step), view.page_size, H, R, dr, self.scale,
                               n_splits)

    def output(self, olat):
        rt = self.rt
        T = olat.shape[0]
        o = torch.empty(T, self.H * self.dv, dtype=rt.dtype, device=olat.device)
        rt.ops.head_project(olat.view(T, self.H * self.R), self.R, self.w_uv, o, self.dv)
        return rt.linear(o, self.w_o, partials=True)

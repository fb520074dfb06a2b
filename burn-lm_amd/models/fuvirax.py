"""The Fuvirax design as a plan of parts.

A decoder over several residual streams (hyper-connections): every layer is a mixer and (usually) a dense xIELU
feed-forward, each read through a layer norm with bias, scaled per channel on the way back, the mixer's input
blended with the token before (token shift).  Mixers, chosen layer by layer: latent attention, HGRN2, and a delta
rule with per-channel decay.  A range of layers may run several times in a row with the same weights; every run is
a place of its own in the order and keeps its own cache and state.  The output is the layer norm of the summed
streams times the embedding table, times ``logit_scale``.

Checkpoint tensor names: ``embed``; per layer i ``l<i>.norm1`` (+ ``.b``), ``l<i>.norm2`` (+ ``.b``), ``l<i>.ls1/2``,
``l<i>.shift``, ``l<i>.hc1/2.in|out|mix``, ``l<i>.mix.*``, ``l<i>.mlp.up|down|act``; ``final.norm`` (+ ``.b``)."""
from __future__ import annotations

from ..config.fuvirax import DEFAULT_LOW_RANK, MAX_POSITIONS, FuviraxConfig
from ..parts.base import PartSpec
from ..registry import Architecture, register_architecture
from ..weights.random_init import Normal, Ones, Uniform
from .plan import LayerPlan, ModelPlan, Place



def _shape_of(checkpoint, name):
    """Shape of a tensor in the checkpoint (a mapping name -> shape), or None."""
    if isinstance(checkpoint, dict) and checkpoint.get(name) is not None:
        return tuple(checkpoint[name])
    return None


def _ranks(m, prefix, checkpoint):
    """Inner widths of the delta mixer's two low-rank projections: from the checkpoint's shapes, else from the
    configuration, else the default of fresh random weights."""
    a1, g1 = _shape_of(checkpoint, prefix + "a1"), _shape_of(checkpoint, prefix + "g1")
    return (a1[0] if a1 else m.decay_rank or DEFAULT_LOW_RANK), (g1[0] if g1 else m.gate_rank or DEFAULT_LOW_RANK)


def _mixer(cfg, i, m, checkpoint, positions):
    p = f"l{i}.mix."
    D = cfg.width
    if m.type == "latent_attention":
        key = f"rope_{m.rot_dim}_{m.rot_dims}_{m.rot_base!r}"
        positions.setdefault(key, PartSpec("rope", dict(head_dim=m.rot_dim, theta=m.rot_base, pairing="half",
                                                        rotary_dim=m.rot_dims, scaling=None)))
        spec = PartSpec("latent_attention",
                        dict(width=D, heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim, kv_rank=m.kv_rank,
                             scale=m.scale, rot_dims=m.rot_dims, eps=cfg.eps),
                        dict(q=p + "q", dkv=p + "dkv", dkv_norm=p + "dkv.norm", uk=p + "uk", uv=p + "uv", o=p + "o"))
        return spec, key
    if m.type == "hgrn2":
        return PartSpec("hgrn2", dict(width=D, heads=m.heads, dim=m.dim, vdim=m.vdim, eps=cfg.eps),
                        dict(q=p + "q", f=p + "f", f_bias=p + "f.b", lower=p + "lower", v=p + "v", norm=p + "norm",
                             o=p + "o")), None
    ra, rg = _ranks(m, p, checkpoint)
    return PartSpec("channel_delta",
                    dict(width=D, heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, conv=m.conv,
                         decay_rank=ra, gate_rank=rg, eps=cfg.eps),
                    dict(q=p + "q", k=p + "k", v=p + "v", q_conv=p + "q.conv", k_conv=p + "k.conv", v_conv=p + "v.conv",
                         b=p + "b", A_log=p + "A_log", norm=p + "norm", a1=p + "a1", a2=p + "a2", dt_bias=p + "dt_bias",
                         g1=p + "g1", g2=p + "g2", o=p + "o")), None


def plan(cfg: FuviraxConfig, checkpoint=None) -> ModelPlan:
    D, S = cfg.width, cfg.streams
    positions = {}
    layers = []
    norm = lambda name, **kw: PartSpec("layernorm", dict(width=D, eps=cfg.eps, streams=S, **kw),
                                       dict(weight=name, bias=name + ".b"))
    for i, layer in enumerate(cfg.layers):
        l = f"l{i}."
        link = lambda q, shift: PartSpec("hyper", dict(width=D, streams=S, shift=shift),
                                         dict(read=f"{l}hc{q}.in", write=f"{l}hc{q}.out", mix=f"{l}hc{q}.mix",
                                              scale=f"{l}ls{q}", shift=l + "shift"))
        mixer, position = _mixer(cfg, i, layer.mixer, checkpoint, positions)
        parts = dict(mixer_link=link(1, True), mixer_norm=norm(l + "norm1"), mixer=mixer)
        if layer.ff is None:
            layers.append(LayerPlan("hyper_mixer_only", parts, position=position))
            continue
        parts.update(ffn_link=link(2, False), ffn_norm=norm(l + "norm2"),
                     feed_forward=PartSpec("dense_xielu", dict(width=D, inner=layer.ff),
                                           dict(up=l + "mlp.up", down=l + "mlp.down", act=l + "mlp.act")))
        layers.append(LayerPlan("hyper", parts, position=position))
    ignorable = [rf"^l{i}\.(norm2(\.b)?|ls2|hc2\.(in|out|mix))$" for i, layer in enumerate(cfg.layers) if layer.ff is None]
    return ModelPlan(
        vocab_size=cfg.vocab, width=D, max_positions=MAX_POSITIONS,
        embedding=PartSpec("table", dict(vocab=cfg.vocab, width=D, copies=S), dict(weight="embed")),
        layers=layers, order=[Place(i) for i in cfg.order()],
        final_norm=norm("final.norm", out_scale=cfg.logit_scale),
        head=PartSpec("linear", dict(vocab=cfg.vocab, width=D), dict(weight="embed")),
        positions=positions, stop_ids=(), ignorable_tensors=tuple(ignorable))


def checkpoint_tensors(cfg: FuviraxConfig):
    """Name -> (shape, initialiser) of a fresh checkpoint: matrices N(0, 1/sqrt(fan-in)), norms near one, the
    streams' mixing matrices near the identity, gates and decays in the range where the recurrences neither
    forget at once nor never."""
    D, S = cfg.width, cfg.streams
    lin = lambda n_out, n_in: ((n_out, n_in), Normal(n_in ** -0.5))
    out = {"embed": ((cfg.vocab, D), Normal(1.0, layout="table"))}
    for i, layer in enumerate(cfg.layers):
        l, m = f"l{i}.", layer.mixer
        for q in (1, 2) if layer.ff is not None else (1,):
            out[f"{l}norm{q}"] = ((D,), Ones(0.1))
            out[f"{l}norm{q}.b"] = ((D,), Normal(0.05))
            out[f"{l}ls{q}"] = ((D,), Uniform(0.3, 1.0))
            out[f"{l}hc{q}.in"] = ((S,), Uniform(0.1, 0.6))
            out[f"{l}hc{q}.out"] = ((S,), Uniform(0.2, 1.0))
            out[f"{l}hc{q}.mix"] = ((S, S), Uniform(0.0, 2.0 / S))
        out[l + "shift"] = ((D,), Uniform(0.0, 1.0))
        p = l + "mix."
        if m.type == "latent_attention":
            out[p + "q"] = lin(m.heads * (m.dim + m.rot_dim), D)
            out[p + "dkv"] = lin(m.kv_rank + m.rot_dim, D)
            out[p + "dkv.norm"] = ((m.kv_rank,), Ones(0.1))
            out[p + "uk"] = lin(m.heads * m.dim, m.kv_rank)
            out[p + "uv"] = lin(m.heads * m.vdim, m.kv_rank)
            out[p + "o"] = lin(D, m.heads * m.vdim)
        elif m.type == "hgrn2":
            out[p + "q"] = lin(m.heads * m.dim, D)
            out[p + "f"] = lin(m.heads * m.dim, D)
            out[p + "f.b"] = ((m.heads * m.dim,), Normal(0.5))
            out[p + "lower"] = ((m.heads * m.dim,), Uniform(0.0, 0.9))
            out[p + "v"] = lin(m.heads * m.vdim, D)
            out[p + "norm"] = ((m.vdim,), Ones(0.1))
            out[p + "o"] = lin(D, m.heads * m.vdim)
        else:
            ra, rg = _ranks(m, p, None)
            out[p + "q"] = lin(m.kv_heads * m.dim, D)
            out[p + "q.conv"] = ((m.kv_heads * m.dim, m.conv), Normal(m.conv ** -0.5))
            out[p + "k"] = lin(m.kv_heads * m.dim, D)
            out[p + "k.conv"] = ((m.kv_heads * m.dim, m.conv), Normal(m.conv ** -0.5))
            out[p + "v"] = lin(m.heads * m.vdim, D)
            out[p + "v.conv"] = ((m.heads * m.vdim, m.conv), Normal(m.conv ** -0.5))
            out[p + "b"] = lin(m.heads, D)
            out[p + "A_log"] = ((m.heads,), Uniform(-3.0, 0.5))
            out[p + "norm"] = ((m.vdim,), Ones(0.1))
            out[p + "a1"] = lin(ra, D)
            out[p + "a2"] = lin(m.heads * m.dim, ra)
            out[p + "dt_bias"] = ((m.heads * m.dim,), Uniform(-4.0, 0.0))
            out[p + "g1"] = lin(rg, D)
            out[p + "g2"] = lin(m.heads * m.vdim, rg)
            out[p + "o"] = lin(D, m.heads * m.vdim)
        if layer.ff is not None:
            out[l + "mlp.up"] = lin(layer.ff, D)
            out[l + "mlp.down"] = lin(D, layer.ff)
            out[l + "mlp.act"] = ((2,), Normal(0.5))
    out["final.norm"] = ((D,), Ones(0.1))
    out["final.norm.b"] = ((D,), Normal(0.05))
    return out


FUVIRAX = Architecture(name="Fuvirax", read_config=FuviraxConfig.from_dict, plan=plan,
                       checkpoint_tensors=checkpoint_tensors, display_name="Fuvirax", created_by="")
register_architecture(FUVIRAX, "fuvirax")

"""The Digasun design as a plan of parts.

A decoder whose layers run their mixer and their feed-forward side by side on the same rows: one layer norm with
bias, a short causal convolution added to what each sublayer reads, the mixer (attention with a window, a softmax
sink and head mixing, some layers borrowing an earlier layer's keys and values; or gated linear attention) beside a
clamped dense feed-forward or a mixture of experts with a shared expert, then a gated side input per token from a
second embedding table.  The embedding is scaled; the output is the layer norm of the residual times a head matrix
of its own.

Checkpoint tensor names: ``embed``, ``side.embed``, ``head``, ``final.norm`` (+ ``.b``); per layer i ``l<i>.norm1``
(+ ``.b``), ``l<i>.canon1/2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.side.gate|proj|norm``."""
from __future__ import annotations

from ..config.digasun import DEFAULT_DECAY_RANK, MAX_POSITIONS, DigasunConfig
from ..parts.base import PartSpec
from ..registry import Architecture, register_architecture
from ..weights.random_init import Normal, Ones, Uniform
from .plan import LayerPlan, ModelPlan, Place


def _shape_of(checkpoint, name):
    if isinstance(checkpoint, dict) and checkpoint.get(name) is not None:
        return tuple(checkpoint[name])
    return None


def _decay_rank(m, prefix, checkpoint):
    a1 = _shape_of(checkpoint, prefix + "a1")
    return a1[0] if a1 else m.decay_rank or DEFAULT_DECAY_RANK


def _cache_window(cfg, i):
    """What layer i's cache must keep: the largest window among the layer and those that read its keys and values
    (0, everything, if one of them sees every earlier key)."""
    windows = [cfg.layers[i].mixer.window] + [l.mixer.window for l in cfg.layers
                                              if l.mixer.type == "attention" and l.mixer.kv_from == i]
    return 0 if 0 in windows else max(windows)


def _mixer(cfg, i, checkpoint, positions):
    m, p, D = cfg.layers[i].mixer, f"l{i}.mix.", cfg.width
    if m.type == "gla":
        return PartSpec("gla", dict(width=D, heads=m.heads, dim=m.dim, vdim=m.vdim, tau=m.tau, eps=cfg.eps,
                                    decay_rank=_decay_rank(m, p, checkpoint)),
                        dict(q=p + "q", k=p + "k", v=p + "v", g=p + "g", a1=p + "a1", a2=p + "a2", a2_bias=p + "a2.b",
                             norm=p + "norm", o=p + "o")), None
    key = None
    if m.rot_dims:
        key = f"rope_{m.rot_dims}_{m.rot_base!r}"
        positions.setdefault(key, PartSpec("rope", dict(head_dim=m.rot_dims, theta=m.rot_base, pairing="half",
                                                        scaling=None)))
    borrows = m.kv_from is not None
    names = dict(q=p + "q", q_bias=p + "q.b", o=p + "o", o_bias=p + "o.b", sink=p + "sink", talk=p + "talk")
    if not borrows:
        names.update(k=p + "k", k_bias=p + "k.b", v=p + "v", v_bias=p + "v.b")
    src = m.kv_from if borrows else i
    return PartSpec("sink_attention",
                    dict(width=D, heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale,
                         window=m.window, cache_window=_cache_window(cfg, src), rot_dims=m.rot_dims, borrows=borrows),
                    names), key


def _feed_forward(cfg, i):
    f, p, D = cfg.layers[i].mlp, f"l{i}.mlp.", cfg.width
    if f.kind == "dense":
        return PartSpec("clamped_glu", dict(width=D, inner=f.ff, limit=f.limit, alpha=1.702),
                        dict(gate=p + "gate", up=p + "up", down=p + "down"))
    names = dict(router=p + "router", router_bias=p + "router.b")
    for e in range(f.experts):
        names.update({f"e{e}.{r}": f"{p}e{e}.{r}" for r in ("gate", "up", "down")})
    if f.shared_ff:
        names.update({f"shared.{r}": f"{p}shared.{r}" for r in ("gate", "up", "down", "sg")})
    return PartSpec("routed_experts", dict(width=D, experts=f.experts, top=f.top, expert_inner=f.ff,
                                           shared_inner=f.shared_ff), names)


def plan(cfg: DigasunConfig, checkpoint=None) -> ModelPlan:
    D, L = cfg.width, len(cfg.layers)
    positions = {}
    layers = []
    norm = lambda name: PartSpec("layernorm", dict(width=D, eps=cfg.eps), dict(weight=name, bias=name + ".b"))
    for i, layer in enumerate(cfg.layers):
        l = f"l{i}."
        mixer, position = _mixer(cfg, i, checkpoint, positions)
        readers = 2 if layer.mlp is not None else 1
        parts = dict(norm=norm(l + "norm1"),
                     input=PartSpec("causal_conv", dict(width=D, taps=cfg.taps, readers=readers),
                                    {f"w{r}": f"{l}canon{r + 1}" for r in range(readers)}),
                     mixer=mixer,
                     side=PartSpec("token_side", dict(width=D, dim=cfg.side_dim, vocab=cfg.vocab, columns=L * cfg.side_dim,
                                                      column=i * cfg.side_dim, eps=cfg.eps),
                                   dict(table="side.embed", gate=l + "side.gate", proj=l + "side.proj", norm=l + "side.norm")))
        if layer.mlp is None:
            layers.append(LayerPlan("parallel_mixer_only", parts, position=position))
        else:
            parts["feed_forward"] = _feed_forward(cfg, i)
            layers.append(LayerPlan("parallel", parts, position=position))
    order = [Place(i, reads_cache_of=layer.mixer.kv_from if layer.mixer.type == "attention" else None)
             for i, layer in enumerate(cfg.layers)]
    ignorable = [rf"^l{i}\.canon2$" for i, layer in enumerate(cfg.layers) if layer.mlp is None]
    return ModelPlan(
        vocab_size=cfg.vocab, width=D, max_positions=MAX_POSITIONS,
        embedding=PartSpec("table", dict(vocab=cfg.vocab, width=D, scale=cfg.embedding_scale), dict(weight="embed")),
        layers=layers, order=order, final_norm=norm("final.norm"),
        head=PartSpec("linear", dict(vocab=cfg.vocab, width=D), dict(weight="head")),
        positions=positions, stop_ids=(), ignorable_tensors=tuple(ignorable))


def checkpoint_tensors(cfg: DigasunConfig):
    """Name -> (shape, initialiser) of a fresh checkpoint: matrices N(0, 1/sqrt(fan-in)), norms near one, sinks and
    router biases of a size that matters, the heads' mixing matrices near the identity, decays in the range where
    the recurrence neither forgets at once nor never."""
    D, L = cfg.width, len(cfg.layers)
    lin = lambda n_out, n_in: ((n_out, n_in), Normal(n_in ** -0.5))
    out = {"embed": ((cfg.vocab, D), Normal(1.0, layout="table")),
           "side.embed": ((cfg.vocab, L * cfg.side_dim), Normal(1.0, layout="table")),
           "head": lin(cfg.vocab, D), "final.norm": ((D,), Ones(0.1)), "final.norm.b": ((D,), Normal(0.05))}
    for i, layer in enumerate(cfg.layers):
        l, m, f = f"l{i}.", layer.mixer, layer.mlp
        out[l + "norm1"] = ((D,), Ones(0.1))
        out[l + "norm1.b"] = ((D,), Normal(0.05))
        out[l + "canon1"] = ((D, cfg.taps), Normal(cfg.taps ** -0.5))
        if f is not None:
            out[l + "canon2"] = ((D, cfg.taps), Normal(cfg.taps ** -0.5))
        out[l + "side.gate"] = lin(cfg.side_dim, D)
        out[l + "side.proj"] = lin(D, cfg.side_dim)
        out[l + "side.norm"] = ((D,), Uniform(0.2, 0.6))
        p = l + "mix."
        if m.type == "gla":
            r = _decay_rank(m, p, None)
            out[p + "q"], out[p + "k"] = lin(m.heads * m.dim, D), lin(m.heads * m.dim, D)
            out[p + "v"], out[p + "g"] = lin(m.heads * m.vdim, D), lin(m.heads * m.vdim, D)
            out[p + "a1"], out[p + "a2"] = lin(r, D), lin(m.heads * m.dim, r)
            out[p + "a2.b"] = ((m.heads * m.dim,), Uniform(0.0, 4.0))
            out[p + "norm"] = ((m.vdim,), Ones(0.1))
            out[p + "o"] = lin(D, m.heads * m.vdim)
        else:
            out[p + "q"], out[p + "q.b"] = lin(m.heads * m.dim, D), ((m.heads * m.dim,), Normal(0.1))
            if m.kv_from is None:
                out[p + "k"], out[p + "k.b"] = lin(m.kv_heads * m.dim, D), ((m.kv_heads * m.dim,), Normal(0.1))
                out[p + "v"], out[p + "v.b"] = lin(m.kv_heads * m.vdim, D), ((m.kv_heads * m.vdim,), Normal(0.1))
            out[p + "talk"] = ((m.heads, m.heads), Uniform(-0.2, 2.0 / m.heads + 0.2))
            out[p + "sink"] = ((m.heads,), Normal(1.0))
            out[p + "o"], out[p + "o.b"] = lin(D, m.heads * m.vdim), ((D,), Normal(0.05))
        if f is None:
            continue
        p = l + "mlp."
        if f.kind == "dense":
            out[p + "gate"], out[p + "up"], out[p + "down"] = lin(f.ff, D), lin(f.ff, D), lin(D, f.ff)
            continue
        out[p + "router"], out[p + "router.b"] = lin(f.experts, D), ((f.experts,), Normal(0.3))
        for e in range(f.experts):
            out[f"{p}e{e}.gate"], out[f"{p}e{e}.up"], out[f"{p}e{e}.down"] = lin(f.ff, D), lin(f.ff, D), lin(D, f.ff)
        if f.shared_ff:
            out[p + "shared.gate"], out[p + "shared.up"] = lin(f.shared_ff, D), lin(f.shared_ff, D)
            out[p + "shared.down"], out[p + "shared.sg"] = lin(D, f.shared_ff), lin(1, D)
    return out


DIGASUN = Architecture(name="Digasun", read_config=DigasunConfig.from_dict, plan=plan,
                       checkpoint_tensors=checkpoint_tensors, display_name="Digasun", created_by="")
register_architecture(DIGASUN, "digasun")

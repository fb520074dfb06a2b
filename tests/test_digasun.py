"""The Digasun design in the engine against the plain implementation of tests/plain_digasun.py.

The configurations and weights are made here.  The CPU tests cover the configuration reader, the plan, the cache's
lending of keys and values between places with several needs, and the plain implementation's own consistency; the
GPU tests run the engine's step function, cache, scheduler and kernels: every mixer and feed-forward alone, whole
prompts against token-by-token decoding, prompts in portions, unequal batches, slots and pages used again, keys far
back, at page borders and at the edges of the windows (in prompts and in decoding), the sink, long decoding through
recorded graphs, odd sizes, and greedy generation through the server."""
import json
import math

import numpy as np
import pytest
import torch

import plain_digasun as P
from helpers import rel_err

TOL = {"float32": 2e-5, "bfloat16": 8e-2}


class Rows:
    """Collects rows of logits beside what they should be.  float32: every row within the tolerance.  bfloat16: a
    rounding can tip a router's choice between two experts whose logits are close, which changes that token's row by
    far more than roundings do and is no fault, so nine rows in ten must be within the tolerance, and every row finite."""

    def __init__(self, dtype):
        self.dtype, self.errs = dtype, []

    def add(self, got, want, note=None):
        got, want = np.atleast_2d(np.asarray(got, dtype=np.float64)), np.atleast_2d(want)
        assert got.shape == want.shape and np.isfinite(got).all(), note
        scale = max(1e-30, np.abs(want).max())
        self.errs += [(float(np.abs(g - x).max() / scale), note) for g, x in zip(got, want)]

    def check(self):
        tol = TOL[self.dtype]
        bad = [e for e in self.errs if e[0] > tol]
        if self.dtype == "float32":
            assert not bad, bad[:5]
        else:
            assert len(bad) * 10 <= len(self.errs), (len(bad), len(self.errs), bad[:5])


# ---- configurations and weights of the tests --------------------------------------------------
def attn(heads=4, kv_heads=2, dim=16, vdim=24, window=40, rot=12, base=10000.0, kv_from=None, mlp="dense"):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=1.0 / math.sqrt(dim), mask=dict(size=window),
             rot=dict(base=base, dims=rot))
    if kv_from is not None:
        m["kv_from"] = kv_from
    return dict(type="attention", mixer=m, mlp=ff(mlp))


def gla(heads=2, dim=12, vdim=20, tau=8.0, mlp="dense"):
    return dict(type="gla", mixer=dict(heads=heads, dim=dim, vdim=vdim, tau=tau), mlp=ff(mlp))


def ff(kind):
    if kind is None or isinstance(kind, dict):
        return kind
    if kind == "dense":
        return dict(kind="dense", ff=72, limit=1.5)
    if kind == "moe":
        return dict(kind="moe", router=dict(experts=5, top=2), expert=dict(ff=24), shared=dict(ff=40))
    if kind == "moe_top1_no_shared":
        return dict(kind="moe", router=dict(experts=3, top=1), expert=dict(ff=16))
    raise ValueError(kind)


def config(layers, width=48, vocab=101, taps=3, side=6, scale=0.7, eps=1e-5):
    return dict(architecture="Digasun", canon=dict(taps=taps), embedding=dict(scale=scale), layers=layers,
                norm=dict(eps=eps), token_side=dict(dim=side), vocab=vocab, width=width)


# layer 2 borrows layer 1's keys and values and looks further back than layer 1 itself; layer 4 borrows with a
# narrower window; one layer has no feed-forward
MIXED = config([gla(), attn(window=40, mlp="moe"), attn(window=70, kv_from=1, mlp="moe"), gla(mlp=None),
                attn(window=9, kv_from=1, mlp="moe_top1_no_shared")])
# sizes that are no multiples of eight, as many key-value heads as heads and one, keys and values of other sizes
# than each other, lanes that do not turn, two taps and one, one value lane more than a wavefront
ODD = config([attn(heads=3, kv_heads=3, dim=10, vdim=6, window=5, rot=4, mlp="moe_top1_no_shared"),
              gla(heads=3, dim=10, vdim=14, tau=1.0, mlp="moe"),
              attn(heads=5, kv_heads=1, dim=6, vdim=65, window=200, rot=6, base=300.0, mlp=None)],
             width=36, vocab=53, taps=2, side=5, scale=1.3, eps=1e-6)


def make_weights(cfg, seed, rank=5, sharp=1.0):
    """float64 arrays that are exact in bfloat16.  sharp: factor on the query projections of the attention layers,
    so that the softmax singles out few keys."""
    g = np.random.default_rng(seed)
    D, L = cfg["width"], len(cfg["layers"])
    bf = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32)).bfloat16().double().numpy()
    mat = lambda o, i, s=1.0: bf(g.standard_normal((o, i)) * s / math.sqrt(i))
    near_one = lambda n: bf(1 + 0.1 * g.standard_normal(n))
    w = {"embed": bf(g.standard_normal((cfg["vocab"], D))), "final.norm": near_one(D),
         "final.norm.b": bf(0.05 * g.standard_normal(D)), "head": mat(cfg["vocab"], D),
         "side.embed": bf(g.standard_normal((cfg["vocab"], L * cfg["token_side"]["dim"])))}
    taps, sd = cfg["canon"]["taps"], cfg["token_side"]["dim"]
    for i, layer in enumerate(cfg["layers"]):
        l, m, f = f"l{i}.", layer["mixer"], layer["mlp"]
        w[l + "norm1"], w[l + "norm1.b"] = near_one(D), bf(0.05 * g.standard_normal(D))
        w[l + "canon1"] = bf(g.standard_normal((D, taps)) * 0.4)
        if f is not None:
            w[l + "canon2"] = bf(g.standard_normal((D, taps)) * 0.4)
        w[l + "side.gate"], w[l + "side.proj"] = mat(sd, D), mat(D, sd)
        w[l + "side.norm"] = bf(g.uniform(0.2, 0.6, D))
        p = l + "mix."
        if layer["type"] == "gla":
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            w[p + "q"], w[p + "k"], w[p + "v"], w[p + "g"] = mat(H * dk, D), mat(H * dk, D), mat(H * dv, D), mat(H * dv, D)
            w[p + "a1"], w[p + "a2"] = mat(rank, D), mat(H * dk, rank)
            w[p + "a2.b"] = bf(g.uniform(0.0, 4.0, H * dk))
            w[p + "norm"], w[p + "o"] = near_one(dv), mat(D, H * dv)
        else:
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w[p + "q"], w[p + "q.b"] = mat(H * dk, D, sharp), bf(0.1 * g.standard_normal(H * dk))
            if m.get("kv_from") is None:
                w[p + "k"], w[p + "k.b"] = mat(G * dk, D), bf(0.1 * g.standard_normal(G * dk))
                w[p + "v"], w[p + "v.b"] = mat(G * dv, D), bf(0.1 * g.standard_normal(G * dv))
            w[p + "talk"] = bf(np.eye(H) * 0.6 + g.uniform(-0.3, 0.4, (H, H)))
            w[p + "sink"] = bf(g.standard_normal(H))
            w[p + "o"], w[p + "o.b"] = mat(D, H * dv), bf(0.05 * g.standard_normal(D))
        if f is None:
            continue
        p = l + "mlp."
        if f["kind"] == "dense":
            w[p + "gate"], w[p + "up"], w[p + "down"] = mat(f["ff"], D, 2.0), mat(f["ff"], D, 2.0), mat(D, f["ff"])
            continue
        E, fe = f["router"]["experts"], f["expert"]["ff"]
        w[p + "router"], w[p + "router.b"] = mat(E, D, 2.0), bf(0.3 * g.standard_normal(E))
        for e in range(E):
            w[f"{p}e{e}.gate"], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"] = mat(fe, D), mat(fe, D), mat(D, fe)
        if f.get("shared"):
            fs = f["shared"]["ff"]
            w[p + "shared.gate"], w[p + "shared.up"], w[p + "shared.down"] = mat(fs, D), mat(fs, D), mat(D, fs)
            w[p + "shared.sg"] = mat(1, D)
    return w


def write_folder(path, cfg, w):
    from burn_lm_amd.weights import safetensors_io as st
    with open(path / "config.json", "w") as f:
        json.dump(cfg, f)
    st.write_file(str(path / "model.safetensors"), ((k, torch.from_numpy(v).bfloat16()) for k, v in w.items()))
    return str(path)


def tokens_of(cfg, seed, n):
    return [int(x) for x in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


# ---- CPU: configuration, plan, cache, plain implementation --------------------------------------
def test_config_is_read_and_refused_by_key():
    from burn_lm_amd import registry
    from burn_lm_amd.errors import ConfigError
    import burn_lm_amd.models  # noqa: F401
    arch = registry.architecture_of(MIXED)
    assert arch.name == "Digasun"
    cfg = arch.read_config(MIXED)
    assert cfg.layers[2].mixer.kv_from == 1 and cfg.layers[3].mlp is None and cfg.layers[4].mlp.shared_ff == 0
    assert cfg.taps == 3 and cfg.side_dim == 6 and cfg.embedding_scale == 0.7
    for path, value, word in ((("layers", 1, "mixer", "vdim"), None, "vdim"), (("width",), "48", "width"),
                              (("layers", 0, "type"), "mamba", "type"), (("norm",), {}, "eps"),
                              (("layers", 1, "mixer", "kv_heads"), 3, "kv_heads"), (("canon",), None, "taps"),
                              (("layers", 2, "mixer", "kv_from"), 0, "kv_from"), (("layers", 2, "mixer", "kv_from"), 2, "kv_from"),
                              (("layers", 4, "mixer", "kv_from"), 2, "kv_from"), (("layers", 2, "mixer", "vdim"), 8, "differ"),
                              (("layers", 1, "mixer", "rot"), dict(base=10.0, dims=18), "rot"),
                              (("layers", 1, "mlp", "router"), dict(experts=2, top=3), "top"),
                              (("layers", 0, "mlp"), dict(kind="routed", ff=8), "kind")):
        bad = json.loads(json.dumps(MIXED))
        at = bad
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            arch.read_config(bad)


def test_plan_asks_for_the_checkpoints_tensors():
    from burn_lm_amd import registry
    import burn_lm_amd.parts  # noqa: F401
    from burn_lm_amd.engine.model import Model
    for cfg_dict in (MIXED, ODD):
        w = make_weights(cfg_dict, 0)
        arch = registry.architecture_of(cfg_dict)
        cfg = arch.read_config(cfg_dict)
        model = Model(arch.plan(cfg, {k: v.shape for k, v in w.items()}))
        assert {k: tuple(s.shape) for k, s in model.tensor_specs().items()} == {k: tuple(v.shape) for k, v in w.items()}
        assert set(arch.checkpoint_tensors(cfg)) == set(w)
    model = Model(registry.architecture_of(MIXED).plan(registry.architecture_of(MIXED).read_config(MIXED), None))
    assert model.reads_from() == [None, None, 1, None, 1]
    # the lending layer's cache keeps the largest window of those that read it
    needs = model.cache_needs()
    assert needs[1][1].window == 70 and needs[2][1].window == 70 and needs[1][1].value_dim == 24
    assert needs[0][0].shape == (2, 48) and needs[0][1].shape == (2, 12, 20)


def test_cache_lends_keys_between_places_with_several_needs():
    from burn_lm_amd.cache.cache import Cache, CacheError, KVView, StateView
    from burn_lm_amd.parts.base import KVNeed, StateNeed
    kv, st = KVNeed(2, 8, window=16, value_dim=12), StateNeed((3, 4))
    c = Cache([(st, kv), (st, kv), (st, StateNeed((5,))), (st, kv)], [None, 0, None, 0], max_tokens=256, max_seqs=2,
              max_context=128, page_size=64, dtype=torch.float32)
    assert len(c.groups) == 1 and c.groups[0].k_storage.shape[0] == 1       # one plane: the readers keep none
    own, lent = c.views[0][1], c.views[1][1]
    assert isinstance(lent, KVView) and not lent.store and own.store and lent.k.data_ptr() == own.k.data_ptr()
    assert c.views[3][1].v.data_ptr() == own.v.data_ptr() and tuple(own.v.shape[1:]) == (2, 12, 64)
    states = [c.views[i][0] for i in range(4)]
    assert all(isinstance(s, StateView) for s in states) and len({s.tensor.data_ptr() for s in states}) == 4
    with pytest.raises(CacheError, match="keeps keys and values of its own"):
        Cache([(st, kv), (st, kv), (st, kv)], [None, 0, 1], max_tokens=128, max_seqs=2, max_context=128, dtype=torch.float32)
    with pytest.raises(CacheError, match="differ"):
        Cache([(st, kv), (st, KVNeed(2, 8, value_dim=8))], [None, 0], max_tokens=128, max_seqs=2, max_context=128,
              dtype=torch.float32)


def test_random_folder_loads_into_the_plain_implementation(tmp_path):
    import burn_lm_amd
    from burn_lm_amd.weights import safetensors_io as st
    cfg = json.loads(json.dumps(ODD))
    cfg["layers"][1]["mixer"]["decay_rank"] = 4
    folder = burn_lm_amd.write_random_model(str(tmp_path), cfg, seed=5)
    w = {n: f.tensor(n).double().numpy() for n, f in st.open_folder(folder).items()}
    assert w["l1.mix.a1"].shape == (4, 36) and "l2.canon2" not in w and "l2.mix.k" in w
    logits = P.forward(cfg, w, tokens_of(cfg, 0, 9))
    assert logits.shape == (9, 53) and np.isfinite(logits).all() and logits.std() > 0.05


def test_plain_mechanisms_on_cases_worked_by_hand():
    # window: with equal scores and no sink's share to speak of, a query averages exactly the keys it sees
    m = dict(heads=1, kv_heads=1, dim=2, vdim=1, scale=1.0, mask=dict(size=3), rot=dict(base=10.0, dims=2))
    W = {"a.q": np.zeros((2, 2)), "a.q.b": np.zeros(2), "a.sink": np.array([-1e9]), "a.talk": np.array([[1.0]]),
         "a.o": np.array([[1.0]]), "a.o.b": np.zeros(1)}
    v = np.arange(6.0).reshape(6, 1, 1)
    out = P.attention(W, "a.", m, np.zeros((6, 2)), np.zeros((6, 1, 2)), v)
    assert np.allclose(out[:, 0], [0, 0.5, 1, 2, 3, 4])
    # a sink at the score of the keys takes one share more
    W["a.sink"] = np.array([0.0])
    out = P.attention(W, "a.", m, np.zeros((6, 2)), np.zeros((6, 1, 2)), v)
    assert np.allclose(out[:, 0], [0, 1 / 3, 3 / 4, 6 / 4, 9 / 4, 12 / 4])
    # rotation: a quarter turn of the pair (lane 0, lane 1) at the position whose angle is pi / 2; lane 2 passes
    x = np.array([[[1.0, 0.0, 7.0]]])
    assert np.allclose(P.rotate(x, np.array([math.pi / 2]), 2, 10.0), [[[0.0, 1.0, 7.0]]], atol=1e-12)
    # convolution: the last tap is the token itself, zeros before the start
    h = np.array([[1.0], [2.0], [4.0]])
    assert np.allclose(P.causal_conv(h, np.array([[10.0, 1.0]])), [[1.0], [12.0], [24.0]])
    # gated linear attention with alpha = 1 (bias far up) is the plain running sum of k v^T
    g = dict(heads=1, dim=1, vdim=1, tau=1.0)
    W = {"g.q": np.array([[1.0]]), "g.k": np.array([[1.0]]), "g.v": np.array([[1.0]]), "g.g": np.array([[0.0]]),
         "g.a1": np.array([[0.0]]), "g.a2": np.array([[0.0]]), "g.a2.b": np.array([50.0]), "g.norm": np.array([1.0]),
         "g.o": np.array([[1.0]])}
    # o_t = sum_{s<=t} x_s^2 * x_t is positive, so its unit-RMS form is 1, times silu(0) = 0
    assert np.allclose(P.gla(W, "g.", g, np.array([[1.0], [2.0]]), 0.0), 0.0)
    W["g.g"] = np.array([[1.0]])
    assert np.allclose(P.gla(W, "g.", g, np.array([[1.0], [2.0]]), 0.0)[:, 0], [P.silu(1.0), P.silu(2.0)])
    # routing: the two largest logits, weights from those two alone
    f = dict(kind="moe", router=dict(experts=3, top=2), expert=dict(ff=1))
    W = {"m.router": np.array([[1.0], [3.0], [2.0]]), "m.router.b": np.zeros(3)}
    for e in range(3):
        W[f"m.e{e}.gate"], W[f"m.e{e}.up"], W[f"m.e{e}.down"] = np.array([[1.0]]), np.array([[1.0]]), np.array([[10.0 ** e]])
    a = P.silu(1.0)
    assert np.allclose(P.moe_ff(W, "m.", f, np.array([[1.0]])), a * (10 * math.e + 100) / (1 + math.e))


# ---- GPU ----------------------------------------------------------------------------------------
def engine_for(tmp_path, cfg, w, dtype, **kw):
    from burn_lm_amd.engine.loading import load_engine
    kw.setdefault("max_tokens", 1024)
    return load_engine(write_folder(tmp_path, cfg, w), dtype=dtype, **kw)


def whole(eng, toks):
    s = eng.open()
    out = eng.step([(s, toks, list(range(len(toks))))]).double().cpu().numpy()
    eng.close(s)
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("layers", [[gla(mlp=None)], [gla(heads=1, dim=70, vdim=5, tau=1.0, mlp=None)],
                                    [attn(mlp=None)], [attn(heads=6, kv_heads=6, dim=8, vdim=8, window=1000, rot=8, mlp=None)],
                                    [attn(heads=8, kv_heads=1, dim=32, vdim=16, window=64, rot=2, mlp=None)],
                                    [attn(window=64, mlp=None), attn(window=65, kv_from=0, mlp=None)],
                                    [gla(mlp="dense")], [gla(mlp="moe")], [gla(mlp="moe_top1_no_shared")]],
                         ids=["gla", "gla_one_wide_head", "attention", "attention_ungrouped_sees_all", "attention_one_kv_head",
                              "attention_borrowed", "dense", "experts", "experts_top1"])
def test_every_mechanism_alone(tmp_path, layers, dtype):
    cfg = config(layers)
    w = make_weights(cfg, 3)
    eng = engine_for(tmp_path, cfg, w, dtype, graphs=False)
    toks = tokens_of(cfg, 4, 150)       # three pages, past every window but one
    want = P.forward(cfg, w, toks)
    rows = Rows(dtype)
    rows.add(whole(eng, toks), want, "whole")
    # one token at a time from the first one on: the first tokens of a sequence, then a page border
    s = eng.open()
    rows.add(np.stack([eng.step([(s, [t], [0])])[0].double().cpu().numpy() for t in toks[:70]]), want[:70], "one by one")
    eng.close(s)
    rows.check()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_batches_and_slots_used_again(tmp_path, dtype):
    cfg = MIXED
    w = make_weights(cfg, 5, sharp=3.0 if dtype == "float32" else 1.0)
    eng = engine_for(tmp_path, cfg, w, dtype, max_tokens=1536, max_seqs=6)
    reqs = [tokens_of(cfg, 10 + i, n) for i, n in enumerate((200, 7, 66, 129, 1))]
    want = [P.forward(cfg, w, r) for r in reqs]
    rows = Rows(dtype)
    for r, x in zip(reqs, want):
        rows.add(whole(eng, r), x, "whole")
    # a prompt in portions of several sizes, down to two tokens and one (fewer than the convolution's taps)
    for sizes in ((2, 5, 57, 64, 3, 69), (63, 2, 1, 1, 133), (128, 72), (1, 1, 1, 2, 195)):
        s, at = eng.open(), 0
        for n in sizes:
            rows.add(eng.step([(s, reqs[0][at:at + n], list(range(n)))]).double().cpu().numpy(), want[0][at:at + n], sizes)
            at += n
        eng.close(s)
        assert at == 200
    # unequal batches: prompts in one step, then one token each; shorter requests end earlier; the second round
    # finds slots, pages and state that the first one used
    for round_ in range(2):
        order = [0, 1, 2, 3, 4] if round_ == 0 else [3, 4, 0, 2, 1]
        slots = {i: eng.open() for i in order}
        cut = {i: max(1, len(reqs[i]) - 6) for i in order}
        got = eng.step([(slots[i], reqs[i][:cut[i]], list(range(cut[i]))) for i in order]).double().cpu().numpy()
        o = 0
        for i in order:
            rows.add(got[o:o + cut[i]], want[i][:cut[i]], (round_, i))
            o += cut[i]
            if cut[i] == len(reqs[i]):
                eng.close(slots[i])
        for k in range(6):
            live = [i for i in order if cut[i] + k < len(reqs[i])]
            got = eng.step([(slots[i], [reqs[i][cut[i] + k]], [0]) for i in live]).double().cpu().numpy()
            for row, i in enumerate(live):
                rows.add(got[row], want[i][cut[i] + k], (round_, i, k))
            for i in order:
                if cut[i] + k + 1 == len(reqs[i]):
                    eng.close(slots[i])
    rows.check()
    assert eng.cache.pages_in_use() == 0 and eng.cache.free_slots == 6


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_recorded_steps(tmp_path, dtype):
    cfg = MIXED
    w = make_weights(cfg, 6, sharp=2.0 if dtype == "float32" else 1.0)
    eng = engine_for(tmp_path, cfg, w, dtype)
    a, b = tokens_of(cfg, 20, 200), tokens_of(cfg, 21, 150)
    wa, wb = P.forward(cfg, w, a), P.forward(cfg, w, b)
    sa, sb = eng.open(), eng.open()
    rows = Rows(dtype)
    got = eng.step([(sa, a[:30], [29]), (sb, b[:3], [2])]).double().cpu().numpy()
    rows.add(got, np.stack([wa[29], wb[2]]), "prompts")
    for k in range(140):          # across two page borders and past every window; one shape, recorded and replayed
        got = eng.step([(sa, [a[30 + k]], [0]), (sb, [b[3 + k]], [0])]).double().cpu().numpy()
        rows.add(got, np.stack([wa[30 + k], wb[3 + k]]), k)
    rows.check()
    assert eng.graphs.replays >= 100


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_are_no_multiples_of_eight(tmp_path, dtype):
    cfg = ODD
    w = make_weights(cfg, 7, rank=3)
    eng = engine_for(tmp_path, cfg, w, dtype)
    reqs = [tokens_of(cfg, 30 + i, n) for i, n in enumerate((90, 31))]
    want = [P.forward(cfg, w, r) for r in reqs]
    slots = [eng.open(), eng.open()]
    rows = Rows(dtype)
    got = eng.step([(slots[0], reqs[0][:80], list(range(80))), (slots[1], reqs[1][:21], list(range(21)))]).double().cpu().numpy()
    rows.add(got[:80], want[0][:80], "prompt 0")
    rows.add(got[80:], want[1][:21], "prompt 1")
    for k in range(10):
        got = eng.step([(slots[0], [reqs[0][80 + k]], [0]), (slots[1], [reqs[1][21 + k]], [0])]).double().cpu().numpy()
        rows.add(got, np.stack([want[0][80 + k], want[1][21 + k]]), k)
    rows.check()


def drawn_config(seed):
    """A configuration drawn from the seed: two to five layers of either mixer in any order, borrowers of earlier
    attention layers with head counts, windows and scales of their own, any feed-forward or none, sizes that are and are
    not multiples of eight, one tap and several."""
    rng = np.random.default_rng(seed)
    pick = lambda *a: a[int(rng.integers(0, len(a)))]
    layers, lenders = [], []
    for i in range(int(rng.integers(2, 6))):
        kind = pick("dense", "moe", None)
        if kind == "dense":
            mlp = dict(kind="dense", ff=pick(24, 64, 100), limit=pick(0.5, 1.0, 3.0))
        elif kind == "moe":
            E = int(rng.integers(2, 9))
            mlp = dict(kind="moe", router=dict(experts=E, top=int(rng.integers(1, E + 1))), expert=dict(ff=pick(8, 16, 40)))
            if rng.random() < 0.6:
                mlp["shared"] = dict(ff=pick(8, 32, 48))
        else:
            mlp = None
        if rng.random() < 0.4:
            mixer = dict(heads=int(rng.integers(1, 5)), dim=pick(8, 16, 24, 48, 5), vdim=pick(8, 16, 32, 20, 3), tau=pick(1.0, 4.0, 16.0))
            layers.append(dict(type="gla", mixer=mixer, mlp=mlp))
            continue
        if lenders and rng.random() < 0.5:
            j = pick(*lenders)
            mixer = dict(layers[j]["mixer"], kv_from=j, mask=dict(size=pick(1, 3, 17, 64, 65, 100, 300)), scale=pick(0.1, 0.25, 0.5))
            mixer["heads"] = mixer["kv_heads"] * int(rng.integers(1, 5))
        else:
            G, dk = int(rng.integers(1, 5)), pick(8, 16, 24, 32, 48, 64, 12, 6)
            mixer = dict(heads=G * int(rng.integers(1, 5)), kv_heads=G, dim=dk, vdim=pick(8, 16, 24, 48, 64, 10, 72), scale=pick(0.1, 0.25, 0.5),
                         mask=dict(size=pick(1, 3, 17, 64, 65, 100, 300)),
                         rot=dict(base=pick(100.0, 10000.0, 5e5), dims=pick(*[d for d in (2, 4, 6, 8, 12, 16, 24, 32, 48, 64) if d <= dk])))
            lenders.append(i)
        layers.append(dict(type="attention", mixer=mixer, mlp=mlp))
    return config(layers, width=pick(40, 64, 96, 128, 72), vocab=pick(50, 101, 257), taps=int(rng.integers(1, 6)), side=pick(3, 8, 16),
                  scale=pick(0.5, 1.0, 2.0), eps=pick(1e-5, 1e-6))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16])
def test_drawn_configurations(tmp_path, seed, dtype):
    """Unequal prompts in one step, then 32 tokens one by one, for configurations nobody chose by hand."""
    cfg = drawn_config(seed)
    w = make_weights(cfg, 100 + seed, rank=(3, 8, 16)[seed % 3])
    eng = engine_for(tmp_path, cfg, w, dtype, max_tokens=2048)
    reqs = [tokens_of(cfg, 7 + seed + i, n) for i, n in enumerate((330, 9, 140))]
    want = [P.forward(cfg, w, r) for r in reqs]
    rows = Rows(dtype)
    slots = [eng.open() for _ in reqs]
    cut = [max(1, len(r) - 32) for r in reqs]
    got = eng.step([(s, r[:c], list(range(c))) for s, r, c in zip(slots, reqs, cut)]).double().cpu().numpy()
    o = 0
    for i, c in enumerate(cut):
        rows.add(got[o:o + c], want[i][:c], ("prompt", i))
        o += c
    for k in range(32):
        live = [i for i in range(len(reqs)) if cut[i] + k < len(reqs[i])]
        got = eng.step([(slots[i], [reqs[i][cut[i] + k]], [0]) for i in live]).double().cpu().numpy()
        rows.add(got, np.stack([want[i][cut[i] + k] for i in live]), k)
    rows.check()


class _Step:
    """The index arrays that the attention kernels read, for sequences laid out by hand."""

    def __init__(self, news, pasts, slots, dev):
        i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=dev)
        self.n_tokens, self.n_seqs = sum(news), len(news)
        self.positions = i32([p + t for n, p in zip(news, pasts) for t in range(n)])
        self.token_seq = i32([b for b, n in enumerate(news) for _ in range(n)])
        self.cu_seqlens = i32([sum(news[:b]) for b in range(len(news) + 1)])
        self.seq_slots = i32(slots)
        self.lens_after = i32([p + n for n, p in zip(news, pasts)])
        self.max_position = max(p + n for n, p in zip(news, pasts)) - 1
        self.max_new, self.max_len_after = max(news), self.max_position + 1
        self.token_source = None


def _attend(form, *args):
    """The generic kernel, or the matrix-core one with its pages whole or cut into pieces."""
    from burn_lm_amd.csrc import ops
    if form == "generic":
        return ops.sink_attn(*args)
    return ops.sink_attn_mfma(*args, n_splits=1 if form == "matrix" else 3, group_batch=0 if form == "matrix" else 1)


FORMS = [("generic", torch.float32), ("generic", torch.bfloat16), ("matrix", torch.bfloat16), ("matrix_pieces", torch.bfloat16)]
FORM_IDS = ["generic-float32", "generic-bfloat16", "matrix", "matrix_pieces"]


@pytest.mark.gpu
@pytest.mark.parametrize("form,dtype", FORMS, ids=FORM_IDS)
@pytest.mark.parametrize("decode", [False, True], ids=["prompt", "decoding"])
def test_one_key_stands_out_far_back_at_page_borders_and_at_the_windows_edges(form, dtype, decode):
    """Keys and queries are made so that exactly one key's score towers over the rest; the result must be that
    key's value when it is the oldest one the window still holds, and must not know it one token later.  The
    sequence's pages lie scattered and in no order."""
    from burn_lm_amd.csrc import ops
    dev = "cuda"
    H, G, dk, dv, ps, window = 4, 2, 8, 6, 64, 130
    g = torch.Generator().manual_seed(0)
    n_pages, L = 9, 300
    pages = [7, 2, 5, 0, 8]                                    # the sequence's pages; pages 1, 3, 4, 6 hold noise
    kc = torch.randn(n_pages, G, ps, dk, generator=g) * 0.1
    vc = torch.randn(n_pages, G, dv, ps, generator=g)
    table = torch.tensor([pages + [-1] * 3], dtype=torch.int32, device=dev)
    sinks = torch.full((H,), -30.0)
    mix = torch.eye(H)
    marked = [0, 63, 64, 127, 128, 169, 170, 171, 200, 299]     # first token, page borders, around queries' window edges
    value = lambda j: float(j % 97)                             # distinct for the marked keys, exact in bfloat16
    for rank, j in enumerate(marked):
        kc[pages[j // ps], :, j % ps, :] = 0.0
        kc[pages[j // ps], :, j % ps, 0] = float(len(marked) - rank)      # lane 0: the older the key, the larger
        vc[pages[j // ps], :, :, j % ps] = value(j)
    # every query asks by lane 0 alone: scores are 40 * (10 - rank) against noise of a few units, so the oldest marked
    # key that the window still holds wins by e^40: the key at p - window + 1 if it is marked, never the one at p - window
    queries = [(p, min(j for j in marked if p - window < j <= p)) for p in (0, 63, 64, 128, 192, 193, 256, 298, 299)]
    assert (299, 170) in queries and (298, 169) in queries and (256, 127) in queries and (193, 64) in queries \
        and (192, 63) in queries and (128, 0) in queries
    if decode:
        steps = [([1], [p]) for p, _ in queries]
    else:
        steps = [([300], [0])]
    for news, pasts in steps:
        step = _Step(news, pasts, [0], dev)
        T = step.n_tokens
        q = torch.zeros(T, H * dk)
        q.view(T, H, dk)[:, :, 0] = 40.0
        out = torch.empty(T, H * dv, dtype=dtype, device=dev)
        _attend(form, q.to(dev, dtype), out, sinks.to(dev), mix.to(dev), step, table, kc.to(dev, dtype).contiguous(),
                vc.to(dev, dtype).contiguous(), ps, H, G, dk, dv, 1.0, window)
        out = out.float().cpu().view(T, H, dv)
        for p, j in queries:
            row = p - pasts[0] if decode else p
            if 0 <= row < T and (not decode or pasts[0] == p):
                assert torch.allclose(out[row], torch.full((H, dv), value(j)), atol=1e-3), (p, j)


@pytest.mark.gpu
@pytest.mark.parametrize("form,dtype", FORMS, ids=FORM_IDS)
def test_sink_and_head_mixing_kernel_against_the_plain_function(form, dtype):
    """Large sinks (they take most of the weight), a mixing matrix far from the identity, values of another size than
    the keys, three sequences of unequal pasts in one step."""
    dev = "cuda"
    H, G, dk, dv, ps = (6, 3, 10, 7, 64) if form == "generic" else (6, 3, 16, 20, 64)
    rng = np.random.default_rng(1)
    bf = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32)).to(dtype).double().numpy()
    news, pasts = [5, 1, 70], [0, 80, 3]
    lens = [n + p for n, p in zip(news, pasts)]
    k = [bf(rng.standard_normal((L, G, dk))) for L in lens]
    v = [bf(rng.standard_normal((L, G, dv))) for L in lens]
    q = [bf(rng.standard_normal((n, H, dk)) * 2) for n in news]
    sinks, talk = rng.standard_normal(H) * 3 + 2, rng.standard_normal((H, H))
    tables = [[4, 1], [0, 6], [5, 2]]
    kc, vc = torch.zeros(8, G, ps, dk), torch.zeros(8, G, dv, ps)
    for b, L in enumerate(lens):
        for j in range(L):
            kc[tables[b][j // ps], :, j % ps] = torch.from_numpy(k[b][j])
            vc[tables[b][j // ps], :, :, j % ps] = torch.from_numpy(v[b][j])
    for window in (0, 4, 64):
        want = []
        for b, (n, p) in enumerate(zip(news, pasts)):
            for t in range(n):
                i = p + t
                lo = max(0, i - window + 1) if window else 0
                wts = np.zeros((H, i + 1))
                for h in range(H):
                    s = k[b][lo:i + 1, h // (H // G)] @ q[b][t, h] * 0.3
                    mx = max(s.max(), sinks[h])
                    e = np.exp(s - mx)
                    wts[h, lo:] = e / (e.sum() + math.exp(sinks[h] - mx))
                mixed = talk @ wts
                want.append(np.stack([mixed[h] @ v[b][:i + 1, h // (H // G)] for h in range(H)]).reshape(-1))
        step = _Step(news, pasts, [0, 1, 2], dev)
        qq = torch.from_numpy(np.concatenate(q).reshape(sum(news), H * dk)).to(dev, dtype)
        out = torch.empty(sum(news), H * dv, dtype=dtype, device=dev)
        _attend(form, qq, out, torch.tensor(sinks, dtype=torch.float32, device=dev),
                torch.tensor(talk, dtype=torch.float32, device=dev), step,
                torch.tensor(tables, dtype=torch.int32, device=dev), kc.to(dev, dtype).contiguous(),
                vc.to(dev, dtype).contiguous(), ps, H, G, dk, dv, 0.3, window)
        assert rel_err(out.double().cpu().numpy(), np.stack(want)) <= (1e-5 if dtype == torch.float32 else 2e-2), window


@pytest.mark.gpu
def test_block_kernels_against_the_plain_functions():
    from burn_lm_amd.csrc import ops
    dev = "cuda"
    rng = np.random.default_rng(2)
    f32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.float32, device=dev)
    # the input convolution over three sequences, one of which brings fewer tokens than taps and has a past
    D, taps = 20, 4
    news, slots = [6, 2, 1], [2, 0, 3]
    hist = rng.standard_normal((4, taps - 1, D))
    hist[2] = 0.0                                               # a fresh slot: the sequence starts here
    n = rng.standard_normal((sum(news), D))
    ws = [rng.standard_normal((D, taps)) for _ in range(2)]
    step = _Step(news, [0, 9, 5], slots, dev)
    outs = [torch.empty(sum(news), D, dtype=torch.float32, device=dev) for _ in ws]
    hist_dev = f32(hist)
    ops.input_conv(f32(n), hist_dev, [f32(w) for w in ws], outs, step)
    at = 0
    for b, cnt in enumerate(news):
        rows = np.concatenate([hist[slots[b]], n[at:at + cnt]])
        for r, w in enumerate(ws):
            want = n[at:at + cnt] + P.causal_conv(rows, w)[taps - 1:]
            assert np.abs(outs[r][at:at + cnt].double().cpu().numpy() - want).max() < 1e-5, (b, r)
        assert np.abs(hist_dev[slots[b]].double().cpu().numpy() - rows[-(taps - 1):]).max() < 1e-6, b
        at += cnt
    assert np.abs(hist_dev[1].cpu().numpy() - hist[1].astype(np.float32)).max() == 0          # a slot that is not in the step
    # clamped gating at and beyond the limit
    gu = np.array([[-3.0, 0.5, 1.5, 9.0, 0.2, -9.0, 9.0, 1.0]])
    out = ops.clamped_glu(f32(gu), torch.empty(1, 4, dtype=torch.float32, device=dev), 1.5, 1.702)
    g, u = np.minimum(gu[0, :4], 1.5), np.clip(gu[0, 4:], -1.5, 1.5)
    assert np.abs(out.double().cpu().numpy()[0] - g * P.sigmoid(1.702 * g) * (u + 1)).max() < 1e-6
    # routing: ties go to the lower index, weights over the chosen alone, the shared expert's gate at the end
    logits = np.array([[1.0, 3.0, 3.0, -1.0, 0.5, 0, 0, 0], [0.0, 0.0, 0.0, 0.0, -2.0, 0, 0, 0]])
    bias = np.array([0.0, 0.0, -0.5, 3.5])                      # with it: [1, 3, 2.5, 2.5] and [0, 0, -0.5, 3.5]
    wts = ops.moe_route(f32(logits), f32(bias), 4, 2, 4, torch.empty(2, 5, dtype=torch.float32, device=dev)).double().cpu().numpy()
    e, e7 = math.exp(-0.5), math.exp(-3.5)
    assert np.allclose(wts[0], [0, 1 / (1 + e), e / (1 + e), 0, P.sigmoid(0.5)], atol=1e-6)
    assert np.allclose(wts[1], [e7 / (1 + e7), 0, 0, 1 / (1 + e7), P.sigmoid(-2.0)], atol=1e-6)
    # the side input and the norm that hands on a float delta
    z, table = rng.standard_normal((3, 5)), rng.standard_normal((7, 12))
    ids = torch.tensor([6, 0, 3], dtype=torch.int32, device=dev)
    got = ops.side_gate(f32(z), f32(table), 4, ids, torch.empty(3, 5, dtype=torch.float32, device=dev))
    assert np.abs(got.double().cpu().numpy() - P.gelu_tanh(z) * table[[6, 0, 3], 4:9]).max() < 1e-6
    y, wn = rng.standard_normal((2, 3, 20)), rng.uniform(0.5, 1.5, 20)
    got = ops.rms_scale(f32(y), f32(wn), 1e-5, torch.empty(3, 20, dtype=torch.float32, device=dev))
    assert np.abs(got.double().cpu().numpy() - P.rms_unit(y.sum(0), 1e-5) * wn).max() < 1e-5
    # the residual add of two results (one as partial planes) and a bias, with its copy
    h, a, b, bias = rng.standard_normal((3, 20)), rng.standard_normal((2, 3, 20)), rng.standard_normal((3, 20)), rng.standard_normal(20)
    hd, copy = f32(h), torch.empty(3, 20, dtype=torch.bfloat16, device=dev)
    ops.residual_add(hd, f32(a), f32(b).bfloat16(), f32(bias), copy)
    want = h + a.sum(0) + f32(b).bfloat16().double().cpu().numpy() + bias
    assert np.abs(hd.double().cpu().numpy() - want).max() < 1e-5
    assert np.abs(copy.double().cpu().numpy() - want).max() < 2e-2


@pytest.mark.gpu
def test_greedy_generation_through_the_server(tmp_path):
    from burn_lm_amd.server import InferenceServer
    cfg = MIXED
    w = make_weights(cfg, 8)
    folder = write_folder(tmp_path, cfg, w)
    prompts = [tokens_of(cfg, 40 + i, n) for i, n in enumerate((5, 11, 2, 70))]

    def plain_greedy(p, n):
        toks = list(p)
        for _ in range(n):
            toks.append(int(np.argmax(P.forward(cfg, w, toks)[-1])))
        return toks[len(p):]

    want = [plain_greedy(p, 6) for p in prompts]
    server = InferenceServer(folder, dtype="float32", batch_size=3)       # two batches: slots are used again
    server.config.update(max_seq_len=256, sample_len=6, temperature=0.0)
    results, _ = server.generate(prompts, stop_ids=[])
    assert [r.tokens for r in results] == want
    server.unload()

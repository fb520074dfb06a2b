"""The Fuvirax design in the engine against the plain implementation of tests/plain_fuvirax.py.

The configurations and weights are made here.  The CPU tests cover the configuration reader, the plan and the
plain implementation's own consistency; the GPU tests run the engine's step function, cache, scheduler and
kernels: every mixer alone, whole prompts against token-by-token decoding, prompts in portions, unequal
batches, slots and pages used again, rows far back and at page borders, long decoding through recorded graphs,
odd sizes, and greedy generation through the server."""
import json
import math

import numpy as np
import pytest
import torch

import plain_fuvirax as P
from helpers import rel_err

# largest difference of a logit relative to the largest logit.  bfloat16: the models here are narrow and up to seven
# layer runs deep, where roundings alone reach 5e-2; what the float32 runs pin to 2e-5 is the same code path
TOL = {"float32": 2e-5, "bfloat16": 8e-2}


# ---- configurations and weights of the tests --------------------------------------------------
def latent(heads=3, dim=8, rot_dim=8, vdim=12, kv_rank=24, base=10000.0, ff=80, turning=None):
    return dict(type="latent_attention",
                mixer=dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank,
                           rot=dict(base=base, dims=turning or rot_dim), scale=1.0 / math.sqrt(dim + rot_dim)),
                mlp=None if ff is None else dict(kind="dense", ff=ff))


def hgrn(heads=2, dim=12, vdim=20, ff=80):
    return dict(type="hgrn2", mixer=dict(heads=heads, dim=dim, vdim=vdim),
                mlp=None if ff is None else dict(kind="dense", ff=ff))


def delta(heads=4, kv_heads=2, dim=8, vdim=12, conv=4, ff=80):
    return dict(type="channel_delta", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv),
                mlp=None if ff is None else dict(kind="dense", ff=ff))


def config(layers, width=48, vocab=101, streams=3, loop=None, logit_scale=0.7, eps=1e-5):
    c = dict(architecture="Fuvirax", layers=layers, logit_scale=logit_scale, norm=dict(eps=eps), streams=streams,
             vocab=vocab, width=width)
    if loop is not None:
        c["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return c


# the first attention layer has a latent of a size only the generic kernel takes, the second one of a size the
# matrix-core kernel is built for (in bfloat16 runs)
MIXED = config([latent(), hgrn(), delta(), latent(heads=2, dim=16, rot_dim=16, vdim=8, kv_rank=32, ff=None), hgrn(ff=None)],
               loop=(1, 3, 2))
# sizes that are no multiples of eight, one stream, one query/key head, two taps, no loop
ODD = config([latent(heads=3, dim=12, rot_dim=6, vdim=10, kv_rank=20, ff=50), hgrn(heads=3, dim=10, vdim=12, ff=50),
              delta(heads=2, kv_heads=1, dim=6, vdim=10, conv=2, ff=50)], width=36, vocab=53, streams=1, logit_scale=1.3)


def make_weights(cfg, seed, ranks=(5, 7), sharp=1.0):
    """float64 arrays that are exact in bfloat16.  sharp: factor on the query projections of the attention
    layers, so that the softmax singles out few rows."""
    g = np.random.default_rng(seed)
    D, S = cfg["width"], cfg["streams"]
    bf = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32)).bfloat16().double().numpy()
    mat = lambda o, i, s=1.0: bf(g.standard_normal((o, i)) * s / math.sqrt(i))
    w = {"embed": bf(g.standard_normal((cfg["vocab"], D))), "final.norm": bf(1 + 0.1 * g.standard_normal(D)),
         "final.norm.b": bf(0.05 * g.standard_normal(D))}
    for i, layer in enumerate(cfg["layers"]):
        l, m = f"l{i}.", layer["mixer"]
        for q in (1, 2) if layer["mlp"] is not None else (1,):
            w[f"{l}norm{q}"] = bf(1 + 0.1 * g.standard_normal(D))
            w[f"{l}norm{q}.b"] = bf(0.05 * g.standard_normal(D))
            w[f"{l}ls{q}"] = bf(g.uniform(0.3, 1.0, D))
            w[f"{l}hc{q}.in"] = bf(g.uniform(0.1, 0.8, S))
            w[f"{l}hc{q}.out"] = bf(g.uniform(0.2, 1.0, S))
            w[f"{l}hc{q}.mix"] = bf(np.eye(S) * 0.7 + g.uniform(-0.2, 0.3, (S, S)))
        w[l + "shift"] = bf(g.uniform(0.0, 1.0, D))
        p = l + "mix."
        if layer["type"] == "latent_attention":
            H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            w[p + "q"] = mat(H * (dn + dr), D, sharp)
            w[p + "dkv"] = mat(R + dr, D)
            w[p + "dkv.norm"] = bf(1 + 0.1 * g.standard_normal(R))
            w[p + "uk"], w[p + "uv"], w[p + "o"] = mat(H * dn, R), mat(H * dv, R), mat(D, H * dv)
        elif layer["type"] == "hgrn2":
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            w[p + "q"], w[p + "f"], w[p + "v"], w[p + "o"] = mat(H * dk, D), mat(H * dk, D), mat(H * dv, D), mat(D, H * dv)
            w[p + "f.b"] = bf(0.5 * g.standard_normal(H * dk))
            w[p + "lower"] = bf(g.uniform(0.0, 0.9, H * dk))
            w[p + "norm"] = bf(1 + 0.1 * g.standard_normal(dv))
        else:
            H, G, dk, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            ra, rg = ranks
            w[p + "q"], w[p + "k"], w[p + "v"] = mat(G * dk, D), mat(G * dk, D), mat(H * dv, D)
            for r, c in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
                w[p + r + ".conv"] = bf(g.standard_normal((c, taps)) / math.sqrt(taps))
            w[p + "b"] = mat(H, D)
            w[p + "A_log"] = bf(g.uniform(-3.0, 0.5, H))
            w[p + "norm"] = bf(1 + 0.1 * g.standard_normal(dv))
            w[p + "a1"], w[p + "a2"] = mat(ra, D), mat(H * dk, ra)
            w[p + "dt_bias"] = bf(g.uniform(-4.0, 0.0, H * dk))
            w[p + "g1"], w[p + "g2"], w[p + "o"] = mat(rg, D), mat(H * dv, rg), mat(D, H * dv)
        if layer["mlp"] is not None:
            F = layer["mlp"]["ff"]
            w[l + "mlp.up"], w[l + "mlp.down"] = mat(F, D), mat(D, F)
            w[l + "mlp.act"] = bf(0.5 * g.standard_normal(2))
    return w


def write_folder(path, cfg, w):
    from burn_lm_amd.weights import safetensors_io as st
    with open(path / "config.json", "w") as f:
        json.dump(cfg, f)
    st.write_file(str(path / "model.safetensors"), ((k, torch.from_numpy(v).bfloat16()) for k, v in w.items()))
    return str(path)


def tokens_of(cfg, seed, n):
    return [int(x) for x in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


# ---- CPU: configuration, plan, plain implementation ---------------------------------------------
def test_config_is_read_and_refused_by_key():
    from burn_lm_amd import registry
    from burn_lm_amd.errors import ConfigError
    import burn_lm_amd.models  # noqa: F401
    arch = registry.architecture_of(MIXED)
    assert arch.name == "Fuvirax"
    cfg = arch.read_config(MIXED)
    assert cfg.order() == [0, 1, 2, 1, 2, 3, 4] and cfg.streams == 3 and cfg.layers[3].ff is None
    assert arch.read_config(ODD).order() == [0, 1, 2]
    for path, value, word in ((("layers", 0, "mixer", "kv_rank"), None, "kv_rank"), (("width",), "48", "width"),
                              (("layers", 1, "type"), "mamba", "type"), (("norm",), {}, "eps"),
                              (("layers", 2, "mixer", "kv_heads"), 3, "kv_heads"), (("loop",), dict(start=2, stop=9, times=2), "loop"),
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
        specs = model.tensor_specs()
        assert {k: tuple(s.shape) for k, s in specs.items()} == {k: tuple(v.shape) for k, v in w.items()}
        assert len(model.plan.order) == len(P.layer_order(cfg_dict))
        # a fresh random checkpoint has the same names (its low-rank widths come from the configuration or a default)
        assert set(arch.checkpoint_tensors(cfg)) == set(w)


def test_random_folder_loads_into_the_plain_implementation(tmp_path):
    import burn_lm_amd
    from burn_lm_amd.weights import safetensors_io as st
    cfg = json.loads(json.dumps(ODD))
    cfg["layers"][2]["mixer"].update(decay_rank=4, gate_rank=6)
    folder = burn_lm_amd.write_random_model(str(tmp_path), cfg, seed=5)
    files = st.open_folder(folder)
    w = {n: f.tensor(n).double().numpy() for n, f in files.items()}
    assert w["l2.mix.a1"].shape == (4, 36) and w["l2.mix.g2"].shape == (20, 6)
    assert 0 <= w["l1.mix.lower"].min() and w["l1.mix.lower"].max() <= 0.9
    logits = P.forward(tokens_of(cfg, 0, 9), w, cfg)
    assert logits.shape == (9, 53) and np.isfinite(logits).all() and logits.std() > 0.05


def test_plain_recurrences_carry_their_state():
    cfg = MIXED
    w = make_weights(cfg, 1)
    g = np.random.default_rng(0)
    x = g.standard_normal((11, cfg["width"]))
    whole, _ = P.hgrn2(x, w, "l1.mix.", cfg["layers"][1]["mixer"], 1e-5)
    a, s = P.hgrn2(x[:4], w, "l1.mix.", cfg["layers"][1]["mixer"], 1e-5)
    b, _ = P.hgrn2(x[4:], w, "l1.mix.", cfg["layers"][1]["mixer"], 1e-5, s)
    assert np.abs(np.concatenate([a, b]) - whole).max() < 1e-12
    whole, _ = P.channel_delta(x, w, "l2.mix.", cfg["layers"][2]["mixer"], 1e-5)
    parts, s = [], None
    for lo, hi in ((0, 1), (1, 3), (3, 4), (4, 11)):
        y, s = P.channel_delta(x[lo:hi], w, "l2.mix.", cfg["layers"][2]["mixer"], 1e-5, s)
        parts.append(y)
    assert np.abs(np.concatenate(parts) - whole).max() < 1e-12
    mu = g.uniform(0, 1, cfg["width"])
    whole, _ = P.token_shift(x, mu)
    a, last = P.token_shift(x[:5], mu)
    b, _ = P.token_shift(x[5:], mu, last)
    assert np.abs(np.concatenate([a, b]) - whole).max() == 0


def test_plain_latent_attention_is_the_expanded_form():
    """The function that the engine computes from cached latents, written the long way: keys and values of every
    head expanded, one softmax per head over the causal rows."""
    cfg = MIXED
    w = make_weights(cfg, 2)
    m = cfg["layers"][0]["mixer"]
    x = np.random.default_rng(1).standard_normal((9, cfg["width"]))
    y = P.latent_attention(x, w, "l0.mix.", m, 1e-5)
    # the last token alone, with everything before it as context, from absorbed queries
    H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = np.arange(9.0)
    down = x @ w["l0.mix.dkv"].T
    c = P.rms_norm(down[:, :R], w["l0.mix.dkv.norm"], 1e-5)
    kr = P.rotate_half(down[:, R:], pos, m["rot"]["base"], dr)
    q = (x[-1:] @ w["l0.mix.q"].T).reshape(1, H, dn + dr)
    qr = P.rotate_half(q[:, :, dn:], pos[-1:], m["rot"]["base"], dr)[0]
    out = []
    for h in range(H):
        q_lat = w["l0.mix.uk"][h * dn:(h + 1) * dn].T @ q[0, h, :dn]
        s = (c @ q_lat + kr @ qr[h]) * m["scale"]
        p = np.exp(s - s.max())
        out.append(w["l0.mix.uv"][h * dv:(h + 1) * dv] @ ((p / p.sum()) @ c))
    assert np.abs(np.concatenate(out) @ w["l0.mix.o"].T - y[-1]).max() < 1e-10


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
@pytest.mark.parametrize("layer", [latent(ff=None), hgrn(ff=None), delta(ff=None), delta(heads=2, kv_heads=2, conv=1, ff=None),
                                   latent(heads=5, dim=4, rot_dim=12, vdim=4, kv_rank=12, ff=40),
                                   latent(heads=5, dim=8, rot_dim=16, vdim=8, kv_rank=64, ff=None),
                                   latent(heads=20, dim=8, rot_dim=32, vdim=4, kv_rank=64, ff=None),
                                   latent(heads=4, dim=8, rot_dim=16, vdim=8, kv_rank=32, ff=None, turning=8, base=300.0)],
                         ids=["latent", "hgrn2", "delta", "delta_one_tap", "latent_with_ff", "latent_matrix_core_sizes",
                              "latent_more_heads_than_a_tile", "latent_some_lanes_do_not_turn"])
def test_every_mixer_alone(tmp_path, layer, dtype):
    cfg = config([layer], streams=2)
    w = make_weights(cfg, 3)
    eng = engine_for(tmp_path, cfg, w, dtype, graphs=False)
    toks = tokens_of(cfg, 4, 150)       # three pages
    want = P.forward(toks, w, cfg)
    assert rel_err(whole(eng, toks), want) <= TOL[dtype]
    # one token at a time from the first one on: the first tokens of a sequence, then page borders
    s = eng.open()
    got = np.stack([eng.step([(s, [t], [0])])[0].double().cpu().numpy() for t in toks[:70]])
    eng.close(s)
    assert rel_err(got, want[:70]) <= TOL[dtype]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_batches_and_slots_used_again(tmp_path, dtype):
    cfg, tol = MIXED, TOL[dtype]
    # float32: sharp attention, where a wrong or missing row shows at once; bfloat16: the roundings of seven layer
    # runs in a model this narrow already move sharp attention by more than the tolerance
    w = make_weights(cfg, 5, sharp=3.0 if dtype == "float32" else 1.0)
    eng = engine_for(tmp_path, cfg, w, dtype, max_tokens=1536, max_seqs=6)
    reqs = [tokens_of(cfg, 10 + i, n) for i, n in enumerate((200, 7, 66, 129, 1))]
    want = [P.forward(r, w, cfg) for r in reqs]
    for r, x in zip(reqs, want):
        assert rel_err(whole(eng, r), x) <= tol
    # a prompt in portions of several sizes, down to two tokens and one
    for sizes in ((2, 5, 57, 64, 3, 69), (63, 2, 1, 134), (128, 72)):
        s, at, rows = eng.open(), 0, []
        for n in sizes:
            rows.append(eng.step([(s, reqs[0][at:at + n], list(range(n)))]).double().cpu().numpy())
            at += n
        eng.close(s)
        assert at == 200 and rel_err(np.concatenate(rows), want[0]) <= tol, sizes
    # unequal batches: prompts in one step, then one token each; shorter requests end earlier; the second round
    # finds slots, pages and state that the first one used
    for round_ in range(2):
        order = [0, 1, 2, 3, 4] if round_ == 0 else [3, 4, 0, 2, 1]
        slots = {i: eng.open() for i in order}
        cut = {i: max(1, len(reqs[i]) - 6) for i in order}
        got = eng.step([(slots[i], reqs[i][:cut[i]], list(range(cut[i]))) for i in order]).double().cpu().numpy()
        o = 0
        for i in order:
            assert rel_err(got[o:o + cut[i]], want[i][:cut[i]]) <= tol, (round_, i)
            o += cut[i]
            if cut[i] == len(reqs[i]):      # a request that was all prompt ends with the prompt step
                eng.close(slots[i])
        for k in range(6):
            live = [i for i in order if cut[i] + k < len(reqs[i])]
            got = eng.step([(slots[i], [reqs[i][cut[i] + k]], [0]) for i in live]).double().cpu().numpy()
            for row, i in enumerate(live):
                assert rel_err(got[row], want[i][cut[i] + k]) <= tol, (round_, i, k)
            for i in order:
                if cut[i] + k + 1 == len(reqs[i]):
                    eng.close(slots[i])
    assert eng.cache.pages_in_use() == 0 and eng.cache.free_slots == 6


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_recorded_steps(tmp_path, dtype):
    cfg = MIXED
    w = make_weights(cfg, 6, sharp=2.0 if dtype == "float32" else 1.0)
    eng = engine_for(tmp_path, cfg, w, dtype)
    a, b = tokens_of(cfg, 20, 200), tokens_of(cfg, 21, 150)
    wa, wb = P.forward(a, w, cfg), P.forward(b, w, cfg)
    sa, sb = eng.open(), eng.open()
    got = eng.step([(sa, a[:30], [29]), (sb, b[:3], [2])]).double().cpu().numpy()
    assert rel_err(got[0], wa[29]) <= TOL[dtype] and rel_err(got[1], wb[2]) <= TOL[dtype]
    for k in range(140):          # across two page borders; the same shape every time, so it is recorded and replayed
        got = eng.step([(sa, [a[30 + k]], [0]), (sb, [b[3 + k]], [0])]).double().cpu().numpy()
        assert rel_err(got[0], wa[30 + k]) <= TOL[dtype], k
        assert rel_err(got[1], wb[3 + k]) <= TOL[dtype], k
    assert eng.graphs.replays >= 100


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_are_no_multiples_of_eight(tmp_path, dtype):
    cfg = ODD
    w = make_weights(cfg, 7, ranks=(3, 9))
    eng = engine_for(tmp_path, cfg, w, dtype)
    reqs = [tokens_of(cfg, 30 + i, n) for i, n in enumerate((90, 31))]
    want = [P.forward(r, w, cfg) for r in reqs]
    slots = [eng.open(), eng.open()]
    got = eng.step([(slots[0], reqs[0][:80], list(range(80))), (slots[1], reqs[1][:21], list(range(21)))]).double().cpu().numpy()
    assert rel_err(got[:80], want[0][:80]) <= TOL[dtype] and rel_err(got[80:], want[1][:21]) <= TOL[dtype]
    for k in range(10):
        got = eng.step([(slots[0], [reqs[0][80 + k]], [0]), (slots[1], [reqs[1][21 + k]], [0])]).double().cpu().numpy()
        assert rel_err(got[0], want[0][80 + k]) <= TOL[dtype] and rel_err(got[1], want[1][21 + k]) <= TOL[dtype]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_splits", [1, 5])
def test_one_row_far_back_stands_out(dtype, n_splits):
    """Rows of the cache are small and random but one, which lines up with the query: the result must be that
    row's latent, wherever the row lies (first rows, both sides of page borders, the query's own place) and
    whichever pages hold the sequence."""
    from burn_lm_amd.csrc import ops
    from burn_lm_amd.engine.batch import Step
    dev, R, Dr, H, page = torch.device("cuda:0"), 24, 8, 3, 64
    ops.latent_attn_init(dev)
    g = torch.Generator().manual_seed(0)
    pos = 700
    pages = torch.randperm(16, generator=g)[:11].int()          # scattered pages of a pool of 16
    cache = (torch.randn(16, 1, page, R + Dr, generator=g) * 0.05).to(dtype)
    q = torch.randn(1, H, R + Dr, generator=g)
    q = q / q.norm(dim=-1, keepdim=True)
    for target in (0, 1, 63, 64, 65, 127, 128, 448, 639, 640, 699, 700):
        c = cache.clone()
        row = (q[0, 1] * 6.0).to(dtype)                         # head 1's query finds it; the others see noise
        c[pages[target // page], 0, target % page] = row
        step = Step(n_tokens=1, n_seqs=1, n_wanted=1, token_ids=None, positions=torch.tensor([pos], dtype=torch.int32, device=dev),
                    token_seq=torch.zeros(1, dtype=torch.int32, device=dev), seq_slots=None, cu_seqlens=None, lens_after=None,
                    want_rows=None, max_len_after=pos + 1, max_position=pos)
        olat = torch.empty(1, H, R, dtype=torch.float32, device=dev)
        table = pages.view(1, -1).to(dev)
        ops.latent_attn(q.to(dev).contiguous(), olat, c.to(dev), step, table, page, H, R, Dr, 8.0, n_splits)
        torch.cuda.synchronize()
        # plain: softmax over rows 0 .. pos
        rows = torch.cat([c[p, 0] for p in pages]).double()[:pos + 1]
        s = (rows @ q[0].double().T) * 8.0
        p = torch.softmax(s, dim=0)
        want = (p.T @ rows[:, :R])
        assert p[target, 1] > 0.99
        assert (olat[0].double().cpu() - want).abs().max() <= 1e-5, target
        assert (olat[0, 1].double().cpu() - row[:R].double()).abs().max() < 0.05


@pytest.mark.gpu
@pytest.mark.parametrize("n_splits", [1, 3, 11])
def test_one_row_far_back_stands_out_on_the_matrix_cores(n_splits):
    """The same for the matrix-core kernel: two sequences of one token each (decoding), 20 heads (two tiles of
    columns, the second partly empty), the latent also in its transposed pages; rows past the data hold NaN."""
    from burn_lm_amd.csrc import ops
    from burn_lm_amd.engine.batch import Step
    dev, R, Dr, H, page = torch.device("cuda:0"), 64, 16, 20, 64
    ops.latent_attn_init(dev)
    g = torch.Generator().manual_seed(1)
    lens = [701, 130]
    pools = torch.randperm(24, generator=g).int()
    tables = torch.full((2, 11), -1, dtype=torch.int32)
    tables[0, :11], tables[1, :3] = pools[:11], pools[11:14]
    q = torch.randn(2, H, R + Dr, generator=g)
    q = (q / q.norm(dim=-1, keepdim=True)).bfloat16()
    i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=dev)
    step = Step(n_tokens=2, n_seqs=2, n_wanted=0, token_ids=None, positions=i32([700, 129]), token_seq=i32([0, 1]),
                seq_slots=i32([0, 1]), cu_seqlens=i32([0, 1, 2]), lens_after=i32(lens), want_rows=None, max_new=1,
                max_len_after=701, max_position=700)
    for target in (0, 63, 64, 127, 128, 129):
        k = (torch.randn(24, 1, page, R + Dr, generator=g) * 0.05).bfloat16()
        for b in range(2):       # places past each sequence's data: NaN
            last_page, used = tables[b][(lens[b] - 1) // page], (lens[b] - 1) % page + 1
            k[last_page, 0, used:] = float("nan")
        rows = []
        for b in range(2):
            row = (q[b, 7].float() * 6.0).bfloat16()
            k[tables[b][target // page], 0, target % page] = row
            rows.append(row)
        v = k[:, :, :, :R].transpose(2, 3).contiguous()
        olat = torch.empty(2, H, R, dtype=torch.float32, device=dev)
        ops.latent_attn_mfma(q.to(dev), olat, k.to(dev), v.to(dev), step, tables.to(dev), page, H, R, Dr, 8.0, n_splits)
        torch.cuda.synchronize()
        for b in range(2):
            ctx = torch.cat([k[p, 0] for p in tables[b][: (lens[b] + page - 1) // page]]).double()[:lens[b]]
            p = torch.softmax((ctx @ q[b].double().T) * 8.0, dim=0)
            want = p.T @ ctx[:, :R]
            assert p[target, 7] > 0.99
            # probabilities go through bfloat16 on their way into the second product
            assert (olat[b].double().cpu() - want).abs().max() <= 4e-3, (target, b)
            assert (olat[b, 7].double().cpu() - rows[b][:R].double()).abs().max() < 0.05


@pytest.mark.gpu
def test_streams_norm_and_shift_kernels_against_the_plain_functions():
    from burn_lm_amd.csrc import ops
    from burn_lm_amd.engine.batch import Step
    dev = torch.device("cuda:0")
    g = np.random.default_rng(0)
    S, D, T = 3, 40, 9                     # two sequences: 5 tokens from position 0, 4 tokens that go on from a carry
    x = g.standard_normal((T, S, D))
    y = g.standard_normal((2, T, D))       # two planes of partial results
    scale, mix, write, read = g.uniform(0.3, 1, D), g.standard_normal((S, S)), g.standard_normal(S), g.standard_normal(S)
    gamma, beta, mu = 1 + 0.1 * g.standard_normal(D), 0.1 * g.standard_normal(D), g.uniform(0, 1, D)
    carry = g.standard_normal((4, D))
    f = lambda a: torch.tensor(a, dtype=torch.float32, device=dev)
    i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=dev)
    step = Step(n_tokens=T, n_seqs=2, n_wanted=0, token_ids=None, positions=i32([0, 1, 2, 3, 4, 7, 8, 9, 10]),
                token_seq=i32([0] * 5 + [1] * 4), seq_slots=i32([2, 1]), cu_seqlens=i32([0, 5, 9]), lens_after=None, want_rows=None)
    xs, carry_d = f(x), f(carry)
    n = torch.empty(T, D, dtype=torch.float32, device=dev)
    stash = torch.empty(2, D, dtype=torch.float32, device=dev)
    ops.streams_norm(xs, n, f(gamma), f(beta), 1e-5, read=f(read), pending=(f(y), f(scale), f(mix), f(write)),
                     stash=(carry_d, stash, step))
    out = torch.empty(T, D, dtype=torch.float32, device=dev)
    ops.token_shift(n, f(mu), stash, carry_d, out, step)
    streams = P.hyper_write(x.transpose(1, 0, 2), mix, write, y.sum(0) * scale)
    assert np.abs(xs.cpu().numpy() - streams.transpose(1, 0, 2)).max() < 1e-5
    normed = P.layer_norm(P.hyper_read(streams, read), gamma, beta, 1e-5)
    a, last_a = P.token_shift(normed[:5], mu)
    b, last_b = P.token_shift(normed[5:], mu, carry[1])
    assert np.abs(out.cpu().numpy() - np.concatenate([a, b])).max() < 1e-5
    assert np.abs(carry_d[2].cpu().numpy() - last_a).max() < 1e-5 and np.abs(carry_d[1].cpu().numpy() - last_b).max() < 1e-5
    assert np.abs(carry_d[[0, 3]].cpu().numpy() - carry[[0, 3]].astype(np.float32)).max() == 0
    # the listed rows only, nothing written back, the plain sum of the streams, a factor on the result
    rows = i32([7, 2])
    before = xs.clone()
    got = torch.empty(2, D, dtype=torch.float32, device=dev)
    ops.streams_norm(xs, got, f(gamma), f(beta), 1e-5, pending=(f(y[0]), f(scale), f(mix), f(write)), rows=rows,
                     write_x=False, out_scale=1.5)
    s2 = P.hyper_write(streams, mix, write, y[0] * scale)
    want = P.layer_norm(s2.sum(0), gamma, beta, 1e-5)[[7, 2]] * 1.5
    assert np.abs(got.cpu().numpy() - want).max() < 2e-5 and torch.equal(xs, before)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_xielu_kernel(dtype):
    from burn_lm_amd.csrc import ops
    z = torch.linspace(-6, 6, 4001).to(dtype)
    p, q = 0.3, -0.7
    out = torch.empty_like(z, device="cuda:0")
    ops.xielu(z.cuda(), out, P.softplus(np.float64(p)), 0.5 + P.softplus(np.float64(q)))
    want = P.xielu(z.double().numpy(), p, q)
    err = np.abs(out.double().cpu().numpy() - want)
    assert err.max() <= (1e-5 if dtype == torch.float32 else 0.04 * (1 + np.abs(want)).max() / 8)


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
            toks.append(int(np.argmax(P.forward(toks, w, cfg)[-1])))
        return toks[len(p):]

    want = [plain_greedy(p, 6) for p in prompts]
    server = InferenceServer(folder, dtype="float32", batch_size=3)       # two batches: slots are used again
    server.config.update(max_seq_len=256, sample_len=6, temperature=0.0)
    results, _ = server.generate(prompts, stop_ids=[])
    assert [r.tokens for r in results] == want
    server.unload()

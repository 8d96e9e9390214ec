"""The Bitonex design in the engine against the plain implementation of tests/plain_bitonex.py.

The configurations and weights are made here.  The CPU tests cover the configuration reader, the plan, the random
checkpoint and the plain implementation's own consistency on cases worked by hand; the GPU tests run the engine's step
function, cache, scheduler and kernels: each mixer and each added kernel alone, whole prompts against token-by-token
decoding, prompts in portions, unequal batches, slots, pages and states used again, one key that stands out far back
and at page borders (in prompts and in decoding, for the softmax attention and for the latent attention, also through
a layer that reads another's rows), a state that must survive hundreds of tokens, long decoding through recorded
graphs, odd sizes and values of one, configurations drawn from seeds, and greedy generation through the server."""
import json
import math

import numpy as np
import pytest
import torch

import plain_bitonex as P
from helpers import rel_err

TOL = {"float32": 2e-5, "bfloat16": 6e-2}


class Rows:
    """Collects rows of logits beside what they should be: every row within the tolerance, relative to the largest
    logit of what it should be."""

    def __init__(self, dtype):
        self.dtype, self.errs = dtype, []

    def add(self, got, want, note=None):
        got, want = np.atleast_2d(np.asarray(got, dtype=np.float64)), np.atleast_2d(want)
        assert got.shape == want.shape and np.isfinite(got).all(), note
        scale = max(1e-30, np.abs(want).max())
        self.errs += [(float(np.abs(g - x).max() / scale), note) for g, x in zip(got, want)]

    def check(self):
        bad = [e for e in self.errs if e[0] > TOL[self.dtype]]
        assert not bad, (len(bad), len(self.errs), sorted(bad, key=lambda e: -e[0])[:5])


# ---- configurations and weights of the tests --------------------------------------------------
def attention(heads=4, kv_heads=2, dim=16, vdim=16, rot=8, base=10000.0, scale=None, mlp="default"):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale or 1.0 / math.sqrt(dim))
    if rot:
        m["rot"] = dict(base=base, dims=rot)
    return dict(type="attention", mixer=m, mlp=dense() if mlp == "default" else mlp)


def lightning(heads=3, dim=12, vdim=20, decay=(0.5, 0.9, 1.0), mlp="default"):
    return dict(type="lightning", mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay)),
                mlp=dense() if mlp == "default" else mlp)


def latent(heads=3, dim=8, rot_dim=8, vdim=12, kv_rank=24, q_rank=20, rot=None, base=10000.0, scale=None, kv_from=None,
           mlp="default"):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank,
             scale=scale or 1.0 / math.sqrt(dim + rot_dim), rot=dict(base=base, dims=rot_dim if rot is None else rot))
    if kv_from is not None:
        m["kv_from"] = kv_from
    return dict(type="latent_attention", mixer=m, mlp=dense() if mlp == "default" else mlp)


def dense(ff=40):
    return dict(kind="dense", ff=ff)


def config(layers, width=48, vocab=101, mult=0.6, eps=1e-5, cap=20.0):
    cfg = dict(architecture="Bitonex", layers=layers, norm=dict(eps=eps), residual_mult=mult, vocab=vocab, width=width)
    if cap is not None:
        cfg["logit_softcap"] = cap
    return cfg


# every mixer, a layer without a feed-forward, two layers that read the rows of an earlier one (not the layer before),
# layers that differ from each other in every size
MIXED = config([latent(), attention(), lightning(mlp=None), latent(heads=2, dim=16, vdim=8, q_rank=12, kv_from=0),
                attention(heads=6, kv_heads=1, dim=8, vdim=24, rot=2, base=300.0, mlp=dense(24)),
                latent(heads=5, dim=4, vdim=20, q_rank=32, kv_from=0, mlp=None),
                lightning(heads=2, dim=16, vdim=8, decay=(0.97, 0.3))])
# sizes that are no multiples of eight; lanes that do not turn and no rotation at all; one head, one key-value head, as
# many key-value heads as heads; a residual multiplier of one; no soft cap; a single decay for all heads
ODD = config([attention(heads=3, kv_heads=3, dim=10, vdim=6, rot=4, mlp=dense(13)),
              latent(heads=1, dim=5, rot_dim=6, vdim=7, kv_rank=11, q_rank=9, rot=2, mlp=None),
              lightning(heads=1, dim=5, vdim=65, decay=(1.0,), mlp=dense(5)),
              attention(heads=1, kv_heads=1, dim=12, vdim=12, rot=12, base=50.0, mlp=None),
              latent(heads=2, dim=3, rot_dim=6, vdim=5, kv_rank=11, q_rank=4, rot=2, kv_from=1),
              attention(heads=5, kv_heads=1, dim=6, vdim=9, rot=0)],
             width=36, vocab=53, mult=1.0, eps=1e-6, cap=None)
ODD["layers"][2]["mixer"]["decay"] = 0.75        # one number for every head


def make_weights(cfg, seed, sharp=1.0):
    """float64 arrays that are exact in bfloat16.  sharp: factor on the query projections of the softmax mixers, so
    that they single out few keys."""
    g = np.random.default_rng(seed)
    D = cfg["width"]
    bf = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32)).bfloat16().double().numpy()
    mat = lambda o, i, s=1.0: bf(g.standard_normal((o, i)) * s / math.sqrt(i))
    near_one = lambda n: bf(1 + 0.1 * g.standard_normal(n))
    number = lambda: bf(np.asarray(1 + 0.2 * g.standard_normal()))
    w = {"embed": bf(g.standard_normal((cfg["vocab"], D))), "final.norm": number(), "head": mat(cfg["vocab"], D)}
    for i, L in enumerate(cfg["layers"]):
        l, m, f, p = f"l{i}.", L["mixer"], L["mlp"], f"l{i}.mix."
        w[l + "norm1"], w[l + "rg1"], w[l + "rg1.b"] = number(), mat(D, D, 2.0), bf(g.standard_normal(D))
        if L["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w[p + "q"], w[p + "k"], w[p + "v"] = mat(H * dk, D, sharp), mat(G * dk, D), mat(G * dv, D)
            w[p + "temp"], w[p + "g"], w[p + "o"] = bf(g.uniform(0.5, 2.0, H)), mat(H * dv, D, 2.0), mat(D, H * dv)
        elif L["type"] == "lightning":
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            w[p + "q"], w[p + "k"], w[p + "v"], w[p + "g"] = mat(H * dk, D), mat(H * dk, D), mat(H * dv, D), mat(H * dv, D)
            w[p + "norm"], w[p + "o"] = near_one(H * dv), mat(D, H * dv)
        else:
            H, dn, dr, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            w[p + "dq"], w[p + "dq.norm"], w[p + "uq"] = mat(Q, D), near_one(Q), mat(H * (dn + dr), Q, sharp)
            if m.get("kv_from") is None:
                w[p + "dkv"], w[p + "dkv.norm"] = mat(R + dr, D), near_one(R)
            w[p + "uk"], w[p + "uv"], w[p + "o"] = mat(H * dn, R), mat(H * dv, R), mat(D, H * dv)
        if f is None:
            continue
        w[l + "norm2"], w[l + "rg2"], w[l + "rg2.b"] = number(), mat(D, D, 2.0), bf(g.standard_normal(D))
        w[l + "mlp.gate"], w[l + "mlp.up"], w[l + "mlp.down"] = mat(f["ff"], D, 2.0), mat(f["ff"], D), mat(D, f["ff"])
    return w


def write_folder(path, cfg, w):
    from burn_lm_amd.weights import safetensors_io as st
    with open(path / "config.json", "w") as f:
        json.dump(cfg, f)
    st.write_file(str(path / "model.safetensors"), ((k, torch.from_numpy(np.asarray(v)).bfloat16()) for k, v in w.items()))
    return str(path)


def tokens_of(cfg, seed, n):
    return [int(x) for x in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


# ---- CPU: configuration, plan, random checkpoint, plain implementation ----------------------------
def test_config_is_read_and_refused_by_key():
    from burn_lm_amd import registry
    from burn_lm_amd.errors import ConfigError
    import burn_lm_amd.models  # noqa: F401
    arch = registry.architecture_of(MIXED)
    assert arch.name == "Bitonex"
    cfg = arch.read_config(MIXED)
    assert cfg.layers[2].mlp is None and cfg.layers[4].mlp.ff == 24 and cfg.residual_mult == 0.6 and cfg.logit_softcap == 20.0
    assert cfg.layers[3].mixer.kv_from == 0 and cfg.layers[0].mixer.kv_from is None and cfg.layers[4].mixer.rot_dims == 2
    assert cfg.layers[6].mixer.decay == (0.97, 0.3)
    odd = arch.read_config(ODD)
    assert odd.logit_softcap == 0.0 and odd.layers[2].mixer.decay == (0.75,) and odd.layers[5].mixer.rot_dims == 0
    for path, value, word in ((("layers", 1, "mixer", "vdim"), None, "vdim"), (("width",), "48", "width"),
                              (("layers", 0, "type"), "serial", "type"), (("norm",), {}, "eps"),
                              (("layers", 1, "mixer", "kv_heads"), 3, "kv_heads"),
                              (("layers", 1, "mixer", "rot"), dict(base=10.0, dims=18), "rot"),
                              (("layers", 2, "mixer", "decay"), [0.5, 0.5], "decay"),
                              (("layers", 2, "mixer", "decay"), [0.5, 0.5, 1.5], "decay"),
                              (("layers", 3, "mixer", "kv_from"), 3, "kv_from"),
                              (("layers", 3, "mixer", "kv_from"), 1, "kv_from"),
                              (("layers", 5, "mixer", "kv_from"), 3, "kv_from"),
                              (("layers", 3, "mixer", "kv_rank"), 16, "kv_rank"),
                              (("layers", 0, "mixer", "rot_dim"), None, "rot_dim"),
                              (("logit_softcap",), "high", "logit_softcap"),
                              (("layers", 0, "mlp"), dict(kind="moe", ff=8), "kind")):
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
    from burn_lm_amd.parts.base import KVNeed, StateNeed
    for cfg_dict in (MIXED, ODD):
        w = make_weights(cfg_dict, 0)
        arch = registry.architecture_of(cfg_dict)
        cfg = arch.read_config(cfg_dict)
        model = Model(arch.plan(cfg, {k: v.shape for k, v in w.items()}))
        assert {k: tuple(s.shape) for k, s in model.tensor_specs().items()} == {k: tuple(v.shape) for k, v in w.items()}
        assert {k: tuple(v[0]) for k, v in arch.checkpoint_tensors(cfg).items()} == {k: tuple(v.shape) for k, v in w.items()}
    needs = model.cache_needs()
    assert needs[0] == KVNeed(3, 10, 0, value_dim=6) and needs[2] == StateNeed((1, 5, 65))
    assert needs[1] == needs[4] == KVNeed(1, 17, 0, no_values=True)
    assert model.reads_from() == [None, None, None, None, 1, None]
    assert all(b.mixer.graph_safe for b in model.blocks)
    # the size of the queries' latent may be in the checkpoint's shapes alone
    bare = json.loads(json.dumps(MIXED))
    for L in bare["layers"]:
        L["mixer"].pop("q_rank", None)
    w = make_weights(MIXED, 0)
    arch = registry.architecture_of(bare)
    model = Model(arch.plan(arch.read_config(bare), {k: v.shape for k, v in w.items()}))
    assert model.tensor_specs()["l5.mix.uq"].shape == (5 * 12, 32)


def test_random_folder_loads_into_the_plain_implementation(tmp_path):
    import burn_lm_amd
    from burn_lm_amd.weights import safetensors_io as st
    folder = burn_lm_amd.write_random_model(str(tmp_path), ODD, seed=5)
    w = {n: f.tensor(n).double().numpy() for n, f in st.open_folder(folder).items()}
    assert w["l0.norm1"].shape == () and "l1.norm2" not in w and "l4.mix.dkv" not in w and w["l2.mix.norm"].shape == (65,)
    logits = P.forward(w, ODD, tokens_of(ODD, 0, 9))
    assert logits.shape == (9, 53) and np.isfinite(logits).all() and logits.std() > 0.05


def test_plain_mechanisms_on_cases_worked_by_hand():
    # rotation: a quarter turn at the position whose angle is pi / 2.  Pairs half the turning lanes apart: (0, 2) and
    # (1, 3), the second slower (base^(-2/4)); adjacent pairs: (0, 1) and (2, 3); lane 4 passes
    x = np.array([[[1.0, 1.0, 0.0, 0.0, 7.0]]])
    c, s = math.cos(math.pi / 20), math.sin(math.pi / 20)
    assert np.allclose(P.turn(x, np.array([math.pi / 2]), 4, 100.0, "half"), [[[0.0, c, 1.0, s, 7.0]]], atol=1e-12)
    x = np.array([[[1.0, 0.0, 1.0, 0.0, 7.0]]])
    assert np.allclose(P.turn(x, np.array([math.pi / 2]), 4, 100.0, "interleaved"), [[[0.0, 1.0, c, s, 7.0]]], atol=1e-12)
    # equal scores: a query averages the values it sees; an open gate (sigmoid of a large number) lets them through,
    # a gate at zero halves them
    m = dict(heads=1, kv_heads=1, dim=2, vdim=1, scale=1.0, rot=dict(base=10.0, dims=2))
    W = {"a.q": np.zeros((2, 1)), "a.k": np.array([[1.0], [0.0]]), "a.v": np.array([[1.0]]), "a.temp": np.array([3.0]),
         "a.g": np.array([[100.0]]), "a.o": np.eye(1)}
    h = np.arange(1.0, 5.0).reshape(4, 1)
    assert np.allclose(P.attention(W, "a.", m, h)[:, 0], [1, 1.5, 2, 2.5])
    W["a.g"] = np.zeros((1, 1))
    assert np.allclose(P.attention(W, "a.", m, h)[:, 0], [0.5, 0.75, 1, 1.25])
    # the temperature multiplies the scores: two keys whose scores differ by d are weighted e^(d * temp) to one
    m = dict(heads=1, kv_heads=1, dim=1, vdim=1, scale=0.5, rot=dict(base=10.0, dims=0))
    W = {"a.q": np.array([[1.0]]), "a.k": np.array([[1.0]]), "a.v": np.array([[1.0]]), "a.temp": np.array([4.0]),
         "a.g": np.array([[100.0]]), "a.o": np.eye(1)}
    out = P.attention(W, "a.", m, np.array([[0.0], [1.0]]))        # the second query sees keys 0 and 1, values 0 and 1
    assert np.allclose(out[1, 0], math.exp(2.0) / (1 + math.exp(2.0)))
    # lightning attention with decay 1 is the running sum of k v^T; with decay 1/2 older tokens count half as much
    s1 = P.silu(1.0)
    r = dict(heads=1, dim=1, vdim=1, decay=[1.0])
    W = {"r.q": np.array([[1.0]]), "r.k": np.array([[1.0]]), "r.v": np.array([[1.0]]), "r.g": np.array([[0.0]]),
         "r.norm": np.array([1.0]), "r.o": np.array([[1.0]])}
    out, S = P.lightning(W, "r.", r, np.ones((3, 1)), 0.0)
    assert np.allclose(S, 3 * s1 * s1) and np.allclose(out, 0.5)       # o > 0, so its unit-RMS form is 1, times sigmoid(0)
    r["decay"] = [0.5]
    _, S = P.lightning(W, "r.", r, np.ones((3, 1)), 0.0)
    assert np.allclose(S, (1 + 0.5 + 0.25) * s1 * s1)
    _, S2 = P.lightning(W, "r.", r, np.ones((1, 1)), 0.0, state=S)
    assert np.allclose(S2, (1 + 0.5 + 0.25 + 0.125) * s1 * s1)
    # latent attention equals softmax attention over the keys and values that the latent expands to
    g = np.random.default_rng(1)
    m = dict(heads=2, dim=3, rot_dim=4, vdim=5, kv_rank=6, q_rank=7, scale=0.3, rot=dict(base=100.0, dims=4))
    W = {"m." + n: g.standard_normal(s) for n, s in (("dq", (7, 9)), ("dq.norm", (7,)), ("uq", (14, 7)), ("dkv", (10, 9)),
                                                    ("dkv.norm", (6,)), ("uk", (6, 6)), ("uv", (10, 6)), ("o", (9, 10)))}
    h = g.standard_normal((5, 9))
    rows = P.latent_rows(W, "m.", m, h, 1e-5)
    assert np.allclose(((rows[0] / W["m.dkv.norm"]) ** 2).mean(-1), 1.0, atol=1e-4)
    out = P.latent_attention(W, "m.", m, h, 1e-5, rows)
    first = (rows[0][0] @ W["m.uv"].T) @ W["m.o"].T                 # the first token sees only itself
    assert np.allclose(out[0], first)
    # the feed-forward's activation and the residual gate
    assert np.allclose(P.gelu_tanh(np.array([0.0, 10.0, -10.0])), [0.0, 10.0, 0.0], atol=1e-9)
    assert abs(P.gelu_tanh(1.0) - 0.841192) < 1e-6
    assert np.allclose(P.residual_gate({"g": np.array([[2.0]]), "g.b": np.array([-2.0])}, "g", np.array([[1.0]])), 0.5)
    # a norm with one number; the soft cap keeps logits below the cap and small ones as they are
    assert np.allclose(P.rms_norm(np.array([[3.0, 4.0]]), 2.0, 0.0), [[6 / math.sqrt(12.5), 8 / math.sqrt(12.5)]])
    cfg = config([lightning(heads=1, dim=1, vdim=1, decay=(1.0,), mlp=None)], width=1, vocab=2, mult=1.0, cap=3.0)
    W = {"embed": np.array([[1.0], [1.0]]), "final.norm": np.array(1.0), "head": np.array([[100.0], [0.001]]),
         "l0.norm1": np.array(1.0), "l0.rg1": np.zeros((1, 1)), "l0.rg1.b": np.array([-100.0])}
    W.update({"l0.mix." + k: np.ones((1, 1)) for k in ("q", "k", "v", "g", "o")})
    W["l0.mix.norm"] = np.ones(1)
    z = P.forward(W, cfg, [0])
    assert abs(z[0, 0] - 3.0) < 1e-6 and abs(z[0, 1] - 0.001) < 1e-6


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
@pytest.mark.parametrize("layers", [[attention(mlp=None)], [attention(heads=6, kv_heads=6, dim=8, vdim=8, rot=8, mlp=None)],
                                    [attention(heads=8, kv_heads=1, dim=32, vdim=32, rot=2, mlp=None)],
                                    [attention(heads=4, kv_heads=2, dim=32, vdim=64, rot=16, mlp=None)],
                                    [lightning(mlp=None)], [lightning(heads=1, dim=70, vdim=5, decay=(0.99,), mlp=None)],
                                    [latent(mlp=None)], [latent(heads=4, dim=16, rot_dim=16, vdim=16, kv_rank=32, q_rank=8, mlp=None)],
                                    [latent(mlp=None), latent(heads=2, dim=4, vdim=6, q_rank=16, kv_from=0, mlp=None)],
                                    [latent(kv_rank=32, rot_dim=16, mlp=None), lightning(mlp=None),
                                     latent(heads=18, dim=4, vdim=6, kv_rank=32, rot_dim=16, q_rank=16, kv_from=0, mlp=None)],
                                    [lightning(heads=1, dim=8, vdim=8, decay=(0.5,))]],
                         ids=["attention", "attention_ungrouped", "attention_one_kv_head", "attention_wide_values",
                              "lightning", "lightning_one_wide_head", "latent", "latent_larger", "latent_read_by_another", "latent_of_a_matrix_core_size_read_by_another",
                              "feed_forward"])
def test_every_mechanism_alone(tmp_path, layers, dtype):
    cfg = config(layers)
    w = make_weights(cfg, 3)
    eng = engine_for(tmp_path, cfg, w, dtype, graphs=False)
    toks = tokens_of(cfg, 4, 150)       # three pages
    want = P.forward(w, cfg, toks)
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
    want = [P.forward(w, cfg, r) for r in reqs]
    rows = Rows(dtype)
    for r, x in zip(reqs, want):
        rows.add(whole(eng, r), x, "whole")
    # a prompt in portions of several sizes, down to two tokens and one
    for sizes in ((2, 5, 57, 64, 3, 69), (63, 2, 1, 1, 133), (128, 72), (1, 1, 1, 2, 195)):
        s, at = eng.open(), 0
        for n in sizes:
            rows.add(eng.step([(s, reqs[0][at:at + n], list(range(n)))]).double().cpu().numpy(), want[0][at:at + n], sizes)
            at += n
        eng.close(s)
        assert at == 200
    # unequal batches: prompts in one step, then one token each; shorter requests end earlier; the second round
    # finds slots, pages and states that the first one used
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
    wa, wb = P.forward(w, cfg, a), P.forward(w, cfg, b)
    sa, sb = eng.open(), eng.open()
    rows = Rows(dtype)
    got = eng.step([(sa, a[:30], [29]), (sb, b[:3], [2])]).double().cpu().numpy()
    rows.add(got, np.stack([wa[29], wb[2]]), "prompts")
    for k in range(140):          # across two page borders; one shape, recorded and replayed
        got = eng.step([(sa, [a[30 + k]], [0]), (sb, [b[3 + k]], [0])]).double().cpu().numpy()
        rows.add(got, np.stack([wa[30 + k], wb[3 + k]]), k)
    rows.check()
    assert eng.graphs.replays >= 100


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_are_no_multiples_of_eight_and_values_of_one(tmp_path, dtype):
    cfg = ODD
    w = make_weights(cfg, 7)
    w["l3.mix.temp"][:] = 1.0
    eng = engine_for(tmp_path, cfg, w, dtype)
    reqs = [tokens_of(cfg, 30 + i, n) for i, n in enumerate((90, 31))]
    want = [P.forward(w, cfg, r) for r in reqs]
    slots = [eng.open(), eng.open()]
    rows = Rows(dtype)
    got = eng.step([(slots[0], reqs[0][:80], list(range(80))), (slots[1], reqs[1][:21], list(range(21)))]).double().cpu().numpy()
    rows.add(got[:80], want[0][:80], "prompt 0")
    rows.add(got[80:], want[1][:21], "prompt 1")
    for k in range(10):
        got = eng.step([(slots[0], [reqs[0][80 + k]], [0]), (slots[1], [reqs[1][21 + k]], [0])]).double().cpu().numpy()
        rows.add(got, np.stack([want[0][80 + k], want[1][21 + k]]), k)
    rows.check()


def marked(kind, cfg, w, marker):
    """Changes the first layer's weights so that the key of the token `marker` towers over every other key for every
    query, wherever it lies: coordinate 0 of the embeddings is zero but for the marker, coordinate 1 is the same for all
    tokens, one unturned key lane reads coordinate 0 and the same query lane reads coordinate 1."""
    D, m = cfg["width"], cfg["layers"][0]["mixer"]
    w["embed"][:, 0], w["embed"][:, 1] = 0.0, 2.0
    w["embed"][marker, 0] = 8.0
    big = 16.0
    e0, e1 = np.eye(D)[0] * big, np.eye(D)[1] * big
    if kind == "attention":
        lane = m["dim"] - 1                     # a lane that does not turn
        for g in range(m["kv_heads"]):
            w["l0.mix.k"][g * m["dim"] + lane] = e0
        for h in range(m["heads"]):
            w["l0.mix.q"][h * m["dim"] + lane] = e1
    else:
        R, Q, dn, dr = m["kv_rank"], m["q_rank"], m["dim"], m["rot_dim"]
        w["l0.mix.dkv"][0], w["l0.mix.dq"][0] = e0, e1           # latent lane 0 of keys and of queries
        for layer in (0, 1):
            mm = cfg["layers"][layer]["mixer"]
            for h in range(mm["heads"]):
                w[f"l{layer}.mix.uk"][h * mm["dim"]] = np.eye(R)[0] * 4.0
                w[f"l{layer}.mix.uq"][h * (mm["dim"] + mm["rot_dim"])] = np.eye(mm["q_rank"])[0] * 4.0
        w["l1.mix.dq"][0] = e1
    return w


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["attention", "latent"])
def test_one_key_far_back_among_hundreds(tmp_path, kind, dtype):
    """The marker's key towers over hundreds of others, so a logits row is decided by whether the marker is seen: the
    marker as the first token, at the last and first places of pages, and far back; rows before it must not know it; in
    a prompt and token by token.  For the latent attention a second layer reads the first one's rows."""
    if kind == "attention":
        cfg = config([attention(heads=4, kv_heads=2, dim=16, vdim=16, rot=8, scale=0.25, mlp=None)], cap=None)
    else:
        # a latent of a size that the matrix-core kernel takes in bfloat16 runs (float32 runs take the generic one)
        cfg = config([latent(kv_rank=32, rot_dim=16, scale=0.25, mlp=None),
                      latent(heads=2, dim=4, vdim=6, kv_rank=32, rot_dim=16, q_rank=16, scale=0.25, kv_from=0, mlp=None)], cap=None)
    marker = 7
    w = marked(kind, cfg, make_weights(cfg, 9), marker)
    eng = engine_for(tmp_path, cfg, w, dtype, max_tokens=1024)
    base = [t if t != marker else marker + 1 for t in tokens_of(cfg, 50, 400)]
    plain_none = P.forward(w, cfg, base)
    for at in (0, 63, 64, 127, 128, 5):
        toks = list(base)
        toks[at] = marker
        want = P.forward(w, cfg, toks)
        # the test's own premise: seeing the marker changes a row by far more than any tolerance
        assert rel_err(want[399], plain_none[399]) > 0.1 and (at == 0 or rel_err(want[at - 1], plain_none[at - 1]) < 1e-9)
        rows = Rows(dtype)
        rows.add(whole(eng, toks), want, ("prompt", at))
        s = eng.open()
        eng.step([(s, toks[:330], [])])
        got = np.stack([eng.step([(s, [t], [0])])[0].double().cpu().numpy() for t in toks[330:]])
        rows.add(got, want[330:], ("decoding", at))
        eng.close(s)
        rows.check()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_state_that_survives_hundreds_of_tokens(tmp_path, dtype):
    """One lightning head never forgets (decay 1) and one forgets slowly: what the first tokens wrote still decides
    the rows 500 tokens later, in a prompt that ends one past a chunk's edge and in decoding from a carried state."""
    cfg = config([lightning(heads=2, dim=8, vdim=8, decay=(1.0, 0.995), mlp=None)], cap=None)
    w = make_weights(cfg, 11)
    eng = engine_for(tmp_path, cfg, w, dtype, max_tokens=1024)
    toks = tokens_of(cfg, 60, 513)
    want = P.forward(w, cfg, toks)
    other = P.forward(w, cfg, [(toks[0] + 1) % cfg["vocab"]] + toks[1:])
    assert rel_err(other[512], want[512]) > 1e-3
    rows = Rows(dtype)
    rows.add(whole(eng, toks), want, "prompt")
    s = eng.open()
    rows.add(eng.step([(s, toks[:449], list(range(449)))]).double().cpu().numpy(), want[:449], "first portion")
    rows.add(np.stack([eng.step([(s, [t], [0])])[0].double().cpu().numpy() for t in toks[449:]]), want[449:], "decoding")
    eng.close(s)
    rows.check()


def drawn_config(seed):
    """A configuration drawn from the seed: one to five layers of any mixers in any order, head counts and sizes that
    are and are not multiples of eight, any grouping of the queries, rotation of some, all or no lanes, decays from fast
    to none, latent layers that read an earlier one's rows, layers without a feed-forward."""
    rng = np.random.default_rng(seed)
    pick = lambda *a: a[int(rng.integers(0, len(a)))]
    layers, keepers = [], []
    for i in range(int(rng.integers(1, 6))):
        mlp = None if rng.random() < 0.25 else dense(pick(8, 16, 40, 6, 64))
        kind = pick("attention", "lightning", "latent")
        if kind == "attention":
            G, dk = int(rng.integers(1, 4)), pick(8, 16, 24, 32, 48, 64, 12, 6, 80, 128)
            layers.append(attention(heads=G * int(rng.integers(1, 5)), kv_heads=G, dim=dk, vdim=pick(dk, dk, 8, 20, 64),
                                    rot=pick(0, *[d for d in (2, 4, 6, 8, 12, 16, 24, 32, 48, 64, 128) if d <= dk]),
                                    base=pick(100.0, 10000.0, 1e6), scale=pick(0.1, 0.25, 0.5), mlp=mlp))
        elif kind == "lightning":
            H = int(rng.integers(1, 5))
            layers.append(lightning(heads=H, dim=pick(8, 16, 24, 48, 5, 64, 128), vdim=pick(8, 16, 32, 20, 3, 64, 128),
                                    decay=[pick(0.3, 0.8, 0.95, 0.99, 0.999, 1.0) for _ in range(H)], mlp=mlp))
        else:
            src = pick(*keepers) if keepers and rng.random() < 0.5 else None
            if src is None:
                dr = pick(4, 8, 16, 32, 6, 64)
                layers.append(latent(heads=int(rng.integers(1, 7)), dim=pick(4, 8, 16, 32, 5, 64), rot_dim=dr, vdim=pick(8, 16, 12, 32, 64),
                                     kv_rank=pick(16, 32, 24, 64, 40, 128), q_rank=pick(8, 16, 24, 48),
                                     rot=pick(dr, dr, dr // 2 * 2 - 2 or 2), base=pick(100.0, 10000.0, 1e6),
                                     scale=pick(0.1, 0.25), mlp=mlp))
                keepers.append(i)
            else:
                sm = layers[src]["mixer"]
                layers.append(latent(heads=int(rng.integers(1, 7)), dim=pick(4, 8, 16, 5), rot_dim=sm["rot_dim"], vdim=pick(8, 16, 12),
                                     kv_rank=sm["kv_rank"], q_rank=pick(8, 16, 24), rot=sm["rot"]["dims"], base=sm["rot"]["base"],
                                     scale=pick(0.1, 0.25), kv_from=src, mlp=mlp))
    return config(layers, width=pick(40, 64, 96, 128, 72), vocab=pick(50, 101, 257), mult=pick(0.5, 1.0, 1.4),
                  eps=pick(1e-5, 1e-6), cap=pick(None, 10.0, 50.0))


def test_drawn_configurations_are_read():
    from burn_lm_amd import registry
    import burn_lm_amd.models  # noqa: F401
    kinds = set()
    for seed in range(11, 40):
        cfg = drawn_config(seed)
        registry.architecture_of(cfg).read_config(cfg)
        kinds |= {(L["type"], L["mixer"].get("kv_from") is not None) for L in cfg["layers"]}
    assert len(kinds) == 4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16, 17, 18, 19, 20])
def test_drawn_configurations(tmp_path, seed, dtype):
    """Unequal prompts in one step, then 32 tokens one by one, for configurations nobody chose by hand."""
    cfg = drawn_config(seed)
    w = make_weights(cfg, 100 + seed)
    eng = engine_for(tmp_path, cfg, w, dtype, max_tokens=2048)
    reqs = [tokens_of(cfg, 7 + seed + i, n) for i, n in enumerate((330, 9, 140))]
    want = [P.forward(w, cfg, r) for r in reqs]
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
    """The index arrays that the kernels read, for sequences laid out by hand."""

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


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_queries_take_their_heads_temperature_and_the_gates_columns_stay(dtype):
    """Pairs half the turning lanes apart, a factor per query head behind the rotation, keys and values into their
    pages, and the gate's columns behind the values untouched; then the gate on the heads' results."""
    from burn_lm_amd.csrc import ops
    dev = "cuda"
    H, G, dk, dv, rot, ps = 3, 1, 10, 6, 6, 64
    rng = np.random.default_rng(3)
    news, pasts, slots = [3, 1], [62, 130], [0, 1]               # one sequence crosses a page border
    step = _Step(news, pasts, slots, dev)
    T = sum(news)
    n_gate = H * dv
    rows = torch.from_numpy(rng.standard_normal((T, H * dk + G * (dk + dv) + 2 + n_gate))).to(dtype)
    tables = torch.tensor([[4, 1, -1], [0, 5, 2]], dtype=torch.int32, device=dev)
    pos = np.arange(256, dtype=np.float64)[:, None] * (50.0 ** (-2.0 * np.arange(rot // 2) / rot))[None, :]
    cs = torch.from_numpy(np.stack([np.cos(pos), np.sin(pos)], -1).astype(np.float32)).to(dev)
    kc = torch.zeros(6, G, ps, dk, dtype=dtype, device=dev)
    vc = torch.zeros(6, G, dv, ps, dtype=dtype, device=dev)
    temp = torch.tensor([0.5, 1.0, 3.0], device=dev)
    qkv = rows.to(dev).clone()
    ops.qkv_prepare(qkv, None, cs, rot, step, tables, kc, vc, ps, H, G, dk, dv, q_scale=temp)
    x = rows.double().numpy()
    positions = np.array([62, 63, 64, 130])
    q = P.turn(x[:, :H * dk].reshape(T, H, dk), positions, rot, 50.0, "half") * temp.double().cpu().numpy()[None, :, None]
    k = P.turn(x[:, H * dk:(H + G) * dk].reshape(T, G, dk), positions, rot, 50.0, "half")
    v = x[:, (H + G) * dk:(H + G) * dk + G * dv].reshape(T, G, dv)
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert np.abs(qkv[:, :H * dk].double().cpu().numpy().reshape(T, H, dk) - q).max() < tol
    assert torch.equal(qkv[:, H * dk:].cpu(), rows[:, H * dk:])       # keys and values as projected, and the gate
    for t, (b, p) in enumerate([(0, 62), (0, 63), (0, 64), (1, 130)]):
        page = int(tables[b, p // ps])
        assert np.abs(kc[page, :, p % ps].double().cpu().numpy() - k[t]).max() < tol
        assert np.abs(vc[page, :, :, p % ps].double().cpu().numpy() - v[t]).max() == 0
    # the gate: rows and gate columns with strides of their own; widths that are and are not multiples of eight
    for N, pad in ((18, 2), (24, 8), (64, 0)):
        a = torch.from_numpy(rng.standard_normal((5, N + pad))).to(dtype).to(dev)
        gate = torch.from_numpy(rng.standard_normal((5, 2 * N + 8)) * 3).to(dtype).to(dev)
        before = a.clone()
        ops.sigmoid_gate(a[:, :N], gate[:, 8:8 + N])
        want = before[:, :N].double().cpu().numpy() * P.sigmoid(gate[:, 8:8 + N].double().cpu().numpy())
        assert np.abs(a[:, :N].double().cpu().numpy() - want).max() < (1e-6 if dtype == torch.float32 else 2e-2)
        assert torch.equal(a[:, N:], before[:, N:])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_latent_rows_turn_in_adjacent_pairs_and_a_reader_writes_nothing(dtype):
    from burn_lm_amd.csrc import ops
    dev = "cuda"
    H, dn, dr, R, rot, ps = 2, 3, 6, 11, 4, 64
    rng = np.random.default_rng(5)
    news, pasts = [3, 1], [62, 130]
    step = _Step(news, pasts, [0, 1], dev)
    T = sum(news)
    down = torch.from_numpy(rng.standard_normal((T, R + dr + 3))).to(dtype)
    q = torch.from_numpy(rng.standard_normal((T, H * (dn + dr)))).to(dtype)
    norm_w = rng.uniform(0.5, 1.5, R)
    tables = torch.tensor([[4, 1, -1], [0, 5, 2]], dtype=torch.int32, device=dev)
    pos = np.arange(256, dtype=np.float64)[:, None] * (50.0 ** (-2.0 * np.arange(rot // 2) / rot))[None, :]
    cs = torch.from_numpy(np.stack([np.cos(pos), np.sin(pos)], -1).astype(np.float32)).to(dev)
    kc = torch.zeros(6, 1, ps, R + dr, dtype=dtype, device=dev)
    qabs = torch.zeros(T, H, R + dr, dtype=torch.float32, device=dev)
    f32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.float32, device=dev)
    ops.latent_write(down.to(dev), q.to(dev), f32(norm_w), 1e-5, cs, rot, qabs, kc, step, tables, ps, H, dn, R, dr, adjacent=True)
    positions = np.array([62, 63, 64, 130])
    x = down.double().numpy()
    c = P.rms_norm(x[:, :R], norm_w, 1e-5)
    kr = P.turn(x[:, None, R:R + dr], positions, rot, 50.0, "interleaved")[:, 0]
    qr = P.turn(q.double().numpy().reshape(T, H, dn + dr)[..., dn:], positions, rot, 50.0, "interleaved")
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert np.abs(qabs[:, :, R:].double().cpu().numpy() - qr).max() < tol
    for t, (b, p) in enumerate([(0, 62), (0, 63), (0, 64), (1, 130)]):
        row = kc[int(tables[b, p // ps]), 0, p % ps].double().cpu().numpy()
        assert np.abs(row[:R] - c[t]).max() < tol and np.abs(row[R:] - kr[t]).max() < tol
    # a layer that reads another's rows turns its queries and leaves the pages as they are
    kept = kc.clone()
    qabs2 = torch.zeros_like(qabs)
    ops.latent_write(None, q.to(dev), f32(np.ones(R)), 1e-5, cs, rot, qabs2, kc, step, tables, ps, H, dn, R, dr, write_kv=False,
                     adjacent=True)
    assert torch.equal(kc, kept) and torch.equal(qabs2[:, :, R:], qabs[:, :, R:])
    # the norm of a slice of rows (the queries' latent)
    for N in (9, 64, 300):
        src = torch.from_numpy(rng.standard_normal((7, N + 5))).to(dtype).to(dev)
        wn = rng.uniform(0.5, 1.5, N)
        got = ops.rmsnorm_rows(src[:, 2:2 + N], f32(wn), 1e-6, torch.empty(7, N, dtype=dtype, device=dev))
        want = P.rms_norm(src[:, 2:2 + N].double().cpu().numpy(), wn, 1e-6)
        assert np.abs(got.double().cpu().numpy() - want).max() < (1e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_gated_add_activation_and_cap_against_the_plain_functions(dtype):
    from burn_lm_amd.csrc import ops
    dev = "cuda"
    rng = np.random.default_rng(2)
    f32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.float32, device=dev)
    act = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32)).to(dtype).to(dev)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    # widths that take the kernel with four channels per lane and the plain one; planes of partial products and a
    # single plane of the activation type; with and without a bias; all rows and chosen rows
    for T, D, planes in ((5, 20, 0), (7, 18, 3), (40, 64, 2), (3, 2048, 1), (2, 4100, 0)):
        h = rng.standard_normal((T, D))
        y = f32(rng.standard_normal((planes, T, D))) if planes else act(rng.standard_normal((T, D)))
        z, b, gamma = act(rng.standard_normal((T, D)) * 2), rng.standard_normal(D), rng.uniform(0.5, 1.5, D)
        ysum = y.double().cpu().numpy().sum(0) if planes else y.double().cpu().numpy()
        for bias in (b, None):
            gate = P.sigmoid(z.double().cpu().numpy() + (0 if bias is None else bias))
            new_h = h + 0.7 * ysum * gate
            hd = f32(h)
            out = ops.add_rmsnorm(hd, y, f32(gamma), 1e-5, torch.empty(T, D, dtype=dtype, device=dev), gate=z,
                                  gate_bias=None if bias is None else f32(bias), mult=0.7)
            assert np.abs(hd.double().cpu().numpy() - new_h).max() < 1e-5, (T, D, planes)
            assert rel_err(out.double().cpu().numpy(), P.rms_norm(new_h, gamma, 1e-5)) < tol, (T, D, planes)
            hd = f32(h)
            chosen = torch.tensor([T - 1, 0], dtype=torch.int32, device=dev)
            out = ops.add_rmsnorm(hd, y, f32(gamma), 1e-5, torch.empty(2, D, dtype=dtype, device=dev), rows=chosen,
                                  write_h=False, gate=z, gate_bias=None if bias is None else f32(bias), mult=0.7)
            assert torch.equal(hd, f32(h))
            assert rel_err(out.double().cpu().numpy(), P.rms_norm(new_h[[T - 1, 0]], gamma, 1e-5)) < tol
    for T, I in ((5, 24), (3, 13), (130, 64)):
        gu = act(rng.standard_normal((T, 2 * I)) * 3)
        x = gu.double().cpu().numpy()
        got = ops.gelu_glu(gu, torch.empty(T, I, dtype=dtype, device=dev))
        assert rel_err(got.double().cpu().numpy(), P.gelu_tanh(x[:, :I]) * x[:, I:]) < tol
    if dtype == torch.bfloat16:
        # few rows: the activation in the epilogue of the product on packed weights
        for M, K, I in ((1, 64, 32), (5, 96, 48), (16, 256, 128), (40, 128, 64)):
            x, wgu = act(rng.standard_normal((M, K))), act(rng.standard_normal((2 * I, K)) / math.sqrt(K) * 3)
            pre = x.double().cpu().numpy() @ wgu.double().cpu().numpy().T
            got = ops.gemv_mfma(x, ops.pack_weight(wgu, gated=True), torch.empty(M, I, dtype=dtype, device=dev), K, gated=True,
                                activation="gelu_tanh")
            assert rel_err(got.double().cpu().numpy(), P.gelu_tanh(pre[:, :I]) * pre[:, I:]) < tol, (M, K, I)
        # many rows: the activation in the epilogue of the tiled product
        for M, K, I, tile in ((130, 128, 192, (128, 128)), (300, 256, 256, (256, 128)), (70, 64, 40, (128, 64, 6))):
            x, wgu = act(rng.standard_normal((M, K))), act(rng.standard_normal((2 * I, K)) / math.sqrt(K) * 3)
            pre = x.double().cpu().numpy() @ wgu.double().cpu().numpy().T
            got = ops.gemm_mfma(x, wgu, torch.empty(M, I, dtype=dtype, device=dev), gated=True, tile=tile, activation="gelu_tanh")
            assert rel_err(got.double().cpu().numpy(), P.gelu_tanh(pre[:, :I]) * pre[:, I:]) < tol, (M, K, I)
    z = f32(rng.standard_normal((9, 77)) * 40)
    want = 15.0 * np.tanh(z.double().cpu().numpy() / 15.0)
    assert np.abs(ops.softcap(z, 15.0).double().cpu().numpy() - want).max() < 1e-5


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
            toks.append(int(np.argmax(P.forward(w, cfg, toks)[-1])))
        return toks[len(p):]

    want = [plain_greedy(p, 6) for p in prompts]
    server = InferenceServer(folder, dtype="float32", batch_size=3)       # two batches: slots are used again
    server.config.update(max_seq_len=256, sample_len=6, temperature=0.0)
    results, _ = server.generate(prompts, stop_ids=[])
    assert [r.tokens for r in results] == want
    server.unload()

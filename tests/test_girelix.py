"""The Girelix design in the engine against the plain implementation of tests/plain_girelix.py.

The configurations and weights are made here.  The CPU tests cover the configuration reader, the plan, the random
checkpoint and the plain implementation's own consistency on cases worked by hand; the GPU tests run the engine's step
function, cache, scheduler and kernels: each mixer of the pair and each router variant alone, whole prompts against
token-by-token decoding, prompts in portions, unequal batches, slots, pages and states used again, one key that stands
out far back and at page borders (in prompts and in decoding), the sink, a state that must survive hundreds of
tokens, long decoding through recorded graphs, odd sizes, configurations drawn from seeds, and greedy generation
through the server."""
import json
import math

import numpy as np
import pytest
import torch

import plain_girelix as P
from helpers import rel_err

TOL = {"float32": 2e-5, "bfloat16": 8e-2}


class Rows:
    """Collects rows of logits beside what they should be.  float32: every row within the tolerance.  bfloat16: a
    rounding can tip a router's choice between two experts whose scores are close, which changes that token's row by
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
def moe(experts=5, identity=1, top=2, count=3, keep=2, ff=24):
    router = dict(experts=experts, top=top)
    if identity:
        router["identity"] = identity
    if count:
        router["groups"] = dict(count=count, keep=keep)
    return dict(kind="moe", expert=dict(ff=ff), router=router)


def layer(heads=4, kv_heads=2, dim=16, rot=12, base=10000.0, scale=None, r_heads=3, r_dim=12, r_vdim=20,
          decay=(0.5, 0.9, 1.0), left_scale=0.8, right_scale=1.25, mlp="default"):
    left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale or 1.0 / math.sqrt(dim))
    if rot:
        left["rot"] = dict(base=base, dims=rot)
    right = dict(heads=r_heads, dim=r_dim, vdim=r_vdim, decay=list(decay))
    return dict(type="parallel", mixer=dict(left=left, right=right, left_scale=left_scale, right_scale=right_scale),
                mlp=moe() if mlp == "default" else mlp)


def config(layers, width=48, vocab=101, mult=0.6, eps=1e-5):
    return dict(architecture="Girelix", layers=layers, norm=dict(eps=eps), residual_mult=mult, vocab=vocab, width=width)


# layers that differ from each other in every size; one without a feed-forward; routers with and without groups and
# pass-through experts
MIXED = config([layer(), layer(heads=6, kv_heads=1, dim=8, rot=8, r_heads=2, r_dim=16, r_vdim=8, decay=(0.97, 0.3),
                              mlp=moe(experts=4, identity=0, top=1, count=0)),
                layer(heads=2, kv_heads=2, dim=32, rot=2, r_heads=1, r_dim=24, r_vdim=40, decay=(0.999,), mlp=None),
                layer(mlp=moe(experts=2, identity=4, top=3, count=2, keep=1))])
# sizes that are no multiples of eight, lanes that do not turn, no rotation at all, a residual multiplier of one, one
# value lane more than a wavefront, as many pass-through experts as real ones
ODD = config([layer(heads=3, kv_heads=3, dim=10, rot=4, r_heads=3, r_dim=10, r_vdim=14, decay=(0.2, 0.8, 0.95),
                    mlp=moe(experts=3, identity=3, top=2, count=2, keep=2, ff=12)),
              layer(heads=5, kv_heads=1, dim=6, rot=0, r_heads=1, r_dim=5, r_vdim=65, decay=(1.0,), left_scale=1.0,
                    right_scale=0.3, mlp=moe(experts=7, identity=0, top=7, count=1, keep=1, ff=5)),
              layer(heads=2, kv_heads=1, dim=12, rot=12, base=300.0, r_heads=2, r_dim=70, r_vdim=3, decay=(0.6, 0.99), mlp=None)],
             width=36, vocab=53, mult=1.0, eps=1e-6)


def make_weights(cfg, seed, sharp=1.0):
    """float64 arrays that are exact in bfloat16.  sharp: factor on the query projections of the softmax attention,
    so that it singles out few keys."""
    g = np.random.default_rng(seed)
    D = cfg["width"]
    bf = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32)).bfloat16().double().numpy()
    mat = lambda o, i, s=1.0: bf(g.standard_normal((o, i)) * s / math.sqrt(i))
    near_one = lambda n: bf(1 + 0.1 * g.standard_normal(n))
    w = {"embed": bf(g.standard_normal((cfg["vocab"], D))), "final.norm": near_one(D), "head": mat(cfg["vocab"], D)}
    for i, L in enumerate(cfg["layers"]):
        l, a, b, f = f"l{i}.", L["mixer"]["left"], L["mixer"]["right"], L["mlp"]
        w[l + "norm1"], w[l + "ls1"] = near_one(D), bf(g.uniform(0.5, 1.2, D))
        p = l + "mix.left."
        w[p + "q"], w[p + "k"] = mat(a["heads"] * a["dim"], D, sharp), mat(a["kv_heads"] * a["dim"], D)
        w[p + "sink"], w[p + "o"] = bf(g.standard_normal(a["heads"]) + 1.0), mat(D, a["heads"] * a["vdim"])
        p = l + "mix.right."
        H, dk, dv = b["heads"], b["dim"], b["vdim"]
        w[p + "q"], w[p + "k"], w[p + "v"], w[p + "g"] = mat(H * dk, D), mat(H * dk, D), mat(H * dv, D), mat(H * dv, D)
        w[p + "norm"], w[p + "o"] = near_one(H * dv), mat(D, H * dv)
        if f is None:
            continue
        w[l + "ls2"] = bf(g.uniform(0.5, 1.2, D))
        p = l + "mlp."
        E, n = f["router"]["experts"], f["router"]["experts"] + f["router"].get("identity", 0)
        w[p + "router"], w[p + "correction"] = mat(n, D, 2.0), bf(g.standard_normal(n) * 0.5 / n)
        for e in range(E):
            fe = f["expert"]["ff"]
            w[f"{p}e{e}.gate"], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"] = mat(fe, D), mat(fe, D), mat(D, fe)
    return w


def write_folder(path, cfg, w):
    from burn_lm_amd.weights import safetensors_io as st
    with open(path / "config.json", "w") as f:
        json.dump(cfg, f)
    st.write_file(str(path / "model.safetensors"), ((k, torch.from_numpy(v).bfloat16()) for k, v in w.items()))
    return str(path)


def tokens_of(cfg, seed, n):
    return [int(x) for x in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


# ---- CPU: configuration, plan, random checkpoint, plain implementation ----------------------------
def test_config_is_read_and_refused_by_key():
    from burn_lm_amd import registry
    from burn_lm_amd.errors import ConfigError
    import burn_lm_amd.models  # noqa: F401
    arch = registry.architecture_of(MIXED)
    assert arch.name == "Girelix"
    cfg = arch.read_config(MIXED)
    assert cfg.layers[2].mlp is None and cfg.layers[1].mlp.identity == 0 and cfg.layers[1].mlp.groups == 1
    assert cfg.layers[3].mlp.identity == 4 and cfg.layers[3].mlp.keep == 1 and cfg.residual_mult == 0.6
    assert cfg.layers[1].mixer.right.decay == (0.97, 0.3) and cfg.layers[2].mixer.left.rot_dims == 2
    for path, value, word in ((("layers", 1, "mixer", "left", "vdim"), None, "vdim"), (("width",), "48", "width"),
                              (("layers", 0, "type"), "serial", "type"), (("norm",), {}, "eps"),
                              (("layers", 1, "mixer", "left", "kv_heads"), 4, "kv_heads"), (("residual_mult",), None, "residual_mult"),
                              (("layers", 0, "mixer", "left", "vdim"), 8, "keys"),
                              (("layers", 0, "mixer", "left", "rot"), dict(base=10.0, dims=18), "rot"),
                              (("layers", 0, "mixer", "right", "decay"), [0.5, 0.5], "decay"),
                              (("layers", 0, "mixer", "right", "decay"), [0.5, 0.5, 1.5], "decay"),
                              (("layers", 0, "mixer", "left_scale"), None, "left_scale"),
                              (("layers", 0, "mlp", "router", "groups"), dict(count=4, keep=2), "groups"),
                              (("layers", 0, "mlp", "router", "groups"), dict(count=3, keep=4), "groups"),
                              (("layers", 3, "mlp", "router", "top"), 4, "top"),
                              (("layers", 0, "mlp"), dict(kind="dense", ff=8), "kind")):
        bad = json.loads(json.dumps(MIXED))
        at = bad
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            arch.read_config(bad)
    none = json.loads(json.dumps(MIXED))
    none["layers"][0]["mixer"]["left"]["rot"] = dict(base=10000.0, dims=0)      # no lanes turn
    assert arch.read_config(none).layers[0].mixer.left.rot_dims == 0
    one = json.loads(json.dumps(MIXED))
    one["layers"][0]["mixer"]["right"]["decay"] = 0.75      # one number stands for every head
    assert arch.read_config(one).layers[0].mixer.right.decay == (0.75,) * one["layers"][0]["mixer"]["right"]["heads"]


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
    assert needs[0] == (KVNeed(3, 10, 0, value_dim=10), StateNeed((3, 10, 14))) and needs[1][1].shape == (1, 5, 65)
    assert all(b.mixer.graph_safe for b in model.blocks)


def test_random_folder_loads_into_the_plain_implementation(tmp_path):
    import burn_lm_amd
    from burn_lm_amd.weights import safetensors_io as st
    folder = burn_lm_amd.write_random_model(str(tmp_path), ODD, seed=5)
    w = {n: f.tensor(n).double().numpy() for n, f in st.open_folder(folder).items()}
    assert w["l0.mlp.router"].shape == (6, 36) and "l2.ls2" not in w and w["l1.mix.right.norm"].shape == (65,)
    logits = P.forward(w, ODD, tokens_of(ODD, 0, 9))
    assert logits.shape == (9, 53) and np.isfinite(logits).all() and logits.std() > 0.05


def test_plain_mechanisms_on_cases_worked_by_hand():
    # rotation: a quarter turn of the pair (lane 0, lane 1) at the position whose angle is pi / 2; lanes 2 and 3 turn
    # slower (base^(-2/4)); lane 4 passes
    x = np.array([[[1.0, 0.0, 1.0, 0.0, 7.0]]])
    got = P.rotate_pairs(x, np.array([math.pi / 2]), 4, 100.0)
    assert np.allclose(got, [[[0.0, 1.0, math.cos(math.pi / 20), math.sin(math.pi / 20), 7.0]]], atol=1e-12)
    # equal scores: a query averages the keys it sees (the values are the keys), and a sink at their score takes one
    # share more; the key is unrotated as a value
    m = dict(heads=1, kv_heads=1, dim=2, vdim=2, scale=1.0, rot=dict(base=10.0, dims=2))
    W = {"a.q": np.zeros((2, 1)), "a.k": np.array([[1.0], [0.0]]), "a.sink": np.array([-1e9]), "a.o": np.eye(2)}
    h = np.arange(1.0, 5.0).reshape(4, 1)
    assert np.allclose(P.softmax_attention(W, "a.", m, h), [[1, 0], [1.5, 0], [2, 0], [2.5, 0]])
    W["a.sink"] = np.array([0.0])
    assert np.allclose(P.softmax_attention(W, "a.", m, h)[:, 0], [1 / 2, 3 / 3, 6 / 4, 10 / 5])
    # lightning attention with decay 1 is the running sum of k v^T; with decay 1/2 older tokens count half as much
    s1 = P.silu(1.0)
    r = dict(heads=1, dim=1, vdim=1, decay=[1.0])
    W = {"r.q": np.array([[1.0]]), "r.k": np.array([[1.0]]), "r.v": np.array([[1.0]]), "r.g": np.array([[0.0]]),
         "r.norm": np.array([1.0]), "r.o": np.array([[1.0]])}
    out, S = P.lightning_attention(W, "r.", r, np.ones((3, 1)), 0.0)
    assert np.allclose(S, 3 * s1 * s1) and np.allclose(out, 0.5)       # o > 0, so its unit-RMS form is 1, times sigmoid(0)
    r["decay"] = [0.5]
    _, S = P.lightning_attention(W, "r.", r, np.ones((3, 1)), 0.0)
    assert np.allclose(S, (1 + 0.5 + 0.25) * s1 * s1)
    _, S2 = P.lightning_attention(W, "r.", r, np.ones((1, 1)), 0.0, state=S)
    assert np.allclose(S2, (1 + 0.5 + 0.25 + 0.125) * s1 * s1)
    # routing: six outputs in three pairs; expert e multiplies by 10^e; outputs 4 and 5 pass the input through
    scores = np.array([0.30, 0.05, 0.25, 0.02, 0.28, 0.10])
    f = dict(kind="moe", expert=dict(ff=1), router=dict(experts=4, identity=2, top=2, groups=dict(count=3, keep=2)))
    W = {"m.router": np.log(scores).reshape(6, 1), "m.correction": np.array([0, 0, 0, 0.5, -0.2, -0.2])}
    for e in range(4):
        W[f"m.e{e}.gate"], W[f"m.e{e}.up"], W[f"m.e{e}.down"] = np.array([[1.0]]), np.array([[1.0]]), np.array([[10.0 ** e]])
    one = np.array([[1.0]])
    # corrected: [.30 .05 .25 .52 .08 -.10]; pairs rank .30 .52 .08, the last pair is out; chosen 3 and 0 with the
    # weights of the uncorrected scores .02 and .30
    chosen, wts = P.route(W, "m.", f, one)
    assert list(chosen[0]) == [3, 0] and np.allclose(wts[0], [0.02 / 0.32, 0.30 / 0.32])
    assert np.allclose(P.experts(W, "m.", f, one), s1 * (0.9375 + 0.0625 * 1000))
    # without correction and with all groups: the largest scores, one of them a pass-through expert
    W["m.correction"] = np.zeros(6)
    f["router"]["groups"] = dict(count=3, keep=3)
    assert np.allclose(P.experts(W, "m.", f, one), (0.30 * s1 + 0.28 * 1.0) / 0.58)
    # one group kept, two chosen: its second expert is taken although its corrected score is negative and those of
    # the groups left out are not
    W["m.correction"] = np.array([0, 0, 0.5, -0.3, 0, 0])
    f["router"]["groups"] = dict(count=3, keep=1)
    chosen, wts = P.route(W, "m.", f, one)
    assert list(chosen[0]) == [2, 3] and np.allclose(wts[0], [0.25 / 0.27, 0.02 / 0.27])


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
@pytest.mark.parametrize("layers", [[layer(right_scale=0.0, mlp=None)],
                                    [layer(heads=6, kv_heads=6, dim=8, rot=8, right_scale=0.0, mlp=None)],
                                    [layer(heads=8, kv_heads=1, dim=32, rot=2, right_scale=0.0, mlp=None)],
                                    [layer(left_scale=0.0, mlp=None)],
                                    [layer(left_scale=0.0, r_heads=1, r_dim=70, r_vdim=5, decay=(0.99,), mlp=None)],
                                    [layer(mlp=None)], [layer()], [layer(mlp=moe(experts=3, identity=0, top=1, count=0))],
                                    [layer(mlp=moe(experts=1, identity=5, top=2, count=3, keep=1))]],
                         ids=["softmax", "softmax_ungrouped", "softmax_one_kv_head", "lightning", "lightning_one_wide_head",
                              "pair", "experts", "experts_top1_plain", "experts_mostly_pass_through"])
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
def test_sizes_that_are_no_multiples_of_eight(tmp_path, dtype):
    cfg = ODD
    w = make_weights(cfg, 7)
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


def drawn_config(seed):
    """A configuration drawn from the seed: one to four layers, head counts and sizes that are and are not multiples of
    eight, any grouping of the queries, rotation of some, all or no lanes, decays from fast to none, routers with and
    without groups and pass-through experts, layers without a feed-forward."""
    rng = np.random.default_rng(seed)
    pick = lambda *a: a[int(rng.integers(0, len(a)))]
    layers = []
    for _ in range(int(rng.integers(1, 5))):
        G, dk = int(rng.integers(1, 4)), pick(8, 16, 24, 32, 48, 64, 12, 6, 80, 96, 128)
        rh = int(rng.integers(1, 5))
        if rng.random() < 0.25:
            mlp = None
        else:
            count = pick(0, 1, 2, 3, 4)
            per = int(rng.integers(1, 4))
            n = max(1, count) * per if count else int(rng.integers(1, 9))
            identity = int(rng.integers(0, n))
            keep = int(rng.integers(1, count + 1)) if count else 1
            room = keep * per if count else n
            mlp = moe(experts=n - identity, identity=identity, top=int(rng.integers(1, room + 1)), count=count, keep=keep,
                      ff=pick(8, 16, 40, 6))
        layers.append(layer(heads=G * int(rng.integers(1, 5)), kv_heads=G, dim=dk,
                            rot=pick(0, *[d for d in (2, 4, 6, 8, 12, 16, 24, 32, 48, 64, 96, 128) if d <= dk]),
                            base=pick(100.0, 10000.0, 5e5), scale=pick(0.1, 0.25, 0.5), r_heads=rh,
                            r_dim=pick(8, 16, 24, 48, 5, 64, 128), r_vdim=pick(8, 16, 32, 20, 3, 64, 128),
                            decay=[pick(0.3, 0.8, 0.95, 0.99, 0.999, 1.0) for _ in range(rh)],
                            left_scale=pick(0.5, 1.0, 1.5), right_scale=pick(0.5, 1.0, 1.5), mlp=mlp))
    return config(layers, width=pick(40, 64, 96, 128, 72), vocab=pick(50, 101, 257), mult=pick(0.5, 1.0, 1.4), eps=pick(1e-5, 1e-6))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16, 17, 18])
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


def _attend(form, *args):
    """The generic kernel, the matrix-core one with its pages whole or cut into pieces, or the plain attention's
    kernels given the sink (16 or 32 queries per wavefront in prompts, key ranges whole or cut in decoding)."""
    from burn_lm_amd.csrc import ops
    if form == "generic":
        return ops.sink_attn(*args)
    if form.startswith("plain"):
        q, out, sinks, mix, step, table, kc, vc, ps, H, G, dk, dv, scale, window = args
        assert mix is None and dk == dv
        if step.max_new == 1:
            return ops.attn_decode(q, q.stride(0), out, step.positions, step.token_seq, table, kc, vc, ps, H, G, dk, scale,
                                   window, n_splits=3 if form == "plain_cut" else 1, sinks=sinks)
        return ops.attn_prefill_mfma(q, q.stride(0), out, step.positions, step.cu_seqlens, table, kc, vc, ps, step.n_seqs,
                                     step.max_new, H, G, dk, scale, window, queries=32 if form == "plain_cut" else 16, sinks=sinks)
    return ops.sink_attn_mfma(*args, n_splits=1 if form == "matrix" else 3, group_batch=0 if form == "matrix" else 1)


FORMS = [("generic", torch.float32), ("generic", torch.bfloat16), ("matrix", torch.bfloat16), ("matrix_pieces", torch.bfloat16),
         ("plain", torch.bfloat16), ("plain_cut", torch.bfloat16)]
FORM_IDS = ["generic-float32", "generic-bfloat16", "matrix", "matrix_pieces", "plain", "plain_cut"]


@pytest.mark.gpu
@pytest.mark.parametrize("form,dtype", FORMS, ids=FORM_IDS)
@pytest.mark.parametrize("decode", [False, True], ids=["prompt", "decoding"])
def test_one_key_far_back_among_hundreds_and_the_sink(form, dtype, decode):
    """No window and no head mixing.  One key's score towers over hundreds of others: the result must be that key's
    value wherever the key lies (the first token, the last and first places of pages that lie scattered), and must not
    know it before the query reaches it.  Then the sink towers over all keys, and the result must be nothing."""
    dev = "cuda"
    H, G, dk, ps = 4, 2, (32 if form.startswith("plain") else 8), 64
    g = torch.Generator().manual_seed(0)
    pages = [7, 2, 5, 0, 8, 3]                                   # the sequence's pages; pages 1, 4, 6 hold noise
    kc = torch.randn(9, G, ps, dk, generator=g) * 0.1
    vc = torch.randn(9, G, dk, ps, generator=g)
    table = torch.tensor([pages + [-1] * 2], dtype=torch.int32, device=dev)
    marked = [0, 63, 64, 191, 192, 320]                         # the later the key, the larger its score
    value = lambda j: float(j % 97 + 1)
    for rank, j in enumerate(marked):
        kc[pages[j // ps], :, j % ps, :] = 0.0
        kc[pages[j // ps], :, j % ps, 0] = float(rank + 1)
        vc[pages[j // ps], :, :, j % ps] = value(j)
    queries = [(p, max(j for j in marked if j <= p)) for p in (0, 62, 63, 64, 190, 191, 192, 319, 320, 340)]
    steps = [([1], [p]) for p, _ in queries] if decode else [([341], [0])]
    for sink in (-30.0, 500.0):
        for news, pasts in steps:
            step = _Step(news, pasts, [0], dev)
            T = step.n_tokens
            q = torch.zeros(T, H * dk)
            q.view(T, H, dk)[:, :, 0] = 40.0
            out = torch.empty(T, H * dk, dtype=dtype, device=dev)
            _attend(form, q.to(dev, dtype), out, torch.full((H,), sink, device=dev), None, step, table,
                    kc.to(dev, dtype).contiguous(), vc.to(dev, dtype).contiguous(), ps, H, G, dk, dk, 1.0, 0)
            out = out.float().cpu().view(T, H, dk)
            for p, j in queries:
                row = p - pasts[0]
                if 0 <= row < T:
                    want = value(j) if sink < 0 else 0.0
                    assert torch.allclose(out[row], torch.full((H, dk), want), atol=1e-3), (sink, p, j)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_keys_are_turned_in_adjacent_pairs_and_kept_unturned_as_values(dtype):
    from burn_lm_amd.csrc import ops
    dev = "cuda"
    H, G, dk, rot, ps = 3, 2, 10, 6, 64
    rng = np.random.default_rng(3)
    news, pasts, slots = [3, 1], [62, 130], [0, 1]               # one sequence crosses a page border
    step = _Step(news, pasts, slots, dev)
    T = sum(news)
    rows = torch.from_numpy(rng.standard_normal((T, (H + G) * dk + 6))).to(dtype)     # six columns nobody may touch
    tables = torch.tensor([[4, 1, -1], [0, 5, 2]], dtype=torch.int32, device=dev)
    pos = np.arange(256, dtype=np.float64)[:, None] * (50.0 ** (-2.0 * np.arange(rot // 2) / rot))[None, :]
    cs = torch.from_numpy(np.stack([np.cos(pos), np.sin(pos)], -1).astype(np.float32)).to(dev)
    kc = torch.zeros(6, G, ps, dk, dtype=dtype, device=dev)
    vc = torch.zeros(6, G, dk, ps, dtype=dtype, device=dev)
    qkv = rows.to(dev).clone()
    ops.qkv_prepare(qkv, None, cs, rot, step, tables, kc, vc, ps, H, G, dk, dk, adjacent=True, values_are_keys=True)
    x = rows.double().numpy()
    positions = np.array([62, 63, 64, 130])
    q = P.rotate_pairs(x[:, :H * dk].reshape(T, H, dk), positions, rot, 50.0)
    k = x[:, H * dk:(H + G) * dk].reshape(T, G, dk)
    kr = P.rotate_pairs(k, positions, rot, 50.0)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert np.abs(qkv[:, :H * dk].double().cpu().numpy().reshape(T, H, dk) - q).max() < tol
    assert torch.equal(qkv[:, H * dk:].cpu(), rows[:, H * dk:])       # keys as projected, and what lies behind them
    for t, (b, p) in enumerate([(0, 62), (0, 63), (0, 64), (1, 130)]):
        page = int(tables[b, p // ps])
        assert np.abs(kc[page, :, p % ps].double().cpu().numpy() - kr[t]).max() < tol
        assert np.abs(vc[page, :, :, p % ps].double().cpu().numpy() - k[t]).max() == 0
    assert float(kc[[0, 3, 5]].float().abs().sum()) == 0 and float(vc[[0, 3, 5]].float().abs().sum()) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("H,dk,dv", [(3, 12, 20), (10, 4, 250), (2, 128, 128), (3, 70, 33)],
                         ids=["small", "norm_over_2500_lanes", "largest_chunked_heads", "odd"])
@pytest.mark.parametrize("form", ["scan", "chunks"])
@pytest.mark.parametrize("news,slots", [([300, 40, 1], [2, 0, 3]), ([64, 65, 63, 128, 129, 1, 8, 2], [5, 0, 3, 8, 2, 7, 4, 6])],
                         ids=["long", "chunk_edges"])
def test_fading_state_kernel_against_the_plain_function(dtype, H, dk, dv, form, news, slots):
    """Three sequences in one step: a long prompt (walked in segments, or in chunks of 64 tokens whose last one is not
    full), a continuation from a state, one token from a state; heads that forget at once, slowly and never; a state slot
    that is not in the step stays as it was.  The recurrence is written out here once more, on rows that stand for the
    projections' results."""
    from burn_lm_amd.csrc import ops
    if form == "chunks" and not ops.lightning_chunks_supported(dk, dv):
        pytest.skip("heads of this size are not run in chunks")
    dev = "cuda"
    r = dict(heads=H, dim=dk, vdim=dv, decay=([0.05, 0.999, 1.0] * 4)[:H])
    rng = np.random.default_rng(4)
    bf = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32)).to(dtype).double().numpy()
    W = {"r.norm": rng.uniform(0.5, 1.5, H * dv)}
    act = lambda z: bf(P.silu(z))            # the activations are rounded to the rows' type
    states = rng.standard_normal((max(slots) + 1, H, dk, dv))      # slot 1 belongs to no sequence of the step
    states[slots[0]] = 0.0
    width = 2 * H * dk + 2 * H * dv
    proj = bf(rng.standard_normal((sum(news), width)))
    # the plain function projects its input with identities: one input per projection
    want, at = [], 0
    for n, slot in zip(news, slots):
        x = proj[at:at + n]
        q, k, v, gl = np.split(x, [H * dk, 2 * H * dk, 2 * H * dk + H * dv], axis=1)
        S = states[slot].copy()
        o = np.zeros((n, H, dv))
        for t in range(n):
            for hd in range(H):
                S[hd] = r["decay"][hd] * S[hd] + np.outer(act(k[t].reshape(H, dk)[hd]), act(v[t].reshape(H, dv)[hd]))
                o[t, hd] = S[hd].T @ act(q[t].reshape(H, dk)[hd])
        want.append((P.rms_norm(o.reshape(n, H * dv), W["r.norm"], 1e-5) * P.sigmoid(gl), S))
        at += n
    step = _Step(news, [0, 77, 500, 3, 64, 640, 1, 0][:len(news)], slots, dev)
    f32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.float32, device=dev)
    state_dev = f32(states)
    T = sum(news)
    out = torch.empty(T, H * dv, dtype=dtype, device=dev)
    if form == "chunks":
        ops.lightning_chunks_init(dev)
        ops.lightning_chunks(torch.from_numpy(proj).to(dev, dtype), ops.decay_powers(r["decay"], dev), f32(W["r.norm"]), 1e-5, state_dev,
                             torch.zeros(T, H * dv, dtype=torch.float32, device=dev), out, step, H, dk, dv,
                             activation="silu", norm_all=True, gate="sigmoid")
    else:
        ops.gla_scan(torch.from_numpy(proj).to(dev, dtype), None, None, None, f32(W["r.norm"]), 1e-5, state_dev,
                     torch.zeros(T, H * dv, dtype=torch.float32, device=dev), out, step, H, dk, dv,
                     segments=(3, 104) if max(news) > 200 else (2, 72),
                     fixed_decay=f32(np.repeat(r["decay"], dk)), activation="silu", q_scale=1.0, norm_all=True, gate="sigmoid")
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    at = 0
    for (o, S), n, slot in zip(want, news, slots):
        assert rel_err(out[at:at + n].double().cpu().numpy(), o) < tol, slot
        assert rel_err(state_dev[slot].double().cpu().numpy(), S) < 2e-5, slot
        at += n
    assert torch.equal(state_dev[1].cpu(), f32(states)[1].cpu())


@pytest.mark.gpu
def test_routing_and_adding_kernels_against_the_plain_functions():
    from burn_lm_amd.csrc import ops
    dev = "cuda"
    rng = np.random.default_rng(2)
    f32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.float32, device=dev)
    for E, I, count, keep, top in ((5, 3, 4, 2, 3), (6, 0, 1, 1, 2), (1, 5, 3, 3, 6), (9, 3, 6, 1, 2), (4, 4, 2, 1, 4), (7, 0, 0, 1, 7), (30, 10, 4, 3, 20), (100, 28, 8, 4, 9)):
        N, T = E + I, 257
        logits = rng.standard_normal((T, N + 3)) * 2              # three columns of padding behind the logits
        correction = rng.standard_normal(N) * 0.3
        f = dict(router=dict(experts=E, identity=I, top=top))
        if count:
            f["router"]["groups"] = dict(count=count, keep=keep)
        chosen, wts = P.route({"m.router": np.eye(N), "m.correction": correction}, "m.", f, logits[:, :N].astype(np.float32).astype(np.float64))
        want = np.zeros((T, E + 1))
        for t in range(T):
            for e, a in zip(chosen[t], wts[t]):
                want[t, min(e, E)] += a
        got = ops.moe_route_grouped(f32(logits), f32(correction), E, I, count, keep, top,
                                    torch.empty(T, E + 1, dtype=torch.float32, device=dev)).double().cpu().numpy()
        assert np.abs(got - want).max() < 1e-5, (E, I, count, keep, top)
        assert np.allclose(got.sum(1), 1.0, atol=1e-5)
    # sublayer results into the residual, each with its coefficients: float planes, one bfloat16 plane, a factor per
    # token read with a stride, a term without coefficients; widths that are and are not a multiple of four (four
    # channels per lane, or one)
    for T, D in ((5, 20), (7, 18), (300, 64)):
        h = rng.standard_normal((T, D))
        a, b, c, d = rng.standard_normal((2, T, D)), rng.standard_normal((T, D)), rng.standard_normal((1, T, D)), rng.standard_normal((T, D))
        ca, cb = rng.standard_normal(D), rng.standard_normal(D)
        rows = rng.standard_normal((T, 3))
        hd, rows_dev = f32(h), f32(rows)
        b16 = f32(b).bfloat16()
        ops.scaled_add(hd, [(f32(a), f32(ca), None), (b16, f32(cb), rows_dev[:, 2]), (f32(c), None, None), (f32(d), None, rows_dev[:, 0])])
        want = h + ca * a.sum(0) + cb * rows[:, 2:3] * b16.double().cpu().numpy() + c[0] + rows[:, 0:1] * d
        assert np.abs(hd.double().cpu().numpy() - want).max() < 1e-5, (T, D)


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

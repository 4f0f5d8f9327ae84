"""The Kugadra design (layer-list family: norms in front of and behind every sublayer, lightning layers, latent attention with a query
latent, a shared rotated key part and caches that a later layer may read, relu^2 feed-forward, mixture of experts with a softmax
router) on the GPU against the plain float64 restatement in tests/kugadra_ref.py.

Every test makes its own small configuration and random bfloat16-representable weights, writes them as a model folder and loads that
through the product's loader.  float32 plans are held to 2e-4 (root mean square of the logit difference over the root mean square of
the logits), bfloat16 plans to 6e-2.  Where random weights would hide a fault, the first latent layer is turned into a look-up: the
query latent repeats the key latent and the unrotated query entries are a multiple of the unrotated key entries, so that a token
attends to the earlier occurrences of the same token wherever they are; hiding one key, or moving the causal edge by one, then moves
the logits by far more than the bound, and the tests check that on the restatement itself.
"""
import copy
import json
import os
import subprocess

import numpy as np
import pytest

import __graft_entry__ as ge
import kugadra_ref as R

pytestmark = pytest.mark.gpu
F32_TOL, BF16_TOL = 2e-4, 6e-2


@pytest.fixture(scope="module")
def hy():
    from importlib import import_module
    ge.load_package()
    return import_module(ge.PKG_NAME + ".hybrid")


def dense(ff=56):
    return {"kind": "dense", "ff": ff} if ff else None


def moe(experts=6, top=2, ff=24, shared=40, scale=1.7):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}, "shared": {"ff": shared} if shared else None}


def lig(heads=3, dim=16, vdim=24, decay=None, mlp="dense"):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay or [1.0 - 2.0 ** -(2 + i) for i in range(heads)]},
            "mlp": dense() if mlp == "dense" else mlp}


def lat(heads=3, dim=12, rot_dim=8, vdim=20, kv_rank=28, q_rank=36, scale=0.3, base=10000.0, scaling="yarn", kv_from=None, mlp="dense"):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale}
    if rot_dim:
        m["rot"] = {"base": base, "dims": rot_dim}
        if scaling == "yarn":
            m["rot"]["scaling"] = {"factor": 3.0, "original": 48, "fast": 8.0, "slow": 1.0}
        elif scaling:
            m["rot"]["scaling"] = scaling
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": dense() if mlp == "dense" else mlp}


def config(layers, width=88, vocab=131, emb_scale=2.5, eps=1e-5, cap=11.0):
    c = {"architecture": "Kugadra", "vocab": vocab, "width": width, "embedding": {"scale": emb_scale}, "norm": {"eps": eps}, "layers": layers}
    if cap:
        c["logit_softcap"] = cap
    return c


class Model:
    def __init__(self, hy, tmp_path, cfg, seed, tweak=None):
        self.cfg, self.w = cfg, R.random_weights(cfg, seed)
        if tweak:
            tweak(cfg, self.w)
            self.w = {k: R.bf16_round(v) for k, v in self.w.items()}
        self.dir = str(tmp_path / ("m%d" % seed))
        hy.save_model_dir(self.dir, cfg, self.w)
        self.w64 = R.to_f64(self.w)
        self.hy = hy

    def plan(self, dtype="float32", **kw):
        return self.hy.HybridPlan.from_dir(self.dir, dtype=dtype, **kw)

    def ref(self, tokens, **kw):
        return R.forward(self.cfg, self.w64, tokens, **kw)

    def tokens(self, n, seed=0, vocab=None):
        toks = np.random.default_rng(1000 + seed).integers(0, vocab or self.cfg["vocab"], n).astype(np.int32)
        return toks, self.ref(toks)


def err_rows(got, want):
    d = got - want
    d = d - d.mean(axis=-1, keepdims=True)
    w = want - want.mean(axis=-1, keepdims=True)
    return np.sqrt((d ** 2).mean(axis=-1)) / np.sqrt((w ** 2).mean())


def err(got, want):
    return float(err_rows(got, want).max())


def whole(plan, toks, want=None):
    want = list(range(len(toks))) if want is None else want
    s = plan.acquire()
    out = plan.step(s, toks, 0, want)
    plan.release(s)
    return out


def stepwise(plan, toks, sizes):
    """The sequence in steps of the given sizes (the last size repeats), all logits."""
    s = plan.acquire()
    rows, p, i = [], 0, 0
    while p < len(toks):
        c = min(sizes[min(i, len(sizes) - 1)], len(toks) - p)
        rows.append(plan.step(s, toks[p:p + c], p, list(range(c))))
        p += c
        i += 1
    plan.release(s)
    return np.concatenate(rows)


# ---- each mechanism alone: one or two layers, the mechanism's sizes and constants varied ---------------------------------------------
SINGLE = [
    ("lightning_plain", [lig()], {}),
    ("lightning_no_feed_forward", [lig(mlp=None)], {}),
    ("lightning_one_head_wide", [lig(heads=1, dim=72, vdim=130)], {}),
    ("lightning_many_small_heads", [lig(heads=11, dim=4, vdim=6)], {}),
    ("lightning_one_state_row", [lig(heads=2, dim=1, vdim=3)], {}),
    ("lightning_never_forgets_or_at_once", [lig(heads=3, decay=[1.0, 0.0, 0.5])], {}),
    ("latent_plain", [lat()], {}),
    ("latent_no_feed_forward", [lat(mlp=None)], {}),
    ("latent_one_head", [lat(heads=1, dim=40, rot_dim=24, vdim=56, kv_rank=64, q_rank=16)], {}),
    ("latent_many_heads", [lat(heads=12, dim=6, rot_dim=2, vdim=5, kv_rank=10, q_rank=70)], {}),
    ("latent_no_rotated_part", [lat(rot_dim=0)], {}),
    ("latent_all_rotated_small_base", [lat(dim=2, rot_dim=30, base=3.0, scaling=None)], {}),
    ("latent_plain_frequencies", [lat(scaling=None)], {}),
    ("latent_ramp_inside_the_pairs", [lat(rot_dim=32, base=40.0, scaling={"factor": 8.0, "original": 64, "fast": 4.0, "slow": 0.5})], {}),
    ("latent_narrow_ramp", [lat(rot_dim=8, base=5.0, scaling={"factor": 2.0, "original": 20, "fast": 1.5, "slow": 1.4})], {}),
    ("latent_ramp_behind_its_end", [lat(rot_dim=8, base=16.0, scaling={"factor": 2.0, "original": 100, "fast": 0.1, "slow": 8.0})], {}),
    ("latent_wide_rows", [lat(heads=2, dim=64, rot_dim=64, vdim=96, kv_rank=320, q_rank=200)], {"n": 80}),
    ("latent_rows_longer_than_the_direct_form", [lat(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=520, q_rank=24, mlp=None)], {"n": 40}),
    ("shared_cache", [lat(), lat(heads=5, dim=8, vdim=12, q_rank=20, scale=0.5, kv_from=0)], {}),
    ("shared_cache_twice_and_apart", [lat(mlp=None), lig(mlp=None), lat(heads=2, kv_from=0, mlp=None), lat(heads=4, dim=20, kv_from=0)], {}),
    ("dense_feed_forward_odd_width", [lig(mlp=dense(33))], {}),
    ("experts_plain", [lig(mlp=moe())], {}),
    ("experts_without_shared", [lat(mlp=moe(shared=0))], {}),
    ("experts_top_1_scale_1", [lig(mlp=moe(experts=5, top=1, scale=1.0))], {}),
    ("experts_all_chosen", [lig(mlp=moe(experts=4, top=4))], {}),
    ("experts_one", [lig(mlp=moe(experts=1, top=1))], {}),
    ("experts_many", [lat(mlp=moe(experts=70, top=7, ff=8, shared=8))], {}),
    ("no_cap_no_embedding_scale", [lig(), lat()], {"cap": None, "emb_scale": 1.0}),
    ("tight_cap", [lat()], {"cap": 0.8}),
    ("widths_not_multiples_of_four", [lig(heads=3, dim=10, vdim=9, mlp=dense(17)), lat(heads=3, dim=9, rot_dim=6, vdim=11, kv_rank=21, q_rank=13, mlp=moe(ff=9, shared=13))],
     {"width": 75, "vocab": 53}),
    ("wide_model", [lig(heads=2, dim=32, vdim=32, mlp=dense(96)), lat(heads=2, dim=32, rot_dim=32, vdim=32, kv_rank=64, q_rank=96, mlp=moe(ff=64, shared=2048))],
     {"width": 1024, "vocab": 64, "n": 40}),
]


@pytest.mark.parametrize("name,layers,kw", SINGLE, ids=[s[0] for s in SINGLE])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_single_mechanism(hy, tmp_path, name, layers, kw, dtype):
    kw = dict(kw)
    n = kw.pop("n", 75)
    m = Model(hy, tmp_path, config(copy.deepcopy(layers), **kw), seed=len(name))
    toks, ref = m.tokens(n)
    plan = m.plan(dtype, ctx=max(128, n))
    got = whole(plan, toks)
    dec = stepwise(plan, toks[:12], [1])
    plan.close()
    tol = F32_TOL if dtype == "float32" else BF16_TOL
    assert err(got, ref) < tol
    assert err(dec, ref[:12]) < tol


MIXED = [lig(heads=2, dim=24, vdim=16, mlp=None), lat(mlp=moe()),
         lat(heads=6, dim=16, rot_dim=8, vdim=32, kv_rank=28, q_rank=44, scale=0.4, kv_from=1, mlp=dense(24)),
         lig(heads=4, dim=12, vdim=20, mlp=moe(experts=9, top=3, ff=16, shared=0, scale=0.7)),
         lat(heads=2, dim=40, rot_dim=16, vdim=24, kv_rank=48, q_rank=20, base=50.0, scaling=None, mlp=None)]


def test_layer_taps(hy, tmp_path):
    """The residual that leaves every layer against the restatement, layer by layer."""
    m = Model(hy, tmp_path, config(copy.deepcopy(MIXED), width=96), seed=41)
    toks, ref = m.tokens(90)
    plan = m.plan("float32", ctx=96, layer_taps=True)
    taps = []
    m.ref(toks, taps=taps)
    got = whole(plan, toks)
    for l, t in enumerate(taps):
        rows = plan.layer_rows(l, len(toks))
        assert np.abs(rows - t).max() < 1e-4 * max(1.0, np.abs(t).max()), l
    plan.close()
    assert err(got, ref) < F32_TOL


def random_config(seed):
    """Layer order, every size and every constant drawn at random (sizes that are no multiples of anything included)."""
    rng = np.random.default_rng(seed)
    pick = lambda *xs: xs[int(rng.integers(len(xs)))]

    def mlp():
        kind = pick("none", "dense", "moe", "moe")
        if kind == "none":
            return None
        if kind == "dense":
            return dense(int(rng.integers(8, 90)))
        E = int(rng.integers(1, 20))
        return moe(experts=E, top=int(rng.integers(1, E + 1)), ff=int(rng.integers(4, 40)), shared=pick(0, int(rng.integers(4, 60))), scale=float(rng.uniform(0.5, 3.0)))

    layers, caches = [], []
    for i in range(int(rng.integers(2, 7))):
        if rng.random() < 0.45:
            H = int(rng.integers(1, 7))
            layers.append(lig(heads=H, dim=int(rng.integers(2, 40)), vdim=int(rng.integers(2, 50)), decay=[float(1.0 - 2.0 ** -rng.uniform(1.0, 10.0)) for _ in range(H)], mlp=mlp()))
        else:
            src = pick(None, *caches) if caches else None
            R_, P = (layers[src]["mixer"]["kv_rank"], layers[src]["mixer"]["rot_dim"]) if src is not None else (int(rng.integers(4, 70)), 2 * int(rng.integers(0, 17)))
            sc = pick(None, "yarn", {"factor": float(rng.uniform(1.5, 16.0)), "original": int(rng.integers(16, 400)), "fast": float(rng.uniform(4.0, 40.0)), "slow": float(rng.uniform(0.3, 2.0))})
            lay = lat(heads=int(rng.integers(1, 8)), dim=int(rng.integers(2, 36)), rot_dim=P, vdim=int(rng.integers(3, 50)), kv_rank=R_, q_rank=int(rng.integers(4, 80)),
                      scale=float(rng.uniform(0.1, 0.6)), base=float(rng.uniform(5.0, 1e6)), scaling=sc, kv_from=src, mlp=mlp())
            if src is None:
                caches.append(i)
            elif P:
                lay["mixer"]["rot"] = copy.deepcopy(layers[src]["mixer"]["rot"])
            layers.append(lay)
    return config(layers, width=int(rng.integers(20, 140)), vocab=int(rng.integers(30, 300)), emb_scale=float(rng.uniform(0.5, 20.0)), eps=float(10.0 ** -rng.uniform(4, 7)),
                  cap=pick(None, float(rng.uniform(2.0, 40.0))))


@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(hy, tmp_path, seed):
    m = Model(hy, tmp_path, random_config(seed), seed=100 + seed)
    n = 140
    toks, ref = m.tokens(n, seed=seed)
    # float32 holds every position to the bound.  bfloat16: with random routers the choice scores of the last chosen and the first
    # unchosen expert lie within the rounding of the router's bfloat16 input for one token in ten or so (measured on these
    # configurations: median gap 0.008 at scores around 1 / experts), and a token whose expert flips leaves the restatement by far more
    # than rounding.  The bfloat16 plan is therefore held to the restatement with its products' inputs rounded alike (which makes the
    # same choices); against the unrounded one the median row is held to the bound
    refb = m.ref(toks, round_inputs=True)
    for dtype in ("float32", "bfloat16"):
        plan = m.plan(dtype, ctx=n + 4, max_batch=48)
        for got in (whole(plan, toks), stepwise(plan, toks, [50, 2, 1, 31, 7, 1])):
            if dtype == "float32":
                assert err(got, ref) < F32_TOL
            else:
                assert np.quantile(err_rows(got, refb), 0.95) < BF16_TOL / 3 and np.median(err_rows(got, ref)) < BF16_TOL
        plan.close()


# ---- prompts cut into portions, decoding token by token ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_equals_token_by_token_and_portions(hy, tmp_path, dtype):
    m = Model(hy, tmp_path, config(copy.deepcopy(MIXED)), seed=7)
    n = 150
    toks, ref = m.tokens(n)
    if dtype == "float32":
        ok = lambda got: err(got, ref) < F32_TOL
    else:
        # held to the restatement with its products' inputs rounded alike (it chooses the same experts as the plan but for a token whose
        # choice scores tie to the last bits; such a token, and those after it, leave by more than rounding): nine rows in ten
        refb = m.ref(toks, round_inputs=True)
        ok = lambda got: np.quantile(err_rows(got, refb), 0.9) < BF16_TOL / 3 and np.median(err_rows(got, ref)) < BF16_TOL
    plan = m.plan(dtype, ctx=160, max_batch=64)              # the whole prompt runs as portions of 64 inside one step, too
    assert ok(whole(plan, toks))
    assert ok(stepwise(plan, toks, [1]))
    for sizes in ([2, 3, 2, 64, 5, 1, 1, 37, 2, 33], [70, 2, 2, 2, 74], [1, 149], [9, 2], [8, 9, 8]):
        assert ok(stepwise(plan, toks, sizes)), sizes
    plan.close()


def test_logits_do_not_depend_on_the_cut(hy, tmp_path):
    """float32: the same position through different cuts agrees to rounding."""
    m = Model(hy, tmp_path, config(copy.deepcopy(MIXED)), seed=8)
    toks, _ = m.tokens(90)
    plan = m.plan("float32", ctx=128)
    a = whole(plan, toks)
    b = stepwise(plan, toks, [41, 2, 47])
    c = stepwise(plan, toks, [1])
    plan.close()
    assert err(b, a) < 2e-5 and err(c, a) < 2e-5


# ---- slots -------------------------------------------------------------------------------------------------------------------------------
def test_interleaved_requests_and_slot_reuse(hy, tmp_path):
    """Unequal requests whose steps alternate give what each gives alone; a slot that a long request left (latent rows, also those a
    later layer reads, and memory states) is clean for the next."""
    m = Model(hy, tmp_path, config(copy.deepcopy(MIXED)), seed=9)
    (ta, ra), (tb, rb), (tc, rc) = m.tokens(60, 1), m.tokens(45, 2), m.tokens(30, 3)
    plan = m.plan("float32", ctx=64, n_seqs=2)
    a, b = plan.acquire(), plan.acquire()
    assert a != b
    with pytest.raises(hy.hip.Gl3Error):
        plan.acquire()                                   # both slots are taken
    ga, gb = [], []
    ga.append(plan.step(a, ta[:20], 0, list(range(20))))
    gb.append(plan.step(b, tb[:7], 0, list(range(7))))
    ga.append(plan.step(a, ta[20:21], 20, [0]))
    gb.append(plan.step(b, tb[7:40], 7, list(range(33))))
    ga.append(plan.step(a, ta[21:], 21, list(range(39))))
    for i in range(40, 45):
        gb.append(plan.step(b, tb[i:i + 1], i, [0]))
    assert err(np.concatenate(ga), ra) < F32_TOL and err(np.concatenate(gb), rb) < F32_TOL
    plan.release(a)
    c = plan.acquire()
    assert c == a
    gc = [plan.step(c, tc[:1], 0, [0]), plan.step(c, tc[1:3], 1, [0, 1]), plan.step(c, tc[3:], 3, list(range(27)))]
    assert err(np.concatenate(gc), rc) < F32_TOL
    with pytest.raises(hy.hip.Gl3Error):
        plan.step(c, tc[:2], 7, [])                      # neither a continuation nor a restart
    assert err(plan.step(b, tc, 0, list(range(30))), rc) < F32_TOL          # a restart at position 0 on a live slot starts clean as well
    plan.close()


def test_decode_batch_over_slots(hy, tmp_path):
    m = Model(hy, tmp_path, config(copy.deepcopy(MIXED[:3])), seed=10)
    (ta, ra), (tb, rb) = m.tokens(12, 4), m.tokens(9, 5)
    plan = m.plan("float32", ctx=32, n_seqs=2)
    a, b = plan.acquire(), plan.acquire()
    plan.step(a, ta[:11], 0, [])
    plan.step(b, tb[:8], 0, [])
    logits, ids = plan.forward_decode_batch([ta[11], tb[8]], [a, b], [11, 8])
    plan.close()
    assert err(logits, np.stack([ra[11], rb[8]])) < F32_TOL and list(ids) == list(np.argmax(logits, axis=1))


# ---- far keys, the causal edge, key tiles: a token looks for its own earlier occurrences -------------------------------------------------
def lookup_latent(cfg, w, copy_score=8.0):
    """Layer 0 (a latent attention whose q_rank equals its kv_rank) becomes a look-up: the query latent repeats the key latent (same down
    projection, same norm weight), the unrotated query entries are a multiple of the unrotated key entries and the rotated ones are
    zero, so the score of a key depends on the two tokens only and a token finds every earlier copy of itself about `copy_score` above
    the other keys.  The embedding's share of the residual is made small, so that what the attention gathers decides the logits."""
    mx = cfg["layers"][0]["mixer"]
    H, D, P, R = mx["heads"], mx["dim"], mx.get("rot_dim", 0), mx["kv_rank"]
    assert cfg["layers"][0]["type"] == "latent_attention" and mx["q_rank"] == R
    w["l0.mix.dq"] = w["l0.mix.dkv"][:R].copy()
    w["l0.mix.dq.norm"] = w["l0.mix.dkv.norm"].copy()
    uk = w["l0.mix.uk"].reshape(H, D, R)
    uq = np.zeros((H, D + P, R), np.float32)
    # |W_uk c|^2 is about D for a normed latent: the copy's score is scale * mult * D
    uq[:, :D] = uk * (copy_score / (mx["scale"] * D))
    w["l0.mix.uq"] = uq.reshape(H * (D + P), R)
    w["l0.mix.g"] = np.zeros_like(w["l0.mix.g"])
    w["l0.norm1b"] = np.full_like(w["l0.norm1b"], 4.0)


def lookup_model(hy, tmp_path, seed, extra=()):
    layers = [lat(heads=4, dim=16, rot_dim=8, vdim=24, kv_rank=32, q_rank=32, scale=0.5, mlp=None)] + list(extra)
    return Model(hy, tmp_path, config(layers, width=64, vocab=97, emb_scale=1.0), seed=seed, tweak=lookup_latent)


@pytest.mark.parametrize("n,decode_from", [(150, 120), (200, 190), (330, 300), (129, 60), (530, 505)])
def test_causal_edge_and_key_tiles(hy, tmp_path, n, decode_from):
    """A small vocabulary and a look-up layer: every query has earlier copies of its token at all distances, in every key tile (tiles are
    64 keys wide; decode steps split the keys over workgroups by tile), in the prompt and while decoding.  The restatement with the
    causal edge moved by one (a query that also sees the next key) differs by more than 10 times the bound: a kernel that is off by
    one at the edge cannot pass."""
    m = lookup_model(hy, tmp_path, n, extra=[lat(heads=2, dim=12, rot_dim=8, vdim=16, kv_rank=32, q_rank=20, kv_from=0, mlp=dense(16))])
    toks, ref = m.tokens(n, vocab=23)
    assert err(m.ref(toks, causal_shift=1), ref) > 10 * F32_TOL
    plan = m.plan("float32", ctx=n + 8, max_batch=96)
    assert err(whole(plan, toks), ref) < F32_TOL
    s = plan.acquire()
    got = [plan.step(s, toks[:decode_from], 0, list(range(decode_from)))]
    got += [plan.step(s, toks[i:i + 1], i, [0]) for i in range(decode_from, n)]
    plan.release(s)
    assert err(np.concatenate(got), ref) < F32_TOL
    assert err(stepwise(plan, toks, [61, 2, 3, 64, 2, 67]), ref) < F32_TOL
    plan.close()


@pytest.mark.parametrize("far", [0, 3, 63, 64, 127, 128, 191])
def test_one_far_key_among_hundreds(hy, tmp_path, far):
    """One token stands at position `far` and again at the very end, nowhere else: the last query's look-up finds that one key among
    hundreds (at a tile's first or last row, in the first tile or a later one).  Hiding the key in the restatement moves the last logits
    by far more than the bound; the plan follows with the prompt whole, in portions, and with the last tokens decoded (the keys are
    then split over workgroups)."""
    m = lookup_model(hy, tmp_path, 300 + far, extra=[lig(heads=2, dim=8, vdim=8, mlp=None)])
    n = 450
    toks = np.random.default_rng(far).integers(1, 97, n).astype(np.int32)
    toks[far] = toks[n - 1] = 0
    ref = m.ref(toks)
    assert err(m.ref(toks, drop_keys=[far])[-1:], ref[-1:]) > 20 * F32_TOL
    for dtype, tol in (("float32", F32_TOL), ("bfloat16", BF16_TOL)):
        plan = m.plan(dtype, ctx=n, max_batch=200)
        assert err(whole(plan, toks, [n - 1]), ref[-1:]) < tol
        s = plan.acquire()
        plan.step(s, toks[:n - 5], 0, [])
        got = np.concatenate([plan.step(s, toks[i:i + 1], i, [0]) for i in range(n - 5, n)])
        plan.release(s)
        assert err(got, ref[n - 5:]) < tol
        assert err(stepwise(plan, toks, [190, 2, 130, 127, 1])[-1:], ref[-1:]) < tol
        plan.close()


def test_far_tokens_reach_the_memories(hy, tmp_path):
    """The first tokens of a long prompt decide the last logits only through the lightning layers' states (the attention's output
    projection is zero): swapping two early tokens moves the restatement's last logits by far more than the bound, and the plan
    follows, whole and decoded."""
    layers = [lig(heads=2, dim=16, vdim=16, decay=[1.0, 0.999], mlp=None), lat(mlp=None), lig(heads=3, dim=8, vdim=12, decay=[0.9995, 0.5, 0.99], mlp=dense(24))]

    def tweak(cfg, w):
        w["l1.mix.o"] = np.zeros_like(w["l1.mix.o"])

    m = Model(hy, tmp_path, config(layers, width=48, vocab=61), seed=77, tweak=tweak)
    n = 700
    toks, ref = m.tokens(n)
    other = toks.copy()
    other[3], other[4] = (toks[3] + 1) % 61, (toks[4] + 7) % 61
    assert err(m.ref(other)[-1:], ref[-1:]) > 20 * F32_TOL
    plan = m.plan("float32", ctx=n, max_batch=256)
    assert err(whole(plan, toks, [n - 1]), ref[-1:]) < F32_TOL
    s = plan.acquire()
    plan.step(s, toks[:n - 40], 0, [])
    got = np.concatenate([plan.step(s, toks[i:i + 1], i, [0]) for i in range(n - 40, n)])
    plan.release(s)
    plan.close()
    assert err(got, ref[n - 40:]) < F32_TOL


def test_first_tokens(hy, tmp_path):
    """Positions 0 .. 4 and a one-token sequence (through the decode kernels)."""
    m = lookup_model(hy, tmp_path, 21, extra=[lig(heads=2, dim=8, vdim=8, mlp=moe(experts=3, top=2, ff=8, shared=8)), lat(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=32, kv_from=0)])
    toks, ref = m.tokens(5, vocab=2)
    plan = m.plan("float32", ctx=8)
    assert err(whole(plan, toks), ref) < F32_TOL
    assert err(whole(plan, toks[:1]), ref[:1]) < F32_TOL
    assert err(stepwise(plan, toks, [1]), ref) < F32_TOL
    assert err(stepwise(plan, toks, [2]), ref) < F32_TOL
    plan.close()


def test_long_decoding(hy, tmp_path):
    layers = [lat(heads=2, dim=16, rot_dim=16, vdim=16, kv_rank=24, q_rank=16, mlp=dense(16)), lig(heads=2, dim=16, vdim=16, decay=[0.999, 0.96], mlp=moe(experts=4, top=2, ff=8, shared=0)),
              lat(heads=3, dim=8, rot_dim=16, vdim=8, kv_rank=24, q_rank=12, kv_from=0, mlp=None)]
    m = Model(hy, tmp_path, config(layers, width=48, vocab=61), seed=33)
    n = 420
    toks, ref = m.tokens(n)
    for dtype, tol in (("float32", F32_TOL), ("bfloat16", BF16_TOL)):
        plan = m.plan(dtype, ctx=n)
        s = plan.acquire()
        plan.step(s, toks[:3], 0, [])
        got = np.concatenate([plan.step(s, toks[i:i + 1], i, [0]) for i in range(3, n)])
        plan.release(s)
        plan.close()
        assert err(got, ref[3:]) < tol, dtype


def test_rotation_is_by_position_not_by_place_in_the_step(hy, tmp_path):
    """The rotated parts turn by the token's position in the sequence: with a small base and no scaling the turns are large, and a
    portion that starts late must turn by its true positions."""
    m = Model(hy, tmp_path, config([lat(dim=4, rot_dim=24, base=3.0, scaling=None, scale=1.0), lat(dim=4, rot_dim=24, base=3.0, scaling=None, scale=1.0, kv_from=0)]), seed=61)
    toks, ref = m.tokens(70)
    plan = m.plan("float32", ctx=80)
    assert err(stepwise(plan, toks, [33, 2, 1, 20, 14]), ref) < F32_TOL
    plan.close()


def test_router_choice_follows_the_correction(hy, tmp_path):
    """Corrections far larger than any score difference fix the choice (the experts with the largest corrections) whatever the scores,
    while the weights stay the scores': the restatement agrees with itself run on the chosen experts alone, and the plan with it."""
    layers = [lig(mlp=moe(experts=8, top=3, ff=16, shared=0))]

    def tweak(cfg, w):
        w["l0.mlp.correction"] = np.array([0.0, 5.0, 0.0, 7.0, 0.0, 0.0, 6.0, 0.0], np.float32)

    m = Model(hy, tmp_path, config(layers), seed=88, tweak=tweak)
    toks, ref = m.tokens(40)
    h = np.random.default_rng(0).standard_normal((9, 88))
    choice, wts = R.route(h, R.sub(m.w64, "l0.mlp."), m.cfg["layers"][0]["mlp"])
    assert (choice == np.array([3, 6, 1])).all() and np.allclose(wts.sum(axis=1), 1.7)
    plan = m.plan("float32", ctx=64)
    assert err(whole(plan, toks), ref) < F32_TOL
    assert err(stepwise(plan, toks, [1]), ref) < F32_TOL
    plan.close()


# ---- the framework's own entry points ----------------------------------------------------------------------------------------------------
def check_greedy(m, prompt, ids):
    """Every generated id is the reference's arg max given the ids before it (ties within 1e-4 of the maximum are allowed)."""
    full = list(prompt) + list(ids)
    ref = m.ref(np.array(full[:-1], np.int32))
    for i, t in enumerate(ids):
        row = ref[len(prompt) - 1 + i]
        assert row[t] >= row.max() - 1e-4 * max(1.0, abs(row.max())), i


def test_greedy_generation_python_entry(hy, tmp_path):
    m = Model(hy, tmp_path, config(copy.deepcopy(MIXED)), seed=51)
    prompt, _ = m.tokens(37)
    plan = m.plan("float32", ctx=64, max_batch=16)
    ids = plan.generate(prompt, 20)
    check_greedy(m, prompt, ids)
    plan.prefill(prompt[:-1], 0)
    lg = plan.forward_decode(int(prompt[-1]), len(prompt) - 1)
    assert int(np.argmax(lg)) == ids[0]
    plan.prefill(prompt[:-1], 0)
    t = plan.forward_decode_sample(int(prompt[-1]), len(prompt) - 1, 0.7, 0.9, 0.3)
    assert 0 <= t < m.cfg["vocab"]
    plan.close()


def test_greedy_generation_command_line(hy, tmp_path):
    m = Model(hy, tmp_path, config(copy.deepcopy(MIXED)), seed=52)
    prompt, _ = m.tokens(21)
    exe = os.path.join(ge.ROOT, "tools", "gl3_run")
    out = subprocess.run([exe, "-m", m.dir, "--ids", ",".join(map(str, prompt)), "-n", "40", "-b", "8", "--f32"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    ids = [int(x) for x in out.stdout.split("generated:")[1].split()]
    assert len(ids) == 40 - len(prompt) + 1
    check_greedy(m, prompt, ids)


def test_trace_replay_tool(hy, tmp_path):
    m = Model(hy, tmp_path, config(copy.deepcopy(MIXED[:3])), seed=53)
    toks, ref = m.tokens(50)
    outdir = tmp_path / "out"
    outdir.mkdir()
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:30].tolist(), "want": [3, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[30:32].tolist(), "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": toks[32:].tolist(), "want": [17]}], "end": ["x"]},
             {"step": 3, "entries": [{"id": "y", "tokens": toks[:5].tolist(), "want": [4]}], "end": ["y"]}]
    for dtype, tol in (("float32", F32_TOL), ("bfloat16", BF16_TOL)):
        p = subprocess.run([os.path.join(ge.ROOT, "bin", "trace_run"), "--model", m.dir, "--dtype", dtype, "--out", str(outdir), "--max-tokens", "64"],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr
        assert [l for l in p.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
        assert not (outdir / "1.f32").exists()
        got = np.concatenate([np.fromfile(outdir / ("%d.f32" % i), np.float32).reshape(-1, m.cfg["vocab"]) for i in (0, 2, 3)])
        assert err(got, ref[[3, 29, 49, 4]]) < tol


def test_loader_refuses_what_it_cannot_run(hy, tmp_path):
    m = Model(hy, tmp_path, config([lat(mlp=moe()), lig(), lat(kv_from=0, mlp=None)]), seed=54)
    for name in ("l0.mix.dq.norm", "l0.mix.uq", "l0.mix.dkv", "l0.norm1b", "l0.norm2b", "l0.mlp.correction", "l0.mlp.e3.up", "l0.mlp.shared.gate", "l1.mix.norm", "l1.mix.g",
                 "l1.mlp.up", "l2.mix.uk", "l2.mix.dq", "final.norm"):
        w = dict(m.w)
        del w[name]
        hy.save_model_dir(str(tmp_path / "bad"), m.cfg, w)
        with pytest.raises(hy.hip.Gl3Error):
            hy.HybridPlan.from_dir(str(tmp_path / "bad"))
    w = dict(m.w)
    w["l0.mlp.correction"] = np.concatenate([w["l0.mlp.correction"], w["l0.mlp.correction"]])
    hy.save_model_dir(str(tmp_path / "bad"), m.cfg, w)
    with pytest.raises(hy.hip.Gl3Error):
        hy.HybridPlan.from_dir(str(tmp_path / "bad"))
    for layer, path, value in ((0, ("rot", "dims"), 6), (1, ("decay",), [0.5]), (2, ("kv_from",), 1), (2, ("kv_from",), 2), (2, ("kv_rank",), 30), (0, ("rot_dim",), 7)):
        bad = copy.deepcopy(m.cfg)
        node = bad["layers"][layer]["mixer"]
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        hy.save_model_dir(str(tmp_path / "bad"), bad, m.w)
        with pytest.raises(hy.hip.Gl3Error):
            hy.HybridPlan.from_dir(str(tmp_path / "bad"))

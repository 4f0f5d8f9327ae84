"""Host-side tests of the Kugadra design that need no GPU: hand-derived values of the plain restatement (tests/kugadra_ref.py), one per
mechanism, and the native loader's refusals that come before any device call."""
import math

import numpy as np
import pytest

import __graft_entry__ as ge
import kugadra_ref as R


@pytest.fixture(scope="module")
def hy():
    from importlib import import_module
    ge.load_package()
    return import_module(ge.PKG_NAME + ".hybrid")


def test_ref_blended_frequencies_by_hand():
    # 8 entries, 4 pairs, base 16: f = 1, 1/2, 1/4, 1/8.  p(t) = 8 ln(original / (2 pi t)) / (2 ln 16)
    rot = {"dims": 8, "base": 16.0, "scaling": {"factor": 4.0, "original": 100, "fast": 8.0, "slow": 1.0}}
    p = lambda t: 8 * math.log(100 / (2 * math.pi * t)) / (2 * math.log(16))
    lo, hi = max(math.floor(p(8.0)), 0), min(math.ceil(p(1.0)), 7)
    assert (lo, hi) == (0, 4)
    f, mul = R.yarn_frequencies(rot)
    ramp = np.array([0.0, 0.25, 0.5, 0.75])
    plain = np.array([1.0, 0.5, 0.25, 0.125])
    assert np.allclose(f, plain / 4.0 * ramp + plain * (1.0 - ramp))
    assert abs(mul - (0.1 * math.log(4.0) + 1.0)) < 1e-15
    f, mul = R.yarn_frequencies({"dims": 8, "base": 16.0})
    assert np.allclose(f, plain) and mul == 1.0
    # a ramp one pair wide (lo = 2, hi = 3): pairs from 3 on take the divided frequency, the others the plain one
    f, _ = R.yarn_frequencies({"dims": 8, "base": 16.0, "scaling": {"factor": 2.0, "original": 100, "fast": 3.0, "slow": 2.9}})
    assert np.allclose(f, plain * np.array([1.0, 1.0, 1.0, 0.5]))
    # a ramp that starts behind its end (lo = 7 > hi = 1): its width counts as 0.001 and no pair lies on or behind it
    f, _ = R.yarn_frequencies({"dims": 8, "base": 16.0, "scaling": {"factor": 2.0, "original": 100, "fast": 0.1, "slow": 8.0}})
    assert np.allclose(f, plain)


def test_ref_turn_pairs_entry_i_with_i_plus_half():
    x = np.array([[[1.0, 2.0, 3.0, 4.0]]]).repeat(2, axis=0)
    rot = {"dims": 4, "base": 100.0, "scaling": {"factor": 2.0, "original": 10, "fast": 1e9, "slow": 1e-9}}          # lo = 0, hi = 3: ramp 0, 1/3
    mul = 0.1 * math.log(2.0) + 1.0
    a0, a1 = 5.0 * 1.0, 5.0 * (0.1 / 2.0 / 3.0 + 0.1 * 2.0 / 3.0)
    out = R.turn(x, np.array([0.0, 5.0]), rot)
    assert np.allclose(out[0], x[0] * mul)
    want = [1 * np.cos(a0) - 3 * np.sin(a0), 2 * np.cos(a1) - 4 * np.sin(a1), 3 * np.cos(a0) + 1 * np.sin(a0), 4 * np.cos(a1) + 2 * np.sin(a1)]
    assert np.allclose(out[1, 0], np.array(want) * mul)


def test_ref_lightning_is_a_decayed_sum_over_the_past():
    rng = np.random.default_rng(0)
    c = {"heads": 2, "dim": 4, "vdim": 3, "decay": [0.5, 0.9]}
    T, W = 6, 5
    h = rng.standard_normal((T, W))
    p = {n: rng.standard_normal(s) for n, s in (("q", (8, W)), ("k", (8, W)), ("v", (6, W)), ("g", (6, W)), ("o", (W, 6)), ("norm", (6,)))}
    act = lambda z: z / (1 + np.exp(-z))
    q, k, v = act(h @ p["q"].T).reshape(T, 2, 4), act(h @ p["k"].T).reshape(T, 2, 4), act(h @ p["v"].T).reshape(T, 2, 3)
    o = np.zeros((T, 2, 3))
    for t in range(T):
        for s in range(t + 1):
            for hd in range(2):
                o[t, hd] += c["decay"][hd] ** (t - s) * (q[t, hd] @ k[s, hd]) * v[s, hd]
    o = o.reshape(T, 6)
    o = o / np.sqrt((o ** 2).mean(axis=-1, keepdims=True) + 1e-3) * p["norm"]          # ONE norm over both heads
    want = (o / (1 + np.exp(-(h @ p["g"].T)))) @ p["o"].T
    assert np.allclose(R.lightning(h, p, c, 1e-3), want)


def test_ref_latent_attention_by_hand():
    # one head, one unrotated and no rotated entry, latents of one entry: every projection is a number
    c = {"heads": 1, "dim": 1, "rot_dim": 0, "vdim": 1, "kv_rank": 1, "q_rank": 1, "scale": 2.0}
    p = {"dq": np.array([[1.0]]), "dq.norm": np.array([3.0]), "uq": np.array([[0.5]]), "dkv": np.array([[1.0]]), "dkv.norm": np.array([2.0]),
         "uk": np.array([[1.0]]), "uv": np.array([[5.0]]), "g": np.array([[0.0]]), "o": np.array([[1.0]])}
    h = np.array([[1.0], [-2.0], [0.5]])
    # a normed latent of one entry is its sign times the weight: c = 2 sign(h), q = 0.5 * 3 sign(h), k = c, v = 5 c
    sg = np.sign(h[:, 0])
    q, k, v = 1.5 * sg, 2.0 * sg, 10.0 * sg
    want = []
    for i in range(3):
        s = np.array([2.0 * q[i] * k[j] for j in range(i + 1)])
        w = np.exp(s) / np.exp(s).sum()
        want.append(0.5 * (w * v[:i + 1]).sum())
    assert np.allclose(R.latent_attention(h, p, c, 0.0)[:, 0], want)
    # with a cache handed in the layer reads those rows instead of its own
    other = (np.array([[7.0], [7.0], [7.0]]), np.zeros((3, 0)))
    assert np.allclose(R.latent_attention(h, p, c, 0.0, cache=other)[:, 0], 0.5 * 35.0)


def test_ref_rotated_key_part_is_shared_and_unscaled():
    # two heads, no unrotated score (W_uk = 0): both heads score q_rot . k_rot with the same key part; the latent is normed, the rotated part is not
    c = {"heads": 2, "dim": 1, "rot_dim": 2, "vdim": 1, "kv_rank": 1, "q_rank": 2, "scale": 1.0, "rot": {"dims": 2, "base": 10.0}}
    p = {"dq": np.eye(2), "dq.norm": np.ones(2), "uq": np.array([[0, 0], [1.0, 0], [0, 1.0], [0, 0], [0, 2.0], [-2.0, 0]]), "dkv": np.array([[1.0, 0], [3.0, 0], [0, 3.0]]),
         "dkv.norm": np.ones(1), "uk": np.zeros((2, 1)), "uv": np.ones((2, 1)), "g": np.zeros((2, 2)), "o": np.eye(2)}
    h = np.array([[1.0, 1.0], [1.0, 1.0]])
    lat, kr = R.latent_cache(h, p, c, 0.0)
    assert np.allclose(lat, 1.0)
    a = 1.0                                                              # position 1, frequency 1
    assert np.allclose(kr[0], [3.0, 3.0]) and np.allclose(kr[1], [3 * np.cos(a) - 3 * np.sin(a), 3 * np.cos(a) + 3 * np.sin(a)])
    # a turn keeps dot products of vectors turned by the same angle: head 0's rotated query (1, 1) scores 6 against its own position's key, head 1's (2, -2) scores 0
    out = R.latent_attention(h, p, c, 0.0)
    assert np.allclose(out[0], 0.5)                                      # one key: the value, times the gate's half
    k0 = np.array([3.0, 3.0])
    q1 = [np.array([np.cos(a) - np.sin(a), np.cos(a) + np.sin(a)]), 2.0 * np.array([np.cos(a) + np.sin(a), np.cos(a) - np.sin(a)]) * np.array([1, -1])]
    for hd in range(2):
        s = np.array([q1[hd] @ k0, q1[hd] @ kr[1]])
        assert np.allclose(out[1, hd], 0.5 * 1.0)                         # both values are 1: any weights give 1
        assert np.isfinite(s).all()


def test_ref_router_by_hand():
    c = {"router": {"experts": 4, "top": 2, "scale": 3.0}}
    p = {"router": np.eye(4), "correction": np.array([0.0, 0.0, 0.5, 0.0])}
    z = np.array([[2.0, 1.0, 0.0, -1.0]])
    s = np.exp(z[0]) / np.exp(z[0]).sum()
    choice, w = R.route(z, p, c)
    # expert 2 is chosen for its correction (0.09 + 0.5), ahead of expert 0 (0.64); its weight is its score without the correction
    assert list(choice[0]) == [0, 2] or list(choice[0]) == [2, 0]
    order = list(choice[0])
    assert np.allclose(w[0], 3.0 * s[order] / (s[0] + s[2]))
    # a tie goes to the lower index
    choice, _ = R.route(np.zeros((1, 4)), dict(p, correction=np.zeros(4)), c)
    assert list(choice[0]) == [0, 1]


def test_ref_layer_has_norms_on_both_sides_and_a_capped_tied_head():
    """A lightning layer switched off by a zero output projection would divide zero by the root of eps: with eps > 0 its share is zero and
    the feed-forward alone moves x."""
    cfg = {"vocab": 3, "width": 2, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-6}, "logit_softcap": 1.5,
           "layers": [{"type": "lightning", "mixer": {"heads": 1, "dim": 1, "vdim": 1, "decay": [0.5]}, "mlp": {"kind": "dense", "ff": 1}}]}
    w = {"embed": np.array([[1.0, 0.5], [0.0, 1.0], [2.0, 2.0]]), "l0.norm1": np.array([1.0, 2.0]), "l0.norm1b": np.array([1.0, 1.0]), "l0.mix.q": np.ones((1, 2)),
         "l0.mix.k": np.ones((1, 2)), "l0.mix.v": np.ones((1, 2)), "l0.mix.g": np.ones((1, 2)), "l0.mix.o": np.zeros((2, 1)), "l0.mix.norm": np.ones(1),
         "l0.norm2": np.array([1.0, 3.0]), "l0.norm2b": np.array([0.5, 2.0]), "l0.mlp.up": np.array([[1.0, -1.0]]), "l0.mlp.down": np.array([[1.0], [-2.0]]),
         "final.norm": np.array([1.0, 1.0])}
    x0 = np.array([4.0, 4.0])                                            # token 2 times the embedding scale
    hn = x0 / np.sqrt(16.0 + 1e-6) * np.array([1.0, 3.0])
    up = hn[0] - hn[1]
    assert up < 0                                                        # relu: nothing passes; the feed-forward's output is zero and stays zero behind its norm
    assert np.allclose(R.forward(cfg, w, [2])[0], 1.5 * np.tanh(w["embed"] @ (x0 / np.sqrt(16.0 + 1e-6)) / 1.5))
    w["l0.mlp.up"] = np.array([[-1.0, 1.0]])
    y = (hn[1] - hn[0]) ** 2 * np.array([1.0, -2.0])
    x = x0 + y / np.sqrt((y ** 2).mean() + 1e-6) * np.array([0.5, 2.0])
    xn = x / np.sqrt((x ** 2).mean() + 1e-6)
    assert np.allclose(R.forward(cfg, w, [2])[0], 1.5 * np.tanh(w["embed"] @ xn / 1.5))


def test_native_loader_refuses_before_touching_a_device(hy, tmp_path):
    L = hy.hip.lib()
    base = '{"architecture": "Kugadra", "vocab": 8, "width": 8, "norm": {"eps": 1e-6}, "layers": [%s]}'
    la = '{"type": "latent_attention", "mixer": {"heads": 2, "dim": 4, "rot_dim": 2, "vdim": 4, "kv_rank": 4, "q_rank": 4, "scale": 1.0%s}%s}'
    rot = ', "rot": {"base": 10.0, "dims": 2}'
    for i, text in enumerate(['{"architecture": "Kugadra", "vocab": 8}', base % '{"type": "conv", "mixer": {"heads": 1, "dim": 1, "vdim": 1}}', base % '{"type": "lightning"}',
                              base % '{"type": "lightning", "mixer": {"heads": 2, "dim": 4, "vdim": 4, "decay": [0.5]}}',
                              base % (la % ("", "")),                                                    # a rotated part without rot
                              base % (la % (', "rot": {"base": 10.0, "dims": 4}', "")),               # rot.dims differs from rot_dim
                              base % (la % (rot + ', "kv_from": 0', "")),                               # no earlier layer to read from
                              base % (la % (rot, ', "mlp": {"kind": "glu", "ff": 4}')),
                              base % (la % (rot, ', "mlp": {"kind": "moe", "expert": {"ff": 4}}'))]):
        d = tmp_path / ("c%d" % i)
        d.mkdir()
        (d / "config.json").write_text(text)
        assert L.gl3_is_model_dir(str(d).encode()) == 1
        with pytest.raises(hy.hip.Gl3Error) as e:
            hy.HybridPlan.from_dir(str(d))
        assert e.value.code in (hy.hip.E_ARG, hy.hip.E_UNSUPPORTED) and len(str(e.value)) > 20

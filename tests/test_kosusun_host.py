"""Host-side tests of the Kosusun design that need no GPU: hand-derived values of the plain restatement (tests/kosusun_ref.py), one per
mechanism, and the native loader's refusals that come before any device call."""
import numpy as np
import pytest

import __graft_entry__ as ge
import kosusun_ref as R


@pytest.fixture(scope="module")
def hy():
    from importlib import import_module
    ge.load_package()
    return import_module(ge.PKG_NAME + ".hybrid")


def test_ref_rotary_pairs_in_both_layouts():
    # 6 entries, the first 4 turn; entry pair i turns by pos * base^(-2 i / 4) / factor
    x = np.array([[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]]).repeat(2, axis=0)
    rot = {"dims": 4, "base": 100.0, "scaling": {"factor": 2.0}}
    a0, a1 = 3.0 / 2.0, 3.0 * 100.0 ** -0.5 / 2.0
    out = R.turn(x, np.array([0.0, 3.0]), rot, interleaved=True)
    assert np.allclose(out[0], x[0])
    want = [1 * np.cos(a0) - 2 * np.sin(a0), 2 * np.cos(a0) + 1 * np.sin(a0), 3 * np.cos(a1) - 4 * np.sin(a1), 4 * np.cos(a1) + 3 * np.sin(a1), 5.0, 6.0]
    assert np.allclose(out[1, 0], want)
    out = R.turn(x, np.array([0.0, 3.0]), rot, interleaved=False)
    want = [1 * np.cos(a0) - 3 * np.sin(a0), 2 * np.cos(a1) - 4 * np.sin(a1), 3 * np.cos(a0) + 1 * np.sin(a0), 4 * np.cos(a1) + 2 * np.sin(a1), 5.0, 6.0]
    assert np.allclose(out[1, 0], want)


def test_ref_window_and_blocks_seen():
    # window of 4, blocks of 3: query 9 holds positions 6 .. 9 and sees the blocks that end at or before position 5: blocks 0 and 1
    assert R.window_lo(9, 4) == 6 and R.blocks_seen(9, 4, 3) == 2
    # query 8 holds 5 .. 8; block 1 ends at 5 > 8 - 4: only block 0, and position 4 is seen neither way
    assert R.window_lo(8, 4) == 5 and R.blocks_seen(8, 4, 3) == 1
    assert R.blocks_seen(3, 4, 3) == 0 and R.blocks_seen(6, 4, 3) == 1 and R.blocks_seen(5, 4, 3) == 0
    assert R.blocks_seen(100, 4, 0) == 0


def one_head(**over):
    c = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 1.0, "mask": {"size": 2, "pool": 2}, "rot": None}
    c.update(over)
    return c


def test_ref_attention_sink_window_and_pooled_block_by_hand():
    # queries zeroed by their norm's weight: every seen key scores 0, the sink scores z: weights 1 / (n + e^z)
    z = np.log(2.0)
    p = {"q": np.eye(2), "q.b": np.zeros(2), "q.norm": np.zeros(2), "k": np.eye(2), "k.b": np.zeros(2), "k.norm": np.ones(2),
         "v": np.eye(2), "v.b": np.array([0.5, 0.0]), "sink": np.array([z]), "o": np.eye(2)}
    h = np.array([[1.0, 0.0], [0.0, 1.0], [2.0, 2.0], [0.0, 4.0], [6.0, 0.0]])
    v = h + p["v.b"]
    out = R.pooled_window_attention(h, p, one_head(), 0.0)
    assert np.allclose(out[0], v[0] / 3.0)                                      # one key and the sink's two units
    assert np.allclose(out[1], (v[0] + v[1]) / 4.0)
    assert np.allclose(out[2], (v[1] + v[2]) / 4.0)                             # position 0 has left the window, its block ends at 1 > 2 - 2
    assert np.allclose(out[3], ((v[0] + v[1]) / 2.0 + v[2] + v[3]) / 5.0)        # block 0 (positions 0, 1) is seen as ONE key
    assert np.allclose(out[4], ((v[0] + v[1]) / 2.0 + v[3] + v[4]) / 5.0)        # position 2 is in no window and in no complete block before it
    # the norm is over the whole projection: two heads of one entry each share one root mean square
    c2 = one_head(heads=2, kv_heads=2, dim=1, vdim=1)
    p2 = dict(p, q=np.eye(2), k=np.eye(2), sink=np.array([z, z]), **{"q.norm": np.array([1.0, 3.0])})
    h1 = np.array([[3.0, 4.0]])
    rms = np.sqrt(12.5)
    s = np.array([3.0 / rms * 3.0 / rms, 3.0 * 4.0 / rms * 4.0 / rms])         # q . k per head
    want = (h1[0] + p["v.b"]) * np.exp(s) / (np.exp(s) + 2.0)
    assert np.allclose(R.pooled_window_attention(h1, p2, c2, 0.0)[0], want)


def test_ref_retention_is_a_decayed_sum_over_the_past():
    rng = np.random.default_rng(0)
    c = {"heads": 2, "dim": 4, "vdim": 3, "rot": {"dims": 2, "base": 7.0}, "decay": [0.5, 0.9]}
    T, W = 6, 5
    h = rng.standard_normal((T, W))
    p = {n: rng.standard_normal(s) for n, s in (("q", (8, W)), ("k", (8, W)), ("v", (6, W)), ("g", (6, W)), ("o", (W, 6)))}
    pos = np.arange(T, dtype=np.float64)
    q = R.turn((h @ p["q"].T).reshape(T, 2, 4), pos, c["rot"], False)
    k = R.turn((h @ p["k"].T).reshape(T, 2, 4), pos, c["rot"], False) / 2.0
    v = (h @ p["v"].T).reshape(T, 2, 3)
    o = np.zeros((T, 2, 3))
    for t in range(T):
        for s in range(t + 1):
            for hd in range(2):
                o[t, hd] += c["decay"][hd] ** (t - s) * (q[t, hd] @ k[s, hd]) * v[s, hd]
    o = o / np.sqrt((o ** 2).mean(axis=-1, keepdims=True) + 1e-3)
    g = h @ p["g"].T
    want = (o.reshape(T, 6) * g / (1 + np.exp(-g))) @ p["o"].T
    assert np.allclose(R.retention(h, p, c, 1e-3), want)


def test_ref_mlstm_first_steps_by_hand():
    # one head, one key entry, one value entry; all projections are numbers
    c = {"heads": 1, "dim": 1, "vdim": 1, "gate_cap": 2.0}
    p = {"q": np.array([[1.0]]), "k": np.array([[1.0]]), "v": np.array([[1.0]]), "g": np.array([[0.0]]), "o": np.array([[1.0]]), "norm": np.array([3.0]),
         "i": np.array([[1.0]]), "i.b": np.array([0.5]), "f": np.array([[0.0]]), "f.b": np.array([1.0])}
    h = np.array([[2.0], [-1.0]])
    i0, i1 = 2.0 * np.tanh(2.5 / 2.0), 2.0 * np.tanh(-0.5 / 2.0)
    f = -np.log1p(np.exp(-2.0 * np.tanh(0.5)))
    m0 = max(f + 0.0, i0)                                                       # the running maximum starts at 0
    S0 = np.exp(i0 - m0) * 2.0 * 2.0
    n0 = np.exp(i0 - m0) * 2.0
    o0 = S0 * 2.0 / (max(abs(n0 * 2.0), np.exp(-m0)) + 1e-6)
    m1 = max(f + m0, i1)
    S1 = np.exp(f + m0 - m1) * S0 + np.exp(i1 - m1) * -1.0 * -1.0
    n1 = np.exp(f + m0 - m1) * n0 + np.exp(i1 - m1) * -1.0
    o1 = S1 * -1.0 / (max(abs(n1 * -1.0), np.exp(-m1)) + 1e-6)
    want = [np.sign(o) * 3.0 * 0.5 for o in (o0, o1)]                           # one entry per head: unit-RMS leaves its sign
    got = R.mlstm(h, p, c, 0.0)
    assert np.allclose(got[:, 0], want) and o0 != 0 and o1 != 0
    # the head's size matters before the norm only through the floor e^(-m): with a tiny query the floor rules the denominator
    p2 = dict(p, q=np.array([[1e-3]]))
    c2 = dict(c, vdim=2)
    p2.update(v=np.array([[1.0], [0.0]]), g=np.zeros((2, 1)), o=np.eye(2), norm=np.array([1.0, 1.0]))
    got = R.mlstm(h, p2, c2, 0.0)
    assert np.allclose(np.abs(got[:, 0]), np.sqrt(2.0) * 0.5) and np.allclose(got[:, 1], 0.0)


def test_ref_parallel_block_has_one_norm_and_one_residual_update():
    """A layer whose mixer is switched off by zero output projections: x <- x + mult * ff(norm1 x), then the logits' scale."""
    cfg = {"vocab": 3, "width": 2, "embedding": {"scale": 2.0}, "norm": {"eps": 0.0}, "residual_mult": 0.25, "logit_scale": 3.0,
           "layers": [{"type": "mlstm", "mixer": {"heads": 1, "dim": 1, "vdim": 1, "gate_cap": 1.0}, "mlp": {"kind": "dense", "ff": 1}}]}
    w = {"embed": np.array([[1.0, 0.5], [0.0, 1.0], [2.0, 2.0]]), "l0.norm1": np.array([1.0, 2.0]), "l0.mix.q": np.ones((1, 2)), "l0.mix.k": np.ones((1, 2)),
         "l0.mix.v": np.ones((1, 2)), "l0.mix.g": np.ones((1, 2)), "l0.mix.o": np.zeros((2, 1)), "l0.mix.norm": np.ones(1), "l0.mix.i": np.ones((1, 2)),
         "l0.mix.i.b": np.zeros(1), "l0.mix.f": np.ones((1, 2)), "l0.mix.f.b": np.zeros(1), "l0.mlp.gate": np.array([[1.0, 0.0]]),
         "l0.mlp.up": np.array([[0.0, 1.0]]), "l0.mlp.down": np.array([[1.0], [-2.0]]), "final.norm": np.array([1.0, 1.0]), "head": np.eye(2)}
    x0 = np.array([4.0, 4.0])                                                   # token 2 times the embedding scale
    hn = np.array([1.0, 2.0])                                                   # unit-RMS of equal entries is one, times norm1
    ff = R.gelu_tanh(hn[0]) * hn[1] * np.array([1.0, -2.0])
    x = x0 + 0.25 * ff
    want = x / np.sqrt((x ** 2).mean()) * 3.0
    assert np.allclose(R.forward(cfg, w, [2])[0], want)
    assert abs(R.gelu_tanh(1.0) - 0.8411919906082768) < 1e-12


def test_native_loader_refuses_before_touching_a_device(hy, tmp_path):
    L = hy.hip.lib()
    base = '{"architecture": "Kosusun", "vocab": 8, "width": 8, "norm": {"eps": 1e-6}, "layers": [%s]}'
    left = '"left": {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 1.0, "mask": {"size": 4, "pool": 2}, "rot": {"base": 10.0, "dims": 2}}'
    right = '"right": {"heads": 2, "dim": 4, "vdim": 4, "decay": [0.5, 0.9], "rot": {"base": 10.0, "dims": 2}}'
    for i, text in enumerate(['{"architecture": "Kosusun", "vocab": 8}', base % '{"type": "conv", "mixer": {}}', base % '{"type": "parallel"}',
                              base % ('{"type": "parallel", "mixer": {%s}}' % left),
                              base % ('{"type": "parallel", "mixer": {%s, %s}}' % (left, right.replace("[0.5, 0.9]", "[0.5]"))),
                              base % ('{"type": "parallel", "mlp": {"kind": "moe", "ff": 4}, "mixer": {%s, %s}}' % (left, right)),
                              base % '{"type": "mlstm", "mixer": {"heads": 2, "dim": 4, "vdim": 4}}']):
        d = tmp_path / ("c%d" % i)
        d.mkdir()
        (d / "config.json").write_text(text)
        assert L.gl3_is_model_dir(str(d).encode()) == 1
        with pytest.raises(hy.hip.Gl3Error) as e:
            hy.HybridPlan.from_dir(str(d))
        assert e.value.code in (hy.hip.E_ARG, hy.hip.E_UNSUPPORTED) and len(str(e.value)) > 20

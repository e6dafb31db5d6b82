"""The plain Vitudra oracle (tests/vitudra_oracle.py) pinned by closed forms: each mechanism on inputs whose answer is known by hand, and a demonstration that
switching any mechanism off moves the logits far beyond the tolerance the device path is held to.  CPU only."""
import copy

import numpy as np

import vitudra_oracle as vo
from test_hip_vitudra import config, tokens, want_of


def test_masks_by_hand():
    w = vo.window_mask(6, 3)
    assert w[5].tolist() == [False, False, False, True, True, True] and w[1].tolist() == [True, True, False, False, False, False]
    c = vo.chunk_mask(7, 3)
    assert c[5].tolist() == [False, False, False, True, True, True, False] and c[3].tolist() == [False, False, False, True, False, False, False]
    assert c[2].tolist() == [True, True, True, False, False, False, False]
    assert vo.window_mask(4, 1).tolist() == np.eye(4, dtype=bool).tolist()


def test_rotation_turns_neighbours_and_scaling_divides_the_angle():
    x = np.zeros((5, 1, 6)); x[:, 0, 0] = 1.0; x[:, 0, 2] = 1.0; x[:, 0, 5] = 3.0
    y = vo.rotate_pairs(x, 4, 100.0, 2.0)
    p = np.arange(5)
    np.testing.assert_allclose(y[:, 0, 0], np.cos(p / 2.0)); np.testing.assert_allclose(y[:, 0, 1], np.sin(p / 2.0))
    np.testing.assert_allclose(y[:, 0, 2], np.cos(p * 100.0 ** -0.5 / 2.0)); np.testing.assert_allclose(y[:, 0, 3], np.sin(p * 100.0 ** -0.5 / 2.0))
    assert (y[:, 0, 4:] == x[:, 0, 4:]).all()             # the channels beyond `dims` pass
    np.testing.assert_allclose((y ** 2).sum(-1), (x ** 2).sum(-1))


def test_attention_pieces():
    np.testing.assert_allclose(vo.distance_slopes(8), 2.0 ** -np.arange(1, 9))
    np.testing.assert_allclose(vo.query_temperature(130, 0.5, 64)[[0, 62, 63, 127, 128]], 1 + 0.5 * np.log([1, 1, 2, 3, 3]))
    rng = np.random.default_rng(0)
    q, k, v = rng.standard_normal((4, 2, 3)), rng.standard_normal((4, 1, 3)), rng.standard_normal((4, 1, 5))
    o = vo.softmax_attention(q, k, v, vo.window_mask(4, 1), 1.0)
    np.testing.assert_allclose(o[:, 0], v[:, 0]); np.testing.assert_allclose(o[:, 1], v[:, 0])      # one visible key: its value
    # two keys, scores 0: the bias alone decides, exp(-slope) against 1
    o = vo.softmax_attention(np.zeros((2, 1, 3)), k[:2], v[:2], vo.causal_mask(2), 1.0, 0.0, np.array([0.7]))
    e = np.exp(-0.7)
    np.testing.assert_allclose(o[1, 0], (e * v[0, 0] + v[1, 0]) / (1 + e))
    # a cap far below the scores makes them equal: the average of the values
    o = vo.softmax_attention(100 * np.ones((2, 1, 3)), np.ones((2, 1, 3)), v[:2], vo.causal_mask(2), 1.0, 1e-3)
    np.testing.assert_allclose(o[1, 0], v[:2, 0].mean(0), rtol=1e-9)


def test_short_convolution_and_the_delta_rule_by_hand():
    x = np.arange(1.0, 5.0)[:, None]
    np.testing.assert_allclose(vo.short_conv(x, np.array([[100.0, 10.0, 1.0]]))[:, 0], [1, 12, 123, 234])
    # one token: S = k (beta v)^T, read with q
    cfg = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "conv": 1}
    W, eye = 2, np.eye(2)
    t = {"q": eye, "k": eye, "v": eye, "q.conv": np.ones((2, 1)), "k.conv": np.ones((2, 1)), "v.conv": np.ones((2, 1)), "b": np.zeros((1, W)), "a": np.zeros((1, W)),
         "A_log": np.zeros(1), "dt_bias": np.zeros(1), "norm": np.ones(2), "g": eye, "o": eye}
    h = np.array([[1.0, 2.0]])
    s = vo.silu(h[0]); unit = s / np.sqrt((s * s).sum() + 1e-6)
    o = 0.5 * s * (unit @ unit) * 2 ** -0.5               # beta = 1/2; k . q = 1 / sqrt(dim)
    want = vo.rms_unit(o, 1e-5) * vo.silu(h[0])
    np.testing.assert_allclose(vo.gated_delta(h, cfg, t, "", 1e-5)[0], want, rtol=1e-6)


def test_wkv_by_hand():
    m = {"heads": 1, "dim": 2}
    eye = np.eye(2)
    t = {"mu." + s: np.zeros(2) for s in "rkvgw"}
    t.update({"r": eye, "k": eye, "v": eye, "g": eye, "w1": np.zeros((1, 2)), "w2": np.zeros((2, 1)), "w0": np.zeros(2), "u": np.array([[2.0, 3.0]]), "norm": np.ones(2), "o": eye})
    h = np.array([[1.0, 2.0], [0.5, -1.0]])
    # token 0: o = (u k r summed) v = (2 * 1 + 3 * 4) v; token 1: the state k0 v0^T decayed by exp(-1)... read before the decay applies, plus the bonus term
    o0 = (2 * 1 + 3 * 4) * h[0]
    o1 = (h[1] @ h[0]) * h[0] + (2 * 0.25 + 3 * 1.0) * h[1]
    want = np.stack([vo.rms_unit(o0, 1e-5), vo.rms_unit(o1, 1e-5)]) * vo.silu(h)
    np.testing.assert_allclose(vo.wkv_mixer(h, m, t, "", 1e-5), want, rtol=1e-9)
    # the token shift: mu = 1 hands every projection the token before
    t2 = dict(t, **{"mu." + s: np.ones(2) for s in "rkvgw"})
    got = vo.wkv_mixer(h, m, t2, "", 1e-5)
    assert np.abs(got[0]).max() == 0.0                    # the first token's predecessor is zero


def test_offset_norm_and_feed_forward():
    x = np.array([[3.0, 4.0]])
    np.testing.assert_allclose(vo.offset_norm(x, np.zeros(2), 0.0), x / np.sqrt(12.5))
    np.testing.assert_allclose(vo.offset_norm(x, np.array([1.0, -1.0]), 0.0), [[2 * 3 / np.sqrt(12.5), 0.0]])
    np.testing.assert_allclose(vo.dense_ff(x, np.eye(2), 2 * np.eye(2), np.eye(2)), vo.silu(x) * 2 * x)


def test_every_mechanism_moves_the_logits():
    """the oracle with one mechanism switched off differs far beyond the tolerance: a device path that left it out could not pass"""
    cfg = config()
    w = vo.random_tensors(cfg, 3)
    toks = tokens(cfg, 40)
    base = want_of(cfg, w, toks)

    def moved(c2=None, w2=None):
        return np.abs(want_of(c2 or cfg, w2 or w, toks) - base).max() / np.abs(base).max()

    def edit(path, value):
        c2 = copy.deepcopy(cfg)
        node = c2
        for k in path[:-1]:
            node = node[k]
        if value is None:
            node.pop(path[-1], None)
        else:
            node[path[-1]] = value
        return c2
    assert moved(edit(["residual_mult"], 0.5)) > 1e-2
    assert moved(edit(["layers", 2, "mixer", "mask", "size"], 12)) > 1e-3            # a window one longer
    assert moved(edit(["layers", 2, "mixer", "q_temp"], None)) > 1e-3
    assert moved(edit(["layers", 1, "mixer", "left", "mask", "size"], 10)) > 1e-3    # chunks one longer
    assert moved(edit(["layers", 1, "mixer", "left", "softcap"], None)) > 1e-4
    assert moved(edit(["layers", 1, "mixer", "left", "rot", "scaling", "factor"], 1.0)) > 1e-3
    assert moved(edit(["layers", 1, "mixer", "left", "rot"], None)) > 1e-3
    assert moved(edit(["layers", 1, "mixer", "right_scale"], 0.0)) > 1e-2
    assert moved(edit(["layers", 1, "mixer", "left_scale"], 0.0)) > 1e-2
    assert moved(w2={**w, "l0.mix.u": np.zeros_like(w["l0.mix.u"])}) > 1e-3
    assert moved(w2={**w, "l0.mix.mu.k": np.zeros_like(w["l0.mix.mu.k"])}) > 1e-3
    assert moved(w2={**w, "l0.mix.w0": w["l0.mix.w0"] + 1.0}) > 1e-3
    assert moved(w2={**w, "l1.mix.right.dt_bias": w["l1.mix.right.dt_bias"] + 2.0}) > 1e-4
    assert moved(w2={**w, "l1.mix.right.q.conv": np.roll(w["l1.mix.right.q.conv"], 1, axis=1)}) > 1e-4
    assert moved(w2={**w, "l0.norm1": np.zeros_like(w["l0.norm1"])}) > 1e-3
    c2 = edit(["layers", 4, "mixer", "kv_from"], None)                               # the sharing layer with projections of its own
    w2 = vo.random_tensors(c2, 3)
    assert moved(c2, {**w2, **w}) > 1e-3

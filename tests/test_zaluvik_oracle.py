"""The plain Zaluvik oracle (tests/zaluvik_oracle.py) pinned by closed forms: each mechanism on inputs whose answer is known by hand, and a demonstration
that switching any mechanism off (or moving a window by one) moves the logits far beyond the tolerance the device path is held to.  CPU only."""
import copy
import math

import numpy as np

import zaluvik_oracle as zo
from test_hip_zaluvik import attn, config, dense, lat, moe, tokens, want_of


def test_norms_by_hand():
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    y = zo.layer_norm(x, np.array([1.0, 1.0, 2.0, 1.0]), np.array([0.0, 0.5, 0.0, 0.0]), 0.0)
    sd = math.sqrt((4 + 1 + 0 + 9) / 4)
    np.testing.assert_allclose(y[0], [-2 / sd, -1 / sd + 0.5, 0.0, 3 / sd])
    np.testing.assert_allclose(zo.unit_rms(np.array([3.0, 4.0]), 0.0), np.array([3.0, 4.0]) / math.sqrt(12.5))
    np.testing.assert_allclose(zo.unit_rms(np.array([0.0, 0.0]), 1e-4), [0.0, 0.0])      # eps sits inside the root


def test_window_by_hand():
    v = zo.visible(6, 3)
    assert v[5].tolist() == [False, False, False, True, True, True] and v[1].tolist() == [True, True, False, False, False, False]
    assert zo.visible(4, 1).tolist() == np.eye(4, dtype=bool).tolist()
    assert zo.visible(3, None).tolist() == np.tril(np.ones((3, 3), bool)).tolist()


def test_rotation_pairs_a_channel_with_the_one_half_the_span_away():
    x = np.zeros((5, 6)); x[:, 0] = 1.0; x[:, 1] = 1.0; x[:, 5] = 3.0
    y = zo.rotate_half(x, np.arange(5.0), 4, 100.0)
    p = np.arange(5)
    np.testing.assert_allclose(y[:, 0], np.cos(p)); np.testing.assert_allclose(y[:, 2], np.sin(p))
    np.testing.assert_allclose(y[:, 1], np.cos(p * 100.0 ** -0.5)); np.testing.assert_allclose(y[:, 3], np.sin(p * 100.0 ** -0.5))
    assert (y[:, 4:] == x[:, 4:]).all()                    # the channels beyond `dims` pass
    np.testing.assert_allclose((y ** 2).sum(-1), (x ** 2).sum(-1))


def test_sigmoid_attention_by_hand():
    """two tokens, one head of one dimension: unit q and k are signs, weights are sigmoids that do not sum to one, the mixing matrix scales them"""
    m = {"heads": 1, "kv_heads": 1, "dim": 1, "vdim": 1, "scale": 2.0, "mask": {"size": 2}}
    one = np.ones((1, 1))
    h = np.array([[1.0], [-3.0]])
    out = zo.sigmoid_attention(h, m, one, one, one, np.zeros((1, 1)), one, np.array([[0.5]]), np.array([0.25]), 0.0)
    s = lambda z: 1 / (1 + math.exp(-z))
    np.testing.assert_allclose(out[0, 0], 0.5 * s(2.25) * 1.0 * 0.5)                                  # gate sigmoid(0) = 1/2
    np.testing.assert_allclose(out[1, 0], 0.5 * (s(-1.75) * 1.0 + s(2.25) * -3.0) * 0.5)
    m["mask"] = {"size": 1}
    out = zo.sigmoid_attention(h, m, one, one, one, np.zeros((1, 1)), one, np.array([[0.5]]), np.array([0.25]), 0.0)
    np.testing.assert_allclose(out[1, 0], 0.5 * s(2.25) * -3.0 * 0.5)


def test_heads_are_mixed_before_the_values_are_summed():
    rng = np.random.default_rng(0)
    m = {"heads": 2, "kv_heads": 2, "dim": 3, "vdim": 2, "scale": 1.0}
    W = 5
    wq, wk, wv, wg = rng.standard_normal((6, W)), rng.standard_normal((6, W)), rng.standard_normal((4, W)), np.zeros((4, W))
    h = rng.standard_normal((4, W))
    plain = zo.sigmoid_attention(h, m, wq, wk, wv, wg, np.eye(4), np.eye(2), np.zeros(2), 1e-5) * 2
    swap = zo.sigmoid_attention(h, m, wq, wk, wv, wg, np.eye(4), np.array([[0.0, 1.0], [1.0, 0.0]]), np.zeros(2), 1e-5) * 2
    # with the heads' weights swapped, head 0 applies head 1's weights to ITS OWN values
    q = zo.unit_rms((h @ wq.T).reshape(4, 2, 3), 1e-5); k = zo.unit_rms((h @ wk.T).reshape(4, 2, 3), 1e-5); v = (h @ wv.T).reshape(4, 2, 2)
    w1 = zo.sigmoid(q[:, 1] @ k[:, 1].T) * np.tril(np.ones((4, 4)))
    np.testing.assert_allclose(swap[:, :2], w1 @ v[:, 0])
    assert np.abs(plain - swap).max() > 0.1


def test_latent_attention_with_one_visible_key_hands_the_value_through():
    rng = np.random.default_rng(1)
    m = {"heads": 2, "dim": 3, "rot_dim": 2, "vdim": 4, "kv_rank": 5, "scale": 0.7, "mask": {"size": 1}, "rot": {"base": 10.0, "dims": 2}}
    W = 6
    t = [rng.standard_normal(s) for s in ((10, W), (7, W), (5,), (6, 5), (8, 5), (2, W), (W, 8))]
    h = rng.standard_normal((3, W))
    out = zo.latent_attention(h, m, *t, 1e-5)
    c = zo.unit_rms((h @ t[1].T)[:, :5], 1e-5) * t[2]
    v = (c @ t[4].T).reshape(3, 2, 4) * zo.sigmoid(h @ t[5].T)[:, :, None]
    np.testing.assert_allclose(out, v.reshape(3, 8) @ t[6].T)


def test_rotated_scores_depend_on_the_distance_only():
    """shifting every position by the same amount leaves the rotated part of the scores unchanged"""
    rng = np.random.default_rng(2)
    q, k = rng.standard_normal((6, 4)), rng.standard_normal((6, 4))
    a = zo.rotate_half(q, np.arange(6.0), 4, 50.0) @ zo.rotate_half(k, np.arange(6.0), 4, 50.0).T
    b = zo.rotate_half(q, np.arange(6.0) + 11, 4, 50.0) @ zo.rotate_half(k, np.arange(6.0) + 11, 4, 50.0).T
    np.testing.assert_allclose(a, b, atol=1e-12)


def test_router_by_hand():
    f = {"router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}}}
    # scores rise with the logit.  groups (0,1) (2,3) (4,5): sums of the two largest decide, not the single largest
    z = np.array([[3.0, -9.0, 1.0, 1.5, 0.0, 0.1]])
    wr = np.eye(6)
    idx, wts = zo.route(z, f, wr)
    s = zo.sigmoid(z[0])
    assert s[0] + s[1] < s[2] + s[3]                       # the group with the single best expert loses
    assert idx[0].tolist() == [3, 2]
    np.testing.assert_allclose(wts[0], [s[3] / (s[2] + s[3]), s[2] / (s[2] + s[3])])
    f["router"]["groups"] = {"count": 3, "keep": 2}
    assert zo.route(z, f, wr)[0][0].tolist() == [3, 2]     # the second open group is (4, 5): the best expert's group stays shut
    f["router"]["groups"] = {"count": 3, "keep": 3}
    idx, wts = zo.route(z, f, wr)
    assert idx[0].tolist() == [0, 3]                       # every group is open and the largest scores win
    del f["router"]["groups"]
    assert zo.route(z, f, wr)[0][0].tolist() == [0, 3]


def test_feed_forwards_by_hand():
    np.testing.assert_allclose(zo.gelu_erf(np.array([0.0, 1.0, -1.0])), [0.0, 0.5 * (1 + math.erf(2 ** -0.5)), -0.5 * (1 - math.erf(2 ** -0.5))])
    h = np.array([[2.0]])
    np.testing.assert_allclose(zo.gated_expert(h, np.array([[1.0]]), np.array([[3.0]]), np.array([[0.5]])), [[2.0 / (1 + math.exp(-2.0)) * 6.0 * 0.5]])


def test_the_loop_runs_its_layers_again_with_the_input_product_in_front():
    cfg = config([attn(dense()), lat(), attn()], loop=(1, 3, 2))
    assert zo.run_order(cfg) == [(0, False), (1, True), (2, False), (1, True), (2, False)]
    assert zo.run_order(config([attn()], loop=None)) == [(0, False)]
    w = zo.random_tensors(cfg, 0)
    toks = tokens(cfg, 9)
    st = []
    zo.forward(cfg, w, toks, st)
    assert len(st) == 5
    one = copy.deepcopy(cfg); one["loop"]["times"] = 1
    st1 = []
    zo.forward(one, w, toks, st1)
    np.testing.assert_allclose(st1[2], st[2])              # the first pass is the same; the second starts from W_loop [x; x0]
    x0 = np.asarray(w["embed"], np.float64)[toks] * cfg["embedding"]["scale"]
    x = np.concatenate([st[2], x0], -1) @ np.asarray(w["loop.in"], np.float64).T
    eps = cfg["norm"]["eps"]
    h = zo.layer_norm(x, w["l1.norm1"], w["l1.norm1.b"], eps)
    y = zo.latent_attention(h, cfg["layers"][1]["mixer"], *[w["l1.mix." + n] for n in ("q", "dkv", "dkv.norm", "uk", "uv", "g", "o")], eps)
    np.testing.assert_allclose(st[3], x + cfg["residual_mult"] * zo.layer_norm(y, w["l1.norm1b"], w["l1.norm1b.b"], eps))


def test_every_mechanism_moves_the_logits():
    """each switch changes the logits by far more than the 1e-4 the device path is held to in fp32"""
    cfg = config()
    w = zo.random_tensors(cfg, 3)
    toks = tokens(cfg, 30)
    base = want_of(cfg, w, toks)
    scale = np.abs(base).max()

    def moved(c=None, ww=None):
        return np.abs(want_of(c or cfg, ww or w, toks) - base).max() / scale

    def with_cfg(fn):
        c = copy.deepcopy(cfg); fn(c); return c

    def with_w(**kw):
        ww = dict(w); ww.update(kw); return ww

    assert moved(with_cfg(lambda c: c["layers"][0]["mixer"]["mask"].update(size=10))) > 1e-2        # a window one shorter
    assert moved(with_cfg(lambda c: c["layers"][1]["mixer"]["mask"].update(size=14))) > 1e-3        # a latent window one longer
    assert moved(with_cfg(lambda c: c["loop"].update(times=1))) > 1e-2
    assert moved(with_cfg(lambda c: c.pop("loop"))) > 1e-2                                            # no input product at all
    assert moved(with_cfg(lambda c: c["embedding"].update(scale=1.0))) > 1e-2
    assert moved(with_cfg(lambda c: c.update(residual_mult=1.0))) > 1e-2
    assert moved(with_cfg(lambda c: c["layers"][1]["mixer"]["rot"].update(base=10000.0))) > 1e-3
    assert moved(with_cfg(lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=3))) > 1e-3
    assert moved(with_cfg(lambda c: c["layers"][1]["mlp"]["router"].update(top=1))) > 1e-3
    assert moved(ww=with_w(**{"l0.mix.talk": np.eye(4)})) > 1e-2
    assert moved(ww=with_w(**{"l0.mix.pb": np.zeros(4)})) > 1e-3
    assert moved(ww=with_w(**{"l0.norm1b.b": np.zeros(24)})) > 1e-3
    assert moved(ww=with_w(**{"final.norm.b": np.zeros(24)})) > 1e-3
    assert moved(ww=with_w(**{"l1.mlp.shared.down": np.zeros_like(w["l1.mlp.shared.down"])})) > 1e-3
    assert moved(ww=with_w(**{"l1.mix.g": np.zeros_like(w["l1.mix.g"])})) > 1e-3

"""A plain, slow restatement of the Zaluvik design in numpy float64: one function per mechanism, whole sequences only (no cache, no batching, no
pages), written from the design's equations and sharing no code with the product.  The GPU tests compare the library with it.

Notation.  x: the residual stream [T][W]; h: a sublayer's input; a config dictionary `cfg` is the checkpoint's config.json; `w` maps checkpoint names
to arrays.  Positions count from 0.

  embedding     x = embed[token] * embedding.scale; x0 = that x
  layer         x += m * LN_1b(mixer(LN_1(x))); x += m * LN_2b(ff(LN_2(x)))       m = residual_mult; LN has a weight and a bias ("<name>", "<name>.b")
  loop          layers start .. stop - 1 run `times` times in a row (same weights); in front of the first of them, every pass: x = W_loop [x; x0]
  attention     unit-RMS q and k per head, score = q . k * scale, window of mask.size, weight = sigmoid(score + pb[head]) (not normalised), weights mixed
                across heads by `talk`, value sums per head over its own key / value head, times sigmoid(W_g h) per channel, W_o
  latent        q = [plain | rotated] per head; dkv = [latent (RMS norm with weight) | one rotated key part]; k_plain = W_uk c, v = W_uv c;
                score = (q_plain . k_plain + rot(q_rot) . rot(k_rot)) * scale; window; softmax; times sigmoid(W_g h) per head; W_o
  dense         W_down gelu(W_up h), gelu with erf
  experts       s = sigmoid(W_r h); groups of neighbours, a group counts as the sum of its two largest s, the best `keep` groups stay; the `top` largest s
                among them; weights = s / (sum + 1e-20); experts W_down (silu(W_gate h) * W_up h); a shared expert added for every token
  output        logits = embed LN_final(x)
"""
import math

import numpy as np


def bf16_round(a):
    """round-to-nearest-even onto the bfloat16 grid (as float32 values)"""
    u = np.asarray(a, np.float32).reshape(-1).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def layer_norm(x, weight, bias, eps):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * weight + bias


def unit_rms(x, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def visible(T, size):
    """[T][T] True where query i sees key j: 0 <= i - j < size (size None: every j <= i)"""
    d = np.arange(T)[:, None] - np.arange(T)[None, :]
    return (d >= 0) & ((d < size) if size else True)


def sigmoid_attention(h, m, wq, wk, wv, wg, wo, talk, pb, eps):
    T = h.shape[0]
    H, G, D, VD = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = unit_rms((h @ wq.T).reshape(T, H, D), eps)
    k = unit_rms((h @ wk.T).reshape(T, G, D), eps)
    v = (h @ wv.T).reshape(T, G, VD)
    see = visible(T, (m.get("mask") or {}).get("size"))
    wts = np.zeros((H, T, T))
    for g in range(H):
        wts[g] = sigmoid(q[:, g] @ k[:, g // (H // G)].T * m["scale"] + pb[g]) * see
    mixed = np.einsum("hg,gij->hij", talk, wts)
    out = np.zeros((T, H, VD))
    for hh in range(H):
        out[:, hh] = mixed[hh] @ v[:, hh // (H // G)]
    return (out.reshape(T, H * VD) * sigmoid(h @ wg.T)) @ wo.T


def rotate_half(x, pos, dims, base):
    """the first `dims` entries of the last axis turn: entry i pairs with i + dims / 2, angle pos * base^(-2i / dims); x [T][...][n]"""
    out = np.array(x, np.float64)
    half = dims // 2
    for i in range(half):
        ang = pos * base ** (-2.0 * i / dims)
        c, s = np.cos(ang), np.sin(ang)
        shape = (-1,) + (1,) * (x.ndim - 2)
        c, s = c.reshape(shape), s.reshape(shape)
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * c - v * s
        out[..., i + half] = v * c + u * s
    return out


def latent_attention(h, m, wq, wdkv, lat_w, wuk, wuv, wg, wo, eps):
    T = h.shape[0]
    H, D, RD, VD, R = m["heads"], m["dim"], m.get("rot_dim", 0), m.get("vdim", m["dim"]), m["kv_rank"]
    pos = np.arange(T, dtype=np.float64)
    q = (h @ wq.T).reshape(T, H, D + RD)
    dkv = h @ wdkv.T
    c = unit_rms(dkv[:, :R], eps) * lat_w
    q_plain, q_rot, k_rot = q[..., :D], q[..., D:], dkv[:, R:]
    if RD:
        rot = m.get("rot") or {}
        dims, base = rot.get("dims", RD), rot.get("base", 10000.0)
        q_rot, k_rot = rotate_half(q_rot, pos, dims, base), rotate_half(k_rot, pos, dims, base)
    k_plain = (c @ wuk.T).reshape(T, H, D)
    v = (c @ wuv.T).reshape(T, H, VD)
    see = visible(T, (m.get("mask") or {}).get("size"))
    gate = sigmoid(h @ wg.T)                                 # [T][H]
    out = np.zeros((T, H, VD))
    for hh in range(H):
        s = (q_plain[:, hh] @ k_plain[:, hh].T + q_rot[:, hh] @ k_rot.T) * m["scale"]
        s = np.where(see, s, -np.inf)
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        out[:, hh] = (p @ v[:, hh]) * gate[:, hh:hh + 1]
    return out.reshape(T, H * VD) @ wo.T


def gelu_erf(z):
    return 0.5 * z * (1.0 + np.vectorize(math.erf)(z / math.sqrt(2.0)))


def dense_ff(h, wup, wdown):
    return gelu_erf(h @ wup.T) @ wdown.T


def gated_expert(h, wgate, wup, wdown):
    g = h @ wgate.T
    return (g * sigmoid(g) * (h @ wup.T)) @ wdown.T


def route(h, f, wr):
    """chosen experts [T][top] and their weights, token by token"""
    r = f["router"]
    E, top = r["experts"], r["top"]
    grp = r.get("groups") or {}
    n_g, keep = grp.get("count", 1), grp.get("keep", grp.get("count", 1))
    s = sigmoid(np.asarray(h, np.float32).astype(np.float64) @ wr.T)
    idx, wts = np.zeros((len(h), top), int), np.zeros((len(h), top))
    for t in range(len(h)):
        ok = np.ones(E, bool)
        if n_g > 1:
            per = E // n_g
            gs = [np.sort(s[t, g * per:(g + 1) * per])[-2:].sum() for g in range(n_g)]
            best = sorted(range(n_g), key=lambda g: (-gs[g], g))[:keep]
            ok = np.array([e // per in best for e in range(E)])
        order = sorted([e for e in range(E) if ok[e]], key=lambda e: (-s[t, e], e))[:top]
        idx[t] = order
        wts[t] = s[t, order] / (s[t, order].sum() + 1e-20)
    return idx, wts


def moe_ff(h, f, w, p):
    idx, wts = route(h, f, w[p + "router"])
    out = np.zeros_like(h)
    for t in range(len(h)):
        for e, a in zip(idx[t], wts[t]):
            out[t] += a * gated_expert(h[t:t + 1], w[f"{p}e{e}.gate"], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"])[0]
    if f.get("shared"):
        out += gated_expert(h, w[p + "shared.gate"], w[p + "shared.up"], w[p + "shared.down"])
    return out


def run_order(cfg):
    """(layer, whether the loop's input product comes first) in the order the layers run"""
    n, lp = len(cfg["layers"]), cfg.get("loop")
    if not lp or lp["stop"] <= lp["start"]:
        return [(i, False) for i in range(n)]
    order = [(i, False) for i in range(lp["start"])]
    for _ in range(lp["times"]):
        order += [(i, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return order + [(i, False) for i in range(lp["stop"], n)]


def forward(cfg, w, tokens, streams=None):
    """logits [T][vocab] of a whole sequence; `streams` (a list) receives the residual stream after every layer run"""
    w = {k: np.asarray(v, np.float64) for k, v in w.items()}
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    ln = lambda v, n: layer_norm(v, w[n], w[n + ".b"], eps)
    x = w["embed"][np.asarray(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    x0 = x
    for i, first in run_order(cfg):
        if first:
            x = np.concatenate([x, x0], -1) @ w["loop.in"].T
        l, p = cfg["layers"][i], f"l{i}."
        h = ln(x, p + "norm1")
        if l["type"] == "attention":
            y = sigmoid_attention(h, l["mixer"], w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"], w[p + "mix.g"], w[p + "mix.o"], w[p + "mix.talk"], w[p + "mix.pb"], eps)
        else:
            y = latent_attention(h, l["mixer"], w[p + "mix.q"], w[p + "mix.dkv"], w[p + "mix.dkv.norm"], w[p + "mix.uk"], w[p + "mix.uv"], w[p + "mix.g"], w[p + "mix.o"], eps)
        x = x + m * ln(y, p + "norm1b")
        f = l.get("mlp")
        if f:
            h = ln(x, p + "norm2")
            y = dense_ff(h, w[p + "mlp.up"], w[p + "mlp.down"]) if f["kind"] == "dense" else moe_ff(h, f, w, p + "mlp.")
            x = x + m * ln(y, p + "norm2b")
        if streams is not None:
            streams.append(x.copy())
    return ln(x, "final.norm") @ w["embed"].T


def tensor_shapes(cfg):
    W, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"])}
    lp = cfg.get("loop")
    if lp and lp["stop"] > lp["start"]:
        out["loop.in"] = (W, 2 * W)
    for i, l in enumerate(cfg["layers"]):
        p, m, f = f"l{i}.", l["mixer"], l.get("mlp")
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if f else ()):
            out[p + n] = (W,); out[p + n + ".b"] = (W,)
        H, D, VD = m["heads"], m["dim"], m.get("vdim", m["dim"])
        if l["type"] == "attention":
            G = m.get("kv_heads", H)
            out.update({p + "mix.q": (H * D, W), p + "mix.k": (G * D, W), p + "mix.v": (G * VD, W), p + "mix.talk": (H, H), p + "mix.pb": (H,), p + "mix.g": (H * VD, W),
                        p + "mix.o": (W, H * VD)})
        else:
            R, RD = m["kv_rank"], m.get("rot_dim", 0)
            out.update({p + "mix.q": (H * (D + RD), W), p + "mix.dkv": (R + RD, W), p + "mix.dkv.norm": (R,), p + "mix.uk": (H * D, R), p + "mix.uv": (H * VD, R),
                        p + "mix.g": (H, W), p + "mix.o": (W, H * VD)})
        if f and f["kind"] == "dense":
            out[p + "mlp.up"] = (f["ff"], W); out[p + "mlp.down"] = (W, f["ff"])
        elif f:
            F = f["expert"]["ff"]
            for e in range(f["router"]["experts"]):
                out[p + f"mlp.e{e}.gate"] = (F, W); out[p + f"mlp.e{e}.up"] = (F, W); out[p + f"mlp.e{e}.down"] = (W, F)
            out[p + "mlp.router"] = (f["router"]["experts"], W)
            if f.get("shared"):
                S = f["shared"]["ff"]
                out[p + "mlp.shared.gate"] = (S, W); out[p + "mlp.shared.up"] = (S, W); out[p + "mlp.shared.down"] = (W, S)
    out["final.norm"] = (W,); out["final.norm.b"] = (W,)
    return out


def random_tensors(cfg, seed=0, overrides=None):
    """weights on the bfloat16 grid, scaled so that every mechanism matters: projections ~ 1 / sqrt(inputs), norm weights around one with biases, a head
    mixing matrix near the identity with sizeable off-diagonal entries, score biases of both signs, router rows large enough to spread the choices"""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if name == "embed":
            v = rng.standard_normal(shape)
        elif leaf == "talk":
            v = np.eye(shape[0]) + rng.standard_normal(shape) * 0.4
        elif leaf == "pb":
            v = rng.uniform(-2.0, 1.0, shape)
        elif leaf == "router":
            v = rng.standard_normal(shape) * 3.0 / np.sqrt(shape[1])
        elif name == "loop.in":
            v = rng.standard_normal(shape) / np.sqrt(shape[1] / 2)
        elif len(shape) == 2:
            v = rng.standard_normal(shape) / np.sqrt(shape[1])
        elif leaf == "b":
            v = rng.standard_normal(shape) * 0.2
        else:
            v = rng.uniform(0.5, 1.5, shape)                 # norm weights
        out[name] = bf16_round(v)
    for k, v in (overrides or {}).items():
        out[k] = bf16_round(v)
    return out

"""Plain numpy (float64) restatement of the Vitudra design, one function per mechanism, whole sequences only (no cache, no state
between calls): the slow restatement that the device path is compared with.  It shares no code with tinygpt_amd.

A model is (cfg, tensors): cfg the dictionary of the checkpoint's config.json, tensors name -> float array.
Notation: T tokens, W width, H query heads, G key / value heads, D key size, E value size.
"""
import math

import numpy as np


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis"""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight is the distance from one"""
    return rms_unit(x, eps) * (1.0 + w)


def silu(z):
    return z / (1.0 + np.exp(-z))


def softplus(z):
    return np.where(z > 30, z, np.log1p(np.exp(np.minimum(z, 30))))


def dense_ff(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


# ---- masks: visible[i][j] for query position i and key position j ------------------------------------------------------------------
def window_mask(T, size):
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (i - j >= 0) & (i - j < size)


def chunk_mask(T, size):
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


def causal_mask(T):
    return np.tril(np.ones((T, T), bool))


def rotate_pairs(x, dims, base, factor):
    """x [T][heads][D]: neighbours (2i, 2i + 1) of the first `dims` channels turn by position * base^(-2i / dims) / factor"""
    T = x.shape[0]
    out = x.copy()
    f = base ** (-2.0 * np.arange(dims // 2) / dims) / factor
    a = np.arange(T)[:, None] * f[None, :]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def softmax_attention(q, k, v, visible, scale, softcap=0.0, slopes=None):
    """q [T][H][D], k [T][G][D], v [T][G][E] -> [T][H][E]; scores * scale, soft cap, minus slope_h * distance, softmax over the visible keys"""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    dist = np.arange(T)[:, None] - np.arange(T)[None, :]
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * np.tanh(s / softcap)
        if slopes is not None:
            s = s - slopes[h] * dist
        s = np.where(visible, s, -np.inf)
        s = s - s.max(axis=1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=1, keepdims=True)
        out[:, h] = p @ v[:, g]
    return out


def distance_slopes(H):
    return np.array([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])


def query_temperature(T, coef, every):
    p = np.arange(T)
    return 1.0 + coef * np.log(np.floor((p + 1) / every) + 1.0)


# ---- the three mixers --------------------------------------------------------------------------------------------------------------
def attention_mixer(h, m, t, pre, eps, kv=None):
    """sliding-window attention without rotation: query temperature, distance bias.  kv: (k, v) of the layer named by kv_from.  Returns (out, (k, v))."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[pre + "q"].T).reshape(T, H, D)
    if kv is None:
        kv = ((h @ t[pre + "k"].T).reshape(T, G, D), (h @ t[pre + "v"].T).reshape(T, G, E))
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(T, qt["coef"], qt["every"])[:, None, None]
    vis = window_mask(T, m["mask"]["size"]) if m.get("mask") else causal_mask(T)
    o = softmax_attention(q, kv[0], kv[1], vis, m["scale"], 0.0, distance_slopes(H))
    return o.reshape(T, H * E) @ t[pre + "o"].T, kv


def rotary_chunk_attention(h, m, t, pre):
    """the left half of a parallel mixer: rotated queries and keys, soft-capped scores, chunked mask"""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[pre + "q"].T).reshape(T, H, D)
    k = (h @ t[pre + "k"].T).reshape(T, G, D)
    v = (h @ t[pre + "v"].T).reshape(T, G, E)
    rot = m.get("rot")
    if rot:
        factor = (rot.get("scaling") or {}).get("factor", 1.0)
        q = rotate_pairs(q, rot["dims"], rot["base"], factor)
        k = rotate_pairs(k, rot["dims"], rot["base"], factor)
    vis = chunk_mask(T, m["mask"]["size"]) if m.get("mask") else causal_mask(T)
    o = softmax_attention(q, k, v, vis, m["scale"], m.get("softcap", 0.0))
    return o.reshape(T, H * E) @ t[pre + "o"].T


def short_conv(x, w):
    """x [T][C], w [C][taps] (last column: the current token), zeros before the start"""
    T, taps = x.shape[0], w.shape[1]
    out = np.zeros_like(x)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            out[back:] += x[:T - back] * w[:, j]
    return out


def gated_delta(h, m, t, pre, eps):
    """the right half: short convolutions, unit queries and keys, a decaying matrix state written by the delta rule"""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ t[pre + "q"].T, t[pre + "q.conv"])).reshape(T, G, D)
    k = silu(short_conv(h @ t[pre + "k"].T, t[pre + "k.conv"])).reshape(T, G, D)
    v = silu(short_conv(h @ t[pre + "v"].T, t[pre + "v.conv"])).reshape(T, H, E)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = 1.0 / (1.0 + np.exp(-(h @ t[pre + "b"].T)))
    decay = np.exp(-np.exp(t[pre + "A_log"]) * softplus(h @ t[pre + "a"].T + t[pre + "dt_bias"]))
    o = np.zeros((T, H, E))
    for hd in range(H):
        g = hd // (H // G)
        S = np.zeros((D, E))
        for i in range(T):
            S = decay[i, hd] * S
            u = beta[i, hd] * (v[i, hd] - S.T @ k[i, g])
            S = S + np.outer(k[i, g], u)
            o[i, hd] = S.T @ q[i, g]
    o = rms_unit(o, eps) * t[pre + "norm"] * silu(h @ t[pre + "g"].T).reshape(T, H, E)
    return o.reshape(T, H * E) @ t[pre + "o"].T


def parallel_mixer(h, m, t, pre, eps):
    return m["left_scale"] * rotary_chunk_attention(h, m["left"], t, pre + "left.") + m["right_scale"] * gated_delta(h, m["right"], t, pre + "right.", eps)


def wkv_mixer(h, m, t, pre, eps):
    """token-shift mixes, data-dependent decay per key channel, a bonus for the current token, per-head unit norm, silu gate"""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    prev = np.vstack([np.zeros((1, h.shape[1])), h[:-1]])
    mix = {s: h + (prev - h) * t[pre + "mu." + s] for s in "rkvgw"}
    r = (mix["r"] @ t[pre + "r"].T).reshape(T, H, D)
    k = (mix["k"] @ t[pre + "k"].T).reshape(T, H, D)
    v = (mix["v"] @ t[pre + "v"].T).reshape(T, H, D)
    gate = silu(mix["g"] @ t[pre + "g"].T)
    w = np.exp(-np.exp(np.tanh(mix["w"] @ t[pre + "w1"].T) @ t[pre + "w2"].T + t[pre + "w0"])).reshape(T, H, D)
    u = t[pre + "u"].reshape(H, D)
    o = np.zeros((T, H, D))
    for hd in range(H):
        S = np.zeros((D, D))
        for i in range(T):
            kv = np.outer(k[i, hd], v[i, hd])
            o[i, hd] = (S + u[hd][:, None] * kv).T @ r[i, hd]
            S = w[i, hd][:, None] * S + kv
    o = rms_unit(o, eps).reshape(T, H * D) * t[pre + "norm"] * gate
    return o @ t[pre + "o"].T


# ---- the model ---------------------------------------------------------------------------------------------------------------------
def forward(cfg, t, ids, layers_out=None):
    """logits [T][vocab] of one sequence; layers_out (a list) receives the stream after every layer"""
    t = {k: np.asarray(v, np.float64) for k, v in t.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = t["embed"][np.asarray(ids)]
    kvs = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = offset_norm(x, t[p + "norm1"], eps)
        m = L["mixer"]
        if L["type"] == "wkv":
            y = wkv_mixer(h, m, t, p + "mix.", eps)
        elif L["type"] == "parallel":
            y = parallel_mixer(h, m, t, p + "mix.", eps)
        elif L["type"] == "attention":
            y, kvs[i] = attention_mixer(h, m, t, p + "mix.", eps, kvs[m["kv_from"]] if "kv_from" in m else None)
        else:
            raise ValueError(L["type"])
        if L.get("mlp"):
            y = y + dense_ff(h, t[p + "mlp.gate"], t[p + "mlp.up"], t[p + "mlp.down"])
        x = x + mult * y
        if layers_out is not None:
            layers_out.append(x.copy())
    return offset_norm(x, t["final.norm"], eps) @ t["head"].T


# ---- random models -----------------------------------------------------------------------------------------------------------------
def tensor_shapes(cfg, decay_rank=5):
    """checkpoint name -> shape; the decay rank of the wkv layers is not part of the configuration (the tensors carry it)"""
    W, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"])}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        out[p + "norm1"] = (W,)
        if L["type"] == "attention":
            H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out[p + "mix.q"] = (H * D, W)
            if "kv_from" not in m:
                out[p + "mix.k"] = (G * D, W); out[p + "mix.v"] = (G * E, W)
            out[p + "mix.o"] = (W, H * E)
        elif L["type"] == "wkv":
            HD = m["heads"] * m["dim"]
            for s in "rkvgw":
                out[p + "mix.mu." + s] = (W,)
            for s in "rkvg":
                out[p + "mix." + s] = (HD, W)
            out.update({p + "mix.w1": (decay_rank, W), p + "mix.w2": (HD, decay_rank), p + "mix.w0": (HD,), p + "mix.u": (m["heads"], m["dim"]),
                        p + "mix.norm": (HD,), p + "mix.o": (W, HD)})
        else:
            l, r = m["left"], m["right"]
            out.update({p + "mix.left.q": (l["heads"] * l["dim"], W), p + "mix.left.k": (l["kv_heads"] * l["dim"], W), p + "mix.left.v": (l["kv_heads"] * l["vdim"], W),
                        p + "mix.left.o": (W, l["heads"] * l["vdim"])})
            gd, vd, q = r["kv_heads"] * r["dim"], r["heads"] * r["vdim"], p + "mix.right."
            for s, n in (("q", gd), ("k", gd), ("v", vd)):
                out[q + s] = (n, W); out[q + s + ".conv"] = (n, r["conv"])
            out.update({q + "b": (r["heads"], W), q + "a": (r["heads"], W), q + "A_log": (r["heads"],), q + "dt_bias": (r["heads"],), q + "norm": (r["vdim"],),
                        q + "g": (vd, W), q + "o": (W, vd)})
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            out.update({p + "mlp.gate": (F, W), p + "mlp.up": (F, W), p + "mlp.down": (W, F)})
    out["final.norm"] = (W,)
    out["head"] = (cfg["vocab"], W)
    return out


def bf16_round(a):
    """round-to-nearest-even onto the bfloat16 grid, so that every storage dtype of the library holds the same numbers"""
    u = np.asarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def random_tensors(cfg, seed=0, overrides=None, decay_rank=5):
    """weights on the bfloat16 grid, scaled so that every mechanism matters: projections ~ 1 / sqrt(inputs), norm weights around zero, decays spread over (0, 1)"""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, decay_rank).items():
        leaf = name.split(".")[-1]
        if name == "embed":
            v = rng.standard_normal(shape)
        elif leaf == "conv":
            v = rng.standard_normal(shape) * 0.6
        elif leaf == "u":
            v = rng.standard_normal(shape) * 0.5
        elif leaf == "w2":
            v = rng.standard_normal(shape) * 0.7
        elif len(shape) == 2:
            v = rng.standard_normal(shape) / np.sqrt(shape[1])
        elif leaf == "norm1" or name == "final.norm":
            v = rng.uniform(-0.3, 0.3, shape)
        elif ".mu." in name:
            v = rng.uniform(0.0, 1.0, shape)
        elif leaf == "w0":
            v = rng.uniform(-3.0, 0.3, shape)
        elif leaf == "A_log":
            v = rng.uniform(-2.5, 0.3, shape)
        elif leaf == "dt_bias":
            v = rng.uniform(-1.0, 1.0, shape)
        elif leaf == "norm":
            v = rng.uniform(0.5, 1.5, shape)
        else:
            v = rng.standard_normal(shape) * 0.3
        out[name] = bf16_round(v)
    for k, v in (overrides or {}).items():
        out[k] = bf16_round(v)
    return out

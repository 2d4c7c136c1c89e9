"""Plain, slow float64 statement of the Zifetar design, one function per mechanism, for the tests of the layer-stack model class.

It shares nothing with the product path: numpy only, one whole sequence at a time, token-by-token recurrences, no cache, no pages,
no state slots.  `forward` takes the config.json dict of a model and its tensors (name -> float array) and returns the logits of every
position of ONE sequence (and, on request, the residual stream after every layer).

Notation: x residual stream [T, width]; positions p = 0..T-1; N(v; w) = v / sqrt(mean(v^2) + eps) * (1 + w).
A layer is  x <- x + N(mixer(N(x; n1)); n1b),  x <- x + N(ff(N(x; n2)); n2b).
"""
import math

import numpy as np


def sigmoid(z):
    return 0.5 * (1.0 + np.tanh(0.5 * np.asarray(z, np.float64)))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    z = np.asarray(z, np.float64)
    return np.maximum(z, 0.0) + np.log1p(np.exp(-np.abs(z)))


def rms(v, eps):
    """v / sqrt(mean(v^2) + eps) over the last axis"""
    return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps)


def norm1p(v, w, eps):
    """RMS norm whose weight is stored around zero"""
    return rms(v, eps) * (1.0 + w)


def embed_tokens(tokens, embed, bigram, scale, buckets, mul_prev, mul_cur):
    """embedding row times a constant, plus a row of a hashed (previous token, token) table; the first token takes the table's last row"""
    tokens = np.asarray(tokens, np.int64)
    x = embed[tokens] * scale
    rows = np.empty(len(tokens), np.int64)
    rows[0] = buckets
    rows[1:] = (tokens[:-1] * mul_prev + tokens[1:] * mul_cur) % buckets
    return x + bigram[rows]


def rotary_freqs(dims, base, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2; optional wavelength-dependent slowdown: long waves are divided by `factor`, short ones kept,
    those between blended linearly in original/wavelength"""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], np.float64)
    if scaling:
        fac, lo, hi, orig = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"]), float(scaling["original"])
        out = f.copy()
        for i, fi in enumerate(f):
            wl = 2.0 * math.pi / fi
            if wl < orig / hi:
                out[i] = fi
            elif wl > orig / lo:
                out[i] = fi / fac
            else:
                s = (orig / wl - lo) / (hi - lo)
                out[i] = (1.0 - s) * fi / fac + s * fi
        f = out
    return f


def rotate_half(v, pos, freqs):
    """v [T, heads, dim]; dimension i pairs with i + n/2 (n = 2 len(freqs)) inside the first n dimensions; the rest pass"""
    n = 2 * len(freqs)
    if n == 0:
        return v.copy()
    ang = np.asarray(pos, np.float64)[:, None] * freqs[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    a, b = v[..., :n // 2], v[..., n // 2:n]
    out = v.copy()
    out[..., :n // 2] = a * c - b * s
    out[..., n // 2:n] = b * c + a * s
    return out


def causal_conv_silu(z, w):
    """z [T, C], w [C, taps] (last column = the current token), zeros before the start; then silu"""
    T, C = z.shape
    taps = w.shape[1]
    pad = np.concatenate([np.zeros((taps - 1, C)), z], 0)
    out = np.zeros((T, C))
    for j in range(taps):
        out += pad[j:j + T] * w[:, j][None, :]
    return silu(out)


def linear_recurrence(q, k, v, decay, beta=None):
    """Per head a matrix state S [dim, vdim] from zero:  S <- decay_t * S (decay [T, H, dim] on the rows);  without beta  S <- S + k v^T;
    with beta (delta rule)  u = beta (v - S^T k),  S <- S + k u^T;  o_t = S^T q_t after the write.  q, k [T, H, dim], v [T, H, vdim]."""
    T, H, D = q.shape
    V = v.shape[-1]
    S = np.zeros((H, D, V))
    o = np.zeros((T, H, V))
    for t in range(T):
        S = S * decay[t][:, :, None]
        if beta is None:
            u = v[t]
        else:
            u = beta[t][:, None] * (v[t] - np.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    return o


def mixer_channel_delta(h, mx, w, p, eps):
    """gated delta rule with a decay per key channel"""
    T = h.shape[0]
    H, G, D, V = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx.get("vdim", mx["dim"])
    q = causal_conv_silu(h @ w[p + "q"].T, w[p + "q.conv"]).reshape(T, G, D)
    k = causal_conv_silu(h @ w[p + "k"].T, w[p + "k.conv"]).reshape(T, G, D)
    v = causal_conv_silu(h @ w[p + "v"].T, w[p + "v.conv"]).reshape(T, H, V)
    unit = lambda a: a / np.sqrt((a * a).sum(-1, keepdims=True) + 1e-6)
    q, k = unit(q) * D ** -0.5, unit(k)
    rep = H // G
    q, k = np.repeat(q, rep, 1), np.repeat(k, rep, 1)
    beta = sigmoid(h @ w[p + "b"].T)
    dt = softplus((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).reshape(T, H, D)
    g = np.exp(-np.exp(w[p + "A_log"])[None, :, None] * dt)
    o = linear_recurrence(q, k, v, g, beta)
    o = rms(o, eps) * w[p + "norm"][None, None, :]
    gate = sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).reshape(T, H, V)
    return (o * gate).reshape(T, H * V) @ w[p + "o"].T


def mixer_retention(h, mx, w, p, eps):
    """linear attention with a constant decay per head; rotary on q and k"""
    T = h.shape[0]
    H, D, V = mx["heads"], mx["dim"], mx.get("vdim", mx["dim"])
    rot = mx.get("rot") or {}
    fr = rotary_freqs(int(rot.get("dims", 0)), float(rot.get("base", 10000.0)), rot.get("scaling")) if rot.get("dims") else np.zeros(0)
    pos = np.arange(T)
    q = rotate_half((h @ w[p + "q"].T).reshape(T, H, D), pos, fr)
    k = rotate_half((h @ w[p + "k"].T).reshape(T, H, D), pos, fr) * D ** -0.5
    v = (h @ w[p + "v"].T).reshape(T, H, V)
    decay = np.broadcast_to(np.asarray(mx["decay"], np.float64)[None, :, None], (T, H, D))
    o = rms(linear_recurrence(q, k, v, decay), eps)
    return (o.reshape(T, H * V) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def chunk_visible(T, size):
    """[T, T] bool: key j visible from query i iff j <= i and both lie in the same block of `size` positions (size <= 0: plain causal)"""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    m = j <= i
    if size and size > 0:
        m = m & (i // size == j // size)
    return m


def softmax_attention(q, k, v, scale, visible):
    """q [T, H, D], k [T, G, D], v [T, G, V] -> [T, H, V]; ordinary softmax over the visible keys"""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[-1]))
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * scale
        s = np.where(visible, s, -np.inf)
        s = s - s.max(-1, keepdims=True)
        e = np.exp(s)
        out[:, hd] = (e / e.sum(-1, keepdims=True)) @ v[:, g]
    return out


def branch_chunked_attention(h, mx, w, p, eps):
    T = h.shape[0]
    H, G, D, V = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx.get("vdim", mx["dim"])
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, D)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, V)
    q = rms(q, eps) * w[p + "q.norm"]
    k = rms(k, eps) * w[p + "k.norm"]
    rot = mx.get("rot") or {}
    fr = rotary_freqs(int(rot.get("dims", 0)), float(rot.get("base", 10000.0)), rot.get("scaling")) if rot.get("dims") else np.zeros(0)
    pos = np.arange(T)
    q, k = rotate_half(q, pos, fr), rotate_half(k, pos, fr)
    vis = chunk_visible(T, int((mx.get("mask") or {}).get("size", 0)))
    o = softmax_attention(q, k, v, float(mx["scale"]), vis)
    return o.reshape(T, H * V) @ w[p + "o"].T


def branch_gated_linear(h, mx, w, p, eps):
    """linear attention whose decay per key channel comes from the token: alpha = sigmoid(z)^(1/tau)"""
    T = h.shape[0]
    H, D, V = mx["heads"], mx["dim"], mx.get("vdim", mx["dim"])
    q = (h @ w[p + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).reshape(T, H, D)
    v = (h @ w[p + "v"].T).reshape(T, H, V)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = np.exp(np.log(sigmoid(z)) / float(mx["tau"])).reshape(T, H, D)
    o = rms(linear_recurrence(q, k, v, alpha), eps) * w[p + "norm"][None, None, :]
    return (o.reshape(T, H * V) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def mixer_parallel(h, mx, w, p, eps):
    return float(mx["left_scale"]) * branch_chunked_attention(h, mx["left"], w, p + "left.", eps) + \
        float(mx["right_scale"]) * branch_gated_linear(h, mx["right"], w, p + "right.", eps)


def moe(h, mlp, w, p):
    """router in full precision, the `top` largest logits, softmax over the chosen ones, weighted sum of the experts' outputs"""
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    z = h @ w[p + "router"].T + w[p + "router.b"]
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        pick = np.argsort(-z[t], kind="stable")[:top]
        e = np.exp(z[t, pick] - z[t, pick].max())
        wt = e / e.sum()
        for j, ex in enumerate(pick):
            pe = p + "e%d." % ex
            out[t] += wt[j] * ((silu(h[t] @ w[pe + "gate"].T) * (h[t] @ w[pe + "up"].T)) @ w[pe + "down"].T)
    return out


MIXERS = {"channel_delta": mixer_channel_delta, "retention": mixer_retention, "parallel": mixer_parallel}


def forward(cfg, w, tokens, layers_out=None):
    """logits [T, vocab] of one sequence; layers_out (a list) receives the residual stream after every layer"""
    w = {k: np.asarray(v, np.float64) for k, v in w.items()}
    eps = float(cfg["norm"]["eps"])
    em = cfg["embedding"]
    bg = em["bigram"]
    x = embed_tokens(tokens, w["embed"], w["bigram"], float(em["scale"]), int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"]))
    x = norm1p(x, w["embed.norm"], eps)
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = MIXERS[layer["type"]](norm1p(x, w[p + "norm1"], eps), layer["mixer"], w, p + "mix.", eps)
        x = x + norm1p(m, w[p + "norm1b"], eps)
        if layer.get("mlp"):
            f = moe(norm1p(x, w[p + "norm2"], eps), layer["mlp"], w, p + "mlp.")
            x = x + norm1p(f, w[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return norm1p(x, w["final.norm"], eps) @ w["head"].T


def bf16_round(a):
    """float32 array rounded to bfloat16 (nearest even), returned as float32"""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32).reshape(np.shape(a))


def tensor_shapes(cfg, rank=8):
    """name -> shape of every tensor a model of this config has; `rank` (or a mixer's "rank_a" / "rank_g") sizes the low-rank projections,
    which a config does not carry"""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "bigram": (cfg["embedding"]["bigram"]["buckets"] + 1, W), "embed.norm": (W,), "head": (V, W), "final.norm": (W,)}
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        for n in ("norm1", "norm1b", "norm2", "norm2b") if layer.get("mlp") else ("norm1", "norm1b"):
            out[p + n] = (W,)
        mx, m = layer["mixer"], p + "mix."
        if layer["type"] == "channel_delta":
            H, G, D, Vd = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx.get("vdim", mx["dim"])
            ra, rg, taps = mx.get("rank_a", rank), mx.get("rank_g", rank), mx["conv"]
            out.update({m + "q": (G * D, W), m + "q.conv": (G * D, taps), m + "k": (G * D, W), m + "k.conv": (G * D, taps), m + "v": (H * Vd, W),
                        m + "v.conv": (H * Vd, taps), m + "b": (H, W), m + "A_log": (H,), m + "norm": (Vd,), m + "a1": (ra, W), m + "a2": (H * D, ra),
                        m + "dt_bias": (H * D,), m + "g1": (rg, W), m + "g2": (H * Vd, rg), m + "o": (W, H * Vd)})
        elif layer["type"] == "retention":
            H, D, Vd = mx["heads"], mx["dim"], mx.get("vdim", mx["dim"])
            out.update({m + "q": (H * D, W), m + "k": (H * D, W), m + "v": (H * Vd, W), m + "g": (H * Vd, W), m + "o": (W, H * Vd)})
        else:
            le, ri = mx["left"], mx["right"]
            H, G, D, Vd = le["heads"], le.get("kv_heads", le["heads"]), le["dim"], le.get("vdim", le["dim"])
            out.update({m + "left.q": (H * D, W), m + "left.q.b": (H * D,), m + "left.k": (G * D, W), m + "left.k.b": (G * D,), m + "left.v": (G * Vd, W),
                        m + "left.v.b": (G * Vd,), m + "left.q.norm": (D,), m + "left.k.norm": (D,), m + "left.o": (W, H * Vd)})
            H, D, Vd, ra = ri["heads"], ri["dim"], ri.get("vdim", ri["dim"]), ri.get("rank_a", rank)
            out.update({m + "right.q": (H * D, W), m + "right.k": (H * D, W), m + "right.v": (H * Vd, W), m + "right.g": (H * Vd, W),
                        m + "right.o": (W, H * Vd), m + "right.norm": (Vd,), m + "right.a1": (ra, W), m + "right.a2": (H * D, ra), m + "right.a2.b": (H * D,)})
        if layer.get("mlp"):
            f, E = layer["mlp"]["expert"]["ff"], layer["mlp"]["router"]["experts"]
            out.update({p + "mlp.router": (E, W), p + "mlp.router.b": (E,)})
            for e in range(E):
                out.update({p + "mlp.e%d.gate" % e: (f, W), p + "mlp.e%d.up" % e: (f, W), p + "mlp.e%d.down" % e: (W, f)})
    return out


def random_tensors(cfg, seed, rank=8):
    """bfloat16-representable float32 tensors: projections ~ N(0, 1.5 / sqrt(fan in)), norm weights around zero (plain ones around one),
    decay inputs spread so that some channels forget within a few tokens and others keep hundreds"""
    r = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, rank).items():
        last = name.split(".")[-1]
        if last in ("norm1", "norm1b", "norm2", "norm2b") or name in ("embed.norm", "final.norm"):
            a = 0.2 * r.standard_normal(shape)
        elif last == "norm":
            a = 1.0 + 0.2 * r.standard_normal(shape)
        elif name.endswith("a2.b"):
            a = 2.0 + 2.0 * r.standard_normal(shape)
        elif last == "dt_bias":
            a = -2.0 + 1.5 * r.standard_normal(shape)
        elif last == "A_log":
            a = -1.0 + 0.7 * r.standard_normal(shape)
        elif last == "b" and len(shape) == 1:
            a = 0.3 * r.standard_normal(shape)
        elif last == "conv":
            a = 0.4 * r.standard_normal(shape) + 0.3
        elif name in ("embed", "bigram"):
            a = r.standard_normal(shape)
        else:
            a = 1.5 * r.standard_normal(shape) / math.sqrt(shape[-1])
        out[name] = bf16_round(np.asarray(a, np.float32))
    return out

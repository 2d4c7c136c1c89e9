"""Float64 numpy statement of the Sudosun design: one function per mechanism, a whole sequence at a time, recurrences token by token, no cache, no
pages, no slots.  Shares no code with the product path; the tests compare the engine with it.

A model is (cfg, w): cfg the dict of a config.json of the design, w a dict tensor name -> float64 array.
"""
import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.maximum(z, 0.0) + np.log1p(np.exp(-np.abs(z)))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis"""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def dyt(x, w, name):
    """Dynamic Tanh: a learned slope, a weight and an offset; no statistics of the row"""
    return np.tanh(float(w[name + ".alpha"]) * x) * w[name] + w[name + ".b"]


def causal_conv(x, taps_w, bias=None):
    """x [T, C], taps_w [C, K]: the last column weighs the current token, zeros stand before the sequence"""
    T, C = x.shape
    K = taps_w.shape[1]
    y = np.zeros_like(x)
    for j in range(K):
        back = K - 1 - j
        if back < T:
            y[back:] += x[:T - back] * taps_w[:, j]
    if bias is not None:
        y = y + bias
    return y


# ------------------------------------------------------------------------------------------------ rotary
def rotary_table(rot, positions):
    """-> cos, sin [T, dims / 2] for neighbouring pairs (2i, 2i + 1); YaRN: pairs that turn fewer than `slow` times over the original length are
    slowed down by `factor`, those that turn more than `fast` times are kept, a linear ramp over the pair index lies between; cos and sin grow
    by 0.1 ln(factor) + 1"""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def pair_of(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(pair_of(float(sc["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(sc["slow"]))), dims - 1)
        ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = np.asarray(positions, np.float64)[:, None] * f[None, :]
    return np.cos(ang) * mag, np.sin(ang) * mag


def rotate_pairs(x, cos, sin):
    """x [T, H, dim]; the first 2 * cos.shape[1] dimensions turn, the rest pass"""
    n = cos.shape[1] * 2
    out = x.copy()
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    c, s = cos[:, None, :], sin[:, None, :]
    out[..., 0:n:2] = u * c - v * s
    out[..., 1:n:2] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------------ mixers
def mixer_lightning(h, mx, w, p, eps):
    """linear attention with one constant decay per head: S <- d S + k v^T, o = S^T q; q, k, v through silu"""
    T = h.shape[0]
    H, D, V = int(mx["heads"]), int(mx["dim"]), int(mx.get("vdim", mx["dim"]))
    q = silu(h @ w[p + "q"].T).reshape(T, H, D)
    k = silu(h @ w[p + "k"].T).reshape(T, H, D)
    v = silu(h @ w[p + "v"].T).reshape(T, H, V)
    decay = [float(d) for d in mx["decay"]]
    o = np.zeros((T, H, V))
    for hd in range(H):
        S = np.zeros((D, V))
        for t in range(T):
            S = decay[hd] * S + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = rms(o.reshape(T, H * V), eps) * w[p + "norm"]
    o = o * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def mixer_delta(h, mx, w, p, eps):
    """gated delta rule with one decay per head and token"""
    T = h.shape[0]
    H, G, D, V = int(mx["heads"]), int(mx.get("kv_heads", mx["heads"])), int(mx["dim"]), int(mx.get("vdim", mx["dim"]))
    q = silu(causal_conv(h @ w[p + "q"].T, w[p + "q.conv"])).reshape(T, G, D)
    k = silu(causal_conv(h @ w[p + "k"].T, w[p + "k.conv"])).reshape(T, G, D)
    v = silu(causal_conv(h @ w[p + "v"].T, w[p + "v.conv"])).reshape(T, H, V)
    q = q / np.sqrt(np.sum(q * q, -1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt(np.sum(k * k, -1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ w[p + "b"].T)
    g = np.exp(-np.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    o = np.zeros((T, H, V))
    rep = H // G
    for hd in range(H):
        S = np.zeros((D, V))
        for t in range(T):
            kt, qt = k[t, hd // rep], q[t, hd // rep]
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ kt)
            S = S + np.outer(kt, u)
            o[t, hd] = S.T @ qt
    o = rms(o, eps) * w[p + "norm"]
    o = o.reshape(T, H * V) * silu(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def attention_window_sink(h, mx, w, p, eps, positions):
    """softmax attention over a sliding window with a sink in the denominator, per-head temperature, per-head output gate"""
    T = h.shape[0]
    H, G, D, V = int(mx["heads"]), int(mx.get("kv_heads", mx["heads"])), int(mx["dim"]), int(mx.get("vdim", mx["dim"]))
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, D)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, V)
    q = rms(q, eps) * w[p + "q.norm"]
    k = rms(k, eps) * w[p + "k.norm"]
    rot = mx.get("rot")
    if rot and int(rot.get("dims", 0)) > 0:
        cos, sin = rotary_table(rot, positions)
        q, k = rotate_pairs(q, cos, sin), rotate_pairs(k, cos, sin)
    window = int((mx.get("mask") or {}).get("size", 0))
    pos = np.asarray(positions)
    dist = pos[:, None] - pos[None, :]
    vis = (dist >= 0) & ((dist < window) if window > 0 else True)
    gate = sigmoid(h @ w[p + "g"].T)  # [T, H]
    out = np.zeros((T, H, V))
    rep = H // G
    for hd in range(H):
        s = (q[:, hd] @ k[:, hd // rep].T) * float(mx["scale"]) * w[p + "temp"][hd]
        s = np.where(vis, s, -np.inf)
        sink = w[p + "sink"][hd]
        m = np.maximum(s.max(-1), sink)
        e = np.exp(s - m[:, None])
        den = e.sum(-1) + np.exp(sink - m)
        out[:, hd] = (e / den[:, None]) @ v[:, hd // rep] * gate[:, hd:hd + 1]
    return out.reshape(T, H * V) @ w[p + "o"].T


def gated_linear_unit(h, mx, w, p):
    """two branches: gelu on one, on the other a short convolution and a real-gated diagonal recurrence
    S <- a S + sqrt(1 - a^2) i u,  a = exp(-8 r softplus(lam)),  r and i from block-diagonal sigmoid gates of u"""
    T = h.shape[0]
    C, nb = int(mx["width"]), int(mx["blocks"])
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_conv(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"], w[p + "conv.b"])
    bw = C // nb
    ub = u.reshape(T, nb, bw)
    r = sigmoid(np.einsum("tbi,boi->tbo", ub, w[p + "ra"]) + w[p + "ra.b"]).reshape(T, C)
    i = sigmoid(np.einsum("tbi,boi->tbo", ub, w[p + "ri"]) + w[p + "ri.b"]).reshape(T, C)
    a = np.exp(-8.0 * r * softplus(w[p + "lam"]))
    S = np.zeros(C)
    out = np.zeros((T, C))
    for t in range(T):
        S = a[t] * S + np.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return (out * y) @ w[p + "o"].T


def mixer_parallel(h, mx, w, p, eps, positions):
    left = attention_window_sink(h, mx["left"], w, p + "left.", eps, positions)
    right = gated_linear_unit(h, mx["right"], w, p + "right.")
    return 0.5 * (rms(left, eps) * w[p + "left.out"] + rms(right, eps) * w[p + "right.out"])


# ------------------------------------------------------------------------------------------------ feed-forwards
def ff_dense(h, mlp, w, p):
    lim = float(mlp["limit"])
    g = np.minimum(h @ w[p + "gate"].T, lim)
    u = np.clip(h @ w[p + "up"].T, -lim, lim)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def route(h, router, w, p):
    """-> chosen [T, top] (indices over experts + identity experts), weights [T, top]: softmax over all router outputs; the choice adds a
    correction and is restricted to the groups whose best corrected score is among the `keep` largest; the weights are the plain scores"""
    z = h @ w[p + "router"].T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z)
    s = s / s.sum(-1, keepdims=True)
    c = s + w[p + "correction"]
    n, top = s.shape[1], int(router["top"])
    groups = router.get("groups")
    if groups:
        cnt, keep = int(groups["count"]), int(groups["keep"])
        gs = c.reshape(-1, cnt, n // cnt).max(-1)
        order = np.argsort(-gs, axis=-1, kind="stable")[:, :keep]
        ok = np.zeros_like(gs, bool)
        np.put_along_axis(ok, order, True, -1)
        c = np.where(np.repeat(ok, n // cnt, axis=1), c, -np.inf)
    chosen = np.argsort(-c, axis=-1, kind="stable")[:, :top]
    return chosen, np.take_along_axis(s, chosen, -1)


def ff_moe(h, mlp, w, p):
    router = mlp["router"]
    n_real = int(router["experts"])
    chosen, wt = route(h, router, w, p)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t], wt[t]):
            if e >= n_real:  # an identity expert hands its input back
                out[t] += a * h[t]
            else:
                pe = "%se%d." % (p, e)
                out[t] += a * ((silu(h[t] @ w[pe + "gate"].T) * (h[t] @ w[pe + "up"].T)) @ w[pe + "down"].T)
    return out


# ------------------------------------------------------------------------------------------------ the model
def forward(cfg, w, tokens, return_layers=False):
    """-> logits [T, vocab] (and the residual stream after every layer [L, T, width])"""
    eps = float(cfg["norm"]["eps"])
    tokens = np.asarray(tokens)
    positions = np.arange(len(tokens))
    x = w["embed"][tokens]
    trace = []
    for li, layer in enumerate(cfg["layers"]):
        p = "l%d." % li
        h = dyt(x, w, p + "norm1")
        kind, mx = layer["type"], layer["mixer"]
        if kind == "lightning":
            m = mixer_lightning(h, mx, w, p + "mix.", eps)
        elif kind == "delta":
            m = mixer_delta(h, mx, w, p + "mix.", eps)
        elif kind == "parallel":
            m = mixer_parallel(h, mx, w, p + "mix.", eps, positions)
        else:
            raise ValueError(kind)
        x = x + dyt(m, w, p + "norm1b")
        mlp = layer.get("mlp")
        if mlp:
            h = dyt(x, w, p + "norm2")
            f = ff_moe(h, mlp, w, p + "mlp.") if mlp["kind"] == "moe" else ff_dense(h, mlp, w, p + "mlp.")
            x = x + dyt(f, w, p + "norm2b")
        trace.append(x.copy())
    logits = (dyt(x, w, "final.norm") @ w["embed"].T) * float(cfg.get("logit_scale", 1.0))
    return (logits, np.stack(trace)) if return_layers else logits


def greedy(cfg, w, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(forward(cfg, w, toks)[-1])))
    return toks[len(prompt):]

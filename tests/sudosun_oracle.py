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
def constant_decay_recurrence(q, k, v, decay):
    """q, k [T, H, D], v [T, H, V]: per head S <- decay_h S + k v^T, o = S^T q (the read-out sees the current token's write)"""
    T, H, D = q.shape
    o = np.zeros((T, H, v.shape[-1]))
    for hd in range(H):
        S = np.zeros((D, v.shape[-1]))
        for t in range(T):
            S = decay[hd] * S + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    return o


def delta_rule_recurrence(q, k, v, beta, g):
    """q, k [T, G, D], v [T, H, V], beta, g [T, H]: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q"""
    T, G, D = q.shape
    H, V = v.shape[1], v.shape[2]
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
    return o


def unit(x):
    return x / np.sqrt(np.sum(x * x, -1, keepdims=True) + 1e-6)


def mixer_lightning(h, mx, w, p, eps):
    """linear attention with one constant decay per head: S <- d S + k v^T, o = S^T q; q, k, v through silu"""
    T = h.shape[0]
    H, D, V = int(mx["heads"]), int(mx["dim"]), int(mx.get("vdim", mx["dim"]))
    q = silu(h @ w[p + "q"].T).reshape(T, H, D)
    k = silu(h @ w[p + "k"].T).reshape(T, H, D)
    v = silu(h @ w[p + "v"].T).reshape(T, H, V)
    o = constant_decay_recurrence(q, k, v, [float(d) for d in mx["decay"]])
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
    q, k = unit(q) * D ** -0.5, unit(k)
    beta = sigmoid(h @ w[p + "b"].T)
    g = np.exp(-np.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    o = rms(delta_rule_recurrence(q, k, v, beta, g), eps) * w[p + "norm"]
    o = o.reshape(T, H * V) * silu(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def window_visible(positions, window):
    """[T, T]: query i sees key j iff 0 <= p_i - p_j < window (window 0: every earlier key)"""
    pos = np.asarray(positions)
    dist = pos[:, None] - pos[None, :]
    return (dist >= 0) & ((dist < window) if window > 0 else True)


def softmax_window_sink(q, k, v, head_scale, sink, vis):
    """q [T, H, D], k [T, G, D], v [T, G, V]: scores q . k times head_scale[h]; the denominator also holds exp(sink[h]), which has no value"""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[-1]))
    for hd in range(H):
        g = hd // (H // G)
        s = np.where(vis, (q[:, hd] @ k[:, g].T) * head_scale[hd], -np.inf)
        m = np.maximum(s.max(-1), sink[hd])
        e = np.exp(s - m[:, None])
        out[:, hd] = (e / (e.sum(-1) + np.exp(sink[hd] - m))[:, None]) @ v[:, g]
    return out


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
    out = softmax_window_sink(q, k, v, float(mx["scale"]) * w[p + "temp"], w[p + "sink"], window_visible(positions, window))
    out = out * sigmoid(h @ w[p + "g"].T)[:, :, None]  # one gate per head
    return out.reshape(T, H * V) @ w[p + "o"].T


def gated_diagonal_recurrence(u, r, i, lam):
    """u, r, i [T, C]: a = exp(-8 r softplus(lam)); S <- a S + sqrt(1 - a^2) i u from S = 0, the first token included"""
    a = np.exp(-8.0 * r * softplus(lam))
    S = np.zeros(u.shape[1])
    out = np.zeros_like(u)
    for t in range(u.shape[0]):
        S = a[t] * S + np.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return out


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
    return (gated_diagonal_recurrence(u, r, i, w[p + "lam"]) * y) @ w[p + "o"].T


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
    w = {k: np.asarray(v, np.float64) for k, v in w.items()}
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


# ------------------------------------------------------------------------------------------------ random models for the tests
def bf16_round(a):
    """float32 array rounded to bfloat16 (nearest even), returned as float32"""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32).reshape(np.shape(a))


def tensor_shapes(cfg):
    W = int(cfg["width"])
    out = {"embed": (int(cfg["vocab"]), W)}

    def norm(name):
        out[name], out[name + ".b"], out[name + ".alpha"] = (W,), (W,), ()
    norm("final.norm")
    for li, layer in enumerate(cfg["layers"]):
        p, mx = "l%d." % li, layer["mixer"]
        norm(p + "norm1"), norm(p + "norm1b")
        if layer.get("mlp"):
            norm(p + "norm2"), norm(p + "norm2b")
        m = p + "mix."
        if layer["type"] == "delta":
            H, G, D, V, K = int(mx["heads"]), int(mx.get("kv_heads", mx["heads"])), int(mx["dim"]), int(mx.get("vdim", mx["dim"])), int(mx.get("conv", 1))
            out.update({m + "q": (G * D, W), m + "q.conv": (G * D, K), m + "k": (G * D, W), m + "k.conv": (G * D, K), m + "v": (H * V, W),
                        m + "v.conv": (H * V, K), m + "b": (H, W), m + "a": (H, W), m + "A_log": (H,), m + "dt_bias": (H,), m + "norm": (V,),
                        m + "g": (H * V, W), m + "o": (W, H * V)})
        elif layer["type"] == "lightning":
            H, D, V = int(mx["heads"]), int(mx["dim"]), int(mx.get("vdim", mx["dim"]))
            out.update({m + "q": (H * D, W), m + "k": (H * D, W), m + "v": (H * V, W), m + "g": (H * V, W), m + "o": (W, H * V), m + "norm": (H * V,)})
        else:
            le, ri = mx["left"], mx["right"]
            H, G, D, V = int(le["heads"]), int(le.get("kv_heads", le["heads"])), int(le["dim"]), int(le.get("vdim", le["dim"]))
            C, nb, K = int(ri["width"]), int(ri["blocks"]), int(ri.get("conv", 1))
            a, b = m + "left.", m + "right."
            out.update({a + "q": (H * D, W), a + "q.b": (H * D,), a + "k": (G * D, W), a + "k.b": (G * D,), a + "v": (G * V, W), a + "v.b": (G * V,),
                        a + "q.norm": (D,), a + "k.norm": (D,), a + "temp": (H,), a + "sink": (H,), a + "g": (H, W), a + "o": (W, H * V), a + "out": (W,),
                        b + "y": (C, W), b + "y.b": (C,), b + "x": (C, W), b + "x.b": (C,), b + "conv": (C, K), b + "conv.b": (C,),
                        b + "ra": (nb, C // nb, C // nb), b + "ra.b": (nb, C // nb), b + "ri": (nb, C // nb, C // nb), b + "ri.b": (nb, C // nb),
                        b + "lam": (C,), b + "o": (W, C), b + "out": (W,)})
        mlp = layer.get("mlp")
        f = p + "mlp."
        if mlp and mlp["kind"] == "dense":
            out.update({f + "gate": (int(mlp["ff"]), W), f + "up": (int(mlp["ff"]), W), f + "down": (W, int(mlp["ff"]))})
        elif mlp:
            r, ff = mlp["router"], int(mlp["expert"]["ff"])
            n = int(r["experts"]) + int(r.get("identity", 0))
            out.update({f + "router": (n, W), f + "correction": (n,)})
            for e in range(int(r["experts"])):
                out.update({"%se%d.gate" % (f, e): (ff, W), "%se%d.up" % (f, e): (ff, W), "%se%d.down" % (f, e): (W, ff)})
    return out


def random_tensors(cfg, seed):
    """bfloat16-representable float32 tensors: projections ~ N(0, 1.5 / sqrt(fan in)), norm weights around one with slopes below one, decay
    inputs spread so that some channels forget within a few tokens and others keep hundreds"""
    r = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if last == "alpha":
            a = 0.3 + 0.5 * r.random(shape)
        elif last in ("norm1", "norm1b", "norm2", "norm2b", "norm", "out", "temp") or name == "final.norm":
            a = 1.0 + 0.2 * r.standard_normal(shape)
        elif last == "dt_bias":
            a = -2.0 + 1.5 * r.standard_normal(shape)
        elif last == "A_log":
            a = -1.0 + 0.7 * r.standard_normal(shape)
        elif last == "lam":
            a = -3.0 + 1.5 * r.standard_normal(shape)
        elif last == "sink":
            a = r.standard_normal(shape)
        elif last == "correction":
            a = 0.05 * r.standard_normal(shape)
        elif last == "b" and (len(shape) == 1 or name.endswith(("ra.b", "ri.b"))):
            a = 0.3 * r.standard_normal(shape)
        elif last == "conv":
            a = 0.4 * r.standard_normal(shape) + 0.3
        elif name == "embed":
            a = r.standard_normal(shape)
        elif last == "router":
            a = 3.0 * r.standard_normal(shape) / math.sqrt(shape[-1])
        else:
            a = 1.5 * r.standard_normal(shape) / math.sqrt(shape[-1])
        out[name] = bf16_round(np.asarray(a, np.float32))
    return out

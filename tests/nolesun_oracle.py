"""A plain, slow numpy (float64) implementation of the Nolesun decoder, whole sequences at
a time, one function per mechanism.  It shares no code with the package: the tests compare
the engine (paged cache, state slots, step packing, kernels) against it.

Weights are a dict of float64 arrays under the checkpoint's names; ``cfg`` is the parsed
config.json."""
import numpy as np


def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def silu(x):
    return x / (1.0 + np.exp(-x))


def logistic(x):
    return 1.0 / (1.0 + np.exp(-x))


def softplus(x):
    return np.logaddexp(0.0, x)


def layer_runs(cfg):
    """[(layer, pass number if the run opens a pass of the loop, else None)]."""
    n, lp = len(cfg["layers"]), cfg.get("loop")
    if not lp:
        return [(i, None) for i in range(n)]
    a, b = lp["start"], lp["stop"]
    runs = [(i, None) for i in range(a)]
    for t in range(lp["times"]):
        runs += [(i, t if i == a else None) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, n)]


def short_conv(x, taps, bias=None):
    """x [T, C], taps [C, K]: y[t] = sum_j taps[:, j] * x[t - (K - 1) + j], zeros before 0."""
    T, C = x.shape
    K = taps.shape[1]
    y = np.zeros((T, C))
    for t in range(T):
        for j in range(K):
            s = t - (K - 1) + j
            if s >= 0:
                y[t] += taps[:, j] * x[s]
    return y if bias is None else y + bias


def rotate(x, dims, base, interleaved):
    """x [T, heads, d]: the first ``dims`` dimensions of every head turn with the position."""
    out = x.copy()
    for i in range(dims // 2):
        a, b = (2 * i, 2 * i + 1) if interleaved else (i, i + dims // 2)
        ang = np.arange(x.shape[0]) * base ** (-2.0 * i / dims)
        c, s = np.cos(ang)[:, None], np.sin(ang)[:, None]
        out[..., a] = x[..., a] * c - x[..., b] * s
        out[..., b] = x[..., b] * c + x[..., a] * s
    return out


def attention(h, W, p, m, second):
    """Causal softmax attention with grouped key/value heads.  ``second``: biases, pairs
    (2i, 2i + 1), capped scores and a sigmoid gate on the concatenated heads."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ W[p + "q"].T, h @ W[p + "k"].T, h @ W[p + "v"].T
    if second:
        q, k, v = q + W[p + "q.b"], k + W[p + "k.b"], v + W[p + "v.b"]
    q, k, v = q.reshape(T, H, d), k.reshape(T, G, d), v.reshape(T, G, dv)
    rot = m.get("rot")
    if rot and rot["dims"]:
        q = rotate(q, rot["dims"], rot["base"], second)
        k = rotate(k, rot["dims"], rot["base"], second)
    out = np.zeros((T, H, dv))
    for hd in range(H):
        g = hd // (H // G)
        for t in range(T):
            sc = (k[: t + 1, g] @ q[t, hd]) * m["scale"]
            if second and m.get("softcap"):
                sc = m["softcap"] * np.tanh(sc / m["softcap"])
            w = np.exp(sc - sc.max())
            out[t, hd] = (w / w.sum()) @ v[: t + 1, g]
    o = out.reshape(T, H * dv)
    if second:
        o = o * logistic(h @ W[p + "g"].T)
    y = o @ W[p + "o"].T
    return y + W[p + "o.b"] if second else y


def mamba2(h, W, p, m, eps):
    T = h.shape[0]
    H, V, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * V
    u = h @ W[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner: 2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = silu(short_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, V)
    B = xbc[:, inner: inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    step = softplus(dt + W[p + "dt_bias"])
    rate = np.exp(W[p + "A_log"])
    y = np.zeros((T, H, V))
    for hd in range(H):
        g = hd // (H // G)
        S = np.zeros((N, V))
        for t in range(T):
            S = np.exp(-rate[hd] * step[t, hd]) * S + step[t, hd] * np.outer(B[t, g], x[t, hd])
            y[t, hd] = C[t, g] @ S + W[p + "D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    parts = m.get("norm_groups", 1)
    y = unit_rms(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def gated_delta(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ W[p + "q"].T, W[p + "q.conv"])).reshape(T, G, d)
    k = silu(short_conv(h @ W[p + "k"].T, W[p + "k.conv"])).reshape(T, G, d)
    v = silu(short_conv(h @ W[p + "v"].T, W[p + "v.conv"])).reshape(T, H, dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) / np.sqrt(d)
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    strength = logistic(h @ W[p + "b"].T)
    keep = np.exp(-np.exp(W[p + "A_log"]) * softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    o = np.zeros((T, H, dv))
    for hd in range(H):
        g = hd // (H // G)
        S = np.zeros((d, dv))
        for t in range(T):
            S = keep[t, hd] * S
            u = strength[t, hd] * (v[t, hd] - k[t, g] @ S)
            S = S + np.outer(k[t, g], u)
            o[t, hd] = q[t, g] @ S
    o = unit_rms(o, eps) * W[p + "norm"]
    return (o.reshape(T, H * dv) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def feed_forward(h, W, p, f, margins=None):
    """``margins``: per token, the gap between the last chosen and the first unchosen
    router logit is appended (routed layers)."""
    if f["kind"] == "dense":
        return np.maximum(h @ W[p + "up"].T, 0.0) ** 2 @ W[p + "down"].T
    E, top = f["router"]["experts"], f["router"]["top"]
    logits = h @ W[p + "router"].T + W[p + "router.b"]
    out = np.zeros_like(h)
    gaps = np.full(h.shape[0], np.inf)
    for t in range(h.shape[0]):
        order = np.argsort(-logits[t], kind="stable")
        chosen = order[:top]
        if top < E:
            gaps[t] = logits[t, order[top - 1]] - logits[t, order[top]]
        w = np.exp(logits[t, chosen] - logits[t, chosen].max())
        w /= w.sum()
        for e, we in zip(chosen, w):
            pe = p + "e%d." % e
            a = silu(W[pe + "gate"] @ h[t]) * (W[pe + "up"] @ h[t])
            out[t] += we * (W[pe + "down"] @ a)
    if margins is not None:
        margins.append(gaps)
    return out


def mixer(h, W, p, layer, eps):
    m = layer["mixer"]
    second = layer["type"] == "parallel_2"
    left = attention(h, W, p + "left.", m["left"], second)
    right = (gated_delta if second else mamba2)(h, W, p + "right.", m["right"], eps)
    return m.get("left_scale", 1.0) * left + m.get("right_scale", 1.0) * right


def forward(cfg, W, tokens, taps=None, margins=None):
    """Logits [T, vocab] of a whole sequence.  ``taps``: the residual stream after every
    layer run is appended."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    first = x.copy()
    for i, opens in layer_runs(cfg):
        if opens is not None:
            x = np.concatenate([x, first], axis=-1) @ W["loop.in"].T + W["loop.step"][opens]
        layer, p = cfg["layers"][i], "l%d." % i
        h = unit_rms(x, eps) * (1.0 + W[p + "norm1"])
        y = mixer(h, W, p + "mix.", layer, eps)
        x = x + unit_rms(y, eps) * (1.0 + W[p + "norm1b"]) * W[p + "ls1"]
        if layer.get("mlp"):
            h = unit_rms(x, eps) * (1.0 + W[p + "norm2"])
            y = feed_forward(h, W, p + "mlp.", layer["mlp"], margins)
            x = x + unit_rms(y, eps) * (1.0 + W[p + "norm2b"]) * W[p + "ls2"]
        if taps is not None:
            taps.append(x.copy())
    return (unit_rms(x, eps) * (1.0 + W["final.norm"])) @ W["head"].T

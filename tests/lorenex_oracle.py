"""Plain float64 implementation of the Lorenex decoder, one function per mechanism, whole
sequences at a time.  It shares no code with the package: numpy only, weights as a dict of
float64 arrays under the checkpoint's tensor names, the configuration as the dict that
config.json holds.

  x = embed[token] * embedding.scale + pos[p]
  per layer:  x += m * rms(mixer(x)) * norm1;   x += m * rms(ff(x)) * norm2     (m: residual_mult)
  logits = embed @ (rms(x) * final.norm)
with rms(v) = v / sqrt(mean(v^2) + eps).  The sublayers read x itself.
"""
from __future__ import annotations

import numpy as np


def rms(v, eps):
    return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def causal_conv(u, w, bias=None):
    """u [T, C], w [C, K]: y[t] = sum_j w[:, j] * u[t - (K - 1) + j], zeros before t = 0."""
    T, C = u.shape
    K = w.shape[1]
    pad = np.concatenate([np.zeros((K - 1, C)), u], 0)
    y = np.zeros((T, C))
    for j in range(K):
        y += pad[j:j + T] * w[:, j]
    return y if bias is None else y + bias


# ------------------------------------------------------------------ gated linear attention
def gla_scan(q, k, v, alpha):
    """q, k, alpha [T, H, d], v [T, H, dv]:  S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,
    o_t = S_t^T q_t  ->  [T, H, dv]."""
    T, H, d = q.shape
    S = np.zeros((H, d, v.shape[2]))
    o = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    return o


def gla_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ W[p + "k"].T).reshape(T, H, d)
    v = (h @ W[p + "v"].T).reshape(T, H, dv)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / m["tau"])).reshape(T, H, d)
    o = rms(gla_scan(q, k, v, alpha), eps) * W[p + "norm"]
    return (o.reshape(T, H * dv) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


# ------------------------------------------------------------------ attention beside Mamba
def query_temperature(T, qt):
    """1 + coef * ln(floor((p + 1) / every) + 1) for p < T."""
    if not qt:
        return np.ones(T)
    p = np.arange(T)
    return 1.0 + qt["coef"] * np.log(np.floor((p + 1) / qt["every"]) + 1.0)


def softmax_attention(q, k, v, scale):
    """q [T, H, d], k [T, G, d], v [T, G, dv], causal -> [T, H, dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    o = np.zeros((T, H, v.shape[2]))
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * scale
        s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
        s = np.exp(s - s.max(-1, keepdims=True))
        o[:, hh] = (s / s.sum(-1, keepdims=True)) @ v[:, g]
    return o


def left_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]

    def proj(n):
        u = h @ W[p + n].T + W[p + n + ".b"]
        return causal_conv(u, W[p + n + ".conv"]) if m.get("conv") else u
    q = rms(proj("q").reshape(T, H, d), eps) * query_temperature(T, m.get("q_temp"))[:, None, None]
    k = rms(proj("k").reshape(T, G, d), eps)
    v = rms(proj("v").reshape(T, G, dv), eps)
    return softmax_attention(q, k, v, m["scale"]).reshape(T, H * dv) @ W[p + "o"].T


def selective_scan(x, dt, A, B, C, D):
    """x, dt [T, I], A [I, N], B, C [T, N], D [I]:
    S <- exp(dt A) S + dt x B;  y = S C + D x."""
    T, I = x.shape
    S = np.zeros(A.shape)
    y = np.zeros((T, I))
    for t in range(T):
        S = np.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + D * x[t]
    return y


def right_mixer(h, W, p, m):
    I, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = h @ W[p + "in"].T
    x = silu(causal_conv(xz[:, :I], W[p + "conv"], W[p + "conv.b"]))
    dbc = x @ W[p + "x"].T
    dt = softplus(dbc[:, :R] @ W[p + "dt"].T + W[p + "dt.b"])
    y = selective_scan(x, dt, -np.exp(W[p + "A_log"]), dbc[:, R:R + N], dbc[:, R + N:R + 2 * N],
                       W[p + "D"])
    return (y * silu(xz[:, I:])) @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    return (m.get("left_scale", 1.0) * left_mixer(h, W, p + "left.", m["left"], eps)
            + m.get("right_scale", 1.0) * right_mixer(h, W, p + "right.", m["right"]))


# ------------------------------------------------------------------ feed-forwards
def polynorm_mlp(h, W, p, eps):
    z = h @ W[p + "up"].T
    a, b, c, e = W[p + "act"]
    return (a * rms(z, eps) + b * rms(z ** 2, eps) + c * rms(z ** 3, eps) + e) @ W[p + "down"].T


def route(h, W, p, top, margins=None):
    """-> (weights [T, top], expert ids [T, top]); ids >= experts name identity experts.
    ``margins`` receives, per token, how far the last chosen output's choice score lies above
    the first one left out, relative to the chosen scores' size."""
    z = h @ W[p + "router"].T
    s = np.exp(z - z.max(-1, keepdims=True))
    s = s / s.sum(-1, keepdims=True)
    c = s + W[p + "correction"]
    order = np.argsort(-c, axis=-1, kind="stable")
    ids = order[:, :top]
    if margins is not None and top < c.shape[1]:
        cs = np.take_along_axis(c, order, 1)
        margins.append((cs[:, top - 1] - cs[:, top]) / np.abs(cs[:, :top]).max(-1))
    return np.take_along_axis(s, ids, 1), ids


def expert(h, W, p, limit):
    g = np.minimum(h @ W[p + "gate"].T, limit)
    u = np.clip(h @ W[p + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def moe_mlp(h, W, p, mlp, margins=None):
    E, top, limit = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["limit"]
    w, ids = route(h, W, p, top, margins)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(ids[t, j])
            y = h[t] if e >= E else expert(h[t:t + 1], W, f"{p}e{e}.", limit)[0]
            out[t] += w[t, j] * y
    return out


# ------------------------------------------------------------------ the model
def forward(cfg: dict, W: dict, tokens, taps: list = None, margins: list = None):
    """-> logits [T, vocab]; ``taps`` receives the residual stream after every layer,
    ``margins`` every routed layer's routing margins (see ``route``)."""
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    tokens = np.asarray(tokens)
    T = len(tokens)
    x = W["embed"][tokens] * cfg.get("embedding", {}).get("scale", 1.0) + W["pos"][:T]
    for i, L in enumerate(cfg["layers"]):
        j = i
        while cfg["layers"][j].get("weights_of", j) != j:
            j = cfg["layers"][j]["weights_of"]
        p = f"l{j}."
        if L["type"] == "gla":
            y = gla_mixer(x, W, p + "mix.", L["mixer"], eps)
        elif L["type"] == "parallel":
            y = parallel_mixer(x, W, p + "mix.", L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        x = x + m * rms(y, eps) * W[p + "norm1"]
        mlp = L.get("mlp")
        if mlp:
            y = (polynorm_mlp(x, W, p + "mlp.", eps) if mlp["kind"] == "dense"
                 else moe_mlp(x, W, p + "mlp.", mlp, margins))
            x = x + m * rms(y, eps) * W[p + "norm2"]
        if taps is not None:
            taps.append(x.copy())
    return (rms(x, eps) * W["final.norm"]) @ W["embed"].T


# ------------------------------------------------------------------ random models for tests
def random_weights(cfg: dict, seed: int = 0, bf16=True) -> dict:
    """Random weights under the checkpoint's names, rounded to bfloat16 values (as float64
    arrays) so that a bf16 and an fp32 engine load exactly what the oracle uses."""
    rng = np.random.default_rng(seed)
    Wd, V = cfg["width"], cfg["vocab"]
    out = {}

    def put(name, *shape, std=None, base=0.0):
        a = rng.standard_normal(shape) * (std if std is not None else shape[-1] ** -0.5) + base
        if bf16:
            b = a.astype(np.float32).view(np.uint32)
            b = ((b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
            a = b.view(np.float32).astype(np.float64)
        out[name] = a
    put("embed", V, Wd, std=0.3)
    put("pos", cfg["max_positions"], Wd, std=0.3)
    put("final.norm", Wd, std=0.1, base=1.0)
    for i, L in enumerate(cfg["layers"]):
        if "weights_of" in L:
            continue
        p, m = f"l{i}.", L["mixer"]
        put(p + "norm1", Wd, std=0.1, base=1.0)
        if L["type"] == "gla":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            r = m.get("_rank", 8)
            put(p + "mix.q", H * d, Wd)
            put(p + "mix.k", H * d, Wd)
            put(p + "mix.v", H * dv, Wd)
            put(p + "mix.g", H * dv, Wd)
            put(p + "mix.o", Wd, H * dv)
            put(p + "mix.norm", dv, std=0.1, base=1.0)
            put(p + "mix.a1", r, Wd)
            put(p + "mix.a2", H * d, r, std=1.0)
            put(p + "mix.a2.b", H * d, std=1.0, base=2.0)
        else:
            l, rr = m["left"], m["right"]
            H, G, d, dv = l["heads"], l.get("kv_heads", l["heads"]), l["dim"], l["vdim"]
            for n, c in (("q", H * d), ("k", G * d), ("v", G * dv)):
                put(p + f"mix.left.{n}", c, Wd)
                put(p + f"mix.left.{n}.b", c, std=0.3)
                if l.get("conv"):
                    put(p + f"mix.left.{n}.conv", c, l["conv"], std=0.5)
            put(p + "mix.left.o", Wd, H * dv)
            I, N, R = rr["inner"], rr["state"], rr["dt_rank"]
            put(p + "mix.right.in", 2 * I, Wd)
            put(p + "mix.right.conv", I, rr["conv"], std=0.5)
            put(p + "mix.right.conv.b", I, std=0.3)
            put(p + "mix.right.x", R + 2 * N, I)
            put(p + "mix.right.dt", I, R)
            put(p + "mix.right.dt.b", I, std=0.5, base=-2.0)
            out[p + "mix.right.A_log"] = np.log(1.0 + 7.0 * rng.random((I, N)))
            if bf16:
                a = out[p + "mix.right.A_log"].astype(np.float32).view(np.uint32)
                out[p + "mix.right.A_log"] = (a & 0xFFFF0000).astype(np.uint32).view(
                    np.float32).astype(np.float64)
            put(p + "mix.right.D", I, std=0.3, base=1.0)
            put(p + "mix.right.o", Wd, I)
        mlp = L.get("mlp")
        if not mlp:
            continue
        put(p + "norm2", Wd, std=0.1, base=1.0)
        if mlp["kind"] == "dense":
            put(p + "mlp.up", mlp["ff"], Wd)
            put(p + "mlp.down", Wd, mlp["ff"])
            put(p + "mlp.act", 4, std=0.5)
        else:
            E, I2 = mlp["router"]["experts"], mlp["router"].get("identity", 0)
            ff = mlp["expert"]["ff"]
            for e in range(E):
                put(p + f"mlp.e{e}.gate", ff, Wd, std=2.0 * Wd ** -0.5)
                put(p + f"mlp.e{e}.up", ff, Wd, std=2.0 * Wd ** -0.5)
                put(p + f"mlp.e{e}.down", Wd, ff)
            put(p + "mlp.router", E + I2, Wd, std=2.0 * Wd ** -0.5)
            put(p + "mlp.correction", E + I2, std=0.05)
    return out

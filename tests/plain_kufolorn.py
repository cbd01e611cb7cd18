"""The Kufolorn decoder written plainly: NumPy float64, whole sequences, no cache, no batches, one
function per mechanism, each from its equations.  It shares no code with the package; the tests compare
the engine with it.

Notation: T tokens, W the model's width.  Weights are a dict name -> array, linear weights [out, in],
applied as y = x @ w.T.  `cfg` is the parsed config.json.
"""
import math

import numpy as np


def silu(z):
    return z / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def offset_norm(x, w, eps):
    """The layers' norm: the weight is stored around zero, y = rms(x) * (1 + w)."""
    return rms(x, eps) * (1.0 + w)


# ------------------------------------------------------------------------------------------ rotation
def rotate_half(x, positions, rot):
    """x [T, heads, d]: column i of the first rot.dims columns is paired with column i + dims/2 and the pair
    turned by the angle p * base^(-2i/dims) / factor; the other columns pass."""
    dims, base = rot["dims"], rot["base"]
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    half = dims // 2
    out = x.copy()
    for i in range(half):
        f = base ** (-2.0 * i / dims) / factor
        a = np.asarray(positions, dtype=np.float64) * f
        c, s = np.cos(a)[:, None], np.sin(a)[:, None]
        u, v = x[:, :, i], x[:, :, i + half]
        out[:, :, i] = u * c - v * s
        out[:, :, i + half] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------ delta rule
def causal_conv(u, w):
    """u [T, C]; w [C, taps], the last column multiplies the current token; zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    out = np.zeros((T, C))
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                out[t] += w[:, j] * u[src]
    return out


def unit(x):
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + 1e-6)


def delta_rule(q, k, v, beta, g):
    """q, k [T, heads, dim], v [T, heads, vdim], beta, g [T, heads].  Per head: S <- g S; u = beta (v - S^T k);
    S <- S + k u^T; o = S^T q."""
    T, H, D = q.shape
    V = v.shape[2]
    out = np.zeros((T, H, V))
    for h in range(H):
        S = np.zeros((D, V))
        for t in range(T):
            S = g[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, h])
            S = S + np.outer(k[t, h], u)
            out[t, h] = S.T @ q[t, h]
    return out


def delta_mixer(h, w, p, m, eps):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ w[p + "q"].T, w[p + "q.conv"])).reshape(T, G, D)
    k = silu(causal_conv(h @ w[p + "k"].T, w[p + "k.conv"])).reshape(T, G, D)
    v = silu(causal_conv(h @ w[p + "v"].T, w[p + "v.conv"])).reshape(T, H, V)
    q = unit(q) * D ** -0.5
    k = unit(k)
    rep = H // G
    q = np.repeat(q, rep, axis=1)
    k = np.repeat(k, rep, axis=1)
    beta = sigmoid(h @ w[p + "b"].T)
    g = np.exp(-np.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    o = delta_rule(q, k, v, beta, g)
    o = rms(o, eps) * w[p + "norm"]
    o = o.reshape(T, H * V) * silu(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


# ------------------------------------------------------------------------------------------ attention with a sink
def sink_attention(h, w, p, m, eps, positions):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[p + "q"].T + w[p + "q.b"]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, V)
    q = (rms(q, eps) * w[p + "q.norm"]).reshape(T, H, D)
    k = (rms(k, eps) * w[p + "k.norm"]).reshape(T, G, D)
    q = rotate_half(q, positions, m["rot"])
    k = rotate_half(k, positions, m["rot"])
    gate = sigmoid(h @ w[p + "g"].T)                       # [T, H]
    out = np.zeros((T, H, V))
    for hd in range(H):
        kv = hd // (H // G)
        for t in range(T):
            s = (k[:t + 1, kv] @ q[t, hd]) * m["scale"]
            sk = w[p + "sink"][hd]
            mx = max(s.max(), sk)
            e = np.exp(s - mx)
            out[t, hd] = (e @ v[:t + 1, kv]) / (e.sum() + math.exp(sk - mx))
    out = out * gate[:, :, None]
    return out.reshape(T, H * V) @ w[p + "o"].T


# ------------------------------------------------------------------------------------------ retention
def retention(h, w, p, m, eps, positions):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = rotate_half((h @ w[p + "q"].T).reshape(T, H, D), positions, m["rot"])
    k = rotate_half((h @ w[p + "k"].T).reshape(T, H, D), positions, m["rot"]) * D ** -0.5
    v = (h @ w[p + "v"].T).reshape(T, H, V)
    out = np.zeros((T, H, V))
    for hd in range(H):
        S = np.zeros((D, V))
        for t in range(T):
            S = m["decay"][hd] * S + np.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.T @ q[t, hd]
    out = rms(out, eps).reshape(T, H * V) * silu(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps, positions):
    return (m["left_scale"] * sink_attention(h, w, p + "left.", m["left"], eps, positions)
            + m["right_scale"] * retention(h, w, p + "right.", m["right"], eps, positions))


# ------------------------------------------------------------------------------------------ feed-forward
def dense_ff(h, w, p):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def expert(h, w, p, limit):
    g = np.minimum(h @ w[p + "gate"].T, limit)
    u = np.clip(h @ w[p + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def route(h, w, p, r, margins=None):
    """(chosen router outputs [T, top], their weights [T, top]).  Router outputs experts .. experts + identity - 1
    are identity experts.  `margins`, a list, receives per token by how much the last chosen output's choice score
    beats the best one that is not chosen (infinity where every allowed output is chosen)."""
    n = r["experts"] + r.get("identity", 0)
    z = h @ w[p + "router"].T
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    s = e / e.sum(axis=-1, keepdims=True)
    choice = s + w[p + "correction"]
    groups = r.get("groups")
    if groups and groups["count"] > 1:
        per = n // groups["count"]
        gs = choice.reshape(-1, groups["count"], per).max(axis=-1)
        kept = np.argsort(-gs, axis=-1, kind="stable")[:, :groups["keep"]]
        mask = np.full_like(choice, -np.inf)
        for t in range(h.shape[0]):
            for gi in kept[t]:
                mask[t, gi * per:(gi + 1) * per] = 0.0
        choice = choice + mask
    order = np.argsort(-choice, axis=-1, kind="stable")
    idx = order[:, :r["top"]]
    if margins is not None:
        ranked = np.take_along_axis(choice, order, axis=-1)
        margins.append(ranked[:, r["top"] - 1] - ranked[:, r["top"]] if r["top"] < n else np.full(h.shape[0], np.inf))
    return idx, np.take_along_axis(s, idx, axis=-1)


def moe_ff(h, w, p, mlp, margins=None):
    r = mlp["router"]
    idx, wt = route(h, w, p, r, margins)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t], wt[t]):
            if e >= r["experts"]:
                out[t] += a * h[t]
            else:
                out[t] += a * expert(h[t:t + 1], w, p + f"e{e}.", mlp["expert"]["limit"])[0]
    return out


# ------------------------------------------------------------------------------------------- model
def forward(cfg, w, ids, taps=None, margins=None):
    """Logits [T, vocab] of a whole sequence.  `taps`, a list, receives the stream after every layer; `margins`, a
    list, an array [T] for every routed layer: how clear each token's choice of experts was (see `route`)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(ids)]
    positions = np.arange(len(ids))
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        if L["type"] == "delta":
            y = delta_mixer(x, w, p + "mix.", L["mixer"], eps)
        elif L["type"] == "parallel":
            y = parallel_mixer(x, w, p + "mix.", L["mixer"], eps, positions)
        else:
            raise ValueError(L["type"])
        x = x + offset_norm(y, w[p + "norm1"], eps)
        mlp = L.get("mlp")
        if mlp is not None:
            y = dense_ff(x, w, p + "mlp.") if mlp["kind"] == "dense" else moe_ff(x, w, p + "mlp.", mlp, margins)
            x = x + offset_norm(y, w[p + "norm2"], eps)
        if taps is not None:
            taps.append(x.copy())
    return head(cfg, w, x)


def head(cfg, w, x):
    logits = offset_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["embed"].T
    cap = cfg.get("logit_softcap") or 0.0
    return cap * np.tanh(logits / cap) if cap else logits

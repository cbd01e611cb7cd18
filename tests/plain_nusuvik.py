"""The Nusuvik decoder written plainly: NumPy float64, whole sequences, no cache, no batches, one
function per mechanism, each from its equations.  It shares no code with the package; the tests compare
the engine with it.

Notation: T tokens, W the model's width.  Weights are a dict name -> array, linear weights [out, in],
applied as y = x @ w.T.  `cfg` is the parsed config.json.
"""
import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def layer_norm(x, w, b, eps):
    """(x - mean) / sqrt(mean of squared deviations + eps) * w + b over the last axis."""
    m = np.mean(x, axis=-1, keepdims=True)
    d = x - m
    return d / np.sqrt(np.mean(d * d, axis=-1, keepdims=True) + eps) * w + b


# --------------------------------------------------------------------------------------- embedding
def bigram_rows(ids, buckets, mul_prev, mul_cur):
    """Row of the bigram table for every token: the last row (number `buckets`) for a sequence's first
    token, else (previous * mul_prev + token * mul_cur) mod buckets."""
    rows = []
    for t, tok in enumerate(ids):
        rows.append(buckets if t == 0 else (int(ids[t - 1]) * mul_prev + int(tok) * mul_cur) % buckets)
    return rows


def embed(ids, W, cfg):
    x = W["embed"][np.asarray(ids)]
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        x = x + W["bigram"][bigram_rows(ids, bg["buckets"], bg["mul_prev"], bg["mul_cur"])]
    return x


# ---------------------------------------------------------------------------------------- rotation
def rotate_half(v, positions, base, dims):
    """v [T, n >= dims]: column i < dims/2 is paired with column i + dims/2; the pair (a, b) at position p
    becomes (a cos t - b sin t, b cos t + a sin t), t = p * base^(-2i/dims).  Columns from `dims` on pass."""
    out = np.array(v, dtype=np.float64)
    half = dims // 2
    for r, p in enumerate(positions):
        for i in range(half):
            t = p * base ** (-2.0 * i / dims)
            a, b = v[r, i], v[r, i + half]
            out[r, i] = a * math.cos(t) - b * math.sin(t)
            out[r, i + half] = b * math.cos(t) + a * math.sin(t)
    return out


# ----------------------------------------------------------------------------------------- mixer
def latent_attention(h, W, p, m, eps):
    """h [T, W]; p the tensors' prefix ('l3.mix.'); m the mixer's configuration."""
    T = h.shape[0]
    H, dn, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    pos = np.arange(T)
    cq = rms(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (cq @ W[p + "uq"].T).reshape(T, H, dn + dr)
    down = h @ W[p + "dkv"].T
    c = rms(down[:, :rank], eps) * W[p + "dkv.norm"]
    k_rot = rotate_half(down[:, rank:], pos, base, dims)
    k_plain = (c @ W[p + "uk"].T).reshape(T, H, dn)
    v = (c @ W[p + "uv"].T).reshape(T, H, dv)
    gate = sigmoid(h @ W[p + "g"].T)                       # [T, H]
    out = np.zeros((T, H, dv))
    for hd in range(H):
        q_plain = q[:, hd, :dn]
        q_rot = rotate_half(q[:, hd, dn:], pos, base, dims)
        for i in range(T):
            s = (k_plain[:i + 1, hd] @ q_plain[i] + k_rot[:i + 1] @ q_rot[i]) * m["scale"]
            w = np.exp(s - s.max())
            w = w / w.sum()
            out[i, hd] = (w @ v[:i + 1, hd]) * gate[i, hd]
    return out.reshape(T, H * dv) @ W[p + "o"].T


# ---------------------------------------------------------------------------------- feed-forward
def dense_mlp(h, W, p):
    u = h @ W[p + "up"].T + W[p + "up.b"]
    return gelu_tanh(u) @ W[p + "down"].T + W[p + "down.b"]


def route(h, W, p, r):
    """Per token: (chosen experts, their weights).  Scores s = sigmoid(router logits); the choice uses
    s + correction, restricted to the best groups; the weights use s alone, normalised."""
    E, top = r["experts"], r["top"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    G, keep = groups["count"], groups["keep"]
    per = E // G
    s = sigmoid(h @ W[p + "router"].T)
    choice = s + W[p + "correction"]
    picks, weights = [], []
    for t in range(h.shape[0]):
        gs = [np.sort(choice[t, g * per:(g + 1) * per])[::-1][:2].sum() for g in range(G)]
        best = sorted(range(G), key=lambda g: (-gs[g], g))[:keep]
        allowed = [e for e in range(E) if e // per in best]
        chosen = sorted(allowed, key=lambda e: (-choice[t, e], e))[:top]
        w = np.array([s[t, e] for e in chosen])
        picks.append(chosen)
        weights.append(w / (w.sum() + 1e-20))
    return picks, weights


def expert(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def moe_mlp(h, W, p, mlp):
    picks, weights = route(h, W, p, mlp["router"])
    out = np.zeros((h.shape[0], W[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, w in zip(picks[t], weights[t]):
            out[t] += w * expert(h[t:t + 1], W, f"{p}e{e}.")[0]
    return out


# ------------------------------------------------------------------------------------------ model
def layer(x, W, i, L, eps):
    """Both sublayers read one norm: x + (mixer(h) + ff(h)), h = norm1(x)."""
    p = f"l{i}."
    h = layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps)
    y = latent_attention(h, W, p + "mix.", L["mixer"], eps)
    mlp = L.get("mlp")
    if mlp is not None:
        y = y + (dense_mlp(h, W, p + "mlp.") if mlp["kind"] == "dense" else moe_mlp(h, W, p + "mlp.", mlp))
    return x + y


def layer_runs(cfg):
    """The order in which layers run: (layer, first of a pass?) with layers start..stop-1 `times` times."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["stop"] <= loop["start"]:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(loop["start"])]
    for _ in range(loop["times"]):
        runs += [(i, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, False) for i in range(loop["stop"], n)]


def forward(ids, W, cfg, streams=None):
    """Logits [T, vocab] of one whole sequence.  `streams`: a list that takes the stream after every layer run."""
    eps = cfg["norm"]["eps"]
    x0 = embed(ids, W, cfg)
    x = x0
    for i, enters in layer_runs(cfg):
        if enters:
            x = np.concatenate([x, x0], axis=1) @ W["loop.in"].T
        x = layer(x, W, i, cfg["layers"][i], eps)
        if streams is not None:
            streams.append(x.copy())
    z = layer_norm(x, W["final.norm"], W["final.norm.b"], eps) @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * np.tanh(z / cap) if cap else z

"""Plain, slow restatement of the Fekotar decoder, one function per mechanism (test infrastructure only: nothing under
aphrodite_engine_amd/ imports this, and this imports nothing from there).  float64 numpy, no cache: every call recomputes a
whole sequence, and the attention materialises every head's keys and values from the latent.

Notation: x [T, W] is the residual stream of one sequence, positions 0 .. T-1.  Weights come as a dict name -> array, named as
in the checkpoint; the configuration is the checkpoint's config.json as a dict."""
import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w


def pair_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the pair table for every position: a hash of (previous token, token); the first position takes row `buckets`."""
    return [buckets] + [(int(tokens[i - 1]) * mul_prev + int(tokens[i]) * mul_cur) % buckets for i in range(1, len(tokens))]


def embed(tokens, table, pair_table, hashing):
    x = table[np.asarray(tokens)]
    if hashing is None:
        return x
    return x + pair_table[pair_rows(tokens, hashing["buckets"], hashing["mul_prev"], hashing["mul_cur"])]


def rotary_frequencies(rot):
    """(f [dims / 2], factor on cos and sin).  With scaling: number(t) = dims ln(original / (2 pi t)) / (2 ln base) is the
    (fractional) index that turns t times over the original length; between number(fast) and number(slow) a ramp goes from the
    original frequency to the one divided by `factor`."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    number = lambda t: dims * math.log(sc["original"] / (2 * math.pi * t)) / (2 * math.log(base))
    lo, hi = max(math.floor(number(sc["fast"])), 0), min(math.ceil(number(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(x, positions, rot):
    """x [T, ..., n]: the first rot.dims numbers of the last axis are turned, number i with number i + dims / 2."""
    dims = int(rot["dims"])
    f, mult = rotary_frequencies(rot)
    half = dims // 2
    a = np.asarray(positions, np.float64)[:, None] * f[None]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (half,)
    cos, sin = (np.cos(a) * mult).reshape(shape), (np.sin(a) * mult).reshape(shape)
    u, v = x[..., :half], x[..., half:dims]
    return np.concatenate([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], -1)


def latent_attention(h, W, p, mc, eps):
    """The mixer of one layer on a whole sequence; p is the tensor prefix ('l3.mix.')."""
    T = h.shape[0]
    H, d, r, e, R = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
    pos = np.arange(T)
    cq = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).reshape(T, H, d + r)
    down = h @ W[p + "dkv"].T
    c = rms_norm(down[:, :R], W[p + "dkv.norm"], eps)
    k_rot = rotate(down[:, R:], pos, mc["rot"])                       # one per token, shared by the heads
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], pos, mc["rot"])
    k_plain = (c @ W[p + "uk"].T).reshape(T, H, d)
    v = (c @ W[p + "uv"].T).reshape(T, H, e)
    out = np.zeros((T, H, e))
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * mc["scale"]
        for i in range(T):
            w = np.exp(s[i, :i + 1] - s[i, :i + 1].max())
            out[i, a] = (w / w.sum()) @ v[:i + 1, a]
    gated = out.reshape(T, H * e) * sigmoid(h @ W[p + "g"].T)
    return gated @ W[p + "o"].T


def dense_ff(h, W, p, mlp):
    lim = mlp["limit"]
    g = np.minimum(h @ W[p + "gate"].T + W[p + "gate.b"], lim)
    u = np.clip(h @ W[p + "up"].T + W[p + "up.b"], -lim, lim)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T + W[p + "down.b"]


def route(z, top, groups, keep, scale):
    """z [experts] router outputs of one token -> (chosen experts, their weights)."""
    s = sigmoid(z)
    E = len(s)
    per = E // groups
    group_score = [np.sort(s[g * per:(g + 1) * per])[-2:].sum() for g in range(groups)]
    kept = sorted(range(groups), key=lambda g: (-group_score[g], g))[:keep]
    allowed = [j for j in range(E) if j // per in kept]
    chosen = sorted(allowed, key=lambda j: (-s[j], j))[:top]
    return chosen, [s[j] * scale for j in chosen]


def moe_ff(h, W, p, mlp):
    r = mlp["router"]
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        chosen, weights = route(W[p + "router"] @ h[t], r["top"], r["groups"]["count"], r["groups"]["keep"], r.get("scale", 1.0))
        for j, w in zip(chosen, weights):
            e = f"{p}e{j}."
            a = W[e + "gate"] @ h[t]
            out[t] += w * (W[e + "down"] @ (a * sigmoid(a) * (W[e + "up"] @ h[t])))
    return out


def forward(cfg, W, tokens, trace=None):
    """Logits [T, vocab] of one sequence; ``trace`` (a list) receives the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    hashing = (cfg.get("embedding") or {}).get("bigram")
    x = embed(tokens, W["embed"], W.get("bigram"), hashing).astype(np.float64)
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_norm(x, W[p + "norm1"], eps)
        y = latent_attention(h, W, p + "mix.", lc["mixer"], eps)
        mlp = lc.get("mlp")
        if mlp is not None:
            y = y + (dense_ff(h, W, p + "mlp.", mlp) if mlp["kind"] == "dense" else moe_ff(h, W, p + "mlp.", mlp))
        x = x + y
        if trace is not None:
            trace.append(x.copy())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T * cfg.get("logit_scale", 1.0)

"""Plain, slow restatement of the Pagulix decoder, one function per mechanism (test infrastructure only: nothing under
aphrodite_engine_amd/ imports this, and this imports nothing from there).  float64 numpy, no cache: every call recomputes a
whole sequence token by token; the latent attention materialises every head's keys and values from the latent.

Notation: x [T, W] is one residual stream of one sequence, positions 0 .. T-1.  Weights come as a dict name -> array, named as
in the checkpoint; the configuration is the checkpoint's config.json as a dict."""
import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis (w None: no weight)."""
    y = x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)
    return y if w is None else y * w


# ---- rotation --------------------------------------------------------------------------------------------------------------
def rotary_frequencies(rot):
    """f_i = base^(-2 i / dims), i < dims / 2; with `scaling` (factor, low, high, original) every frequency whose wavelength
    l = 2 pi / f is longer than original / low is divided by factor, one whose wavelength is shorter than original / high is
    kept, and between the two s = (original / l - low) / (high - low) blends (1 - s) f / factor + s f."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f
    out = f.copy()
    for i, fi in enumerate(f):
        wave = 2.0 * math.pi / fi
        if wave < sc["original"] / sc["high"]:
            continue
        if wave > sc["original"] / sc["low"]:
            out[i] = fi / sc["factor"]
        else:
            s = (sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])
            out[i] = (1.0 - s) * fi / sc["factor"] + s * fi
    return out


def rotate(x, positions, rot, layout):
    """x [T, ..., n]: the first rot.dims numbers of the last axis are turned by position * f_i; layout "half" pairs number i
    with number i + dims / 2, layout "interleaved" pairs number 2 i with number 2 i + 1."""
    dims = int(rot["dims"])
    f = rotary_frequencies(rot)
    a = np.asarray(positions, np.float64)[:, None] * f[None]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (dims // 2,)
    cos, sin = np.cos(a).reshape(shape), np.sin(a).reshape(shape)
    out = x.copy()
    if layout == "half":
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2], out[..., dims // 2:dims] = u * cos - v * sin, v * cos + u * sin
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2], out[..., 1:dims:2] = u * cos - v * sin, v * cos + u * sin
    return out


# ---- softmax attention over visible keys, with an optional window and sink ---------------------------------------------------
def masked_attention(q, k, v, scale, window=0, sink=None):
    """q [T, d], k [T, d], v [T, e] of one head.  Row i sees j <= i, and with a window only i - j < window.  `sink`: a number
    whose exponential joins the denominator (no key, no value, not scaled)."""
    T = q.shape[0]
    out = np.zeros((T, v.shape[1]))
    for i in range(T):
        lo = max(0, i - window + 1) if window else 0
        s = (k[lo:i + 1] @ q[i]) * scale
        m = s.max() if sink is None else max(s.max(), sink)
        w = np.exp(s - m)
        den = w.sum() + (0.0 if sink is None else math.exp(sink - m))
        out[i] = (w / den) @ v[lo:i + 1]
    return out


def attention(h, W, p, mc, eps, v_first=None):
    """Grouped-query attention with a rotation of the first rot.dims numbers of every head ("half" layout), unit RMS of q and k
    after the rotation, and values blended with `v_first` (the first value-mixing layer's values) by the layer's lambda.
    Returns (output, this layer's values as cached)."""
    T = h.shape[0]
    H, G, d, e = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    pos = np.arange(T)
    q = rotate((h @ W[p + "q"].T).reshape(T, H, d), pos, mc["rot"], "half")
    k = rotate((h @ W[p + "k"].T).reshape(T, G, d), pos, mc["rot"], "half")
    q, k = rms_norm(q, None, eps), rms_norm(k, None, eps)
    v = (h @ W[p + "v"].T).reshape(T, G, e)
    if mc.get("v_mix") and v_first is not None:
        lam = float(W[p + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    out = np.zeros((T, H, e))
    for a in range(H):
        g = a // (H // G)
        out[:, a] = masked_attention(q[:, a], k[:, g], v[:, g], mc["scale"])
    return out.reshape(T, H * e) @ W[p + "o"].T, v


def latent_attention(h, W, p, mc, eps):
    """Keys and values as products of a normed latent c; one rotated key part shared by all heads ("interleaved" layout);
    sliding window; a per-head sink in the softmax denominator."""
    T = h.shape[0]
    H, d, r, e, R = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
    pos = np.arange(T)
    q = (h @ W[p + "q"].T).reshape(T, H, d + r)
    down = h @ W[p + "dkv"].T
    c = rms_norm(down[:, :R], W[p + "dkv.norm"], eps)
    k_rot = rotate(down[:, R:], pos, mc["rot"], "interleaved")
    q_rot = rotate(q[..., d:], pos, mc["rot"], "interleaved")
    k_plain = (c @ W[p + "uk"].T).reshape(T, H, d)
    v = (c @ W[p + "uv"].T).reshape(T, H, e)
    window = int((mc.get("mask") or {}).get("size", 0))
    out = np.zeros((T, H, e))
    for a in range(H):
        qa = np.concatenate([q[:, a, :d], q_rot[:, a]], -1)
        ka = np.concatenate([k_plain[:, a], k_rot], -1)
        sink = float(W[p + "sink"][a]) if p + "sink" in W else None
        out[:, a] = masked_attention(qa, ka, v[:, a], mc["scale"], window, sink)
    return out.reshape(T, H * e) @ W[p + "o"].T


# ---- gated delta rule ------------------------------------------------------------------------------------------------------
def causal_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_{t - taps + 1 + j}, zeros before the sequence."""
    T, taps = u.shape[0], w.shape[1]
    pad = np.concatenate([np.zeros((taps - 1, u.shape[1])), u], 0)
    return sum(pad[j:j + T] * w[:, j] for j in range(taps))


def delta_rule(q, k, v, beta, g):
    """One head: q, k [T, d], v [T, e], beta, g [T].  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, d = q.shape
    S = np.zeros((d, v.shape[1]))
    out = np.zeros_like(v)
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def delta_mixer(h, W, p, mc, eps):
    T = h.shape[0]
    H, G, d, e = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    q = silu(causal_conv(h @ W[p + "q"].T, W[p + "q.conv"])).reshape(T, G, d)
    k = silu(causal_conv(h @ W[p + "k"].T, W[p + "k.conv"])).reshape(T, G, d)
    v = silu(causal_conv(h @ W[p + "v"].T, W[p + "v.conv"])).reshape(T, H, e)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * d ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ W[p + "b"].T)
    g = np.exp(-np.exp(W[p + "A_log"]) * softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    gate = silu(h @ W[p + "g"].T).reshape(T, H, e)
    out = np.zeros((T, H, e))
    for a in range(H):
        j = a // (H // G)
        out[:, a] = delta_rule(q[:, j], k[:, j], v[:, a], beta[:, a], g[:, a])
    out = rms_norm(out, W[p + "norm"], eps) * gate
    return out.reshape(T, H * e) @ W[p + "o"].T


# ---- feed-forward ----------------------------------------------------------------------------------------------------------
def glu(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(z, top):
    """z [experts] router logits of one token -> (chosen experts, softmax over the chosen logits).  Ties go to the lower index."""
    chosen = sorted(range(len(z)), key=lambda j: (-z[j], j))[:top]
    w = np.exp(z[chosen] - z[chosen].max())
    return chosen, w / w.sum()


def moe_ff(h, W, p, mlp):
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        z = W[p + "router"] @ h[t] + W[p + "router.b"]
        chosen, weights = route(z, mlp["router"]["top"])
        for j, w in zip(chosen, weights):
            out[t] += w * glu(h[t:t + 1], W, f"{p}e{j}.")[0]
    if mlp.get("shared"):
        out = out + glu(h, W, p + "shared.")
    return out


# ---- the stack -------------------------------------------------------------------------------------------------------------
def forward(cfg, W, tokens, trace=None):
    """Logits [T, vocab] of one sequence; ``trace`` (a list) receives the sum of the streams after every layer."""
    eps, m, n = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0), int(cfg.get("streams", 1))
    x0 = W["embed"][np.asarray(tokens)].astype(np.float64)
    xs = [x0.copy() for _ in range(n)]
    v_first = None
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        for q in (1, 2):
            if q == 2 and lc.get("mlp") is None:
                continue
            hc = f"{p}hc{q}."
            u = sum(W[hc + "in"][s] * xs[s] for s in range(n)) if hc + "in" in W else xs[0]
            hin = rms_norm(u, W[f"{p}norm{q}"], eps)
            if q == 2:
                y = moe_ff(hin, W, p + "mlp.", lc["mlp"])
            elif lc["type"] == "delta":
                y = delta_mixer(hin, W, p + "mix.", lc["mixer"], eps)
            elif lc["type"] == "latent_attention":
                y = latent_attention(hin, W, p + "mix.", lc["mixer"], eps)
            else:
                y, v = attention(hin, W, p + "mix.", lc["mixer"], eps, v_first)
                if lc["mixer"].get("v_mix") and v_first is None:
                    v_first = v
            if f"{p}ls{q}" in W:
                y = y * W[f"{p}ls{q}"]
            if hc + "in" in W:
                xs = [sum(W[hc + "mix"][s, t] * xs[s] for s in range(n)) + m * W[hc + "out"][t] * y for t in range(n)]
            else:
                xs = [xs[0] + m * y]
        if trace is not None:
            trace.append(sum(xs))
    z = rms_norm(sum(xs), W["final.norm"], eps) @ W["embed"].T
    cap = cfg.get("logit_softcap")
    return cap * np.tanh(z / cap) if cap else z

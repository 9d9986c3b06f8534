"""
A plain, slow float64 implementation of the Dikopel design, written from its equations: one function per mechanism, token by token where the
design is recurrent, sharing no code with the product path.  Test infrastructure only.

Weights are a dict name -> float64 numpy array (the names a checkpoint uses); `cfg` is the parsed config.json.  Sequences are processed one at a
time and whole, so nothing here knows about steps, slots, pages or batches.
"""
from __future__ import annotations
import math
import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def logsigmoid(z):
    return -np.logaddexp(0.0, -z)


def rms_unit(x, eps):
    """x over the root of its mean square (last axis)."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(axis=-1, keepdims=True)
    d = x - mu
    return d / np.sqrt(np.mean(d * d, axis=-1, keepdims=True) + eps) * w + b


def position_vectors(count, width):
    """[count, width]: entry 2i = sin(p f_i), entry 2i + 1 = cos(p f_i), f_i = 10000^(-2i / width)."""
    out = np.zeros((count, width))
    for i in range((width + 1) // 2):
        f = 10000.0 ** (-2.0 * i / width)
        a = np.arange(count) * f
        out[:, 2 * i] = np.sin(a)
        if 2 * i + 1 < width:
            out[:, 2 * i + 1] = np.cos(a)
    return out


def causal_conv(h, w, identity):
    """h [T, C], w [C, taps]: sum_j w[:, j] h[t - taps + 1 + j] with zeros before the start; `identity` adds h itself."""
    T, C = h.shape
    taps = w.shape[1]
    out = h.copy() if identity else np.zeros_like(h)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def mlstm(h, W, pre, m, eps):
    """Matrix memory with exponential gating and a running maximum that starts at 0."""
    H, d, dv, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
    T = h.shape[0]
    q = (h @ W[pre + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ W[pre + "k"].T).reshape(T, H, d)
    v = (h @ W[pre + "v"].T).reshape(T, H, dv)
    ig = cap * np.tanh((h @ W[pre + "i"].T + W[pre + "i.b"]) / cap)
    fg = logsigmoid(cap * np.tanh((h @ W[pre + "f"].T + W[pre + "f.b"]) / cap))
    out = np.zeros((T, H, dv))
    for a in range(H):
        S, n, mx = np.zeros((d, dv)), np.zeros(d), 0.0
        for t in range(T):
            m_new = max(fg[t, a] + mx, ig[t, a])
            df, di = math.exp(fg[t, a] + mx - m_new), math.exp(ig[t, a] - m_new)
            S = df * S + di * np.outer(k[t, a], v[t, a])
            n = df * n + di * k[t, a]
            mx = m_new
            out[t, a] = (S.T @ q[t, a]) / (max(abs(n @ q[t, a]), math.exp(-mx)) + 1e-6)
    o = rms_unit(out, eps).reshape(T, H * dv) * W[pre + "norm"] * sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T


def sigmoid_attention(h, W, pre, m):
    """Causal attention without softmax: every visible key weighs sigmoid(scale q.k + bias_head), weights are not normalised."""
    H, G, d, dv, scale = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"])
    T = h.shape[0]
    q = (h @ W[pre + "q"].T).reshape(T, H, d)
    k = (h @ W[pre + "k"].T).reshape(T, G, d)
    v = (h @ W[pre + "v"].T).reshape(T, G, dv)
    out = np.zeros((T, H, dv))
    vis = np.tril(np.ones((T, T)))
    for a in range(H):
        g = a // (H // G)
        wgt = sigmoid(q[:, a] @ k[:, g].T * scale + W[pre + "pb"][a]) * vis
        out[:, a] = wgt @ v[:, g]
    return out.reshape(T, H * dv) @ W[pre + "o"].T


def gated_delta(h, W, pre, m, eps):
    """Delta-rule memory with a scalar decay per head: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    short = lambda nm: silu(causal_conv(h @ W[pre + nm].T, W[pre + nm + ".conv"], identity=False))
    q, k, v = short("q").reshape(T, G, d), short("k").reshape(T, G, d), short("v").reshape(T, H, dv)
    unit = lambda x: x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + 1e-6)
    q, k = unit(q) * d ** -0.5, unit(k)
    beta = sigmoid(h @ W[pre + "b"].T)
    decay = np.exp(-np.exp(W[pre + "A_log"]) * softplus(h @ W[pre + "a"].T + W[pre + "dt_bias"]))
    out = np.zeros((T, H, dv))
    for a in range(H):
        g = a // (H // G)
        S = np.zeros((d, dv))
        for t in range(T):
            S = decay[t, a] * S
            u = beta[t, a] * (v[t, a] - S.T @ k[t, g])
            S = S + np.outer(k[t, g], u)
            out[t, a] = S.T @ q[t, g]
    o = rms_unit(out, eps) * W[pre + "norm"] * silu(h @ W[pre + "g"].T).reshape(T, H, dv)
    return o.reshape(T, H * dv) @ W[pre + "o"].T


def parallel_mixer(h, W, pre, m, eps):
    left = sigmoid_attention(h, W, pre + "left.", m["left"])
    right = gated_delta(h, W, pre + "right.", m["right"], eps)
    return 0.5 * (rms_unit(left, eps) * W[pre + "left.out"] + rms_unit(right, eps) * W[pre + "right.out"])


def gated_ff(h, W, pre):
    return (silu(h @ W[pre + "gate"].T) * (h @ W[pre + "up"].T)) @ W[pre + "down"].T


def route(z, corr, r):
    """z [E] router logits -> (chosen experts, weights).  Choice by sigmoid + correction inside the kept groups, weights from the bare sigmoids."""
    E, top = int(r["experts"]), int(r["top"])
    s = sigmoid(z)
    c = s + corr
    grp = r.get("groups") or {}
    count, keep = int(grp.get("count", 1)), int(grp.get("keep", grp.get("count", 1)))
    if count > 1 and keep < count:
        per = E // count
        gs = [np.sort(c[g * per:(g + 1) * per])[::-1][:2].sum() for g in range(count)]
        order = sorted(range(count), key=lambda g: (-gs[g], g))[:keep]
        c = np.array([c[e] if (e // per) in order else -np.inf for e in range(E)])
    chosen = sorted(range(E), key=lambda e: (-c[e], e))[:top]
    w = s[chosen]
    return chosen, w / (w.sum() + 1e-20) * float(r.get("scale", 1.0))


def moe(h, W, pre, f):
    T = h.shape[0]
    out = np.zeros((T, W[pre + "e0.down"].shape[0]))
    z = h @ W[pre + "router"].T
    corr = W.get(pre + "correction")
    if corr is None:
        corr = np.zeros(z.shape[1])
    for t in range(T):
        chosen, w = route(z[t], corr, f["router"])
        for e, we in zip(chosen, w):
            out[t] += we * gated_ff(h[t:t + 1], W, f"{pre}e{e}.")[0]
    if f.get("shared"):
        out += gated_ff(h, W, pre + "shared.") * sigmoid(h @ W[pre + "shared.sg"].T)
    return out


def forward(cfg, W, tokens, taps_out=None):
    """tokens of ONE sequence -> logits [T, vocab] (float64).  taps_out: a list that receives the residual stream after every layer."""
    width, eps = int(cfg["width"]), float(cfg["norm"]["eps"])
    T = len(tokens)
    x = W["embed"][np.asarray(tokens)] * float(cfg["embedding"]["scale"]) + position_vectors(T, width)
    mult = float(cfg.get("residual_mult", 1.0))
    for i, L in enumerate(cfg["layers"]):
        src = int(L["weights_of"]) if L.get("weights_of") is not None else i
        pre = f"l{src}."
        h = layer_norm(x, W[pre + "norm1"], W[pre + "norm1.b"], eps)
        hm = causal_conv(h, W[pre + "canon1"], identity=True)
        if L["type"] == "mlstm":
            y = mlstm(hm, W, pre + "mix.", L["mixer"], eps)
        elif L["type"] == "parallel":
            y = parallel_mixer(hm, W, pre + "mix.", L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        f = L.get("mlp")
        if f is not None:
            y = y + (gated_ff(h, W, pre + "mlp.") if f["kind"] == "dense" else moe(h, W, pre + "mlp.", f))
        x = x + mult * y
        if taps_out is not None:
            taps_out.append(x.copy())
    return layer_norm(x, W["final.norm"], W["final.norm.b"], eps) @ W["head"].T

"""Slow float64 restatement of the Fimunex mechanisms, one function per mechanism, written from their equations and sharing no code with
exllamav3_amd (test infrastructure only).  Weights are a dict name -> tensor (used at the stored values), the configuration is the
config.json dict.  Everything runs on the CPU over whole sequences; nothing is cached, so a whole-sequence pass is the truth for every
way of cutting the same tokens into steps."""
import math
import torch

F64 = torch.float64


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """RMS norm with a one-plus weight: the checkpoint holds w, the norm multiplies by 1 + w."""
    return rms_unit(x, eps) * (1.0 + w)


def causal_taps(h, w):
    """h [T, C], w [C, taps]: h_t + sum_j w[:, j] h_(t - taps + 1 + j), nothing before the sequence's start."""
    T, C = h.shape
    taps = w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotary_half_tables(T, dims, base, scaling=None):
    """cos, sin [T, dims/2] for the pairs (i, i + dims/2); with `scaling` the frequencies are blended with their slowed versions along a
    ramp over the pair index and both tables are multiplied by 0.1 ln(factor) + 1."""
    i = torch.arange(dims // 2, dtype=F64)
    f = float(base) ** (-2.0 * i / dims)
    mag = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])
        at = lambda turns: dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))
        lo = max(math.floor(at(float(scaling["fast"]))), 0)
        hi = min(math.ceil(at(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    a = torch.arange(T, dtype=F64)[:, None] * f[None, :]
    return torch.cos(a) * mag, torch.sin(a) * mag


def rotate_half(x, cos, sin, dims):
    """x [T, ..., d]: entries i and i + dims/2 (i < dims/2) of the last axis turn together; entries from `dims` on pass."""
    out = x.clone()
    half = dims // 2
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = cos.reshape(shape), sin.reshape(shape)
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def chunk_softmax_attention(q, k, v, scale, softcap, chunk):
    """q [T, d], k [T, d], v [T, dv] of one map of one head: token i sees j <= i with i // chunk == j // chunk, i and j being positions in the sequence."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for i in range(T):
        lo = (i // chunk) * chunk if chunk else 0
        s = (k[lo:i + 1] @ q[i]) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        p = torch.softmax(s, 0)
        out[i] = p @ v[lo:i + 1]
    return out


def differential_attention(h, W, pre, m, eps):
    """The attention mixer over a whole sequence h [T, width]; m = the layer's `mixer` dict."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"]))
    diff = float(m["diff"])
    q = (h @ W[pre + "q"].T + W[pre + "q.b"]).reshape(T, H, 2, d)
    k = (h @ W[pre + "k"].T + W[pre + "k.b"]).reshape(T, G, 2, d)
    v = (h @ W[pre + "v"].T + W[pre + "v.b"]).reshape(T, G, dv)
    q = rms_unit(q, eps) * W[pre + "q.norm"]
    k = rms_unit(k, eps) * W[pre + "k.norm"]
    rot = m.get("rot")
    if rot:
        dims = int(rot.get("dims", d))
        cos, sin = rotary_half_tables(T, dims, rot["base"], rot.get("scaling"))
        q, k = rotate_half(q, cos, sin, dims), rotate_half(k, cos, sin, dims)
    lam = torch.exp((W[pre + "lq1"] * W[pre + "lk1"]).sum()) - torch.exp((W[pre + "lq2"] * W[pre + "lk2"]).sum()) + diff
    mask = m.get("mask")
    chunk = int(mask["size"]) if mask else 0
    cap = float(m.get("softcap") or 0.0)
    gate = torch.sigmoid(h @ W[pre + "g"].T)                                  # [T, H]
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        a1 = chunk_softmax_attention(q[:, hh, 0], k[:, g, 0], v[:, g], float(m["scale"]), cap, chunk)
        a2 = chunk_softmax_attention(q[:, hh, 1], k[:, g, 1], v[:, g], float(m["scale"]), cap, chunk)
        o = rms_unit(a1 - lam * a2, eps) * (1.0 - diff)
        heads.append(o * gate[:, hh:hh + 1])
    return torch.cat(heads, 1) @ W[pre + "o"].T + W[pre + "o.b"]


def grouped_router(z, correction, top, groups, keep):
    """z [T, E] logits over all experts (identity experts included).  Returns chosen indices [T, top] and weights [T, top]: scores are a
    softmax over all experts; the choice looks at score + correction, only inside the `keep` groups with the best single choice score; the
    weights are the chosen scores themselves over their sum."""
    T, E = z.shape
    s = torch.softmax(z, 1)
    c = s + correction
    if groups and groups > 1 and keep < groups:
        per = E // groups
        best = c.reshape(T, groups, per).max(2).values
        kept = torch.topk(best, keep, dim=1).indices
        allowed = torch.zeros(T, groups, dtype=torch.bool)
        allowed.scatter_(1, kept, True)
        allowed = allowed[:, :, None].expand(T, groups, per).reshape(T, E)
        c = torch.where(allowed, c, torch.full_like(c, -math.inf))
    idx = torch.topk(c, top, dim=1).indices
    w = torch.gather(s, 1, idx)
    return idx, w / (w.sum(1, keepdim=True) + 1e-20)


def expert_mixture(h, W, pre, f):
    """The feed-forward over h [T, width]; f = the layer's `mlp` dict.  The last `identity` router outputs stand for experts that return
    their input."""
    r = f["router"]
    E, I, top = int(r["experts"]), int(r.get("identity", 0)), int(r["top"])
    g = r.get("groups") or {}
    z = h @ W[pre + "router"].T
    corr = W[pre + "correction"] if (pre + "correction") in W else torch.zeros(E + I, dtype=F64)
    idx, w = grouped_router(z, corr, top, int(g.get("count", 1)), int(g.get("keep", 1)))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            if e >= E:
                y = h[t]
            else:
                y = W[f"{pre}e{e}.down"] @ (torch.relu(W[f"{pre}e{e}.up"] @ h[t]) ** 2)
            out[t] += w[t, j] * y
    return out


def layer_runs(config):
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, t = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * t + list(range(b, n))


def forward(config, W, tokens, taps_out=None):
    """Logits [T, vocab] of one sequence; taps_out (a list) receives the residual stream after every layer run."""
    W = {k: v.to(F64) for k, v in W.items() if v.dtype.is_floating_point}
    eps = float(config["norm"]["eps"])
    x = W["embed"][torch.tensor(tokens, dtype=torch.long)]
    for i in layer_runs(config):
        L = config["layers"][i]
        p = f"l{i}."
        if L["type"] != "attention":
            raise ValueError(L["type"])
        h = causal_taps(norm_one_plus(x, W[p + "norm1"], eps), W[p + "canon1"])
        x = x + differential_attention(h, W, p + "mix.", L["mixer"], eps)
        if L.get("mlp") is not None:
            h = causal_taps(norm_one_plus(x, W[p + "norm2"], eps), W[p + "canon2"])
            x = x + expert_mixture(h, W, p + "mlp.", L["mlp"])
        if taps_out is not None:
            taps_out.append(x.clone())
    logits = norm_one_plus(x, W["final.norm"], eps) @ W["head"].T
    cap = float(config.get("logit_softcap") or 0.0)
    return cap * torch.tanh(logits / cap) if cap else logits


def greedy(config, W, prompt, new_tokens):
    toks, out = list(prompt), []
    for _ in range(new_tokens):
        t = int(torch.argmax(forward(config, W, toks)[-1]))
        out.append(t); toks.append(t)
    return out

"""Plain, slow float64 oracle of the Sefalorn design: one function per
mechanism, explicit loops over tokens and heads, no paging, no batching,
no state objects. It shares no code with fusioninfer_amd; tests compare
the engine (CPU ops or HIP kernels) against it.

Weights use the checkpoint naming (``l<i>.mix.q``, ``l<i>.mix.left.q.b``
...), as a dict of float64 tensors; ``cfg`` is the config.json dict.
"""

import math

import torch

F64 = torch.float64


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0.0)


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w, biased variance, no bias."""
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    var = (d * d).mean(-1, keepdim=True)
    return d / torch.sqrt(var + eps) * w


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


# ---------------------------------------------------------------- lightning

def lightning_mixer(h, P, pre, m, eps):
    """Linear attention with one scalar decay per head. h: [T, width]."""
    H, D, V = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(h @ P[pre + "q"].T).reshape(T, H, D)
    k = silu(h @ P[pre + "k"].T).reshape(T, H, D)
    v = silu(h @ P[pre + "v"].T).reshape(T, H, V)
    o = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, V, dtype=F64)
        lam = float(m["decay"][hd])
        for t in range(T):
            S = lam * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = unit_rms(o.reshape(T, H * V), eps) * P[pre + "norm"]
    o = o * sigmoid(h @ P[pre + "g"].T)
    return o @ P[pre + "o"].T


# ------------------------------------------------- windowed softmax attention

def window_attention(h, P, pre, m):
    """Grouped-query softmax attention without rotation: log-distance
    score penalty per head, scores mixed across heads before the softmax,
    sliding window of ``mask.size`` positions."""
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    win = int(m["mask"]["size"])
    T = h.shape[0]
    q = (h @ P[pre + "q"].T + P[pre + "q.b"]).reshape(T, H, D)
    k = (h @ P[pre + "k"].T + P[pre + "k.b"]).reshape(T, G, D)
    v = (h @ P[pre + "v"].T + P[pre + "v.b"]).reshape(T, G, V)
    r1, r2, talk = P[pre + "r1"], P[pre + "r2"], P[pre + "talk"]
    rep = H // G
    out = torch.zeros(T, H, V, dtype=F64)
    for i in range(T):
        lo = max(0, i - win + 1)               # visible: 0 <= i - j < win
        dist = torch.arange(i - lo, -1, -1, dtype=F64)       # i - j
        sc = torch.zeros(H, i - lo + 1, dtype=F64)
        for hd in range(H):
            g = hd // rep
            sc[hd] = (k[lo:i + 1, g] @ q[i, hd]) * float(m["scale"]) \
                - r1[hd] * torch.log(1.0 + r2[hd] * dist)
        mixed = talk @ sc                      # row h = sum_g talk[h, g] sc[g]
        w = torch.softmax(mixed, dim=-1)
        for hd in range(H):
            out[i, hd] = w[hd] @ v[lo:i + 1, hd // rep]
    return out.reshape(T, H * V) @ P[pre + "o"].T + P[pre + "o.b"]


# ------------------------------------------------------- gated delta rule

def causal_conv(x, w):
    """x: [T, C]; w: [C, taps], last column multiplies the current token;
    zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                y[t] += w[:, j] * x[src]
    return y


def gated_delta_mixer(h, P, pre, m, eps):
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(causal_conv(h @ P[pre + "q"].T, P[pre + "q.conv"])).reshape(T, G, D)
    k = silu(causal_conv(h @ P[pre + "k"].T, P[pre + "k.conv"])).reshape(T, G, D)
    v = silu(causal_conv(h @ P[pre + "v"].T, P[pre + "v.conv"])).reshape(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(h @ P[pre + "b"].T)                       # [T, H]
    dt = softplus(h @ P[pre + "a"].T + P[pre + "dt_bias"])   # [T, H]
    gdec = torch.exp(-torch.exp(P[pre + "A_log"]) * dt)      # [T, H]
    rep = H // G
    o = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        g = hd // rep
        S = torch.zeros(D, V, dtype=F64)
        for t in range(T):
            S = gdec[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, hd] = S.T @ q[t, g]
    o = unit_rms(o, eps) * P[pre + "norm"]
    o = o.reshape(T, H * V) * silu(h @ P[pre + "g"].T)
    return o @ P[pre + "o"].T


def parallel_mixer(h, P, pre, m, eps):
    left = window_attention(h, P, pre + "left.", m["left"])
    right = gated_delta_mixer(h, P, pre + "right.", m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


# ------------------------------------------------------ mixture of experts

def moe(h, P, pre, m):
    E, top = int(m["router"]["experts"]), int(m["router"]["top"])
    scale = float(m["router"]["scale"])
    T = h.shape[0]
    out = torch.zeros(T, P[pre + "e0.down"].shape[0], dtype=F64)
    for t in range(T):
        s = sigmoid(P[pre + "router"] @ h[t])
        order = sorted(range(E), key=lambda e: -float(s[e]))[:top]
        tot = sum(float(s[e]) for e in order) + 1e-20
        for e in order:
            p = pre + "e%d." % e
            a = silu(P[p + "gate"] @ h[t]) * (P[p + "up"] @ h[t])
            out[t] += (float(s[e]) / tot * scale) * (P[p + "down"] @ a)
    return out


# ------------------------------------------------------------------ model

def forward(tokens, P, cfg, return_layers=False):
    """Logits [T, vocab] of one whole sequence (positions 0..T-1)."""
    eps = float(cfg["norm"]["eps"])
    x = P["embed"][torch.as_tensor(tokens, dtype=torch.long)].clone()
    layers = []
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % i
        h = layer_norm(x, P[p + "norm1"], eps)
        if L["type"] == "lightning":
            y = lightning_mixer(h, P, p + "mix.", L["mixer"], eps)
        elif L["type"] == "parallel":
            y = parallel_mixer(h, P, p + "mix.", L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        x = x + y * sigmoid(h @ P[p + "rg1"].T + P[p + "rg1.b"])
        if L.get("mlp"):
            h = layer_norm(x, P[p + "norm2"], eps)
            y = moe(h, P, p + "mlp.", L["mlp"])
            x = x + y * sigmoid(h @ P[p + "rg2"].T + P[p + "rg2.b"])
        layers.append(x.clone())
    h = layer_norm(x, P["final.norm"], eps)
    logits = h @ P["head"].T * float(cfg.get("logit_scale", 1.0))
    if return_layers:
        return logits, torch.stack(layers)
    return logits


def greedy(tokens, P, cfg, n_new):
    """n_new greedy continuations of a prompt (whole-sequence recompute)."""
    toks = list(tokens)
    out = []
    for _ in range(n_new):
        nxt = int(forward(toks, P, cfg)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out

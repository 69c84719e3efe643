"""Plain, slow float64 oracle of the Pinuvik design: one function per
mechanism, explicit loops over tokens and heads, no paging, no batching,
no state objects. It shares no code with fusioninfer_amd; tests compare
the engine (CPU ops or HIP kernels) against it.

Weights use the checkpoint naming (``l<i>.mix.left.q`` ...), as a dict of
float64 tensors; ``cfg`` is the config.json dict.
"""

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, gain, eps):
    return unit_rms(x, eps) * gain


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def token_shift(h, mix, h_before=None):
    """h: [T, W]. Row t moves towards row t-1 of the UNSHIFTED h by
    `mix`; row 0 moves towards h_before (zeros if None)."""
    out = torch.empty_like(h)
    prev = torch.zeros_like(h[0]) if h_before is None else h_before
    for t in range(h.shape[0]):
        out[t] = h[t] + (prev - h[t]) * mix
        prev = h[t]
    return out


def rotate_pairs(x, pos, dims, base):
    """x: [heads, D] at position pos; dims (2i, 2i+1), 2i+1 < dims, turn
    by pos * base^(-2i/dims)."""
    y = x.clone()
    for i in range(dims // 2):
        ang = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(ang), math.sin(ang)
        a, b = x[:, 2 * i], x[:, 2 * i + 1]
        y[:, 2 * i] = a * c - b * s
        y[:, 2 * i + 1] = b * c + a * s
    return y


def visible(i, j, chunk):
    return j <= i and (chunk <= 0 or i // chunk == j // chunk)


def shared_kv_attention(h, W, pre, m, eps, pos0=0):
    """Left half on rows h [T, width] (positions pos0..); returns the
    projected output [T, width]. No cache: all T rows must be given."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    rd, base = m["rot"]["dims"], m["rot"]["base"]
    chunk = m["mask"]["size"]
    q = (h @ W[pre + "q"].T).view(T, H, D)
    kraw = (h @ W[pre + "k"].T).view(T, G, D)
    qn = torch.stack([unit_rms(rotate_pairs(q[t], pos0 + t, rd, base), eps)
                      for t in range(T)])
    kn = torch.stack([unit_rms(rotate_pairs(kraw[t], pos0 + t, rd, base), eps)
                      for t in range(T)])
    out = torch.zeros(T, H, D, dtype=F64)
    for i in range(T):
        js = [j for j in range(T) if visible(pos0 + i, pos0 + j, chunk)]
        for hh in range(H):
            g = hh // (H // G)
            sc = (kn[js, g] * qn[i, hh]).sum(-1) * m["scale"]
            out[i, hh] = torch.softmax(sc, 0) @ kraw[js, g]
    return out.reshape(T, H * D) @ W[pre + "o"].T


def delta_rule_step(S, r, k, v, w, a):
    """One token of one head. S: [D, D] (key x value)."""
    u = k / torch.sqrt((k * k).sum() + 1e-6)
    uS = u @ S
    S = w[:, None] * S - torch.outer(a * u, uS) + torch.outer(k, v)
    return S, S.T @ r


def delta_rule_mixer(h, W, pre, m, eps, state=None):
    """Right half; returns (projected output [T, width], final state
    [heads, D, D])."""
    T = h.shape[0]
    Hn, D = m["heads"], m["dim"]
    r = (h @ W[pre + "r"].T).view(T, Hn, D)
    k = (h @ W[pre + "k"].T).view(T, Hn, D)
    v = (h @ W[pre + "v"].T).view(T, Hn, D)
    lin = torch.tanh(h @ W[pre + "w1"].T) @ W[pre + "w2"].T + W[pre + "w0"]
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(lin)).view(T, Hn, D)
    a = torch.sigmoid(h @ W[pre + "a"].T + W[pre + "a.b"]).view(T, Hn, D)
    gate = torch.sigmoid(h @ W[pre + "g"].T)
    S = torch.zeros(Hn, D, D, dtype=F64) if state is None else state.clone()
    o = torch.zeros(T, Hn, D, dtype=F64)
    for t in range(T):
        for hh in range(Hn):
            S[hh], o[t, hh] = delta_rule_step(S[hh], r[t, hh], k[t, hh],
                                              v[t, hh], w[t, hh], a[t, hh])
    o = unit_rms(o, eps).reshape(T, Hn * D) * W[pre + "norm"] * gate
    return o @ W[pre + "o"].T, S


def layer_runs(cfg):
    lp = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    n = len(cfg["layers"])
    return (list(range(lp["start"]))
            + list(range(lp["start"], lp["stop"])) * lp["times"]
            + list(range(lp["stop"], n)))


def forward(cfg, W, tokens, return_layers=False):
    """Logits [T, vocab] for one whole sequence from position 0."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)]
    streams = []
    for li in layer_runs(cfg):
        L, p = cfg["layers"][li], "l%d." % li
        h = token_shift(scalar_norm(x, W[p + "norm1"], eps), W[p + "shift"])
        left = shared_kv_attention(h, W, p + "mix.left.", L["mixer"]["left"],
                                   eps)
        right, _ = delta_rule_mixer(h, W, p + "mix.right.",
                                    L["mixer"]["right"], eps)
        y = 0.5 * (unit_rms(left, eps) * W[p + "mix.left.out"]
                   + unit_rms(right, eps) * W[p + "mix.right.out"])
        x = x + scalar_norm(y, W[p + "norm1b"], eps)
        if L.get("mlp"):
            h2 = scalar_norm(x, W[p + "norm2"], eps)
            ff = (gelu_tanh(h2 @ W[p + "mlp.gate"].T)
                  * (h2 @ W[p + "mlp.up"].T)) @ W[p + "mlp.down"].T
            x = x + scalar_norm(ff, W[p + "norm2b"], eps)
        streams.append(x.clone())
    logits = scalar_norm(x, W["final.norm"], eps) @ W["head"].T
    return (logits, streams) if return_layers else logits


def greedy(cfg, W, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]

"""Plain float64 oracle of the Muvetar design, one function per mechanism.

Written from the design's equations only: whole sequences, token-by-token
recurrences, a per-token loop over chosen experts, dense attention matrices.
It shares no code with the engine, its ops or their torch reference forms,
reads a checkpoint's tensors by their checkpoint names, and knows nothing of
pages, slots, portions or batches.

Notation: W width, n tokens, x the residual stream [n, W], h a sublayer's
normed input.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def position_vector(n, width, first=0):
    """[n, width]: column 2i = sin(p / 10000^(2i/width)), column 2i+1 = cos of
    the same angle, p = first .. first + n - 1."""
    out = torch.zeros(n, width, dtype=F64)
    for c in range(width):
        i = c // 2
        freq = 10000.0 ** (-2.0 * i / width)
        for r in range(n):
            a = (first + r) * freq
            out[r, c] = math.cos(a) if c % 2 else math.sin(a)
    return out


def mingru(t, p, h):
    """Elementwise gated recurrence; returns the mixer output [n, W]."""
    a = sigmoid(h @ t[p + "z"].T + t[p + "z.b"])
    u = h @ t[p + "x"].T + t[p + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, sigmoid(u))
    state = torch.zeros(u.shape[1], dtype=F64)
    rows = []
    for r in range(h.shape[0]):
        state = (1.0 - a[r]) * state + a[r] * cand[r]
        rows.append(state)
    s = torch.stack(rows)
    return (s * silu(h @ t[p + "g"].T)) @ t[p + "o"].T


def log_bias_attention(t, p, h, m):
    """Causal softmax attention; head a's score for query i and key j <= i is
    q_i.k_j * scale - r1_a * ln(1 + r2_a * (i - j))."""
    n = h.shape[0]
    H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[p + "q"].T).view(n, H, D)
    k = (h @ t[p + "k"].T).view(n, G, D)
    v = (h @ t[p + "v"].T).view(n, G, DV)
    out = torch.zeros(n, H, DV, dtype=F64)
    for a in range(H):
        g = a // (H // G)
        r1, r2 = float(t[p + "r1"][a]), float(t[p + "r2"][a])
        for i in range(n):
            d = torch.arange(i, -1, -1, dtype=F64)             # i - j for j = 0..i
            s = (k[: i + 1, g] @ q[i, a]) * m["scale"] - r1 * torch.log1p(r2 * d)
            w = torch.softmax(s, dim=0)
            out[i, a] = w @ v[: i + 1, g]
    return out.reshape(n, H * DV) @ t[p + "o"].T


def causal_conv(x, w, b):
    """x [n, C]; w [C, K], last column = the current token's tap; zeros
    before the start."""
    n, C = x.shape
    K = w.shape[1]
    out = torch.zeros(n, C, dtype=F64)
    for r in range(n):
        acc = b.clone()
        for k in range(K):
            src = r - (K - 1) + k
            if src >= 0:
                acc = acc + w[:, k] * x[src]
        out[r] = acc
    return out


def mamba(t, p, h, m):
    """Selective scan behind a short convolution; returns [n, W]."""
    n = h.shape[0]
    I, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = h @ t[p + "in"].T
    x, z = xz[:, :I], xz[:, I:]
    x = silu(causal_conv(x, t[p + "conv"], t[p + "conv.b"]))
    proj = x @ t[p + "x"].T
    dt, Bm, Cm = proj[:, :R], proj[:, R:R + N], proj[:, R + N:R + 2 * N]
    step = softplus(dt @ t[p + "dt"].T + t[p + "dt.b"])         # [n, I]
    A = -torch.exp(t[p + "A_log"])                             # [I, N]
    S = torch.zeros(I, N, dtype=F64)
    ys = []
    for r in range(n):
        S = torch.exp(step[r].unsqueeze(1) * A) * S + (step[r] * x[r]).unsqueeze(1) * Bm[r]
        ys.append(S @ Cm[r] + t[p + "D"] * x[r])
    y = torch.stack(ys) * silu(z)
    return y @ t[p + "o"].T


def expert(t, p, h, limit):
    g = torch.clamp(h @ t[p + "gate"].T, max=limit)
    u = torch.clamp(h @ t[p + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ t[p + "down"].T


def route(t, p, h, m):
    """(chosen experts [n, top], their weights [n, top])."""
    s = torch.softmax(h @ t[p + "router"].T, dim=-1)
    w, idx = torch.sort(s, dim=-1, descending=True, stable=True)
    top = m["router"]["top"]
    return idx[:, :top], w[:, :top] * m["router"].get("scale", 1.0)


def moe(t, p, h, m):
    idx, w = route(t, p, h, m)
    out = torch.zeros_like(h)
    for r in range(h.shape[0]):
        for j in range(idx.shape[1]):
            e = int(idx[r, j])
            out[r] += w[r, j] * expert(t, f"{p}e{e}.", h[r:r + 1], m["expert"]["limit"])[0]
    if m.get("shared"):
        out = out + expert(t, p + "shared.", h, m["shared"]["limit"])
    return out


def depth_average(results, coef):
    """results = [X_0, ..., X_k]; returns sum_j coef[j] X_j."""
    out = torch.zeros_like(results[0])
    for j, xj in enumerate(results):
        out = out + coef[j] * xj
    return out


def as_f64(tensors):
    return {k: v.to(F64) for k, v in tensors.items()}


def forward(cfg, tensors, tokens, taps=None):
    """Logits [n, vocab] of a whole token sequence, float64."""
    t = as_f64(tensors)
    n, W, eps = len(tokens), cfg["width"], cfg["norm"]["eps"]
    mult = cfg.get("residual_mult", 1.0)
    x = t["embed"][torch.tensor(tokens)] + position_vector(n, W)
    results = [x]
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = rms_norm(x, t[p + "norm1"], eps)
        if layer["type"] == "mingru":
            y = mingru(t, p + "mix.", h)
        else:
            y = m.get("left_scale", 1.0) * log_bias_attention(t, p + "mix.left.", h, m["left"]) \
                + m.get("right_scale", 1.0) * mamba(t, p + "mix.right.", h, m["right"])
        x = x + mult * y
        if layer["mlp"] is not None:
            x = x + mult * moe(t, p + "mlp.", rms_norm(x, t[p + "norm2"], eps), layer["mlp"])
        results.append(x)
        x = depth_average(results, t[p + "dwa"])
        if taps is not None:
            taps.append(x)
    logits = rms_norm(x, t["final.norm"], eps) @ t["head"].T
    cap = cfg.get("logit_softcap") or 0.0
    return cap * torch.tanh(logits / cap) if cap else logits


def greedy(cfg, tensors, prompt, steps):
    toks = list(prompt)
    for _ in range(steps):
        toks.append(int(forward(cfg, tensors, toks)[-1].argmax()))
    return toks[len(prompt):]

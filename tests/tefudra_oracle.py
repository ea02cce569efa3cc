"""Plain float64 oracle of the Tefudra design, one function per mechanism.

Written from the design's equations only: whole sequences, dense attention
rows, token-by-token recurrences, a per-token loop over chosen experts. It
shares no code with the engine, its ops or their torch reference forms, reads
a checkpoint's tensors by their checkpoint names, and knows nothing of pages,
slots, portions or batches.

Notation: W width, n tokens, x the residual stream [n, W], h a sublayer's
normed input, positions 0 .. n-1.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, w, eps, groups):
    """The vector in `groups` equal consecutive parts, each divided by its own
    root mean square, the whole times w."""
    n, W = x.shape
    parts = x.view(n, groups, W // groups)
    return rms(parts, eps).reshape(n, W) * w


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def log_sigmoid(x):
    return -torch.log1p(torch.exp(-x.abs())) + torch.clamp(x, max=0.0)


def rotate_half(x, first_pos, base, dims, sign=1.0):
    """x [n, ..., d]: pair (i, i + dims/2) of the first `dims` channels turns
    by sign * position * base^(-2i/dims); the rest passes."""
    n = x.shape[0]
    half = dims // 2
    out = x.clone()
    if not half:
        return out
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    pos = torch.arange(first_pos, first_pos + n, dtype=F64)
    ang = sign * pos.view(n, *([1] * (x.dim() - 1))) * freq
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def causal_conv(u, w):
    """u [n, C], w [C, taps]: y_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros
    before the start."""
    n, C = u.shape
    taps = w.shape[1]
    y = torch.zeros(n, C, dtype=F64)
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def sink_window_attention(t, p, h, m, eps):
    """Grouped-head attention whose values are the keys as projected; per-head
    q/k norm, partial rotation, a sliding window that keeps the first tokens,
    and a softmax whose denominator holds one more term exp(sink_head)."""
    n = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    size, keep = m["mask"]["size"], m["mask"].get("keep_first", 0)
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    q = (h @ t[p + "q"].T).view(n, H, D)
    k = (h @ t[p + "k"].T).view(n, G, D)
    v = k.clone()
    q = rotate_half(rms(q, eps) * t[p + "q.norm"], 0, base, dims)
    k = rotate_half(rms(k, eps) * t[p + "k.norm"], 0, base, dims)
    out = torch.zeros(n, H, D, dtype=F64)
    for a in range(H):
        g = a // (H // G)
        sink = float(t[p + "sink"][a])
        for i in range(n):
            js = [j for j in range(i + 1) if i - j < size or j < keep]
            s = torch.stack([(q[i, a] @ k[j, g]) * m["scale"] for j in js])
            top = max(float(s.max()), sink)
            e = torch.exp(s - top)
            den = e.sum() + math.exp(sink - top)
            for wgt, j in zip(e / den, js):
                out[i, a] += wgt * v[j, g]
    return out.reshape(n, H * D) @ t[p + "o"].T


def softcap_window_attention(t, p, h, m, eps):
    """The left half of a parallel mixer: biased projections, a short causal
    convolution on q, k and v, rotation of q and k, unit-norm values that are
    rotated by their own position and turned back at the query's, tanh-capped
    scores, a plain sliding window."""
    n = h.shape[0]
    H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    size = m["mask"]["size"]
    base, dims, cap = m["rot"]["base"], m["rot"]["dims"], m["softcap"]
    q = causal_conv(h @ t[p + "q"].T + t[p + "q.b"], t[p + "q.conv"]).view(n, H, D)
    k = causal_conv(h @ t[p + "k"].T + t[p + "k.b"], t[p + "k.conv"]).view(n, G, D)
    v = causal_conv(h @ t[p + "v"].T + t[p + "v.b"], t[p + "v.conv"]).view(n, G, DV)
    q = rotate_half(q, 0, base, dims)
    k = rotate_half(k, 0, base, dims)
    v = rotate_half(rms(v, eps), 0, base, DV)
    out = torch.zeros(n, H, DV, dtype=F64)
    for a in range(H):
        g = a // (H // G)
        for i in range(n):
            lo = max(0, i - size + 1)
            s = (k[lo:i + 1, g] @ q[i, a]) * m["scale"]
            s = cap * torch.tanh(s / cap)
            w = torch.softmax(s, dim=0)
            out[i, a] = w @ v[lo:i + 1, g]
    out = rotate_half(out, 0, base, DV, sign=-1.0)
    return out.reshape(n, H * DV) @ t[p + "o"].T + t[p + "o.b"]


def matrix_memory(t, p, h, m, eps):
    """The right half: a [dim, vdim] memory per head with a normaliser vector
    and a running maximum that starts at 0."""
    n = h.shape[0]
    H, D, DV, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ t[p + "q"].T).view(n, H, D) * D ** -0.5
    k = (h @ t[p + "k"].T).view(n, H, D)
    v = (h @ t[p + "v"].T).view(n, H, DV)
    gi = cap * torch.tanh((h @ t[p + "i"].T + t[p + "i.b"]) / cap)
    gf = log_sigmoid(cap * torch.tanh((h @ t[p + "f"].T + t[p + "f.b"]) / cap))
    out = torch.zeros(n, H, DV, dtype=F64)
    for a in range(H):
        S = torch.zeros(D, DV, dtype=F64)
        nv = torch.zeros(D, dtype=F64)
        mx = 0.0
        for r in range(n):
            new = max(float(gf[r, a]) + mx, float(gi[r, a]))
            df = math.exp(float(gf[r, a]) + mx - new)
            di = math.exp(float(gi[r, a]) - new)
            S = df * S + di * torch.outer(k[r, a], v[r, a])
            nv = df * nv + di * k[r, a]
            mx = new
            den = max(abs(float(nv @ q[r, a])), math.exp(-mx)) + 1e-6
            out[r, a] = (S.T @ q[r, a]) / den
    y = rms(out, eps).reshape(n, H * DV) * t[p + "norm"]
    y = y * sigmoid(h @ t[p + "g"].T)
    return y @ t[p + "o"].T


def parallel_mixer(t, p, h, m, eps):
    left = softcap_window_attention(t, p + "left.", h, m["left"], eps)
    right = matrix_memory(t, p + "right.", h, m["right"], eps)
    return 0.5 * (rms(left, eps) * t[p + "left.out"] + rms(right, eps) * t[p + "right.out"])


def relu_squared_ff(t, p, h):
    u = torch.clamp(h @ t[p + "up"].T, min=0.0)
    return (u * u) @ t[p + "down"].T


def gelu_erf(x):
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def gelu_ff(t, p, h):
    return gelu_erf(h @ t[p + "up"].T) @ t[p + "down"].T


def routed_experts(t, p, h, mlp):
    """Softmax router over real and identity experts; the choice adds a
    per-expert correction, the weights do not; a shared expert on top."""
    r = mlp["router"]
    E, ident, top = r["experts"], r.get("identity", 0), r["top"]
    z = h @ t[p + "router"].T
    s = torch.softmax(z, dim=-1)
    choice = s + t[p + "correction"]
    out = torch.zeros_like(h)
    for row in range(h.shape[0]):
        chosen = sorted(range(E + ident), key=lambda e: (-float(choice[row, e]), e))[:top]
        total = sum(float(s[row, e]) for e in chosen) + 1e-20
        for e in chosen:
            wgt = float(s[row, e]) / total
            x = h[row:row + 1]
            y = gelu_ff(t, f"{p}e{e}.", x) if e < E else x
            out[row] += wgt * y[0]
    if mlp.get("shared"):
        out = out + gelu_ff(t, p + "shared.", h)
    return out


def forward(cfg, t, ids, layer_outputs=None):
    """Logits [n, vocab] of one whole sequence; t maps checkpoint names to
    float64 tensors."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = t["embed"][torch.as_tensor(ids)]
    for i, lc in enumerate(cfg["layers"]):
        src = lc.get("weights_of", i)
        lp = f"l{src}."
        h = group_norm(x, t[lp + "norm1"], eps, groups)
        if lc["type"] == "attention":
            y = sink_window_attention(t, lp + "mix.", h, lc["mixer"], eps)
        else:
            y = parallel_mixer(t, lp + "mix.", h, lc["mixer"], eps)
        x = x + group_norm(y, t[lp + "norm1b"], eps, groups)
        mlp = lc.get("mlp")
        if mlp:
            h = group_norm(x, t[lp + "norm2"], eps, groups)
            if mlp["kind"] == "dense":
                y = relu_squared_ff(t, lp + "mlp.", h)
            else:
                y = routed_experts(t, lp + "mlp.", h, mlp)
            x = x + group_norm(y, t[lp + "norm2b"], eps, groups)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    x = group_norm(x, t["final.norm"], eps, groups)
    return x @ t["embed"].T


def greedy(cfg, t, ids, n):
    """n greedy continuations of ids, each from a whole forward pass."""
    ids, out = list(ids), []
    for _ in range(n):
        nxt = int(forward(cfg, t, ids)[-1].argmax())
        out.append(nxt)
        ids.append(nxt)
    return out

"""Reference implementations of the engine's hot ops in plain PyTorch.

These are the NUMERICS ORACLES for the HIP kernels (tests compare the
CDNA4 kernels against these at fp32) and the CPU execution path for tests.
They are deliberately simple; nothing here runs in the GPU hot loop.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, offset: float = 0.0) -> torch.Tensor:
    """RMSNorm. Gemma uses weight offset +1 (x * (1 + w))."""
    dtype = x.dtype
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    xf = xf * torch.rsqrt(var + eps)
    return (xf * (weight.float() + offset)).to(dtype)


def norm_add_norm(x, residual, w_post, w_pre, eps, offset=0.0):
    """residual += rmsnorm(x, w_post); x = rmsnorm(residual, w_pre)."""
    t = rmsnorm(x, w_post, eps, offset)
    residual = (residual.float() + t.float()).to(x.dtype)
    out = rmsnorm(residual, w_pre, eps, offset)
    return out, residual


def fused_add_rmsnorm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float, offset: float = 0.0
) -> Tuple[torch.Tensor, torch.Tensor]:
    """residual += x; out = rmsnorm(residual). Returns (out, new_residual)."""
    new_residual = (residual.float() + x.float()).to(x.dtype)
    return rmsnorm(new_residual, weight, eps, offset), new_residual


def build_rope_cache(
    max_positions: int, rotary_dim: int, theta: float, device,
    dtype=torch.float32, rope_scaling=None,
) -> torch.Tensor:
    """[max_positions, rotary_dim]: first half cos, second half sin.

    rope_scaling: HF config.json dict. Supported: "llama3" (Llama-3.1/3.2
    wavelength remap, transformers modeling_rope_utils
    _compute_llama3_parameters) and "linear" (position interpolation —
    dividing inv_freq by factor is identical to dividing positions).
    Unknown types raise rather than silently serving wrong rotations.
    """
    import math as _math

    inv_freq = 1.0 / (
        theta ** (torch.arange(0, rotary_dim, 2, device=device, dtype=torch.float32) / rotary_dim)
    )
    if rope_scaling:
        rtype = rope_scaling.get("rope_type") or rope_scaling.get("type")
        factor = float(rope_scaling.get("factor", 1.0))
        if rtype == "llama3":
            low = float(rope_scaling["low_freq_factor"])
            high = float(rope_scaling["high_freq_factor"])
            orig = float(rope_scaling["original_max_position_embeddings"])
            wavelen = 2 * _math.pi / inv_freq
            smooth = (orig / wavelen - low) / (high - low)
            smoothed = (1 - smooth) * inv_freq / factor + smooth * inv_freq
            inv_freq = torch.where(
                wavelen < orig / high, inv_freq,
                torch.where(wavelen > orig / low, inv_freq / factor, smoothed),
            )
        elif rtype == "linear":
            inv_freq = inv_freq / factor
        elif rtype in (None, "default"):
            pass
        else:
            raise ValueError(f"unsupported rope_scaling type: {rtype!r}")
    t = torch.arange(max_positions, device=device, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)  # [P, rotary_dim/2]
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1).to(dtype)


def rope_inplace(
    q: torch.Tensor,  # [T, num_heads, head_dim]
    k: torch.Tensor,  # [T, num_kv_heads, head_dim]
    positions: torch.Tensor,  # [T]
    cos_sin: torch.Tensor,  # [max_pos, head_dim] (cos || sin)
) -> None:
    """NeoX-style (rotate-half) RoPE applied in place to q and k."""
    half = q.shape[-1] // 2
    cs = cos_sin[positions]  # [T, head_dim]
    cos = cs[:, :half].unsqueeze(1)  # [T, 1, half]
    sin = cs[:, half:].unsqueeze(1)
    for t in (q, k):
        # clone: for f32 inputs .float() aliases, and the first write below
        # would corrupt x1 before the second line reads it
        x1 = t[..., :half].float().clone()
        x2 = t[..., half:].float().clone()
        t[..., :half] = (x1 * cos - x2 * sin).to(t.dtype)
        t[..., half:] = (x2 * cos + x1 * sin).to(t.dtype)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """x = [*, 2*d]: silu(x[..., :d]) * x[..., d:]."""
    d = x.shape[-1] // 2
    a, b = x[..., :d], x[..., d:]
    return (torch.nn.functional.silu(a.float()) * b.float()).to(x.dtype)


def gelu_tanh_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    a, b = x[..., :d], x[..., d:]
    return (torch.nn.functional.gelu(a.float(), approximate="tanh") * b.float()).to(x.dtype)


def reshape_and_cache(
    key: torch.Tensor,  # [T, kv_heads, head_dim]
    value: torch.Tensor,
    k_cache: torch.Tensor,  # [num_blocks, kv_heads, block_size, head_dim]
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,  # [T] int32/int64 global slot ids
) -> None:
    block_size = k_cache.shape[2]
    slots = slot_mapping.long()
    blocks = slots // block_size
    offs = slots % block_size
    k_cache[blocks, :, offs, :] = key.to(k_cache.dtype)
    v_cache[blocks, :, offs, :] = value.to(v_cache.dtype)


def _softcap(scores: torch.Tensor, cap: float) -> torch.Tensor:
    if cap and cap > 0:
        return torch.tanh(scores / cap) * cap
    return scores


def paged_decode_attention(
    q: torch.Tensor,  # [B, num_heads, head_dim]
    k_cache: torch.Tensor,  # [num_blocks, kv_heads, block_size, head_dim]
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [B, max_blocks] int32
    context_lens: torch.Tensor,  # [B] int32 (length INCLUDING current token)
    scale: float,
    softcap: float = 0.0,
    window: int = 0,
) -> torch.Tensor:
    """Single-token decode attention over the paged cache (reference)."""
    B, H, D = q.shape
    KVH = k_cache.shape[1]
    bs = k_cache.shape[2]
    group = H // KVH
    out = torch.empty_like(q)
    for b in range(B):
        L = int(context_lens[b])
        nblocks = (L + bs - 1) // bs
        blocks = block_tables[b, :nblocks].long()
        k = k_cache[blocks].permute(1, 0, 2, 3).reshape(KVH, nblocks * bs, D)[:, :L]
        v = v_cache[blocks].permute(1, 0, 2, 3).reshape(KVH, nblocks * bs, D)[:, :L]
        start = max(0, L - window) if window else 0
        k, v = k[:, start:], v[:, start:]
        qb = q[b].view(KVH, group, D).float()  # [KVH, G, D]
        scores = torch.einsum("hgd,hld->hgl", qb, k.float()) * scale
        scores = _softcap(scores, softcap)
        probs = torch.softmax(scores, dim=-1)
        ob = torch.einsum("hgl,hld->hgd", probs, v.float())
        out[b] = ob.reshape(H, D).to(q.dtype)
    return out


def varlen_prefill_attention(
    q: torch.Tensor,  # [Tq, num_heads, head_dim]
    k: torch.Tensor,  # [Tk, kv_heads, head_dim]
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,  # [B+1] query offsets
    scale: float,
    softcap: float = 0.0,
    window: int = 0,
    cu_seqlens_k: "Optional[torch.Tensor]" = None,  # [B+1] key offsets
) -> torch.Tensor:
    """Causal attention over packed variable-length sequences (reference).

    With cu_seqlens_k, each sequence's K/V may be LONGER than its Q (chunked
    prefill: the queries are the last Tq positions of a Tk-long context);
    query row i has absolute position (Tk - Tq) + i."""
    T, H, D = q.shape
    KVH = k.shape[1]
    group = H // KVH
    cu_k = cu_seqlens if cu_seqlens_k is None else cu_seqlens_k
    out = torch.empty_like(q)
    for b in range(len(cu_seqlens) - 1):
        s, e = int(cu_seqlens[b]), int(cu_seqlens[b + 1])
        sk, ek = int(cu_k[b]), int(cu_k[b + 1])
        Lq, Lk = e - s, ek - sk
        off = Lk - Lq  # absolute position of q row 0
        qb = q[s:e].float()  # [Lq, H, D]
        kb = k[sk:ek].float().repeat_interleave(group, dim=1)  # [Lk, H, D]
        vb = v[sk:ek].float().repeat_interleave(group, dim=1)
        scores = torch.einsum("ihd,jhd->hij", qb, kb) * scale
        scores = _softcap(scores, softcap)
        i = torch.arange(Lq, device=q.device).view(-1, 1) + off
        j = torch.arange(Lk, device=q.device).view(1, -1)
        mask = j > i
        if window:
            mask = mask | (j <= i - window)
        scores.masked_fill_(mask.unsqueeze(0), float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        ob = torch.einsum("hij,jhd->ihd", probs, vb)
        out[s:e] = ob.to(q.dtype)
    return out


def sample_tokens(
    logits: torch.Tensor,  # [B, vocab] float
    temperatures: torch.Tensor,  # [B]
    top_ps: torch.Tensor,  # [B]
    top_ks: torch.Tensor,  # [B] int (0 = off)
    generator: Optional[torch.Generator] = None,
) -> torch.Tensor:
    """Temperature / top-k / top-p sampling; greedy where temperature == 0."""
    B, V = logits.shape
    out = torch.empty(B, dtype=torch.long, device=logits.device)
    greedy_mask = temperatures <= 0
    if greedy_mask.any():
        out[greedy_mask] = logits[greedy_mask].argmax(dim=-1)
    sample_idx = (~greedy_mask).nonzero(as_tuple=True)[0]
    for i in sample_idx.tolist():
        l = logits[i].float() / float(temperatures[i])
        k = int(top_ks[i])
        if k > 0 and k < V:
            kth = torch.topk(l, k).values[-1]
            l = torch.where(l < kth, torch.full_like(l, float("-inf")), l)
        p = float(top_ps[i])
        if p < 1.0:
            sorted_l, sorted_i = torch.sort(l, descending=True)
            probs = torch.softmax(sorted_l, dim=-1)
            cum = torch.cumsum(probs, dim=-1)
            cut = (cum - probs) >= p  # keep tokens whose preceding mass < p
            sorted_l[cut] = float("-inf")
            l = torch.full_like(l, float("-inf")).scatter(0, sorted_i, sorted_l)
        probs = torch.softmax(l, dim=-1)
        out[i] = torch.multinomial(probs, 1, generator=generator).squeeze(0)
    return out


# ----------------------------------------------------- hybrid decoders ----
# Reference forms of the hybrid-decoder ops (fp32 residual stream, block-
# local biased attention over the paged cache, gated-linear-attention
# recurrence over state slots). Same contracts as the HIP kernels.


def rmsnorm_cast(x: torch.Tensor, weight: torch.Tensor, eps: float, offset: float,
                 out_dtype: torch.dtype, groups: int = 1) -> torch.Tensor:
    """groups > 1: the row is split into that many equal consecutive parts,
    each divided by its own root mean square."""
    xf = x.float()
    if groups > 1:
        xf = xf.unflatten(-1, (groups, x.shape[-1] // groups))
    inv = 1.0 / torch.sqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    xf = xf * inv
    if groups > 1:
        xf = xf.flatten(-2)
    return (xf * (weight.float() + offset)).to(out_dtype)


def sandwich_norm_res32(x, residual, w_post, w_pre, eps, offset, groups=1):
    """residual(fp32) += rmsnorm(x)*(w_post+offset); returns
    rmsnorm(residual)*(w_pre+offset) in x's dtype. residual updated in place."""
    residual.add_(rmsnorm_cast(x, w_post, eps, offset, torch.float32, groups))
    return rmsnorm_cast(residual, w_pre, eps, offset, x.dtype, groups)


def act_and_mul(x: torch.Tensor, gelu: bool) -> torch.Tensor:
    return gelu_tanh_and_mul(x) if gelu else silu_and_mul(x)


def qknorm_vmix_cache(q, k, v, q_w, k_w, v_first, lam, k_cache, v_cache, slots, eps):
    """q [T, nq] normalised in place over its whole width; k normalised and
    v (blended with v_first when given) scattered into the paged cache."""
    q.copy_(rmsnorm_cast(q, q_w, eps, 0.0, q.dtype))
    kn = rmsnorm_cast(k, k_w, eps, 0.0, k.dtype)
    vv = v.float()
    if v_first is not None:
        vv = (1.0 - lam) * vv + lam * v_first.float()
    G, bs, D = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    DV = v_cache.shape[3]
    keep = slots >= 0
    s = slots[keep].long()
    k_cache[s // bs, :, s % bs, :] = kn[keep].view(-1, G, D).to(k_cache.dtype)
    v_cache[s // bs, :, s % bs, :] = vv[keep].view(-1, G, DV).to(v_cache.dtype)


def _block_local_attend(qb, kc, vc, bias, pos, span, scale, gate):
    """qb [n, H, D] at absolute positions pos [n]; kc [L, G, D], vc [L, G, DV]
    the sequence's cached keys/values for positions 0..L-1."""
    n, H, _ = qb.shape
    G = kc.shape[1]
    lo = int(pos[0]) // span * span
    kk = kc[lo:].float().repeat_interleave(H // G, dim=1)
    vv = vc[lo:].float().repeat_interleave(H // G, dim=1)
    j = torch.arange(lo, kc.shape[0], device=qb.device).view(1, -1)
    i = pos.view(-1, 1)
    vis = (j <= i) & (j // span == i // span)
    dist = (i - j).clamp_(0, bias.shape[1] - 1)
    scores = torch.einsum("ihd,jhd->hij", qb.float(), kk) * scale
    scores = scores + bias[:, dist]
    scores = scores.masked_fill(~vis.unsqueeze(0), float("-inf"))
    out = torch.einsum("hij,jhd->ihd", torch.softmax(scores, dim=-1), vv)
    if gate is not None:
        out = out * torch.sigmoid(gate.float()).unsqueeze(-1)
    return out


def _gather_seq(cache, table, length):
    bs = cache.shape[2]
    nb = (length + bs - 1) // bs
    blocks = table[:nb].long()
    return cache[blocks].permute(0, 2, 1, 3).reshape(nb * bs, cache.shape[1], cache.shape[3])[:length]


def chunk_bias_attn_prefill(q, gate, k_cache, v_cache, bias, block_tables, cu_q, q_start,
                            span, scale):
    T, H, _ = q.shape
    out = q.new_empty(T, H, v_cache.shape[3])
    for b in range(len(q_start)):
        s, e = int(cu_q[b]), int(cu_q[b + 1])
        if e == s:
            continue
        p0 = int(q_start[b])
        L = p0 + (e - s)
        kc = _gather_seq(k_cache, block_tables[b], L)
        vc = _gather_seq(v_cache, block_tables[b], L)
        pos = torch.arange(p0, L, device=q.device)
        # rows of one portion may straddle several spans: attend span by span
        start = 0
        while start < e - s:
            first = p0 + start
            stop = min(e - s, start + (span - first % span))
            rows = slice(s + start, s + stop)
            out[rows] = _block_local_attend(
                q[rows], kc[: p0 + stop], vc[: p0 + stop], bias, pos[start:stop], span, scale,
                None if gate is None else gate[rows],
            ).to(q.dtype)
            start = stop
    return out


def chunk_bias_attn_decode(q, gate, k_cache, v_cache, bias, block_tables, context_lens,
                           span, scale):
    B, H, _ = q.shape
    out = q.new_empty(B, H, v_cache.shape[3])
    for b in range(B):
        L = int(context_lens[b])
        kc = _gather_seq(k_cache, block_tables[b], L)
        vc = _gather_seq(v_cache, block_tables[b], L)
        pos = torch.tensor([L - 1], device=q.device)
        out[b : b + 1] = _block_local_attend(
            q[b : b + 1], kc, vc, bias, pos, span, scale,
            None if gate is None else gate[b : b + 1],
        ).to(q.dtype)
    return out


def gla_recurrence(q, k, v, z, z_bias, state, cu, slots, fresh, tau):
    """q,k,z [T,H,D], v [T,H,DV] → o [T,H,DV] fp32; state [slots,H,D,DV] fp32
    advanced in place (zero start where fresh)."""
    T, H, D = q.shape
    o = torch.empty(T, H, v.shape[2], dtype=torch.float32, device=q.device)
    zf = z.float() + z_bias.view(1, H, D)
    alpha = torch.exp(torch.nn.functional.logsigmoid(zf) / tau)
    qf = q.float() * (1.0 / (D ** 0.5))
    kf, vf = k.float(), v.float()
    for b in range(len(slots)):
        s, e = int(cu[b]), int(cu[b + 1])
        slot = int(slots[b])
        S = torch.zeros_like(state[slot]) if int(fresh[b]) else state[slot].clone()
        for t in range(s, e):
            S = alpha[t].unsqueeze(-1) * S + kf[t].unsqueeze(-1) * vf[t].unsqueeze(-2)
            o[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[slot] = S
    return o


def gla_out_norm_gate(o, weight, gate, eps, out_dtype):
    T, H, DV = o.shape
    y = o * (1.0 / torch.sqrt(o.pow(2).mean(dim=-1, keepdim=True) + eps)) * weight.float()
    y = y.reshape(T, H * DV) * torch.nn.functional.silu(gate.float())
    return y.to(out_dtype)


# ------------------------------------------- looped hybrid decoders (ref) --
# Reference forms of the ops added for latent attention, lower-bounded
# forget-gate recurrences, gated parallel residuals and expert mixtures.


def _window_attend(qb, kc, vc, pos, window, scale, log_bias=None, keep_first=0, sink=None,
                   softcap=0.0):
    """qb [n, H, D] at absolute positions pos [n]; kc [L, G, D], vc [L, G, DV]
    cached keys/values of positions 0..L-1. Query i sees key j iff j <= i
    and (window == 0 or i - j < window or j < keep_first). log_bias [H, 2] =
    (r1, r2) per head takes r1 * ln(1 + r2 * (i - j)) off the scaled score.
    softcap c > 0: the scaled score becomes c * tanh(score / c). sink [H]:
    the softmax denominator gains exp(sink[h])."""
    n, H, _ = qb.shape
    G = kc.shape[1]
    lo = max(0, int(pos[0]) - window + 1) if window and not keep_first else 0
    kk = kc[lo:].float().repeat_interleave(H // G, dim=1)
    vv = vc[lo:].float().repeat_interleave(H // G, dim=1)
    j = torch.arange(lo, kc.shape[0], device=qb.device).view(1, -1)
    i = pos.view(-1, 1)
    vis = j <= i
    if window:
        vis = vis & ((i - j < window) | (j < keep_first))
    scores = torch.einsum("ihd,jhd->hij", qb.float(), kk) * scale
    if softcap:
        scores = softcap * torch.tanh(scores / softcap)
    if log_bias is not None:
        dist = (i - j).clamp(min=0).float().unsqueeze(0)
        r1, r2 = log_bias[:, 0].float().view(-1, 1, 1), log_bias[:, 1].float().view(-1, 1, 1)
        scores = scores - r1 * torch.log1p(r2 * dist)
    scores = scores.masked_fill(~vis.unsqueeze(0), float("-inf"))
    if sink is not None:
        extra = sink.float().view(-1, 1, 1).expand(H, n, 1)
        w = torch.softmax(torch.cat([scores, extra], dim=-1), dim=-1)[..., :-1]
    else:
        w = torch.softmax(scores, dim=-1)
    return torch.einsum("hij,jhd->ihd", w, vv)


def window_attn_prefill(q, k_cache, v_cache, dv, block_tables, cu_q, q_start, window, scale,
                        log_bias=None, keep_first=0, sink=None, softcap=0.0):
    """Causal / sliding-window softmax attention of packed prompt portions
    over the paged cache. v_cache None: a key row's first dv channels are
    its value."""
    T, H, _ = q.shape
    out = q.new_empty(T, H, dv)
    for b in range(len(q_start)):
        s, e = int(cu_q[b]), int(cu_q[b + 1])
        if e == s:
            continue
        p0 = int(q_start[b])
        L = p0 + (e - s)
        kc = _gather_seq(k_cache, block_tables[b], L)
        vc = kc[..., :dv] if v_cache is None else _gather_seq(v_cache, block_tables[b], L)
        pos = torch.arange(p0, L, device=q.device)
        out[s:e] = _window_attend(q[s:e], kc, vc, pos, window, scale, log_bias, keep_first,
                                  sink, softcap).to(q.dtype)
    return out


def window_attn_decode(q, k_cache, v_cache, dv, block_tables, context_lens, window, scale,
                       log_bias=None, keep_first=0, sink=None, softcap=0.0):
    B, H, _ = q.shape
    out = q.new_empty(B, H, dv)
    for b in range(B):
        L = int(context_lens[b])
        kc = _gather_seq(k_cache, block_tables[b], L)
        vc = kc[..., :dv] if v_cache is None else _gather_seq(v_cache, block_tables[b], L)
        pos = torch.tensor([L - 1], device=q.device)
        out[b : b + 1] = _window_attend(q[b : b + 1], kc, vc, pos, window, scale,
                                        log_bias, keep_first, sink, softcap).to(q.dtype)
    return out


def _rotate(x, positions, inv_freq, rot_dims, interleaved):
    """x [T, ..., n] fp32: rotary positions on its first rot_dims channels."""
    half = rot_dims // 2
    ang = positions.float().view(-1, *([1] * (x.dim() - 2)), 1) * inv_freq.float()
    cos, sin = torch.cos(ang), torch.sin(ang)
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
        out[..., 0:rot_dims:2] = u * cos - v * sin
        out[..., 1:rot_dims:2] = v * cos + u * sin
    else:
        u, v = x[..., :half], x[..., half:rot_dims]
        out[..., :half] = u * cos - v * sin
        out[..., half:rot_dims] = v * cos + u * sin
    return out


def latent_rope_pack(q, q_lat, ckr, c_w, inv_freq, positions, k_cache, slots, dim, rot_dims,
                     interleaved, eps):
    """q [T, H, dim+DR] (projection), q_lat [T, H, R] (its unrotated part
    mapped into the latent), ckr [T, R+DR] (latent ‖ rotated key part).
    Returns the packed query [T, H, R+DR] = q_lat ‖ rotate(q[..., dim:]) and
    scatters rmsnorm(latent)*c_w ‖ rotate(key part) into the paged cache
    [blocks, 1, bs, R+DR]."""
    T, H, _ = q.shape
    R = q_lat.shape[2]
    q_rot = _rotate(q[..., dim:].float(), positions, inv_freq, rot_dims, interleaved)
    out = torch.cat([q_lat.float(), q_rot], dim=-1).to(q.dtype)
    c = rmsnorm_cast(ckr[:, :R], c_w, eps, 0.0, torch.float32)
    k_rot = _rotate(ckr[:, R:].float(), positions, inv_freq, rot_dims, interleaved)
    row = torch.cat([c, k_rot], dim=-1)
    bs = k_cache.shape[2]
    keep = slots >= 0
    s = slots[keep].long()
    k_cache[s // bs, 0, s % bs, :] = row[keep].to(k_cache.dtype)
    return out


def gated_recurrence(q, k, v, z, z_bias, state, cu, slots, fresh, tau, lower, q_silu, q_scale):
    """The diagonal-decay recurrence S <- diag(a) S + w v^T, o = S^T q over
    packed sequences. lower None: a = sigmoid(z + b)^(1/tau), w = k.
    lower given: a = l + (1 - l) * sigmoid(z + b), w = 1 - a (k unused)."""
    T, H, D = q.shape
    o = torch.empty(T, H, v.shape[2], dtype=torch.float32, device=q.device)
    zf = z.float() + z_bias.view(1, H, D)
    if lower is None:
        alpha = torch.exp(torch.nn.functional.logsigmoid(zf) / tau)
        kf = k.float()
    else:
        lo = lower.float().view(1, H, D)
        alpha = lo + (1.0 - lo) * torch.sigmoid(zf)
        kf = 1.0 - alpha
    qf = q.float()
    if q_silu:
        qf = torch.nn.functional.silu(qf)
    qf = qf * q_scale
    vf = v.float()
    for b in range(len(slots)):
        s, e = int(cu[b]), int(cu[b + 1])
        slot = int(slots[b])
        S = torch.zeros_like(state[slot]) if int(fresh[b]) else state[slot].clone()
        for t in range(s, e):
            S = alpha[t].unsqueeze(-1) * S + kf[t].unsqueeze(-1) * vf[t].unsqueeze(-2)
            o[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[slot] = S
    return o


def head_norm(o, weight, eps, out_dtype):
    """Per-head RMSNorm over the value size of o [T, H, DV] fp32 -> [T, H*DV]."""
    T, H, DV = o.shape
    y = o * (1.0 / torch.sqrt(o.pow(2).mean(dim=-1, keepdim=True) + eps)) * weight.float()
    return y.reshape(T, H * DV).to(out_dtype)


def gated_residual_add(res, y1, g1, b1, y2, g2, b2, out_dtype):
    """res (fp32, in place) += sigmoid(g1 + b1) * y1 [+ sigmoid(g2 + b2) * y2];
    returns res rounded to out_dtype."""
    add = torch.sigmoid(g1.float() + b1.float()) * y1.float()
    if y2 is not None:
        add = add + torch.sigmoid(g2.float() + b2.float()) * y2.float()
    res.add_(add)
    return res.to(out_dtype)


def side_gate_mul(a, table, tokens, offset):
    """gelu_tanh(a) * table[tokens, offset : offset + a.shape[1]] in a's dtype."""
    e = table[tokens][:, offset : offset + a.shape[1]].float()
    return (torch.nn.functional.gelu(a.float(), approximate="tanh") * e).to(a.dtype)


def sigmoid_topk(logits, top):
    """Router: scores = sigmoid(logits) (fp32); the `top` largest per row.
    Returns (indices int32 [T, top], scores fp32 [T, top])."""
    s = torch.sigmoid(logits.float())
    w, idx = torch.topk(s, top, dim=-1)
    return idx.to(torch.int32), w


# ------------------------------ scan hybrids (minGRU / selective scan) ref --
# Reference forms of the ops added for decoders built from elementwise gated
# recurrences, selective scans beside attention, softmax-routed clamped
# experts and a learned average over layer outputs.


def sinusoid_inv_freq(width: int) -> torch.Tensor:
    """fp32 table 10000^(-2i/width), one entry per (sin, cos) pair, rounded
    once from float64."""
    i = torch.arange((width + 1) // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(10000.0, dtype=torch.float64), -2.0 * i / width).float()


def embed_sinusoid(embedding, ids, positions, inv_freq):
    """fp32 [T, W]: embedding[ids] plus the sinusoidal position vector, entry
    2i = sin(p * inv_freq[i]), entry 2i+1 = cos of the same angle (fp32)."""
    x = embedding[ids].float()
    W = x.shape[1]
    ang = positions.float().unsqueeze(1) * inv_freq.float().unsqueeze(0)
    pe = torch.stack([torch.sin(ang), torch.cos(ang)], dim=-1).reshape(x.shape[0], -1)[:, :W]
    return x + pe


def scaled_add_norm(res, y, y2, a1, a2, weight, eps, out_dtype):
    """res (fp32, in place) += a1 * y [+ a2 * y2]; returns rmsnorm(res) * weight."""
    add = a1 * y.float()
    if y2 is not None:
        add = add + a2 * y2.float()
    res.add_(add)
    return rmsnorm_cast(res, weight, eps, 0.0, out_dtype)


def depth_mix_norm(stack, n, coef, y, y2, a1, a2, weight, eps, out_dtype):
    """stack [>= n+1, T, W] fp32 holds the embedding output and the layer
    results so far in rows 0..n-1. Row n-1 (in place) += a1 * y [+ a2 * y2];
    row n = sum_j coef[j] * row j (j < n); returns rmsnorm(row n) * weight."""
    add = a1 * y.float()
    if y2 is not None:
        add = add + a2 * y2.float()
    stack[n - 1].add_(add)
    mix = torch.einsum("j,jtw->tw", coef.float()[:n], stack[:n])
    stack[n].copy_(mix)
    return rmsnorm_cast(stack[n], weight, eps, 0.0, out_dtype)


def kv_scatter(k, v, k_cache, v_cache, slots):
    """k [T, G*D], v [T, G*DV] scattered into the paged cache rows `slots`
    (negative: skipped)."""
    G, bs, D = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    DV = v_cache.shape[3]
    keep = slots >= 0
    s = slots[keep].long()
    k_cache[s // bs, :, s % bs, :] = k[keep].reshape(-1, G, D).to(k_cache.dtype)
    v_cache[s // bs, :, s % bs, :] = v[keep].reshape(-1, G, DV).to(v_cache.dtype)


def mingru_scan(z, u, g, z_b, u_b, state, cu, slots, fresh, out_dtype):
    """minGRU over packed sequences. z, u, g [T, n] projections; gate
    a = sigmoid(z + z_b), candidate c = u' + 1/2 (u' >= 0) or sigmoid(u')
    with u' = u + u_b; S <- (1 - a) S + a c per channel (fp32 state
    [slots, n], advanced in place, zero start where fresh); returns
    S_t * silu(g_t) in out_dtype."""
    a = torch.sigmoid(z.float() + z_b.float())
    uu = u.float() + u_b.float()
    c = torch.where(uu >= 0, uu + 0.5, torch.sigmoid(uu))
    out = torch.empty(z.shape, dtype=torch.float32, device=z.device)
    for b in range(len(slots)):
        s, e = int(cu[b]), int(cu[b + 1])
        slot = int(slots[b])
        S = torch.zeros_like(state[slot]) if int(fresh[b]) else state[slot].clone()
        for t in range(s, e):
            S = (1.0 - a[t]) * S + a[t] * c[t]
            out[t] = S
        state[slot] = S
    return (out * torch.nn.functional.silu(g.float())).to(out_dtype)


def causal_conv_silu(x, weight, bias, tail, cu, slots, fresh, silu=True):
    """Per-channel causal convolution (+ SiLU unless silu is False; bias may
    be None) over packed sequences.
    x [T, C]; weight [C, K] fp32 (last column = the current token's tap);
    bias [C] fp32; tail [slots, K-1, C] fp32 holds each sequence's last K-1
    inputs (zeros before the start), advanced in place. Returns [T, C] in
    x's dtype."""
    K = weight.shape[1]
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    xf = x.float()
    for b in range(len(slots)):
        s, e = int(cu[b]), int(cu[b + 1])
        slot = int(slots[b])
        past = torch.zeros_like(tail[slot]) if int(fresh[b]) else tail[slot].clone()
        seq = torch.cat([past, xf[s:e]], dim=0)          # [K-1 + n, C]
        n = e - s
        acc = torch.zeros(n, x.shape[1], dtype=torch.float32, device=x.device)
        if bias is not None:
            acc += bias.float()
        for k in range(K):
            acc += seq[k:k + n] * weight[:, k].float()
        out[s:e] = acc
        if K > 1:
            tail[slot] = seq[seq.shape[0] - (K - 1):]
    return (torch.nn.functional.silu(out) if silu else out).to(x.dtype)


def selective_scan(x, dt, dt_b, A, Bm, Cm, D, z, state, cu, slots, fresh):
    """Selective scan over packed sequences. x, dt, z [T, C]; Bm, Cm [T, N];
    dt_b, D [C] fp32; A [C, N] fp32 (negative); state [slots, C, N] fp32
    advanced in place. step = softplus(dt + dt_b);
    S <- exp(step A) S + step x B;  y = S C + D x;  returns y * silu(z)."""
    step = torch.nn.functional.softplus(dt.float() + dt_b.float())
    xf, Bf, Cf = x.float(), Bm.float(), Cm.float()
    y = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    for b in range(len(slots)):
        s, e = int(cu[b]), int(cu[b + 1])
        slot = int(slots[b])
        S = torch.zeros_like(state[slot]) if int(fresh[b]) else state[slot].clone()
        for t in range(s, e):
            S = torch.exp(step[t].unsqueeze(1) * A) * S \
                + (step[t] * xf[t]).unsqueeze(1) * Bf[t].unsqueeze(0)
            y[t] = S @ Cf[t] + D * xf[t]
        state[slot] = S
    return (y * torch.nn.functional.silu(z.float())).to(x.dtype)


def softmax_topk(logits, top, scale, correction=None, renorm=False):
    """Router: scores = softmax(logits) over all experts (fp32); the `top`
    largest per row, times scale. correction [E]: the choice is made on
    score + correction, the weights stay the plain scores. renorm: the chosen
    scores are divided by their sum (+ 1e-20) first. Returns (indices int32,
    weights fp32)."""
    s = torch.softmax(logits.float(), dim=-1)
    if correction is None:
        w, idx = torch.topk(s, top, dim=-1)
    else:
        idx = torch.topk(s + correction.float(), top, dim=-1).indices
        w = torch.gather(s, 1, idx)
    if renorm:
        w = w / (w.sum(dim=-1, keepdim=True) + 1e-20)
    return idx.to(torch.int32), w * scale


def clamp_swish_mul(x, limit):
    """[*, 2d] -> g * sigmoid(1.702 g) * (u + 1) with g = min(x[..., :d], limit)
    and u = clamp(x[..., d:], -limit, limit)."""
    d = x.shape[-1] // 2
    g = x[..., :d].float().clamp(max=limit)
    u = x[..., d:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)).to(x.dtype)


def softcap(x, cap):
    return cap * torch.tanh(x.float() / cap)


# --------------------------- windowed attention beside a matrix memory (ref) --
# Reference forms of the ops added for decoders whose norms work on groups of
# the width, whose attention keeps its first tokens and a learned term in the
# softmax denominator or rotates its values, and whose recurrent mixer is an
# mLSTM matrix memory.


def qkv_norm_rope_cache(q, k, v, q_w, k_w, inv_freq, rot_dims, positions, k_cache, v_cache,
                        slots, eps, v_unit_norm, v_inv_freq):
    """Per token, between the projections and the attention kernel. q [T, H, D]
    (updated in place), k [T, G, D], v [T, G, DV] or None (the values are then
    the keys as they arrive). q_w / k_w [D] or None: per-head RMSNorm with that
    weight first. Rotary positions (fp32 angle position * inv_freq[i], pairs
    (i, i + rot_dims/2)) on the first rot_dims channels of q and k.
    v_unit_norm: each head's value divided by its root mean square;
    v_inv_freq [DV/2]: the value turned by its position over all DV channels.
    k and v go to the paged cache rows `slots` (negative: skipped)."""
    T, H, D = q.shape
    G = k.shape[1]
    raw_k = k.float()
    qf, kf = q.float(), raw_k
    if q_w is not None:
        qf = qf / torch.sqrt(qf.pow(2).mean(-1, keepdim=True) + eps) * q_w.float()
    if k_w is not None:
        kf = kf / torch.sqrt(kf.pow(2).mean(-1, keepdim=True) + eps) * k_w.float()
    if rot_dims:
        qf = _rotate(qf, positions, inv_freq, rot_dims, False)
        kf = _rotate(kf, positions, inv_freq, rot_dims, False)
    vf = raw_k if v is None else v.float()
    if v_unit_norm:
        vf = vf / torch.sqrt(vf.pow(2).mean(-1, keepdim=True) + eps)
    if v_inv_freq is not None:
        vf = _rotate(vf, positions, v_inv_freq, vf.shape[-1], False)
    q.copy_(qf.to(q.dtype))
    bs = k_cache.shape[2]
    keep = slots >= 0
    s = slots[keep].long()
    k_cache[s // bs, :, s % bs, :] = kf[keep].to(k_cache.dtype)
    v_cache[s // bs, :, s % bs, :] = vf[keep].to(v_cache.dtype)


def rotate_heads(x, positions, inv_freq, inverse):
    """x [T, H, n] in place: every head turned by (minus, if inverse) its
    token's position over all n channels, pairs (i, i + n/2)."""
    ang = inv_freq if not inverse else -inv_freq
    x.copy_(_rotate(x.float(), positions, ang, x.shape[-1], False).to(x.dtype))
    return x


def mlstm_gates(gates, cap, m_state, cu, slots, fresh):
    """gates [T, 2H] fp32 = (input | forget) pre-activations. Per head:
    i = cap tanh(g_i / cap), f = logsigmoid(cap tanh(g_f / cap)),
    m_t = max(f + m_(t-1), i) with m = 0 before a sequence's first token.
    Returns fp32 [T, H] each: decay e^(f + m_(t-1) - m_t), write e^(i - m_t),
    floor e^(-m_t); m_state [slots, H] advanced in place."""
    T, H2 = gates.shape
    H = H2 // 2
    gi = cap * torch.tanh(gates[:, :H].float() / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh(gates[:, H:].float() / cap))
    decay = torch.empty(T, H, dtype=torch.float32, device=gates.device)
    write, floor = torch.empty_like(decay), torch.empty_like(decay)
    for b in range(len(slots)):
        s, e = int(cu[b]), int(cu[b + 1])
        slot = int(slots[b])
        m = torch.zeros(H, dtype=torch.float32, device=gates.device) if int(fresh[b]) \
            else m_state[slot].clone()
        for t in range(s, e):
            new = torch.maximum(gf[t] + m, gi[t])
            decay[t] = torch.exp(gf[t] + m - new)
            write[t] = torch.exp(gi[t] - new)
            floor[t] = torch.exp(-new)
            m = new
        m_state[slot] = m
    return decay, write, floor


def matrix_memory(q, k, v, decay, write, state, cu, slots, fresh, q_scale):
    """S <- decay S + write k v'^T per head over packed sequences with
    v' = [v | 1] (the last column carries the normaliser), o = S^T (q_scale q).
    q, k [T, H, D], v [T, H, DV], decay / write [T, H] fp32; state
    [slots, H, D, DV + 1] fp32 advanced in place. Returns o [T, H, DV + 1]."""
    T, H, D = q.shape
    DV = v.shape[2]
    o = torch.empty(T, H, DV + 1, dtype=torch.float32, device=q.device)
    qf = q.float() * q_scale
    kf = k.float() * write.unsqueeze(-1)
    vf = torch.cat([v.float(), torch.ones(T, H, 1, device=q.device)], dim=-1)
    for b in range(len(slots)):
        s, e = int(cu[b]), int(cu[b + 1])
        slot = int(slots[b])
        S = torch.zeros_like(state[slot]) if int(fresh[b]) else state[slot].clone()
        for t in range(s, e):
            S = decay[t].view(H, 1, 1) * S + kf[t].unsqueeze(-1) * vf[t].unsqueeze(-2)
            o[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[slot] = S
    return o


def mlstm_out_norm_gate(o, floor, weight, gate, eps, out_dtype):
    """o [T, H, DV + 1] (last column n . q), floor [T, H]: each head's
    o[..., :DV] / (max(|n . q|, floor) + 1e-6), divided by its root mean
    square, times weight [H * DV], times sigmoid(gate [T, H * DV])."""
    T, H, DV1 = o.shape
    DV = DV1 - 1
    den = torch.maximum(o[..., DV].abs(), floor) + 1e-6
    y = o[..., :DV] / den.unsqueeze(-1)
    y = y / torch.sqrt(y.pow(2).mean(dim=-1, keepdim=True) + eps)
    y = y.reshape(T, H * DV) * weight.float() * torch.sigmoid(gate.float())
    return y.to(out_dtype)


def dual_norm_mean(a, w_a, b, w_b, eps):
    """(rmsnorm(a) * w_a + rmsnorm(b) * w_b) / 2 in a's dtype."""
    ya = rmsnorm_cast(a, w_a, eps, 0.0, torch.float32)
    yb = rmsnorm_cast(b, w_b, eps, 0.0, torch.float32)
    return (0.5 * (ya + yb)).to(a.dtype)


def unary_act(x, kind):
    """relu2: max(x, 0)^2; gelu_erf: the exact GELU."""
    xf = x.float()
    if kind == "relu2":
        y = torch.relu(xf).pow(2)
    elif kind == "gelu_erf":
        y = torch.nn.functional.gelu(xf)
    else:
        raise ValueError(f"unknown activation {kind!r}")
    return y.to(x.dtype)

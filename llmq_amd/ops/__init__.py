"""Op dispatch: hand-written CDNA4 HIP kernels on GPU, torch reference on CPU.

Policy (per the build contract): on a GPU box the HIP extension MUST be
present and is ALWAYS used — if `torch.cuda.is_available()` and the
extension failed to load, every op raises instead of silently falling back
to eager PyTorch. On CPU (tests, this dev container) the torch reference
implementations run.
"""

from __future__ import annotations

import os
from pathlib import Path
from typing import Optional, Tuple

import torch

from llmq_amd.ops import torch_ref

_EXT = None
_EXT_ERROR: Optional[str] = None
_EXT_TRIED = False


def _try_load_extension() -> None:
    """Lazy: called on first use, NOT at import (so `python -m
    llmq_amd.ops.build` can rebuild without a namespace clash against a
    stale loaded .so)."""
    global _EXT, _EXT_ERROR, _EXT_TRIED
    if _EXT_TRIED:
        return
    _EXT_TRIED = True
    # A build in this very process (ops.build.build / ensure) has already
    # loaded the library it produced: loading the copied file again would
    # register the namespace twice, which aborts the process.
    try:
        torch.ops.llmq_amd.rmsnorm  # noqa: B018
        _EXT = torch.ops.llmq_amd
        return
    except (AttributeError, RuntimeError):
        pass
    here = Path(__file__).parent
    override = os.environ.get("LLMQ_OPS_SO")
    if override:
        candidates = [Path(override)]
    else:
        candidates = sorted(here.glob("_hip_ops*.so"))
    if not candidates:
        _EXT_ERROR = (
            f"HIP extension not built (no _hip_ops*.so under {here}). "
            "Run `python -m llmq_amd.ops.build` (or __graft_entry__.build())."
        )
        return
    try:
        torch.ops.load_library(str(candidates[0]))
        _EXT = torch.ops.llmq_amd
        _EXT_ERROR = None
    except Exception as exc:  # noqa: BLE001
        # If an identical build was already loaded in this process (e.g.
        # right after `build()`), the namespace exists — use it.
        try:
            torch.ops.llmq_amd.rmsnorm  # noqa: B018
            _EXT = torch.ops.llmq_amd
            _EXT_ERROR = None
        except Exception:
            _EXT_ERROR = f"failed to load {candidates[0]}: {exc}"


def has_hip_ext() -> bool:
    _try_load_extension()
    return _EXT is not None


def _use_hip(t: torch.Tensor) -> bool:
    if not t.is_cuda:
        return False
    _try_load_extension()
    if _EXT is None:
        raise RuntimeError(
            f"llmq_amd HIP extension required for GPU execution but unavailable: {_EXT_ERROR}"
        )
    return True


# ---------------------------------------------------------------- norms --


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, offset: float = 0.0) -> torch.Tensor:
    if _use_hip(x):
        out = torch.empty_like(x)
        _EXT.rmsnorm(out, x, weight, eps, offset)
        return out
    return torch_ref.rmsnorm(x, weight, eps, offset)


def fused_add_rmsnorm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float, offset: float = 0.0
) -> Tuple[torch.Tensor, torch.Tensor]:
    """In place on GPU: residual += x, x = rmsnorm(residual). Returns (x, residual)."""
    if _use_hip(x):
        _EXT.fused_add_rmsnorm(x, residual, weight, eps, offset)
        return x, residual
    return torch_ref.fused_add_rmsnorm(x, residual, weight, eps, offset)


def norm_add_norm(
    x: torch.Tensor, residual: torch.Tensor, w_post: torch.Tensor,
    w_pre: torch.Tensor, eps: float, offset: float = 0.0,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gemma-2 sandwich: residual += rmsnorm(x, w_post);
    x = rmsnorm(residual, w_pre). In place on GPU; returns (x, residual)."""
    if _use_hip(x):
        _EXT.norm_add_norm(x, residual, w_post, w_pre, eps, offset)
        return x, residual
    return torch_ref.norm_add_norm(x, residual, w_post, w_pre, eps, offset)


# ----------------------------------------------------------------- rope --


def rope_inplace(
    q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor
) -> None:
    if _use_hip(q):
        _EXT.rope_inplace(q, k, positions, cos_sin)
        return
    torch_ref.rope_inplace(q, k, positions, cos_sin)


build_rope_cache = torch_ref.build_rope_cache


# ----------------------------------------------------------- activations --


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    if _use_hip(x):
        d = x.shape[-1] // 2
        out = torch.empty(*x.shape[:-1], d, dtype=x.dtype, device=x.device)
        _EXT.silu_and_mul(out, x)
        return out
    return torch_ref.silu_and_mul(x)


def gelu_tanh_and_mul(x: torch.Tensor) -> torch.Tensor:
    if _use_hip(x):
        d = x.shape[-1] // 2
        out = torch.empty(*x.shape[:-1], d, dtype=x.dtype, device=x.device)
        _EXT.gelu_tanh_and_mul(out, x)
        return out
    return torch_ref.gelu_tanh_and_mul(x)


def rope_and_cache(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
    k_cache: torch.Tensor, v_cache: torch.Tensor,
    positions: torch.Tensor, cos_sin: torch.Tensor, slot_mapping: torch.Tensor,
) -> None:
    """Fused: RoPE(q, k) in place + scatter rotated k and v into the paged
    cache (one launch instead of two per layer)."""
    if _use_hip(q):
        _EXT.rope_and_cache(q, k, v, k_cache, v_cache, positions, cos_sin, slot_mapping)
        return
    torch_ref.rope_inplace(q, k, positions, cos_sin)
    torch_ref.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)


# ------------------------------------------------------------- KV cache --


def reshape_and_cache(
    key: torch.Tensor,
    value: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    if _use_hip(key):
        _EXT.reshape_and_cache(key, value, k_cache, v_cache, slot_mapping)
        return
    torch_ref.reshape_and_cache(key, value, k_cache, v_cache, slot_mapping)


# ------------------------------------------------------------ attention --


def paged_decode_attention(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    context_lens: torch.Tensor,
    scale: float,
    softcap: float = 0.0,
    window: int = 0,
) -> torch.Tensor:
    if _use_hip(q):
        out = torch.empty_like(q)
        _EXT.paged_decode_attention(
            out, q, k_cache, v_cache, block_tables, context_lens, scale, softcap, window
        )
        return out
    return torch_ref.paged_decode_attention(
        q, k_cache, v_cache, block_tables, context_lens, scale, softcap, window
    )


def varlen_prefill_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,
    max_seqlen: int,
    scale: float,
    softcap: float = 0.0,
    window: int = 0,
    cu_seqlens_k: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Packed causal attention; cu_seqlens_k (key offsets per seq, >= query
    lengths) enables chunked prefill: Q is the last Lq positions of a
    Lk-long context."""
    cu_k = cu_seqlens if cu_seqlens_k is None else cu_seqlens_k
    if _use_hip(q):
        out = torch.empty_like(q)
        _EXT.varlen_prefill_attention(
            out, q, k, v, cu_seqlens, cu_k, int(max_seqlen), scale, softcap, window
        )
        return out
    return torch_ref.varlen_prefill_attention(
        q, k, v, cu_seqlens, scale, softcap, window, cu_seqlens_k=cu_k
    )


# ---------------------------------------------------------- skinny GEMM --


def skinny_gemm(
    x: torch.Tensor,          # [M, K] bf16
    w: torch.Tensor,          # [N, K] bf16 (torch linear weight layout)
    bias: Optional[torch.Tensor] = None,
    splitk: int = 0,          # 0 = auto
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Hand-written skinny-M decode-projection GEMM (out = x @ w.T + bias).

    256x256x64 MFMA tile, glds-staged with source-side st_16x32 swizzle,
    counted-vmcnt pipeline; split-K slabs + fused reduce for narrow-N
    shapes. Falls back to F.linear off-GPU / unsupported shapes."""
    M, K = x.shape
    N = w.shape[0]
    if not (x.is_cuda and x.dtype == torch.bfloat16 and K % 64 == 0
            and N % 4 == 0 and has_hip_ext()):
        import torch.nn.functional as F

        return F.linear(x, w, bias)
    if out is None:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    _EXT.skinny_gemm(out, x, w, bias, splitk)
    return out


# ------------------------------------------------------------- sampling --


def sample_gumbel_argmax(
    out: torch.Tensor,        # [B] int64
    keys: torch.Tensor,       # [B] int64 scratch (packed value|~index)
    logits: torch.Tensor,     # [B, V] fp32
    temps: torch.Tensor,      # [B] fp32 (<= 0 → greedy row)
    req_seeds: torch.Tensor,  # [B] int32 (0 = unseeded)
    req_pos: torch.Tensor,    # [B] int32 output position (seeded rows)
    seed: int,
    step: int,
    bounds: Optional[torch.Tensor] = None,  # [B] fp32 top-k/p keep-bound
) -> None:
    """Fused one-pass sampler: per-row Gumbel-max (== softmax sampling) or
    argmax for greedy rows, optionally truncated to {logit >= bounds[b]}
    (top-k/top-p, from topk_topp_bound). Unseeded rows draw from the
    counter-based (engine seed, step, row) stream; rows with a request seed
    draw from (request_seed, output_position) — reproducible for a given
    request regardless of batch placement."""
    assert _use_hip(logits)
    keys.zero_()
    _EXT.sample_gumbel_argmax(out, keys, logits, temps, req_seeds, req_pos,
                              seed, step, bounds)


def topk_topp_bound(
    logits: torch.Tensor,   # [B, V] fp32
    temps: torch.Tensor,    # [B] fp32
    top_ps: torch.Tensor,   # [B] fp32
    top_ks: torch.Tensor,   # [B] int64 (0 = off)
) -> torch.Tensor:
    """Per-row logit-space keep-bound realising top-p ∧ top-k truncation
    via histogram select (3 streaming passes; no full-vocab sort)."""
    assert _use_hip(logits)
    out = torch.empty(logits.size(0), dtype=torch.float32, device=logits.device)
    _EXT.topk_topp_bound(out, logits, temps, top_ps, top_ks)
    return out


def sample_tokens(
    logits: torch.Tensor,
    temperatures: torch.Tensor,
    top_ps: torch.Tensor,
    top_ks: torch.Tensor,
    generator: Optional[torch.Generator] = None,
) -> torch.Tensor:
    # Generic path (top-k/top-p capable). The serving hot loop uses the
    # fused sample_gumbel_argmax above when no top-k/top-p is requested.
    if logits.is_cuda:
        return _sample_tokens_gpu(logits, temperatures, top_ps, top_ks, generator)
    return torch_ref.sample_tokens(logits, temperatures, top_ps, top_ks, generator)


def _sample_tokens_gpu(
    logits: torch.Tensor,
    temperatures: torch.Tensor,
    top_ps: torch.Tensor,
    top_ks: torch.Tensor,
    generator: Optional[torch.Generator],
) -> torch.Tensor:
    """Batched GPU sampling without per-sequence python loops."""
    B, V = logits.shape
    greedy = temperatures <= 0
    temps = torch.where(greedy, torch.ones_like(temperatures), temperatures)
    scaled = logits.float() / temps.unsqueeze(1)
    need_topk = bool((top_ks > 0).any()) and bool((top_ks < V).any())
    need_topp = bool((top_ps < 1.0).any())
    if need_topk or need_topp:
        # histogram-select keep-bound (3 streaming passes) instead of the
        # full-vocab sort — at B=256 × V=256k the sort was a multi-ms cliff
        bound = topk_topp_bound(logits.float(), temperatures.float(),
                                top_ps.float(), top_ks)
        scaled = torch.where(logits.float() >= bound.unsqueeze(1), scaled,
                             torch.full_like(scaled, float("-inf")))
    # Gumbel-max trick: single fused sample, no multinomial sync.
    u = torch.rand(B, V, device=logits.device, generator=generator)
    gumbel = -torch.log(-torch.log(u.clamp_min(1e-20)).clamp_min(1e-20))
    sampled = (scaled + gumbel).argmax(dim=-1)
    greedy_choice = logits.argmax(dim=-1)
    return torch.where(greedy, greedy_choice, sampled)


# ------------------------------------------------------ hybrid decoders --
# Ops of the hybrid-decoder families (fp32 residual stream, block-local
# biased attention, gated-linear-attention recurrences). They live in a
# library of their own (_hip_hybrid*.so), loaded on first use; the same
# policy applies: on a GPU the HIP kernels run or the op raises.

_HY = None
_HY_ERROR: Optional[str] = None
_HY_TRIED = False


def _try_load_hybrid() -> None:
    global _HY, _HY_ERROR, _HY_TRIED
    if _HY_TRIED:
        return
    _HY_TRIED = True
    try:  # built (and thereby loaded) earlier in this process
        torch.ops.llmq_amd_hybrid.rmsnorm_cast  # noqa: B018
        _HY = torch.ops.llmq_amd_hybrid
        return
    except (AttributeError, RuntimeError):
        pass
    here = Path(__file__).parent
    override = os.environ.get("LLMQ_HYBRID_OPS_SO")
    candidates = [Path(override)] if override else sorted(here.glob("_hip_hybrid*.so"))
    if not candidates:
        _HY_ERROR = (
            f"hybrid HIP extension not built (no _hip_hybrid*.so under {here}). "
            "Run `python -m llmq_amd.ops.build --group hybrid`."
        )
        return
    try:
        torch.ops.load_library(str(candidates[0]))
        _HY = torch.ops.llmq_amd_hybrid
    except Exception as exc:  # noqa: BLE001
        try:
            torch.ops.llmq_amd_hybrid.rmsnorm_cast  # noqa: B018
            _HY = torch.ops.llmq_amd_hybrid
        except Exception:
            _HY_ERROR = f"failed to load {candidates[0]}: {exc}"


def has_hybrid_ext() -> bool:
    _try_load_hybrid()
    return _HY is not None


def _use_hybrid(t: torch.Tensor) -> bool:
    if not t.is_cuda:
        return False
    _try_load_hybrid()
    if _HY is None:
        raise RuntimeError(
            f"llmq_amd hybrid HIP extension required for GPU execution but unavailable: {_HY_ERROR}"
        )
    return True


def rmsnorm_cast(x: torch.Tensor, weight: torch.Tensor, eps: float, offset: float,
                 out_dtype: torch.dtype, groups: int = 1) -> torch.Tensor:
    """RMSNorm of x (fp32 stream or model dtype) written in out_dtype.
    groups > 1: every row is normed in that many equal consecutive parts,
    each by its own root mean square."""
    if _use_hybrid(x):
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _HY.rmsnorm_cast(out, x, weight, eps, offset, int(groups))
        return out
    return torch_ref.rmsnorm_cast(x, weight, eps, offset, out_dtype, groups)


def sandwich_norm_res32(x: torch.Tensor, residual: torch.Tensor, w_post: torch.Tensor,
                        w_pre: torch.Tensor, eps: float, offset: float,
                        groups: int = 1) -> torch.Tensor:
    """residual (fp32, in place) += rmsnorm(x)·(w_post+offset); returns
    rmsnorm(residual)·(w_pre+offset) in x's dtype (x's storage on GPU).
    groups > 1: both norms work on that many equal parts of a row."""
    if _use_hybrid(x):
        _HY.sandwich_norm_res32(x, residual, w_post, w_pre, eps, offset, int(groups))
        return x
    return torch_ref.sandwich_norm_res32(x, residual, w_post, w_pre, eps, offset, groups)


def act_and_mul(x: torch.Tensor, gelu: bool = False) -> torch.Tensor:
    """[*, 2d] → act(x[..., :d]) · x[..., d:], act = SiLU or tanh-GELU."""
    if _use_hybrid(x):
        d = x.shape[-1] // 2
        out = torch.empty(*x.shape[:-1], d, dtype=x.dtype, device=x.device)
        _HY.act_and_mul(out, x, gelu)
        return out
    return torch_ref.act_and_mul(x, gelu)


def qknorm_vmix_cache(q, k, v, q_w, k_w, v_first, lam: float, k_cache, v_cache,
                      slot_mapping, eps: float) -> None:
    """Whole-projection RMSNorm of q (in place) and k, value blending with an
    earlier layer's values, and the paged-cache scatter of k and v — fused."""
    if _use_hybrid(q):
        _HY.qknorm_vmix_cache(q, k, v, q_w, k_w, v_first, float(lam), k_cache, v_cache,
                              slot_mapping, eps)
        return
    torch_ref.qknorm_vmix_cache(q, k, v, q_w, k_w, v_first, lam, k_cache, v_cache,
                                slot_mapping, eps)


# mask modes of the paged attention kernels: keys of the query's own span of
# positions (counted from 0), or the `span` newest positions up to the query
_MASK_BLOCK, _MASK_WINDOW = 0, 1
_NO_WINDOW = (1 << 31) - 1
# bias modes: a table [H, n] indexed by the distance i - j, or per head the
# pair (r1, r2) of a logarithmic distance penalty -r1 * ln(1 + r2 * (i - j))
_BIAS_TABLE, _BIAS_LOG = 0, 1


def chunk_bias_attn_prefill(q, gate, k_cache, v_cache, bias, block_tables, cu_q, q_start,
                            max_q: int, span: int, scale: float) -> torch.Tensor:
    """Block-local causal attention + per-distance bias for packed prompt
    portions; keys/values come from the paged cache. q [T, H, D] → [T, H, DV]."""
    if _use_hybrid(q):
        out = torch.empty(q.shape[0], q.shape[1], v_cache.shape[3], dtype=q.dtype, device=q.device)
        _HY.paged_attn_prefill(out, q, gate, k_cache, v_cache, bias, block_tables, cu_q,
                               q_start, int(max_q), int(span), float(scale), _MASK_BLOCK, 1,
                               _BIAS_TABLE, 0, None, 0.0)
        return out
    return torch_ref.chunk_bias_attn_prefill(q, gate, k_cache, v_cache, bias, block_tables,
                                             cu_q, q_start, span, scale)


def chunk_bias_attn_decode(q, gate, k_cache, v_cache, bias, block_tables, context_lens,
                           span: int, scale: float) -> torch.Tensor:
    """The single-token form: query b sits at position context_lens[b]-1."""
    if _use_hybrid(q):
        out = torch.empty(q.shape[0], q.shape[1], v_cache.shape[3], dtype=q.dtype, device=q.device)
        _HY.paged_attn_decode(out, q, gate, k_cache, v_cache, bias, block_tables,
                              context_lens, int(span), float(scale), _MASK_BLOCK, _BIAS_TABLE,
                              0, None, 0.0)
        return out
    return torch_ref.chunk_bias_attn_decode(q, gate, k_cache, v_cache, bias, block_tables,
                                            context_lens, span, scale)


def gla_recurrence(q, k, v, z, z_bias, state, cu, slots, fresh, tau: float) -> torch.Tensor:
    """Gated-linear-attention recurrence over packed sequences; returns o
    [T, H, DV] fp32 and advances state [slots, H, D, DV] in place."""
    return gated_recurrence(q, k, v, z, z_bias, state, cu, slots, fresh, tau=tau,
                            q_scale=1.0 / (q.shape[2] ** 0.5))


def gated_recurrence(q, k, v, z, z_bias, state, cu, slots, fresh, tau: float = 1.0,
                     lower=None, q_silu: bool = False, q_scale: float = 1.0) -> torch.Tensor:
    """Diagonal-decay recurrence S <- diag(a) S + w v^T, o = S^T (q_scale * act(q))
    over packed sequences, state [slots, H, D, DV] fp32 advanced in place.
    lower None (gated linear attention): a = sigmoid(z + b)^(1/tau), w = k.
    lower [H*D] fp32 (HGRN2): a = l + (1 - l) * sigmoid(z + b), w = 1 - a and
    k is not read. q_silu applies SiLU to q first. Returns o [T, H, DV] fp32."""
    if _use_hybrid(q):
        o = torch.empty(q.shape[0], q.shape[1], v.shape[2], dtype=torch.float32, device=q.device)
        _HY.gla_recurrence(o, q, k, v, z, z_bias, state, cu, slots, fresh, float(tau),
                           lower, bool(q_silu), float(q_scale))
        return o
    return torch_ref.gated_recurrence(q, k, v, z, z_bias, state, cu, slots, fresh, tau, lower,
                                      q_silu, q_scale)


def gla_out_norm_gate(o, weight, gate, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """Per-head RMSNorm of the recurrence output × weight × SiLU(gate)."""
    if _use_hybrid(o):
        T, H, DV = o.shape
        out = torch.empty(T, H * DV, dtype=out_dtype, device=o.device)
        _HY.gla_out_norm_gate(out, o, weight, gate, eps)
        return out
    return torch_ref.gla_out_norm_gate(o, weight, gate, eps, out_dtype)


def head_norm(o, weight, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """Per-head RMSNorm of a recurrence output o [T, H, DV] fp32 x weight [DV]."""
    if _use_hybrid(o):
        T, H, DV = o.shape
        out = torch.empty(T, H * DV, dtype=out_dtype, device=o.device)
        _HY.gla_out_norm_gate(out, o, weight, None, eps)
        return out
    return torch_ref.head_norm(o, weight, eps, out_dtype)


def window_attn_prefill(q, k_cache, v_cache, dv: int, block_tables, cu_q, q_start, max_q: int,
                        window: int, scale: float, log_bias=None, keep_first: int = 0,
                        sink=None, softcap: float = 0.0) -> torch.Tensor:
    """Softmax attention of packed prompt portions over the paged cache:
    query at position i sees keys j <= i with i - j < window (window 0:
    every j <= i) or j < keep_first. v_cache None: the first dv channels of a
    key row are its value (latent caches). log_bias fp32 [H, 2] = (r1, r2)
    per head: the score loses r1 * ln(1 + r2 * (i - j)). softcap c > 0: the
    scaled score becomes c * tanh(score / c). sink fp32 [H]: the softmax
    denominator gains exp(sink[h]). q [T, H, D] -> [T, H, dv]."""
    if _use_hybrid(q):
        out = torch.empty(q.shape[0], q.shape[1], dv, dtype=q.dtype, device=q.device)
        _HY.paged_attn_prefill(out, q, None, k_cache, v_cache, log_bias, block_tables, cu_q,
                               q_start, int(max_q), int(window) or _NO_WINDOW, float(scale),
                               _MASK_WINDOW, 1, _BIAS_LOG if log_bias is not None else _BIAS_TABLE,
                               int(keep_first) if window else 0, sink, float(softcap))
        return out
    return torch_ref.window_attn_prefill(q, k_cache, v_cache, dv, block_tables, cu_q, q_start,
                                         window, scale, log_bias, keep_first, sink, softcap)


def window_attn_decode(q, k_cache, v_cache, dv: int, block_tables, context_lens, window: int,
                       scale: float, log_bias=None, keep_first: int = 0, sink=None,
                       softcap: float = 0.0) -> torch.Tensor:
    """The single-token form: query b sits at position context_lens[b]-1."""
    if _use_hybrid(q):
        B, H, D = q.shape
        out = torch.empty(B, H, dv, dtype=q.dtype, device=q.device)
        bias_mode = _BIAS_LOG if log_bias is not None else _BIAS_TABLE
        keep = int(keep_first) if window else 0
        if (q.dtype == torch.bfloat16 and k_cache.shape[1] == 1 and H >= 8 and D % 8 == 0
                and D <= 256 and q.is_contiguous() and log_bias is None and not keep
                and sink is None and not softcap):
            # one kv head for all query heads: the heads of a token become the
            # rows of one head, all at the token's position, and the step runs
            # on the matrix-core kernel — every key tile staged once for all
            # heads instead of once per head group
            cu = _head_row_offsets(B, H, q.device)
            _HY.paged_attn_prefill(out.view(B * H, 1, dv), q.view(B * H, 1, D), None, k_cache,
                                   v_cache, None, block_tables, cu, context_lens - 1, H,
                                   int(window) or _NO_WINDOW, float(scale), _MASK_WINDOW, 0,
                                   _BIAS_TABLE, 0, None, 0.0)
            return out
        _HY.paged_attn_decode(out, q, None, k_cache, v_cache, log_bias, block_tables,
                              context_lens, int(window) or _NO_WINDOW, float(scale), _MASK_WINDOW,
                              bias_mode, keep, sink, float(softcap))
        return out
    return torch_ref.window_attn_decode(q, k_cache, v_cache, dv, block_tables, context_lens,
                                        window, scale, log_bias, keep_first, sink, softcap)


_HEAD_ROWS = {}


def _head_row_offsets(B: int, H: int, device) -> torch.Tensor:
    """[0, H, 2H, ..., B*H] int32 on the device, made once per (B, H)."""
    key = (B, H, str(device))
    t = _HEAD_ROWS.get(key)
    if t is None:
        t = torch.arange(B + 1, dtype=torch.int32, device=device) * H
        _HEAD_ROWS[key] = t
    return t


def latent_rope_pack(q, q_lat, ckr, c_w, inv_freq, positions, k_cache, slots, dim: int,
                     rot_dims: int, interleaved: bool, eps: float) -> torch.Tensor:
    """Latent attention, between the projections and the attention kernel:
    rotary positions (fp32 angles position * inv_freq[i]) on the rotated part
    of q [T, H, dim+DR] and of ckr [T, R+DR], RMSNorm of the latent, the
    packed query q_lat ‖ rotated part [T, H, R+DR] returned, and latent ‖
    rotated key part scattered into the paged cache [blocks, 1, bs, R+DR]."""
    if _use_hybrid(q):
        T, H, _ = q.shape
        out = torch.empty(T, H, ckr.shape[1], dtype=q.dtype, device=q.device)
        _HY.latent_rope_pack(out, q, q_lat, ckr, c_w, inv_freq, positions, k_cache, slots,
                             int(dim), int(rot_dims), bool(interleaved), float(eps))
        return out
    return torch_ref.latent_rope_pack(q, q_lat, ckr, c_w, inv_freq, positions, k_cache, slots,
                                      dim, rot_dims, interleaved, eps)


def gated_residual_add(res, y1, g1, b1, y2, g2, b2, out_dtype: torch.dtype) -> torch.Tensor:
    """res (fp32, in place) += sigmoid(g1 + b1) * y1 [+ sigmoid(g2 + b2) * y2];
    returns the updated rows rounded to out_dtype. g1/g2 may be column
    slices of a wider projection output."""
    if _use_hybrid(res):
        out = torch.empty(res.shape, dtype=out_dtype, device=res.device)
        _HY.gated_residual_add(out, res, y1, g1, b1, y2, g2, b2)
        return out
    return torch_ref.gated_residual_add(res, y1, g1, b1, y2, g2, b2, out_dtype)


def side_gate_mul(a, table, tokens, offset: int) -> torch.Tensor:
    """gelu_tanh(a) * table[tokens, offset : offset + a.shape[1]]."""
    if _use_hybrid(a):
        out = torch.empty_like(a)
        _HY.side_gate_mul(out, a, table, tokens, int(offset))
        return out
    return torch_ref.side_gate_mul(a, table, tokens, offset)


def sigmoid_topk(logits, top: int):
    """Router scores sigmoid(logits) in fp32 and their `top` largest per
    row: (indices int32 [T, top], scores fp32 [T, top])."""
    if _use_hybrid(logits):
        T = logits.shape[0]
        idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
        w = torch.empty(T, top, dtype=torch.float32, device=logits.device)
        _HY.sigmoid_topk(idx, w, logits, int(top))
        return idx, w
    return torch_ref.sigmoid_topk(logits, top)


# rows (token, expert) pairs up to which the expert mixture runs as
# per-row matrix-vector kernels (no host sync, graph-capturable)
MOE_GEMV_MAX_ROWS = 64
# within the matrix-vector form: from this many rows on (and up to the LDS
# row list's size) rows are grouped by expert inside the kernel
MOE_GROUP_MIN_ROWS = 16
MOE_GROUP_MAX_ROWS = 2048
# from MOE_GROUP_MIN_ROWS rows on, while experts x tokens stays below this: the
# dense form, every expert on every token as one batched GEMM pair (all
# experts' weights are streamed anyway once the rows outnumber the experts)
MOE_DENSE_MAX_PAIRS = 16384


def moe_experts(h, idx, w, gate_up, down, sync_free: bool = False, act: str = "silu",
                limit: float = 0.0, weight_output: bool = False, identity: int = 0) -> torch.Tensor:
    """Sum over a token's chosen experts of down_e(act(gate_e x, up_e x)).
    weight_output False: x = w * h (the router weight scales the expert's
    INPUT); True: x = h and the weight scales the expert's OUTPUT.
    act "silu": silu(g) * u; "clamp_swish": g * sigmoid(1.702 g) * (u + 1)
    with g = min(g, limit), u = clamp(u, +-limit); "gelu_erf" / "relu2":
    ungated experts down_e(act(up_e x)), gate_up then holds [E, F, W].
    identity > 0 (with weight_output): indices E .. E + identity - 1 name
    experts that return their input.
    h [T, W]; idx/w [T, top]; gate_up [E, 2F, W]; down [E, W, F].

    Few rows: one matrix-vector kernel pair that reads only each row's
    expert weights. Decode batches (sync_free, for captured graphs) with
    more rows than that: every expert runs on every token as one batched
    GEMM pair on the matrix cores, and a token's unchosen experts weigh
    nothing in the join. Many rows (prompt portions): rows sorted by expert
    and one GEMM pair per expert on contiguous slices (the per-expert row
    counts cross to the host once)."""
    T, top = idx.shape
    gated = act in _MOE_ACTS
    if identity and not weight_output:
        raise ValueError("identity experts need the weight on the output side")
    E = gate_up.shape[0]

    def middle(gu):
        if not gated:
            return unary_act(gu, act)
        return act_and_mul(gu) if act == "silu" else clamp_swish_mul(gu, limit)

    if h.is_cuda and (sync_free or T * top <= MOE_GEMV_MAX_ROWS):
        _use_hybrid(h)
        F_ = down.shape[2]
        plain = gated and not identity
        if T * top >= MOE_GROUP_MIN_ROWS and (E * T <= MOE_DENSE_MAX_PAIRS or
                                              (sync_free and not plain)):
            wd = torch.zeros(T, E + identity, dtype=torch.float32, device=h.device)
            wd.scatter_(1, idx.long(), w)
            if weight_output:
                xs = h.unsqueeze(0).expand(E, T, h.shape[1])
            else:  # zero input for the experts a token did not choose
                xs = (h.float().unsqueeze(0) * wd.t().unsqueeze(-1)).to(h.dtype)
            gu = torch.bmm(xs, gate_up.transpose(1, 2)).view(E * T, -1)
            yk = torch.bmm(middle(gu).view(E, T, F_), down.transpose(1, 2))
            y = torch.empty_like(h)
            if identity:
                # an identity expert's output is the token itself: one more
                # "expert result" whose weight is the sum of those chosen
                yk = torch.cat([yk, h.unsqueeze(0)], dim=0)
                wd = torch.cat([wd[:, :E], wd[:, E:].sum(dim=1, keepdim=True)], dim=1)
            _HY.moe_combine(y, yk, wd if weight_output else None)
            return y
        if not plain:
            # few rows of ungated experts: the matrix-vector kernels read only
            # the chosen experts; an identity expert's row runs on a stand-in
            # expert with weight 0 and the token itself joins afterwards
            hmid = torch.empty(T * top, F_, dtype=h.dtype, device=h.device)
            real = idx < E
            w_real = torch.where(real, w, torch.zeros_like(w))
            _HY.moe_gate_up_gemv(hmid, h, idx, None if weight_output else w, gate_up,
                                 _MOE_PLAIN_ACTS[act], 0.0)
            y = torch.empty_like(h)
            _HY.moe_down_gemv(y, hmid, idx, down, w_real if weight_output else None)
            if identity:
                w_id = (w - w_real).sum(dim=1, keepdim=True)
                y = torch.addcmul(y.float(), h.float(), w_id).to(h.dtype)
            return y
        if plain:
            act_mode = _MOE_ACTS[act]
            hmid = torch.empty(T * top, F_, dtype=h.dtype, device=h.device)
            w_in = None if weight_output else w
            if MOE_GROUP_MIN_ROWS <= T * top <= MOE_GROUP_MAX_ROWS and \
                    max(h.shape[1], F_) * h.element_size() * 8 <= (128 << 10):
                # enough rows that experts repeat: grouped by expert inside the
                # kernel, a weight row is read once per 8 rows of its expert
                _HY.moe_expert_gemv(hmid, h, idx, w_in, gate_up, True, act_mode, float(limit))
                yk = torch.empty(T * top, h.shape[1], dtype=h.dtype, device=h.device)
                _HY.moe_expert_gemv(yk, hmid, idx, None, down, False, 0, 0.0)
                yk = yk.view(T, top, -1).float()
                if weight_output:
                    yk = yk * w.unsqueeze(-1)
                return yk.sum(dim=1).to(h.dtype)
            _HY.moe_gate_up_gemv(hmid, h, idx, w_in, gate_up, act_mode, float(limit))
            y = torch.empty_like(h)
            _HY.moe_down_gemv(y, hmid, idx, down, w if weight_output else None)
            return y
    flat = idx.reshape(-1).long()
    order = torch.sort(flat, stable=True).indices
    counts = torch.bincount(flat, minlength=E + identity).tolist()
    if weight_output:
        xs = h[order // top]
    else:
        xs = (h.float()[order // top] * w.reshape(-1)[order].unsqueeze(1)).to(h.dtype)
    ys = torch.empty_like(xs)
    at = 0
    for e, n in enumerate(counts):
        if n and e < E:
            gu = torch.nn.functional.linear(xs[at:at + n], gate_up[e])
            ys[at:at + n] = torch.nn.functional.linear(middle(gu), down[e])
        elif n:
            ys[at:at + n] = xs[at:at + n]
        at += n
    inv = torch.empty_like(order)
    inv[order] = torch.arange(order.numel(), device=order.device)
    if h.is_cuda:
        _use_hybrid(h)
        y = torch.empty_like(h)
        _HY.moe_gather_combine(y, ys, inv, w.contiguous() if weight_output else None, top)
        return y
    yk = ys[inv].view(T, top, -1).float()
    if weight_output:
        yk = yk * w.unsqueeze(-1)
    return yk.sum(dim=1).to(h.dtype)


_MOE_ACTS = {"silu": 0, "clamp_swish": 1}
_MOE_PLAIN_ACTS = {"gelu_erf": 2, "relu2": 3}


# ---- scan hybrids: elementwise gated recurrences, selective scans beside
# attention, softmax-routed clamped experts, a learned average over layers --


def embed_sinusoid(embedding, ids, positions, inv_freq) -> torch.Tensor:
    """fp32 [T, W]: embedding[ids] plus the sinusoidal position vector (entry
    2i = sin(p * inv_freq[i]), entry 2i+1 = cos of it, angles in fp32)."""
    if _use_hybrid(embedding):
        out = torch.empty(ids.shape[0], embedding.shape[1], dtype=torch.float32,
                          device=embedding.device)
        _HY.embed_sinusoid(out, embedding, ids, positions, inv_freq)
        return out
    return torch_ref.embed_sinusoid(embedding, ids, positions, inv_freq)


def scaled_add_norm(res, y, y2, a1: float, a2: float, weight, eps: float,
                    out_dtype: torch.dtype) -> torch.Tensor:
    """res (fp32, in place) += a1 * y [+ a2 * y2]; returns rmsnorm(res) * weight
    in out_dtype."""
    if _use_hybrid(res):
        out = torch.empty(res.shape, dtype=out_dtype, device=res.device)
        _HY.scaled_add_norm(out, res, y, y2, float(a1), float(a2), weight, float(eps))
        return out
    return torch_ref.scaled_add_norm(res, y, y2, a1, a2, weight, eps, out_dtype)


def depth_mix_norm(stack, n: int, coef, y, y2, a1: float, a2: float, weight, eps: float,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """The close of a layer under a learned average over layer outputs.
    stack [>= n+1, T, W] fp32: rows 0..n-1 hold the embedding output and the
    layer results so far. Row n-1 (in place) += a1 * y [+ a2 * y2]; row n =
    sum_j coef[j] * row j; returns rmsnorm(row n) * weight in out_dtype."""
    if _use_hybrid(stack):
        out = torch.empty(stack.shape[1:], dtype=out_dtype, device=stack.device)
        _HY.depth_mix_norm(out, stack, int(n), coef, y, y2, float(a1), float(a2), weight,
                           float(eps))
        return out
    return torch_ref.depth_mix_norm(stack, n, coef, y, y2, a1, a2, weight, eps, out_dtype)


def kv_scatter(k, v, k_cache, v_cache, slots) -> None:
    """Rows of k [T, G*D] and v [T, G*DV] (column slices of a projection)
    into the paged cache rows `slots`; a negative slot writes nothing."""
    if _use_hybrid(k):
        _HY.kv_scatter(k, v, k_cache, v_cache, slots)
        return
    torch_ref.kv_scatter(k, v, k_cache, v_cache, slots)


def mingru_scan(z, u, g, z_b, u_b, state, cu, slots, fresh, out_dtype: torch.dtype):
    """minGRU over packed sequences: S <- (1 - a) S + a c per channel with
    a = sigmoid(z + z_b), c = u' + 1/2 (u' >= 0) else sigmoid(u'), u' = u +
    u_b; state [slots, n] fp32 advanced in place; returns S_t * silu(g_t)."""
    if _use_hybrid(z):
        out = torch.empty(z.shape, dtype=out_dtype, device=z.device)
        _HY.mingru_scan(out, z, u, g, z_b, u_b, state, cu, slots, fresh)
        return out
    return torch_ref.mingru_scan(z, u, g, z_b, u_b, state, cu, slots, fresh, out_dtype)


def causal_conv_silu(x, weight, bias, tail, cu, slots, fresh, silu: bool = True) -> torch.Tensor:
    """Per-channel causal convolution (+ bias unless None, + SiLU unless silu
    is False) over packed sequences; tail [slots, K-1, C] fp32 carries each
    sequence's last K-1 inputs."""
    if _use_hybrid(x):
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _HY.causal_conv_silu(out, x, weight, bias, tail, cu, slots, fresh, bool(silu))
        return out
    return torch_ref.causal_conv_silu(x, weight, bias, tail, cu, slots, fresh, silu)


def selective_scan(x, dt, dt_b, A, Bm, Cm, D, z, state, cu, slots, fresh) -> torch.Tensor:
    """Selective scan over packed sequences (see torch_ref.selective_scan);
    state [slots, C, N] fp32 advanced in place; returns y * silu(z)."""
    if _use_hybrid(x):
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _HY.selective_scan(out, x, dt, dt_b, A, Bm, Cm, D, z, state, cu, slots, fresh)
        return out
    return torch_ref.selective_scan(x, dt, dt_b, A, Bm, Cm, D, z, state, cu, slots, fresh)


def softmax_topk(logits, top: int, scale: float = 1.0, correction=None, renorm: bool = False):
    """Router: softmax over all experts in fp32, the `top` largest per row,
    times scale: (indices int32 [T, top], weights fp32 [T, top]). correction
    fp32 [E]: the choice is made on score + correction, the weights stay the
    plain scores. renorm: the chosen scores are divided by their sum first."""
    if _use_hybrid(logits):
        T = logits.shape[0]
        idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
        w = torch.empty(T, top, dtype=torch.float32, device=logits.device)
        _HY.softmax_topk(idx, w, logits, int(top), float(scale), correction, bool(renorm))
        return idx, w
    return torch_ref.softmax_topk(logits, top, scale, correction, renorm)


def clamp_swish_mul(x, limit: float) -> torch.Tensor:
    """[*, 2d] -> g * sigmoid(1.702 g) * (u + 1), g = min(x[..., :d], limit),
    u = clamp(x[..., d:], -limit, limit)."""
    if _use_hybrid(x):
        d = x.shape[-1] // 2
        out = torch.empty(*x.shape[:-1], d, dtype=x.dtype, device=x.device)
        _HY.clamp_swish_mul(out, x, float(limit))
        return out
    return torch_ref.clamp_swish_mul(x, limit)


# ---- windowed attention beside a matrix memory: norms on groups of the
# width, kept first tokens and a learned softmax term, rotated values, mLSTM --


def qkv_norm_rope_cache(q, k, v, q_w, k_w, inv_freq, rot_dims: int, positions, k_cache, v_cache,
                        slots, eps: float, v_unit_norm: bool = False, v_inv_freq=None) -> None:
    """Per token, between the projections and the attention kernel: optional
    per-head RMSNorm of q and k (weights q_w / k_w [D]), rotary positions on
    their first rot_dims channels (q [T, H, D] in place), and the paged-cache
    scatter of k and of the values — v [T, G, DV], or the keys as they arrive
    when v is None — which may be divided by their root mean square per head
    (v_unit_norm) and turned by their position over all channels
    (v_inv_freq fp32 [DV/2])."""
    if _use_hybrid(q):
        _HY.qkv_norm_rope_cache(q, k, v, q_w, k_w, inv_freq, int(rot_dims), positions, k_cache,
                                v_cache, slots, float(eps), bool(v_unit_norm), v_inv_freq)
        return
    torch_ref.qkv_norm_rope_cache(q, k, v, q_w, k_w, inv_freq, rot_dims, positions, k_cache,
                                  v_cache, slots, eps, v_unit_norm, v_inv_freq)


def rotate_heads(x, positions, inv_freq, inverse: bool = False) -> torch.Tensor:
    """x [T, H, n] in place: every head turned by its token's position (by
    minus the position if inverse) over all n channels, pairs (i, i + n/2),
    angles position * inv_freq[i] in fp32."""
    if _use_hybrid(x):
        _HY.rotate_heads(x, positions, inv_freq, bool(inverse))
        return x
    return torch_ref.rotate_heads(x, positions, inv_freq, inverse)


def mlstm_gates(gates, cap: float, m_state, cu, slots, fresh):
    """The gate recurrence of an mLSTM over packed sequences. gates fp32
    [T, 2H] = input | forget pre-activations; returns fp32 [T, H] decay,
    write and floor (see torch_ref.mlstm_gates); m_state [slots, H] fp32
    (the running maximum) advanced in place."""
    if _use_hybrid(gates):
        T, H = gates.shape[0], gates.shape[1] // 2
        out = torch.empty(3, T, H, dtype=torch.float32, device=gates.device)
        _HY.mlstm_gates(out, gates, float(cap), m_state, cu, slots, fresh)
        return out[0], out[1], out[2]
    return torch_ref.mlstm_gates(gates, cap, m_state, cu, slots, fresh)


def matrix_memory(q, k, v, decay, write, state, cu, slots, fresh, q_scale: float) -> torch.Tensor:
    """mLSTM memory update and read-out with per-head scalar gates:
    S <- decay S + write k [v | 1]^T, o = S^T (q_scale q). The state's last
    value column is the normaliser vector, so o's last column is n . q.
    state [slots, H, D, DV + 1] fp32 advanced in place; o [T, H, DV + 1] fp32."""
    if _use_hybrid(q):
        T, H, _ = q.shape
        o = torch.empty(T, H, v.shape[2] + 1, dtype=torch.float32, device=q.device)
        _HY.matrix_memory(o, q, k, v, decay, write, state, cu, slots, fresh, float(q_scale))
        return o
    return torch_ref.matrix_memory(q, k, v, decay, write, state, cu, slots, fresh, q_scale)


def mlstm_out_norm_gate(o, floor, weight, gate, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """Read-out of an mLSTM: o[..., :DV] / (max(|o[..., DV]|, floor) + 1e-6),
    per-head RMS norm, times weight [H*DV], times sigmoid(gate)."""
    if _use_hybrid(o):
        T, H, DV1 = o.shape
        out = torch.empty(T, H * (DV1 - 1), dtype=out_dtype, device=o.device)
        _HY.mlstm_out_norm_gate(out, o, floor, weight, gate, float(eps))
        return out
    return torch_ref.mlstm_out_norm_gate(o, floor, weight, gate, eps, out_dtype)


def dual_norm_mean(a, w_a, b, w_b, eps: float) -> torch.Tensor:
    """(rmsnorm(a) * w_a + rmsnorm(b) * w_b) / 2, norms over the whole row."""
    if _use_hybrid(a):
        out = torch.empty_like(a)
        _HY.dual_norm_mean(out, a, w_a, b, w_b, float(eps))
        return out
    return torch_ref.dual_norm_mean(a, w_a, b, w_b, eps)


_UNARY_ACTS = {"relu2": 0, "gelu_erf": 1}


def unary_act(x, kind: str) -> torch.Tensor:
    """Elementwise activation of an ungated feed-forward: "relu2" =
    max(x, 0)^2, "gelu_erf" = the exact GELU."""
    if _use_hybrid(x):
        out = torch.empty_like(x)
        _HY.unary_act(out, x, _UNARY_ACTS[kind])
        return out
    return torch_ref.unary_act(x, kind)

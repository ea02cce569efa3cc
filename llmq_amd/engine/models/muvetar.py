"""Muvetar: a scan/attention hybrid decoder on an fp32 residual.

The embedding gets a sinusoidal position vector. A layer is pre-norm,

    x += m * mixer(norm1(x));   x += m * ff(norm2(x))

with a fixed multiplier m on every sublayer output, and ends by replacing x
with a learned weighted sum of the embedding output and the results of all
layers so far ("depth average"): x <- sum_j c[j] * X_j.

Mixers: a minGRU (an elementwise gated recurrence whose gate and candidate
read only the current token), or two mixers side by side on the same input —
causal softmax attention with grouped kv heads and a logarithmic distance
penalty instead of a rotation, and a Mamba selective scan behind a short
causal convolution — added with fixed scales. Feed-forward: a mixture of
clamped gated experts picked by a softmax router, plus a shared expert. The
logits pass a tanh soft cap.

MI355X mapping, in the manner of the other hybrid families:

- plain-tensor weights; everything that reads the mixer's input is ONE GEMM
  per layer (minGRU: gate ‖ candidate ‖ output gate; parallel layer:
  q ‖ k ‖ v ‖ scan input ‖ scan gate), segments at 16-byte boundaries;
- the residual stream and the layer outputs the depth average reads stay
  fp32 in one [layers + 2, tokens, width] stack; closing a sublayer (scaled
  add of one or two results, norm for the next reader) is one kernel, and the
  layer's end (last add, depth average, next layer's norm) is one more;
- attention keys and values go through the paged cache and the block
  table for prompt portions and single tokens alike, on the same paged
  attention kernels as the other families with the distance penalty
  computed in the kernel from the head's two numbers;
- minGRU state, scan state and convolution tail live in per-sequence state
  slots; one kernel per recurrence serves portions and single tokens;
- a step's expert mixture runs sorted by expert on vendor GEMMs, or, for few
  rows and inside captured decode graphs, as matrix-vector kernels.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Union

import torch
import torch.nn.functional as F

from llmq_amd import ops
from llmq_amd.engine.forward_meta import DecodeMeta, MixedMeta, PrefillMeta
from llmq_amd.engine.kv_cache import KVCache
from llmq_amd.engine.model_specs import MuvetarSpec
from llmq_amd.ops import torch_ref


class MuvetarLayerWeights:
    def __init__(self) -> None:
        self.t: Dict[str, torch.Tensor] = {}     # packed / checkpoint-shaped tensors
        self.seg: Dict[str, tuple] = {}          # name -> (first row, rows) in t["in"]
        self.A: Optional[torch.Tensor] = None    # fp32 [inner, state] = -exp(A_log)


def _align8(n: int) -> int:
    return -(-n // 8) * 8


class MuvetarLM:
    #: HIP extension groups this family runs on
    ext_groups = ("hybrid",)
    #: prompt portions attend through the block table (no gathered copy)
    paged_prefill = True
    #: mixed steps run their decode and prefill segments one after the other
    #: (the expert GEMMs pick stream-k kernels at some shapes; those must not
    #: share the chip with a second stream's kernels)
    overlap_mixed = False

    def __init__(self, spec: MuvetarSpec, device: torch.device, dtype: torch.dtype,
                 tp_rank: int = 0, tp_size: int = 1):
        if tp_size != 1:
            raise NotImplementedError("the hybrid families run on one GPU per replica")
        self.spec = spec
        self.device = device
        self.dtype = dtype
        self.tp_rank, self.tp_size = tp_rank, tp_size
        self.layers: List[MuvetarLayerWeights] = []
        self.embedding: Optional[torch.Tensor] = None
        self.lm_head: Optional[torch.Tensor] = None
        self.final_norm: Optional[torch.Tensor] = None
        self.inv_freq: Optional[torch.Tensor] = None    # fp32 sinusoid table
        self.taps: Optional[List[torch.Tensor]] = None  # stream after each layer (debug)
        self._alloc()

    # -- layout the engine asks for ---------------------------------------

    def kv_layout(self):
        return [
            (ls.mixer.left.kv_heads, ls.mixer.left.dim, ls.mixer.left.vdim)
            if ls.mixer.kind == "parallel" else None
            for ls in self.spec.layers
        ]

    def state_layout(self):
        out = []
        for ls in self.spec.layers:
            m = ls.mixer
            if m.kind == "mingru":
                out.append((m.width,))
            else:
                r = m.right
                out.append([(r.inner, r.state), (r.conv - 1, r.inner)])
        return out

    # -- weights ---------------------------------------------------------

    def _empty(self, *shape, dtype=None) -> torch.Tensor:
        return torch.empty(*shape, device=self.device, dtype=dtype or self.dtype)

    def _alloc(self) -> None:
        s = self.spec
        W = s.hidden_size
        f32 = torch.float32
        self.embedding = self._empty(s.vocab_size, W)
        self.lm_head = self._empty(s.vocab_size, W)
        self.final_norm = self._empty(W)
        for i, ls in enumerate(s.layers):
            lw = MuvetarLayerWeights()
            m, t = ls.mixer, lw.t
            t["norm1"] = self._empty(W)
            t["dwa"] = self._empty(i + 2, dtype=f32)
            if m.kind == "mingru":
                segs = [("z", m.width), ("u", m.width), ("g", m.width)]
                t["z_b"] = self._empty(m.width, dtype=f32)
                t["u_b"] = self._empty(m.width, dtype=f32)
                t["o"] = self._empty(W, m.width)
            else:
                a, r = m.left, m.right
                segs = [("q", a.heads * a.dim), ("k", a.kv_heads * a.dim),
                        ("v", a.kv_heads * a.vdim), ("x", r.inner), ("gate", r.inner)]
                t["r12"] = self._empty(a.heads, 2, dtype=f32)       # (r1, r2) per head
                t["attn_o"] = self._empty(W, a.heads * a.vdim)
                t["conv_w"] = self._empty(r.inner, r.conv, dtype=f32)
                t["conv_b"] = self._empty(r.inner, dtype=f32)
                t["xproj"] = self._empty(r.dt_rank + 2 * r.state, r.inner)   # dt ‖ B ‖ C
                t["dt"] = self._empty(r.inner, r.dt_rank)
                t["dt_b"] = self._empty(r.inner, dtype=f32)
                t["A_log"] = self._empty(r.inner, r.state, dtype=f32)
                t["D"] = self._empty(r.inner, dtype=f32)
                t["scan_o"] = self._empty(W, r.inner)
            at = 0
            for name, n in segs:
                lw.seg[name] = (at, n)
                at += _align8(n)
            t["in"] = self._empty(at, W)
            t["in"].zero_()
            if ls.moe:
                e = ls.moe
                t["norm2"] = self._empty(W)
                t["router"] = self._empty(e.experts, W, dtype=f32)
                t["e_gate_up"] = self._empty(e.experts, 2 * e.ff, W)
                t["e_down"] = self._empty(e.experts, W, e.ff)
                if e.shared_ff:
                    t["s_gate_up"] = self._empty(2 * e.shared_ff, W)
                    t["s_down"] = self._empty(W, e.shared_ff)
            self.layers.append(lw)

    @torch.no_grad()
    def finalize(self) -> None:
        """Derive what the kernels read from the loaded tensors."""
        self.inv_freq = torch_ref.sinusoid_inv_freq(self.spec.hidden_size).to(self.device)
        for lw in self.layers:
            if "A_log" in lw.t:
                lw.A = -torch.exp(lw.t["A_log"])

    @torch.no_grad()
    def random_init(self, seed: int = 0, fast: bool = False) -> None:
        if fast and self.device.type == "cuda":
            gen = torch.Generator(device=self.device).manual_seed(seed)

            def fill(t: torch.Tensor, std: float, mean: float = 0.0) -> None:
                t.normal_(mean, std, generator=gen)
        else:
            gen = torch.Generator(device="cpu").manual_seed(seed)

            def fill(t: torch.Tensor, std: float, mean: float = 0.0) -> None:
                cpu = torch.randn(t.shape, generator=gen, dtype=torch.float32) * std + mean
                t.copy_(cpu.to(t.dtype))

        W = self.spec.hidden_size
        fill(self.embedding, 1.0)
        fill(self.lm_head, 1.0 / math.sqrt(W))
        fill(self.final_norm, 0.1, 1.0)
        for lw in self.layers:
            for name, t in lw.t.items():
                if name in ("norm1", "norm2"):
                    fill(t, 0.1, 1.0)
                elif name == "dwa":
                    # mostly the newest layer output, a little of the others
                    fill(t, 0.1)
                    t[-1] += 1.0
                elif name == "r12":
                    fill(t, 0.2, 0.6)
                    t.abs_()
                elif name == "A_log":
                    fill(t, 0.5)
                elif name == "D":
                    fill(t, 0.3, 1.0)
                elif name == "dt_b":
                    fill(t, 0.5, -2.0)
                elif name in ("z_b", "u_b", "conv_b"):
                    fill(t, 0.5)
                elif name == "conv_w":
                    fill(t, 0.5)
                elif name == "in":
                    fill(t, 1.0 / math.sqrt(W))
                    keep = torch.zeros(t.shape[0], dtype=torch.bool)
                    for at, n in lw.seg.values():
                        keep[at:at + n] = True
                    t[~keep.to(t.device)] = 0
                else:
                    fill(t, 1.0 / math.sqrt(t.shape[-1]))
        self.finalize()

    def named_tensors(self) -> Dict[str, torch.Tensor]:
        out = {"embedding": self.embedding, "lm_head": self.lm_head,
               "final_norm": self.final_norm}
        for i, lw in enumerate(self.layers):
            for name, t in lw.t.items():
                out[f"layers.{i}.{name}"] = t
        return out

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.named_tensors().values())

    # -- mixers ----------------------------------------------------------

    def _seg(self, p: torch.Tensor, lw: MuvetarLayerWeights, name: str) -> torch.Tensor:
        at, n = lw.seg[name]
        return p[:, at:at + n]

    def _mingru(self, p, lw, i, kv_cache, meta):
        rm = meta.recurrent
        y = ops.mingru_scan(self._seg(p, lw, "z"), self._seg(p, lw, "u"), self._seg(p, lw, "g"),
                            lw.t["z_b"], lw.t["u_b"], kv_cache.recurrent.state[i],
                            rm.cu, rm.slots, rm.fresh, self.dtype)
        return F.linear(y, lw.t["o"])

    def _attention(self, p, lw, a, i, kv_cache, meta):
        T = p.shape[0]
        q = self._seg(p, lw, "q").unflatten(1, (a.heads, a.dim))
        kc, vc = kv_cache.k[i], kv_cache.v[i]
        ops.kv_scatter(self._seg(p, lw, "k"), self._seg(p, lw, "v"), kc, vc, meta.slot_mapping)
        bias = lw.t["r12"]
        if meta.is_prefill:
            att = ops.window_attn_prefill(
                q, kc, vc, a.vdim, meta.block_tables, meta.cu_seqlens, meta.q_start,
                meta.max_seqlen, 0, a.scale, log_bias=bias)
        elif meta.is_mixed:
            nd, pm, dm = meta.n_decode, meta.prefill, meta.decode
            att_d = ops.window_attn_decode(
                q[:nd], kc, vc, a.vdim, dm.block_tables, dm.context_lens, 0, a.scale,
                log_bias=bias)
            att_p = ops.window_attn_prefill(
                q[nd:], kc, vc, a.vdim, pm.block_tables, pm.cu_seqlens, pm.q_start,
                pm.max_seqlen, 0, a.scale, log_bias=bias)
            att = torch.cat([att_d, att_p], dim=0)
        else:
            att = ops.window_attn_decode(
                q, kc, vc, a.vdim, meta.block_tables, meta.context_lens, 0, a.scale,
                log_bias=bias)
        return F.linear(att.reshape(T, a.heads * a.vdim), lw.t["attn_o"])

    def _mamba(self, p, lw, r, i, kv_cache, meta):
        rm = meta.recurrent
        state, tail = kv_cache.recurrent.state[i]
        x = ops.causal_conv_silu(self._seg(p, lw, "x"), lw.t["conv_w"], lw.t["conv_b"], tail,
                                 rm.cu, rm.slots, rm.fresh)
        dbc = F.linear(x, lw.t["xproj"])
        R, N = r.dt_rank, r.state
        dt = F.linear(dbc[:, :R], lw.t["dt"])
        y = ops.selective_scan(x, dt, lw.t["dt_b"], lw.A, dbc[:, R:R + N], dbc[:, R + N:R + 2 * N],
                               lw.t["D"], self._seg(p, lw, "gate"), state,
                               rm.cu, rm.slots, rm.fresh)
        return F.linear(y, lw.t["scan_o"])

    def _moe(self, h, lw, e, meta):
        logits = F.linear(h.float(), lw.t["router"])
        idx, w = ops.softmax_topk(logits, e.top, e.scale)
        decode_only = not (meta.is_prefill or meta.is_mixed)
        y = ops.moe_experts(h, idx, w, lw.t["e_gate_up"], lw.t["e_down"], sync_free=decode_only,
                            act="clamp_swish", limit=e.limit, weight_output=True)
        ys = None
        if e.shared_ff:
            mid = ops.clamp_swish_mul(F.linear(h, lw.t["s_gate_up"]), e.shared_limit)
            ys = F.linear(mid, lw.t["s_down"])
        return y, ys

    # -- forward ---------------------------------------------------------

    @torch.no_grad()
    def forward(
        self,
        input_ids: torch.Tensor,
        positions: torch.Tensor,
        kv_cache: KVCache,
        meta: Union[PrefillMeta, DecodeMeta, MixedMeta],
    ) -> torch.Tensor:
        s = self.spec
        eps, mult = s.rms_eps, s.residual_mult
        n = len(self.layers)
        T, W = input_ids.shape[0], s.hidden_size
        # rows 0..i+1 hold the embedding output and the results of layers
        # 0..i; a layer accumulates its result in place in row i+1, which the
        # previous layer's depth average initialised with the layer's input
        stack = torch.empty(n + 2, T, W, dtype=torch.float32, device=input_ids.device)
        x0 = ops.embed_sinusoid(self.embedding, input_ids, positions, self.inv_freq)
        stack[0].copy_(x0)
        stack[1].copy_(x0)
        first = self.layers[0].t["norm1"] if n else self.final_norm
        h = ops.rmsnorm_cast(stack[1], first, eps, 0.0, self.dtype)
        for i, (ls, lw) in enumerate(zip(s.layers, self.layers)):
            m = ls.mixer
            res = stack[i + 1]
            p = F.linear(h, lw.t["in"])
            if m.kind == "mingru":
                y, y2 = self._mingru(p, lw, i, kv_cache, meta), None
                a1 = a2 = mult
            else:
                y = self._attention(p, lw, m.left, i, kv_cache, meta)
                y2 = self._mamba(p, lw, m.right, i, kv_cache, meta)
                a1, a2 = mult * m.left_scale, mult * m.right_scale
            w_next = self.layers[i + 1].t["norm1"] if i + 1 < n else self.final_norm
            if ls.moe:
                h = ops.scaled_add_norm(res, y, y2, a1, a2, lw.t["norm2"], eps, self.dtype)
                y, y2 = self._moe(h, lw, ls.moe, meta)
                a1 = a2 = mult
            h = ops.depth_mix_norm(stack, i + 2, lw.t["dwa"], y, y2, a1, a2, w_next, eps,
                                   self.dtype)
            if self.taps is not None:
                self.taps.append(stack[i + 2].clone())
        return h

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """final-normed hidden [N, width] -> logits [N, vocab] fp32."""
        logits = F.linear(hidden, self.lm_head).float()
        cap = self.spec.logit_softcap
        return torch_ref.softcap(logits, cap) if cap else logits

"""Tefudra: windowed attention and a matrix memory on an fp32 residual.

Every sublayer sits between two norms,

    x += norm_b(mixer(norm_1(x)));   x += norm_2b(ff(norm_2(x)))    (ff may be absent)

and every such norm splits the row into `groups` equal consecutive parts,
each divided by its own root mean square. Two kinds of mixer:

* sink attention — grouped key/value heads whose values are the keys as
  projected; q and k get a per-head RMSNorm and a rotation of their first
  rot.dims channels; position i sees j <= i with i - j < window or
  j < keep_first; the softmax denominator holds one more learned term per head.
* an averaged pair — capped attention (biased projections, a short causal
  convolution on q, k and v, tanh-capped scores, a plain sliding window,
  unit-norm values rotated by their own position and the head's output turned
  back by the query's) beside an mLSTM matrix memory (exponential gating with
  a running maximum, a normaliser vector, per-head norm and a sigmoid output
  gate); each output is RMS-normed over the width and the two are averaged.

Feed-forwards: dense with a squared ReLU, or a softmax-routed mixture of
exact-GELU experts (choice by score + correction, weights the renormalised
plain scores, identity experts that return their input) plus a shared expert.
A layer may run on another layer's tensors with a cache and state of its own.
The output head is the embedding table.

MI355X mapping, in the manner of the other hybrid families:

- plain-tensor weights; everything that reads the mixer's input in the model
  dtype is ONE GEMM per layer (attention: q ‖ k; pair: q ‖ k ‖ v of the left,
  then q ‖ k ‖ v ‖ gate of the right), segments at 16-byte boundaries, the
  left's biases folded into the GEMM; the memory's two gate rows per head run
  as a small fp32 GEMM beside it, like a router;
- the residual stays fp32; closing a sublayer and opening the next (post
  norm, add, pre norm, all grouped) is one kernel;
- keys and values go through the paged cache and the block table for prompt
  portions and single tokens alike; one kernel per token does the per-head
  norms, the rotations and the scatter; the paged attention kernels of the
  other families take the kept first tokens, the extra softmax term and the
  score cap as options;
- the convolution tail, the memory [dim, vdim + 1] per head (its last column
  is the normaliser, so n . q leaves the recurrence kernel as one more output
  column) and the running maximum live in per-sequence state slots; the
  memory runs on the diagonal-decay recurrence kernel of the other families in
  its scalar-gate mode, fed by a small kernel that walks the gates;
- a step's expert mixture runs sorted by expert on vendor GEMMs, or, inside
  captured decode graphs, as one batched GEMM pair over all experts.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Union

import torch
import torch.nn.functional as F

from llmq_amd import ops
from llmq_amd.engine.forward_meta import DecodeMeta, MixedMeta, PrefillMeta
from llmq_amd.engine.kv_cache import KVCache
from llmq_amd.engine.model_specs import TefudraSpec
from llmq_amd.engine.models.kosalorn import rotary_inv_freq


class TefudraLayerWeights:
    def __init__(self) -> None:
        self.t: Dict[str, torch.Tensor] = {}     # packed / checkpoint-shaped tensors
        self.seg: Dict[str, tuple] = {}          # name -> (first row, rows) in t["in"]
        self.inv_freq: Optional[torch.Tensor] = None     # fp32 rotary table of q and k
        self.v_inv_freq: Optional[torch.Tensor] = None   # fp32 rotary table of the values
        self.conv_cols = 0                       # columns of the packed projection the conv reads


def _align8(n: int) -> int:
    return -(-n // 8) * 8


class TefudraLM:
    #: HIP extension groups this family runs on
    ext_groups = ("hybrid",)
    #: prompt portions attend through the block table (no gathered copy)
    paged_prefill = True
    #: mixed steps run their decode and prefill segments one after the other
    #: (the expert GEMMs pick stream-k kernels at some shapes; those must not
    #: share the chip with a second stream's kernels)
    overlap_mixed = False

    def __init__(self, spec: TefudraSpec, device: torch.device, dtype: torch.dtype,
                 tp_rank: int = 0, tp_size: int = 1):
        if tp_size != 1:
            raise NotImplementedError("the hybrid families run on one GPU per replica")
        self.spec = spec
        self.device = device
        self.dtype = dtype
        self.tp_rank, self.tp_size = tp_rank, tp_size
        # one entry per layer of the spec; a layer that runs on another's
        # tensors shares that layer's weight object
        self.layers: List[TefudraLayerWeights] = []
        self.embedding: Optional[torch.Tensor] = None
        self.final_norm: Optional[torch.Tensor] = None
        self.taps: Optional[List[torch.Tensor]] = None  # stream after each layer (debug)
        self._alloc()

    @property
    def lm_head(self) -> torch.Tensor:
        return self.embedding

    # -- layout the engine asks for: one entry per layer, shared weights or not

    def kv_layout(self):
        out = []
        for ls in self.spec.layers:
            m = ls.mixer
            if m.kind == "sink_attention":
                out.append((m.kv_heads, m.dim, m.dim))
            else:
                out.append((m.left.kv_heads, m.left.dim, m.left.vdim))
        return out

    def state_layout(self):
        out = []
        for i, ls in enumerate(self.spec.layers):
            m = ls.mixer
            if m.kind == "sink_attention":
                out.append(None)
                continue
            r = m.right
            shapes = [(r.heads, r.dim, r.vdim + 1), (r.heads,)]
            if m.left.conv > 1:
                shapes.append((m.left.conv - 1, self.layers[i].conv_cols))
            out.append(shapes)
        return out

    # -- weights ---------------------------------------------------------

    def _empty(self, *shape, dtype=None) -> torch.Tensor:
        return torch.empty(*shape, device=self.device, dtype=dtype or self.dtype)

    def _alloc(self) -> None:
        s = self.spec
        W = s.hidden_size
        f32 = torch.float32
        self.embedding = self._empty(s.vocab_size, W)
        self.final_norm = self._empty(W)
        for i, ls in enumerate(s.layers):
            if ls.weights_of is not None:
                self.layers.append(None)
                continue
            lw = TefudraLayerWeights()
            m, t = ls.mixer, lw.t
            t["norm1"] = self._empty(W)
            t["norm1b"] = self._empty(W)
            if m.kind == "sink_attention":
                segs = [("q", m.heads * m.dim), ("k", m.kv_heads * m.dim)]
                t["q_norm"] = self._empty(m.dim)
                t["k_norm"] = self._empty(m.dim)
                t["sink"] = self._empty(m.heads, dtype=f32)
                t["o"] = self._empty(W, m.heads * m.dim)
            else:
                a, r = m.left, m.right
                segs = [("q", a.heads * a.dim), ("k", a.kv_heads * a.dim),
                        ("v", a.kv_heads * a.vdim)]
                lw.conv_cols = sum(_align8(n) for _, n in segs)
                segs += [("mq", r.heads * r.dim), ("mk", r.heads * r.dim),
                         ("mv", r.heads * r.vdim), ("mg", r.heads * r.vdim)]
                t["conv_w"] = self._empty(lw.conv_cols, a.conv, dtype=f32)
                t["o"] = self._empty(W, a.heads * a.vdim)
                t["o_b"] = self._empty(W)
                t["left_out"] = self._empty(W)
                t["gates"] = self._empty(2 * r.heads, W, dtype=f32)      # input | forget rows
                t["gates_b"] = self._empty(2 * r.heads, dtype=f32)
                t["m_norm"] = self._empty(r.heads * r.vdim)
                t["m_o"] = self._empty(W, r.heads * r.vdim)
                t["right_out"] = self._empty(W)
            at = 0
            for name, n in segs:
                lw.seg[name] = (at, n)
                at += _align8(n)
            t["in"] = self._empty(at, W)
            t["in"].zero_()
            if m.kind == "parallel":
                t["in_b"] = self._empty(at)
                t["in_b"].zero_()
                t["conv_w"].zero_()
            if ls.ff or ls.moe:
                t["norm2"] = self._empty(W)
                t["norm2b"] = self._empty(W)
            if ls.ff:
                t["up"] = self._empty(ls.ff, W)
                t["down"] = self._empty(W, ls.ff)
            if ls.moe:
                e = ls.moe
                t["router"] = self._empty(e.experts + e.identity, W, dtype=f32)
                t["correction"] = self._empty(e.experts + e.identity, dtype=f32)
                t["e_up"] = self._empty(e.experts, e.ff, W)
                t["e_down"] = self._empty(e.experts, W, e.ff)
                if e.shared_ff:
                    t["s_up"] = self._empty(e.shared_ff, W)
                    t["s_down"] = self._empty(W, e.shared_ff)
            self.layers.append(lw)
        for i in range(len(self.layers)):
            if self.layers[i] is None:
                self.layers[i] = self.layers[s.owner(i)]

    def owned_layers(self):
        """(index, spec, weights) of the layers that hold tensors of their own."""
        return [(i, ls, self.layers[i]) for i, ls in enumerate(self.spec.layers)
                if ls.weights_of is None]

    @torch.no_grad()
    def finalize(self) -> None:
        """Derive what the kernels read from the loaded tensors."""
        for _, ls, lw in self.owned_layers():
            m = ls.mixer
            a = m if m.kind == "sink_attention" else m.left
            lw.inv_freq = rotary_inv_freq(a.rot.base, a.rot.dims).to(self.device) \
                if a.rot.dims else None
            if m.kind == "parallel":
                lw.v_inv_freq = rotary_inv_freq(a.rot.base, a.vdim).to(self.device)

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
        fill(self.final_norm, 0.1, 1.0)
        for _, ls, lw in self.owned_layers():
            keep = torch.zeros(lw.t["in"].shape[0], dtype=torch.bool)
            for at, n in lw.seg.values():
                keep[at:at + n] = True
            keep = keep.to(self.device)
            biased = torch.zeros_like(keep)
            biased[:lw.conv_cols] = keep[:lw.conv_cols]
            for name, t in lw.t.items():
                if name in ("norm1", "norm2", "q_norm", "k_norm", "m_norm"):
                    fill(t, 0.1, 1.0)
                elif name in ("norm1b", "norm2b", "left_out", "right_out"):
                    fill(t, 0.05, 0.5)
                elif name == "sink":
                    fill(t, 1.0)
                elif name == "correction":
                    fill(t, 0.02)
                elif name in ("o_b", "gates_b"):
                    fill(t, 0.5)
                elif name == "in":
                    fill(t, 1.0 / math.sqrt(W))
                    t[~keep] = 0
                elif name == "in_b":
                    fill(t, 0.3)
                    t[~biased] = 0
                elif name == "conv_w":
                    fill(t, 0.5)
                    t[~keep[:lw.conv_cols]] = 0
                else:
                    fill(t, 1.0 / math.sqrt(t.shape[-1]))
        self.finalize()

    def named_tensors(self) -> Dict[str, torch.Tensor]:
        out = {"embedding": self.embedding, "final_norm": self.final_norm}
        for i, _, lw in self.owned_layers():
            for name, t in lw.t.items():
                out[f"layers.{i}.{name}"] = t
        return out

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.named_tensors().values())

    # -- mixers ----------------------------------------------------------

    @staticmethod
    def _cols(p: torch.Tensor, lw: TefudraLayerWeights, name: str) -> torch.Tensor:
        at, n = lw.seg[name]
        return p[:, at:at + n]

    def _attend(self, q, kc, vc, dv, a, meta, **extra):
        if meta.is_prefill:
            return ops.window_attn_prefill(
                q, kc, vc, dv, meta.block_tables, meta.cu_seqlens, meta.q_start, meta.max_seqlen,
                a.window, a.scale, **extra)
        if meta.is_mixed:
            nd, pm, dm = meta.n_decode, meta.prefill, meta.decode
            att_d = ops.window_attn_decode(
                q[:nd], kc, vc, dv, dm.block_tables, dm.context_lens, a.window, a.scale, **extra)
            att_p = ops.window_attn_prefill(
                q[nd:], kc, vc, dv, pm.block_tables, pm.cu_seqlens, pm.q_start, pm.max_seqlen,
                a.window, a.scale, **extra)
            return torch.cat([att_d, att_p], dim=0)
        return ops.window_attn_decode(
            q, kc, vc, dv, meta.block_tables, meta.context_lens, a.window, a.scale, **extra)

    def _sink_attention(self, p, lw, a, i, positions, kv_cache, meta):
        T = p.shape[0]
        q = self._cols(p, lw, "q").unflatten(1, (a.heads, a.dim))
        k = self._cols(p, lw, "k").unflatten(1, (a.kv_heads, a.dim))
        kc, vc = kv_cache.k[i], kv_cache.v[i]
        ops.qkv_norm_rope_cache(q, k, None, lw.t["q_norm"], lw.t["k_norm"], lw.inv_freq,
                                a.rot.dims, positions, kc, vc, meta.slot_mapping,
                                self.spec.rms_eps)
        att = self._attend(q, kc, vc, a.dim, a, meta, keep_first=a.keep_first, sink=lw.t["sink"])
        return F.linear(att.reshape(T, a.heads * a.dim), lw.t["o"])

    def _capped_attention(self, p, lw, a, i, positions, kv_cache, meta):
        T = p.shape[0]
        rm = meta.recurrent
        x = p[:, :lw.conv_cols]
        if a.conv > 1:
            x = ops.causal_conv_silu(x, lw.t["conv_w"], None, kv_cache.recurrent.state[i][2],
                                     rm.cu, rm.slots, rm.fresh, silu=False)
        else:
            x = (x.float() * lw.t["conv_w"][:, 0]).to(x.dtype)
        q = self._cols(x, lw, "q").unflatten(1, (a.heads, a.dim))
        k = self._cols(x, lw, "k").unflatten(1, (a.kv_heads, a.dim))
        v = self._cols(x, lw, "v").unflatten(1, (a.kv_heads, a.vdim))
        kc, vc = kv_cache.k[i], kv_cache.v[i]
        ops.qkv_norm_rope_cache(q, k, v, None, None, lw.inv_freq, a.rot.dims, positions, kc, vc,
                                meta.slot_mapping, self.spec.rms_eps, v_unit_norm=True,
                                v_inv_freq=lw.v_inv_freq)
        att = self._attend(q, kc, vc, a.vdim, a, meta, softcap=a.softcap)
        att = ops.rotate_heads(att, positions, lw.v_inv_freq, inverse=True)
        return F.linear(att.reshape(T, a.heads * a.vdim), lw.t["o"], lw.t["o_b"])

    def _memory(self, h32, p, lw, r, i, kv_cache, meta):
        rm = meta.recurrent
        S, m_state = kv_cache.recurrent.state[i][0], kv_cache.recurrent.state[i][1]
        gates = F.linear(h32, lw.t["gates"], lw.t["gates_b"])
        decay, write, floor = ops.mlstm_gates(gates, r.gate_cap, m_state, rm.cu, rm.slots, rm.fresh)
        q = self._cols(p, lw, "mq").unflatten(1, (r.heads, r.dim))
        k = self._cols(p, lw, "mk").unflatten(1, (r.heads, r.dim))
        v = self._cols(p, lw, "mv").unflatten(1, (r.heads, r.vdim))
        o = ops.matrix_memory(q, k, v, decay, write, S, rm.cu, rm.slots, rm.fresh,
                              r.dim ** -0.5)
        y = ops.mlstm_out_norm_gate(o, floor, lw.t["m_norm"], self._cols(p, lw, "mg"),
                                    self.spec.rms_eps, self.dtype)
        return F.linear(y, lw.t["m_o"])

    def _moe(self, h, h32, lw, e, meta):
        logits = F.linear(h32, lw.t["router"])
        idx, w = ops.softmax_topk(logits, e.top, 1.0, correction=lw.t["correction"], renorm=True)
        decode_only = not (meta.is_prefill or meta.is_mixed)
        y = ops.moe_experts(h, idx, w, lw.t["e_up"], lw.t["e_down"], sync_free=decode_only,
                            act="gelu_erf", weight_output=True, identity=e.identity)
        if e.shared_ff:
            mid = ops.unary_act(F.linear(h, lw.t["s_up"]), "gelu_erf")
            y = torch.addmm(y, mid, lw.t["s_down"].t())     # the join rides on the GEMM
        return y

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
        eps, groups = s.rms_eps, s.norm_groups
        n = len(self.layers)
        res = F.embedding(input_ids, self.embedding).float()
        first = self.layers[0].t["norm1"] if n else self.final_norm
        h = ops.rmsnorm_cast(res, first, eps, 0.0, self.dtype, groups)
        for i, (ls, lw) in enumerate(zip(s.layers, self.layers)):
            m = ls.mixer
            p = F.linear(h, lw.t["in"], lw.t.get("in_b"))
            if m.kind == "sink_attention":
                y = self._sink_attention(p, lw, m, i, positions, kv_cache, meta)
            else:
                yl = self._capped_attention(p, lw, m.left, i, positions, kv_cache, meta)
                yr = self._memory(h.float(), p, lw, m.right, i, kv_cache, meta)
                y = ops.dual_norm_mean(yl, lw.t["left_out"], yr, lw.t["right_out"], eps)
            w_next = self.layers[i + 1].t["norm1"] if i + 1 < n else self.final_norm
            if ls.ff or ls.moe:
                h = ops.sandwich_norm_res32(y, res, lw.t["norm1b"], lw.t["norm2"], eps, 0.0, groups)
                if ls.ff:
                    y = F.linear(ops.unary_act(F.linear(h, lw.t["up"]), "relu2"), lw.t["down"])
                else:
                    y = self._moe(h, h.float(), lw, ls.moe, meta)
                h = ops.sandwich_norm_res32(y, res, lw.t["norm2b"], w_next, eps, 0.0, groups)
            else:
                h = ops.sandwich_norm_res32(y, res, lw.t["norm1b"], w_next, eps, 0.0, groups)
            if self.taps is not None:
                self.taps.append(res.clone())
        return h

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """final-normed hidden [N, width] -> logits [N, vocab] fp32."""
        return F.linear(hidden, self.embedding).float()

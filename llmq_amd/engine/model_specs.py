"""Model architecture specs for the Llama/Qwen2/Gemma-2 families.

The reference serves Tower-Plus-{2B,9B,72B}, Llama-3.2 and Gemma-2 via vLLM
(README.md:98-108,169). All of those are decoder-only
RMSNorm+RoPE+GQA transformers differing in a handful of switches, captured
here as one ModelSpec:

  qkv_bias          Qwen2 adds bias to q/k/v projections
  tied_embeddings   small models tie lm_head to the embedding
  gelu              Gemma uses GeGLU (gelu_tanh) instead of SiLU
  post_norms        Gemma-2 adds post-attention/post-mlp norms
  attn_softcap /    Gemma-2 logit soft-capping
  final_softcap
  sliding_window    Gemma-2 alternates local/global attention layers
  embedding_scale   Gemma scales embeddings by sqrt(hidden)

A spec can be loaded from a HF checkpoint directory's config.json or picked
from the built-in presets by name (synthetic/random-init benchmarking —
no network in this environment).
"""

from __future__ import annotations

import json
import math
from dataclasses import dataclass, field
from pathlib import Path
from typing import Optional


@dataclass
class ModelSpec:
    name: str
    family: str  # "llama" | "qwen2" | "gemma2"
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    rms_eps: float = 1e-6
    rope_theta: float = 10000.0
    max_position_embeddings: int = 8192
    qkv_bias: bool = False
    tied_embeddings: bool = False
    gelu: bool = False
    post_norms: bool = False
    attn_softcap: float = 0.0
    final_softcap: float = 0.0
    sliding_window: int = 0  # 0 = none; Gemma-2: applied on even layers
    embedding_scale: bool = False
    attn_scale: Optional[float] = None  # default 1/sqrt(head_dim)
    rope_scaling: Optional[dict] = None  # HF rope_scaling (llama3/linear)
    eos_token_id: int = 2
    bos_token_id: int = 1

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def scale(self) -> float:
        if self.attn_scale is not None:
            return self.attn_scale
        return 1.0 / math.sqrt(self.head_dim)

    def layer_uses_sliding_window(self, layer_idx: int) -> bool:
        if self.sliding_window <= 0:
            return False
        # Gemma-2 alternates local/global layers; Mistral windows every layer.
        if self.family == "gemma2":
            return layer_idx % 2 == 0
        return True

    def param_count(self) -> int:
        embed = self.vocab_size * self.hidden_size
        per_layer = (
            self.hidden_size * (self.q_size + 2 * self.kv_size)  # qkv
            + self.q_size * self.hidden_size  # o
            + 3 * self.hidden_size * self.intermediate_size  # gate/up/down
            + 2 * self.hidden_size  # norms
        )
        if self.post_norms:
            per_layer += 2 * self.hidden_size
        total = embed + self.num_layers * per_layer + self.hidden_size
        if not self.tied_embeddings:
            total += embed
        return total


def _llama(name, vocab, hidden, inter, layers, heads, kv_heads, head_dim=None, **kw):
    return ModelSpec(
        name=name, family="llama", vocab_size=vocab, hidden_size=hidden,
        intermediate_size=inter, num_layers=layers, num_heads=heads,
        num_kv_heads=kv_heads, head_dim=head_dim or hidden // heads,
        rms_eps=1e-5, **kw,
    )


def _qwen2(name, vocab, hidden, inter, layers, heads, kv_heads, head_dim=None, **kw):
    return ModelSpec(
        name=name, family="qwen2", vocab_size=vocab, hidden_size=hidden,
        intermediate_size=inter, num_layers=layers, num_heads=heads,
        num_kv_heads=kv_heads, head_dim=head_dim or hidden // heads, rms_eps=1e-6,
        rope_theta=1000000.0, qkv_bias=True, **kw,
    )


def _gemma2(name, vocab, hidden, inter, layers, heads, kv_heads, head_dim, **kw):
    kw.setdefault("sliding_window", 4096)
    return ModelSpec(
        name=name, family="gemma2", vocab_size=vocab, hidden_size=hidden,
        intermediate_size=inter, num_layers=layers, num_heads=heads,
        num_kv_heads=kv_heads, head_dim=head_dim, rms_eps=1e-6,
        gelu=True, post_norms=True, attn_softcap=50.0, final_softcap=30.0,
        embedding_scale=True, tied_embeddings=True,
        eos_token_id=1, bos_token_id=2, **kw,
    )


# Llama-3.1/3.2 ship rope_scaling in config.json (rope_type "llama3");
# real checkpoints are wrong without it, so the presets carry it too.
_LLAMA31_ROPE = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                 "high_freq_factor": 4.0,
                 "original_max_position_embeddings": 8192}
_LLAMA32_ROPE = {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                 "high_freq_factor": 4.0,
                 "original_max_position_embeddings": 8192}

PRESETS = {
    # tiny configs for CPU tests
    # head_dim 64 (not hidden/heads = 16): the HIP attention kernels support
    # D in {64, 128, 256}, and the GPU consistency tests run these presets.
    "tiny-llama": _llama("tiny-llama", 512, 64, 128, 2, 4, 2, head_dim=64,
                         rope_theta=10000.0,
                         max_position_embeddings=512, tied_embeddings=True),
    "tiny-llama-d128": _llama("tiny-llama-d128", 512, 64, 128, 2, 4, 2,
                              head_dim=128, rope_theta=10000.0,
                              max_position_embeddings=512, tied_embeddings=True),
    "tiny-qwen2": _qwen2("tiny-qwen2", 512, 64, 128, 2, 4, 2, head_dim=64,
                         max_position_embeddings=512, tied_embeddings=True),
    "tiny-gemma2": _gemma2("tiny-gemma2", 512, 64, 128, 2, 4, 2, 64,
                           sliding_window=64, max_position_embeddings=512),
    # Llama 3.2 (vocab 128256, rope theta 500k)
    "llama-3.2-1b": _llama("llama-3.2-1b", 128256, 2048, 8192, 16, 32, 8,
                           head_dim=64, rope_theta=500000.0,
                           rope_scaling=_LLAMA32_ROPE,
                           max_position_embeddings=131072, tied_embeddings=True,
                           eos_token_id=128001, bos_token_id=128000),
    "llama-3.2-3b": _llama("llama-3.2-3b", 128256, 3072, 8192, 28, 24, 8,
                           head_dim=128, rope_theta=500000.0,
                           rope_scaling=_LLAMA32_ROPE,
                           max_position_embeddings=131072, tied_embeddings=True,
                           eos_token_id=128001, bos_token_id=128000),
    # Qwen2.5 family (Tower-Plus-2B = Qwen2.5-1.5B arch; -72B = Qwen2.5-72B)
    "qwen2.5-1.5b": _qwen2("qwen2.5-1.5b", 151936, 1536, 8960, 28, 12, 2,
                           max_position_embeddings=32768, tied_embeddings=True,
                           eos_token_id=151645, bos_token_id=151643),
    "qwen2.5-7b": _qwen2("qwen2.5-7b", 152064, 3584, 18944, 28, 28, 4,
                         max_position_embeddings=32768,
                         eos_token_id=151645, bos_token_id=151643),
    "qwen2.5-72b": _qwen2("qwen2.5-72b", 152064, 8192, 29568, 80, 64, 8,
                          max_position_embeddings=32768,
                          eos_token_id=151645, bos_token_id=151643),
    "qwen2.5-32b": _qwen2("qwen2.5-32b", 152064, 5120, 27648, 64, 40, 8,
                          max_position_embeddings=32768,
                          eos_token_id=151645, bos_token_id=151643),
    # Llama-3.1-8B / 70B (same layout; 70B pairs with TP=8 or fits 1 GPU)
    "llama-3.1-8b": _llama("llama-3.1-8b", 128256, 4096, 14336, 32, 32, 8,
                           head_dim=128, rope_theta=500000.0,
                           rope_scaling=_LLAMA31_ROPE,
                           max_position_embeddings=131072,
                           eos_token_id=128001, bos_token_id=128000),
    "llama-3.1-70b": _llama("llama-3.1-70b", 128256, 8192, 28672, 80, 64, 8,
                            head_dim=128, rope_theta=500000.0,
                            rope_scaling=_LLAMA31_ROPE,
                            max_position_embeddings=131072,
                            eos_token_id=128001, bos_token_id=128000),
    # Mistral-7B (llama layout, 4096-token sliding window on every layer)
    "mistral-7b": _llama("mistral-7b", 32000, 4096, 14336, 32, 32, 8,
                         rope_theta=10000.0, max_position_embeddings=32768,
                         sliding_window=4096, eos_token_id=2, bos_token_id=1),
    # Gemma-2 (Tower-Plus-9B is built on Gemma-2-9B)
    "gemma-2-9b": _gemma2("gemma-2-9b", 256000, 3584, 14336, 42, 16, 8, 256,
                          max_position_embeddings=8192),
    # 27b: query_pre_attn_scalar = hidden/heads = 144 (NOT head_dim as on
    # 9b) -> attention scale 1/sqrt(144)
    "gemma-2-27b": _gemma2("gemma-2-27b", 256000, 4608, 36864, 46, 32, 16, 128,
                           attn_scale=144.0 ** -0.5,
                           max_position_embeddings=8192),
}

# Aliases for the model names the reference's production configs use.
ALIASES = {
    "tower-plus-2b": "qwen2.5-1.5b",
    "unbabel/tower-plus-2b": "qwen2.5-1.5b",
    "tower-plus-9b": "gemma-2-9b",
    "unbabel/tower-plus-9b": "gemma-2-9b",
    "tower-plus-72b": "qwen2.5-72b",
    "unbabel/tower-plus-72b": "qwen2.5-72b",
    "llama-3.2-1b-instruct": "llama-3.2-1b",
    "meta-llama/llama-3.2-1b-instruct": "llama-3.2-1b",
    "llama-3.2-3b-instruct": "llama-3.2-3b",
    "meta-llama/llama-3.2-3b-instruct": "llama-3.2-3b",
    "google/gemma-2-9b": "gemma-2-9b",
    "google/gemma-2-9b-it": "gemma-2-9b",
    "google/gemma-2-27b": "gemma-2-27b",
    "meta-llama/llama-3.1-8b-instruct": "llama-3.1-8b",
    "llama-3.1-8b-instruct": "llama-3.1-8b",
    "meta-llama/llama-3.1-70b-instruct": "llama-3.1-70b",
    "llama-3.1-70b-instruct": "llama-3.1-70b",
    "qwen/qwen2.5-32b-instruct": "qwen2.5-32b",
}


# ---------------------------------------------------------------------------
# Hybrid decoders: a per-layer list of sequence mixers (block-local biased
# attention, gated linear attention) with optional gated feed-forwards, an
# fp32 residual stream and a zero-centred norm sandwich round every sublayer.


@dataclass
class BlockBiasAttnSpec:
    """Attention whose keys are limited to the query's own span of `span`
    positions (counted from position 0), with a learned bias per bucketed
    distance, one RMSNorm over the whole q / k projection, optional value
    blending with the first blending layer, and a sigmoid gate per head."""

    heads: int
    kv_heads: int
    dim: int            # per-head q/k size
    vdim: int           # per-head v size
    scale: float
    span: int           # mask span
    bias_far: float     # distance at which the log buckets reach the last row
    bias_rows: int = 16  # rows of the bias table (read from the tensor's shape)
    v_mix: bool = False
    kind: str = "attention"


@dataclass
class GLASpec:
    """Gated linear attention: per head S ← diag(a) S + k vᵀ, o = Sᵀ q, with
    a = sigmoid(low-rank(h) + b)^(1/tau) per key channel."""

    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int = 16  # inner size of the decay projection (tensor shape)
    kind: str = "gla"


@dataclass
class HybridLayerSpec:
    mixer: object                 # BlockBiasAttnSpec | GLASpec
    ff: int = 0                   # 0 = the layer has no feed-forward
    ff_kind: str = "dense"


@dataclass
class HybridSpec:
    name: str
    family: str                   # "kakovik"
    vocab_size: int
    hidden_size: int
    layers: list = field(default_factory=list)
    rms_eps: float = 1e-6
    logit_scale: float = 1.0
    # no positional table: the limit only bounds block tables
    max_position_embeddings: int = 1 << 17
    tied_embeddings: bool = False
    eos_token_id: int = 2
    bos_token_id: int = 1

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def param_count(self) -> int:
        w = self.hidden_size
        total = 2 * self.vocab_size * w + w
        for ls in self.layers:
            m = ls.mixer
            total += 2 * w
            if m.kind == "attention":
                nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
                total += w * (nq + nk + nv + m.heads) + nq + nk
                total += m.heads * m.vdim * w + m.bias_rows * m.heads + 1
            else:
                nk, nv = m.heads * m.dim, m.heads * m.vdim
                total += w * (2 * nk + 2 * nv + m.decay_rank) + m.decay_rank * nk + nk
                total += nv * w + m.vdim
            if ls.ff:
                total += 2 * w + 3 * w * ls.ff
        return total


def _safetensors_shapes(path: Path) -> dict:
    """name → shape from a safetensors header (8-byte length + JSON); no
    tensor data is read."""
    import struct

    with open(path, "rb") as fh:
        (n,) = struct.unpack("<Q", fh.read(8))
        header = json.loads(fh.read(n))
    return {k: v["shape"] for k, v in header.items() if k != "__metadata__"}


def kakovik_spec_from_config(cfg: dict, name: str, shapes: Optional[dict] = None) -> HybridSpec:
    """Kakovik config.json → HybridSpec. Sizes the config does not carry
    (bias-table rows, decay rank) come from the checkpoint's tensor shapes."""
    shapes = shapes or {}
    layers = []
    for i, lc in enumerate(cfg["layers"]):
        mc = lc["mixer"]
        kind = lc["type"]
        if kind == "attention":
            rel = shapes.get(f"l{i}.mix.rel")
            mixer = BlockBiasAttnSpec(
                heads=mc["heads"], kv_heads=mc.get("kv_heads", mc["heads"]),
                dim=mc["dim"], vdim=mc.get("vdim", mc["dim"]),
                scale=float(mc["scale"]), span=int(mc["mask"]["size"]),
                bias_far=float(mc["bias_max"]),
                bias_rows=int(rel[0]) if rel else 16,
                v_mix=bool(mc.get("v_mix", False)),
            )
        elif kind == "gla":
            a1 = shapes.get(f"l{i}.mix.a1")
            mixer = GLASpec(
                heads=mc["heads"], dim=mc["dim"], vdim=mc.get("vdim", mc["dim"]),
                tau=float(mc["tau"]), decay_rank=int(a1[0]) if a1 else 16,
            )
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        mlp = lc.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        layers.append(HybridLayerSpec(mixer=mixer, ff=int(mlp["ff"]) if mlp else 0))
    return HybridSpec(
        name=name, family="kakovik", vocab_size=int(cfg["vocab"]),
        hidden_size=int(cfg["width"]), layers=layers,
        rms_eps=float(cfg["norm"]["eps"]), logit_scale=float(cfg.get("logit_scale", 1.0)),
    )


def _kakovik(name, vocab, width, n_layers, heads, kv_heads, dim, vdim, ff, span,
             gla_every=3, gla_heads=None, gla_dim=None, gla_vdim=None, **kw):
    """Preset builder: every `gla_every`-th layer is a gated-linear-attention
    layer without feed-forward, the others attention + dense feed-forward."""
    layers = []
    for i in range(n_layers):
        if gla_every and i % gla_every == gla_every - 1:
            layers.append(HybridLayerSpec(GLASpec(
                heads=gla_heads or heads, dim=gla_dim or dim, vdim=gla_vdim or vdim,
                tau=16.0, decay_rank=16)))
        else:
            layers.append(HybridLayerSpec(BlockBiasAttnSpec(
                heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=dim ** -0.5,
                span=span, bias_far=float(span), bias_rows=32, v_mix=True), ff=ff))
    return HybridSpec(name=name, family="kakovik", vocab_size=vocab, hidden_size=width,
                      layers=layers, **kw)


HYBRID_PRESETS = {
    # CPU/GPU test config: unequal q/v sizes, grouped kv heads, short spans
    "tiny-kakovik": _kakovik("tiny-kakovik", 512, 64, 3, 4, 2, 32, 16, 128, 24,
                             gla_every=2, gla_heads=2, gla_dim=16, gla_vdim=32),
    # benchmark configs at the layer sizes of llama-3.2-1b / -3b (the closest
    # existing models): same width, heads, head size, feed-forward and depth
    "kakovik-1b": _kakovik("kakovik-1b", 128256, 2048, 16, 32, 8, 64, 64, 8192, 2048,
                           gla_every=4, gla_heads=16, gla_dim=64, gla_vdim=128),
    "kakovik-3b": _kakovik("kakovik-3b", 128256, 3072, 28, 24, 8, 128, 128, 8192, 2048,
                           gla_every=4, gla_heads=12, gla_dim=128, gla_vdim=256),
}


# ---------------------------------------------------------------------------
# Kosalorn: a looped hybrid decoder. One norm per layer feeds a sequence
# mixer (latent attention or an HGRN2 recurrence) and a feed-forward (dense
# or a mixture of experts) in parallel, each behind a sigmoid gate, followed
# by a per-layer token-indexed side input. A range of layers may run several
# times in a row with the same weights (each pass with its own cache/state).


@dataclass
class RotarySpec:
    """Rotary positions on the first `dims` coordinates of a vector: pair i
    turns by position * base^(-2i/dims). layout "half": pair (i, i+dims/2);
    "interleaved": pair (2i, 2i+1)."""

    base: float
    dims: int
    layout: str = "half"


@dataclass
class LatentAttnSpec:
    """Attention over a shared low-rank latent: per token only the normed
    latent (kv_rank) and one rotated key part (rot_dim) are cached; per-head
    keys and values are linear maps of the latent. q_rank > 0: the query goes
    through a normed latent too. window 0 = causal, else position i sees
    j with 0 <= i - j < window."""

    heads: int
    dim: int            # per-head unrotated q/k size
    rot_dim: int        # per-head rotated q size = shared rotated key size
    vdim: int
    kv_rank: int
    scale: float
    rot: RotarySpec = None
    q_rank: int = 0
    window: int = 0
    kind: str = "latent_attention"


@dataclass
class HGRN2Spec:
    """Linear attention whose forget gate f = l + (1-l)*sigmoid(.) also sets
    the write strength: S <- diag(f) S + (1-f) v^T, o = S^T q."""

    heads: int
    dim: int
    vdim: int
    kind: str = "hgrn2"


@dataclass
class MoESpec:
    """Mixture of gated feed-forward experts: sigmoid router scores, the
    `top` best experts per token, the score scales the expert's INPUT."""

    experts: int
    top: int
    ff: int             # per-expert inner size


@dataclass
class KosalornLayerSpec:
    mixer: object                 # LatentAttnSpec | HGRN2Spec
    ff: int = 0                   # dense feed-forward inner size (0 = none)
    moe: Optional[MoESpec] = None


@dataclass
class KosalornSpec:
    name: str
    family: str                   # "kosalorn"
    vocab_size: int
    hidden_size: int
    layers: list = field(default_factory=list)
    rms_eps: float = 1e-6
    side_dim: int = 0             # per-layer token side input width (0 = none)
    loop_start: int = 0           # layers [loop_start, loop_stop) run
    loop_stop: int = 0            # loop_times times in a row
    loop_times: int = 1
    max_position_embeddings: int = 1 << 17
    tied_embeddings: bool = False
    eos_token_id: int = 2
    bos_token_id: int = 1

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> list:
        """Execution order: [(layer index, adds the embedding output first)].
        A looped layer appears once per pass; every entry owns its own cache
        or state."""
        n = len(self.layers)
        a, b, times = self.loop_start, self.loop_stop, self.loop_times
        if times == 1 or b <= a:
            return [(i, False) for i in range(n)]
        order = [(i, False) for i in range(a)]
        for p in range(times):
            order += [(i, p > 0 and i == a) for i in range(a, b)]
        return order + [(i, False) for i in range(b, n)]

    def param_count(self) -> int:
        w = self.hidden_size
        total = 2 * self.vocab_size * w + 2
        total += self.vocab_size * self.side_dim * len(self.layers)
        for ls in self.layers:
            m = ls.mixer
            total += 1 + (2 if (ls.ff or ls.moe) else 1) * (w * w + w)
            if m.kind == "hgrn2":
                nk, nv = m.heads * m.dim, m.heads * m.vdim
                total += 2 * nk * w + 2 * nk + nv * w + m.vdim + w * nv
            else:
                nq = m.heads * (m.dim + m.rot_dim)
                total += (m.q_rank * (w + 1 + nq)) if m.q_rank else nq * w
                total += (m.kv_rank + m.rot_dim) * w + m.kv_rank
                total += m.kv_rank * m.heads * (m.dim + m.vdim) + w * m.heads * m.vdim
            if ls.ff:
                total += 3 * w * ls.ff
            if ls.moe:
                total += ls.moe.experts * (3 * w * ls.moe.ff + w)
            if self.side_dim:
                total += 2 * w * self.side_dim + w
        return total


def kosalorn_spec_from_config(cfg: dict, name: str) -> KosalornSpec:
    """Kosalorn config.json -> KosalornSpec. Every size and constant comes
    from the config; the layer type fixes the rotary layout and whether the
    query has a latent."""
    layers = []
    for i, lc in enumerate(cfg["layers"]):
        mc, kind = lc["mixer"], lc["type"]
        if kind in ("latent_attention", "latent_attention_2"):
            rot = mc["rot"]
            mask = mc.get("mask")
            mixer = LatentAttnSpec(
                heads=int(mc["heads"]), dim=int(mc["dim"]), rot_dim=int(mc["rot_dim"]),
                vdim=int(mc["vdim"]), kv_rank=int(mc["kv_rank"]),
                scale=float(mc.get("scale", (int(mc["dim"]) + int(mc["rot_dim"])) ** -0.5)),
                rot=RotarySpec(base=float(rot["base"]), dims=int(rot["dims"]),
                               layout="half" if kind == "latent_attention" else "interleaved"),
                q_rank=int(mc.get("q_rank", 0)) if kind == "latent_attention" else 0,
                window=int(mask["size"]) if mask else 0,
            )
            if kind == "latent_attention" and not mixer.q_rank:
                raise ValueError(f"layer {i}: latent_attention needs q_rank")
            if mixer.rot.dims > mixer.rot_dim or mixer.rot.dims % 2:
                raise ValueError(f"layer {i}: rot.dims must be even and at most rot_dim")
        elif kind == "hgrn2":
            mixer = HGRN2Spec(heads=int(mc["heads"]), dim=int(mc["dim"]), vdim=int(mc["vdim"]))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        mlp = lc.get("mlp")
        ff, moe = 0, None
        if mlp is not None:
            if mlp.get("kind", "dense") == "dense":
                ff = int(mlp["ff"])
            elif mlp["kind"] == "moe":
                moe = MoESpec(experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
                              ff=int(mlp["expert"]["ff"]))
                if not 1 <= moe.top <= moe.experts:
                    raise ValueError(f"layer {i}: top must be within 1..experts")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
        layers.append(KosalornLayerSpec(mixer=mixer, ff=ff, moe=moe))
    loop = cfg.get("loop") or {}
    side = cfg.get("token_side") or {}
    spec = KosalornSpec(
        name=name, family="kosalorn", vocab_size=int(cfg["vocab"]),
        hidden_size=int(cfg["width"]), layers=layers, rms_eps=float(cfg["norm"]["eps"]),
        side_dim=int(side.get("dim", 0)),
        loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
        loop_times=int(loop.get("times", 1)),
    )
    if not 0 <= spec.loop_start <= spec.loop_stop <= len(layers):
        raise ValueError("loop range outside the layer list")
    return spec


def _kosalorn(name, vocab, width, n_layers, heads, dim, rot_dim, vdim, kv_rank, q_rank, ff,
              window=0, rec_every=4, rec_heads=None, rec_dim=None, rec_vdim=None,
              moe_every=0, experts=8, top=2, expert_ff=None, side_dim=0, loop=None, **kw):
    """Preset builder: every `rec_every`-th layer is an HGRN2 layer, the
    others latent attention (alternating the windowed query-latent form and
    the causal direct-query form); every `moe_every`-th feed-forward is a
    mixture of experts, the others dense."""
    layers = []
    for i in range(n_layers):
        if rec_every and i % rec_every == rec_every - 1:
            mixer = HGRN2Spec(heads=rec_heads or heads, dim=rec_dim or dim, vdim=rec_vdim or vdim)
        elif i % 2 == 0:
            mixer = LatentAttnSpec(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim,
                                   kv_rank=kv_rank, scale=(dim + rot_dim) ** -0.5,
                                   rot=RotarySpec(250000.0, rot_dim, "half"),
                                   q_rank=q_rank, window=window)
        else:
            mixer = LatentAttnSpec(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim,
                                   kv_rank=kv_rank, scale=(dim + rot_dim) ** -0.5,
                                   rot=RotarySpec(500000.0, rot_dim, "interleaved"))
        if moe_every and i % moe_every == moe_every - 1:
            layers.append(KosalornLayerSpec(mixer, moe=MoESpec(experts, top, expert_ff or ff)))
        else:
            layers.append(KosalornLayerSpec(mixer, ff=ff))
    a, b, times = loop or (0, 0, 1)
    return KosalornSpec(name=name, family="kosalorn", vocab_size=vocab, hidden_size=width,
                        layers=layers, side_dim=side_dim, loop_start=a, loop_stop=b,
                        loop_times=times, **kw)


KOSALORN_PRESETS = {
    # CPU/GPU test config: every mixer and feed-forward kind, a looped range
    "tiny-kosalorn": _kosalorn("tiny-kosalorn", 512, 64, 4, 4, 16, 8, 24, 40, 24, 96,
                               window=24, rec_every=3, rec_heads=2, rec_dim=16, rec_vdim=32,
                               moe_every=2, experts=6, top=2, expert_ff=32, side_dim=8,
                               loop=(1, 3, 2)),
    # benchmark configs at the layer sizes of llama-3.2-1b / -3b (the closest
    # existing models): same width, head count, feed-forward and depth; the
    # head size is split into an unrotated and a rotated part, the latent is
    # four heads wide
    "kosalorn-1b": _kosalorn("kosalorn-1b", 128256, 2048, 16, 32, 32, 32, 64, 192, 768, 8192,
                             window=2048, rec_every=4, rec_heads=16, rec_dim=64, rec_vdim=128),
    "kosalorn-3b": _kosalorn("kosalorn-3b", 128256, 3072, 28, 24, 64, 64, 128, 192, 1536, 8192,
                             window=2048, rec_every=4, rec_heads=12, rec_dim=128, rec_vdim=256),
    # the same with every second feed-forward a mixture of 8 experts, 2 per
    # token, each a quarter of the dense inner size
    "kosalorn-1b-moe": _kosalorn("kosalorn-1b-moe", 128256, 2048, 16, 32, 32, 32, 64, 192, 768,
                                 8192, window=2048, rec_every=4, rec_heads=16, rec_dim=64,
                                 rec_vdim=128, moe_every=2, experts=8, top=2, expert_ff=2048,
                                 side_dim=64),
}


# ---------------------------------------------------------------------------
# Muvetar: a hybrid decoder on an fp32 residual whose layers carry either a
# minGRU recurrence or two mixers side by side (softmax attention with a
# logarithmic distance penalty, and a Mamba selective scan), a mixture-of-
# experts feed-forward with a shared expert, and a learned average over the
# outputs of all earlier layers ("depth average") at every layer's end.
# Positions enter through a sinusoidal vector added to the embedding and
# through the attention's distance penalty only.


@dataclass
class MinGRUSpec:
    """Gated recurrence whose gates read only the current token:
    S_t = (1 - z_t) S_{t-1} + z_t c_t with z = sigmoid(.), c = g(.),
    g(u) = u + 1/2 for u >= 0 and sigmoid(u) below; the output is
    W_o (S_t * silu(W_g h))."""

    width: int
    kind: str = "mingru"


@dataclass
class LogBiasAttnSpec:
    """Causal softmax attention with grouped key/value heads and no rotation;
    head a's score for distance d = i - j is q.k * scale - r1_a ln(1 + r2_a d)."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    kind: str = "log_bias_attention"


@dataclass
class MambaSpec:
    """Selective scan: a short causal convolution per channel, then per
    channel c and state n  S <- exp(dt_c A[c, n]) S + dt_c x_c B_n,
    y_c = sum_n S C_n + D_c x_c, gated by silu(z)."""

    inner: int
    state: int
    dt_rank: int
    conv: int
    kind: str = "mamba"


@dataclass
class ParallelMixerSpec:
    """Two mixers reading the same input; their outputs are added with fixed
    scales."""

    left: LogBiasAttnSpec
    right: MambaSpec
    left_scale: float = 1.0
    right_scale: float = 1.0
    kind: str = "parallel"


@dataclass
class SoftmaxMoESpec:
    """Mixture of clamped gated experts: scores = softmax of the router
    logits over ALL experts, the `top` largest chosen, their scores times
    `scale` (not renormalised) weight the experts' OUTPUTS. Expert:
    g = min(W_gate h, limit), u = clamp(W_up h, +-limit),
    W_down(g * sigmoid(1.702 g) * (u + 1)). shared_ff > 0: one more expert of
    the same form (own inner size and limit) runs for every token."""

    experts: int
    top: int
    ff: int
    limit: float
    scale: float = 1.0
    shared_ff: int = 0
    shared_limit: float = 0.0


@dataclass
class MuvetarLayerSpec:
    mixer: object                          # MinGRUSpec | ParallelMixerSpec
    moe: Optional[SoftmaxMoESpec] = None   # None: the layer has no feed-forward


@dataclass
class MuvetarSpec:
    name: str
    family: str                   # "muvetar"
    vocab_size: int
    hidden_size: int
    layers: list = field(default_factory=list)
    rms_eps: float = 1e-6
    residual_mult: float = 1.0    # every sublayer output is scaled by this
    logit_softcap: float = 0.0    # 0 = none
    max_position_embeddings: int = 1 << 17
    tied_embeddings: bool = False
    eos_token_id: int = 2
    bos_token_id: int = 1

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def param_count(self) -> int:
        w = self.hidden_size
        total = 2 * self.vocab_size * w + w
        for i, ls in enumerate(self.layers):
            m = ls.mixer
            total += w + (i + 2)
            if m.kind == "mingru":
                total += 3 * m.width * w + 2 * m.width + w * m.width
            else:
                a, r = m.left, m.right
                total += (a.heads * a.dim + a.kv_heads * (a.dim + a.vdim)) * w
                total += 2 * a.heads + w * a.heads * a.vdim
                total += 2 * r.inner * w + r.inner * (r.conv + 1)
                total += (r.dt_rank + 2 * r.state) * r.inner + r.inner * (r.dt_rank + 1)
                total += r.inner * r.state + r.inner + w * r.inner
            if ls.moe:
                e = ls.moe
                total += w + e.experts * (3 * w * e.ff + w) + 3 * w * e.shared_ff
        return total


def muvetar_spec_from_config(cfg: dict, name: str) -> MuvetarSpec:
    """Muvetar config.json -> MuvetarSpec: every size and constant comes from
    the config."""
    layers = []
    for i, lc in enumerate(cfg["layers"]):
        mc, kind = lc["mixer"], lc["type"]
        if kind == "mingru":
            mixer = MinGRUSpec(width=int(mc.get("width", cfg["width"])))
        elif kind == "parallel":
            lt, rt = mc["left"], mc["right"]
            heads = int(lt["heads"])
            left = LogBiasAttnSpec(
                heads=heads, kv_heads=int(lt.get("kv_heads", heads)), dim=int(lt["dim"]),
                vdim=int(lt.get("vdim", lt["dim"])), scale=float(lt["scale"]))
            if left.heads % left.kv_heads:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            right = MambaSpec(inner=int(rt["inner"]), state=int(rt["state"]),
                              dt_rank=int(rt["dt_rank"]), conv=int(rt["conv"]))
            if right.conv < 1:
                raise ValueError(f"layer {i}: the convolution needs at least one tap")
            mixer = ParallelMixerSpec(left=left, right=right,
                                      left_scale=float(mc.get("left_scale", 1.0)),
                                      right_scale=float(mc.get("right_scale", 1.0)))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        mlp, moe = lc.get("mlp"), None
        if mlp is not None:
            if mlp.get("kind", "moe") != "moe":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            rt, ex, sh = mlp["router"], mlp["expert"], mlp.get("shared")
            moe = SoftmaxMoESpec(
                experts=int(rt["experts"]), top=int(rt["top"]), ff=int(ex["ff"]),
                limit=float(ex["limit"]), scale=float(rt.get("scale", 1.0)),
                shared_ff=int(sh["ff"]) if sh else 0,
                shared_limit=float(sh["limit"]) if sh else 0.0)
            if not 1 <= moe.top <= moe.experts:
                raise ValueError(f"layer {i}: top must be within 1..experts")
        layers.append(MuvetarLayerSpec(mixer=mixer, moe=moe))
    return MuvetarSpec(
        name=name, family="muvetar", vocab_size=int(cfg["vocab"]),
        hidden_size=int(cfg["width"]), layers=layers, rms_eps=float(cfg["norm"]["eps"]),
        residual_mult=float(cfg.get("residual_mult", 1.0)),
        logit_softcap=float(cfg.get("logit_softcap") or 0.0),
    )


def _muvetar(name, vocab, width, n_layers, heads, kv_heads, dim, vdim, inner, state, dt_rank,
             experts, top, ff, shared_ff, parallel_every=2, gru_width=None, conv=4,
             left_scale=1.0, right_scale=1.0, limit=7.0, router_scale=1.0, **kw):
    """Preset builder: every `parallel_every`-th layer (starting with the
    first) carries attention beside a selective scan, the others a minGRU;
    every layer has the expert mixture with a shared expert."""
    layers = []
    for i in range(n_layers):
        if i % parallel_every == 0:
            mixer = ParallelMixerSpec(
                LogBiasAttnSpec(heads, kv_heads, dim, vdim, dim ** -0.5),
                MambaSpec(inner, state, dt_rank, conv), left_scale, right_scale)
        else:
            mixer = MinGRUSpec(gru_width or width)
        layers.append(MuvetarLayerSpec(mixer, SoftmaxMoESpec(
            experts, top, ff, limit, router_scale, shared_ff, limit)))
    return MuvetarSpec(name=name, family="muvetar", vocab_size=vocab, hidden_size=width,
                       layers=layers, **kw)


MUVETAR_PRESETS = {
    # CPU/GPU test config: both layer types, grouped kv heads, q/k size != v
    # size, a recurrence narrower than the model, a state size that is no
    # power of two
    "tiny-muvetar": _muvetar("tiny-muvetar", 512, 64, 4, 4, 2, 16, 24, 96, 12, 6, 6, 2, 32, 48,
                             gru_width=48, conv=3, left_scale=1.1, right_scale=0.8,
                             limit=1.5, router_scale=1.3, residual_mult=0.5,
                             logit_softcap=20.0),
    # benchmark configs at the layer sizes of llama-3.2-1b / -3b and of the
    # Kosalorn expert-mixture preset: same width, head count and depth; the
    # scan is two model widths wide with 16 states per channel; 8 experts,
    # 2 per token, each a quarter of the dense inner size, plus a shared one
    "muvetar-1b": _muvetar("muvetar-1b", 128256, 2048, 16, 32, 8, 64, 64, 4096, 16, 128,
                           8, 2, 2048, 2048),
    "muvetar-3b": _muvetar("muvetar-3b", 128256, 3072, 28, 24, 8, 128, 128, 6144, 16, 192,
                           8, 2, 2048, 2048),
}


# ---------------------------------------------------------------------------
# Tefudra: a hybrid decoder on an fp32 residual whose norms work on equal
# consecutive groups of the width. A layer carries either softmax attention
# whose values are its keys (per-head q/k norm, partial rotation, a sliding
# window that also keeps the first tokens, a learned extra term per head in
# the softmax denominator), or two mixers side by side whose normed outputs
# are averaged: tanh-capped sliding-window attention behind a short causal
# convolution with position-rotated unit-norm values, and an mLSTM matrix
# memory. Feed-forwards are dense (squared ReLU) or a softmax-routed mixture
# of GELU experts with identity experts and a shared expert. A layer may run
# on another layer's weights with a cache and state of its own.


@dataclass
class SinkAttnSpec:
    """Softmax attention with grouped key/value heads whose values are the
    keys as projected (before norm and rotation). Position i sees j <= i with
    i - j < window (window 0: every j <= i) or j < keep_first; the softmax
    denominator holds one more term exp(sink_head)."""

    heads: int
    kv_heads: int
    dim: int
    scale: float
    rot: RotarySpec = None
    window: int = 0
    keep_first: int = 0
    kind: str = "sink_attention"

    @property
    def vdim(self) -> int:
        return self.dim


@dataclass
class CappedConvAttnSpec:
    """Sliding-window softmax attention with biased projections, a causal
    convolution of `conv` taps per channel on q, k and v, scores passed
    through softcap * tanh(. / softcap) (softcap 0: none), values divided by
    their root mean square per head and rotated by their own position over
    all of vdim; a head's output is turned back by the query's position."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotarySpec = None
    window: int = 0
    softcap: float = 0.0
    conv: int = 1
    kind: str = "capped_conv_attention"


@dataclass
class MLSTMSpec:
    """Matrix memory per head with exponential gating: log input gate
    i = cap tanh(. / cap), log forget gate f = logsigmoid(cap tanh(. / cap)),
    running maximum m_t = max(f + m_(t-1), i) from m = 0,
    S_t = e^(f + m_(t-1) - m_t) S_(t-1) + e^(i - m_t) k v^T, n_t alike with k,
    o = S_t^T q / (max(|n_t . q|, e^(-m_t)) + 1e-6)."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float
    kind: str = "mlstm"


@dataclass
class AveragedPairSpec:
    """Two mixers on the same input; the result is half the sum of their
    outputs, each RMS-normed over the model width with its own weight."""

    left: CappedConvAttnSpec
    right: MLSTMSpec
    kind: str = "parallel"


@dataclass
class RoutedFFSpec:
    """Mixture of ungated experts W_down gelu(W_up h) (exact GELU). Scores =
    softmax of the router logits over experts + identity experts; the `top`
    largest of score + correction are chosen, their scores divided by their
    sum weigh the outputs; an identity expert returns its input. shared_ff >
    0: one more expert of the same form runs for every token."""

    experts: int
    top: int
    ff: int
    identity: int = 0
    shared_ff: int = 0


@dataclass
class TefudraLayerSpec:
    mixer: object                           # SinkAttnSpec | AveragedPairSpec
    ff: int = 0                             # dense feed-forward inner size (0 = none)
    moe: Optional[RoutedFFSpec] = None
    weights_of: Optional[int] = None        # runs on this layer's tensors


@dataclass
class TefudraSpec:
    name: str
    family: str                   # "tefudra"
    vocab_size: int
    hidden_size: int
    layers: list = field(default_factory=list)
    rms_eps: float = 1e-6
    norm_groups: int = 1
    max_position_embeddings: int = 1 << 17
    tied_embeddings: bool = True
    eos_token_id: int = 2
    bos_token_id: int = 1

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def owner(self, i: int) -> int:
        """The layer whose tensors layer i runs on."""
        seen = set()
        while self.layers[i].weights_of is not None:
            if i in seen:
                raise ValueError("weights_of forms a cycle")
            seen.add(i)
            i = self.layers[i].weights_of
        return i

    def param_count(self) -> int:
        w = self.hidden_size
        total = self.vocab_size * w + w
        for ls in self.layers:
            if ls.weights_of is not None:
                continue
            m = ls.mixer
            total += 4 * w if (ls.ff or ls.moe) else 2 * w
            if m.kind == "sink_attention":
                total += (m.heads + m.kv_heads) * m.dim * w + 2 * m.dim + m.heads
                total += w * m.heads * m.dim
            else:
                a, r = m.left, m.right
                n = a.heads * a.dim + a.kv_heads * (a.dim + a.vdim)
                total += n * (w + 1 + a.conv) + w * a.heads * a.vdim + w
                total += r.heads * (2 * r.dim + 2 * r.vdim) * w + r.heads * r.vdim
                total += w * r.heads * r.vdim + 2 * r.heads * (w + 1) + 2 * w
            if ls.ff:
                total += 2 * w * ls.ff
            if ls.moe:
                e = ls.moe
                total += (e.experts + e.identity) * (w + 1)
                total += 2 * w * (e.experts * e.ff + e.shared_ff)
        return total


def _rotary_from(rc: dict, size: int, where: str) -> RotarySpec:
    rot = RotarySpec(base=float(rc["base"]), dims=int(rc.get("dims", size)), layout="half")
    if rot.dims % 2 or not 0 <= rot.dims <= size:
        raise ValueError(f"{where}: rot.dims must be even and at most the head size")
    return rot


def tefudra_spec_from_config(cfg: dict, name: str) -> TefudraSpec:
    """Tefudra config.json -> TefudraSpec: every size and constant comes from
    the config."""
    layers = []
    raw = cfg["layers"]
    for i, lc in enumerate(raw):
        mc, kind = lc["mixer"], lc["type"]
        if kind == "attention":
            heads = int(mc["heads"])
            mask = mc.get("mask") or {}
            mixer = SinkAttnSpec(
                heads=heads, kv_heads=int(mc.get("kv_heads", heads)), dim=int(mc["dim"]),
                scale=float(mc.get("scale", int(mc["dim"]) ** -0.5)),
                rot=_rotary_from(mc["rot"], int(mc["dim"]), f"layer {i}"),
                window=int(mask.get("size", 0)), keep_first=int(mask.get("keep_first", 0)))
            if int(mc.get("vdim", mixer.dim)) != mixer.dim:
                raise ValueError(f"layer {i}: values are the keys, so vdim must equal dim")
            pairs = [mixer]
        elif kind == "parallel":
            lt, rt = mc["left"], mc["right"]
            heads = int(lt["heads"])
            mask = lt.get("mask") or {}
            left = CappedConvAttnSpec(
                heads=heads, kv_heads=int(lt.get("kv_heads", heads)), dim=int(lt["dim"]),
                vdim=int(lt.get("vdim", lt["dim"])),
                scale=float(lt.get("scale", int(lt["dim"]) ** -0.5)),
                rot=_rotary_from(lt["rot"], int(lt["dim"]), f"layer {i}"),
                window=int(mask.get("size", 0)), softcap=float(lt.get("softcap") or 0.0),
                conv=int(lt.get("conv", 1)))
            if left.vdim % 2:
                raise ValueError(f"layer {i}: rotated values need an even vdim")
            if left.conv < 1:
                raise ValueError(f"layer {i}: the convolution needs at least one tap")
            right = MLSTMSpec(heads=int(rt["heads"]), dim=int(rt["dim"]), vdim=int(rt["vdim"]),
                              gate_cap=float(rt["gate_cap"]))
            mixer = AveragedPairSpec(left=left, right=right)
            pairs = [left]
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        for a in pairs:
            if a.heads % a.kv_heads:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
        mlp = lc.get("mlp")
        ff, moe = 0, None
        if mlp is not None:
            if mlp.get("kind", "dense") == "dense":
                ff = int(mlp["ff"])
            elif mlp["kind"] == "moe":
                rt, sh = mlp["router"], mlp.get("shared")
                moe = RoutedFFSpec(experts=int(rt["experts"]), top=int(rt["top"]),
                                   ff=int(mlp["expert"]["ff"]), identity=int(rt.get("identity", 0)),
                                   shared_ff=int(sh["ff"]) if sh else 0)
                if not 1 <= moe.top <= moe.experts + moe.identity:
                    raise ValueError(f"layer {i}: top must be within 1..experts + identity")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
        src = lc.get("weights_of")
        if src is not None and not 0 <= int(src) < len(raw):
            raise ValueError(f"layer {i}: weights_of names no layer")
        layers.append(TefudraLayerSpec(mixer=mixer, ff=ff, moe=moe,
                                       weights_of=None if src is None else int(src)))
    spec = TefudraSpec(
        name=name, family="tefudra", vocab_size=int(cfg["vocab"]),
        hidden_size=int(cfg["width"]), layers=layers, rms_eps=float(cfg["norm"]["eps"]),
        norm_groups=int(cfg["norm"].get("groups", 1)))
    if spec.hidden_size % spec.norm_groups:
        raise ValueError("norm.groups must divide the width")
    for i in range(len(layers)):
        spec.owner(i)
    return spec


def _tefudra(name, vocab, width, n_layers, heads, kv_heads, dim, ff, window, keep_first=4,
             groups=4, attn_every=3, left_dim=None, left_vdim=None, left_window=None, conv=4,
             softcap=20.0, mem_heads=None, mem_dim=None, mem_vdim=None, gate_cap=15.0,
             moe_every=0, experts=8, identity=2, top=2, expert_ff=None, shared_ff=0,
             rot_dims=None, share_last=False, **kw):
    """Preset builder: every `attn_every`-th layer is a sink-attention layer,
    the others carry capped attention beside a matrix memory; every
    `moe_every`-th feed-forward is a routed mixture, the others dense;
    share_last: the last layer runs on the weights of the nearest earlier
    layer of its kind."""
    layers = []
    ld, lv = left_dim or dim, left_vdim or left_dim or dim
    for i in range(n_layers):
        if attn_every and i % attn_every == attn_every - 1:
            mixer = SinkAttnSpec(heads, kv_heads, dim, dim ** -0.5,
                                 RotarySpec(1000000.0, rot_dims or dim, "half"), window, keep_first)
        else:
            mixer = AveragedPairSpec(
                CappedConvAttnSpec(heads, kv_heads, ld, lv, ld ** -0.5,
                                   RotarySpec(250000.0, ld, "half"), left_window or window,
                                   softcap, conv),
                MLSTMSpec(mem_heads or heads, mem_dim or dim, mem_vdim or dim, gate_cap))
        if moe_every and i % moe_every == moe_every - 1:
            layers.append(TefudraLayerSpec(mixer, moe=RoutedFFSpec(
                experts, top, expert_ff or ff, identity, shared_ff)))
        else:
            layers.append(TefudraLayerSpec(mixer, ff=ff))
    if share_last and n_layers > 1:
        for j in range(n_layers - 2, -1, -1):
            if layers[j].mixer.kind == layers[-1].mixer.kind:
                layers[-1] = TefudraLayerSpec(layers[j].mixer, layers[j].ff, layers[j].moe, j)
                break
    return TefudraSpec(name=name, family="tefudra", vocab_size=vocab, hidden_size=width,
                       layers=layers, norm_groups=groups, **kw)


TEFUDRA_PRESETS = {
    # CPU/GPU test config: both layer types, both feed-forwards, grouped kv
    # heads, q/k size != v size, partial rotation, a shared-weights layer
    "tiny-tefudra": _tefudra("tiny-tefudra", 512, 64, 6, 4, 2, 16, 96, 24, keep_first=3,
                             groups=2, attn_every=3, left_dim=24, left_vdim=16, left_window=20,
                             conv=3, softcap=8.0, mem_heads=2, mem_dim=8, mem_vdim=24,
                             gate_cap=10.0, moe_every=2, experts=5, identity=2, top=3,
                             expert_ff=32, shared_ff=48, rot_dims=8, share_last=True),
    # benchmark configs at the layer sizes of llama-3.2-1b / -3b (and of the
    # other hybrid presets): same width, head count, feed-forward and depth;
    # every 4th layer sink attention, window 2048
    "tefudra-1b": _tefudra("tefudra-1b", 128256, 2048, 16, 32, 8, 64, 8192, 2048, attn_every=4,
                           mem_heads=16, mem_dim=64, mem_vdim=128),
    "tefudra-1b-moe": _tefudra("tefudra-1b-moe", 128256, 2048, 16, 32, 8, 64, 8192, 2048,
                               attn_every=4, mem_heads=16, mem_dim=64, mem_vdim=128,
                               moe_every=2, experts=8, identity=2, top=2, expert_ff=2048,
                               shared_ff=2048),
    "tefudra-3b": _tefudra("tefudra-3b", 128256, 3072, 28, 24, 8, 128, 8192, 2048, attn_every=4,
                           mem_heads=12, mem_dim=128, mem_vdim=256),
}


def spec_from_hf_config(path: Path, name: str) -> ModelSpec:
    """Build a spec from a HF checkpoint directory's config.json."""
    with open(path / "config.json", "r", encoding="utf-8") as fh:
        cfg = json.load(fh)
    if str(cfg.get("architecture", "")).lower() == "kosalorn":
        return kosalorn_spec_from_config(cfg, name)
    if str(cfg.get("architecture", "")).lower() == "muvetar":
        return muvetar_spec_from_config(cfg, name)
    if str(cfg.get("architecture", "")).lower() == "tefudra":
        return tefudra_spec_from_config(cfg, name)
    if str(cfg.get("architecture", "")).lower() == "kakovik":
        st = path / "model.safetensors"
        return kakovik_spec_from_config(
            cfg, name, _safetensors_shapes(st) if st.is_file() else None)
    arch = (cfg.get("architectures") or [""])[0].lower()
    model_type = cfg.get("model_type", "").lower()
    if "gemma2" in arch or model_type == "gemma2":
        family = "gemma2"
    elif "qwen2" in arch or model_type == "qwen2":
        family = "qwen2"
    elif "mistral" in arch or model_type == "mistral":
        family = "mistral"  # llama layout + sliding window on every layer
    else:
        family = "llama"
    heads = cfg["num_attention_heads"]
    hidden = cfg["hidden_size"]
    head_dim = cfg.get("head_dim") or hidden // heads
    # rope config: transformers <=4.x puts rope_theta at top level and the
    # scaling dict under "rope_scaling"; transformers 5.x nests BOTH under
    # "rope_parameters". Normalise to (theta, scaling-or-None).
    rope_params = cfg.get("rope_scaling") or cfg.get("rope_parameters") or {}
    rope_theta = cfg.get("rope_theta") or rope_params.get("rope_theta") or 10000.0
    rope_type = rope_params.get("rope_type") or rope_params.get("type")
    rope_scaling = dict(rope_params) if rope_type not in (None, "default") else None
    spec = ModelSpec(
        name=name,
        family=family,
        vocab_size=cfg["vocab_size"],
        hidden_size=hidden,
        intermediate_size=cfg["intermediate_size"],
        num_layers=cfg["num_hidden_layers"],
        num_heads=heads,
        num_kv_heads=cfg.get("num_key_value_heads", heads),
        head_dim=head_dim,
        rms_eps=cfg.get("rms_norm_eps", 1e-6),
        rope_theta=rope_theta,
        rope_scaling=rope_scaling,
        max_position_embeddings=cfg.get("max_position_embeddings", 8192),
        qkv_bias=family == "qwen2",
        tied_embeddings=cfg.get("tie_word_embeddings", False),
        gelu=family == "gemma2",
        post_norms=family == "gemma2",
        attn_softcap=cfg.get("attn_logit_softcapping") or 0.0,
        final_softcap=cfg.get("final_logit_softcapping") or 0.0,
        sliding_window=(
            (cfg.get("sliding_window") or 0) if family in ("gemma2", "mistral") else 0
        ),
        embedding_scale=family == "gemma2",
        attn_scale=(
            cfg.get("query_pre_attn_scalar") and 1.0 / math.sqrt(cfg["query_pre_attn_scalar"])
        ),
        eos_token_id=_first(cfg.get("eos_token_id"), 2),
        bos_token_id=_first(cfg.get("bos_token_id"), 1),
    )
    return spec


def _first(x, default: int = 2) -> int:
    # HF configs may carry an int, a list, or null (e.g. Qwen2 bos_token_id).
    if x is None:
        return default
    if isinstance(x, list):
        return int(x[0]) if x else default
    return int(x)


def resolve_spec(model: str) -> ModelSpec:
    """Resolve a model name or checkpoint path to a spec."""
    path = Path(model)
    if path.is_dir() and (path / "config.json").is_file():
        return spec_from_hf_config(path, path.name)
    key = model.lower()
    key = ALIASES.get(key, key)
    if key in PRESETS:
        return PRESETS[key]
    if key in HYBRID_PRESETS:
        return HYBRID_PRESETS[key]
    if key in KOSALORN_PRESETS:
        return KOSALORN_PRESETS[key]
    if key in MUVETAR_PRESETS:
        return MUVETAR_PRESETS[key]
    if key in TEFUDRA_PRESETS:
        return TEFUDRA_PRESETS[key]
    raise ValueError(
        f"Unknown model '{model}'. Provide a checkpoint directory with config.json "
        f"or one of: {sorted(PRESETS) + sorted(HYBRID_PRESETS) + sorted(KOSALORN_PRESETS) + sorted(MUVETAR_PRESETS) + sorted(TEFUDRA_PRESETS) + sorted(ALIASES)}"
    )

"""Safetensors checkpoint loading (HF layout → packed in-tree layout).

Reference counterpart: vLLM's weight loader, consumed implicitly through
AsyncLLMEngine.from_engine_args (vllm_worker.py:105-123). Handles the
Llama/Qwen2/Gemma-2 HF naming and packs q/k/v and gate/up into the fused
GEMM tensors. Tensor-parallel loads take each rank's shard only.
"""

from __future__ import annotations

import logging
from pathlib import Path
from typing import Dict, List

import torch

logger = logging.getLogger(__name__)


def _shard_rows(t: torch.Tensor, rank: int, size: int) -> torch.Tensor:
    if size == 1:
        return t
    n = t.shape[0] // size
    return t[rank * n : (rank + 1) * n]


def _shard_cols(t: torch.Tensor, rank: int, size: int) -> torch.Tensor:
    if size == 1:
        return t
    n = t.shape[1] // size
    return t[:, rank * n : (rank + 1) * n]


def load_safetensors_weights(model, path: Path) -> None:
    loader = _FAMILY_LOADERS.get(model.spec.family)
    if loader:
        loader(model, path)
        return
    from safetensors import safe_open  # noqa: PLC0415

    spec = model.spec
    rank, size = model.tp_rank, model.tp_size
    files = sorted(path.glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors under {path}")

    # name → file handle lazily
    tensors: Dict[str, torch.Tensor] = {}
    for f in files:
        with safe_open(str(f), framework="pt", device="cpu") as sf:
            for name in sf.keys():
                tensors[name] = sf.get_tensor(name)

    def get(name: str) -> torch.Tensor:
        for candidate in (name, "model." + name):
            if candidate in tensors:
                return tensors[candidate]
        raise KeyError(f"missing tensor {name} (have {len(tensors)})")

    def copy_(dst: torch.Tensor, src: torch.Tensor) -> None:
        if dst.shape != src.shape:
            raise ValueError(f"shape mismatch: {tuple(dst.shape)} vs {tuple(src.shape)}")
        dst.copy_(src.to(dst.dtype))

    copy_(model.embedding, get("embed_tokens.weight"))
    copy_(model.final_norm, get("norm.weight"))
    if not spec.tied_embeddings:
        copy_(model.lm_head, tensors.get("lm_head.weight", get("embed_tokens.weight")))

    for i, lw in enumerate(model.layers):
        p = f"layers.{i}."
        copy_(lw.input_norm, get(p + "input_layernorm.weight"))
        q = _shard_rows(get(p + "self_attn.q_proj.weight"), rank, size)
        k = _shard_rows(get(p + "self_attn.k_proj.weight"), rank, size)
        v = _shard_rows(get(p + "self_attn.v_proj.weight"), rank, size)
        copy_(lw.qkv, torch.cat([q, k, v], dim=0))
        if lw.qkv_bias is not None:
            qb = _shard_rows(get(p + "self_attn.q_proj.bias"), rank, size)
            kb = _shard_rows(get(p + "self_attn.k_proj.bias"), rank, size)
            vb = _shard_rows(get(p + "self_attn.v_proj.bias"), rank, size)
            copy_(lw.qkv_bias, torch.cat([qb, kb, vb], dim=0))
        copy_(lw.o, _shard_cols(get(p + "self_attn.o_proj.weight"), rank, size))
        gate = _shard_rows(get(p + "mlp.gate_proj.weight"), rank, size)
        up = _shard_rows(get(p + "mlp.up_proj.weight"), rank, size)
        copy_(lw.gate_up, torch.cat([gate, up], dim=0))
        copy_(lw.down, _shard_cols(get(p + "mlp.down_proj.weight"), rank, size))
        if spec.post_norms:
            copy_(lw.post_attn_norm, get(p + "post_attention_layernorm.weight"))
            copy_(lw.pre_mlp_norm, get(p + "pre_feedforward_layernorm.weight"))
            copy_(lw.post_mlp_norm, get(p + "post_feedforward_layernorm.weight"))
        else:
            copy_(lw.pre_mlp_norm, get(p + "post_attention_layernorm.weight"))
    logger.info("loaded %d tensors from %s", len(tensors), path)


def load_kakovik_weights(model, path: Path) -> None:
    """Kakovik checkpoint names → the packed in-tree tensors.

    Checkpoint: 'embed', 'head', 'final.norm', and per layer 'l<i>.norm1',
    'l<i>.norm1b' (+ 'norm2', 'norm2b' with a feed-forward), the mixer under
    'l<i>.mix.' and the feed-forward under 'l<i>.mlp.'; linear weights are
    [out, in]. Packing: attention q‖k‖v‖g → qkvg, GLA q‖k‖v‖g‖a1 → qkvga,
    feed-forward gate‖up → gate_up."""
    from safetensors import safe_open  # noqa: PLC0415

    files = sorted(path.glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors under {path}")
    tensors: Dict[str, torch.Tensor] = {}
    for f in files:
        with safe_open(str(f), framework="pt", device="cpu") as sf:
            for name in sf.keys():
                tensors[name] = sf.get_tensor(name)
    used = set()

    def get(name: str) -> torch.Tensor:
        if name not in tensors:
            raise KeyError(f"missing tensor {name}")
        used.add(name)
        return tensors[name]

    def copy_(dst: torch.Tensor, src: torch.Tensor) -> None:
        if dst.shape != src.shape:
            raise ValueError(f"shape mismatch: {tuple(dst.shape)} vs {tuple(src.shape)}")
        dst.copy_(src.to(dst.dtype))

    copy_(model.embedding, get("embed"))
    copy_(model.lm_head, get("head"))
    copy_(model.final_norm, get("final.norm"))
    for i, (ls, lw) in enumerate(zip(model.spec.layers, model.layers)):
        p, t = f"l{i}.", lw.t
        copy_(t["norm1"], get(p + "norm1"))
        copy_(t["norm1b"], get(p + "norm1b"))
        mx = p + "mix."
        if ls.mixer.kind == "attention":
            packed = torch.cat([get(mx + "q"), get(mx + "k"), get(mx + "v"), get(mx + "g")], dim=0)
            t["qkvg"].zero_()  # trailing alignment rows
            copy_(t["qkvg"][: packed.shape[0]], packed)
            copy_(t["q_norm"], get(mx + "q.norm"))
            copy_(t["k_norm"], get(mx + "k.norm"))
            copy_(t["rel"], get(mx + "rel"))
            copy_(t["vmix"], get(mx + "vmix"))
            copy_(t["o"], get(mx + "o"))
        else:
            copy_(t["qkvga"], torch.cat([get(mx + "q"), get(mx + "k"), get(mx + "v"),
                                         get(mx + "g"), get(mx + "a1")], dim=0))
            copy_(t["a2"], get(mx + "a2"))
            copy_(t["a2_b"], get(mx + "a2.b"))
            copy_(t["norm"], get(mx + "norm"))
            copy_(t["o"], get(mx + "o"))
        if ls.ff:
            copy_(t["norm2"], get(p + "norm2"))
            copy_(t["norm2b"], get(p + "norm2b"))
            copy_(t["gate_up"], torch.cat([get(p + "mlp.gate"), get(p + "mlp.up")], dim=0))
            copy_(t["down"], get(p + "mlp.down"))
    unused = sorted(set(tensors) - used)
    if unused:
        raise ValueError(f"checkpoint tensors the model does not know: {unused[:8]}")
    model.finalize()
    logger.info("loaded %d tensors from %s", len(tensors), path)


def _read_all(path: Path) -> Dict[str, torch.Tensor]:
    from safetensors import safe_open  # noqa: PLC0415

    files = sorted(path.glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors under {path}")
    tensors: Dict[str, torch.Tensor] = {}
    for f in files:
        with safe_open(str(f), framework="pt", device="cpu") as sf:
            for name in sf.keys():
                tensors[name] = sf.get_tensor(name)
    return tensors


def load_kosalorn_weights(model, path: Path) -> None:
    """Kosalorn checkpoint names -> the packed in-tree tensors.

    Checkpoint: 'embed', 'embed.norm', 'head', 'final.norm', 'side.embed', and
    per layer 'l<i>.norm1', the gates 'l<i>.rg1' / '.rg1.b' / '.rg2' /
    '.rg2.b', the mixer under 'l<i>.mix.', the feed-forward under
    'l<i>.mlp.' (experts 'e<j>.'), the side input under 'l<i>.side.'; linear
    weights are [out, in]. Packing: mixer input projections ‖ rg1 ‖ rg2 ->
    'in' (segments at multiples of 8 rows), feed-forward gate‖up -> gate_up,
    experts stacked [E, ...]; uk / uv split per head."""
    tensors = _read_all(path)
    used = set()

    def get(name: str) -> torch.Tensor:
        if name not in tensors:
            raise KeyError(f"missing tensor {name}")
        used.add(name)
        return tensors[name]

    def copy_(dst: torch.Tensor, src: torch.Tensor) -> None:
        if dst.shape != src.shape:
            raise ValueError(f"shape mismatch: {tuple(dst.shape)} vs {tuple(src.shape)}")
        dst.copy_(src.to(dst.dtype))

    spec = model.spec
    copy_(model.embedding, get("embed"))
    copy_(model.embed_norm, get("embed.norm"))
    copy_(model.lm_head, get("head"))
    copy_(model.final_norm, get("final.norm"))
    if spec.side_dim:
        copy_(model.side_embed, get("side.embed"))
    for i, (ls, lw) in enumerate(zip(spec.layers, model.layers)):
        p, t, m = f"l{i}.", lw.t, ls.mixer
        mx = p + "mix."
        copy_(t["norm1"], get(p + "norm1"))

        def put(seg: str, src: torch.Tensor, lw=lw, t=t) -> None:
            at, n = lw.seg[seg]
            copy_(t["in"][at:at + n], src)

        t["in"].zero_()  # alignment rows between segments
        if m.kind == "hgrn2":
            put("q", get(mx + "q"))
            put("f", get(mx + "f"))
            put("v", get(mx + "v"))
            copy_(t["f_b"], get(mx + "f.b"))
            copy_(t["lower"], get(mx + "lower"))
            copy_(t["norm"], get(mx + "norm"))
        else:
            if m.q_rank:
                put("dq", get(mx + "dq"))
                copy_(t["dq_norm"], get(mx + "dq.norm"))
                copy_(t["uq"], get(mx + "uq"))
            else:
                put("q", get(mx + "q"))
            put("dkv", get(mx + "dkv"))
            copy_(t["dkv_norm"], get(mx + "dkv.norm"))
            copy_(t["uk"], get(mx + "uk").view(m.heads, m.dim, m.kv_rank))
            copy_(t["uv"], get(mx + "uv").view(m.heads, m.vdim, m.kv_rank))
        copy_(t["o"], get(mx + "o"))
        put("rg1", get(p + "rg1"))
        copy_(t["rg1_b"], get(p + "rg1.b"))
        if ls.ff or ls.moe:
            put("rg2", get(p + "rg2"))
            copy_(t["rg2_b"], get(p + "rg2.b"))
        if ls.ff:
            copy_(t["gate_up"], torch.cat([get(p + "mlp.gate"), get(p + "mlp.up")], dim=0))
            copy_(t["down"], get(p + "mlp.down"))
        if ls.moe:
            copy_(t["router"], get(p + "mlp.router"))
            for e in range(ls.moe.experts):
                ep = f"{p}mlp.e{e}."
                copy_(t["e_gate_up"][e], torch.cat([get(ep + "gate"), get(ep + "up")], dim=0))
                copy_(t["e_down"][e], get(ep + "down"))
        if spec.side_dim:
            copy_(t["side_gate"], get(p + "side.gate"))
            copy_(t["side_proj"], get(p + "side.proj"))
            copy_(t["side_norm"], get(p + "side.norm"))
    unused = sorted(set(tensors) - used)
    if unused:
        logger.warning("checkpoint tensors this configuration does not use: %s", unused[:8])
    model.finalize()
    logger.info("loaded %d tensors from %s", len(tensors), path)


def load_muvetar_weights(model, path: Path) -> None:
    """Muvetar checkpoint names -> the packed in-tree tensors.

    Checkpoint: 'embed', 'head', 'final.norm', and per layer 'l<i>.norm1',
    'l<i>.norm2', 'l<i>.dwa', the mixer under 'l<i>.mix.' (a parallel layer's
    two mixers under '.left.' and '.right.'), the feed-forward under
    'l<i>.mlp.' (experts 'e<j>.', the shared expert 'shared.'); linear weights
    are [out, in]. Packing: everything that reads the mixer's input -> 'in'
    (segments at multiples of 8 rows), gate‖up -> one tensor, experts stacked
    [E, ...], the attention's two distance numbers -> [heads, 2]."""
    tensors = _read_all(path)
    used = set()

    def get(name: str) -> torch.Tensor:
        if name not in tensors:
            raise KeyError(f"missing tensor {name}")
        used.add(name)
        return tensors[name]

    def copy_(dst: torch.Tensor, src: torch.Tensor) -> None:
        if dst.shape != src.shape:
            raise ValueError(f"shape mismatch: {tuple(dst.shape)} vs {tuple(src.shape)}")
        dst.copy_(src.to(dst.dtype))

    spec = model.spec
    copy_(model.embedding, get("embed"))
    copy_(model.lm_head, get("head"))
    copy_(model.final_norm, get("final.norm"))
    for i, (ls, lw) in enumerate(zip(spec.layers, model.layers)):
        p, t, m = f"l{i}.", lw.t, ls.mixer
        mx = p + "mix."
        copy_(t["norm1"], get(p + "norm1"))
        copy_(t["dwa"], get(p + "dwa"))

        def put(seg: str, src: torch.Tensor, lw=lw, t=t) -> None:
            at, n = lw.seg[seg]
            copy_(t["in"][at:at + n], src)

        t["in"].zero_()  # alignment rows between segments
        if m.kind == "mingru":
            put("z", get(mx + "z"))
            put("u", get(mx + "x"))
            put("g", get(mx + "g"))
            copy_(t["z_b"], get(mx + "z.b"))
            copy_(t["u_b"], get(mx + "x.b"))
            copy_(t["o"], get(mx + "o"))
        else:
            lf, rt, r = mx + "left.", mx + "right.", m.right
            put("q", get(lf + "q"))
            put("k", get(lf + "k"))
            put("v", get(lf + "v"))
            copy_(t["r12"], torch.stack([get(lf + "r1").float(), get(lf + "r2").float()], dim=1))
            copy_(t["attn_o"], get(lf + "o"))
            w_in = get(rt + "in")
            if w_in.shape[0] != 2 * r.inner:
                raise ValueError(f"{rt}in: expected {2 * r.inner} rows")
            put("x", w_in[: r.inner])
            put("gate", w_in[r.inner:])
            copy_(t["conv_w"], get(rt + "conv"))
            copy_(t["conv_b"], get(rt + "conv.b"))
            copy_(t["xproj"], get(rt + "x"))
            copy_(t["dt"], get(rt + "dt"))
            copy_(t["dt_b"], get(rt + "dt.b"))
            copy_(t["A_log"], get(rt + "A_log"))
            copy_(t["D"], get(rt + "D"))
            copy_(t["scan_o"], get(rt + "o"))
        if ls.moe:
            e = ls.moe
            copy_(t["norm2"], get(p + "norm2"))
            copy_(t["router"], get(p + "mlp.router"))
            for j in range(e.experts):
                ep = f"{p}mlp.e{j}."
                copy_(t["e_gate_up"][j], torch.cat([get(ep + "gate"), get(ep + "up")], dim=0))
                copy_(t["e_down"][j], get(ep + "down"))
            if e.shared_ff:
                sp = p + "mlp.shared."
                copy_(t["s_gate_up"], torch.cat([get(sp + "gate"), get(sp + "up")], dim=0))
                copy_(t["s_down"], get(sp + "down"))
    unused = sorted(set(tensors) - used)
    if unused:
        logger.warning("checkpoint tensors this configuration does not use: %s", unused[:8])
    model.finalize()
    logger.info("loaded %d tensors from %s", len(tensors), path)


def load_tefudra_weights(model, path: Path) -> None:
    """Tefudra checkpoint names -> the packed in-tree tensors.

    Checkpoint: 'embed' (also the output head), 'final.norm', and per layer
    that owns tensors 'l<i>.norm1', '.norm1b', '.norm2', '.norm2b', the mixer
    under 'l<i>.mix.' (an averaged pair's two mixers under '.left.' and
    '.right.', their output norms '.left.out' / '.right.out'), the
    feed-forward under 'l<i>.mlp.' (experts 'e<j>.', the shared expert
    'shared.'); linear weights are [out, in], a bias is the weight's name +
    '.b', a short convolution's taps the weight's name + '.conv'. Packing:
    everything that reads the mixer's input in the model dtype -> 'in' (+ the
    biases -> 'in_b', the taps -> 'conv_w', segments at multiples of 8 rows),
    the memory's input and forget gate rows -> one fp32 'gates', experts
    stacked [E, ...]."""
    tensors = _read_all(path)
    used = set()

    def get(name: str) -> torch.Tensor:
        if name not in tensors:
            raise KeyError(f"missing tensor {name}")
        used.add(name)
        return tensors[name]

    def copy_(dst: torch.Tensor, src: torch.Tensor) -> None:
        if dst.shape != src.shape:
            raise ValueError(f"shape mismatch: {tuple(dst.shape)} vs {tuple(src.shape)}")
        dst.copy_(src.to(dst.dtype))

    copy_(model.embedding, get("embed"))
    copy_(model.final_norm, get("final.norm"))
    for i, ls, lw in model.owned_layers():
        p, t, m = f"l{i}.", lw.t, ls.mixer
        mx = p + "mix."
        copy_(t["norm1"], get(p + "norm1"))
        copy_(t["norm1b"], get(p + "norm1b"))

        def put(seg: str, src: torch.Tensor, dst: str = "in", lw=lw, t=t) -> None:
            at, n = lw.seg[seg]
            copy_(t[dst][at:at + n], src)

        t["in"].zero_()  # alignment rows between segments
        if m.kind == "sink_attention":
            put("q", get(mx + "q"))
            put("k", get(mx + "k"))
            copy_(t["q_norm"], get(mx + "q.norm"))
            copy_(t["k_norm"], get(mx + "k.norm"))
            copy_(t["sink"], get(mx + "sink"))
            copy_(t["o"], get(mx + "o"))
        else:
            lf, rt = mx + "left.", mx + "right."
            t["in_b"].zero_()
            t["conv_w"].zero_()
            for seg in ("q", "k", "v"):
                put(seg, get(lf + seg))
                put(seg, get(lf + seg + ".b"), "in_b")
                put(seg, get(lf + seg + ".conv"), "conv_w")
            copy_(t["o"], get(lf + "o"))
            copy_(t["o_b"], get(lf + "o.b"))
            copy_(t["left_out"], get(lf + "out"))
            for seg, name in (("mq", "q"), ("mk", "k"), ("mv", "v"), ("mg", "g")):
                put(seg, get(rt + name))
            copy_(t["gates"], torch.cat([get(rt + "i"), get(rt + "f")], dim=0))
            copy_(t["gates_b"], torch.cat([get(rt + "i.b"), get(rt + "f.b")], dim=0))
            copy_(t["m_norm"], get(rt + "norm"))
            copy_(t["m_o"], get(rt + "o"))
            copy_(t["right_out"], get(rt + "out"))
        if ls.ff or ls.moe:
            copy_(t["norm2"], get(p + "norm2"))
            copy_(t["norm2b"], get(p + "norm2b"))
        if ls.ff:
            copy_(t["up"], get(p + "mlp.up"))
            copy_(t["down"], get(p + "mlp.down"))
        if ls.moe:
            e = ls.moe
            copy_(t["router"], get(p + "mlp.router"))
            copy_(t["correction"], get(p + "mlp.correction"))
            for j in range(e.experts):
                copy_(t["e_up"][j], get(f"{p}mlp.e{j}.up"))
                copy_(t["e_down"][j], get(f"{p}mlp.e{j}.down"))
            if e.shared_ff:
                copy_(t["s_up"], get(p + "mlp.shared.up"))
                copy_(t["s_down"], get(p + "mlp.shared.down"))
    unused = sorted(set(tensors) - used)
    if unused:
        logger.warning("checkpoint tensors this configuration does not use: %s", unused[:8])
    model.finalize()
    logger.info("loaded %d tensors from %s", len(tensors), path)


_FAMILY_LOADERS = {"kakovik": load_kakovik_weights, "kosalorn": load_kosalorn_weights,
                   "muvetar": load_muvetar_weights, "tefudra": load_tefudra_weights}

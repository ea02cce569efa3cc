"""Muvetar (scan/attention hybrid decoder) against the plain oracle in
muvetar_oracle.py.

Every test builds its own small configuration and random checkpoint, loads
it through the engine's own entry points (config reader, weight loader,
scheduler, cache and state managers) and compares logits with the oracle.
The scenarios run on the CPU (torch reference ops) and, marked ``gpu``, on
the HIP kernels in fp32 (sharp) and bf16.

Expert routing is a discrete choice: a bf16 run rounds the router's input,
so a near-tie may fall the other way than in the float64 oracle. Whole-model
bf16 scenarios therefore use mixtures in which every expert is chosen (the
scores still weigh the outputs); the choice itself is checked in fp32 at
model level and in bf16 at op level, where the oracle sees the same inputs.
"""

from __future__ import annotations

import json
import math

import pytest
import torch

import muvetar_oracle as oracle
from llmq_amd import ops
from llmq_amd.engine.config import EngineConfig
from llmq_amd.engine.engine import LLMEngine
from llmq_amd.engine.sampling_params import SamplingParams


# --------------------------------------------------------------- fixtures --

def moe_cfg(experts=5, top=2, ff=24, limit=1.5, scale=1.3, shared=(20, 0.8)):
    cfg = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
           "router": {"experts": experts, "top": top, "scale": scale}}
    cfg["shared"] = {"ff": shared[0], "limit": shared[1]} if shared else None
    return cfg


def gru(width=40, mlp="moe"):
    return {"type": "mingru", "mixer": {"width": width},
            "mlp": moe_cfg() if mlp == "moe" else mlp}


def par(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.3, inner=40, state=6, dt_rank=3, conv=3,
        left_scale=1.1, right_scale=0.7, mlp="moe"):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                               "scale": scale},
                      "right": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv},
                      "left_scale": left_scale, "right_scale": right_scale},
            "mlp": moe_cfg() if mlp == "moe" else mlp}


def make_config(layers, width=48, vocab=128, eps=1e-5, mult=0.6, softcap=12.0):
    return {"architecture": "Muvetar", "layers": layers, "norm": {"eps": eps},
            "residual_mult": mult, "logit_softcap": softcap, "vocab": vocab, "width": width}


def make_tensors(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(shape, generator=g) * std + mean).to(torch.bfloat16)

    def lin(out, inn, gain=1.0):
        return rnd(out, inn, std=gain / math.sqrt(inn))

    W, V = cfg["width"], cfg["vocab"]
    t = {"embed": rnd(V, W), "head": lin(V, W, 2.0), "final.norm": rnd(W, std=0.1, mean=0.9)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        t[p + "norm1"] = rnd(W, std=0.1, mean=1.1)
        coef = torch.randn(i + 2, generator=g) * 0.25
        coef[-1] += 0.8
        t[p + "dwa"] = coef.to(torch.bfloat16)
        if layer["type"] == "mingru":
            w = m["width"]
            t[p + "mix.z"], t[p + "mix.z.b"] = lin(w, W, 2.0), rnd(w, std=1.0)
            t[p + "mix.x"], t[p + "mix.x.b"] = lin(w, W, 2.0), rnd(w, std=0.5)
            t[p + "mix.g"], t[p + "mix.o"] = lin(w, W, 2.0), lin(W, w, 2.0)
        else:
            a, r = m["left"], m["right"]
            H, G, D, DV = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            t[p + "mix.left.q"], t[p + "mix.left.k"] = lin(H * D, W, 1.5), lin(G * D, W, 1.5)
            t[p + "mix.left.v"], t[p + "mix.left.o"] = lin(G * DV, W), lin(W, H * DV, 2.0)
            t[p + "mix.left.r1"] = (torch.rand(H, generator=g) * 1.5 + 0.1).to(torch.bfloat16)
            t[p + "mix.left.r2"] = (torch.rand(H, generator=g) * 2.0 + 0.05).to(torch.bfloat16)
            I, N, R, K = r["inner"], r["state"], r["dt_rank"], r["conv"]
            t[p + "mix.right.in"] = lin(2 * I, W, 1.0)
            t[p + "mix.right.conv"] = rnd(I, K, std=0.9 / math.sqrt(K))
            t[p + "mix.right.conv.b"] = rnd(I, std=0.3)
            t[p + "mix.right.x"] = lin(R + 2 * N, I, 1.0)
            t[p + "mix.right.dt"] = lin(I, R, 1.0)
            t[p + "mix.right.dt.b"] = rnd(I, std=0.7, mean=-1.5)
            t[p + "mix.right.A_log"] = rnd(I, N, std=0.5, mean=-0.5)
            t[p + "mix.right.D"] = rnd(I, std=0.3, mean=0.8)
            t[p + "mix.right.o"] = lin(W, I, 2.0)
        mlp = layer["mlp"]
        if mlp is not None:
            t[p + "norm2"] = rnd(W, std=0.1, mean=1.0)
            ff = mlp["expert"]["ff"]
            t[p + "mlp.router"] = lin(mlp["router"]["experts"], W, 1.0)
            for e in range(mlp["router"]["experts"]):
                q = f"{p}mlp.e{e}."
                t[q + "gate"], t[q + "up"], t[q + "down"] = lin(ff, W, 2.0), lin(ff, W, 2.0), lin(W, ff)
            if mlp.get("shared"):
                sf, q = mlp["shared"]["ff"], p + "mlp.shared."
                t[q + "gate"], t[q + "up"], t[q + "down"] = lin(sf, W, 2.0), lin(sf, W, 2.0), lin(W, sf)
    return t


def write_checkpoint(path, cfg, tensors):
    from safetensors.torch import save_file

    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(path / "model.safetensors"))
    return str(path)


def mixed_layers(route):
    """Every switch at once: a recurrence first, parallel layers with grouped
    and ungrouped heads, a layer without feed-forward, a mixture without a
    shared expert, a recurrence narrower and one wider than the model."""
    moe = (lambda **kw: moe_cfg(experts=5, top=2, **kw)) if route else \
        (lambda **kw: moe_cfg(experts=3, top=3, **kw))
    return [
        gru(width=40, mlp=moe()),
        par(heads=4, kv_heads=2, dim=8, vdim=12, inner=40, state=6, dt_rank=3, conv=3, mlp=moe()),
        gru(width=56, mlp=None),
        par(heads=3, kv_heads=3, dim=16, vdim=8, scale=0.2, inner=24, state=20, dt_rank=5, conv=4,
            left_scale=0.9, right_scale=1.2, mlp=moe(shared=None)),
        par(heads=2, kv_heads=1, dim=12, vdim=12, inner=72, state=3, dt_rank=2, conv=2,
            mlp=moe(ff=10, limit=0.7)),
    ]


def tokens_for(n, vocab, seed):
    g = torch.Generator().manual_seed(3000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


DEVICES = [
    pytest.param(("cpu", "float32"), id="cpu"),
    pytest.param(("cuda", "float32"), id="hip-fp32", marks=pytest.mark.gpu),
    pytest.param(("cuda", "bfloat16"), id="hip-bf16", marks=pytest.mark.gpu),
]


def make_engine(path, target, blocks=64, block_size=16, max_seqs=4, prefill_budget=4096,
                max_len=1024):
    device, dtype = target
    return LLMEngine(EngineConfig(
        model=path, device=device, dtype=dtype, max_num_seqs=max_seqs, max_model_len=max_len,
        num_kv_blocks=blocks, kv_block_size=block_size, max_prefill_tokens=prefill_budget))


def tolerance(target):
    """(worst row, mean over rows) of the relative rms error. fp32 is the
    sharp comparison; bf16 rounds every GEMM input and output of a deep
    stack and only has to stay at rounding level."""
    return (8e-2, 2.5e-2) if target[1] == "bfloat16" else (2e-4, 5e-5)


def assert_close(got, want, target, what=""):
    got, want = got.double().cpu(), want.double()
    err = (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt()
    worst, mean = float(err.max()), float(err.mean())
    lim_worst, lim_mean = tolerance(target)
    assert worst < lim_worst, f"{what}: worst row error {worst:.3e} at row {int(err.argmax())}"
    assert mean < lim_mean, f"{what}: mean row error {mean:.3e}"


def replay(engine, rid, toks, cuts, end=True):
    """One request alone, cut into the given portion sizes; all logits."""
    out, at = [], 0
    for n in cuts:
        last = at + n == len(toks)
        out.append(engine.replay_step(
            [{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}],
            end=[rid] if (last and end) else []))
        at += n
    assert at == len(toks)
    return torch.cat(out)


_MODELS = {}


@pytest.fixture(scope="module")
def mixed_model(tmp_path_factory):
    """(config, tensors, path, oracle cache) of the all-switches model;
    `route` picks the variant with a real expert choice (fp32) or with every
    expert chosen (bf16)."""
    def get(target):
        route = target[1] != "bfloat16"
        if route not in _MODELS:
            cfg = make_config(mixed_layers(route))
            tensors = make_tensors(cfg, seed=11)
            path = write_checkpoint(tmp_path_factory.mktemp("mv") / "m", cfg, tensors)
            _MODELS[route] = (cfg, tensors, path)
        return _MODELS[route]
    return get


_WANT = {}


def oracle_logits(cfg, tensors, toks):
    key = (id(tensors), tuple(toks))
    if key not in _WANT:
        _WANT[key] = oracle.forward(cfg, tensors, toks)
    return _WANT[key]


def dev_dtype(target):
    return target[0], (torch.bfloat16 if target[1] == "bfloat16" else torch.float32)


# ------------------------------------------------------ config and order --

def test_config_reader_takes_everything_from_config(tmp_path):
    from llmq_amd.engine.model_specs import resolve_spec

    cfg = make_config(mixed_layers(True))
    tensors = make_tensors(cfg)
    path = write_checkpoint(tmp_path / "m", cfg, tensors)
    spec = resolve_spec(path)
    assert spec.family == "muvetar" and spec.num_layers == 5 and spec.hidden_size == 48
    assert [ls.mixer.kind for ls in spec.layers] == [
        "mingru", "parallel", "mingru", "parallel", "parallel"]
    assert (spec.residual_mult, spec.logit_softcap, spec.rms_eps) == (0.6, 12.0, 1e-5)
    assert spec.layers[0].mixer.width == 40 and spec.layers[2].mixer.width == 56
    a, r = spec.layers[3].mixer.left, spec.layers[3].mixer.right
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale) == (3, 3, 16, 8, 0.2)
    assert (r.inner, r.state, r.dt_rank, r.conv) == (24, 20, 5, 4)
    assert (spec.layers[3].mixer.left_scale, spec.layers[3].mixer.right_scale) == (0.9, 1.2)
    e = spec.layers[1].moe
    assert (e.experts, e.top, e.ff, e.limit, e.scale, e.shared_ff, e.shared_limit) == \
        (5, 2, 24, 1.5, 1.3, 20, 0.8)
    assert spec.layers[2].moe is None and spec.layers[3].moe.shared_ff == 0
    assert spec.layers[4].moe.ff == 10 and spec.layers[4].moe.limit == 0.7
    assert spec.param_count() == sum(v.numel() for v in tensors.values())
    # attention layers own key/value pages, every layer a state entry
    eng = make_engine(path, ("cpu", "float32"))
    assert [k is not None for k in eng.kv_cache.k] == [False, True, False, True, True]
    assert eng.kv_cache.k[1].shape[1:] == (2, 16, 8) and eng.kv_cache.v[1].shape[1:] == (2, 16, 12)
    assert eng.state_cache.state[0].shape[1:] == (40,)
    scan, tail = eng.state_cache.state[3]
    assert scan.shape[1:] == (24, 20) and tail.shape[1:] == (3, 24)
    with pytest.raises(ValueError):
        bad = make_config([dict(gru(), type="lstm")])
        resolve_spec(write_checkpoint(tmp_path / "bad", bad, {}))


# ------------------------------------------------------ mechanisms alone --

@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("layers,kw", [
    ([gru(width=48, mlp=None)], {}),
    ([gru(width=24, mlp=None)], {"mult": 1.0, "softcap": 0.0}),
    ([par(mlp=None)], {}),
    ([par(left_scale=1.0, right_scale=0.0, mlp=None)], {}),          # attention alone
    ([par(left_scale=0.0, right_scale=1.0, mlp=None)], {}),          # scan alone
    ([par(heads=1, kv_heads=1, dim=32, vdim=32, conv=1, dt_rank=1, state=1, mlp=None)], {}),
    ([par(heads=6, kv_heads=1, dim=4, vdim=20, inner=136, state=40, conv=8, mlp=None)], {}),
    ([gru(mlp=moe_cfg(experts=4, top=4))], {}),
    ([gru(mlp=moe_cfg(experts=3, top=3, shared=None, scale=1.0))], {}),
    ([gru(mlp=moe_cfg(experts=1, top=1, limit=0.3))], {}),
    ([gru(mlp=None), gru(mlp=None), gru(mlp=None)], {}),             # the depth average alone
], ids=["gru", "gru-narrow-plain", "parallel", "attention", "scan", "ones", "wide", "moe-all",
        "moe-no-shared", "moe-single", "depth-average"])
def test_mechanism_alone(tmp_path, target, layers, kw):
    cfg = make_config(layers, **kw)
    tensors = make_tensors(cfg, seed=3)
    path = write_checkpoint(tmp_path / "m", cfg, tensors)
    toks = tokens_for(37, cfg["vocab"], 1)
    eng = make_engine(path, target)
    eng.model.taps = []
    got = replay(eng, "a", toks, [37])
    taps = []
    want = oracle.forward(cfg, tensors, toks, taps)
    for i, (g, w) in enumerate(zip(eng.model.taps, taps)):
        assert_close(g, w, target, f"stream after layer {i}")
    assert_close(got, want, target, "logits")


@pytest.mark.parametrize("target", DEVICES)
def test_sizes_that_fit_no_vector_width(tmp_path, target):
    layers = [par(heads=3, kv_heads=1, dim=5, vdim=7, inner=13, state=5, dt_rank=3, conv=3,
                  mlp=moe_cfg(experts=3, top=3, ff=9, shared=(7, 1.1))),
              gru(width=11, mlp=moe_cfg(experts=3, top=3, ff=5, shared=None))]
    cfg = make_config(layers, width=27, vocab=61)
    tensors = make_tensors(cfg, seed=5)
    path = write_checkpoint(tmp_path / "m", cfg, tensors)
    toks = tokens_for(41, 61, 2)
    want = oracle.forward(cfg, tensors, toks)
    eng = make_engine(path, target)
    assert_close(replay(eng, "a", toks, [41]), want, target, "whole")
    assert_close(replay(eng, "b", toks, [7, 1, 1, 30, 2]), want, target, "portions")


@pytest.mark.parametrize("target", DEVICES[:2])
@pytest.mark.parametrize("experts,top", [(5, 1), (5, 2), (7, 3), (2, 1), (13, 4)])
def test_expert_choice_in_the_model(tmp_path, target, experts, top):
    cfg = make_config([gru(mlp=moe_cfg(experts=experts, top=top)),
                       par(mlp=moe_cfg(experts=experts, top=top, shared=None))])
    tensors = make_tensors(cfg, seed=experts * 10 + top)
    path = write_checkpoint(tmp_path / "m", cfg, tensors)
    toks = tokens_for(33, cfg["vocab"], 6)
    assert_close(replay(make_engine(path, target), "a", toks, [30, 1, 1, 1]),
                 oracle.forward(cfg, tensors, toks), target, f"{experts} experts, top {top}")


# ------------------------------------------- schedules: cuts, batches, reuse --

@pytest.mark.parametrize("target", DEVICES)
def test_prefill_equals_token_by_token(mixed_model, target):
    cfg, tensors, path = mixed_model(target)
    toks = tokens_for(90, cfg["vocab"], 2)
    want = oracle_logits(cfg, tensors, toks)
    eng = make_engine(path, target)
    assert_close(replay(eng, "w", toks, [90]), want, target, "whole prompt")
    assert_close(replay(eng, "d", toks, [1] * 90), want, target, "token by token")
    assert eng.allocator.num_free == eng.allocator.num_blocks
    assert eng.slot_allocator.num_free == 4


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("cuts", [
    [2, 2, 3, 13, 2, 40, 1, 1, 16, 10],
    [16, 16, 16, 16, 16, 10],                 # on page borders
    [15, 17, 1, 31, 2, 24],                   # just off them
    [3, 3, 3, 3, 3, 3, 3, 3, 66],             # the longest convolution's reach
    [89, 1],
    [1, 1, 1, 87],                            # the first tokens alone
    [2] * 45,
])
def test_portions(mixed_model, target, cuts):
    cfg, tensors, path = mixed_model(target)
    toks = tokens_for(90, cfg["vocab"], 3)
    want = oracle_logits(cfg, tensors, toks)
    eng = make_engine(path, target)
    assert_close(replay(eng, "c", toks, cuts), want, target, f"cuts {cuts}")


@pytest.mark.parametrize("target", DEVICES)
def test_mixed_batches_equal_alone_and_reuse(mixed_model, target):
    """Six unequal requests through four slots and a pool that cannot hold
    them all at once: portions beside single tokens, requests that pause,
    blocks and slots handed on to later requests."""
    cfg, tensors, path = mixed_model(target)
    lens = {"a": 70, "b": 9, "c": 41, "d": 130, "e": 25, "f": 3}
    toks = {r: tokens_for(n, cfg["vocab"], 10 + i) for i, (r, n) in enumerate(lens.items())}
    want = {r: oracle_logits(cfg, tensors, t) for r, t in toks.items()}
    eng = make_engine(path, target, blocks=14, block_size=16)
    at = {r: 0 for r in lens}
    got = {r: [] for r in lens}
    plan = [
        {"a": 33, "b": 2, "c": 17},
        {"a": 1, "b": 1, "c": 24, "d": 40},
        {"a": 1, "b": 6, "d": 2},              # c pauses at its end; b ends
        {"a": 35, "d": 1, "e": 25},            # e takes b's slot and blocks
        {"d": 1, "e": 0, "c": 0},
        {"d": 86, "f": 3},                     # a, c, e ended; f reuses
    ]
    ends = [[], [], ["b"], ["a", "e"], ["c"], ["d", "f"]]
    slots_seen = set()
    for step, end in zip(plan, ends):
        entries = []
        for r, n in step.items():
            if n:
                entries.append({"id": r, "tokens": toks[r][at[r]:at[r] + n], "want": list(range(n))})
        out = eng.replay_step(entries, end=[])
        for s in eng._seqs.values():
            slots_seen.add(s.state_slot)
        eng.replay_step([], end=end)
        k = 0
        for ent in entries:
            n = len(ent["tokens"])
            got[ent["id"]].append(out[k:k + n])
            at[ent["id"]] += n
            k += n
    assert at == lens
    assert slots_seen <= {0, 1, 2, 3}
    for r in lens:
        assert_close(torch.cat(got[r]), want[r], target, f"request {r}")
    assert eng.allocator.num_free == 14 and eng.slot_allocator.num_free == 4


@pytest.mark.parametrize("target", DEVICES)
def test_stale_pages_and_slots_do_not_leak(mixed_model, target):
    """A request that runs in blocks and a slot another one just left sees
    nothing of it: same logits as in a fresh engine."""
    cfg, tensors, path = mixed_model(target)
    first = tokens_for(64, cfg["vocab"], 30)
    second = tokens_for(50, cfg["vocab"], 31)
    want = oracle_logits(cfg, tensors, second)
    eng = make_engine(path, target, blocks=4, max_seqs=1)
    replay(eng, "x", first, [60, 1, 1, 1, 1])
    assert_close(replay(eng, "y", second, [3, 1, 1, 45]), want, target, "after reuse")


@pytest.mark.parametrize("target", DEVICES)
def test_long_decode_across_pages(mixed_model, target):
    cfg, tensors, path = mixed_model(target)
    toks = tokens_for(5 + 150, cfg["vocab"], 4)
    want = oracle_logits(cfg, tensors, toks)
    eng = make_engine(path, target)
    assert_close(replay(eng, "l", toks, [5] + [1] * 150), want, target, "long decode")


# ------------------------------------------ edges made visible by design --

def _needle_case(device, dtype, key_pos, query_pos, decode, r1, r2, H=2, G=1, D=16, DV=8,
                 block_size=16):
    """Every key scores 0 and has value 0, but the needle at key_pos: raw score
    8, value 1 in channel 1. The output's channel 1 is then the softmax weight
    the needle gets after the distance penalty; the caller compares it with
    the dense formula. Pages are handed out in reverse order."""
    n = query_pos + 1
    nblocks = (n + block_size - 1) // block_size
    kc = torch.zeros(nblocks + 2, G, block_size, D, dtype=dtype)
    vc = torch.zeros(nblocks + 2, G, block_size, DV, dtype=dtype)
    table = torch.arange(nblocks + 1, 0, -1, dtype=torch.int32).view(1, -1)   # reversed pages
    b, o = int(table[0, key_pos // block_size]), key_pos % block_size
    kc[b, :, o, 0] = 8.0
    vc[b, :, o, 1] = 1.0
    kc, vc, table = kc.to(device), vc.to(device), table.to(device)
    bias = torch.tensor([[r1, r2]] * H, dtype=torch.float32, device=device)
    if decode:
        q = torch.zeros(1, H, D, dtype=dtype, device=device)
        q[0, :, 0] = 1.0
        out = ops.window_attn_decode(
            q, kc, vc, DV, table, torch.tensor([n], dtype=torch.int32, device=device), 0, 1.0,
            log_bias=bias)
        return float(out[0, H - 1, 1])
    start = max(0, query_pos - 4)            # a portion whose last row is the query
    rows = query_pos - start + 1
    q = torch.zeros(rows, H, D, dtype=dtype, device=device)
    q[:, :, 0] = 1.0
    out = ops.window_attn_prefill(
        q, kc, vc, DV, table, torch.tensor([0, rows], dtype=torch.int32, device=device),
        torch.tensor([start], dtype=torch.int32, device=device), rows, 0, 1.0, log_bias=bias)
    return float(out[-1, H - 1, 1])


def _needle_weight(key_pos, query_pos, r1, r2):
    """Dense formula: softmax weight of the needle among query_pos + 1 keys."""
    s = torch.zeros(query_pos + 1, dtype=torch.float64)
    s[key_pos] = 8.0
    d = torch.arange(query_pos, -1, -1, dtype=torch.float64)
    return float(torch.softmax(s - r1 * torch.log1p(r2 * d), 0)[key_pos])


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("decode", [False, True], ids=["portion", "single"])
def test_far_keys_page_borders_and_the_distance_penalty(target, decode):
    """A lone strong key far back, on either side of page borders, at the
    sequence's first positions and right at the query: its weight follows
    the dense formula, for a weak and a strong distance penalty."""
    device, dtype = dev_dtype(target)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-4
    for r1, r2 in ((0.0, 1.0), (0.5, 0.25), (1.5, 3.0)):
        for key_pos, query_pos in ((0, 700), (1, 700), (15, 700), (16, 700), (17, 700),
                                   (350, 700), (699, 700), (700, 700), (0, 0), (0, 1),
                                   (63, 64), (64, 64), (3, 255), (3, 256)):
            got = _needle_case(device, dtype, key_pos, query_pos, decode, r1, r2)
            want = _needle_weight(key_pos, query_pos, r1, r2)
            assert abs(got - want) < tol * max(want, 0.05), (r1, r2, key_pos, query_pos, got, want)


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("D,DV", [(16, 8), (12, 20)])
def test_a_query_does_not_see_the_keys_after_it(target, D, DV):
    """A portion whose later rows carry a key that would swamp everything: the
    rows before it must not notice, the row at it and the rows after it must."""
    device, dtype = dev_dtype(target)
    H, bs, start, rows, hot = 2, 16, 90, 40, 111          # the portion spans two page borders
    n = start + rows
    nb = (n + bs - 1) // bs
    kc = torch.zeros(nb, 1, bs, D, dtype=dtype)
    vc = torch.zeros(nb, 1, bs, DV, dtype=dtype)
    kc[hot // bs, 0, hot % bs, 0] = 30.0
    vc[hot // bs, 0, hot % bs, 1] = 1.0
    q = torch.zeros(rows, H, D, dtype=dtype)
    q[:, :, 0] = 1.0
    table = torch.arange(nb, dtype=torch.int32).view(1, -1).to(device)
    out = ops.window_attn_prefill(
        q.to(device), kc.to(device), vc.to(device), DV, table,
        torch.tensor([0, rows], dtype=torch.int32, device=device),
        torch.tensor([start], dtype=torch.int32, device=device), rows, 0, 1.0,
        log_bias=torch.tensor([[0.3, 0.5]] * H, device=device)).float().cpu()
    seen = out[:, :, 1]
    assert float(seen[: hot - start].abs().max()) == 0.0
    assert float(seen[hot - start:].min()) > 0.99


@pytest.mark.parametrize("target", DEVICES)
def test_penalty_numbers_are_per_head(target):
    """Heads with different (r1, r2) over the same keys and grouped kv heads."""
    device, dtype = dev_dtype(target)
    H, G, D, DV, n, bs = 6, 2, 8, 8, 70, 16
    g = torch.Generator().manual_seed(5)
    k = torch.randn(n, G, D, generator=g)
    v = torch.randn(n, G, DV, generator=g)
    q = torch.randn(n, H, D, generator=g)
    r12 = torch.stack([torch.linspace(0.0, 2.0, H), torch.linspace(3.0, 0.1, H)], 1)
    nb = (n + bs - 1) // bs
    kc = torch.zeros(nb, G, bs, D)
    vc = torch.zeros(nb, G, bs, DV)
    for p in range(n):
        kc[p // bs, :, p % bs], vc[p // bs, :, p % bs] = k[p], v[p]
    table = torch.arange(nb, dtype=torch.int32).view(1, -1).to(device)
    cast = lambda x: x.to(dtype).to(device)
    got = ops.window_attn_prefill(
        cast(q), cast(kc), cast(vc), DV, table, torch.tensor([0, n], dtype=torch.int32, device=device),
        torch.tensor([0], dtype=torch.int32, device=device), n, 0, 0.4, log_bias=r12.to(device))
    qd, kd, vd = (x.to(dtype).double() for x in (q, k, v))
    want = torch.zeros(n, H, DV, dtype=torch.float64)
    for a in range(H):
        for i in range(n):
            d = torch.arange(i, -1, -1, dtype=torch.float64)
            s = (kd[: i + 1, a // (H // G)] @ qd[i, a]) * 0.4 \
                - float(r12[a, 0]) * torch.log1p(float(r12[a, 1]) * d)
            want[i, a] = torch.softmax(s, 0) @ vd[: i + 1, a // (H // G)]
    tol = 3e-2 if dtype == torch.bfloat16 else 1e-4
    assert (got.double().cpu() - want).abs().max() < tol


def _seq_meta(lens, slots, fresh, device):
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=device)
    return (cu, torch.tensor(slots, dtype=torch.int32, device=device),
            torch.tensor(fresh, dtype=torch.int32, device=device))


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("n", [1, 40, 300])
def test_mingru_op_keeps_a_far_input(target, n):
    """Gates near zero after the first token: the state written at token 0
    must still be there hundreds of tokens later, through portion cuts and a
    slot handed over from another sequence."""
    device, dtype = dev_dtype(target)
    C, T = n, 260
    z = torch.full((T, C), -12.0)
    z[0] = 9.0                                     # token 0 writes, the rest keep
    u = torch.zeros(T, C)
    u[0] = torch.linspace(-2.0, 2.0, C)
    g = torch.full((T, C), 1.5)
    zero = torch.zeros(C, device=device)
    zd, ud = z.to(dtype).double(), u.to(dtype).double()
    a = oracle.sigmoid(zd)
    cand = torch.where(ud >= 0, ud + 0.5, oracle.sigmoid(ud))
    silu_g = oracle.silu(g.to(dtype).double())
    S, want = torch.zeros(C, dtype=torch.float64), []
    for t in range(T):
        S = (1 - a[t]) * S + a[t] * cand[t]
        want.append(S * silu_g[t])
    want = torch.stack(want)
    assert float((want[259] - want[0]).abs().max()) < 0.05 * float(want[0].abs().max())
    state = torch.full((3, C), 77.0, device=device)    # stale values of an earlier owner
    outs, at = [], 0
    for cut in (1, 2, 97, 1, 1, 158):
        cu, slots, fresh = _seq_meta([cut], [1], [int(at == 0)], device)
        sl = slice(at, at + cut)
        outs.append(ops.mingru_scan(z[sl].to(dtype).to(device), u[sl].to(dtype).to(device),
                                    g[sl].to(dtype).to(device), zero, zero, state, cu, slots,
                                    fresh, dtype))
        at += cut
    got = torch.cat(outs).double().cpu()
    assert (got - want).abs().max() < (3e-2 if dtype == torch.bfloat16 else 2e-4)
    assert float(state[0].min()) == 77.0 and float(state[2].max()) == 77.0


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("lens", [[200, 1, 3, 130], [1, 1, 1], [17, 40], [700]])
def test_mingru_op_unequal_sequences_in_one_call(target, lens):
    """Long and very short sequences side by side (the long ones run split
    over time), strided inputs, a state carried in from an earlier call."""
    device, dtype = dev_dtype(target)
    C, T = 70, sum(lens)
    g = torch.Generator().manual_seed(T)
    p = (torch.randn(T, 3 * C + 5, generator=g) * 1.5).to(dtype)
    zb, ub = torch.randn(C, generator=g), torch.randn(C, generator=g) * 0.5
    start = torch.randn(len(lens) + 1, C, generator=g)
    fresh = [i % 2 for i in range(len(lens))]
    slots = list(range(len(lens), 0, -1))
    cu, sl, fr = _seq_meta(lens, slots, fresh, device)
    state = start.clone().to(device)
    pd = p.to(device)
    got = ops.mingru_scan(pd[:, 1:C + 1], pd[:, C + 2:2 * C + 2], pd[:, 2 * C + 3:3 * C + 3],
                          zb.to(device), ub.to(device), state, cu, sl, fr, dtype).double().cpu()
    pz, pu, pg = (p[:, a:a + C].double() for a in (1, C + 2, 2 * C + 3))
    at = 0
    tol = 3e-2 if dtype == torch.bfloat16 else 1e-4
    for b, n in enumerate(lens):
        S = torch.zeros(C, dtype=torch.float64) if fresh[b] else start[slots[b]].double()
        for t in range(at, at + n):
            a = oracle.sigmoid(pz[t] + zb.double())
            uu = pu[t] + ub.double()
            S = (1 - a) * S + a * torch.where(uu >= 0, uu + 0.5, oracle.sigmoid(uu))
            want = S * oracle.silu(pg[t])
            assert (got[t] - want).abs().max() < tol * max(1.0, float(want.abs().max())), (b, t)
        assert (state[slots[b]].double().cpu() - S).abs().max() < 1e-4
        at += n
    assert torch.equal(state[0].cpu(), start[0])


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("C,K", [(5, 4), (64, 3), (300, 8), (7, 2), (9, 1), (33, 16)])
def test_conv_op_across_cuts_shorter_than_its_reach(target, C, K):
    device, dtype = dev_dtype(target)
    g = torch.Generator().manual_seed(C * 10 + K)
    T = 45
    x = torch.randn(T, C, generator=g).to(dtype)
    w = torch.randn(C, K, generator=g)
    b = torch.randn(C, generator=g)
    want = oracle.silu(oracle.causal_conv(x.double(), w.double(), b.double()))
    tail = torch.full((3, max(K - 1, 0), C), 55.0, device=device)
    outs, at = [], 0
    for cut in (1, 1, 2, 1, 3, 20, 2, 15):
        cu, slots, fresh = _seq_meta([cut], [2], [int(at == 0)], device)
        outs.append(ops.causal_conv_silu(x[at:at + cut].to(device), w.to(device), b.to(device),
                                         tail, cu, slots, fresh))
        at += cut
    got = torch.cat(outs).double().cpu()
    assert ((got - want).abs() / want.abs().clamp(min=1.0)).max() < \
        (2e-2 if dtype == torch.bfloat16 else 1e-5)
    # several sequences in one call, a padded strided input, unequal lengths
    wide = torch.randn(T, C + 3, generator=g).to(dtype).to(device)
    xs = wide[:, 1:C + 1]
    lens = [3, 1, 30, 11]
    cu, slots, fresh = _seq_meta(lens, [0, 2, 1, 3], [1, 1, 1, 1], device)
    tail4 = torch.zeros(5, max(K - 1, 0), C, device=device)
    got = ops.causal_conv_silu(xs, w.to(device), b.to(device), tail4, cu, slots, fresh).double().cpu()
    at = 0
    for n in lens:
        ref = oracle.silu(oracle.causal_conv(xs[at:at + n].double().cpu(), w.double(), b.double()))
        assert ((got[at:at + n] - ref).abs() / ref.abs().clamp(min=1.0)).max() < \
            (2e-2 if dtype == torch.bfloat16 else 1e-5)
        at += n
    if K > 1:
        assert torch.equal(tail4[2, -1].cpu(), xs[3].float().cpu())      # the one-token sequence
        assert float(tail4[2, 0].abs().max()) == 0.0 or K == 2


def _scan_reference(x, dt, dt_b, A, Bm, Cm, D, z):
    """Token-by-token selective scan in float64 (one sequence)."""
    step = oracle.softplus(dt + dt_b)
    S = torch.zeros(A.shape, dtype=torch.float64)
    ys = []
    for r in range(x.shape[0]):
        S = torch.exp(step[r].unsqueeze(1) * A) * S + (step[r] * x[r]).unsqueeze(1) * Bm[r]
        ys.append(S @ Cm[r] + D * x[r])
    return torch.stack(ys) * oracle.silu(z), S


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("C,N", [(40, 6), (24, 20), (72, 3), (13, 5), (300, 16), (8, 1), (16, 40)])
def test_selective_scan_op_against_token_by_token(target, C, N):
    device, dtype = dev_dtype(target)
    g = torch.Generator().manual_seed(C + N)
    T = 380
    rn = lambda *s: torch.randn(*s, generator=g)
    x, dt, z = rn(T, C).to(dtype), (rn(T, C) - 1.0).to(dtype), rn(T, C).to(dtype)
    bc = rn(T, 2 * N + 3).to(dtype)
    dt_b, A, D = rn(C) * 0.5, -torch.exp(rn(C, N) * 0.7 - 0.5), rn(C)
    Bm, Cm = bc[:, 1:N + 1], bc[:, N + 1:2 * N + 1]
    want, S_end = _scan_reference(x.double(), dt.double(), dt_b.double(), A.double(), Bm.double(),
                                  Cm.double(), D.double(), z.double())
    state = torch.full((4, C, N), 9.0, device=device)
    dev = lambda t: t.to(device)
    outs, at = [], 0
    for cut in (1, 2, 30, 1, 1, 40, 205, 100):      # the long ones run split over time
        cu, slots, fresh = _seq_meta([cut], [3], [int(at == 0)], device)
        sl = slice(at, at + cut)
        outs.append(ops.selective_scan(dev(x[sl]), dev(dt[sl]), dev(dt_b), dev(A), dev(bc)[sl, 1:N + 1],
                                       dev(bc)[sl, N + 1:2 * N + 1], dev(D), dev(z[sl]), state, cu,
                                       slots, fresh))
        at += cut
    got = torch.cat(outs).double().cpu()
    scale = want.abs().max()
    tol = 2e-2 if dtype == torch.bfloat16 else 2e-5
    assert (got - want).abs().max() < tol * scale
    assert (state[3].double().cpu() - S_end).abs().max() < tol * S_end.abs().max().clamp(min=1.0)
    assert float(state[0].min()) == 9.0 and float(state[2].max()) == 9.0
    # three sequences in one call equal each alone, short and long ones mixed
    for lens in ([20, 1, 54], [300, 2, 78], [5, 370, 5]):
        cu, slots, fresh = _seq_meta(lens, [2, 0, 1], [1, 1, 1], device)
        st = torch.zeros(4, C, N, device=device)
        n_all = sum(lens)
        got = ops.selective_scan(dev(x)[:n_all], dev(dt)[:n_all], dev(dt_b), dev(A),
                                 dev(bc)[:n_all, 1:N + 1], dev(bc)[:n_all, N + 1:2 * N + 1], dev(D),
                                 dev(z)[:n_all], st, cu, slots, fresh).double().cpu()
        at = 0
        for n in lens:
            sl = slice(at, at + n)
            ref, _ = _scan_reference(x[sl].double(), dt[sl].double(), dt_b.double(), A.double(),
                                     Bm[sl].double(), Cm[sl].double(), D.double(), z[sl].double())
            assert (got[sl] - ref).abs().max() < tol * scale, lens
            at += n


@pytest.mark.parametrize("target", DEVICES)
def test_selective_scan_keeps_a_far_input(target):
    """Slow decay and an input only at token 0: what reaches token 400 is
    exp(sum of steps * A) of it, through cuts and single tokens."""
    device, dtype = dev_dtype(target)
    C, N, T = 12, 4, 401
    x = torch.zeros(T, C)
    x[0] = 1.0
    dt = torch.full((T, C), -3.0)
    A = -torch.full((C, N), 0.01) * torch.arange(1, N + 1)
    Bm = torch.ones(T, N)
    Cm = torch.ones(T, N)
    z = torch.full((T, C), 2.0)
    zero = torch.zeros(C)
    want, _ = _scan_reference(x.double(), dt.double(), zero.double(), A.double(), Bm.double(),
                              Cm.double(), zero.double(), z.double())
    state = torch.zeros(2, C, N, device=device)
    dev = lambda t: t.to(dtype).to(device)
    outs, at = [], 0
    for cut in [1, 1, 2, 196] + [1] * 100 + [101]:
        cu, slots, fresh = _seq_meta([cut], [0], [int(at == 0)], device)
        sl = slice(at, at + cut)
        outs.append(ops.selective_scan(dev(x[sl]), dev(dt[sl]), zero.to(device), A.to(device),
                                       dev(Bm[sl]), dev(Cm[sl]), zero.to(device), dev(z[sl]), state,
                                       cu, slots, fresh))
        at += cut
    got = torch.cat(outs).double().cpu()
    assert float(want[400].min()) > 1e-3
    assert ((got - want).abs() / want.abs().clamp(min=1e-3)).max() < \
        (3e-2 if dtype == torch.bfloat16 else 1e-4)


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("W,F,E,top,T", [(48, 24, 5, 2, 9), (40, 20, 10, 4, 3), (36, 10, 3, 3, 130),
                                         (64, 32, 8, 1, 24), (27, 9, 70, 5, 6)])
def test_router_and_expert_mixture_ops(target, W, F, E, top, T):
    device, dtype = dev_dtype(target)
    g = torch.Generator().manual_seed(W + E)
    h = torch.randn(T, W, generator=g).to(dtype)
    router = torch.randn(E, W, generator=g) * 0.4
    gate_up = (torch.randn(E, 2 * F, W, generator=g) * 0.3).to(dtype)
    down = (torch.randn(E, W, F, generator=g) * 0.3).to(dtype)
    logits = h.float() @ router.T
    idx, w = ops.softmax_topk(logits.to(device), top, 1.7)
    s = torch.softmax(logits.double(), -1)
    w_ref, i_ref = torch.sort(s, dim=-1, descending=True, stable=True)
    assert torch.equal(idx.cpu().long(), i_ref[:, :top])
    assert (w.double().cpu() - 1.7 * w_ref[:, :top]).abs().max() < 1e-5
    tensors = {"router": router.double()}
    for e in range(E):
        tensors[f"e{e}.gate"], tensors[f"e{e}.up"] = gate_up[e, :F].double(), gate_up[e, F:].double()
        tensors[f"e{e}.down"] = down[e].double()
    want = torch.zeros(T, W, dtype=torch.float64)
    for r in range(T):
        for j in range(top):
            want[r] += float(w[r, j]) * oracle.expert(tensors, f"e{int(idx[r, j])}.",
                                                      h[r:r + 1].double(), 0.9)[0]
    tol = 4e-2 if dtype == torch.bfloat16 else 1e-4
    for sync_free in (False, True):
        got = ops.moe_experts(h.to(device), idx, w, gate_up.to(device), down.to(device),
                              sync_free=sync_free, act="clamp_swish", limit=0.9,
                              weight_output=True)
        assert (got.double().cpu() - want).abs().max() < tol * want.abs().max(), sync_free
    x2 = torch.randn(T, 2 * F, generator=g).to(dtype) * 2
    got = ops.clamp_swish_mul(x2.to(device), 0.9).double().cpu()
    gd, ud = x2[:, :F].double().clamp(max=0.9), x2[:, F:].double().clamp(-0.9, 0.9)
    assert (got - gd * oracle.sigmoid(1.702 * gd) * (ud + 1)).abs().max() < \
        (2e-2 if dtype == torch.bfloat16 else 1e-6)


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("W", [48, 27, 2048, 2056])
def test_embedding_joins_and_depth_average_ops(target, W):
    device, dtype = dev_dtype(target)
    g = torch.Generator().manual_seed(W)
    T, V, n = 5, 30, 4
    emb = torch.randn(V, W, generator=g).to(dtype)
    ids = torch.tensor([3, 0, 29, 7, 7])
    pos = torch.tensor([0, 1, 900, 77, 4000])
    from llmq_amd.ops.torch_ref import sinusoid_inv_freq
    got = ops.embed_sinusoid(emb.to(device), ids.to(device), pos.to(device),
                             sinusoid_inv_freq(W).to(device)).double().cpu()
    for r in range(T):
        want = emb[ids[r]].double() + oracle.position_vector(1, W, int(pos[r]))[0]
        assert (got[r] - want).abs().max() < 5e-4, r       # fp32 angle at position 4000
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    res = torch.randn(T, W, generator=g)
    y, y2, w = (torch.randn(T, W, generator=g).to(dtype) for _ in range(3))
    w = w[0]
    for second in (None, y2):
        r = res.clone().to(device)
        h = ops.scaled_add_norm(r, y.to(device), None if second is None else second.to(device),
                                0.7, -0.4, w.to(device), 1e-5, dtype)
        want = res.double() + 0.7 * y.double() + (0 if second is None else -0.4 * second.double())
        assert (r.double().cpu() - want).abs().max() < 1e-5
        assert (h.double().cpu() - oracle.rms_norm(want, w.double(), 1e-5)).abs().max() < tol * 4
    stack = torch.randn(n + 2, T, W, generator=g)
    coef = torch.randn(n, generator=g)
    for second in (None, y2):
        st = stack.clone().to(device)
        h = ops.depth_mix_norm(st, n, coef.to(device), y.to(device),
                               None if second is None else second.to(device), 0.3, 0.9,
                               w.to(device), 1e-5, dtype)
        last = stack[n - 1].double() + 0.3 * y.double() + (0 if second is None else 0.9 * second.double())
        mix = oracle.depth_average([stack[j].double() for j in range(n - 1)] + [last], coef.double())
        assert (st[n - 1].double().cpu() - last).abs().max() < 1e-5
        assert (st[n].double().cpu() - mix).abs().max() < 1e-5
        assert torch.equal(st[:n - 1].cpu(), stack[:n - 1]) and torch.equal(st[n + 1].cpu(), stack[n + 1])
        assert (h.double().cpu() - oracle.rms_norm(mix, w.double(), 1e-5)).abs().max() < tol * 4


# ------------------------------------------- generation through the engine --

@pytest.mark.parametrize("target", DEVICES[:2])
def test_greedy_generation_through_the_scheduler(mixed_model, target):
    """add_request / step: the scheduler's own admission, chunked prefill
    (a budget smaller than the prompts), decode batching and sampler."""
    cfg, tensors, path = mixed_model(target)
    prompts = {"p": tokens_for(21, cfg["vocab"], 40), "q": tokens_for(5, cfg["vocab"], 41),
               "r": tokens_for(34, cfg["vocab"], 42)}
    eng = make_engine(path, target, prefill_budget=16)
    params = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
    for rid, toks in prompts.items():
        eng.add_request(rid, prompt_token_ids=toks, params=params)
    got = {rid: [] for rid in prompts}
    while eng.has_unfinished():
        for out in eng.step():
            got[out.request_id].extend(out.new_token_ids)
    for rid, toks in prompts.items():
        assert got[rid] == oracle.greedy(cfg, tensors, toks, 6), rid
    assert eng.allocator.num_free == eng.allocator.num_blocks


def test_preset_runs_through_generate():
    eng = LLMEngine(EngineConfig(model="tiny-muvetar", device="cpu", max_num_seqs=2,
                                 max_model_len=64, num_kv_blocks=8))
    out = eng.generate_batch(["ab", "c"], SamplingParams(temperature=0.0, max_tokens=4,
                                                         ignore_eos=True))
    assert len(out) == 2


@pytest.mark.gpu
def test_decode_graph_replays_equal_eager(mixed_model):
    """Captured decode steps replayed several times, with eager work between
    the replays, against the same steps run eagerly."""
    target = ("cuda", "float32")
    cfg, tensors, path = mixed_model(target)
    # eight sequences: enough (token, expert) rows that the captured steps run
    # the expert mixture in its dense batched form
    toks = {r: tokens_for(n, cfg["vocab"], 50 + i) for i, (r, n) in enumerate(
        {"a": 30, "b": 12, "c": 19, "d": 9, "e": 25, "f": 14, "g": 11, "h": 21}.items())}
    results = []
    for eager in (True, False):
        device, dtype = target
        eng = LLMEngine(EngineConfig(model=path, device=device, dtype=dtype, max_num_seqs=8,
                                     max_model_len=256, num_kv_blocks=32, enforce_eager=eager))
        assert eng.runner.use_graphs == (not eager)
        rows = []
        eng.replay_step([{"id": r, "tokens": t[:-8], "want": []} for r, t in toks.items()])
        for k in range(8, 0, -1):
            rows.append(eng.replay_step(
                [{"id": r, "tokens": [t[len(t) - k]], "want": [0]} for r, t in toks.items()]))
            torch.cuda.synchronize()
        results.append(torch.cat(rows))
    assert (results[0] - results[1]).abs().max() < 2e-4
    want = torch.cat([torch.stack([oracle_logits(cfg, tensors, t)[len(t) - k] for t in toks.values()])
                      for k in range(8, 0, -1)])
    assert_close(results[1], want, target, "graph replays")


def test_trace_runner_cli(tmp_path, mixed_model):
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    cfg, tensors, path = mixed_model(("cpu", "float32"))
    toks = tokens_for(20, cfg["vocab"], 60)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": toks[:13], "want": [0, 12]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": toks[13:15], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": toks[15:], "want": [4]}], "end": ["a"]},
    ]
    out = tmp_path / "out"
    root = Path(__file__).resolve().parent.parent
    proc = subprocess.run(
        [sys.executable, str(root / "bin" / "trace_run"), "--model", path, "--dtype", "float32",
         "--out", str(out), "--max-tokens", "64"],
        input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
        timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [ln for ln in proc.stdout.splitlines() if ln.startswith("done")] == \
        ["done 0", "done 1", "done 2"]
    want = oracle_logits(cfg, tensors, toks)
    a = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1).copy())
    b = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1).copy())
    assert not (out / "1.f32").exists()
    assert_close(torch.cat([a, b]), want[[0, 12, 19]], ("cpu", "float32"), "trace runner")

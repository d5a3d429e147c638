"""Kosalorn (looped hybrid decoder) against the plain oracle in
kosalorn_oracle.py.

Every test builds its own small configuration and random checkpoint, loads
it through the engine's own entry points (config reader, weight loader,
scheduler, cache and state managers) and compares logits with the oracle.
The scenarios run on the CPU (torch reference ops) and, marked ``gpu``, on
the HIP kernels in fp32 (sharp) and bf16.

Expert routing is a discrete choice: a bf16 run rounds the router's input,
so a near-tie may fall the other way than in the float64 oracle. Whole-model
bf16 scenarios therefore use mixtures in which every expert is chosen (the
scores still weigh the inputs); the choice itself is checked in fp32 at
model level and in bf16 at op level, where the oracle sees the same inputs.
"""

from __future__ import annotations

import json
import math

import pytest
import torch

import kosalorn_oracle as oracle
from llmq_amd.engine.config import EngineConfig
from llmq_amd.engine.engine import LLMEngine
from llmq_amd.engine.sampling_params import SamplingParams


# --------------------------------------------------------------- fixtures --

def latent(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, q_rank=16, window=11,
           base=1000.0, scale=0.3, mlp="dense"):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
                      "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
                      "rot": {"base": base, "dims": rot_dim}, "mask": {"size": window}},
            "mlp": mlp_cfg(mlp)}


def latent2(heads=2, dim=16, rot_dim=8, vdim=24, kv_rank=24, base=50000.0, scale=0.2,
            mlp="dense"):
    return {"type": "latent_attention_2",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
                      "kv_rank": kv_rank, "scale": scale, "rot": {"base": base, "dims": rot_dim}},
            "mlp": mlp_cfg(mlp)}


def hgrn2(heads=2, dim=8, vdim=24, mlp="dense"):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim},
            "mlp": mlp_cfg(mlp)}


def mlp_cfg(kind):
    if kind is None:
        return None
    if kind == "dense":
        return {"kind": "dense", "ff": 40}
    experts, top = kind                     # ("moe", ...) given as (experts, top)
    return {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": experts, "top": top}}


def make_config(layers, width=48, vocab=128, eps=1e-5, side=6, loop=None):
    cfg = {"architecture": "Kosalorn", "layers": layers, "norm": {"eps": eps},
           "vocab": vocab, "width": width}
    if side:
        cfg["token_side"] = {"dim": side}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_tensors(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(shape, generator=g) * std + mean).to(torch.bfloat16)

    def lin(out, inn, gain=1.0):
        return rnd(out, inn, std=gain / math.sqrt(inn))

    W, V = cfg["width"], cfg["vocab"]
    side = cfg.get("token_side", {}).get("dim", 0)
    t = {"embed": rnd(V, W), "embed.norm": rnd(std=0.1, mean=1.3), "head": lin(V, W),
         "final.norm": rnd(std=0.1, mean=0.8)}
    if side:
        t["side.embed"] = rnd(V, side * len(cfg["layers"]))
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        t[p + "norm1"] = rnd(std=0.1, mean=1.1)
        t[p + "rg1"], t[p + "rg1.b"] = lin(W, W), rnd(W, std=0.5)
        if layer["type"] == "hgrn2":
            nk, nv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            t[p + "mix.q"], t[p + "mix.f"], t[p + "mix.v"] = lin(nk, W), lin(nk, W, 2.0), lin(nv, W)
            t[p + "mix.f.b"] = rnd(nk, mean=1.0)
            t[p + "mix.lower"] = (torch.rand(nk, generator=g) * 0.9).to(torch.bfloat16)
            t[p + "mix.norm"] = rnd(m["vdim"], std=0.2, mean=1.0)
            t[p + "mix.o"] = lin(W, nv)
        else:
            nq = m["heads"] * (m["dim"] + m["rot_dim"])
            R = m["kv_rank"]
            if layer["type"] == "latent_attention":
                t[p + "mix.dq"] = lin(m["q_rank"], W)
                t[p + "mix.dq.norm"] = rnd(m["q_rank"], std=0.2, mean=1.0)
                t[p + "mix.uq"] = lin(nq, m["q_rank"], 2.0)
            else:
                t[p + "mix.q"] = lin(nq, W, 2.0)
            t[p + "mix.dkv"] = lin(R + m["rot_dim"], W, 2.0)
            t[p + "mix.dkv.norm"] = rnd(R, std=0.2, mean=1.0)
            t[p + "mix.uk"] = lin(m["heads"] * m["dim"], R, 2.0)
            t[p + "mix.uv"] = lin(m["heads"] * m["vdim"], R)
            t[p + "mix.o"] = lin(W, m["heads"] * m["vdim"])
        mlp = layer["mlp"]
        if mlp is not None:
            t[p + "rg2"], t[p + "rg2.b"] = lin(W, W), rnd(W, std=0.5)
            if mlp["kind"] == "dense":
                ff = mlp["ff"]
                t[p + "mlp.gate"], t[p + "mlp.up"], t[p + "mlp.down"] = lin(ff, W), lin(ff, W), lin(W, ff)
            else:
                ff = mlp["expert"]["ff"]
                t[p + "mlp.router"] = lin(mlp["router"]["experts"], W, 3.0)
                for e in range(mlp["router"]["experts"]):
                    q = f"{p}mlp.e{e}."
                    t[q + "gate"], t[q + "up"], t[q + "down"] = lin(ff, W, 2.0), lin(ff, W, 2.0), lin(W, ff)
        if side:
            t[p + "side.gate"], t[p + "side.proj"] = lin(side, W), lin(W, side)
            t[p + "side.norm"] = rnd(W, std=0.2, mean=0.5)
    return t


def write_checkpoint(path, cfg, tensors):
    from safetensors.torch import save_file

    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(path / "model.safetensors"))
    return str(path)


def mixed_layers(route):
    """Every switch at once: a recurrent layer first and outside the loop, a
    loop that starts after it and runs three times over a windowed and a
    causal attention layer, a layer without feed-forward, mixtures beside
    dense feed-forwards, a recurrent layer inside no loop at the end."""
    moe = (5, 2) if route else (3, 3)
    return [
        hgrn2(heads=2, dim=8, vdim=24, mlp="dense"),
        latent(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, q_rank=16, window=11, mlp=moe),
        latent2(heads=2, dim=16, rot_dim=8, vdim=24, kv_rank=24, mlp=None),
        latent(heads=1, dim=12, rot_dim=6, vdim=8, kv_rank=10, q_rank=28, window=37, mlp="dense"),
        hgrn2(heads=3, dim=12, vdim=8, mlp=moe),
    ]


MIXED_LOOP = (1, 3, 3)


def tokens_for(n, vocab, seed):
    g = torch.Generator().manual_seed(2000 + seed)
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
    """(config, tensors, path) of the all-switches model; `route` picks the
    variant with a real expert choice (fp32) or with every expert chosen."""
    def get(target):
        route = target[1] != "bfloat16"
        if route not in _MODELS:
            cfg = make_config(mixed_layers(route), loop=MIXED_LOOP)
            tensors = make_tensors(cfg, seed=7)
            path = write_checkpoint(tmp_path_factory.mktemp("ks") / "m", cfg, tensors)
            _MODELS[route] = (cfg, tensors, path)
        return _MODELS[route]
    return get


# ------------------------------------------------------ config and order --

def test_config_reader_takes_everything_from_config(tmp_path):
    from llmq_amd.engine.model_specs import resolve_spec

    cfg = make_config(mixed_layers(True), loop=MIXED_LOOP)
    path = write_checkpoint(tmp_path / "m", cfg, make_tensors(cfg))
    spec = resolve_spec(path)
    assert spec.family == "kosalorn" and spec.num_layers == 5 and spec.hidden_size == 48
    assert [ls.mixer.kind for ls in spec.layers] == [
        "hgrn2", "latent_attention", "latent_attention", "latent_attention", "hgrn2"]
    a, b, c = spec.layers[1].mixer, spec.layers[2].mixer, spec.layers[3].mixer
    assert (a.q_rank, a.window, a.rot.layout, a.rot.base) == (16, 11, "half", 1000.0)
    assert (b.q_rank, b.window, b.rot.layout, b.rot.base) == (0, 0, "interleaved", 50000.0)
    assert (c.heads, c.dim, c.rot_dim, c.vdim, c.kv_rank, c.window) == (1, 12, 6, 8, 10, 37)
    assert spec.layers[1].moe.experts == 5 and spec.layers[1].moe.top == 2
    assert spec.layers[2].ff == 0 and spec.layers[2].moe is None and spec.layers[0].ff == 40
    assert spec.side_dim == 6 and spec.rms_eps == 1e-5
    assert [i for i, _ in spec.runs()] == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert [add for _, add in spec.runs()] == [False, False, False, True, False, True, False,
                                               False, False]
    assert [i for i, _ in spec.runs()] == [i for i, _ in oracle.layer_order(cfg)]
    for loop in ((0, 5, 2), (2, 2, 3), (4, 5, 1), (1, 4, 0)):
        c2 = make_config(mixed_layers(True), loop=loop)
        p2 = write_checkpoint(tmp_path / ("m%d%d%d" % loop), c2, make_tensors(c2))
        assert resolve_spec(p2).runs() == oracle.layer_order(c2), loop
    # every run owns a cache or a state entry
    eng = make_engine(path, ("cpu", "float32"))
    assert len(eng.kv_cache.k) == 9 and len(eng.state_cache.state) == 9
    assert eng.kv_cache.k[1].shape[1:] == (1, 16, 24) and eng.kv_cache.v[1] is None
    assert eng.kv_cache.k[0] is None and eng.state_cache.state[0].shape[1:] == (2, 8, 24)
    assert eng.kv_cache.k[3].data_ptr() != eng.kv_cache.k[1].data_ptr()
    assert eng.spec.param_count() == sum(
        v.numel() for v in make_tensors(cfg).values())


# ------------------------------------------------------ mechanisms alone --

@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("layers,side,loop", [
    pytest.param([latent(mlp=None)], 0, None, id="windowed-query-latent"),
    pytest.param([latent(heads=1, dim=4, rot_dim=2, vdim=4, kv_rank=4, q_rank=4, window=1,
                         mlp=None)], 0, None, id="window-of-one"),
    pytest.param([latent2(mlp=None)], 0, None, id="causal-direct-query"),
    pytest.param([latent2(heads=5, dim=6, rot_dim=10, vdim=7, kv_rank=9, mlp=None)], 0, None,
                 id="causal-odd-sizes"),
    pytest.param([hgrn2(mlp=None)], 0, None, id="hgrn2"),
    pytest.param([hgrn2(heads=1, dim=40, vdim=70, mlp=None)], 0, None, id="hgrn2-wide"),
    pytest.param([hgrn2(mlp="dense")], 0, None, id="dense-ff"),
    pytest.param([hgrn2(mlp=(4, 4))], 0, None, id="mixture-all-experts"),
    pytest.param([hgrn2(mlp=None)], 5, None, id="side-input"),
    pytest.param([latent2(mlp="dense"), hgrn2(mlp="dense")], 3, (0, 2, 2), id="loop-all"),
    pytest.param([hgrn2(mlp=None), latent(mlp=None), hgrn2(mlp=None)], 0, (1, 2, 4),
                 id="loop-one-layer"),
    pytest.param([], 0, None, id="no-layers"),
])
def test_mechanism_alone(tmp_path, target, layers, side, loop):
    cfg = make_config(layers, side=side, loop=loop)
    tensors = make_tensors(cfg, seed=len(layers) + side)
    path = write_checkpoint(tmp_path / "m", cfg, tensors)
    eng = make_engine(path, target)
    toks = tokens_for(47, cfg["vocab"], 1)
    eng.model.taps = []
    got = replay(eng, "a", toks, [47])
    want, want_runs = (oracle.forward(cfg, tensors, toks, return_layers=True)
                       if layers else (oracle.forward(cfg, tensors, toks), None))
    if layers and target[1] == "float32":
        assert len(eng.model.taps) == len(want_runs)
        for i, tap in enumerate(eng.model.taps):
            assert_close(tap, want_runs[i], target, f"residual after layer run {i}")
    assert_close(got, want, target, "logits")


@pytest.mark.parametrize("target", DEVICES)
def test_sizes_that_fit_no_vector_width(tmp_path, target):
    """Width, vocabulary, ranks and head sizes that are multiples of nothing:
    every kernel takes its scalar path, GEMM operands are unaligned."""
    layers = [
        latent(heads=3, dim=5, rot_dim=6, vdim=7, kv_rank=11, q_rank=9, window=13, mlp="dense"),
        hgrn2(heads=3, dim=7, vdim=9, mlp=(3, 3)),
        latent2(heads=9, dim=6, rot_dim=2, vdim=5, kv_rank=14, mlp=None),
    ]
    cfg = make_config(layers, width=50, vocab=101, side=5, loop=(0, 2, 2))
    tensors = make_tensors(cfg, seed=3)
    path = write_checkpoint(tmp_path / "m", cfg, tensors)
    toks = tokens_for(60, cfg["vocab"], 6)
    want = oracle.forward(cfg, tensors, toks)
    eng = make_engine(path, target)
    assert_close(replay(eng, "a", toks, [60]), want, target, "whole")
    assert_close(replay(eng, "b", toks, [7, 2, 30, 1, 1, 19]), want, target, "cut")


@pytest.mark.parametrize("target", DEVICES[:2])
@pytest.mark.parametrize("experts,top", [(5, 1), (5, 2), (7, 3), (2, 1)])
def test_expert_choice_in_the_model(tmp_path, target, experts, top):
    cfg = make_config([hgrn2(mlp=(experts, top)), latent2(mlp=(experts, top))], side=0)
    tensors = make_tensors(cfg, seed=experts * 10 + top)
    path = write_checkpoint(tmp_path / "m", cfg, tensors)
    toks = tokens_for(80, cfg["vocab"], 5)
    want = oracle.forward(cfg, tensors, toks)
    eng = make_engine(path, target)
    assert_close(replay(eng, "a", toks, [80]), want, target, "whole (sorted by expert)")
    assert_close(replay(eng, "b", toks, [70] + [1] * 10), want, target, "tail token by token")


# -------------------------------------------------- cuts, batches, reuse --

@pytest.mark.parametrize("target", DEVICES)
def test_prefill_equals_token_by_token(mixed_model, target):
    cfg, tensors, path = mixed_model(target)
    toks = tokens_for(90, cfg["vocab"], 2)
    want = oracle.forward(cfg, tensors, toks)
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
    [11, 11, 11, 11, 11, 11, 11, 11, 2],      # the short window's size
    [37, 37, 16],                             # the long window's size
    [89, 1],
    [1, 1, 1, 87],                            # the first tokens alone
])
def test_portions(mixed_model, target, cuts):
    cfg, tensors, path = mixed_model(target)
    toks = tokens_for(90, cfg["vocab"], 3)
    want = oracle.forward(cfg, tensors, toks)
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
    want = {r: oracle.forward(cfg, tensors, t) for r, t in toks.items()}
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
    want = oracle.forward(cfg, tensors, second)
    eng = make_engine(path, target, blocks=4, max_seqs=1)
    replay(eng, "x", first, [60, 1, 1, 1, 1])
    assert_close(replay(eng, "y", second, [3, 1, 1, 45]), want, target, "after reuse")


@pytest.mark.parametrize("target", DEVICES)
def test_long_decode_across_windows_and_pages(mixed_model, target):
    cfg, tensors, path = mixed_model(target)
    toks = tokens_for(5 + 150, cfg["vocab"], 4)
    want = oracle.forward(cfg, tensors, toks)
    eng = make_engine(path, target)
    assert_close(replay(eng, "l", toks, [5] + [1] * 150), want, target, "long decode")


# ------------------------------------------ edges made visible by design --

def _needle_case(device, dtype, window, key_pos, query_pos, decode, block_size=16, DV=8, D=16,
                 heads=2):
    """One latent cache, two heads (or more: many heads take another kernel); every key scores 0 but the needle, whose
    first channel is 40: the output is the needle's value prefix iff the
    query may see it. Values are the first DV channels of the key rows."""
    from llmq_amd import ops

    n = query_pos + 1
    nblocks = (n + block_size - 1) // block_size
    kc = torch.zeros(nblocks + 2, 1, block_size, D, dtype=dtype)
    table = torch.arange(nblocks + 1, 0, -1, dtype=torch.int32).view(1, -1)  # reversed pages
    for p in range(n):
        b, o = int(table[0, p // block_size]), p % block_size
        kc[b, 0, o, 1] = 1.0                  # channel 1 marks "any key"
    b, o = int(table[0, key_pos // block_size]), key_pos % block_size
    kc[b, 0, o, 0] = 40.0                      # the needle's score channel
    kc[b, 0, o, 1] = -3.0
    kc, table = kc.to(device), table.to(device)
    if decode:
        q = torch.zeros(1, heads, D, dtype=dtype, device=device)
        q[0, :, 0] = 1.0
        out = ops.window_attn_decode(
            q, kc, None, DV, table, torch.tensor([n], dtype=torch.int32, device=device),
            window, 1.0)
        assert out.shape == (1, heads, DV)
        assert torch.equal(out[0, 1], out[0, heads - 1])
        return float(out[0, 1, 1])
    start = max(0, query_pos - 4)            # a portion whose last row is the query
    rows = query_pos - start + 1
    q = torch.zeros(rows, heads, D, dtype=dtype, device=device)
    q[:, :, 0] = 1.0
    out = ops.window_attn_prefill(
        q, kc, None, DV, table, torch.tensor([0, rows], dtype=torch.int32, device=device),
        torch.tensor([start], dtype=torch.int32, device=device), rows, window, 1.0)
    return float(out[-1, 1, 1])


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("decode", [False, True], ids=["portion", "single"])
def test_window_edges_with_a_needle(target, decode):
    device, dtype = target[0], getattr(torch, target[1])
    for window in (1, 7, 16, 50, 300):
        for query_pos in (window - 1, window, window + 1, 2 * window + 5, 331):
            if query_pos < 0:
                continue
            oldest = max(0, query_pos - window + 1)      # the oldest key still seen
            seen = _needle_case(device, dtype, window, oldest, query_pos, decode)
            assert seen < -2.9, (window, query_pos, seen)
            many = _needle_case(device, dtype, window, oldest, query_pos, decode, heads=19)
            assert many < -2.9, (window, query_pos, many)
            newest = _needle_case(device, dtype, window, query_pos, query_pos, decode)
            assert newest < -2.9, (window, query_pos, newest)
            if oldest > 0:                                # one further back is outside
                unseen = _needle_case(device, dtype, window, oldest - 1, query_pos, decode)
                assert unseen > 0.99, (window, query_pos, unseen)
                many = _needle_case(device, dtype, window, oldest - 1, query_pos, decode, heads=19)
                assert many > 0.99, (window, query_pos, many)
                assert _needle_case(device, dtype, window, 0, query_pos, decode) > 0.99


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("decode", [False, True], ids=["portion", "single"])
def test_causal_sees_far_keys_and_page_borders(target, decode):
    """No window: a needle among hundreds of keys is found wherever it sits —
    position 0, either side of a page border, the query itself."""
    device, dtype = target[0], getattr(torch, target[1])
    for query_pos in (0, 1, 15, 16, 17, 700):
        for key_pos in {0, 15, 16, 17, 31, 32, 255, 256, query_pos - 1, query_pos}:
            if 0 <= key_pos <= query_pos:
                got = _needle_case(device, dtype, 0, key_pos, query_pos, decode)
                assert got < -2.9, (query_pos, key_pos, got)


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("H,D,DV,window", [
    (4, 48, 40, 24),          # two MFMA k-steps
    (6, 40, 24, 50),          # key size not a multiple of 32
    (2, 72, 64, 130),
    (2, 136, 128, 300),
    (1, 256, 192, 70),        # the widest instantiation
    (3, 20, 10, 9),           # not a multiple of 8: the fp32-ALU kernel in bf16 too
    (8, 288, 256, 40),        # wider than the matrix-core kernel's tiles; 8 heads a group
    (2, 320, 300, 50),        # values wider than 256
    (12, 24, 16, 33),         # 4 heads a group
    (16, 64, 48, 70),         # many heads on one latent: single tokens on the matrix cores
    (70, 136, 128, 0),        # more heads than one workgroup's rows
    (2, 24, 24, 0),           # values = the whole key row, no window
])
def test_window_attention_ops_against_dense(target, H, D, DV, window):
    """Both attention kernels over a key-only cache on shuffled pages against
    dense float64 attention, for portions that start mid-window and mid-page."""
    from llmq_amd import ops

    device, dtype = target[0], getattr(torch, target[1])
    g = torch.Generator().manual_seed(H * 1000 + D)
    bs, L = 16, 333
    q = torch.randn(L, H, D, generator=g).to(dtype)
    rows = torch.randn(L, D, generator=g).to(dtype)
    scale = 0.9 / math.sqrt(D)
    nblk = (L + bs - 1) // bs
    table = (torch.randperm(nblk + 3, generator=g)[:nblk]).to(torch.int32).view(1, -1)
    kc = torch.zeros(nblk + 3, 1, bs, D, dtype=dtype)
    for t in range(L):
        kc[int(table[0, t // bs]), 0, t % bs] = rows[t]
    kc = kc.to(device)
    sc = torch.einsum("ihd,jd->hij", q.double(), rows.double()) * scale
    sc = sc.masked_fill(~oracle.visibility(L, window or None).unsqueeze(0), float("-inf"))
    want = torch.einsum("hij,jd->ihd", torch.softmax(sc, -1), rows.double()[:, :DV])
    cuts = [0, 5, min(5 + max(window, 20) + 3, 150), 200, 290, 291, 293] + list(range(294, L + 1))
    got = []
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        qq = q[lo:hi].to(device)
        if hi - lo == 1 and lo > 0:
            got.append(ops.window_attn_decode(
                qq, kc, None, DV, table.to(device),
                torch.tensor([hi], dtype=torch.int32, device=device), window, scale))
        else:
            got.append(ops.window_attn_prefill(
                qq, kc, None, DV, table.to(device),
                torch.tensor([0, hi - lo], dtype=torch.int32, device=device),
                torch.tensor([lo], dtype=torch.int32, device=device), hi - lo, window, scale))
    got = torch.cat(got).double().cpu()
    err = (got - want).abs().max() / want.abs().max()
    assert float(err) < (2e-2 if dtype == torch.bfloat16 else 2e-5), float(err)


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("interleaved", [False, True], ids=["half", "interleaved"])
@pytest.mark.parametrize("H,dim,DR,R,rot_dims", [(3, 8, 4, 20, 4), (2, 16, 8, 24, 8),
                                                 (1, 5, 12, 7, 6), (4, 0, 2, 3, 2)])
def test_rotary_norm_and_cache_step(target, interleaved, H, dim, DR, R, rot_dims):
    """The step between projections and attention against the oracle's
    rotation and norm: packed query, cache rows at their slots, padding rows
    (slot -1) written nowhere, rotation of part of the rotated vector only."""
    from llmq_amd import ops
    from llmq_amd.engine.models.kosalorn import rotary_inv_freq

    device, dtype = target[0], getattr(torch, target[1])
    g = torch.Generator().manual_seed(R + DR)
    T, bs, base, eps = 9, 4, 777.0, 1e-5
    pos = torch.tensor([0, 1, 2, 3, 40, 41, 1000, 1001, 5])
    q = torch.randn(T, H, dim + DR, generator=g).to(dtype)
    q_lat = torch.randn(T, H, R, generator=g).to(dtype)
    ckr = torch.randn(T, R + DR + 3, generator=g).to(dtype)[:, :R + DR]   # a row-strided slice
    cw = (1 + 0.2 * torch.randn(R, generator=g)).to(dtype)
    slots = torch.tensor([12, 13, 14, 15, 0, 1, 6, 7, -1])
    cache = torch.full((5, 1, bs, R + DR), 9.0, dtype=dtype, device=device)
    out = ops.latent_rope_pack(q.to(device), q_lat.to(device), ckr.to(device), cw.to(device),
                               rotary_inv_freq(base, rot_dims).to(device), pos.to(device), cache,
                               slots.to(device), dim, rot_dims, interleaved, eps)
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=1e-5, atol=2e-5)

    def rot_at(x, p):   # the oracle rotates row t by position t: place x at row p
        buf = torch.zeros(p + 1, *x.shape, dtype=torch.float64)
        buf[p] = x.double()
        return oracle.rotate(buf, base, rot_dims, interleaved)[p]

    for t in range(T):
        p = int(pos[t])
        want_q = torch.cat([q_lat[t].double(), rot_at(q[t, :, dim:], p)], dim=-1)
        assert torch.allclose(out[t].double().cpu(), want_q, **tol), t
        if int(slots[t]) >= 0:
            want_row = torch.cat([oracle.plain_norm(ckr[t, :R].double(), cw.double(), eps),
                                  rot_at(ckr[t, R:], p)])
            s = int(slots[t])
            assert torch.allclose(cache[s // bs, 0, s % bs].double().cpu(), want_row, **tol), t
    touched = {int(s) for s in slots if s >= 0}
    flat = cache.view(-1, R + DR).float().cpu()
    for s in range(flat.shape[0]):
        if s not in touched:
            assert torch.all(flat[s] == 9.0), s


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("H,D,DV", [(2, 16, 32), (3, 40, 72), (1, 128, 200), (5, 6, 5)])
def test_hgrn2_recurrence_against_token_by_token(target, H, D, DV):
    """The lower-bounded mode of the recurrence kernel and the head norm for
    several packed sequences with old and fresh slots against float64."""
    from llmq_amd import ops

    device, dtype = target[0], getattr(torch, target[1])
    g = torch.Generator().manual_seed(D * 7 + DV)
    lens, slots, fresh = [70, 21, 2, 1], [3, 0, 5, 1], [1, 0, 0, 1]
    T = sum(lens)
    q = torch.randn(T, H, D, generator=g).to(dtype)
    v = torch.randn(T, H, DV, generator=g).to(dtype)
    z = (2 * torch.randn(T, H, D, generator=g)).to(dtype)
    zb = torch.randn(H * D, generator=g)
    low = torch.rand(H * D, generator=g)
    state0 = torch.randn(6, H, D, DV, generator=g)
    w = (1 + 0.2 * torch.randn(DV, generator=g)).to(dtype)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    st = state0.clone().to(device)
    o = ops.gated_recurrence(q.to(device), None, v.to(device), z.to(device), zb.to(device), st,
                             cu.to(device), torch.tensor(slots, dtype=torch.int32, device=device),
                             torch.tensor(fresh, dtype=torch.int32, device=device),
                             lower=low.to(device), q_silu=True)
    y = ops.head_norm(o, w.to(device), 1e-5, dtype)
    lo = low.double().view(1, H, D)
    f = lo + (1 - lo) * torch.sigmoid(z.double() + zb.double().view(1, H, D))
    qa = oracle.silu(q.double())
    want_o = torch.empty(T, H, DV, dtype=torch.float64)
    want_state = state0.double().clone()
    at = 0
    for n, slot, fr in zip(lens, slots, fresh):
        S = torch.zeros(H, D, DV, dtype=torch.float64) if fr else state0[slot].double().clone()
        for t in range(at, at + n):
            S = f[t].unsqueeze(-1) * S + (1 - f[t]).unsqueeze(-1) * v[t].double().unsqueeze(-2)
            want_o[t] = torch.einsum("hdv,hd->hv", S, qa[t])
        want_state[slot] = S
        at += n
    assert float((o.double().cpu() - want_o).abs().max() / want_o.abs().max()) < 1e-5
    assert float((st.double().cpu() - want_state).abs().max() / want_state.abs().max()) < 1e-5
    want_y = oracle.plain_norm(want_o, w.double(), 1e-5).reshape(T, H * DV)
    err = float((y.double().cpu() - want_y).abs().max() / want_y.abs().max())
    assert err < (1e-2 if dtype == torch.bfloat16 else 1e-5), err


@pytest.mark.parametrize("target", DEVICES)
def test_hgrn2_gate_limits(target):
    """Gate pre-activation +60: f = 1, nothing is written and the old state
    answers unchanged, however the rows are cut. Pre-activation -60: f is
    the lower bound, so the state is l*S + (1-l)*v exactly."""
    from llmq_amd import ops

    device, dtype = target[0], getattr(torch, target[1])
    H, D, DV, n = 1, 4, 8, 24
    q = torch.zeros(n, H, D, dtype=dtype)
    q[:, 0, 2] = 30.0                          # silu(30) = 30
    v = torch.arange(n * DV, dtype=torch.float32).view(n, 1, DV).remainder(7).to(dtype)
    zb = torch.zeros(H * D)
    low = torch.full((H * D,), 0.25)
    state = torch.full((3, H, D, DV), 99.0)
    state[1] = torch.arange(D * DV, dtype=torch.float32).view(1, D, DV) / 8
    state = state.to(device)
    args = lambda lo, hi, fr: (  # noqa: E731
        zb.to(device), state, torch.tensor([0, hi - lo], dtype=torch.int32, device=device),
        torch.tensor([1], dtype=torch.int32, device=device),
        torch.tensor([fr], dtype=torch.int32, device=device))
    keep = state[1, 0, 2].clone().cpu()
    z = torch.full((n, H, D), 60.0, dtype=dtype)
    for lo, hi in ((0, 9), (9, 10), (10, 12), (12, 24)):
        o = ops.gated_recurrence(q[lo:hi].to(device), None, v[lo:hi].to(device),
                                 z[lo:hi].to(device), *args(lo, hi, 0),
                                 lower=low.to(device), q_silu=True)
        assert torch.allclose(o.cpu()[:, 0], (30.0 * keep).expand(hi - lo, DV), rtol=1e-5)
    assert torch.all(state[0] == 99.0) and torch.all(state[2] == 99.0)
    z = torch.full((n, H, D), -60.0, dtype=dtype)
    o = ops.gated_recurrence(q.to(device), None, v.to(device), z.to(device), *args(0, n, 1),
                             lower=low.to(device), q_silu=True)
    S = torch.zeros(DV, dtype=torch.float64)
    for t in range(n):
        S = 0.25 * S + 0.75 * v[t, 0].double()
        assert torch.allclose(o[t, 0].double().cpu(), 30.0 * S, rtol=1e-5, atol=1e-5), t


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("W,F,E,top,T", [(48, 24, 5, 2, 9), (40, 20, 12, 1, 3), (36, 10, 3, 3, 130),
                                         (64, 32, 8, 2, 200), (33, 7, 70, 4, 5)])
def test_router_and_expert_mixture_ops(target, W, F, E, top, T):
    """sigmoid_topk and moe_experts — the matrix-vector form for few rows and
    inside decode graphs, the sorted form for many — against the oracle's
    mixture on the same inputs."""
    from llmq_amd import ops

    device, dtype = target[0], getattr(torch, target[1])
    g = torch.Generator().manual_seed(W + E)
    h = torch.randn(T, W, generator=g).to(dtype)
    w = {"router": (3.0 / math.sqrt(W)) * torch.randn(E, W, generator=g)}
    for e in range(E):
        w[f"e{e}.gate"] = (torch.randn(F, W, generator=g) * 2 / math.sqrt(W)).to(dtype)
        w[f"e{e}.up"] = (torch.randn(F, W, generator=g) * 2 / math.sqrt(W)).to(dtype)
        w[f"e{e}.down"] = (torch.randn(W, F, generator=g) / math.sqrt(F)).to(dtype)
    logits = torch.nn.functional.linear(h.float(), w["router"])
    idx, sc = ops.sigmoid_topk(logits.to(device), top)
    s = torch.sigmoid(logits.double())
    ws, wi = torch.topk(s, top, dim=-1)
    assert idx.dtype == torch.int32 and torch.equal(idx.cpu().long(), wi)
    assert torch.allclose(sc.double().cpu(), ws, rtol=1e-5, atol=1e-6)
    gate_up = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)]).to(device)
    down = torch.stack([w[f"e{e}.down"] for e in range(E)]).to(device)
    want = oracle.expert_mixture(
        h.double(), {k: v.double() for k, v in w.items()},
        {"router": {"experts": E, "top": top}})
    for sync_free in (False, True):
        got = ops.moe_experts(h.to(device), idx, sc, gate_up, down, sync_free=sync_free)
        err = float((got.double().cpu() - want).abs().max() / want.abs().max())
        assert err < (3e-2 if dtype == torch.bfloat16 else 1e-5), (sync_free, err)


@pytest.mark.parametrize("target", DEVICES)
def test_gated_join_and_side_gate_ops(target):
    from llmq_amd import ops

    device, dtype = target[0], getattr(torch, target[1])
    g = torch.Generator().manual_seed(11)
    for W in (48, 33, 256):
        T = 7
        res = torch.randn(T, W, generator=g)
        wide = torch.randn(T, 3 * W + 16, generator=g).to(dtype)   # gates are slices of it
        g1, g2 = wide[:, 8:8 + W], wide[:, 16 + W:16 + 2 * W]
        y1, y2 = torch.randn(T, W, generator=g).to(dtype), torch.randn(T, W, generator=g).to(dtype)
        b1, b2 = torch.randn(W, generator=g), torch.randn(W, generator=g)
        want1 = res.double() + torch.sigmoid(g1.double() + b1.double()) * y1.double()
        want2 = want1 + torch.sigmoid(g2.double() + b2.double()) * y2.double()
        wd = wide.to(device)
        for two, want in ((False, want1), (True, want2)):
            r = res.clone().to(device)
            out = ops.gated_residual_add(
                r, y1.to(device), wd[:, 8:8 + W], b1.to(device),
                y2.to(device) if two else None, wd[:, 16 + W:16 + 2 * W] if two else None,
                b2.to(device) if two else None, dtype)
            assert r.dtype == torch.float32 and out.dtype == dtype
            assert_close(r, want, (device, "float32"), "residual")
            assert_close(out, want, target, "rounded copy")
    a = torch.randn(5, 6, generator=g).to(dtype)
    table = torch.randn(20, 30, generator=g).to(dtype)
    toks = torch.tensor([3, 19, 0, 3, 7])
    got = ops.side_gate_mul(a.to(device), table.to(device), toks.to(device), 12)
    want = oracle.gelu_tanh(a.double()) * table.double()[toks][:, 12:18]
    assert_close(got, want, target, "side gate")


# ----------------------------------- the engine's own entry point: greedy --

@pytest.mark.parametrize("target", DEVICES[:2])
def test_greedy_generation_through_the_scheduler(mixed_model, target):
    """add_request + step(): budgeted chunked prefill, continuous batching,
    preemption by recompute in a small pool, hipGraph decode on the GPU —
    greedy tokens equal the oracle's."""
    cfg, tensors, path = mixed_model(target)
    prompts = [tokens_for(n, cfg["vocab"], 40 + i) for i, n in enumerate((37, 5, 18, 1, 26))]
    n_new = 20
    want = [oracle.greedy(cfg, tensors, p, n_new) for p in prompts]
    eng = make_engine(path, target, blocks=7, block_size=16, max_seqs=3, prefill_budget=16)
    params = SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True)
    for i, p in enumerate(prompts):
        eng.add_request(f"g{i}", prompt_token_ids=p, params=params)
    got = {f"g{i}": [] for i in range(len(prompts))}
    seqs = list(eng._seqs.values())
    kinds = set()
    while eng.has_unfinished():
        for out in eng.step():
            got[out.request_id].extend(out.new_token_ids)
        kinds.add(eng.last_step_kind)
    assert {"prefill", "decode", "mixed"} <= kinds
    # the pool is too small for three grown sequences: one was evicted, lost
    # its blocks and state slot, and recomputed its context from position 0
    assert sum(s.num_preemptions for s in seqs) > 0
    for i in range(len(prompts)):
        assert got[f"g{i}"] == want[i], f"request {i}"
    assert eng.allocator.num_free == 7 and eng.slot_allocator.num_free == 3


def test_preset_runs_through_generate(tmp_path):
    """A preset name is a valid model: random weights, sampling, detokenised text."""
    eng = LLMEngine(EngineConfig(model="tiny-kosalorn", device="cpu", max_num_seqs=2,
                                 max_model_len=64, load_weights=False, num_kv_blocks=16))
    outs = eng.generate_batch(["a b", "c"], SamplingParams(temperature=0.8, max_tokens=5,
                                                           ignore_eos=True, seed=3))
    assert len(outs) == 2


def test_trace_runner_cli(tmp_path, mixed_model):
    """bin/trace_run end to end on the CPU: steps in, logits files out."""
    import os
    import subprocess
    import sys

    import numpy as np

    cfg, tensors, path = mixed_model(("cpu", "float32"))
    toks = tokens_for(30, cfg["vocab"], 50)
    steps = [
        {"step": 0, "entries": [{"id": "q", "tokens": toks[:20], "want": [0, 19]}], "end": []},
        {"step": 1, "entries": [{"id": "q", "tokens": toks[20:21], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "q", "tokens": toks[21:], "want": [8]}], "end": ["q"]},
    ]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, HIP_VISIBLE_DEVICES="", CUDA_VISIBLE_DEVICES="")
    res = subprocess.run(
        [sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype",
         "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64"],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True,
        timeout=120, env=env)
    assert res.returncode == 0, res.stderr[-2000:]
    assert [l for l in res.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = oracle.forward(cfg, tensors, toks)
    a = np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(2, -1)
    b = np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4").reshape(1, -1)
    assert not (tmp_path / "o" / "1.f32").exists()
    got = torch.from_numpy(np.concatenate([a, b]))
    assert_close(got, want[[0, 19, 29]], ("cpu", "float32"))

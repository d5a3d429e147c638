"""Kakovik (hybrid decoder) against the plain oracle in kakovik_oracle.py.

Every test builds its own small configuration and random checkpoint, loads
it through the engine's own entry points (config reader, weight loader,
scheduler, cache and state managers) and compares logits with the oracle.
The scenarios run on the CPU (torch reference ops) and, marked ``gpu``, on
the HIP kernels in fp32 (sharp) and bf16.
"""

from __future__ import annotations

import json
import math

import pytest
import torch

import kakovik_oracle as oracle
from llmq_amd.engine.config import EngineConfig
from llmq_amd.engine.engine import LLMEngine
from llmq_amd.engine.sampling_params import SamplingParams


# --------------------------------------------------------------- fixtures --

def attn(heads=4, kv_heads=2, dim=16, vdim=24, span=20, far=37, v_mix=True, ff=48, scale=0.3):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                      "scale": scale, "bias_max": far, "mask": {"size": span}, "v_mix": v_mix},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def gla(heads=2, dim=8, vdim=24, tau=3.0, ff=0):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(layers, width=40, vocab=96, eps=1e-5, logit_scale=1.7):
    return {"architecture": "Kakovik", "layers": layers, "logit_scale": logit_scale,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def make_tensors(cfg, seed=0, bias_rows=10, rank=6):
    g = torch.Generator().manual_seed(seed)

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16)

    def lin(out, inn):
        return rnd(out, inn, std=1.0 / math.sqrt(inn))

    W, V = cfg["width"], cfg["vocab"]
    t = {"embed": rnd(V, W), "head": lin(V, W), "final.norm": rnd(W, std=0.2)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        t[p + "norm1"], t[p + "norm1b"] = rnd(W, std=0.2), rnd(W, std=0.2)
        if layer["type"] == "attention":
            nq, nk, nv = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"] = lin(nq, W), lin(nk, W), lin(nv, W)
            t[p + "mix.q.norm"] = rnd(nq, std=0.2, mean=1.0)
            t[p + "mix.k.norm"] = rnd(nk, std=0.2, mean=1.0)
            t[p + "mix.rel"] = rnd(bias_rows, m["heads"])
            t[p + "mix.vmix"] = torch.tensor(0.2 + 0.1 * i).to(torch.bfloat16)
            t[p + "mix.g"] = lin(m["heads"], W)
            t[p + "mix.o"] = lin(W, m["heads"] * m["vdim"])
        else:
            nk, nv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            t[p + "mix.q"], t[p + "mix.k"] = lin(nk, W), lin(nk, W)
            t[p + "mix.v"], t[p + "mix.g"] = lin(nv, W), lin(nv, W)
            t[p + "mix.a1"], t[p + "mix.a2"] = lin(rank, W), lin(nk, rank)
            t[p + "mix.a2.b"] = rnd(nk, mean=1.0)
            t[p + "mix.norm"] = rnd(m["vdim"], std=0.2, mean=1.0)
            t[p + "mix.o"] = lin(W, nv)
        if layer["mlp"]:
            ff = layer["mlp"]["ff"]
            t[p + "norm2"], t[p + "norm2b"] = rnd(W, std=0.2), rnd(W, std=0.2)
            t[p + "mlp.gate"], t[p + "mlp.up"], t[p + "mlp.down"] = lin(ff, W), lin(ff, W), lin(W, ff)
    return t


def write_checkpoint(path, cfg, tensors):
    from safetensors.torch import save_file

    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(path / "model.safetensors"))
    return str(path)


# a config that differs from a plain stack in every switch: GLA first, an
# attention layer that does not blend before the first blending one, grouped
# kv heads, a layer without feed-forward, a GLA layer with one, attention last
MIXED_LAYERS = [
    gla(heads=2, dim=8, vdim=24, tau=3.0, ff=32),
    attn(heads=4, kv_heads=2, dim=16, vdim=24, span=20, far=37, v_mix=False, ff=0),
    attn(heads=4, kv_heads=1, dim=8, vdim=48, span=33, far=20, v_mix=True, ff=48),
    gla(heads=3, dim=12, vdim=8, tau=1.0),
    attn(heads=2, kv_heads=2, dim=24, vdim=24, span=7, far=100, v_mix=True, ff=48),
    attn(heads=6, kv_heads=3, dim=8, vdim=16, span=64, far=64, v_mix=True, ff=0),
]


def tokens_for(n, vocab, seed):
    g = torch.Generator().manual_seed(1000 + seed)
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
    sharp comparison; bf16 rounds every GEMM input and output of a six-layer
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
    for k, n in enumerate(cuts):
        last = at + n == len(toks)
        out.append(engine.replay_step(
            [{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}],
            end=[rid] if (last and end) else []))
        at += n
    assert at == len(toks)
    return torch.cat(out)


# ------------------------------------------------------ mechanisms alone --

@pytest.mark.parametrize("rows,far", [(10, 37.0), (16, 120.0), (8, 16.0), (32, 1000.0), (6, 3.5)])
def test_distance_bucket_matches_oracle(rows, far):
    from llmq_amd.engine.models.kakovik import distance_bucket

    for n in range(0, 2500):
        assert distance_bucket(n, rows, far) == oracle.distance_bucket(n, rows, far)
    # identity below half, last row from `far` on, monotone
    half = rows // 2
    assert [distance_bucket(n, rows, far) for n in range(half)] == list(range(half))
    assert distance_bucket(int(math.ceil(far)), rows, far) == rows - 1
    seq = [distance_bucket(n, rows, far) for n in range(3000)]
    assert seq == sorted(seq) and seq[-1] == rows - 1


@pytest.mark.parametrize("target", DEVICES)
def test_norm_ops(target):
    from llmq_amd import ops

    device, dtype = target[0], getattr(torch, target[1])
    g = torch.Generator().manual_seed(3)
    for width in (40, 33, 256):
        res = torch.randn(9, width, generator=g)
        y = torch.randn(9, width, generator=g).to(dtype)
        w1 = (0.2 * torch.randn(width, generator=g)).to(dtype)
        w2 = (0.2 * torch.randn(width, generator=g)).to(dtype)
        want_res = res.double() + oracle.zero_centred_rmsnorm(y.double(), w1.double(), 1e-5)
        want_h = oracle.zero_centred_rmsnorm(want_res, w2.double(), 1e-5)
        r = res.clone().to(device)
        h = ops.sandwich_norm_res32(y.clone().to(device), r, w1.to(device), w2.to(device), 1e-5, 1.0)
        assert r.dtype == torch.float32
        assert_close(r, want_res, (device, "float32"), "residual")
        assert_close(h, want_h, target, "normed")
        h0 = ops.rmsnorm_cast(res.to(device), w1.to(device), 1e-5, 1.0, dtype)
        assert_close(h0, oracle.zero_centred_rmsnorm(res.double(), w1.double(), 1e-5), target)


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("layers", [
    pytest.param([attn(ff=0)], id="attention"),
    pytest.param([attn(heads=3, kv_heads=3, dim=8, vdim=8, span=9, far=9, ff=0)], id="attention-eq"),
    pytest.param([gla()], id="gla"),
    pytest.param([gla(heads=1, dim=40, vdim=70, tau=0.7)], id="gla-wide"),
    pytest.param([attn(v_mix=True, ff=0), attn(v_mix=True, ff=0)], id="value-blend"),
    pytest.param([attn(ff=48)], id="attention+ff"),
    pytest.param([], id="no-layers"),
])
def test_mechanism_alone(tmp_path, target, layers):
    cfg = make_config(layers)
    tensors = make_tensors(cfg, seed=len(layers))
    path = write_checkpoint(tmp_path / "m", cfg, tensors)
    eng = make_engine(path, target)
    toks = tokens_for(47, cfg["vocab"], 1)
    eng.model.taps = []
    got = replay(eng, "a", toks, [47])
    want, want_layers = (oracle.forward(cfg, tensors, toks, return_layers=True)
                         if layers else (oracle.forward(cfg, tensors, toks), None))
    if layers and target[1] == "float32":
        for i, tap in enumerate(eng.model.taps):
            assert_close(tap, want_layers[i], target, f"residual after layer {i}")
    assert_close(got, want, target, "logits")


# -------------------------------------------------- cuts, batches, reuse --

@pytest.fixture(scope="module")
def mixed_model(tmp_path_factory):
    cfg = make_config(MIXED_LAYERS, width=48, vocab=128)
    tensors = make_tensors(cfg, seed=7)
    path = write_checkpoint(tmp_path_factory.mktemp("kk") / "m", cfg, tensors)
    return cfg, tensors, path


@pytest.mark.parametrize("target", DEVICES)
def test_prefill_equals_token_by_token(mixed_model, target):
    cfg, tensors, path = mixed_model
    toks = tokens_for(90, cfg["vocab"], 2)
    want = oracle.forward(cfg, tensors, toks)
    eng = make_engine(path, target)
    assert_close(replay(eng, "w", toks, [90]), want, target, "whole prompt")
    assert_close(replay(eng, "d", toks, [1] * 90), want, target, "token by token")
    # everything was given back
    assert eng.allocator.num_free == eng.allocator.num_blocks
    assert eng.slot_allocator.num_free == 4


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("cuts", [
    [2, 2, 3, 13, 2, 40, 1, 1, 16, 10],
    [16, 16, 16, 16, 16, 10],          # on page borders
    [15, 17, 1, 31, 2, 24],            # just off them
    [7, 7, 7, 7, 7, 7, 7, 7, 7, 7, 7, 7, 6],  # the shortest span's size
    [89, 1],
])
def test_portions(mixed_model, target, cuts):
    cfg, tensors, path = mixed_model
    toks = tokens_for(90, cfg["vocab"], 3)
    want = oracle.forward(cfg, tensors, toks)
    eng = make_engine(path, target)
    assert_close(replay(eng, "c", toks, cuts), want, target, f"cuts {cuts}")


@pytest.mark.parametrize("target", DEVICES)
def test_mixed_batches_equal_alone_and_reuse(mixed_model, target):
    """Six unequal requests through four slots and a pool that cannot hold
    them all at once: portions beside single tokens, requests that pause,
    blocks and slots handed on to later requests."""
    cfg, tensors, path = mixed_model
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
    cfg, tensors, path = mixed_model
    first = tokens_for(64, cfg["vocab"], 30)
    second = tokens_for(50, cfg["vocab"], 31)
    want = oracle.forward(cfg, tensors, second)
    eng = make_engine(path, target, blocks=4, max_seqs=1)
    replay(eng, "x", first, [60, 1, 1, 1, 1])
    assert_close(replay(eng, "y", second, [3, 1, 1, 45]), want, target, "after reuse")


@pytest.mark.parametrize("target", DEVICES)
def test_long_decode_across_spans_and_pages(mixed_model, target):
    cfg, tensors, path = mixed_model
    toks = tokens_for(5 + 150, cfg["vocab"], 4)
    want = oracle.forward(cfg, tensors, toks)
    eng = make_engine(path, target)
    assert_close(replay(eng, "l", toks, [5] + [1] * 150), want, target, "long decode")


# ------------------------------------------ edges made visible by design --

def _needle_case(device, dtype, span, key_pos, query_pos, decode, block_size=16):
    """One head; every key scores 0 but the needle, which scores +40: the
    output is the needle's value iff the query may see it."""
    from llmq_amd import ops

    D, DV, n = 8, 8, query_pos + 1
    nblocks = (n + block_size - 1) // block_size
    kc = torch.zeros(nblocks + 2, 1, block_size, D, dtype=dtype)
    vc = torch.zeros(nblocks + 2, 1, block_size, DV, dtype=dtype)
    table = torch.arange(nblocks + 1, 0, -1, dtype=torch.int32).view(1, -1)  # reversed pages
    for p in range(n):
        b, o = int(table[0, p // block_size]), p % block_size
        vc[b, 0, o, :] = 1.0
    b, o = int(table[0, key_pos // block_size]), key_pos % block_size
    kc[b, 0, o, 0] = 40.0
    vc[b, 0, o, :] = -3.0
    bias = torch.zeros(1, span)
    kc, vc, bias, table = kc.to(device), vc.to(device), bias.to(device), table.to(device)
    if decode:
        q = torch.zeros(1, 1, D, dtype=dtype, device=device)
        q[0, 0, 0] = 1.0
        out = ops.chunk_bias_attn_decode(
            q, None, kc, vc, bias, table, torch.tensor([n], dtype=torch.int32, device=device),
            span, 1.0)
        return float(out[0, 0, 0])
    start = max(0, query_pos - 4)            # a portion whose last row is the query
    rows = query_pos - start + 1
    q = torch.zeros(rows, 1, D, dtype=dtype, device=device)
    q[:, 0, 0] = 1.0
    out = ops.chunk_bias_attn_prefill(
        q, None, kc, vc, bias, table,
        torch.tensor([0, rows], dtype=torch.int32, device=device),
        torch.tensor([start], dtype=torch.int32, device=device), rows, span, 1.0)
    return float(out[-1, 0, 0])


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("decode", [False, True], ids=["portion", "single"])
def test_span_edges_with_a_needle(target, decode):
    device, dtype = target[0], getattr(torch, target[1])
    for span in (7, 16, 50, 300):
        for blk in (1, 2):
            first = blk * span                 # first position of the query's span
            for query_pos in (first, first + 1, first + span - 1):
                # the span's first key is seen, the one before it is not
                seen = _needle_case(device, dtype, span, first, query_pos, decode)
                unseen = _needle_case(device, dtype, span, first - 1, query_pos, decode)
                assert seen < -2.9, (span, query_pos, seen)
                assert unseen > 0.99, (span, query_pos, unseen)
            # a far key among hundreds, still inside
            if span == 300:
                far = _needle_case(device, dtype, span, first + 1, first + 298, decode)
                assert far < -2.9


@pytest.mark.parametrize("target", DEVICES)
def test_bias_moves_attention_by_distance(target):
    """All scores equal: the weights are softmax(bias[i - j]) alone."""
    from llmq_amd import ops

    device, dtype = target[0], getattr(torch, target[1])
    span, n, bs = 12, 12, 16
    kc = torch.zeros(2, 1, bs, 8, dtype=dtype, device=device)
    vc = torch.zeros(2, 1, bs, 16, dtype=dtype, device=device)
    for p in range(n):
        vc[1, 0, p, p] = 1.0                 # value p marks position p
    bias = torch.linspace(-2, 2, span).view(1, span).to(device)
    table = torch.tensor([[1]], dtype=torch.int32, device=device)
    q = torch.zeros(1, 1, 8, dtype=dtype, device=device)
    out = ops.chunk_bias_attn_decode(q, None, kc, vc, bias, table,
                                     torch.tensor([n], dtype=torch.int32, device=device), span, 1.0)
    want = torch.softmax(bias[0].flip(0).double().cpu(), 0)  # key j at distance n-1-j
    assert_close(out[0, 0, :n].view(1, -1), want.view(1, -1), target)


@pytest.mark.parametrize("target", DEVICES)
def test_gla_state_is_carried_exactly(target):
    """Decay 1 (huge positive pre-activation) and q = k = one-hot: o_t must be
    the running sum of every earlier value, however the rows are cut."""
    from llmq_amd import ops

    device, dtype = target[0], getattr(torch, target[1])
    H, D, DV, n = 1, 4, 8, 40
    q = torch.zeros(n, H, D, dtype=dtype)
    q[:, 0, 1] = 2.0                           # q scale D^-1/2 = 1/2 → 1
    k = torch.zeros(n, H, D, dtype=dtype)
    k[:, 0, 1] = 1.0
    v = torch.arange(n * DV, dtype=torch.float32).view(n, 1, DV).remainder(7).to(dtype)
    z = torch.full((n, H, D), 60.0, dtype=dtype)
    zb = torch.zeros(H * D)
    state = torch.full((3, H, D, DV), 99.0).to(device)  # stale content of a reused slot
    want = v.float().cumsum(0)
    outs = []
    for lo, hi in ((0, 17), (17, 18), (18, 20), (20, 40)):
        outs.append(ops.gla_recurrence(
            q[lo:hi].to(device), k[lo:hi].to(device), v[lo:hi].to(device), z[lo:hi].to(device),
            zb.to(device), state,
            torch.tensor([0, hi - lo], dtype=torch.int32, device=device),
            torch.tensor([1], dtype=torch.int32, device=device),
            torch.tensor([int(lo == 0)], dtype=torch.int32, device=device), 1.0))
    got = torch.cat(outs).cpu()[:, 0]
    assert torch.allclose(got, want[:, 0], rtol=1e-5, atol=1e-4)
    # only slot 1 and only key channel 1 moved
    st = state.cpu()
    assert torch.all(st[0] == 99.0) and torch.all(st[2] == 99.0)
    assert torch.allclose(st[1, 0, 1], want[-1, 0], rtol=1e-5, atol=1e-4)
    assert torch.all(st[1, 0, 0] == 0) and torch.all(st[1, 0, 2:] == 0)


@pytest.mark.parametrize("target", DEVICES)
def test_gla_decay_forgets(target):
    """A strong decay (pre-activation -20, tau 1) wipes the state each token:
    o_t depends on token t alone."""
    from llmq_amd import ops

    device, dtype = target[0], getattr(torch, target[1])
    H, D, DV, n = 2, 6, 5, 9
    g = torch.Generator().manual_seed(5)
    q, k = torch.randn(n, H, D, generator=g).to(dtype), torch.randn(n, H, D, generator=g).to(dtype)
    v = torch.randn(n, H, DV, generator=g).to(dtype)
    z = torch.full((n, H, D), -20.0, dtype=dtype)
    state = torch.zeros(1, H, D, DV, device=device)
    o = ops.gla_recurrence(q.to(device), k.to(device), v.to(device), z.to(device),
                           torch.zeros(H * D, device=device), state,
                           torch.tensor([0, n], dtype=torch.int32, device=device),
                           torch.zeros(1, dtype=torch.int32, device=device),
                           torch.ones(1, dtype=torch.int32, device=device), 1.0)
    want = (q.double() * k.double()).sum(-1, keepdim=True) * D ** -0.5 * v.double()
    assert torch.allclose(o.cpu().double(), want, rtol=1e-4, atol=1e-5)


# ----------------------------------- the engine's own entry point: greedy --

@pytest.mark.parametrize("target", [DEVICES[0], DEVICES[1]])
def test_greedy_generation_through_the_scheduler(mixed_model, target):
    """add_request + step(): budgeted chunked prefill, continuous batching,
    preemption by recompute in a small pool, hipGraph decode on the GPU —
    greedy tokens equal the oracle's."""
    cfg, tensors, path = mixed_model
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


def test_config_reader_takes_sizes_from_config_and_shapes(tmp_path):
    from llmq_amd.engine.model_specs import resolve_spec

    cfg = make_config(MIXED_LAYERS, width=48, vocab=128)
    path = write_checkpoint(tmp_path / "m", cfg, make_tensors(cfg, bias_rows=14, rank=5))
    spec = resolve_spec(path)
    assert spec.family == "kakovik" and spec.num_layers == 6 and spec.hidden_size == 48
    assert [ls.mixer.kind for ls in spec.layers] == ["gla", "attention", "attention", "gla",
                                                     "attention", "attention"]
    assert spec.layers[1].mixer.bias_rows == 14 and spec.layers[0].mixer.decay_rank == 5
    assert spec.layers[2].mixer.span == 33 and spec.layers[2].mixer.bias_far == 20
    assert spec.layers[0].ff == 32 and spec.layers[1].ff == 0
    assert spec.logit_scale == 1.7 and spec.rms_eps == 1e-5


def test_trace_runner_cli(tmp_path, mixed_model):
    """bin/trace_run end to end on the CPU: steps in, logits files out."""
    import os
    import subprocess
    import sys

    import numpy as np

    cfg, tensors, path = mixed_model
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


# ------------------------------ kernel envelopes: sizes beyond the models --

@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("H,G,D,DV,span", [
    (4, 2, 32, 16, 24),       # one MFMA k-step, one channel tile
    (6, 3, 40, 72, 50),       # q/k size not a multiple of 32, five channel tiles
    (2, 1, 64, 48, 130),
    (2, 2, 128, 136, 300),    # the widest instantiation
    (1, 1, 256, 256, 70),
    (3, 3, 20, 10, 9),        # not a multiple of 8: the fp32-ALU kernel in bf16 too
])
def test_attention_ops_against_dense(target, H, G, D, DV, span):
    """qknorm_vmix_cache + both attention kernels on shuffled pages against
    dense float64 attention, for portions that start mid-span and mid-page."""
    from llmq_amd import ops

    device, dtype = target[0], getattr(torch, target[1])
    g = torch.Generator().manual_seed(H * 1000 + D)
    bs, L = 16, 333
    nq, nk, nv = H * D, G * D, G * DV
    proj = torch.randn(L, nq + nk + nv + H, generator=g).to(dtype)
    v_first = torch.randn(L, nv, generator=g).to(dtype)
    qw = (1 + 0.2 * torch.randn(nq, generator=g)).to(dtype)
    kw = (1 + 0.2 * torch.randn(nk, generator=g)).to(dtype)
    bias = torch.randn(H, span, generator=g)
    lam, scale, eps = 0.35, 0.7 / math.sqrt(D), 1e-5
    nblk = (L + bs - 1) // bs
    table = (torch.randperm(nblk + 3, generator=g)[:nblk]).to(torch.int32).view(1, -1)
    kc = torch.zeros(nblk + 3, G, bs, D, dtype=dtype, device=device)
    vc = torch.zeros(nblk + 3, G, bs, DV, dtype=dtype, device=device)
    # dense reference
    pd = proj.double()
    qn = oracle.plain_rmsnorm(pd[:, :nq], qw.double(), eps).view(L, H, D)
    kn = oracle.plain_rmsnorm(pd[:, nq:nq + nk], kw.double(), eps).view(L, G, D)
    vm = ((1 - lam) * pd[:, nq + nk:nq + nk + nv] + lam * v_first.double()).view(L, G, DV)
    if dtype == torch.bfloat16:   # what the cache holds
        qn, kn, vm = (t.to(dtype).double() for t in (qn, kn, vm))
    kh, vh = kn.repeat_interleave(H // G, 1), vm.repeat_interleave(H // G, 1)
    i = torch.arange(L).view(-1, 1)
    j = torch.arange(L).view(1, -1)
    sc = torch.einsum("ihd,jhd->hij", qn, kh) * scale + bias.double()[:, (i - j).clamp(0, span - 1)]
    sc = sc.masked_fill(~oracle.block_causal_mask(L, span).unsqueeze(0), float("-inf"))
    want = torch.einsum("hij,jhd->ihd", torch.softmax(sc, -1), vh)
    want = want * torch.sigmoid(pd[:, nq + nk + nv:]).unsqueeze(-1)
    # engine ops: portions, the last rows one by one
    cuts = [0, 5, min(5 + span + 3, 150), 200, 290, 291, 293] + list(range(294, L + 1))
    got = []
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        p = proj[lo:hi].clone().to(device)
        q, k, v = p[:, :nq], p[:, nq:nq + nk], p[:, nq + nk:nq + nk + nv]
        gate = p[:, nq + nk + nv:]
        slots = torch.tensor([int(table[0, t // bs]) * bs + t % bs for t in range(lo, hi)],
                             dtype=torch.long, device=device)
        ops.qknorm_vmix_cache(q, k, v, qw.to(device), kw.to(device), v_first[lo:hi].to(device),
                              lam, kc, vc, slots, eps)
        q3 = q.view(hi - lo, H, D)
        if hi - lo == 1 and lo > 0:
            got.append(ops.chunk_bias_attn_decode(
                q3, gate, kc, vc, bias.to(device), table.to(device),
                torch.tensor([hi], dtype=torch.int32, device=device), span, scale))
        else:
            got.append(ops.chunk_bias_attn_prefill(
                q3, gate, kc, vc, bias.to(device), table.to(device),
                torch.tensor([0, hi - lo], dtype=torch.int32, device=device),
                torch.tensor([lo], dtype=torch.int32, device=device), hi - lo, span, scale))
    got = torch.cat(got).double().cpu()
    err = (got - want).abs().max() / want.abs().max()
    assert float(err) < (2e-2 if dtype == torch.bfloat16 else 2e-5), float(err)


@pytest.mark.parametrize("target", DEVICES)
@pytest.mark.parametrize("H,D,DV,tau", [(2, 16, 32, 16.0), (3, 40, 72, 4.0), (1, 128, 200, 1.0),
                                        (1, 256, 24, 0.5), (5, 6, 5, 2.0)])
def test_gla_ops_against_recurrence(target, H, D, DV, tau):
    """gla_recurrence + gla_out_norm_gate for several packed sequences with
    old and fresh slots against the token-by-token float64 recurrence."""
    from llmq_amd import ops

    device, dtype = target[0], getattr(torch, target[1])
    g = torch.Generator().manual_seed(D * 7 + DV)
    lens, slots, fresh = [70, 21, 2, 1], [3, 0, 5, 1], [1, 0, 0, 1]
    T = sum(lens)
    q = torch.randn(T, H, D, generator=g).to(dtype)
    k = torch.randn(T, H, D, generator=g).to(dtype)
    v = torch.randn(T, H, DV, generator=g).to(dtype)
    z = (2 * torch.randn(T, H, D, generator=g)).to(dtype)
    zb = torch.randn(H * D, generator=g)
    state0 = torch.randn(6, H, D, DV, generator=g)
    w = (1 + 0.2 * torch.randn(DV, generator=g)).to(dtype)
    gate = torch.randn(T, H * DV, generator=g).to(dtype)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    st = state0.clone().to(device)
    o = ops.gla_recurrence(q.to(device), k.to(device), v.to(device), z.to(device), zb.to(device),
                           st, cu.to(device), torch.tensor(slots, dtype=torch.int32, device=device),
                           torch.tensor(fresh, dtype=torch.int32, device=device), tau)
    y = ops.gla_out_norm_gate(o, w.to(device), gate.to(device), 1e-5, dtype)
    alpha = torch.sigmoid(z.double() + zb.double().view(1, H, D)).pow(1.0 / tau)
    want_o = torch.empty(T, H, DV, dtype=torch.float64)
    want_state = state0.double().clone()
    at = 0
    for n, slot, fr in zip(lens, slots, fresh):
        S = torch.zeros(H, D, DV, dtype=torch.float64) if fr else state0[slot].double().clone()
        for t in range(at, at + n):
            S = alpha[t].unsqueeze(-1) * S + k[t].double().unsqueeze(-1) * v[t].double().unsqueeze(-2)
            want_o[t] = torch.einsum("hdv,hd->hv", S, q[t].double() * D ** -0.5)
        want_state[slot] = S
        at += n
    assert float((o.double().cpu() - want_o).abs().max() / want_o.abs().max()) < 1e-5
    assert float((st.double().cpu() - want_state).abs().max() / want_state.abs().max()) < 1e-5
    want_y = oracle.plain_rmsnorm(want_o, w.double(), 1e-5).reshape(T, H * DV) * \
        torch.nn.functional.silu(gate.double())
    err = float((y.double().cpu() - want_y).abs().max() / want_y.abs().max())
    assert err < (1e-2 if dtype == torch.bfloat16 else 1e-5), err

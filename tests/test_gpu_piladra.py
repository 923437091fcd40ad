"""The looped pre-norm hybrid decoder (Piladra: grouped norms, a causal convolution in front of every sublayer, gated latent
attention, a selective-scan layer, windowed attention with a sink and normed values, experts weighted on their input, a run
of layers repeated with the same weights) on the GPU against the plain restatement in tests/piladra_oracle.py: small
configurations and random weights made here, the engine's own step function, cache, state slots and kernels on one side,
whole-sequence float64 arithmetic on the other.

fp32 engines are held to 2e-4 of the largest reference value (the sharp test); bf16 engines to the rounding of a 16-bit
product chain.  Where random weights would hide a fault the inputs are built so that it shows: one key whose score stands far
above all others just inside and just outside a window, a sink that takes most of a softmax, state rows that still hold their
last owner's state.
"""
from __future__ import annotations

import json

import pytest
import torch

import piladra_oracle as O
from test_gpu_hybrid import alone, rel, replay, tokens_of

pytestmark = pytest.mark.gpu

FP32_TOL = 2e-4
BF16_TOL = 6e-2


# ----------------------------------------------------------------------------------------- configurations
def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=24, shared=40):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def lat(heads=3, dim=12, rot_dim=8, vdim=20, kv_rank=24, base=10000.0, scale=0.2, mlp=None):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "rot": {"base": base, "dims": rot_dim}}}


SCALING = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}


def att(heads=4, kv_heads=2, dim=16, vdim=12, dims=8, base=500.0, scale=0.3, window=9, scaling=SCALING, mlp=None):
    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = scaling
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if window:
        m["mask"] = {"size": window}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def mam(inner=40, state=12, dt_rank=5, conv=3, mlp=None):
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}, "mlp": mlp}


def config(layers, width=48, vocab=80, eps=1e-5, groups=3, taps=3, mult=0.6, cap=8.0, loop=None):
    cfg = {"architecture": "Piladra", "layers": layers, "norm": {"eps": eps, "groups": groups}, "residual_mult": mult, "vocab": vocab,
           "width": width}
    if taps:
        cfg["canon"] = {"taps": taps}
    if cap:
        cfg["logit_softcap"] = cap
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


FULL = config([mam(mlp=dense()), att(mlp=moe()), lat(mlp=dense(ff=40)), att(heads=6, kv_heads=1, dim=8, vdim=8, dims=4, window=20, mlp=None),
               mam(inner=24, state=16, dt_rank=3, conv=4, mlp=moe(experts=4, top=1, ff=16, shared=0))], loop=(1, 4, 2))


# ----------------------------------------------------------------------------------------- harness
_ENGINES: dict = {}


def engine_for(cfg_json, dtype, max_tokens=512, rows=4, page_size=16, graphs=None, seed=5):
    """(engine, checkpoint-named weights on the host) for a configuration; engines are kept for the session."""
    from mini_sglang_amd.engine import Engine, EngineConfig
    from mini_sglang_amd.hybrid import piladra_config

    key = (json.dumps(cfg_json, sort_keys=True), dtype, max_tokens, rows, page_size, tuple(graphs or ()), seed)
    if key not in _ENGINES:
        pages = max_tokens // page_size
        eng = Engine(EngineConfig(model=piladra_config(cfg_json), dtype=dtype, max_running_req=rows, page_size=page_size,
                                  num_page_override=pages, max_seq_len_override=pages * page_size, cuda_graph_bs=list(graphs or []),
                                  gemm_tune="off", refine_in_graph=False, seed=seed), torch.device("cuda:0"))
        _ENGINES[key] = (eng, eng.model.export_state())
    return _ENGINES[key]


def check(eng_state, cfg_json, steps, seqs, tol, allow=0.0):
    """Every position of every request within `tol` of the restatement (`allow`: the share of positions that may miss it: 16-bit
    runs only, where a router choice that rests on a close call flips under rounding)."""
    eng, state = eng_state
    got = replay(eng, steps)
    for rid, toks in seqs.items():
        ref = O.forward(cfg_json, state, toks)[0]
        assert got[rid].shape == ref.shape
        per = (got[rid] - ref).abs().amax(1) / ref.abs().max()
        bad = (per > tol).nonzero().flatten().tolist()
        assert len(bad) <= allow * len(toks), f"request {rid}: {len(bad)} of {len(toks)} positions above {tol} " \
                                              f"(worst {float(per.max()):.3e}, first at {bad[0]})"
    return got


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


# ----------------------------------------------------------------------------------------- each mechanism alone
@pytest.mark.parametrize("layer", [
    lat(), lat(heads=1, dim=8, rot_dim=16, vdim=8, kv_rank=24), lat(heads=5, dim=10, rot_dim=6, vdim=14, kv_rank=20, base=500.0),
    lat(heads=18, dim=8, rot_dim=2, vdim=8, kv_rank=16),
    att(), att(heads=3, kv_heads=3, dim=10, vdim=6, dims=10, scaling=None), att(heads=6, kv_heads=2, dim=8, vdim=72, dims=0, window=0),
    att(heads=1, kv_heads=1, dim=40, vdim=8, dims=2, scale=1.0, window=1), att(heads=34, kv_heads=1, dim=8, vdim=8, dims=4, window=64),
    att(window=200, base=2.0, scaling={"factor": 16.0, "low": 2.0, "high": 3.0, "original": 20}),
    mam(), mam(inner=24, state=16, dt_rank=1, conv=1), mam(inner=300, state=7, dt_rank=9, conv=2), mam(inner=16, state=40, conv=6),
    mam(inner=8, state=72, dt_rank=2, conv=4),
], ids=["latent", "latent-one-head", "latent-odd-sizes", "latent-many-heads", "attention", "attention-ungrouped-unscaled",
        "attention-wide-v-no-rotation-no-window", "attention-one-head-window-1", "attention-34-per-key-head", "attention-wide-window-other-ramp",
        "scan", "scan-16-one-tap", "scan-wide-7", "scan-40-six-taps", "scan-72"])
def test_mixer_alone_fp32(layer):
    cfg = config([layer])
    toks = tokens_of(70, cfg["vocab"], 1)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [70]), {"a": toks}, FP32_TOL)


@pytest.mark.parametrize("mlp", [dense(), dense(ff=300), moe(), moe(experts=4, top=1, shared=0), moe(experts=5, top=5, ff=8, shared=16),
                                 moe(experts=70, top=3, ff=8, shared=8), None],
                         ids=["dense", "dense-wide", "experts", "top-1-no-shared", "all-experts", "70-experts", "none"])
def test_feed_forward_alone_fp32(mlp):
    cfg = config([lat(heads=1, dim=4, rot_dim=2, vdim=4, kv_rank=4, mlp=mlp)])
    toks = tokens_of(50, cfg["vocab"], 2)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [50]), {"a": toks}, FP32_TOL)


@pytest.mark.parametrize("kw", [dict(groups=1), dict(groups=16), dict(taps=0), dict(taps=1), dict(taps=2), dict(taps=6), dict(mult=1.0, cap=0),
                                dict(cap=0.5), dict(width=40, groups=5, eps=1e-2)],
                         ids=["one-group", "16-groups", "no-conv", "one-tap", "two-taps", "six-taps", "no-multiplier-no-cap", "tight-cap", "width-40"])
def test_stream_variants_fp32(kw):
    """Norm groups, taps of the input convolution (none, one: no state, more than a short portion holds), the residual multiplier
    and the cap of the logits; cut into portions so that the convolution's inputs come from the state rows as well."""
    cfg = config([mam(mlp=dense()), att(mlp=moe())], **kw)
    toks = tokens_of(40, cfg["vocab"], 3)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [1, 2, 7, 1, 29]), {"a": toks}, FP32_TOL)


@pytest.mark.parametrize("loop", [None, (0, 3, 1), (0, 3, 3), (1, 2, 4), (2, 2, 5), (2, 3, 2)],
                         ids=["none", "once", "all-thrice", "middle-four-times", "empty-run", "last-twice"])
def test_loops_fp32(loop):
    """A run of layers repeated with the same weights: every pass has cache rows and state of its own and adds its own vector."""
    cfg = config([att(mlp=dense()), mam(mlp=None), lat(mlp=moe())], loop=loop)
    toks = tokens_of(45, cfg["vocab"], 4)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [30, 1, 14]), {"a": toks}, FP32_TOL)


def test_layer_outputs_fp32():
    """The residual stream after every layer run, not only the logits."""
    eng, state = engine_for(FULL, torch.float32)
    toks = tokens_of(40, FULL["vocab"], 3)
    mine: list = []
    orig = eng.model.forward
    eng.model.forward = lambda ctx, b, logits_out=None: orig(ctx, b, logits_out, layer_outputs=mine)
    try:
        replay(eng, alone("a", toks, [40]))
    finally:
        eng.model.forward = orig
    ref = O.forward(FULL, state, toks)[1]
    assert len(mine) == ref.shape[0] == 1 + 2 * 3 + 1
    for i, a in enumerate(mine):
        assert rel(a.double().cpu(), ref[i]) < FP32_TOL, f"layer run {i}"


def test_sinks_gates_and_steps_matter_fp32():
    """Weights set so that a dropped term shows: sinks of +4 (most of every softmax) and -9 (next to nothing), loop vectors and
    convolution taps of size one, a latent gate far from one half."""
    cfg = config([att(mlp=dense()), lat(mlp=moe(top=1))], loop=(0, 2, 2))
    eng, state = engine_for(cfg, torch.float32, seed=6)
    state = {k: v.clone() for k, v in state.items()}
    state["l0.mix.sink"] = torch.tensor([4.0, -9.0, 0.5, 2.0])
    state["loop.step"] = torch.stack([torch.linspace(-1.0, 1.0, 48), torch.linspace(2.0, -2.0, 48)])
    state["l0.canon1"], state["l1.canon2"] = torch.ones(48, 3), -torch.ones(48, 3)
    state["l1.mix.g"] = state["l1.mix.g"] * 30.0
    eng.model.load_state(state)  # this engine (its own seed) serves no other test
    toks = tokens_of(45, cfg["vocab"], 13)
    got = check((eng, eng.model.export_state()), cfg, alone("a", toks, [20, 1, 24]), {"a": toks}, FP32_TOL)["a"]
    for name, val in (("l0.mix.sink", torch.full((4,), -30.0)), ("loop.step", torch.zeros(2, 48)), ("l0.canon1", torch.zeros(48, 3)),
                      ("l1.canon2", torch.zeros(48, 3)), ("l1.mix.g", torch.zeros_like(state["l1.mix.g"]))):
        other = dict(state)
        other[name] = val
        assert rel(O.forward(cfg, other, toks)[0], got) > 20 * FP32_TOL, name  # the restatement itself moves when the term goes


def test_expert_weight_is_inside_the_expert_fp32():
    """Scores far from one: an engine that weighted the experts' outputs instead of their inputs would miss by far more than the tolerance."""
    cfg = config([lat(heads=1, dim=4, rot_dim=2, vdim=4, kv_rank=4, mlp=moe(experts=3, top=2, ff=32, shared=0))], mult=1.0)
    eng, state = engine_for(cfg, torch.float32, seed=8)
    state = {k: v.clone() for k, v in state.items()}
    state["l0.mlp.router"] = state["l0.mlp.router"] * 0.05 - 0.0  # scores near one half
    for e in range(3):
        state[f"l0.mlp.e{e}.gate"] = state[f"l0.mlp.e{e}.gate"] * 6.0  # a strongly non-linear expert
    eng.model.load_state(state)
    toks = tokens_of(30, cfg["vocab"], 17)
    check((eng, eng.model.export_state()), cfg, alone("a", toks, [30]), {"a": toks}, FP32_TOL)


# ----------------------------------------------------------------------------------------- kernels on built inputs
def _paged(dev, T, k, v, dtype, g):
    slots = torch.randperm(1024, generator=g)[:T].to(torch.int32)
    table = torch.zeros((3, 640), dtype=torch.int32)
    table[2, :T] = slots
    kc = torch.zeros((1024, k[0].numel()), dtype=dtype, device=dev)
    vc = torch.zeros((1024, v[0].numel()), dtype=dtype, device=dev)
    kc[slots.long().to(dev)] = k.reshape(T, -1).to(dtype).to(dev)
    vc[slots.long().to(dev)] = v.reshape(T, -1).to(dtype).to(dev)
    return table.to(dev), kc, vc


def _pieces(T, cut, singles):
    end = min(T, cut + singles)
    return [(0, cut)] + [(t, t + 1) for t in range(cut, end)] + ([(end, T)] if end < T else [])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("splits", [1, 3], ids=["one-range", "three-ranges"])
@pytest.mark.parametrize("loud,window", [(0, 0), (15, 64), (16, 17), (63, 64), (64, 65), (100, 1), (255, 96), (256, 40), (299, 300), (200, 0)])
def test_window_attention_one_loud_key(dev, dtype, splits, loud, window):
    """One key scores far above all others: every query that still sees it (the last: `window - 1` tokens later) returns its value,
    the next query returns something else.  The sequence is a prompt portion, then single decoded tokens, then a second portion, on
    slots scattered over the pool, so the window's edge falls inside a portion for some cases and among decoded tokens for others;
    the keys of a step in one range and cut into three; one head has a sink that outweighs ordinary keys."""
    from mini_sglang_amd import mixops

    H, G, d, dv, scale = 6, 2, 16, 24, 0.5
    T = 420
    g = torch.Generator().manual_seed(loud)
    q = torch.randn(T, H, d, generator=g, dtype=torch.float64) * 0.3
    k = torch.randn(T, G, d, generator=g, dtype=torch.float64) * 0.3
    v = torch.randn(T, G, dv, generator=g, dtype=torch.float64)
    sink = torch.tensor([-30.0, 3.0, 0.0, -2.0, 1.0, -30.0], dtype=torch.float64)
    k[:, :, 0] = 0.0
    k[loud, :, 0] = 12.0
    q[:, :, 0] = 5.0  # the loud key scores 30 with every query, 24 above the sink of head 1
    q, k, v = (t.to(dtype).double() for t in (q, k, v))
    ref = O.windowed_sink_softmax(q, k, v, scale, window, sink)
    table, kc, vc = _paged(dev, T, k, v, dtype, g)
    got = torch.empty((T, H * dv), dtype=dtype, device=dev)
    qd = q.reshape(T, -1).float().to(dev)
    for lo, hi in _pieces(T, 290, 40):
        part = torch.empty((hi - lo, H * dv + 8), dtype=dtype, device=dev)[:, : H * dv]  # a view with a row stride
        mixops.sink_attn(part, qd[lo:hi].contiguous(), kc, vc, table, torch.tensor([2], dtype=torch.int32, device=dev),
                         torch.tensor([hi], dtype=torch.int32, device=dev), torch.tensor([0, hi - lo], dtype=torch.int32, device=dev),
                         1, H, G, d, dv, scale, window, sink.float().to(dev), splits=splits)
        got[lo:hi] = part
    got = got.double().cpu().view(T, H, dv)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert float((got - ref).abs().max()) < tol * float(ref.abs().max())
    want = v[loud].repeat_interleave(H // G, 0)
    last = T - 1 if window == 0 else min(T - 1, loud + window - 1)
    for t in {loud, min(loud + 1, last), last}:
        assert float((got[t] - want).abs().max()) < 2e-2 * float(want.abs().max()) + 1e-3, t
    if last + 1 < T:
        assert float((got[last + 1] - want).abs().max()) > 0.2 * float(want.abs().max()), "the key just outside the window was read"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_window_attention_sinks_and_batches(dev, dtype):
    """Sinks from far below every score to far above, three requests of unequal length in one launch (a portion that continues a
    cached prefix, a fresh prompt, one decoded token), head sizes off every tile."""
    from mini_sglang_amd import mixops

    H, G, d, dv, scale, window = 3, 3, 20, 40, 0.4, 33
    g = torch.Generator().manual_seed(5)
    sink = torch.tensor([12.0, -40.0, 0.5], dtype=torch.float64)
    lens, new = [150, 47, 90], [60, 47, 1]
    seqs = [(torch.randn(n, H, d, generator=g, dtype=torch.float64).to(dtype).double(),
             torch.randn(n, G, d, generator=g, dtype=torch.float64).to(dtype).double(),
             torch.randn(n, G, dv, generator=g, dtype=torch.float64).to(dtype).double()) for n in lens]
    kc = torch.zeros((1024, G * d), dtype=dtype, device=dev)
    vc = torch.zeros((1024, G * dv), dtype=dtype, device=dev)
    table = torch.zeros((4, 256), dtype=torch.int32)
    perm = torch.randperm(1024, generator=g).to(torch.int32)
    at = 0
    for b, (_, k, v) in enumerate(seqs):
        sl = perm[at: at + lens[b]]
        at += lens[b]
        table[b + 1, : lens[b]] = sl
        kc[sl.long().to(dev)] = k.reshape(lens[b], -1).to(dtype).to(dev)
        vc[sl.long().to(dev)] = v.reshape(lens[b], -1).to(dtype).to(dev)
    qd = torch.cat([q[n - m:].reshape(m, -1) for (q, _, _), n, m in zip(seqs, lens, new)]).float().to(dev)
    cu = torch.tensor([0, 60, 107, 108], dtype=torch.int32, device=dev)
    for splits in (1, 2):
        out = torch.empty((108, H * dv), dtype=dtype, device=dev)
        mixops.sink_attn(out, qd, kc, vc, table.to(dev), torch.tensor([1, 2, 3], dtype=torch.int32, device=dev),
                         torch.tensor(lens, dtype=torch.int32, device=dev), cu, 3, H, G, d, dv, scale, window, sink.float().to(dev), splits=splits)
        got, at = out.double().cpu().view(108, H, dv), 0
        for (q, k, v), n, m in zip(seqs, lens, new):
            ref = O.windowed_sink_softmax(q, k, v, scale, window, sink)[n - m:]
            for h in range(H):  # per head: the heads differ by orders of magnitude
                assert float((got[at: at + m, h] - ref[:, h]).abs().max()) < (1e-5 if dtype == torch.float32 else 2e-2) * float(ref[:, h].abs().max()), h
            at += m
        assert float(got[:, 0].abs().max()) < 1e-2 * float(got[:, 1].abs().max())


@pytest.mark.parametrize("H,G,d,dv", [(4, 4, 32, 32), (8, 2, 64, 64), (6, 3, 48, 40), (3, 1, 96, 80), (16, 2, 128, 128), (2, 1, 192, 104), (8, 1, 256, 256),
                                      (5, 5, 72, 136)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_window_attention_head_sizes(dev, dtype, H, G, d, dv):
    """Every matrix-core instance (and the plain kernel beside it): head sizes from 32 to 256, one to eight query heads per key head,
    a window that ends inside a tile, a portion after a cached prefix and single tokens, keys in one range and in two."""
    from mini_sglang_amd import mixops

    T, window, scale = 150, 45, d ** -0.5
    g = torch.Generator().manual_seed(d + dv)
    q, k, v = (torch.randn(T, n, w, generator=g, dtype=torch.float64).to(dtype).double() for n, w in ((H, d), (G, d), (G, dv)))
    sink = torch.randn(H, generator=g, dtype=torch.float64)
    ref = O.windowed_sink_softmax(q, k, v, scale, window, sink)
    table, kc, vc = _paged(dev, T, k, v, dtype, g)
    qd = q.reshape(T, -1).float().to(dev)
    for splits in (1, 2):
        got = torch.empty((T, H * dv), dtype=dtype, device=dev)
        for lo, hi in _pieces(T, 70, 30):
            part = torch.empty((hi - lo, H * dv), dtype=dtype, device=dev)
            mixops.sink_attn(part, qd[lo:hi].contiguous(), kc, vc, table, torch.tensor([2], dtype=torch.int32, device=dev),
                             torch.tensor([hi], dtype=torch.int32, device=dev), torch.tensor([0, hi - lo], dtype=torch.int32, device=dev),
                             1, H, G, d, dv, scale, window, sink.float().to(dev), splits=splits)
            got[lo:hi] = part
        assert rel(got.double().cpu().view(T, H, dv), ref) < (1e-5 if dtype == torch.float32 else 2e-2), splits


@pytest.mark.parametrize("chunk", [0, 1, 5], ids=["whole", "chunks-of-1", "chunks-of-5"])
def test_selective_scan_kernel_state_slots_and_cuts(dev, chunk):
    """The recurrence kernel alone: two requests in one launch on state rows that hold garbage, then continued in a second
    launch; whole portions, and portions cut into pieces that run in parallel and are joined by the scan; inputs as row views."""
    from mini_sglang_amd import mixops

    for C, N in ((40, 12), (300, 16), (9, 33), (20, 70)):
        g = torch.Generator().manual_seed(N)
        lens = [23, 9]
        seq = {b: {k: torch.randn(n, w, generator=g, dtype=torch.float64) for k, w in (("x", C), ("z", C), ("dt", C), ("B", N), ("C", N))}
               for b, n in enumerate(lens)}
        A = -torch.exp(torch.randn(C, N, generator=g, dtype=torch.float64) * 0.5)
        dtb, D = torch.randn(C, generator=g, dtype=torch.float64) * 0.5, torch.randn(C, generator=g, dtype=torch.float64)
        state = torch.randn((3, C, N), generator=g, dtype=torch.float32).to(dev)  # garbage: a fresh request must not read it
        outs = {b: [] for b in seq}
        for lo, hi in ((0.0, 0.6), (0.6, 1.0)):
            cuts = {b: (int(lo * n), int(hi * n)) for b, n in enumerate(lens)}
            wide = torch.cat([torch.cat([seq[b][n][s:e] for n in ("x", "z", "dt", "B", "C")], 1) for b, (s, e) in cuts.items()]).float().to(dev)
            x, z, dt_in, bc = wide[:, :C], wide[:, C: 2 * C], wide[:, 2 * C: 3 * C], wide[:, 3 * C:]
            cu = torch.tensor([0, cuts[0][1] - cuts[0][0], wide.shape[0]], dtype=torch.int32, device=dev)
            chunks = None
            if chunk:
                items, firsts = [], [0]
                for bb, (s0, e0) in cuts.items():
                    items += [[bb, c, min(c + chunk, e0 - s0)] for c in range(0, e0 - s0, chunk)]
                    firsts.append(len(items))
                chunks = (torch.tensor(items, dtype=torch.int32, device=dev).view(-1), torch.tensor(firsts, dtype=torch.int32, device=dev),
                          len(items))
            out = mixops.selective_scan(x, z, dt_in, bc, A.float().to(dev), dtb.float().to(dev), D.float().to(dev), state, cu,
                                        torch.tensor([cuts[0][1], cuts[1][1]], dtype=torch.int32, device=dev),
                                        torch.tensor([2, 0], dtype=torch.int32, device=dev), 2, chunks=chunks)
            outs[0].append(out[: cu[1]].cpu())
            outs[1].append(out[cu[1]:].cpu())
        for b, n in enumerate(lens):
            s = seq[b]
            y, S = O.selective_scan(s["x"], O.softplus(s["dt"] + dtb), A, s["B"], s["C"], D)
            assert rel(torch.cat(outs[b]).double(), y * O.silu(s["z"])) < 1e-5, (C, N, b)
            assert rel(state[[2, 0][b]].double().cpu(), S) < 1e-5, (C, N, b)


@pytest.mark.parametrize("taps,groups", [(3, 2), (1, 1), (4, 7), (2, 56)])
def test_norm_conv_kernel_state_rows_and_cuts(dev, taps, groups):
    """The sum + grouped norm + input convolution kernel alone: two requests in one launch on state rows that hold garbage, continued
    over several launches with portions of one and two tokens (shorter than the taps), two sets of parts, a vector added to the sum."""
    from mini_sglang_amd import mixops

    W, mult, eps = 56, 0.7, 1e-3
    g = torch.Generator().manual_seed(taps)
    lens = [19, 11]
    xs = [torch.randn(n, W, generator=g, dtype=torch.float64) for n in lens]
    y0 = [torch.randn(n, 2, W, generator=g, dtype=torch.float64) for n in lens]
    y1 = [torch.randn(n, W, generator=g, dtype=torch.float64) for n in lens]
    add, w, tp = (torch.randn(s, generator=g, dtype=torch.float64) for s in ((W,), (W,), (W, taps)))
    state = torch.randn((3, max(taps - 1, 1), W), generator=g, dtype=torch.float32).to(dev)
    got = {0: [], 1: []}
    sums = {0: [], 1: []}
    for cuts in (((0, 1), (0, 2)), ((1, 3), (2, 3)), ((3, 4), (3, 10)), ((4, 19), (10, 11))):
        cat = lambda ts: torch.cat([t[s:e] for t, (s, e) in zip(ts, cuts)]).float().to(dev).contiguous()  # noqa: E731
        x, a, b = cat(xs), cat(y0), cat(y1)
        n0, n1 = cuts[0][1] - cuts[0][0], cuts[1][1] - cuts[1][0]
        h = torch.empty((n0 + n1, W), dtype=torch.float32, device=dev)
        x_out = torch.empty_like(x)
        staging = torch.empty((2, taps - 1, W), dtype=torch.float32, device=dev)
        kw = dict(state=state, staging=staging, cu_q=torch.tensor([0, n0, n0 + n1], dtype=torch.int32, device=dev),
                  seq_lens=torch.tensor([cuts[0][1], cuts[1][1]], dtype=torch.int32, device=dev),
                  req_rows=torch.tensor([2, 0], dtype=torch.int32, device=dev), batch=2) if taps > 1 else {}
        mixops.norm_conv(x, w.float().to(dev), eps, groups, h, parts=(a, b), mult=mult, add=add.float().to(dev), x_out=x_out,
                         taps=tp.float().to(dev).contiguous(), **kw)
        if taps > 1:
            mixops.commit_rows(state.view(1, 3, -1), staging.view(1, 2, -1), kw["req_rows"], 2, kw["cu_q"])
        got[0].append(h[:n0].cpu()), got[1].append(h[n0:].cpu())
        sums[0].append(x_out[:n0].cpu()), sums[1].append(x_out[n0:].cpu())
    for b in range(2):
        s = xs[b] + mult * (y0[b].sum(1) + y1[b]) + add
        ref = O.input_conv(O.group_norm(s, w, groups, eps), tp)
        assert rel(torch.cat(sums[b]).double(), s) < 1e-6, b
        assert rel(torch.cat(got[b]).double(), ref) < 1e-5, b


# ----------------------------------------------------------------------------------------- schedules
@pytest.mark.parametrize("dtype,tol", [(torch.float32, FP32_TOL), (torch.bfloat16, BF16_TOL)], ids=["fp32", "bf16"])
def test_whole_prompt(dtype, tol):
    toks = tokens_of(150, FULL["vocab"], 21)
    check(engine_for(FULL, dtype), FULL, alone("a", toks, [150]), {"a": toks}, tol, allow=0.05 if dtype == torch.bfloat16 else 0.0)


def test_prefill_against_token_by_token_fp32():
    eng = engine_for(FULL, torch.float32)
    toks = tokens_of(60, FULL["vocab"], 22)
    whole = check(eng, FULL, alone("a", toks, [60]), {"a": toks}, FP32_TOL)["a"]
    single = check(eng, FULL, alone("a", toks, [1]), {"a": toks}, FP32_TOL)["a"]
    assert rel(single, whole) < FP32_TOL


@pytest.mark.parametrize("sizes", [[2], [3, 1], [5, 2, 17], [16], [64, 1, 1, 2], [33, 31]],
                         ids=["twos", "3-1", "5-2-17", "pages", "64-then-short", "33-31"])
def test_portions_fp32(sizes):
    """Prompts cut anywhere: inside a page, a window, the taps of a convolution; portions down to two tokens and one."""
    toks = tokens_of(100, FULL["vocab"], 23)
    check(engine_for(FULL, torch.float32), FULL, alone("a", toks, sizes), {"a": toks}, FP32_TOL)


def test_long_portions_run_as_parallel_chunks_fp32():
    """Portions long enough that the scan runs as parallel pieces joined by a second launch, continued from a carried state, and the
    norm kernel walks several tokens per workgroup."""
    cfg = config([mam(mlp=dense()), att(window=150, mlp=None), mam(inner=24, state=16, dt_rank=3, conv=4, mlp=None)], loop=(0, 2, 2))
    toks = tokens_of(1300, cfg["vocab"], 24)
    eng = engine_for(cfg, torch.float32, max_tokens=1536)
    got = check(eng, cfg, alone("a", toks, [1100, 3, 197]), {"a": toks}, FP32_TOL)["a"]
    again = replay(eng[0], alone("a", toks, [150, 640, 510]))["a"]
    assert rel(again, got) < FP32_TOL


def test_long_decoding_fp32():
    """A short prompt, then 150 tokens one by one: the window passes over decoded tokens, the states are carried 150 times."""
    toks = tokens_of(170, FULL["vocab"], 25)
    check(engine_for(FULL, torch.float32), FULL, alone("a", toks, [20] + [1] * 150), {"a": toks}, FP32_TOL)


def test_first_tokens_fp32():
    """Sequences of one, two and three tokens: shorter than the taps, the windows and a page."""
    eng = engine_for(FULL, torch.float32)
    for n in (1, 2, 3):
        toks = tokens_of(n, FULL["vocab"], 30 + n)
        check(eng, FULL, alone("a", toks, [n]), {"a": toks}, FP32_TOL)
        check(eng, FULL, alone("a", toks, [1]), {"a": toks}, FP32_TOL)


def test_mixed_batches_against_each_alone_fp32():
    """Four requests of unequal length: portions of some beside single tokens of others, requests that sit out steps."""
    eng = engine_for(FULL, torch.float32)
    seqs = {r: tokens_of(n, FULL["vocab"], 40 + i) for i, (r, n) in enumerate((("a", 90), ("b", 37), ("c", 5), ("d", 61)))}
    a, b, c, d = (seqs[r] for r in "abcd")
    steps = [[("a", a[:50], False), ("b", b[:2], False)],
             [("a", a[50:51], False), ("b", b[2:30], False), ("c", c[:3], False)],
             [("d", d[:40], False), ("a", a[51:52], False), ("c", c[3:4], False)],
             [("a", a[52:88], False), ("b", b[30:], True), ("c", c[4:], True), ("d", d[40:41], False)],
             [("d", d[41:], True), ("a", a[88:], True)]]
    got = check(eng, FULL, steps, seqs, FP32_TOL)
    for r, toks in seqs.items():
        assert rel(replay(eng[0], alone(r, toks, [len(toks)]))[r], got[r]) < FP32_TOL, r


def test_pages_and_state_slots_used_again_fp32():
    """A pool of six pages and two request rows serving six requests in turn: every page and every state row is handed on with its
    last owner's contents."""
    eng = engine_for(FULL, torch.float32, max_tokens=96, rows=2)
    steps, seqs = [], {}
    for i in range(6):
        r, toks = f"r{i}", tokens_of(30 + 3 * i, FULL["vocab"], 50 + i)
        seqs[r] = toks
        steps += alone(r, toks, [17, 1, 40])
    check(eng, FULL, steps, seqs, FP32_TOL)


def test_other_orders_and_sizes_bf16():
    cfg = config([lat(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=64, mlp=moe(experts=8, top=2, ff=64, shared=64)),
                  mam(inner=128, state=16, dt_rank=8, conv=4, mlp=dense(ff=128)),
                  att(heads=8, kv_heads=2, dim=32, vdim=32, dims=16, window=40, mlp=dense(ff=96))], width=128, vocab=200, groups=4, loop=(1, 3, 2))
    a, b = tokens_of(140, 200, 61), tokens_of(33, 200, 62)
    steps = [[("a", a[:100], False)], [("a", a[100:101], False), ("b", b[:20], False)], [("a", a[101:], True), ("b", b[20:], True)]]
    check(engine_for(cfg, torch.bfloat16), cfg, steps, {"a": a, "b": b}, BF16_TOL, allow=0.05)


def test_wider_model_with_odd_head_sizes_bf16():
    """Head sizes, ranks and channel counts that are no powers of two, three key heads, two input taps, three norm groups, a run of two
    layers three times; two requests whose portions and single tokens share steps."""
    cfg = config([att(heads=6, kv_heads=3, dim=48, vdim=40, dims=24, window=33, mlp=moe(experts=5, top=3, ff=40, shared=24)),
                  mam(inner=384, state=8, dt_rank=6, conv=2, mlp=dense(ff=200)),
                  lat(heads=3, dim=48, rot_dim=32, vdim=56, kv_rank=80, mlp=None)], width=192, vocab=333, groups=3, taps=2, loop=(0, 2, 3))
    a, b = tokens_of(120, 333, 63), tokens_of(70, 333, 64)
    steps = [[("a", a[:64], False)], [("a", a[64:65], False), ("b", b[:50], False)], [("a", a[65:66], False), ("b", b[50:51], False)],
             [("a", a[66:], True), ("b", b[51:], True)]]
    check(engine_for(cfg, torch.bfloat16), cfg, steps, {"a": a, "b": b}, BF16_TOL, allow=0.05)
    check(engine_for(cfg, torch.float32), cfg, steps, {"a": a, "b": b}, FP32_TOL)


@pytest.mark.parametrize("graphs", [None, [1, 2, 4]], ids=["eager", "graphs"])
def test_greedy_generation_through_the_scheduler(graphs):
    """OfflineRunner.generate (chunked prefill with a small budget, continuous decode, the sampler's argmax, captured decode
    graphs) against greedy decoding with the restatement; a step whose two best logits are closer than the fp32 tolerance ends
    the comparison for that request."""
    from mini_sglang_amd.core import SamplingParams
    from mini_sglang_amd.offline import OfflineRunner

    eng, state = engine_for(FULL, torch.float32, max_tokens=512, graphs=graphs)
    prompts = [tokens_of(n, FULL["vocab"], 60 + n) for n in (9, 31, 47)]
    run = OfflineRunner(eng, max_extend_tokens=32, seed=2)
    n_new = 12
    run.generate(prompts, [SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True)] * len(prompts))
    compared = 0
    for p, st in zip(prompts, run.last_states):
        out = run.output_ids(st)
        assert len(out) == n_new
        seq = list(p)
        for tok in out:
            lg = O.forward(FULL, state, seq)[0][-1]
            top2 = lg.topk(2).values
            if float(top2[0] - top2[1]) < 1e-3 * float(lg.abs().max()):
                break
            assert tok == int(lg.argmax()), (len(seq), tok)
            seq.append(tok)
            compared += 1
    assert compared >= 2 * n_new


def test_trace_command_line(tmp_path):
    """bin/trace_run end to end in its own process on a checkpoint folder written here: the model class comes from config.json."""
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np
    from safetensors.torch import save_file

    from mini_sglang_amd.hybrid import HybridDecoder, piladra_config

    cfg = config([att(heads=3, kv_heads=1, dim=10, vdim=14, dims=4, window=12, mlp=moe(experts=5, top=2, ff=20, shared=12)),
                  mam(inner=30, state=11, dt_rank=4, conv=3, mlp=dense(ff=44)),
                  lat(heads=2, dim=5, rot_dim=6, vdim=7, kv_rank=18)], width=100, vocab=131, groups=5, taps=2, loop=(0, 2, 2))
    model = HybridDecoder(piladra_config(cfg), dtype=torch.bfloat16, device=torch.device("cpu"), seed=9)
    state = {k: (v.to(torch.bfloat16) if v.is_floating_point() else v) for k, v in model.export_state().items()}
    mdir, out = tmp_path / "model", tmp_path / "out"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(cfg))
    save_file(state, str(mdir / "model.safetensors"))
    a, b = tokens_of(45, cfg["vocab"], 70), tokens_of(9, cfg["vocab"], 71)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:8], "want": []}, {"id": "a", "tokens": a[30:31], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[31:], "want": [13]}, {"id": "b", "tokens": b[8:], "want": [0]}], "end": ["a", "b"]}]
    root = Path(__file__).resolve().parent.parent
    pr = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(mdir), "--dtype", "float32", "--out", str(out),
                         "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n", text=True, capture_output=True,
                        timeout=110)
    assert pr.returncode == 0, pr.stderr[-2000:]
    assert [ln for ln in pr.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    ra, rb = O.forward(cfg, state, a)[0], O.forward(cfg, state, b)[0]
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)).double()
    got1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1)).double()
    got2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1)).double()
    scale = float(ra.abs().max())
    assert float((got0 - ra[[0, 29]]).abs().max()) < FP32_TOL * scale
    assert float((got1 - ra[[30]]).abs().max()) < FP32_TOL * scale
    assert float((got2[0] - ra[44]).abs().max()) < FP32_TOL * scale and float((got2[1] - rb[8]).abs().max()) < FP32_TOL * scale

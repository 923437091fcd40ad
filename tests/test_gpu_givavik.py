"""The parallel-residual hybrid decoder (Givavik: one norm per layer feeding a token-shifted mixer and a feed-forward side by
side; latent attention with a sink, sigmoid attention beside a state-space layer, a pair embedding) on the GPU against the
plain restatement in tests/givavik_oracle.py: small configurations and random weights made here, the engine's own step
function, cache, state slots and kernels on one side, whole-sequence float64 arithmetic on the other.

fp32 engines are held to 2e-4 of the largest reference value (the sharp test); bf16 engines to the rounding of a 16-bit
product chain.  Where random weights would hide a fault the inputs are built so that it shows: one key far back whose weight
is (nearly) one while every other key's is (nearly) zero, a sink that takes most of a softmax, state rows that still hold
their last owner's state.
"""
from __future__ import annotations

import json
import math

import pytest
import torch

import givavik_oracle as O
from test_gpu_hybrid import alone, rel, replay, tokens_of

pytestmark = pytest.mark.gpu

FP32_TOL = 2e-4
BF16_TOL = 6e-2


# ----------------------------------------------------------------------------------------- configurations
def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def lat(heads=3, dim=12, rot_dim=8, vdim=20, kv_rank=24, kv_from=None, base=10000.0, scale=0.2, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def pair(heads=4, kv_heads=2, dim=24, vdim=20, dims=10, base=10000.0, scale=0.4, softcap=5.0, s_heads=3, s_vdim=12, state=20, groups=1,
         conv=3, norm_groups=3, left_scale=0.8, right_scale=1.3, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
            "rot": {"base": base, "dims": dims}}
    right = {"heads": s_heads, "vdim": s_vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}, "mlp": mlp}


def config(layers, width=48, vocab=80, eps=1e-5, scale=3.0, bigram=(37, 5, 11)):
    e = {"scale": scale}
    if bigram:
        e["bigram"] = {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}
    return {"architecture": "Givavik", "embedding": e, "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


FULL = config([pair(mlp=dense()), lat(mlp=dense(ff=40)), pair(heads=6, kv_heads=2, dim=16, vdim=8, dims=16, s_heads=4, s_vdim=8, state=16,
                                                              groups=2, conv=4, norm_groups=1, mlp=None),
               lat(kv_from=1, heads=2, dim=16, vdim=12, mlp=dense()), lat(heads=4, dim=8, rot_dim=4, vdim=8, kv_rank=16, mlp=dense(ff=24)),
               lat(kv_from=4, heads=1, dim=4, rot_dim=4, vdim=24, kv_rank=16, mlp=None)])


# ----------------------------------------------------------------------------------------- harness
_ENGINES: dict = {}


def engine_for(cfg_json, dtype, max_tokens=512, rows=4, page_size=16, graphs=None, seed=5):
    """(engine, checkpoint-named weights on the host) for a configuration; engines are kept for the session."""
    from mini_sglang_amd.engine import Engine, EngineConfig
    from mini_sglang_amd.hybrid import givavik_config

    key = (json.dumps(cfg_json, sort_keys=True), dtype, max_tokens, rows, page_size, tuple(graphs or ()), seed)
    if key not in _ENGINES:
        pages = max_tokens // page_size
        eng = Engine(EngineConfig(model=givavik_config(cfg_json), dtype=dtype, max_running_req=rows, page_size=page_size,
                                  num_page_override=pages, max_seq_len_override=pages * page_size, cuda_graph_bs=list(graphs or []),
                                  gemm_tune="off", refine_in_graph=False, seed=seed), torch.device("cuda:0"))
        _ENGINES[key] = (eng, eng.model.export_state())
    return _ENGINES[key]


def check(eng_state, cfg_json, steps, seqs, tol, allow=0.0):
    """Every position of every request within `tol` of the restatement (`allow`: the share of positions that may miss it)."""
    eng, state = eng_state
    got = replay(eng, steps)
    for rid, toks in seqs.items():
        ref = O.forward(cfg_json, state, toks)
        assert got[rid].shape == ref.shape
        per = (got[rid] - ref).abs().amax(1) / ref.abs().max()
        bad = (per > tol).nonzero().flatten().tolist()
        assert len(bad) <= allow * len(toks), f"request {rid}: {len(bad)} of {len(toks)} positions above {tol} " \
                                              f"(worst {float(per.max()):.3e}, first at {bad[0]})"
    return got


# ----------------------------------------------------------------------------------------- each mechanism alone
@pytest.mark.parametrize("layer", [
    lat(), lat(heads=1, dim=8, rot_dim=16, vdim=8, kv_rank=24), lat(heads=5, dim=10, rot_dim=6, vdim=14, kv_rank=20, base=500.0),
    lat(heads=18, dim=8, rot_dim=2, vdim=8, kv_rank=16),
    pair(), pair(heads=3, kv_heads=3, dim=10, vdim=6, dims=10, softcap=0.0), pair(heads=6, kv_heads=2, dim=8, vdim=72, dims=0),
    pair(heads=1, kv_heads=1, dim=40, vdim=8, dims=2, scale=1.0, softcap=1.0), pair(heads=34, kv_heads=1, dim=8, vdim=8, dims=4),
    pair(s_heads=4, s_vdim=8, state=16, groups=4, norm_groups=1), pair(s_heads=2, s_vdim=72, state=32, groups=1, conv=1, norm_groups=2),
    pair(s_heads=1, s_vdim=8, state=64, conv=6, norm_groups=8), pair(s_heads=2, s_vdim=4, state=128, groups=2, conv=2, norm_groups=1),
    pair(s_heads=1, s_vdim=8, state=136, conv=2, norm_groups=1),
], ids=["latent", "latent-one-head", "latent-odd-sizes", "latent-many-heads", "pair", "pair-ungrouped-no-cap", "pair-wide-v-no-rotation",
        "pair-one-head", "pair-34-per-key-head", "state-16-grouped", "state-32-wide-p-one-tap", "state-64-six-taps", "state-128",
        "state-136"])
def test_mixer_alone_fp32(layer):
    cfg = config([layer])
    toks = tokens_of(70, cfg["vocab"], 1)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [70]), {"a": toks}, FP32_TOL)


@pytest.mark.parametrize("mlp", [dense(), dense(ff=300), None], ids=["dense", "dense-wide", "none"])
def test_feed_forward_alone_fp32(mlp):
    cfg = config([lat(heads=1, dim=4, rot_dim=2, vdim=4, kv_rank=4, mlp=mlp)])
    toks = tokens_of(50, cfg["vocab"], 2)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [50]), {"a": toks}, FP32_TOL)


@pytest.mark.parametrize("kw", [dict(bigram=None), dict(bigram=(1, 3, 7), scale=1.0), dict(bigram=(997, 1000003, 65537), scale=0.25),
                                dict(bigram=(80, 1, 0))], ids=["no-pairs", "one-bucket", "large-multipliers", "previous-token-only"])
def test_embedding_variants_fp32(kw):
    """The pair table with one bucket, with multipliers whose products pass 2^31, keyed by the previous token alone, and absent;
    cut into portions so that the previous token comes from the request's state row as well as from the same step."""
    cfg = config([lat(mlp=dense())], vocab=3000 if kw.get("bigram") and kw["bigram"][0] == 997 else 80, **kw)
    toks = tokens_of(40, cfg["vocab"], 3)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [1, 2, 7, 1, 29]), {"a": toks}, FP32_TOL)


def test_borrowed_keys_across_layers_fp32():
    """Layers that read another layer's cached rows with their own queries and up-projections, a pair layer between them."""
    cfg = config([lat(mlp=dense()), pair(), lat(kv_from=0, heads=2, dim=6, vdim=30), lat(kv_from=0, heads=5, dim=12, vdim=4, scale=1.0)])
    toks = tokens_of(60, cfg["vocab"], 11)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [31, 1, 28]), {"a": toks}, FP32_TOL)


def test_layer_outputs_fp32():
    """The residual stream after every layer, not only the logits."""
    eng, state = engine_for(FULL, torch.float32)
    toks = tokens_of(40, FULL["vocab"], 3)
    mine: list = []
    orig = eng.model.forward
    eng.model.forward = lambda ctx, b, logits_out=None: orig(ctx, b, logits_out, layer_outputs=mine)
    try:
        replay(eng, alone("a", toks, [40]))
    finally:
        eng.model.forward = orig
    ref: list = []
    O.forward(FULL, state, toks, layer_outputs=ref)
    assert len(mine) == len(ref) == len(FULL["layers"])
    for i, (a, b) in enumerate(zip(mine, ref)):
        assert rel(a.double().cpu(), b) < FP32_TOL, f"layer {i}"


def test_sink_and_layer_scales_matter_fp32():
    """Weights set so that a dropped term shows: sinks of +4 (most of every softmax) and -9 (next to nothing), layer scales and
    shifts far from their neutral values, an output bias of size one."""
    cfg = config([lat(mlp=dense()), pair(mlp=dense())])
    eng, state = engine_for(cfg, torch.float32, seed=6)
    state = {k: v.clone() for k, v in state.items()}
    state["l0.mix.sink"] = torch.tensor([4.0, -9.0, 0.5])
    state["l0.ls1"], state["l0.ls2"] = torch.full((48,), 2.5), torch.linspace(-1.0, 1.0, 48)
    state["l1.shift"], state["l0.shift"] = torch.linspace(-0.5, 1.5, 48), torch.ones(48)
    state["l1.mix.left.o.b"] = torch.ones(48)
    state["l1.mix.left.pb"] = torch.tensor([-3.0, 0.0, 2.0, -1.0])
    eng.model.load_state(state)  # this engine (its own seed) serves no other test
    toks = tokens_of(45, cfg["vocab"], 13)
    got = check((eng, eng.model.export_state()), cfg, alone("a", toks, [20, 1, 24]), {"a": toks}, FP32_TOL)["a"]
    for name, val in (("l0.mix.sink", torch.full((3,), -30.0)), ("l1.mix.left.o.b", torch.zeros(48)), ("l0.shift", torch.zeros(48))):
        other = dict(state)
        other[name] = val
        assert rel(O.forward(cfg, other, toks), got) > 20 * FP32_TOL, name  # the restatement itself moves when the term goes


# ----------------------------------------------------------------------------------------- kernels on built inputs
def _paged(dev, T, width_k, width_v, k, v, dtype, g):
    slots = torch.randperm(1024, generator=g)[:T].to(torch.int32)
    table = torch.zeros((3, 640), dtype=torch.int32)
    table[2, :T] = slots
    kc = torch.zeros((1024, width_k), dtype=dtype, device=dev)
    vc = torch.zeros((1024, width_v), dtype=dtype, device=dev)
    kc[slots.long().to(dev)] = k.reshape(T, -1).to(dtype).to(dev)
    vc[slots.long().to(dev)] = v.reshape(T, -1).to(dtype).to(dev)
    return table.to(dev), kc, vc


def _pieces(T, cut, singles):
    end = min(T, cut + singles)
    return [(0, cut)] + [(t, t + 1) for t in range(cut, end)] + ([(end, T)] if end < T else [])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("splits", [1, 3], ids=["one-range", "three-ranges"])
@pytest.mark.parametrize("loud", [0, 15, 16, 63, 64, 255, 256, 300])
def test_sigmoid_attention_one_far_key(dev, dtype, splits, loud):
    """Every key's weight is (nearly) zero except one key's, far back, at a page or tile border: each later query must return
    that key's value, each earlier one (nearly) nothing.  The sequence is a prompt portion, then single decoded tokens, then a
    second portion, on slots scattered over the pool; the keys of a step in one range and cut into three."""
    from mini_sglang_amd import mixops

    H, G, d, dv, scale, cap = 6, 2, 16, 24, 0.5, 30.0
    T = 420
    g = torch.Generator().manual_seed(loud)
    q = torch.randn(T, H, d, generator=g, dtype=torch.float64) * 0.3
    k = torch.randn(T, G, d, generator=g, dtype=torch.float64) * 0.3
    v = torch.randn(T, G, dv, generator=g, dtype=torch.float64)
    pb = torch.full((H,), -14.0, dtype=torch.float64)
    k[:, :, 0] = 0.0
    k[loud, :, 0] = 12.0
    q[:, :, 0] = 5.0  # the loud key scores 30 with every query, before the cap
    q, k, v = (t.to(dtype).double() for t in (q, k, v))
    ref = O.sigmoid_weighted_sum(q, k, v, pb, scale, cap) * 0.7
    table, kc, vc = _paged(dev, T, G * d, G * dv, k, v, dtype, g)
    got = torch.empty((T, H * dv), dtype=dtype, device=dev)
    qd = q.reshape(T, -1).float().to(dev)
    for lo, hi in _pieces(T, 290, 40):
        part = torch.empty((hi - lo, H * dv + 8), dtype=dtype, device=dev)[:, : H * dv]  # a view with a row stride
        mixops.sigmoid_attn(part, qd[lo:hi].contiguous(), kc, vc, table, torch.tensor([2], dtype=torch.int32, device=dev),
                            torch.tensor([hi], dtype=torch.int32, device=dev), torch.tensor([0, hi - lo], dtype=torch.int32, device=dev),
                            1, H, G, d, dv, scale, cap, pb.float().to(dev), out_scale=0.7, splits=splits)
        got[lo:hi] = part
    got = got.double().cpu().view(T, H, dv)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert float((got - ref).abs().max()) < tol * float(ref.abs().max())
    want = 0.7 * v[loud].repeat_interleave(H // G, 0)
    for t in (loud, loud + 1, 289, 290, 329, 330, T - 1):
        if loud <= t < T:
            assert float((got[t] - want).abs().max()) < 2e-2 * float(want.abs().max()) + 1e-3, t
    if loud:
        assert float(got[loud - 1].abs().max()) < 1e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("splits", [1, 3], ids=["one-range", "three-ranges"])
def test_latent_attention_sink(dev, dtype, splits):
    """The shared-key attention kernel with a sink per head: sinks far above every score (the output shrinks to a sliver), far
    below (no effect), and in between; key counts on both sides of the tile and page sizes; portions and single tokens."""
    from mini_sglang_amd import mixops

    H, R, r, scale = 5, 32, 8, 0.3
    T = 330
    g = torch.Generator().manual_seed(splits)
    qa = torch.randn(T, H, R + r, generator=g, dtype=torch.float64) * 0.5
    rows = torch.randn(T, R + r, generator=g, dtype=torch.float64)
    sink = torch.tensor([12.0, -40.0, 0.0, 2.5, -1.0], dtype=torch.float64)
    rows = rows.to(dtype).double()
    if dtype == torch.bfloat16:
        qa = qa.to(dtype).double()
    ref = torch.zeros(T, H, R, dtype=torch.float64)
    for h in range(H):
        for i in range(T):
            ref[i, h] = O.sink_softmax_rows((rows[: i + 1] @ qa[i, h]) * scale, rows[: i + 1, :R], float(sink[h]))
    table, cache, _ = _paged(dev, T, R + r, 1, rows, torch.zeros(T, 1), dtype, g)
    got = torch.empty((T, H, R), dtype=torch.float32, device=dev)
    for lo, hi in _pieces(T, 200, 70):
        part = torch.empty((hi - lo, H, R), dtype=torch.float32, device=dev)
        mixops.latent_attn(part, qa[lo:hi].float().to(dev).contiguous(), cache, table, torch.tensor([2], dtype=torch.int32, device=dev),
                           torch.tensor([hi], dtype=torch.int32, device=dev), torch.tensor([0, hi - lo], dtype=torch.int32, device=dev),
                           1, R, scale, splits=splits, sink=sink.float().to(dev))
        got[lo:hi] = part
    got = got.double().cpu()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for h in range(H):  # per head: the heads differ by orders of magnitude
        assert float((got[:, h] - ref[:, h]).abs().max()) < tol * float(ref[:, h].abs().max()), h
    assert float(ref[:, 0].abs().max()) < 1e-2 * float(ref[:, 1].abs().max())


@pytest.mark.parametrize("chunk", [0, 1, 5], ids=["whole", "chunks-of-1", "chunks-of-5"])
def test_state_space_kernel_state_slots_and_cuts(dev, chunk):
    """The recurrence kernel alone: two requests in one launch on state rows that hold garbage, then continued in a second
    launch; grouped B / C; whole portions, and portions cut into pieces that run in parallel and are joined by the scan."""
    from mini_sglang_amd import mixops

    for H, G, N, P in ((4, 2, 12, 20), (2, 1, 32, 70), (3, 3, 64, 8)):
        g = torch.Generator().manual_seed(N)
        lens = [23, 9]
        seq = {}
        for b, n in enumerate(lens):
            seq[b] = dict(x=torch.randn(n, H, P, generator=g, dtype=torch.float64), B=torch.randn(n, G, N, generator=g, dtype=torch.float64),
                          C=torch.randn(n, G, N, generator=g, dtype=torch.float64), dt=torch.randn(n, H, generator=g, dtype=torch.float64))
        A = torch.exp(torch.randn(H, generator=g, dtype=torch.float64) * 0.5)
        dtb, D = torch.randn(H, generator=g, dtype=torch.float64) * 0.5, torch.randn(H, generator=g, dtype=torch.float64)
        state = torch.randn((3, H, N, P), generator=g, dtype=torch.float32).to(dev)  # garbage: a fresh request must not read it
        outs = {b: [] for b in seq}
        for lo, hi in ((0.0, 0.6), (0.6, 1.0)):
            cuts = {b: (int(lo * n), int(hi * n)) for b, n in enumerate(lens)}
            xbc = torch.cat([torch.cat([seq[b][n][s:e].reshape(e - s, -1) for n in ("x", "B", "C")], 1) for b, (s, e) in cuts.items()])
            dt_raw = torch.cat([seq[b]["dt"][s:e] for b, (s, e) in cuts.items()]).float().to(dev)
            xbc = xbc.float().to(dev)
            cu = torch.tensor([0, cuts[0][1] - cuts[0][0], xbc.shape[0]], dtype=torch.int32, device=dev)
            out = torch.empty((xbc.shape[0], H * P), dtype=torch.float32, device=dev)
            chunks = None
            if chunk:
                items, firsts = [], [0]
                for bb, (s0, e0) in cuts.items():
                    items += [[bb, c, min(c + chunk, e0 - s0)] for c in range(0, e0 - s0, chunk)]
                    firsts.append(len(items))
                chunks = (torch.tensor(items, dtype=torch.int32, device=dev).view(-1), torch.tensor(firsts, dtype=torch.int32, device=dev),
                          len(items))
            mixops.ssd(out, xbc, dt_raw, state, (-A).float().to(dev), dtb.float().to(dev), D.float().to(dev), cu,
                       torch.tensor([cuts[0][1], cuts[1][1]], dtype=torch.int32, device=dev),
                       torch.tensor([2, 0], dtype=torch.int32, device=dev), 2, G, chunks=chunks)
            outs[0].append(out[: cu[1]].cpu())
            outs[1].append(out[cu[1]:].cpu())
        for b, n in enumerate(lens):
            s = seq[b]
            ref, S = O.state_space_scan(s["x"], s["B"], s["C"], O.softplus(s["dt"] + dtb), A, D)
            got = torch.cat(outs[b]).double().view(n, H, P)
            assert rel(got, ref) < 1e-5, (N, b)
            assert rel(state[[2, 0][b]].double().cpu(), S) < 1e-5, (N, b)


# ----------------------------------------------------------------------------------------- schedules
@pytest.mark.parametrize("dtype,tol", [(torch.float32, FP32_TOL), (torch.bfloat16, BF16_TOL)], ids=["fp32", "bf16"])
def test_whole_prompt(dtype, tol):
    toks = tokens_of(150, FULL["vocab"], 4)
    check(engine_for(FULL, dtype), FULL, alone("a", toks, [150]), {"a": toks}, tol)


def test_prefill_against_token_by_token_fp32():
    eng_state = engine_for(FULL, torch.float32)
    toks = tokens_of(90, FULL["vocab"], 5)
    whole = check(eng_state, FULL, alone("a", toks, [90]), {"a": toks}, FP32_TOL)["a"]
    single = check(eng_state, FULL, alone("a", toks, [1]), {"a": toks}, FP32_TOL)["a"]
    assert rel(single, whole) < 2e-5


@pytest.mark.parametrize("sizes", [[2], [3, 2, 5], [16], [15, 17], [64, 1, 63, 2], [33, 1, 1, 1, 7], [1, 2, 1, 3]])
def test_portions_fp32(sizes):
    """Portions shorter than the convolutions' reach (2, 1 and 3 tokens against up to 4 taps), ending at and next to page
    borders; the token before a portion comes from the request's state rows in every layer."""
    eng_state = engine_for(FULL, torch.float32)
    toks = tokens_of(131, FULL["vocab"], 6)
    check(eng_state, FULL, alone("a", toks, sizes), {"a": toks}, FP32_TOL)


def test_long_portions_run_as_parallel_chunks_fp32():
    """Portions long enough for the state-space layers to cut them into pieces (states joined by a scan): first a long portion
    from position 0, then a single token, then a long portion that continues from a carried state, beside a short request;
    lengths off the piece size."""
    eng_state = engine_for(FULL, torch.float32, max_tokens=2048)
    a, b = tokens_of(700, FULL["vocab"], 30), tokens_of(6, FULL["vocab"], 31)
    steps = [[("a", a[:300], False)], [("a", a[300:301], False), ("b", b[:5], False)], [("b", b[5:], True), ("a", a[301:], True)]]
    got = check(eng_state, FULL, steps, {"a": a, "b": b}, FP32_TOL)
    whole = replay(eng_state[0], alone("a", a, [257, 443]))["a"]
    assert rel(got["a"], whole) < 2e-5


def test_very_long_portion_against_shorter_ones_fp32():
    """A 2300-token portion (the norm-and-shift launch then walks two tokens per workgroup and keeps the row before in LDS)
    beside a short request, against the same tokens in portions that take the one-token-per-workgroup path."""
    eng, _ = engine_for(FULL, torch.float32, max_tokens=4096)
    a, b = tokens_of(2300, FULL["vocab"], 32), tokens_of(7, FULL["vocab"], 33)
    long = replay(eng, [[("b", b[:3], False), ("a", a, True)], [("b", b[3:], True)]])
    short = replay(eng, [[("a", a[:700], False)], [("a", a[700:1600], False), ("b", b, True)], [("a", a[1600:], True)]])
    assert rel(long["a"], short["a"]) < 2e-5 and rel(long["b"], short["b"]) < 2e-5


def test_long_decoding_fp32():
    """A short prompt, then 260 tokens one by one: keys far back stay visible, the states carry everything else."""
    cfg = config([pair(mlp=dense()), lat(mlp=None), pair(s_heads=2, s_vdim=20, state=12, norm_groups=2), lat(kv_from=1, mlp=dense())])
    toks = tokens_of(270, cfg["vocab"], 7)
    steps = [[("a", toks[:10], False)]] + [[("a", [t], j == 259)] for j, t in enumerate(toks[10:])]
    check(engine_for(cfg, torch.float32), cfg, steps, {"a": toks}, FP32_TOL)


def test_first_tokens_fp32():
    """Positions 0, 1, 2 of a sequence: a one-token request, and requests whose first portion is one or two tokens."""
    eng_state = engine_for(FULL, torch.float32)
    one = tokens_of(1, FULL["vocab"], 8)
    check(eng_state, FULL, alone("a", one, [1]), {"a": one}, FP32_TOL)
    toks = tokens_of(20, FULL["vocab"], 9)
    check(eng_state, FULL, alone("a", toks, [1, 2, 17]), {"a": toks}, FP32_TOL)
    check(eng_state, FULL, alone("a", toks, [2, 1, 17]), {"a": toks}, FP32_TOL)


def test_mixed_batches_against_each_alone_fp32():
    """Four unequal requests: portions of some beside single tokens of others, requests that sit out steps and that end
    while others go on.  Every request must come out as it does alone."""
    eng_state = engine_for(FULL, torch.float32, max_tokens=512)
    seqs = {i: tokens_of(n, FULL["vocab"], 20 + k) for k, (i, n) in enumerate([("a", 97), ("b", 40), ("c", 5), ("d", 130)])}
    at = {i: 0 for i in seqs}
    plan = [{"a": 30, "b": 1, "d": 64}, {"a": 1, "b": 17, "c": 2}, {"d": 2, "a": 1}, {"a": 33, "b": 1, "c": 3, "d": 1},
            {"b": 21, "d": 63}, {"a": 32}]
    steps = []
    for p in plan:
        step = []
        for i, c in p.items():
            t = seqs[i][at[i]: at[i] + c]
            at[i] += len(t)
            step.append((i, t, at[i] == len(seqs[i])))
        steps.append(step)
    assert all(at[i] == len(seqs[i]) for i in seqs)
    mixed = check(eng_state, FULL, steps, seqs, FP32_TOL)
    for i, toks in seqs.items():
        solo = replay(eng_state[0], alone(i, toks, [len(toks)]))[i]
        assert rel(mixed[i], solo) < 2e-5, i


def test_pages_and_state_slots_used_again_fp32():
    """A pool of 8 pages and two request rows: every request after the first runs on pages and on state rows (recurrent state,
    convolution inputs, the last normed row of every layer, the last token id) that still hold another request's."""
    cfg = config([pair(conv=4), lat(mlp=dense()), pair(s_heads=2, s_vdim=8, state=8, conv=3, norm_groups=2, mlp=dense()), lat(kv_from=1)])
    eng_state = engine_for(cfg, torch.float32, max_tokens=128, rows=2)
    seqs = {i: tokens_of(n, cfg["vocab"], 40 + k) for k, (i, n) in enumerate([("a", 60), ("b", 64), ("c", 50), ("d", 33), ("e", 64)])}
    steps = [[("a", seqs["a"][:40], False), ("b", seqs["b"][:30], False)],
             [("a", seqs["a"][40:], True), ("b", seqs["b"][30:], True)],
             [("c", seqs["c"][:2], False)],
             [("c", seqs["c"][2:], True), ("d", seqs["d"][:1], False)],
             [("d", seqs["d"][1:], True)],
             [("e", seqs["e"], True)]]
    check(eng_state, cfg, steps, seqs, FP32_TOL)


def test_other_orders_and_sizes_bf16():
    """Another order of layers, widths that are not powers of two, no feed-forward in a layer: the 16-bit path end to end."""
    cfg = config([lat(heads=2, dim=12, rot_dim=4, vdim=20, kv_rank=40, mlp=dense(ff=90)),
                  lat(kv_from=0, heads=3, dim=20, rot_dim=4, vdim=12, kv_rank=40),
                  pair(heads=4, kv_heads=4, dim=12, vdim=20, dims=12, s_heads=3, s_vdim=28, state=24, groups=3, norm_groups=1, mlp=dense()),
                  pair(heads=2, kv_heads=1, dim=40, vdim=12, dims=6, softcap=0.0, s_heads=2, s_vdim=10, state=10, conv=2, norm_groups=2)],
                 width=72, vocab=101, eps=1e-6, bigram=(13, 2, 9))
    toks = tokens_of(120, cfg["vocab"], 10)
    check(engine_for(cfg, torch.bfloat16), cfg, alone("a", toks, [50, 1, 1, 30, 2, 36]), {"a": toks}, BF16_TOL)


# ----------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("graphs", [None, [1, 2, 4]], ids=["eager", "graphs"])
def test_greedy_generation_through_the_scheduler(graphs):
    """OfflineRunner.generate (chunked prefill with a small budget, continuous decode, the sampler's argmax, captured
    decode graphs) against greedy decoding with the restatement; a step whose two best logits are closer than the fp32
    tolerance ends the comparison for that request."""
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
            lg = O.forward(FULL, state, seq)[-1]
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

    from mini_sglang_amd.hybrid import HybridDecoder, givavik_config

    cfg = config([lat(heads=3, dim=10, rot_dim=6, vdim=14, kv_rank=18, mlp=dense(ff=44)),
                  pair(heads=3, kv_heads=1, dim=10, vdim=14, dims=4, s_heads=2, s_vdim=9, state=11, conv=3, norm_groups=2, mlp=dense(ff=26)),
                  lat(kv_from=0, heads=2, dim=5, rot_dim=6, vdim=7, kv_rank=18)], width=100, vocab=131)
    model = HybridDecoder(givavik_config(cfg), dtype=torch.bfloat16, device=torch.device("cpu"), seed=9)
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
    ra, rb = O.forward(cfg, state, a), O.forward(cfg, state, b)
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)).double()
    got1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1)).double()
    got2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1)).double()
    scale = float(ra.abs().max())
    assert float((got0 - ra[[0, 29]]).abs().max()) < FP32_TOL * scale
    assert float((got1 - ra[[30]]).abs().max()) < FP32_TOL * scale
    assert float((got2[0] - ra[44]).abs().max()) < FP32_TOL * scale and float((got2[1] - rb[8]).abs().max()) < FP32_TOL * scale

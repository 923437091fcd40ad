"""CPU-side tests of the looped pre-norm hybrid decoder (Piladra): configuration reader, registry, the order of layer runs,
rotary table, checkpoint round trip, cache layout and byte counts, and the plain restatement's own consistency
(tests/piladra_oracle.py).  No GPU."""
from __future__ import annotations

import json
import math

import pytest
import torch

import piladra_oracle as O


def _cfg():
    att = {"type": "attention", "mlp": {"kind": "moe", "expert": {"ff": 10}, "router": {"experts": 5, "top": 2}, "shared": {"ff": 14}},
           "mixer": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "scale": 0.35, "mask": {"size": 7},
                     "rot": {"base": 100.0, "dims": 4, "scaling": {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 16}}}}
    lat = {"type": "latent_attention", "mlp": {"kind": "dense", "ff": 20},
           "mixer": {"heads": 2, "dim": 6, "rot_dim": 4, "vdim": 10, "kv_rank": 12, "scale": 0.3, "rot": {"base": 777.0, "dims": 4}}}
    mam = {"type": "mamba1", "mlp": None, "mixer": {"inner": 18, "state": 5, "dt_rank": 3, "conv": 4}}
    return {"architecture": "Piladra", "vocab": 50, "width": 24, "norm": {"eps": 1e-5, "groups": 3}, "layers": [mam, att, lat, mam],
            "canon": {"taps": 3}, "residual_mult": 0.5, "logit_softcap": 12.0, "loop": {"start": 1, "stop": 3, "times": 2}}


def test_config_reader_and_registry(tmp_path):
    from mini_sglang_amd.hybrid import DenseFfSpec, HybridConfig, HybridDecoder, MoeSpec, piladra_config
    from mini_sglang_amd.registry import architecture_of, load_model_dir, model_class

    raw = _cfg()
    assert architecture_of(raw) == "Piladra"
    cfg = piladra_config(raw)
    assert isinstance(cfg, HybridConfig) and cfg.residual == "pre_norm_conv" and model_class(cfg) is HybridDecoder
    assert (cfg.norm_groups, cfg.conv_taps, cfg.residual_mult, cfg.logit_softcap, cfg.loop) == (3, 3, 0.5, 12.0, (1, 3, 2))
    m, a, l, _ = cfg.layers
    assert (m.kind, m.vdim, m.dim, m.dt_rank, m.conv, m.mlp, m.recurrent) == ("mamba1", 18, 5, 3, 4, None, True)
    assert (a.kind, a.heads, a.kv_heads, a.window, a.sink, a.v_norm, a.rot_dims, a.rot_base) == ("sink_attention", 4, 2, 7, True, True, 4, 100.0)
    assert dict(a.rot_scaling) == {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 16.0}
    assert isinstance(a.mlp, MoeSpec) and (a.mlp.experts, a.mlp.top, a.mlp.ff, a.mlp.shared_ff, a.mlp.pick) == (5, 2, 10, 14, "sigmoid_input")
    assert (l.kind, l.out_gate, l.interleaved, l.sink, l.rot_dims) == ("latent_attention", True, False, False, 4)
    assert isinstance(l.mlp, DenseFfSpec) and l.mlp.act == "silu_gate"
    # the run of layers 1 .. 2 twice, every pass opened by its own vector; one cache layer per run
    assert cfg.runs == ((0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None))
    assert [s.kind for s in cfg.cache_layers] == ["mamba1", "sink_attention", "latent_attention", "sink_attention", "latent_attention", "mamba1"]
    assert O.layer_runs(raw) == list(cfg.runs)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    got, name = load_model_dir(tmp_path)
    assert name == "Piladra" and got == cfg
    plain = _cfg()
    del plain["loop"], plain["canon"], plain["logit_softcap"], plain["residual_mult"]
    plain["norm"] = {"eps": 1e-6}
    c2 = piladra_config(plain)
    assert (c2.loop, c2.conv_taps, c2.logit_softcap, c2.residual_mult, c2.norm_groups) == (None, 0, 0.0, 1.0, 1)
    assert c2.runs == tuple((i, None) for i in range(4))
    for edit in (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), lambda c: c["norm"].update(groups=5),
                 lambda c: c["loop"].update(stop=9), lambda c: c["layers"][2]["mixer"]["rot"].update(dims=2),
                 lambda c: c["layers"][1]["mlp"]["router"].update(top=6), lambda c: c["layers"][0].update(type="lightning")):
        bad = _cfg()
        edit(bad)
        with pytest.raises(ValueError):
            piladra_config(bad)


def test_rotary_table_with_rescaled_frequencies():
    from mini_sglang_amd.hybrid import wavelength_scaled_rotary_table

    sc = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    t = wavelength_scaled_rotary_table(12, 50.0, sc, 40, "cpu")
    f = O.rotary_freqs(12, 50.0, sc)
    pos = torch.arange(40, dtype=torch.float64)[:, None]
    assert t.shape == (40, 12) and t.dtype == torch.float32
    assert torch.allclose(t.double(), torch.cat(((pos * f).cos(), (pos * f).sin()), 1), atol=1e-7)
    plain = O.rotary_freqs(12, 50.0, None)
    waves = 2 * math.pi / plain
    assert bool((f[waves < 16] == plain[waves < 16]).all()) and torch.allclose(f[waves > 64], plain[waves > 64] / 8.0)
    mid = (waves >= 16) & (waves <= 64)
    assert bool(mid.any()) and bool(((f[mid] <= plain[mid]) & (f[mid] >= plain[mid] / 8.0)).all())
    assert torch.equal(wavelength_scaled_rotary_table(12, 50.0, None, 40, "cpu").double()[:, :6], (pos * plain).cos().float().double())


def test_checkpoint_round_trip_and_cache_layout():
    from mini_sglang_amd.hybrid import HybridDecoder, piladra_config
    from mini_sglang_amd.kvcache import HybridCache

    cfg = piladra_config(_cfg())
    a = HybridDecoder(cfg, dtype=torch.float32, device=torch.device("cpu"), seed=1)
    b = HybridDecoder(cfg, dtype=torch.float32, device=torch.device("cpu"), seed=2)
    state = a.export_state()
    assert state["head"].shape == (50, 24) and state["loop.step"].shape == (2, 24) and state["final.norm"].shape == (24,)
    assert state["l0.mix.in"].shape == (36, 24) and state["l0.mix.conv"].shape == (18, 4) and state["l0.mix.conv.b"].shape == (18,)
    assert state["l0.mix.x"].shape == (3 + 10, 18) and state["l0.mix.dt"].shape == (18, 3) and state["l0.mix.A_log"].shape == (18, 5)
    assert state["l0.mix.D"].shape == (18,) and state["l0.mix.o"].shape == (24, 18) and "l0.norm2" not in state and "l0.canon2" not in state
    assert state["l0.canon1"].shape == (24, 3) and state["l1.canon2"].shape == (24, 3)
    assert state["l1.mix.q"].shape == (32, 24) and state["l1.mix.k"].shape == (16, 24) and state["l1.mix.v"].shape == (12, 24)
    assert state["l1.mix.sink"].shape == (4,) and state["l1.mlp.router"].shape == (5, 24) and "l1.mlp.router.b" not in state
    assert state["l1.mlp.e4.gate"].shape == (10, 24) and state["l1.mlp.e0.down"].shape == (24, 10) and state["l1.mlp.shared.up"].shape == (14, 24)
    assert state["l2.mix.q"].shape == (20, 24) and state["l2.mix.dkv"].shape == (16, 24) and state["l2.mix.g"].shape == (20, 24)
    assert state["l2.mix.uk"].shape == (12, 12) and state["l2.mlp.gate"].shape == (20, 24) and state["l2.mlp.down"].shape == (24, 20)
    b.load_state(state)
    again = b.export_state()
    assert set(again) == set(state)
    for k, v in state.items():
        assert torch.allclose(again[k].float(), v.float(), atol=1e-6), k
    layers = cfg.cache_layers
    kv = HybridCache(layers, num_pages=4, page_size=16, state_rows=3, dtype=torch.bfloat16, device=torch.device("cpu"), conv_in=(3, 24))
    assert kv.num_layers == 6 and kv.state(0).shape == (3, 18, 5) and kv.state(5).dtype == torch.float32 and kv.conv_state(5).shape == (3, 3, 18)
    k1, v1 = kv.kv_rows(1)
    k3, _ = kv.kv_rows(3)
    assert k1.shape == (64, 16) and v1.shape == (64, 12) and k1.data_ptr() != k3.data_ptr()  # every pass has rows of its own
    assert kv.latent_rows(2).shape == (64, 16) and kv.latent_rows(4).data_ptr() != kv.latent_rows(2).data_ptr()
    assert kv.conv_in_states.shape == (6, 2, 3, 2, 24) and kv.conv_in_state(4, 1).shape == (3, 2, 24) and kv.conv_in_states.dtype == torch.float32
    assert HybridCache.bytes_per_page(layers, 16, torch.bfloat16) == 2 * (16 + 12 + 16) * 2 * 16
    assert HybridCache.state_bytes(layers, 3, torch.bfloat16, conv_in=(3, 24)) == 2 * 3 * (4 * 18 * 5 + 2 * 3 * 18) + 4 * 2 * 2 * 24 * 6 * 3
    none = HybridCache(layers, num_pages=1, page_size=16, state_rows=2, dtype=torch.float32, device=torch.device("cpu"))
    assert none.conv_in_states is None


def test_restatement_by_hand():
    f = torch.float64
    # two groups of two: each is divided by its own root mean square
    x = torch.tensor([[3.0, 4.0, 0.0, 2.0]], dtype=f)
    got = O.group_norm(x, torch.tensor([1.0, 1.0, 2.0, 2.0], dtype=f), 2, 0.0)
    assert torch.allclose(got, torch.tensor([[3 / math.sqrt(12.5), 4 / math.sqrt(12.5), 0.0, 2 * 2 / math.sqrt(2.0)]], dtype=f))
    # taps (a, b, c): out[t] = h[t] + a h[t-2] + b h[t-1] + c h[t], zeros before the sequence
    h = torch.tensor([[1.0], [10.0], [100.0]], dtype=f)
    got = O.input_conv(h, torch.tensor([[2.0, 3.0, 5.0]], dtype=f))
    assert torch.allclose(got, torch.tensor([[1 + 5.0], [10 + 3 + 50.0], [100 + 2 + 30 + 500.0]], dtype=f))
    # a quarter turn at position 1 with one frequency of pi / 2: (u, v) -> (-v, u); entries past the rotated ones pass
    v = torch.tensor([[[1.0, 2.0, 3.0]], [[1.0, 2.0, 3.0]]], dtype=f)
    got = O.rotate(v, torch.tensor([math.pi / 2], dtype=f), torch.arange(2))
    assert torch.allclose(got, torch.tensor([[[1.0, 2.0, 3.0]], [[-2.0, 1.0, 3.0]]], dtype=f), atol=1e-12)
    # one key with score 0 and a sink of 0: half of the value; window 1: every token sees itself only
    q, k, vv = torch.zeros(3, 1, 1, dtype=f), torch.zeros(3, 1, 1, dtype=f), torch.tensor([[[4.0]], [[6.0]], [[8.0]]], dtype=f)
    assert torch.allclose(O.windowed_sink_softmax(q, k, vv, 1.0, 1, torch.zeros(1, dtype=f))[:, 0, 0], torch.tensor([2.0, 3.0, 4.0], dtype=f))
    # window 2 without a sink: the mean of a token's value and the one before
    assert torch.allclose(O.windowed_sink_softmax(q, k, vv, 1.0, 2, None)[:, 0, 0], torch.tensor([4.0, 5.0, 7.0], dtype=f))
    # one channel, one state: S <- exp(dt A) S + dt x B; y = S C + D x
    y, S = O.selective_scan(torch.tensor([[1.0], [2.0]], dtype=f), torch.tensor([[0.5], [0.25]], dtype=f), torch.tensor([[-2.0]], dtype=f),
                            torch.tensor([[3.0], [1.0]], dtype=f), torch.tensor([[1.0], [2.0]], dtype=f), torch.tensor([10.0], dtype=f))
    s1 = 0.5 * 1.0 * 3.0
    s2 = math.exp(-0.5) * s1 + 0.25 * 2.0 * 1.0
    assert torch.allclose(y[:, 0], torch.tensor([s1 + 10.0, 2 * s2 + 20.0], dtype=f)) and abs(float(S) - s2) < 1e-12


def test_restatement_is_causal_and_counts_layer_runs():
    from mini_sglang_amd.hybrid import HybridDecoder, piladra_config

    raw = _cfg()
    state = HybridDecoder(piladra_config(raw), dtype=torch.float32, device=torch.device("cpu"), seed=3).export_state()
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, 50, (20,), generator=g).tolist()
    logits, after = O.forward(raw, state, toks)
    assert logits.shape == (20, 50) and after.shape == (6, 20, 24) and float(logits.abs().max()) <= 12.0
    head, _ = O.forward(raw, state, toks[:13])
    assert torch.allclose(head, logits[:13], atol=1e-9)
    # the experts' weight sits inside the expert: scaling the router's logits moves the output of a non-linear expert
    y = O.moe_ff(torch.randn(4, 24, generator=g, dtype=torch.float64), state, "l1.mlp.", raw["layers"][1]["mlp"])
    assert y.shape == (4, 24)
    # a selective scan continued from a carried state equals the whole
    x, dt = torch.randn(9, 3, generator=g, dtype=torch.float64), torch.rand(9, 3, generator=g, dtype=torch.float64)
    A, D = -torch.rand(3, 4, generator=g, dtype=torch.float64), torch.randn(3, generator=g, dtype=torch.float64)
    Bm, Cm = torch.randn(9, 4, generator=g, dtype=torch.float64), torch.randn(9, 4, generator=g, dtype=torch.float64)
    whole, S = O.selective_scan(x, dt, A, Bm, Cm, D)
    y1, S1 = O.selective_scan(x[:4], dt[:4], A, Bm[:4], Cm[:4], D)
    y2, S2 = O.selective_scan(x[4:], dt[4:], A, Bm[4:], Cm[4:], D, S0=S1)
    assert torch.allclose(torch.cat([y1, y2]), whole, atol=1e-12) and torch.allclose(S2, S, atol=1e-12)

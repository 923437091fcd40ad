"""CPU-side tests of the parallel-residual hybrid decoder (Givavik): configuration reader, registry, checkpoint round trip,
cache layout, and the plain restatement's own consistency (tests/givavik_oracle.py)."""
from __future__ import annotations

import json
import math

import pytest
import torch

import givavik_oracle as O


def _cfg():
    lat = {"type": "latent_attention", "mlp": {"kind": "dense", "ff": 20},
           "mixer": {"heads": 2, "dim": 6, "rot_dim": 4, "vdim": 10, "kv_rank": 12, "scale": 0.3, "rot": {"base": 777.0, "dims": 4}}}
    borrow = json.loads(json.dumps(lat))
    borrow["mixer"].update(kv_from=0, heads=3, vdim=4)
    borrow["mlp"] = None
    par = {"type": "parallel", "mlp": {"kind": "dense", "ff": 16},
           "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "scale": 0.35, "softcap": 9.0, "rot": {"base": 100.0, "dims": 4}},
                     "right": {"heads": 3, "vdim": 4, "state": 5, "groups": 1, "conv": 3, "norm_groups": 2},
                     "left_scale": 1.5, "right_scale": 0.25}}
    return {"architecture": "Givavik", "vocab": 50, "width": 24, "norm": {"eps": 1e-5}, "layers": [lat, par, borrow],
            "embedding": {"scale": 2.0, "bigram": {"buckets": 7, "mul_prev": 3, "mul_cur": 5}}}


def test_config_reader_and_registry(tmp_path):
    from mini_sglang_amd.hybrid import DenseFfSpec, HybridConfig, HybridDecoder, givavik_config
    from mini_sglang_amd.registry import architecture_of, load_model_dir, model_class

    raw = _cfg()
    assert architecture_of(raw) == "Givavik"
    cfg = givavik_config(raw)
    assert isinstance(cfg, HybridConfig) and cfg.residual == "parallel_shift" and model_class(cfg) is HybridDecoder
    assert cfg.token_shift and cfg.embed_scale == 2.0 and cfg.pair_embed == (7, 3, 5)
    a, p, b = cfg.layers
    assert (a.kind, a.sink, a.interleaved, a.rot_dims, a.rot_base, a.kv_from) == ("latent_attention", True, True, 4, 777.0, None)
    assert isinstance(a.mlp, DenseFfSpec) and a.mlp.act == "xielu" and b.kv_from == 0 and b.mlp is None and not a.recurrent
    assert p.kind == "parallel" and p.recurrent and (p.left_scale, p.right_scale) == (1.5, 0.25)
    assert (p.left.kind, p.left.heads, p.left.kv_heads, p.left.softcap, p.left.rot_dims) == ("sigmoid_attention", 4, 2, 9.0, 4)
    assert (p.right.kind, p.right.heads, p.right.dim, p.right.vdim, p.right.conv, p.right.norm_groups) == ("state_space", 3, 5, 4, 3, 2)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    got, name = load_model_dir(tmp_path)
    assert name == "Givavik" and got == cfg
    bad = _cfg()
    bad["layers"][2]["mixer"]["kv_from"] = 1  # a pair layer caches no latent rows
    with pytest.raises(ValueError):
        givavik_config(bad)
    bad = _cfg()
    bad["layers"][1]["mixer"]["right"]["norm_groups"] = 5
    with pytest.raises(ValueError):
        givavik_config(bad)


def test_checkpoint_round_trip_and_cache_layout():
    from mini_sglang_amd.hybrid import HybridDecoder, givavik_config
    from mini_sglang_amd.kvcache import HybridCache

    cfg = givavik_config(_cfg())
    a = HybridDecoder(cfg, dtype=torch.float32, device=torch.device("cpu"), seed=1)
    b = HybridDecoder(cfg, dtype=torch.float32, device=torch.device("cpu"), seed=2)
    state = a.export_state()
    assert state["bigram"].shape == (8, 24) and state["head"].shape == (50, 24) and state["l0.mix.sink"].shape == (2,)
    assert state["l0.mix.dkv"].shape == (16, 24) and "l2.mix.dkv" not in state and "l2.ls2" not in state and state["l2.ls1"].shape == (24,)
    assert state["l1.mix.left.q"].shape == (32, 24) and state["l1.mix.left.k.b"].shape == (16,) and state["l1.mix.left.o"].shape == (24, 24)
    assert state["l1.mix.right.in"].shape == (2 * 12 + 2 * 5 + 3, 24) and state["l1.mix.right.conv"].shape == (22, 3)
    assert state["l1.mix.right.o"].shape == (24, 12) and state["l1.mix.right.norm"].shape == (12,) and state["l1.mlp.act"].shape == (2,)
    b.load_state(state)
    again = b.export_state()
    assert set(again) == set(state)
    for k, v in state.items():
        assert torch.allclose(again[k].float(), v.float(), atol=1e-6), k
    assert torch.allclose(b.layers[1].sum_bias, state["l1.mix.left.o.b"] * 1.5 * state["l1.ls1"])
    kv = HybridCache(cfg.layers, num_pages=4, page_size=16, state_rows=3, dtype=torch.bfloat16, device=torch.device("cpu"),
                     shift_width=cfg.hidden_size, prev_token=True)
    assert kv.latent_rows(0).shape == (64, 16) and kv.latent_rows(2) is kv.latent_rows(0) and not kv.owns_latent(2)
    k, v = kv.kv_rows(1)
    assert k.shape == (64, 16) and v.shape == (64, 12) and kv.state(1).shape == (3, 3, 5, 4) and kv.state(1).dtype == torch.float32
    assert kv.conv_state(1).shape == (3, 2, 22) and kv.shift_state(2).shape == (3, 24) and kv.shift_states.dtype == torch.float32
    assert kv.prev_token.shape == (3,) and kv.prev_token.dtype == torch.int32
    assert HybridCache.bytes_per_page(cfg.layers, 16, torch.bfloat16) == (16 + 16 + 12) * 2 * 16
    assert HybridCache.state_bytes(cfg.layers, 3, torch.bfloat16, shift_width=24) == 3 * (4 * 3 * 5 * 4 + 2 * 2 * 22) + 4 * 24 * 3 * 3


def test_restatement_by_hand():
    z = torch.tensor([2.0, -1.0, 0.0], dtype=torch.float64)
    p, q = torch.tensor(0.0, dtype=torch.float64), torch.tensor(0.0, dtype=torch.float64)
    ln2 = math.log(2.0)
    want = torch.tensor([ln2 * 4 + 1.0, (0.5 + ln2) * (math.exp(-1.0) - 1 + 1.0) - 0.5, 0.0], dtype=torch.float64)
    assert torch.allclose(O.xielu(z, p, q), want, atol=1e-12)
    # a quarter turn of the first pair at position 1 with base 1 and two rotated entries: (u, v) -> (-v, u); the rest passes
    v = torch.tensor([[1.0, 2.0, 3.0], [1.0, 2.0, 3.0]], dtype=torch.float64)
    got = O.rotate_pairs(v, torch.tensor([0.0, math.pi / 2]), 2, 1.0)
    assert torch.allclose(got, torch.tensor([[1.0, 2.0, 3.0], [-2.0, 1.0, 3.0]], dtype=torch.float64), atol=1e-12)
    # one key with score 0 and a sink of 0: half of the value
    assert torch.allclose(O.sink_softmax_rows(torch.zeros(1, dtype=torch.float64), torch.tensor([[4.0]], dtype=torch.float64), 0.0),
                          torch.tensor([2.0], dtype=torch.float64))
    # sigmoid weights do not sum to one: two identical keys give twice one key's output
    qq, kk = torch.ones(2, 1, 1, dtype=torch.float64), torch.ones(2, 1, 1, dtype=torch.float64)
    vv = torch.ones(2, 1, 1, dtype=torch.float64)
    out = O.sigmoid_weighted_sum(qq, kk, vv, torch.zeros(1, dtype=torch.float64), 1.0, 0.0)
    assert torch.allclose(out[1], 2 * out[0]) and abs(float(out[0]) - 1 / (1 + math.exp(-1.0))) < 1e-12


def test_restatement_carries_over_a_cut():
    g = torch.Generator().manual_seed(3)
    T, H, G, N, P = 17, 4, 2, 5, 3
    xs = torch.randn(T, H, P, generator=g, dtype=torch.float64)
    Bm, Cm = (torch.randn(T, G, N, generator=g, dtype=torch.float64) for _ in range(2))
    dt = torch.rand(T, H, generator=g, dtype=torch.float64)
    A, D = torch.rand(H, generator=g, dtype=torch.float64), torch.randn(H, generator=g, dtype=torch.float64)
    whole, S = O.state_space_scan(xs, Bm, Cm, dt, A, D)
    y1, S1 = O.state_space_scan(xs[:6], Bm[:6], Cm[:6], dt[:6], A, D)
    y2, S2 = O.state_space_scan(xs[6:], Bm[6:], Cm[6:], dt[6:], A, D, S0=S1)
    assert torch.allclose(torch.cat([y1, y2]), whole, atol=1e-12) and torch.allclose(S2, S, atol=1e-12)
    h = torch.randn(5, 4, generator=g, dtype=torch.float64)
    sh = O.token_shift(h, torch.tensor([0.0, 1.0, 0.5, 2.0], dtype=torch.float64))
    assert torch.allclose(sh[0], h[0] * torch.tensor([1.0, 0.0, 0.5, -1.0], dtype=torch.float64))
    assert torch.allclose(sh[3, 1], h[2, 1]) and torch.allclose(sh[3, 0], h[3, 0])

"""`bench.py --givavik`: prefill and decode throughput of the parallel-residual hybrid decoder (Givavik: latent attention with a
sink, sigmoid attention beside a state-space layer, token shift, dense feed-forwards) at layer sizes that resemble a real
model's, beside the repository's closest model, the post-norm hybrid decoder (Nidorax: latent attention + lightning recurrence +
routed experts) of equal width, depth, head count, head size and active feed-forward width, and each new kernel alone against its
roofline beside its like kernel.

Random weights, synthetic token ids, bf16.  One JSON line on stdout; does not touch bench.py's default workload.

    python bench.py --givavik [--givavik-args --sizes s m --prompt 2048 --batch 32 --steps 20 --no-twin --no-kernels]
"""
from __future__ import annotations

import argparse
import json

import torch

from tools.hybrid_bench import HBM_TBS, MFMA_TFLOPS, VALU_TFLOPS, _time_us, run_engine

# name -> (width, layers: L = latent attention, B = latent attention on the keys of the L before it, P = sigmoid attention beside a
#          state-space layer; heads, key heads of the sigmoid attention, head size, latent size, rotated size, state-space heads, their
#          value size, state size, groups, conv taps, dense ff, vocab; experts / top / expert ff of the twin's feed-forward)
SIZES = {
    "s": (1024, "LPLP", 8, 2, 128, 256, 64, 16, 64, 128, 1, 4, 2048, 32000, 16, 2, 1024),
    "m": (2048, "LPBPLP", 16, 4, 128, 512, 64, 32, 64, 128, 2, 4, 4096, 32000, 32, 4, 1024),
}


def givavik_json(name: str) -> dict:
    W, order, H, G, D, R, r, Hs, P, N, Gs, taps, ff, V, _, _, _ = SIZES[name]
    mlp = {"kind": "dense", "ff": ff}
    layers, last_l = [], None
    for i, c in enumerate(order):
        if c == "P":
            left = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5, "softcap": 30.0, "rot": {"base": 1e6, "dims": D // 2}}
            right = {"heads": Hs, "vdim": P, "state": N, "groups": Gs, "conv": taps, "norm_groups": Gs}
            layers.append({"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": 1.0, "right_scale": 1.0}, "mlp": mlp})
        else:
            m = {"heads": H, "dim": D, "rot_dim": r, "vdim": D, "kv_rank": R, "scale": (D + r) ** -0.5, "rot": {"base": 1e6, "dims": r}}
            if c == "B":
                m["kv_from"] = last_l
            else:
                last_l = i
            layers.append({"type": "latent_attention", "mixer": m, "mlp": mlp})
    return {"architecture": "Givavik", "layers": layers, "norm": {"eps": 1e-5}, "vocab": V, "width": W,
            "embedding": {"scale": 1.0, "bigram": {"buckets": 65521, "mul_prev": 31, "mul_cur": 17}}}


def twin_json(name: str) -> dict:
    """The post-norm hybrid decoder of equal width, depth, heads and head size: the same latent attention (without sink), lightning
    layers where this design has pair layers, routed experts whose active width equals the dense feed-forward's."""
    import math

    W, order, H, G, D, R, r, Hs, P, N, Gs, taps, ff, V, E, top, eff = SIZES[name]
    mlp = {"kind": "moe", "expert": {"ff": eff}, "router": {"experts": E, "top": top, "groups": {"count": 4, "keep": 2}}}
    rot = {"base": 1e6, "dims": r, "scaling": {"factor": 8.0, "fast": 32.0, "original": 4096, "slow": 1.0}}
    layers, last_l = [], None
    for i, c in enumerate(order):
        if c == "P":
            decay = [math.exp(-2.0 ** (-(1 + 7 * h / max(H - 1, 1)))) for h in range(H)]
            layers.append({"type": "lightning", "mixer": {"heads": H, "dim": D, "vdim": D, "decay": decay}, "mlp": mlp})
        else:
            m = {"heads": H, "dim": D, "rot_dim": r, "vdim": D, "kv_rank": R, "rot": rot, "scale": (D + r) ** -0.5}
            if c == "B":
                m["kv_from"] = last_l
            else:
                last_l = i
            layers.append({"type": "latent_attention", "mixer": m, "mlp": mlp})
    return {"architecture": "Nidorax", "layers": layers, "norm": {"eps": 1e-6}, "postln_alpha": 2.0, "vocab": V, "width": W}


def _entry(us: float, flops: float, byts: float, flop_peak: float) -> dict:
    return {"us": round(us, 1), "tflops": round(flops / us / 1e6, 2), "tb_s": round(byts / us / 1e6, 3),
            "of_roofline": round(max(flops / us / 1e6 / flop_peak, byts / us / 1e6 / HBM_TBS), 4)}


def kernel_rooflines(name: str, prompt: int, batch: int, device, ssd_chunk: int = 0) -> dict:
    """Each new kernel alone at the size's shapes, beside its like kernel of the other hybrid decoders: microseconds and the share
    of the roofline that bounds it (matrix cores for a prompt portion's attention products, the fp32 vector rate for the
    recurrences, HBM for everything a decode step streams)."""
    from mini_sglang_amd import mixops
    from mini_sglang_amd.attention import MixAttnBackend

    ssd_chunk = ssd_chunk or MixAttnBackend.SSD_CHUNK
    W, order, H, G, D, R, r, Hs, P, N, Gs, taps, ff, V, _, _, _ = SIZES[name]
    bf = torch.bfloat16
    out = {}

    def rnd(*shape, dtype=bf, scale=1.0):
        return (torch.randn(shape, device=device, dtype=torch.float32) * scale).to(dtype)

    def i32(v):
        return torch.tensor(v, dtype=torch.int32, device=device)

    def chunk_list(q_len, reqs, size):
        if q_len < 2 * size:
            return None
        n = -(-q_len // size)
        items = i32([[b, c * size, min((c + 1) * size, q_len)] for b in range(reqs) for c in range(n)]).view(-1)
        return items, i32([b * n for b in range(reqs + 1)]), reqs * n

    for phase, T, reqs, ctx in (("prefill", prompt, 1, prompt), ("decode", batch, batch, prompt)):
        q_len = T // reqs
        cu, seq, rows = i32([i * q_len for i in range(reqs + 1)]), i32([ctx] * reqs), i32(list(range(reqs)))
        pos = i32([ctx - q_len + i for _ in range(reqs) for i in range(q_len)])
        slots = reqs * ctx
        table = torch.arange(slots, dtype=torch.int32, device=device).view(reqs, ctx)
        first = ctx - q_len
        pairs = reqs * (q_len * first + q_len * (q_len + 1) // 2)
        # --- sigmoid attention (+ like kernels: windowed attention without a window at the same heads; latent attention)
        q = rnd(T, H * D, dtype=torch.float32, scale=D ** -0.5)
        kc, vc = rnd(slots, G * D), rnd(slots, G * D)
        pb = torch.full((H,), -2.0, dtype=torch.float32, device=device)
        o = torch.empty(T, H * D, dtype=bf, device=device)
        sp = mixops.sigmoid_attn_splits(reqs, T, H, G, ctx) if q_len <= 16 else 1
        us = _time_us(lambda: mixops.sigmoid_attn(o, q, kc, vc, table, rows, seq, cu, reqs, H, G, D, D, D ** -0.5, 30.0, pb, splits=sp))
        attn_bytes = reqs * ctx * 2 * G * D * 2 + T * H * D * (4 + 2)
        out[f"{phase}.sigmoid_attn"] = _entry(us, 4.0 * pairs * H * D, attn_bytes, MFMA_TFLOPS)
        src = rnd(T, H * D + H, scale=0.3)
        talk = torch.eye(H, device=device)
        ws = mixops.window_attn_splits(reqs, T, 0, ctx)
        us = _time_us(lambda: mixops.window_attn(o, src, H * D, kc, vc, table, rows, seq, cu, reqs, H, G, D, D, 0, D ** -0.5, talk, splits=ws))
        out[f"{phase}.window_attn (like)"] = _entry(us, 2.0 * pairs * H * (2 * D + H), attn_bytes, MFMA_TFLOPS)
        cache, q_abs = rnd(slots, R + r), rnd(T, H, R + r, dtype=torch.float32, scale=0.1)
        o_lat = torch.empty(T, H, R, dtype=torch.float32, device=device)
        sink = torch.zeros(H, dtype=torch.float32, device=device)
        ls = mixops.latent_attn_splits(reqs, T, H, ctx) if q_len <= 16 else 1
        lat_args = (2.0 * pairs * H * (2 * R + r), reqs * ctx * (R + r) * 2 + T * H * (2 * R + r) * 4, MFMA_TFLOPS)
        us = _time_us(lambda: mixops.latent_attn(o_lat, q_abs, cache, table, rows, seq, cu, reqs, R, 0.1, splits=ls, sink=sink))
        out[f"{phase}.latent_attn_sink"] = _entry(us, *lat_args)
        us = _time_us(lambda: mixops.latent_attn(o_lat, q_abs, cache, table, rows, seq, cu, reqs, R, 0.1, splits=ls))
        out[f"{phase}.latent_attn (like)"] = _entry(us, *lat_args)
        # --- q / k preparation (like: the latent layer's preparation)
        n_left = (H + G) * D + G * D
        proj = rnd(T, n_left, scale=0.5)
        bias = torch.zeros(n_left, dtype=torch.float32, device=device)
        from mini_sglang_amd.hybrid import plain_rotary_table
        cs = plain_rotary_table(D // 2, 1e6, ctx, device)
        out_loc = table.view(-1)[: T] if reqs == 1 else table[:, ctx - 1].contiguous()
        us = _time_us(lambda: mixops.qk_prep(proj, bias, kc, vc, out_loc, pos, cs, 1e-5, H, G, D, D, interleaved=True, unit=True))
        out[f"{phase}.qk_prep"] = _entry(us, 0.0, T * (n_left * 2 + H * D * 4 + 2 * G * D * 2), VALU_TFLOPS)
        # --- state space: short convolution (same kernel as the delta layers'), recurrence (+ like: lightning), gated grouped norm
        inner, C = Hs * P, Hs * P + 2 * Gs * N
        pr = rnd(T, 2 * inner + 2 * Gs * N + Hs, scale=0.5)
        tap_w, tap_b = rnd(C, taps, scale=0.5), rnd(C, scale=0.1)
        conv_state = torch.zeros(reqs, taps - 1, C, dtype=bf, device=device)
        us = _time_us(lambda: mixops.short_conv(pr[:, inner: inner + C], C, tap_w, conv_state, cu, seq, rows, reqs, 0, 0, 1, bias=tap_b))
        out[f"{phase}.short_conv"] = _entry(us, 0.0, T * C * (2 + 4) + reqs * (taps - 1) * C * 4, VALU_TFLOPS)
        xbc = mixops.short_conv(pr[:, inner: inner + C], C, tap_w, conv_state, cu, seq, rows, reqs, 0, 0, 1, bias=tap_b)
        state = torch.zeros(reqs, Hs, N, P, dtype=torch.float32, device=device)
        rate, dtb, skip = -torch.rand(Hs, device=device), torch.zeros(Hs, device=device), torch.ones(Hs, device=device)
        y = torch.empty(T, inner, dtype=torch.float32, device=device)
        chunks = chunk_list(q_len, reqs, ssd_chunk)
        us = _time_us(lambda: mixops.ssd(y, xbc, pr[:, inner + C:], state, rate, dtb, skip, cu, seq, rows, reqs, Gs, chunks=chunks))
        out[f"{phase}.ssd"] = _entry(us, 5.0 * T * Hs * N * P, 2 * reqs * Hs * N * P * 4 + T * C * 4 + T * inner * 4, VALU_TFLOPS)
        lq = rnd(T, 4 * H * D, scale=0.5)
        lstate = torch.zeros(reqs, H, D, D, dtype=torch.float32, device=device)
        decay = torch.full((H,), 0.97, dtype=torch.float32, device=device)
        od = torch.empty(T, H * D, dtype=torch.float32, device=device)
        us = _time_us(lambda: mixops.lightning(od, lq, lstate, decay, cu, seq, rows, reqs, chunks=chunk_list(q_len, reqs, 128)))
        out[f"{phase}.lightning (like)"] = _entry(us, 4.0 * T * H * D * D, 2 * reqs * H * D * D * 4 + T * 3 * H * D * 2 + T * H * D * 4, VALU_TFLOPS)
        cat = torch.empty(T, H * D + inner, dtype=bf, device=device)
        nw = torch.ones(inner, dtype=torch.float32, device=device)
        us = _time_us(lambda: mixops.gate_group_norm(cat[:, H * D:], y, pr[:, :inner], nw, 1e-5, Gs))
        out[f"{phase}.gate_group_norm"] = _entry(us, 0.0, T * inner * (4 + 2 + 2), VALU_TFLOPS)
        gate, gw = rnd(T, H * D), rnd(H * D, scale=0.1)
        us = _time_us(lambda: mixops.gated_norm(od, gate, gw, 1e-6))
        out[f"{phase}.gated_norm (like)"] = _entry(us, 0.0, T * H * D * (4 + 2 + 2), VALU_TFLOPS)
        # --- residual sum of two parts + bias, norm, token shift (like: the post-norm)
        x, y0, y1 = rnd(T, W, dtype=torch.float32), rnd(T, W), rnd(T, W)
        vecs = [torch.ones(W, dtype=torch.float32, device=device) for _ in range(5)]
        x_out, h_out, g_out = torch.empty_like(x), torch.empty(T, W, dtype=bf, device=device), torch.empty(T, W, dtype=bf, device=device)
        shift_state = torch.zeros(reqs, W, dtype=torch.float32, device=device)
        staging = torch.empty(reqs, W, dtype=torch.float32, device=device)
        us = _time_us(lambda: mixops.shift_norm(x, vecs[0], 1e-5, dtype=bf, w_offset=1.0, parts=[(y0, vecs[1]), (y1, vecs[2])], bias=vecs[3],
                                                x_out=x_out, h_out=h_out, g_out=g_out, shift=vecs[4], state=shift_state, staging=staging,
                                                positions=pos, cu_q=cu, req_rows=rows, batch=reqs))
        out[f"{phase}.shift_norm"] = _entry(us, 0.0, T * W * (4 + 2 + 2 + 4 + 2 + 2), VALU_TFLOPS)
        nw2 = rnd(W, scale=0.1)
        us = _time_us(lambda: mixops.postnorm(x, nw2, 1e-6, y=y0, alpha=2.0, x_out=x_out, h_out=h_out))
        out[f"{phase}.postnorm (like)"] = _entry(us, 0.0, T * W * (4 + 2 + 4 + 2), VALU_TFLOPS)
        # --- feed-forward activation (like: the polynomial activation)
        z = rnd(T, ff)
        pq = torch.tensor([0.3, -0.4], dtype=torch.float32, device=device)
        us = _time_us(lambda: mixops.xielu(z, pq))
        out[f"{phase}.xielu"] = _entry(us, 0.0, T * ff * 4, VALU_TFLOPS)
        coef = torch.tensor([1.0, 0.3, 0.1, 0.0], dtype=torch.float32, device=device)
        us = _time_us(lambda: mixops.poly_act(z, coef, 1e-6))
        out[f"{phase}.poly_act (like)"] = _entry(us, 0.0, T * ff * 6, VALU_TFLOPS)
    return out


def main(argv=None) -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--sizes", nargs="*", default=["s", "m"], choices=sorted(SIZES))
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-twin", action="store_true", help="skip the post-norm hybrid decoder of equal size")
    ap.add_argument("--no-kernels", action="store_true")
    ap.add_argument("--no-engine", action="store_true", help="kernel rooflines only")
    ap.add_argument("--ssd-chunk", type=int, default=0, help="piece size of long portions in the state-space kernel's own measurement")
    args = ap.parse_args(argv)
    from mini_sglang_amd.hybrid import HybridConfig, givavik_config

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    report = {"metric": "givavik_decoder_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
              "prompt": args.prompt, "batch": args.batch, "steps": args.steps, "sizes": {}}
    keys = ("width", "layers", "heads", "kv_heads", "head", "latent", "rotated", "ss_heads", "ss_vdim", "ss_state", "ss_groups", "taps", "ff",
            "vocab", "twin_experts", "twin_top", "twin_ff")
    if not args.no_engine:  # the process's first engine pays for library loading and allocator growth: one untimed pass
        run_engine(givavik_config(givavik_json(args.sizes[0])), args.prompt, args.batch, 1, 1, device)
    for name in args.sizes:
        entry = {"shape": dict(zip(keys, SIZES[name]))}
        if not args.no_engine:
            entry["givavik"] = run_engine(givavik_config(givavik_json(name)), args.prompt, args.batch, args.steps, args.warmup, device)
            print(f"[givavik bench] {name}: " + json.dumps(entry["givavik"]), flush=True)
            if not args.no_twin:
                entry["post_norm_hybrid"] = run_engine(HybridConfig.from_json(twin_json(name)), args.prompt, args.batch, args.steps, args.warmup,
                                                       device)
                print(f"[givavik bench] {name} twin: " + json.dumps(entry["post_norm_hybrid"]), flush=True)
        if not args.no_kernels:
            entry["kernels"] = kernel_rooflines(name, args.prompt, args.batch, device, args.ssd_chunk)
        report["sizes"][name] = entry
    print(json.dumps(report))


if __name__ == "__main__":
    main()

"""`bench.py --piladra`: prefill and decode throughput of the looped pre-norm hybrid decoder (Piladra: grouped norms, input
convolutions, gated latent attention, a selective-scan layer, windowed attention with a sink, experts weighted on their input)
at layer sizes that resemble a real model's, beside the repository's closest model, the parallel-residual hybrid decoder (Givavik:
latent attention, sigmoid attention beside a state-space layer, dense feed-forwards) of equal width, depth, head count, head size
and active feed-forward width, and each new kernel alone against its roofline beside its like kernel.

Random weights, synthetic token ids, bf16.  One JSON line on stdout; does not touch bench.py's default workload.

    python bench.py --piladra [--piladra-args --sizes s m --prompt 2048 --batch 32 --steps 20 --no-twin --no-kernels]
"""
from __future__ import annotations

import argparse
import json

import torch

from tools.givavik_bench import SIZES as TWIN_SIZES
from tools.givavik_bench import givavik_json
from tools.hybrid_bench import HBM_TBS, MFMA_TFLOPS, VALU_TFLOPS, _time_us, run_engine

# name -> (width, layers: M = selective scan, A = windowed attention with a sink, L = gated latent attention; loop (start, stop, times)
#          or None; heads, key heads of the windowed attention, head size, latent size, rotated size, scan channels, state size, inner
#          size of the step projection, scan taps, window, taps of the input convolutions, norm groups, dense ff, experts, top, expert ff,
#          shared ff, vocab).  Layers alternate dense and routed feed-forwards; the twin is the Givavik size of the same name.
SIZES = {
    "s": (1024, "MALM", None, 8, 2, 128, 256, 64, 2048, 16, 64, 4, 1024, 4, 4, 2048, 16, 2, 512, 1024, 32000),
    "m": (2048, "MALM", (1, 3, 2), 16, 4, 128, 512, 64, 4096, 16, 128, 4, 2048, 4, 4, 4096, 32, 4, 512, 2048, 32000),
}


def piladra_json(name: str) -> dict:
    W, order, loop, H, G, D, R, r, C, N, dr, taps, window, ctaps, groups, ff, E, top, eff, sff, V = SIZES[name]
    dense = {"kind": "dense", "ff": ff}
    moe = {"kind": "moe", "expert": {"ff": eff}, "router": {"experts": E, "top": top}, "shared": {"ff": sff}}
    layers = []
    for i, c in enumerate(order):
        mlp = moe if i % 2 else dense
        if c == "M":
            layers.append({"type": "mamba1", "mixer": {"inner": C, "state": N, "dt_rank": dr, "conv": taps}, "mlp": mlp})
        elif c == "A":
            rot = {"base": 1e6, "dims": D, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}
            layers.append({"type": "attention", "mlp": mlp,
                           "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5, "mask": {"size": window}, "rot": rot}})
        else:
            layers.append({"type": "latent_attention", "mlp": mlp,
                           "mixer": {"heads": H, "dim": D, "rot_dim": r, "vdim": D, "kv_rank": R, "scale": (D + r) ** -0.5,
                                     "rot": {"base": 1e6, "dims": r}}})
    cfg = {"architecture": "Piladra", "layers": layers, "norm": {"eps": 1e-6, "groups": groups}, "canon": {"taps": ctaps}, "residual_mult": 0.7,
           "logit_softcap": 30.0, "vocab": V, "width": W}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def _entry(us: float, flops: float, byts: float, flop_peak: float) -> dict:
    return {"us": round(us, 1), "tflops": round(flops / us / 1e6, 2), "tb_s": round(byts / us / 1e6, 3),
            "of_roofline": round(max(flops / us / 1e6 / flop_peak, byts / us / 1e6 / HBM_TBS), 4)}


def kernel_rooflines(name: str, prompt: int, batch: int, device, scan_chunk: int = 0) -> dict:
    """Each new kernel alone at the size's shapes, beside its like kernel of the other hybrid decoders: microseconds and the share
    of the roofline that bounds it (matrix cores for a prompt portion's attention products, the fp32 vector rate for the
    recurrences, HBM for everything a decode step streams and for the row kernels)."""
    from mini_sglang_amd import mixops
    from mini_sglang_amd.attention import MixAttnBackend

    W, order, loop, H, G, D, R, r, C, N, dr, taps, window, ctaps, groups, ff, E, top, eff, sff, V = SIZES[name]
    Hs, P, Ns, Gs = TWIN_SIZES[name][7], TWIN_SIZES[name][8], TWIN_SIZES[name][9], TWIN_SIZES[name][10]
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
        slots = reqs * ctx
        table = torch.arange(slots, dtype=torch.int32, device=device).view(reqs, ctx)
        first = ctx - q_len
        # --- windowed attention with a sink: every earlier key visible (the like kernel's work), and the size's window
        q = rnd(T, H * D, dtype=torch.float32, scale=D ** -0.5)
        kc, vc = rnd(slots, G * D), rnd(slots, G * D)
        sink = torch.zeros(H, dtype=torch.float32, device=device)
        pb = torch.full((H,), -2.0, dtype=torch.float32, device=device)
        o = torch.empty(T, H * D, dtype=bf, device=device)
        for label, win in (("sink_attn", 0), ("sink_attn (window %d)" % (window // 2), window // 2)):
            keys = lambda p: min(p + 1, win) if win else p + 1  # noqa: E731
            pairs = reqs * sum(keys(first + i) for i in range(q_len))
            read = reqs * (min(ctx, win + q_len) if win else ctx)
            sp = mixops.sink_attn_splits(reqs, T, H, G, win, ctx) if q_len <= 16 else 1
            us = _time_us(lambda: mixops.sink_attn(o, q, kc, vc, table, rows, seq, cu, reqs, H, G, D, D, D ** -0.5, win, sink, splits=sp))
            out[f"{phase}.{label}"] = _entry(us, 4.0 * pairs * H * D, read * 2 * G * D * 2 + T * H * D * (4 + 2), MFMA_TFLOPS)
        pairs = reqs * (q_len * first + q_len * (q_len + 1) // 2)
        sp = mixops.sigmoid_attn_splits(reqs, T, H, G, ctx) if q_len <= 16 else 1
        us = _time_us(lambda: mixops.sigmoid_attn(o, q, kc, vc, table, rows, seq, cu, reqs, H, G, D, D, D ** -0.5, 30.0, pb, splits=sp))
        out[f"{phase}.sigmoid_attn (like)"] = _entry(us, 4.0 * pairs * H * D, reqs * ctx * 2 * G * D * 2 + T * H * D * (4 + 2), MFMA_TFLOPS)
        # --- selective scan (like: the state-space recurrence with one decay per head), its convolution (the same kernel)
        pr = rnd(T, 2 * C, scale=0.5)
        tap_w, tap_b = rnd(C, taps, scale=0.5), rnd(C, scale=0.1)
        conv_state = torch.zeros(reqs, taps - 1, C, dtype=bf, device=device)
        us = _time_us(lambda: mixops.short_conv(pr, C, tap_w, conv_state, cu, seq, rows, reqs, 0, 0, 1, bias=tap_b, model_dtype=True))
        out[f"{phase}.short_conv"] = _entry(us, 0.0, T * C * (2 + 2) + reqs * (taps - 1) * C * 4, VALU_TFLOPS)
        x = mixops.short_conv(pr, C, tap_w, conv_state, cu, seq, rows, reqs, 0, 0, 1, bias=tap_b, model_dtype=True)
        dbc, dt_in = rnd(T, dr + 2 * N, scale=0.5), rnd(T, C, scale=0.5)
        A = -torch.exp(torch.randn(C, N, device=device) * 0.5)
        dtb, skip = torch.full((C,), -2.0, device=device), torch.ones(C, device=device)
        state = torch.zeros(reqs, C, N, dtype=torch.float32, device=device)
        chunks = chunk_list(q_len, reqs, scan_chunk or MixAttnBackend.SCAN_CHUNK)
        us = _time_us(lambda: mixops.selective_scan(x, pr[:, C:], dt_in, dbc[:, dr:], A, dtb, skip, state, cu, seq, rows, reqs, chunks=chunks))
        out[f"{phase}.selective_scan"] = _entry(us, 5.0 * T * C * N, 2 * reqs * C * N * 4 + T * C * 2 * 4 + T * 2 * N * 2, VALU_TFLOPS)
        inner, Cs = Hs * P, Hs * P + 2 * Gs * Ns
        xbc = rnd(T, Cs, dtype=torch.float32, scale=0.5)
        dt_raw = rnd(T, Hs, scale=0.5)
        sstate = torch.zeros(reqs, Hs, Ns, P, dtype=torch.float32, device=device)
        rate, dtb2, skip2 = -torch.rand(Hs, device=device), torch.zeros(Hs, device=device), torch.ones(Hs, device=device)
        y = torch.empty(T, inner, dtype=torch.float32, device=device)
        us = _time_us(lambda: mixops.ssd(y, xbc, dt_raw, sstate, rate, dtb2, skip2, cu, seq, rows, reqs, Gs,
                                         chunks=chunk_list(q_len, reqs, MixAttnBackend.SSD_CHUNK)))
        out[f"{phase}.ssd (like)"] = _entry(us, 5.0 * T * Hs * Ns * P, 2 * reqs * Hs * Ns * P * 4 + T * Cs * 4 + T * inner * 4, VALU_TFLOPS)
        # --- residual sum of two parts + grouped norm + input convolution (like: sum + norm + token shift)
        xr, y0, y1 = rnd(T, W, dtype=torch.float32), rnd(T, top, W), rnd(T, W)
        nw, ctw = rnd(W, scale=0.1), rnd(W, ctaps, scale=0.3)
        x_out, h_out = torch.empty_like(xr), torch.empty(T, W, dtype=bf, device=device)
        cstate = torch.zeros(reqs, ctaps - 1, W, dtype=torch.float32, device=device)
        cstage = torch.empty(reqs, ctaps - 1, W, dtype=torch.float32, device=device)
        us = _time_us(lambda: mixops.norm_conv(xr, nw, 1e-6, groups, h_out, parts=(y0, y1), mult=0.7, x_out=x_out, taps=ctw, state=cstate,
                                               staging=cstage, cu_q=cu, seq_lens=seq, req_rows=rows, batch=reqs))
        out[f"{phase}.norm_conv ({top} + 1 parts)"] = _entry(us, 0.0, T * W * (4 + 2 * (top + 1) + 4 + 2), VALU_TFLOPS)
        us = _time_us(lambda: mixops.norm_conv(xr, nw, 1e-6, groups, h_out, parts=(y1,), mult=0.7, x_out=x_out, taps=ctw, state=cstate,
                                               staging=cstage, cu_q=cu, seq_lens=seq, req_rows=rows, batch=reqs))
        out[f"{phase}.norm_conv (1 part)"] = _entry(us, 0.0, T * W * (4 + 2 + 4 + 2), VALU_TFLOPS)
        vecs = [torch.ones(W, dtype=torch.float32, device=device) for _ in range(5)]
        g_out = torch.empty(T, W, dtype=bf, device=device)
        pos = i32([ctx - q_len + i for _ in range(reqs) for i in range(q_len)])
        sstage, shstate = torch.empty(reqs, W, dtype=torch.float32, device=device), torch.zeros(reqs, W, dtype=torch.float32, device=device)
        y0s = rnd(T, W)
        us = _time_us(lambda: mixops.shift_norm(xr, vecs[0], 1e-5, dtype=bf, w_offset=1.0, parts=[(y0s, vecs[1]), (y1, vecs[2])], bias=vecs[3],
                                                x_out=x_out, h_out=h_out, g_out=g_out, shift=vecs[4], state=shstate, staging=sstage,
                                                positions=pos, cu_q=cu, req_rows=rows, batch=reqs))
        out[f"{phase}.shift_norm (like)"] = _entry(us, 0.0, T * W * (4 + 2 + 2 + 4 + 2 + 2), VALU_TFLOPS)
        # --- router + weighted expert inputs (like: the router on logits with softmax weights)
        hh, router = rnd(T, W), rnd(E, W, scale=W ** -0.5)
        us = _time_us(lambda: mixops.scale_rows(hh, mixops.route_sigmoid(hh, router, top)[1]))
        out[f"{phase}.route_sigmoid + scale_rows"] = _entry(us, 2.0 * T * E * W, T * W * 2 * (1 + top) + E * W * 2, MFMA_TFLOPS)
        us = _time_us(lambda: mixops.route_top(hh, router, None, top))
        out[f"{phase}.route_top (like)"] = _entry(us, 2.0 * T * E * W, T * W * 2 + E * W * 2, MFMA_TFLOPS)
        # --- the latent layer's output gate (like: the gated norm over the concatenated heads), the cap of the logits
        o32, gate = rnd(T, H * D, dtype=torch.float32), rnd(T, H * D + 64)[:, 64:]
        us = _time_us(lambda: mixops.sigmoid_gate(o32, gate))
        out[f"{phase}.sigmoid_gate"] = _entry(us, 0.0, T * H * D * (4 + 2 + 2), VALU_TFLOPS)
        gw = rnd(H * D, scale=0.1)
        us = _time_us(lambda: mixops.gated_norm(o32, gate, gw, 1e-6))
        out[f"{phase}.gated_norm (like)"] = _entry(us, 0.0, T * H * D * (4 + 2 + 2), VALU_TFLOPS)
        lg = rnd(reqs, V)
        us = _time_us(lambda: mixops.softcap(lg, 30.0))
        out[f"{phase}.softcap"] = _entry(us, 0.0, reqs * V * 4, VALU_TFLOPS)
    return out


def main(argv=None) -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--sizes", nargs="*", default=["s", "m"], choices=sorted(SIZES))
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-twin", action="store_true", help="skip the parallel-residual hybrid decoder of equal size")
    ap.add_argument("--no-kernels", action="store_true")
    ap.add_argument("--no-engine", action="store_true", help="kernel rooflines only")
    ap.add_argument("--scan-chunk", type=int, default=0, help="piece size of long portions in the selective scan's own measurement")
    args = ap.parse_args(argv)
    from mini_sglang_amd.hybrid import givavik_config, piladra_config

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    report = {"metric": "piladra_decoder_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
              "prompt": args.prompt, "batch": args.batch, "steps": args.steps, "sizes": {}}
    keys = ("width", "layers", "loop", "heads", "kv_heads", "head", "latent", "rotated", "scan_channels", "scan_state", "dt_rank", "scan_taps",
            "window", "input_taps", "norm_groups", "ff", "experts", "top", "expert_ff", "shared_ff", "vocab")
    if not args.no_engine:  # the process's first engine pays for library loading and allocator growth: one untimed pass
        run_engine(piladra_config(piladra_json(args.sizes[0])), args.prompt, args.batch, 1, 1, device)
    for name in args.sizes:
        entry = {"shape": dict(zip(keys, SIZES[name]))}
        if not args.no_engine:
            entry["piladra"] = run_engine(piladra_config(piladra_json(name)), args.prompt, args.batch, args.steps, args.warmup, device)
            print(f"[piladra bench] {name}: " + json.dumps(entry["piladra"]), flush=True)
            if not args.no_twin:
                entry["parallel_residual_hybrid"] = run_engine(givavik_config(givavik_json(name)), args.prompt, args.batch, args.steps,
                                                               args.warmup, device)
                print(f"[piladra bench] {name} twin: " + json.dumps(entry["parallel_residual_hybrid"]), flush=True)
        if not args.no_kernels:
            entry["kernels"] = kernel_rooflines(name, args.prompt, args.batch, device, args.scan_chunk)
        report["sizes"][name] = entry
    print(json.dumps(report))


if __name__ == "__main__":
    main()

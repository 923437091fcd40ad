"""A plain, slow restatement of the Givavik design in float64 torch, one function per mechanism, token loops where the
design has a recurrence.  It shares no code with the product path: tests hand it a configuration dictionary (the layout of a
Givavik config.json) and a checkpoint-style dictionary of tensors and compare what the engine computes with what this
computes.

Design in short (sizes and constants from the configuration):
  x_0[t]   = embed[tok_t] * s_e + bigram[(tok_(t-1) * m_p + tok_t * m_c) mod B]   (row B for a sequence's first token)
  layer    : h = rms(x) * (1 + w);  g = h + (h_(t-1) - h) * shift  (h_(-1) = 0);  x <- x + ls1 * mixer(g) + ls2 * ff(h)
  mixers   : latent attention with a per-head sink in the softmax denominator (optionally on another layer's cached rows), or
             a pair running side by side: sigmoid attention (grouped heads, biases, rotation, unit-RMS q and k, tanh soft cap,
             weights sigmoid(score + b_h), no normalisation over keys) + a Mamba-2 state-space layer.
  ff       : W_down xielu(W_up h)
  output   : rms(x) * (1 + w_final), then the head matrix.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def xielu(z: torch.Tensor, p: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    pos = softplus(p) * z * z + 0.5 * z
    zn = torch.clamp(z, max=0.0)
    neg = (0.5 + softplus(q)) * (torch.expm1(zn) - zn) + 0.5 * zn
    return torch.where(z > 0, pos, neg)


def rotate_pairs(v: torch.Tensor, pos: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """v [T, ..., n]: entries (2i, 2i + 1), i < dims / 2, turn by pos * base^(-2i / dims); the rest pass."""
    out = v.clone()
    shape = [v.shape[0]] + [1] * (v.dim() - 2)
    for i in range(dims // 2):
        ang = pos.to(F64) * (float(base) ** (-2.0 * i / dims))
        c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
        a, b = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def embedding(cfg: dict, st: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    e = cfg["embedding"]
    x = st["embed"].to(F64)[tokens] * float(e["scale"])
    bg = e.get("bigram")
    if bg:
        B = int(bg["buckets"])
        rows = [B if t == 0 else (tokens[t - 1] * int(bg["mul_prev"]) + tokens[t] * int(bg["mul_cur"])) % B for t in range(len(tokens))]
        x = x + st["bigram"].to(F64)[rows]
    return x


def token_shift(h: torch.Tensor, shift: torch.Tensor) -> torch.Tensor:
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (prev - h) * shift


def latent_rows(m: dict, st, p: str, g: torch.Tensor, eps: float):
    """-> (latent c [T, R], rotated shared key part [T, r]) of a layer that owns its keys."""
    R, r = int(m["kv_rank"]), int(m["rot_dim"])
    T = g.shape[0]
    kv = g @ st[p + "dkv"].to(F64).T
    c = rms_unit(kv[:, :R], eps) * st[p + "dkv.norm"].to(F64)
    kr = rotate_pairs(kv[:, R:], torch.arange(T), int(m["rot"]["dims"]), float(m["rot"]["base"]))
    return c, kr


def sink_softmax_rows(s: torch.Tensor, v: torch.Tensor, sink: float) -> torch.Tensor:
    """One query: scores s [n] over its visible keys, values v [n, e]; the denominator holds one more term exp(sink)."""
    top = max(float(s.max()), float(sink))
    e = torch.exp(s - top)
    return (e @ v) / (e.sum() + math.exp(float(sink) - top))


def sigmoid_weighted_sum(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, pb: torch.Tensor, scale: float, cap: float) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, e] of one sequence -> [T, H, e]: every visible key weighs sigmoid(cap tanh(s / cap) + pb_h),
    s = scale q.k, nothing is normalised (cap <= 0: no soft cap)."""
    T, H, _ = q.shape
    rep = H // k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for h in range(H):
        for i in range(T):
            s = (k[: i + 1, h // rep] @ q[i, h]) * scale
            if cap > 0:
                s = cap * torch.tanh(s / cap)
            out[i, h] = torch.sigmoid(s + pb[h]) @ v[: i + 1, h // rep]
    return out


def state_space_scan(xs: torch.Tensor, Bm: torch.Tensor, Cm: torch.Tensor, dt: torch.Tensor, A: torch.Tensor, D: torch.Tensor,
                     S0: Optional[torch.Tensor] = None):
    """xs [T, H, P], Bm / Cm [T, G, N], dt [T, H] (already positive), A [H] > 0, D [H] -> (y [T, H, P], final state [H, N, P])."""
    T, H, P = xs.shape
    G, N = Bm.shape[1], Bm.shape[2]
    y = torch.zeros(T, H, P, dtype=F64)
    S = torch.zeros(H, N, P, dtype=F64) if S0 is None else S0.clone()
    for h in range(H):
        gi = h // (H // G)
        for t in range(T):
            S[h] = torch.exp(-A[h] * dt[t, h]) * S[h] + dt[t, h] * torch.outer(Bm[t, gi], xs[t, h])
            y[t, h] = S[h].T @ Cm[t, gi] + D[h] * xs[t, h]
    return y, S


def latent_attention(m: dict, st, p: str, g: torch.Tensor, c: torch.Tensor, kr: torch.Tensor) -> torch.Tensor:
    H, d, r, dv, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    T = g.shape[0]
    q = (g @ st[p + "q"].to(F64).T).view(T, H, d + r)
    qn, qr = q[..., :d], rotate_pairs(q[..., d:], torch.arange(T), int(m["rot"]["dims"]), float(m["rot"]["base"]))
    k = (c @ st[p + "uk"].to(F64).T).view(T, H, d)
    v = (c @ st[p + "uv"].to(F64).T).view(T, H, dv)
    sink = st[p + "sink"].to(F64)
    out = torch.zeros(T, H, dv, dtype=F64)
    for h in range(H):
        for i in range(T):
            s = (k[: i + 1, h] @ qn[i, h] + kr[: i + 1] @ qr[i, h]) * float(m["scale"])
            out[i, h] = sink_softmax_rows(s, v[: i + 1, h], float(sink[h]))
    return out.reshape(T, H * dv) @ st[p + "o"].to(F64).T


def sigmoid_attention(m: dict, st, p: str, g: torch.Tensor, eps: float) -> torch.Tensor:
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = g.shape[0]
    pos = torch.arange(T)
    lin = lambda n: g @ st[p + n].to(F64).T + st[p + n + ".b"].to(F64)
    rot = m.get("rot") or {}
    dims, base = int(rot.get("dims", 0)), float(rot.get("base", 10000.0))
    q = rms_unit(rotate_pairs(lin("q").view(T, H, d), pos, dims, base), eps)
    k = rms_unit(rotate_pairs(lin("k").view(T, G, d), pos, dims, base), eps)
    v = lin("v").view(T, G, dv)
    out = sigmoid_weighted_sum(q, k, v, st[p + "pb"].to(F64), float(m["scale"]), float(m.get("softcap") or 0.0))
    return out.reshape(T, H * dv) @ st[p + "o"].to(F64).T + st[p + "o.b"].to(F64)


def state_space(m: dict, st, p: str, g: torch.Tensor, eps: float) -> torch.Tensor:
    """Mamba-2 layer: in-projection [z | x | B | C | dt], causal convolution + SiLU over x, B, C, the recurrence
    S <- exp(-exp(A) dt) S + dt B x^T,  y = S^T C + D x, then y * silu(z), a grouped RMS norm, the output projection."""
    H, P, N, G, taps, ng = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"]), int(m["norm_groups"])
    inner, T = H * P, g.shape[0]
    u = g @ st[p + "in"].to(F64).T
    z, xbc, dt = u[:, :inner], u[:, inner: 2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    w, b = st[p + "conv"].to(F64), st[p + "conv.b"].to(F64)
    padded = torch.cat([torch.zeros(taps - 1, xbc.shape[1], dtype=F64), xbc], dim=0)
    conv = torch.stack([(padded[t: t + taps].T * w).sum(dim=1) + b for t in range(T)])
    conv = silu(conv)
    xs = conv[:, :inner].view(T, H, P)
    Bm = conv[:, inner: inner + G * N].view(T, G, N)
    Cm = conv[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + st[p + "dt_bias"].to(F64))
    A, D = torch.exp(st[p + "A_log"].to(F64)), st[p + "D"].to(F64)
    y, _ = state_space_scan(xs, Bm, Cm, dt, A, D)
    y = y.reshape(T, inner) * silu(z)
    y = rms_unit(y.view(T, ng, inner // ng), eps).reshape(T, inner) * st[p + "norm"].to(F64)
    return y @ st[p + "o"].to(F64).T


def feed_forward(st, p: str, h: torch.Tensor) -> torch.Tensor:
    a = st[p + "act"].to(F64)
    return xielu(h @ st[p + "up"].to(F64).T, a[0], a[1]) @ st[p + "down"].to(F64).T


def forward(cfg: dict, st: Dict[str, torch.Tensor], tokens: List[int], layer_outputs: Optional[list] = None) -> torch.Tensor:
    """-> logits [T, vocab] (float64) of one sequence from its first token."""
    eps = float(cfg["norm"]["eps"])
    x = embedding(cfg, st, list(tokens))
    kept = {}
    for i, entry in enumerate(cfg["layers"]):
        m, p = entry["mixer"], f"l{i}.mix."
        h = rms_unit(x, eps) * (1.0 + st[f"l{i}.norm1"].to(F64))
        g = token_shift(h, st[f"l{i}.shift"].to(F64))
        if entry["type"] == "latent_attention":
            if m.get("kv_from") is None:
                kept[i] = latent_rows(m, st, p, g, eps)
            c, kr = kept[i if m.get("kv_from") is None else int(m["kv_from"])]
            y = latent_attention(m, st, p, g, c, kr)
        elif entry["type"] == "parallel":
            y = float(m["left_scale"]) * sigmoid_attention(m["left"], st, p + "left.", g, eps) \
                + float(m["right_scale"]) * state_space(m["right"], st, p + "right.", g, eps)
        else:
            raise ValueError(entry["type"])
        upd = st[f"l{i}.ls1"].to(F64) * y
        if entry.get("mlp") is not None:
            upd = upd + st[f"l{i}.ls2"].to(F64) * feed_forward(st, f"l{i}.mlp.", h)
        x = x + upd
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    hf = rms_unit(x, eps) * (1.0 + st["final.norm"].to(F64))
    return hf @ st["head"].to(F64).T

"""A plain, slow restatement of the Piladra design in float64 torch: one function per mechanism, whole sequences only, token
loops where the design has a recurrence.  It shares no code with the product path; tests hand it a configuration dictionary
(the layout of the design's config.json) and a checkpoint dictionary (checkpoint tensor names) and compare.

Notation: T tokens of one sequence, positions 0 .. T - 1; W = width; every weight matrix is [out, in] and applied as x @ M^T.
"""
from __future__ import annotations

import math
from typing import Any, Dict, List, Optional, Tuple

import torch

F64 = torch.float64


def _w(state: Dict[str, torch.Tensor], name: str) -> torch.Tensor:
    return state[name].to(F64)


def group_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """Every one of `groups` equal consecutive parts of a row is divided by sqrt(mean(part^2) + eps); then the row times w."""
    T, W = x.shape
    p = x.reshape(T, groups, W // groups)
    p = p / torch.sqrt((p * p).mean(dim=-1, keepdim=True) + eps)
    return p.reshape(T, W) * w


def causal_taps(u: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """out[t, c] = sum_j taps[c, j] u[t - (n - 1) + j, c] with u = 0 before the sequence (the last tap is the current token's)."""
    T, C = u.shape
    n = taps.shape[1]
    out = torch.zeros_like(u)
    for t in range(T):
        for j in range(n):
            s = t - (n - 1) + j
            if s >= 0:
                out[t] += taps[:, j] * u[s]
    return out


def input_conv(h: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    return h + causal_taps(h, taps)


def rotary_freqs(dims: int, base: float, scaling: Optional[Dict[str, float]]) -> torch.Tensor:
    i = torch.arange(dims // 2, dtype=F64)
    f = float(base) ** (-2.0 * i / dims)
    if scaling:
        factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        out = []
        for fi in f.tolist():
            wave = 2.0 * math.pi / fi
            if wave < orig / high:
                out.append(fi)
            elif wave > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wave - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = torch.tensor(out, dtype=F64)
    return f


def rotate(v: torch.Tensor, freqs: torch.Tensor, pos: torch.Tensor) -> torch.Tensor:
    """v [T, heads, n]: the first 2 * len(freqs) entries of each head turn, entry i paired with entry i + len(freqs)."""
    half = freqs.shape[0]
    if half == 0:
        return v
    a = pos.to(F64)[:, None, None] * freqs[None, None, :]
    c, s = torch.cos(a), torch.sin(a)
    u, w = v[..., :half], v[..., half: 2 * half]
    return torch.cat((u * c - w * s, w * c + u * s, v[..., 2 * half:]), dim=-1)


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def latent_attention(h: torch.Tensor, st: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, d, r, dv, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(T)
    q = (h @ _w(st, p + "q").T).reshape(T, H, d + r)
    dkv = h @ _w(st, p + "dkv").T
    c = dkv[:, :R]
    c = c / torch.sqrt((c * c).mean(dim=-1, keepdim=True) + eps) * _w(st, p + "dkv.norm")
    rot = m.get("rot") or {}
    freqs = rotary_freqs(int(rot.get("dims", r)), float(rot["base"]), rot.get("scaling"))
    k_rot = rotate(dkv[:, None, R:], freqs, pos)[:, 0]
    q_rot = rotate(q[:, :, d:], freqs, pos)
    k = (c @ _w(st, p + "uk").T).reshape(T, H, d)
    v = (c @ _w(st, p + "uv").T).reshape(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        s = (torch.einsum("hd,jhd->hj", q[i, :, :d], k[: i + 1]) + q_rot[i] @ k_rot[: i + 1].T) * float(m["scale"])
        a = torch.softmax(s, dim=-1)
        out[i] = torch.einsum("hj,jhv->hv", a, v[: i + 1])
    gated = out.reshape(T, H * dv) * sigmoid(h @ _w(st, p + "g").T)
    return gated @ _w(st, p + "o").T


def selective_scan(x: torch.Tensor, dt: torch.Tensor, A: torch.Tensor, B: torch.Tensor, C: torch.Tensor, D: torch.Tensor,
                   S0: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """x, dt [T, channels]; A [channels, N]; B, C [T, N]; D [channels] -> (y [T, channels], the state after the last token)."""
    T, ch = x.shape
    S = torch.zeros(ch, A.shape[1], dtype=F64) if S0 is None else S0.clone()
    y = torch.zeros(T, ch, dtype=F64)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + D * x[t]
    return y, S


def mamba1(h: torch.Tensor, st: Dict[str, torch.Tensor], p: str, m: Dict[str, Any]) -> torch.Tensor:
    inner, N, dr = int(m["inner"]), int(m["state"]), int(m["dt_rank"])
    xz = h @ _w(st, p + "in").T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_taps(x, _w(st, p + "conv")) + _w(st, p + "conv.b"))
    dbc = x @ _w(st, p + "x").T
    dt = softplus(dbc[:, :dr] @ _w(st, p + "dt").T + _w(st, p + "dt.b"))
    y, _ = selective_scan(x, dt, -torch.exp(_w(st, p + "A_log")), dbc[:, dr: dr + N], dbc[:, dr + N: dr + 2 * N], _w(st, p + "D"))
    return (y * silu(z)) @ _w(st, p + "o").T


def windowed_sink_softmax(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int,
                          sink: Optional[torch.Tensor]) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]: token i weighs the keys j with 0 <= i - j < window (window 0: all j <= i)
    by exp(score) over the sum of these and exp(sink[h])."""
    T, H, _ = q.shape
    G, dv = k.shape[1], v.shape[2]
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        lo = max(0, i - window + 1) if window > 0 else 0
        for hh in range(H):
            g = hh // (H // G)
            s = (k[lo: i + 1, g] @ q[i, hh]) * scale
            mx = s.max() if sink is None else torch.maximum(s.max(), sink[hh])
            e = torch.exp(s - mx)
            den = e.sum() + (torch.exp(sink[hh] - mx) if sink is not None else 0.0)
            out[i, hh] = (e / den) @ v[lo: i + 1, g]
    return out


def window_attention(h: torch.Tensor, st: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q = (h @ _w(st, p + "q").T).reshape(T, H, d)
    k = (h @ _w(st, p + "k").T).reshape(T, G, d)
    v = (h @ _w(st, p + "v").T).reshape(T, G, dv)
    rot = m.get("rot") or {}
    if rot.get("dims"):
        freqs = rotary_freqs(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        q, k = rotate(q, freqs, pos), rotate(k, freqs, pos)
    v = v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    window = int((m.get("mask") or {}).get("size", 0))
    sink = _w(st, p + "sink") if (p + "sink") in st else None
    out = windowed_sink_softmax(q, k, v, float(m["scale"]), window, sink)
    return out.reshape(T, H * dv) @ _w(st, p + "o").T


def gated_ff(h: torch.Tensor, st: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (silu(h @ _w(st, p + "gate").T) * (h @ _w(st, p + "up").T)) @ _w(st, p + "down").T


def moe_ff(h: torch.Tensor, st: Dict[str, torch.Tensor], p: str, mlp: Dict[str, Any]) -> torch.Tensor:
    """Sigmoid scores, the `top` largest chosen, the score multiplies the chosen expert's INPUT; a shared expert is added."""
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    s = sigmoid(h @ _w(st, p + "router").T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        best = torch.topk(s[t], top).indices.tolist()
        for e in best:
            out[t] += gated_ff((s[t, e] * h[t])[None], st, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, st, p + "shared.")
    return out


def layer_runs(cfg: Dict[str, Any]) -> List[Tuple[int, Optional[int]]]:
    """[(layer, pass number when the layer is the first of a loop pass else None)] in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs: List[Tuple[int, Optional[int]]] = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t if i == a else None) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, n)]


def forward(cfg: Dict[str, Any], st: Dict[str, torch.Tensor], tokens) -> Tuple[torch.Tensor, torch.Tensor]:
    """-> (logits [T, vocab], the residual stream after every layer run [runs, T, W]) in float64."""
    eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"].get("groups", 1))
    mult = float(cfg.get("residual_mult", 1.0))
    x = _w(st, "embed")[torch.as_tensor(tokens, dtype=torch.long)]
    after = []
    for i, first_of_pass in layer_runs(cfg):
        if first_of_pass is not None:
            x = x + _w(st, "loop.step")[first_of_pass]
        entry = cfg["layers"][i]
        h = group_norm(x, _w(st, f"l{i}.norm1"), groups, eps)
        if f"l{i}.canon1" in st:
            h = input_conv(h, _w(st, f"l{i}.canon1"))
        kind, m, p = entry["type"], entry["mixer"], f"l{i}.mix."
        if kind == "latent_attention":
            y = latent_attention(h, st, p, m, eps)
        elif kind == "mamba1":
            y = mamba1(h, st, p, m)
        elif kind == "attention":
            y = window_attention(h, st, p, m, eps)
        else:
            raise ValueError(kind)
        x = x + mult * y
        mlp = entry.get("mlp")
        if mlp is not None:
            h = group_norm(x, _w(st, f"l{i}.norm2"), groups, eps)
            if f"l{i}.canon2" in st:
                h = input_conv(h, _w(st, f"l{i}.canon2"))
            y = gated_ff(h, st, f"l{i}.mlp.") if mlp["kind"] == "dense" else moe_ff(h, st, f"l{i}.mlp.", mlp)
            x = x + mult * y
        after.append(x.clone())
    h = group_norm(x, _w(st, "final.norm"), groups, eps)
    logits = h @ _w(st, "head").T
    cap = float(cfg.get("logit_softcap") or 0.0)
    if cap > 0.0:
        logits = cap * torch.tanh(logits / cap)
    return logits, torch.stack(after)

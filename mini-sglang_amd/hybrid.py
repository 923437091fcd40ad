"""Hybrid decoder stack: latent-attention layers and linear-recurrence ("lightning") layers with routed-expert
feed-forwards and norm-after-sum residuals (the Nidorax design; any order and any sizes, all read from its config.json).

Per layer   x <- norm1(alpha x + mixer(x));  x <- norm2(alpha x + ff(x)),  norm(s) = s / sqrt(mean(s^2) + eps) * (1 + w).
The residual stream x lives in fp32; `h` is its copy in the model dtype that the projections read.

latent attention   q = W_q h per head [d unrotated | r rotated];  W_dkv h = [latent (RMS-normed, weight dkv.norm) | one
                   rotated key part shared by the heads];  cached per token: the latent c and the rotated part (R + r numbers).
                   The per-head key W_uk c is never built: the query is carried into latent space once per token
                   (q_abs = W_uk^T q_unrotated, a grouped product over heads), scores are q_abs . c + q_r . k_r, the softmax-
                   weighted LATENT is accumulated and W_uv is applied to it afterwards (grouped product), so prefill portions
                   and decoded tokens read the same R + r numbers per key whatever the head count.  A layer with `kv_from`
                   reads the rows another layer wrote in the same forward.
lightning          S <- decay_h S + k v^T, o = S^T q with q, k, v = SiLU(projections); fp32 state per (request, head) in the
                   cache's state rows; heads concatenated, RMS-normed (plain weight), gated by sigmoid(W_g h).
feed-forward       fp32 router (softmax, bias-corrected choice, group-limited top-k) inside the launch of the norm before it
                   (short batches) or on product-kernel logits (long ones), (token, choice) pairs bucketed by expert on the
                   device, two segmented grouped products (up with ReLU^2, down), the weighted sum of a token's choices folded
                   into the norm that follows.

A second residual scheme, `pre_norm_depth` (the Bedarax design), runs the same loop with other pieces:

stream             X_0 = rms_unit(embed[token]) * w_e;  per layer  s = x + mixer(norm1(x)),  X_(i+1) = s + ff(norm2(s)),
                   x <- sum_{j <= i+1} c_i[j] X_j  (every layer averages the whole history with its own weights); norms have
                   plain weights; the LM head is its own matrix.  The history is one fp32 tensor [layers + 1, tokens, W].
attention          q, k, v projections without rotation; the heads' scores are mixed by an H x H table before the softmax;
                   only the last `window` keys are visible; from the second value-mixing layer on, the cached v is blended
                   with the first such layer's v of the same token; a sigmoid gate per head scales the output.  Cached per
                   token: k [G d] and the blended v [G dv] in the pool's token slots.
delta / channel_delta   q, k, v pass a short causal convolution over time (+ SiLU), q and k become unit vectors per head;
                   S <- g S, u = beta (v - S^T k), S <- S + k u^T, o = S^T q with one decay g per head (delta) or per key
                   channel through a low-rank projection (channel_delta); per-head RMS norm, gated by SiLU / sigmoid.
                   State per request: S in fp32 and the last taps - 1 inputs of the convolution.
feed-forward       dense with a polynomial activation of row-normalised powers, or routed experts silu(W_g h) * (W_u h)
                   chosen by the largest router logits (softmax over the chosen logits only).

A third scheme, `parallel_shift` (the Givavik design), has ONE norm per layer that feeds the mixer and the feed-forward side by side:

stream             x_0 = s_e embed[token] + pair[(previous token * m_p + token * m_c) mod B] (row B for a sequence's first token);
                   per layer  h = rms_unit(x) (1 + w),  g = h + (h of the token before - h) * shift  (zero before the first token),
                   x <- x + ls1 * mixer(g) + ls2 * ff(h);  final norm, then the LM head matrix.  Per request the state rows keep
                   the last token id and, for every layer, the last h (fp32).
latent attention   as above, with the rotated parts paired (2i, 2i + 1) and a learned sink per head: one more term exp(sink_h) in
                   the softmax denominator that has no key and no value.
parallel           two mixers on the same g, their results scaled and added:
  sigmoid attention  H query heads over G key/value heads with projection biases, rotation of the leading entries of each head,
                   q and k divided by their root mean square, score = cap tanh(scale q.k / cap), weight of a visible key =
                   sigmoid(score + b_h), no normalisation over keys.  Cached per token: k [G d] and v [G dv].
  state space      Mamba-2: in-projection [z | x | B | C | dt], causal convolution + SiLU over x, B, C, dt = softplus(dt + bias),
                   S <- exp(-exp(A) dt) S + dt B x^T, y = S^T C + D x, y * silu(z) RMS-normed in equal groups, output projection.
                   State per request: S in fp32 and the last taps - 1 inputs of the convolution.
                   Both mixers share one input projection and one output projection (their outputs side by side in one row).
feed-forward       W_down xielu(W_up h) with two learned numbers per layer.

A fourth scheme, `pre_norm_conv` (the Piladra design): plain pre-norm residuals with a multiplier, norms in groups, a short causal
convolution in front of every sublayer, and a run of layers that is repeated with the same weights:

stream             x_0 = embed[token];  per layer  x <- x + m mixer(c1(norm1(x))),  x <- x + m ff(c2(norm2(x)));  a norm divides every
                   one of `groups` equal parts of a row by its own root mean square, then multiplies by w;  c(h)[t] = h[t] + sum_j
                   taps[:, j] h[t - (n - 1) + j] per channel (zero before the sequence; the last n - 1 normed rows of every sublayer are
                   part of a request's state).  Layers start .. stop - 1 run `times` times in a row with the same weights, every pass
                   with cache and state of its own; before the first layer of pass t the vector step[t] is added to x.  Output:
                   final norm, head matrix, logits <- cap tanh(logits / cap).
latent attention   as above with the rotated parts split in halves, an unscaled rotation, and the concatenated heads multiplied by
                   sigmoid(W_g h) before the output projection.
sink_attention     H query heads over G key/value heads, rotation of the leading entries of each head (frequencies rescaled by
                   wavelength: short ones kept, long ones divided by a factor, a linear blend between), every value head divided by
                   its root mean square before it is cached, keys 0 <= i - j < window visible, softmax with one more term
                   exp(sink_h) in the denominator.  Cached per token: k [G d] and the normed v [G dv].
mamba1             in-projection [x | z], causal convolution (+ bias) + SiLU over x, W_x x = [dt | B | C], dt = softplus(W_dt dt +
                   bias), S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n, y_c = sum_n S[c, n] C_n + D_c x_c, y silu(z), output
                   projection.  State per request: S [inner, state] in fp32 and the last taps - 1 inputs of the convolution.
feed-forward       W_down (silu(W_gate h) * (W_up h)), or routed experts of that form: scores = sigmoid(router logits), the `top`
                   largest chosen, a chosen expert runs on score * h (the weight enters BEFORE the expert, so the choices' outputs are
                   summed as they are), plus a shared expert that every token runs.

Kernels: csrc/seqmix.hip, csrc/mix_delta.hip, csrc/mix_par.hip and csrc/mix_scan.hip through mixops.py; plain projections through the library GEMM
(mixops.linear).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

import torch

from . import flashinfer_compat as fi
from . import mixops


@dataclass(frozen=True)
class MoeSpec:
    experts: int
    top: int
    ff: int
    groups: int = 1
    keep: int = 1
    gated: bool = False             # expert = W_down (silu(W_gate h) * (W_up h)) instead of W_down relu(W_up h)^2
    pick: str = "scores"            # "scores": softmax over all experts, corrected group-limited choice; "logits": the largest
                                    # logits (+ bias) win and the weights are the softmax over the winners; "sigmoid_input": the
                                    # largest logits win, weight = sigmoid(logit), and it multiplies the expert's INPUT
    shared_ff: int = 0              # inner size of a shared expert that every token runs (0: none)


@dataclass(frozen=True)
class DenseFfSpec:
    ff: int
    act: str = "poly_norm"          # "poly_norm": c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 with N = divide a row by its root mean square;
                                    # "xielu": softplus(p) z^2 + z / 2 above zero, (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2 below
                                    # "silu_gate": W_down (silu(W_gate h) * (W_up h))


@dataclass(frozen=True)
class LayerSpec:
    kind: str                       # "latent_attention" | "lightning" | "attention" | "delta" | "channel_delta" | "parallel" |
                                    # "sink_attention" | "mamba1";
                                    # inside a "parallel" pair: "sigmoid_attention" | "state_space"
    heads: int
    dim: int                        # unrotated query/key size per head (lightning: query/key size)
    vdim: int
    rot_dim: int = 0
    kv_rank: int = 0
    kv_from: Optional[int] = None
    scale: float = 1.0
    rot_dims: int = 0               # how many entries of the rotated part turn
    rot_base: float = 10000.0
    rot_scaling: Optional[Tuple[Tuple[str, float], ...]] = None
    decay: Tuple[float, ...] = ()
    mlp: Optional[Any] = None       # MoeSpec | DenseFfSpec | None
    kv_heads: int = 0               # attention / delta kinds: key (and attention: value) heads; query head h reads h // (heads / kv_heads)
    window: int = 0                 # attention: keys i - window < j <= i are visible; 0 = all earlier keys
    v_mix: bool = False             # attention: blends its values with those of the first such layer
    conv: int = 1                   # delta kinds: taps of the causal convolution over q, k, v
    decay_rank: int = 0             # channel_delta: inner sizes of the two-step decay and gate projections
    gate_rank: int = 0
    interleaved: bool = False       # rotation pairs entries (2i, 2i + 1) instead of (i, i + half)
    sink: bool = False              # latent attention: a learned term per head in the softmax denominator
    softcap: float = 0.0            # sigmoid attention: score <- cap tanh(score / cap); 0 = none
    norm_groups: int = 1            # state space: the gated output is RMS-normed in this many equal parts
    left: Optional["LayerSpec"] = None   # parallel: the two mixers that read the same input, and the scales of their sum
    right: Optional["LayerSpec"] = None
    left_scale: float = 1.0
    right_scale: float = 1.0
    out_gate: bool = False          # latent attention: the concatenated heads are multiplied by sigmoid(W_g h)
    v_norm: bool = False            # sink attention: every value head is divided by its root mean square before it is cached
    dt_rank: int = 0                # mamba1: inner size of the two-step step-size projection
    # state space: heads x vdim = inner size, dim = state size per head, kv_heads = groups of B / C, conv = taps
    # mamba1: heads = 1, vdim = inner size (channels), dim = state size per channel, conv = taps

    @property
    def recurrent(self) -> bool:
        return self.kind in ("lightning", "delta", "channel_delta", "state_space", "mamba1") or \
            (self.kind == "parallel" and (self.left.recurrent or self.right.recurrent))


@dataclass(frozen=True)
class HybridConfig:
    """What a Nidorax config.json states, nothing else; `max_position` is the engine's sequence limit (the design has none)."""
    vocab_size: int
    hidden_size: int
    layers: Tuple[LayerSpec, ...]
    rms_norm_eps: float
    postln_alpha: float = 1.0
    max_position: int = 1 << 20
    name: str = "Nidorax"
    residual: str = "post_norm"     # "post_norm": x <- norm(alpha x + f(x)), weights stored as offsets from one, tied head;
                                    # "pre_norm_depth": x + f(norm(x)), depth-averaged history, normed embedding, own head;
                                    # "parallel_shift": x + ls1 mixer(shift(norm(x))) + ls2 ff(norm(x)), own head
    embed_scale: float = 1.0        # parallel_shift: the embedding row is multiplied by this
    pair_embed: Optional[Tuple[int, int, int]] = None  # (buckets, multiplier of the previous id, multiplier of the id) of the pair table
    token_shift: bool = False       # every layer's mixer reads a blend of this token's and the previous token's normed row
    # "pre_norm_conv": x + m f(conv(norm(x))), norms in groups, a looped run of layers, capped logits, own head
    norm_groups: int = 1            # a norm divides each of this many equal parts of a row by its own root mean square
    conv_taps: int = 0              # taps of the causal convolution in front of every sublayer (0: none)
    residual_mult: float = 1.0
    logit_softcap: float = 0.0      # logits <- cap tanh(logits / cap); 0 = none
    loop: Optional[Tuple[int, int, int]] = None   # (start, stop, times): layers start .. stop - 1 run `times` times in a row

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def runs(self) -> Tuple[Tuple[int, Optional[int]], ...]:
        """(layer, pass number if the layer opens a pass of the loop else None) in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return tuple((i, None) for i in range(n))
        a, b, times = self.loop
        out: List[Tuple[int, Optional[int]]] = [(i, None) for i in range(a)]
        for t in range(times):
            out += [(i, t if i == a else None) for i in range(a, b)]
        return tuple(out + [(i, None) for i in range(b, n)])

    @property
    def cache_layers(self) -> Tuple[LayerSpec, ...]:
        """One spec per layer RUN: every pass of a looped layer has cache rows and state of its own."""
        return tuple(self.layers[i] for i, _ in self.runs)

    @staticmethod
    def from_json(cfg: Dict[str, Any], name: str = "Nidorax") -> "HybridConfig":
        layers: List[LayerSpec] = []
        for i, entry in enumerate(cfg["layers"]):
            m, mlp = entry["mixer"], entry.get("mlp")
            moe = None
            if mlp is not None:
                if mlp.get("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                r, g = mlp["router"], mlp["router"].get("groups") or {}
                moe = MoeSpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]),
                              groups=int(g.get("count", 1)), keep=int(g.get("keep", g.get("count", 1))))
            if entry["type"] == "latent_attention":
                rot = m["rot"]
                sc = rot.get("scaling")
                layers.append(LayerSpec(
                    kind="latent_attention", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                    rot_dim=int(m["rot_dim"]), kv_rank=int(m["kv_rank"]),
                    kv_from=None if m.get("kv_from") is None else int(m["kv_from"]), scale=float(m["scale"]),
                    rot_dims=int(rot.get("dims", m["rot_dim"])), rot_base=float(rot["base"]),
                    rot_scaling=None if not sc else tuple(sorted((k, float(v)) for k, v in sc.items())), mlp=moe))
            elif entry["type"] == "lightning":
                layers.append(LayerSpec(kind="lightning", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                                        decay=tuple(float(x) for x in m["decay"]), mlp=moe))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {entry['type']!r}")
        for i, s in enumerate(layers):
            if s.kind == "latent_attention" and s.kv_from is not None:
                o = layers[s.kv_from] if 0 <= s.kv_from < i else None
                if o is None or o.kind != "latent_attention" or o.kv_from is not None or \
                        (o.kv_rank, o.rot_dim) != (s.kv_rank, s.rot_dim):
                    raise ValueError(f"layer {i}: kv_from = {s.kv_from} is not an earlier latent layer with its own keys of equal size")
            if s.kind == "lightning" and len(s.decay) != s.heads:
                raise ValueError(f"layer {i}: {len(s.decay)} decays for {s.heads} heads")
        return HybridConfig(vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=tuple(layers),
                            rms_norm_eps=float(cfg["norm"]["eps"]), postln_alpha=float(cfg["postln_alpha"]), name=name)


def _ff_spec(i: int, mlp: Optional[Dict[str, Any]]):
    if mlp is None:
        return None
    kind = mlp.get("kind")
    if kind == "dense":
        return DenseFfSpec(ff=int(mlp["ff"]))
    if kind == "moe":
        r = mlp["router"]
        return MoeSpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]), gated=True, pick="logits")
    raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")


def bedarax_config(cfg: Dict[str, Any], shapes: Optional[Dict[str, Tuple[int, ...]]] = None, name: str = "Bedarax") -> HybridConfig:
    """config.json of a Bedarax model -> HybridConfig.  `shapes` (tensor name -> shape, from the checkpoint's header) gives the
    sizes config.json leaves to the tensors: the inner sizes of a channel_delta layer's two-step projections."""
    shapes = shapes or {}
    layers: List[LayerSpec] = []
    for i, entry in enumerate(cfg["layers"]):
        m, kind = entry["mixer"], entry["type"]
        ff = _ff_spec(i, entry.get("mlp"))
        H, G = int(m["heads"]), int(m.get("kv_heads", m["heads"]))
        if H % G:
            raise ValueError(f"layer {i}: {H} heads over {G} key heads")
        if kind == "attention":
            layers.append(LayerSpec(kind="attention", heads=H, kv_heads=G, dim=int(m["dim"]), vdim=int(m["vdim"]),
                                    scale=float(m["scale"]), window=int((m.get("mask") or {}).get("size", 0)),
                                    v_mix=bool(m.get("v_mix", False)), mlp=ff))
        elif kind in ("delta", "channel_delta"):
            d = int(m["dim"])
            ra = rg = 0
            if kind == "channel_delta":
                ra = int(shapes.get(f"l{i}.mix.a1", (max(d // 2, 8),))[0])
                rg = int(shapes.get(f"l{i}.mix.g1", (max(d // 2, 8),))[0])
            taps = m.get("conv") or shapes.get(f"l{i}.mix.q.conv", (0, 1))[1]  # config.json, else the taps tensor's width
            layers.append(LayerSpec(kind=kind, heads=H, kv_heads=G, dim=d, vdim=int(m["vdim"]), conv=int(taps),
                                    decay_rank=ra, gate_rank=rg, mlp=ff))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
    mixing = [s for s in layers if s.kind == "attention" and s.v_mix]
    if any((s.kv_heads, s.vdim) != (mixing[0].kv_heads, mixing[0].vdim) for s in mixing):
        raise ValueError("value-mixing attention layers must agree in key heads and value size")
    return HybridConfig(vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=tuple(layers),
                        rms_norm_eps=float(cfg["norm"]["eps"]), name=name, residual="pre_norm_depth")


def _rot(m: Dict[str, Any], default_dims: int) -> Tuple[int, float]:
    rot = m.get("rot") or {}
    return int(rot.get("dims", default_dims)), float(rot.get("base", 10000.0))


def givavik_config(cfg: Dict[str, Any], name: str = "Givavik") -> HybridConfig:
    """config.json of a Givavik model -> HybridConfig."""
    layers: List[LayerSpec] = []
    for i, entry in enumerate(cfg["layers"]):
        m, kind, mlp = entry["mixer"], entry["type"], entry.get("mlp")
        ff = None
        if mlp is not None:
            if mlp.get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            ff = DenseFfSpec(ff=int(mlp["ff"]), act="xielu")
        if kind == "latent_attention":
            dims, base = _rot(m, int(m["rot_dim"]))
            layers.append(LayerSpec(
                kind="latent_attention", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), rot_dim=int(m["rot_dim"]),
                kv_rank=int(m["kv_rank"]), kv_from=None if m.get("kv_from") is None else int(m["kv_from"]), scale=float(m["scale"]),
                rot_dims=dims, rot_base=base, interleaved=True, sink=True, mlp=ff))
        elif kind == "parallel":
            a, b = m["left"], m["right"]
            H, G = int(a["heads"]), int(a.get("kv_heads", a["heads"]))
            dims, base = _rot(a, 0)
            left = LayerSpec(kind="sigmoid_attention", heads=H, kv_heads=G, dim=int(a["dim"]), vdim=int(a["vdim"]), scale=float(a["scale"]),
                             softcap=float(a.get("softcap") or 0.0), rot_dims=dims, rot_base=base, interleaved=True)
            Hs, Gs = int(b["heads"]), int(b.get("groups", 1))
            right = LayerSpec(kind="state_space", heads=Hs, kv_heads=Gs, dim=int(b["state"]), vdim=int(b["vdim"]), conv=int(b["conv"]),
                              norm_groups=int(b.get("norm_groups", 1)))
            if H % G or Hs % Gs or (Hs * right.vdim) % right.norm_groups or dims % 2 or dims > left.dim:
                raise ValueError(f"layer {i}: head / group / rotation sizes do not divide")
            layers.append(LayerSpec(kind="parallel", heads=H, dim=left.dim, vdim=left.vdim, left=left, right=right,
                                    left_scale=float(m.get("left_scale", 1.0)), right_scale=float(m.get("right_scale", 1.0)), mlp=ff))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
    for i, s in enumerate(layers):
        if s.kind == "latent_attention" and s.kv_from is not None:
            o = layers[s.kv_from] if 0 <= s.kv_from < i else None
            if o is None or o.kind != "latent_attention" or o.kv_from is not None or \
                    (o.kv_rank, o.rot_dim, o.rot_dims, o.rot_base) != (s.kv_rank, s.rot_dim, s.rot_dims, s.rot_base):
                raise ValueError(f"layer {i}: kv_from = {s.kv_from} is not an earlier latent layer with its own keys of equal size and rotation")
    e = cfg.get("embedding") or {}
    bg = e.get("bigram")
    pair = None if not bg else (int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"]))
    return HybridConfig(vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=tuple(layers), rms_norm_eps=float(cfg["norm"]["eps"]),
                        name=name, residual="parallel_shift", embed_scale=float(e.get("scale", 1.0)), pair_embed=pair, token_shift=True)


def piladra_config(cfg: Dict[str, Any], name: str = "Piladra") -> HybridConfig:
    """config.json of a Piladra model -> HybridConfig."""
    layers: List[LayerSpec] = []
    for i, entry in enumerate(cfg["layers"]):
        m, kind, mlp = entry["mixer"], entry["type"], entry.get("mlp")
        ff = None
        if mlp is not None:
            if mlp.get("kind") == "dense":
                ff = DenseFfSpec(ff=int(mlp["ff"]), act="silu_gate")
            elif mlp.get("kind") == "moe":
                r, sh = mlp["router"], mlp.get("shared")
                ff = MoeSpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]), gated=True, pick="sigmoid_input",
                             shared_ff=int(sh["ff"]) if sh else 0)
                if not 1 <= ff.top <= ff.experts:
                    raise ValueError(f"layer {i}: top {ff.top} of {ff.experts} experts")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        if kind == "latent_attention":
            r = int(m["rot_dim"])
            dims, base = _rot(m, r)
            if dims != r or r % 2:
                raise ValueError(f"layer {i}: the rotated part has {r} entries, the rotation turns {dims}")
            layers.append(LayerSpec(kind="latent_attention", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), rot_dim=r,
                                    kv_rank=int(m["kv_rank"]), scale=float(m["scale"]), rot_dims=dims, rot_base=base, out_gate=True, mlp=ff))
        elif kind == "attention":
            H, G = int(m["heads"]), int(m.get("kv_heads", m["heads"]))
            dims, base = _rot(m, 0)
            sc = (m.get("rot") or {}).get("scaling")
            if H % G or dims % 2 or dims > int(m["dim"]):
                raise ValueError(f"layer {i}: head / rotation sizes do not divide")
            layers.append(LayerSpec(kind="sink_attention", heads=H, kv_heads=G, dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]),
                                    window=int((m.get("mask") or {}).get("size", 0)), rot_dims=dims, rot_base=base,
                                    rot_scaling=None if not sc else tuple(sorted((k, float(v)) for k, v in sc.items())),
                                    sink=True, v_norm=True, mlp=ff))
        elif kind == "mamba1":
            layers.append(LayerSpec(kind="mamba1", heads=1, dim=int(m["state"]), vdim=int(m["inner"]), conv=int(m["conv"]),
                                    dt_rank=int(m["dt_rank"]), mlp=ff))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
    loop = cfg.get("loop")
    lp = None
    if loop:
        lp = (int(loop["start"]), int(loop["stop"]), int(loop["times"]))
        if not (0 <= lp[0] <= lp[1] <= len(layers) and lp[2] >= 1):
            raise ValueError(f"loop {lp} over {len(layers)} layers")
    W, groups = int(cfg["width"]), int(cfg["norm"].get("groups", 1))
    if W % groups:
        raise ValueError(f"a row of {W} in {groups} groups")
    return HybridConfig(vocab_size=int(cfg["vocab"]), hidden_size=W, layers=tuple(layers), rms_norm_eps=float(cfg["norm"]["eps"]), name=name,
                        residual="pre_norm_conv", norm_groups=groups, conv_taps=int((cfg.get("canon") or {}).get("taps", 0)),
                        residual_mult=float(cfg.get("residual_mult", 1.0)), logit_softcap=float(cfg.get("logit_softcap") or 0.0), loop=lp)


def wavelength_scaled_rotary_table(dims: int, base: float, scaling: Optional[Dict[str, float]], max_position: int, device) -> torch.Tensor:
    """fp32 [max_position, dims] = cos | sin of position * f_i, f_i = base^(-2i / dims) rescaled by wavelength l = 2 pi / f: kept where
    l < original / high, divided by `factor` where l > original / low, blended linearly in original / l between; float64, rounded once."""
    f = float(base) ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims)
    if scaling:
        factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        wave = 2.0 * math.pi / f
        blend = (orig / wave - low) / (high - low) if high != low else torch.zeros_like(f)
        mixed = (1.0 - blend) * f / factor + blend * f
        f = torch.where(wave < orig / high, f, torch.where(wave > orig / low, f / factor, mixed))
    ang = torch.arange(max_position, dtype=torch.float64)[:, None] * f[None, :]
    return torch.cat((ang.cos(), ang.sin()), dim=-1).to(torch.float32).to(device)


def plain_rotary_table(dims: int, base: float, max_position: int, device) -> torch.Tensor:
    """fp32 [max_position, dims] = cos | sin of position * base^(-2i / dims), i < dims / 2; angles in float64, rounded once."""
    f = float(base) ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims)
    ang = torch.arange(max_position, dtype=torch.float64)[:, None] * f[None, :]
    return torch.cat((ang.cos(), ang.sin()), dim=-1).to(torch.float32).to(device)


def rotary_table(spec: LayerSpec, max_position: int, device) -> torch.Tensor:
    """fp32 [max_position, rot_dims] = cos | sin of the layer's (scaled) rotary angles, amplitude folded in."""
    sc = dict(spec.rot_scaling) if spec.rot_scaling else None
    factor = sc["factor"] if sc else 1.0
    scaling = dict(rope_type="yarn", factor=factor, original_max_position_embeddings=sc["original"] if sc else 1.0,
                   beta_fast=sc["fast"] if sc else 2.0, beta_slow=sc["slow"] if sc else 1.0, hi_cap=spec.rot_dims - 1,
                   min_span=0.001, amplitude=0.1 * math.log(factor) + 1.0, float64_table=True)
    return fi.build_cos_sin_cache(spec.rot_dims, max_position, spec.rot_base, scaling, device=device)


class _Layer:
    __slots__ = ("spec", "w_in", "o", "norm1", "norm2", "uk_t", "uv", "c_norm", "cos_sin", "out_norm", "decay", "router",
                 "bias", "up", "down", "talk", "lam", "taps", "rate", "dt_bias", "a2", "g2", "act", "depth_w",
                 "sink", "ls1", "ls2", "shift", "in_bias", "out_bias", "pb", "skip", "conv_b", "sum_bias", "canon1", "canon2", "w_x", "w_dt",
                 "sh_up", "sh_down")

    def __init__(self, spec: LayerSpec) -> None:
        self.spec = spec
        for k in self.__slots__[1:]:
            setattr(self, k, None)


class HybridDecoder:
    ROUTE_FUSE_MAX_TOKENS = 128

    def __init__(self, cfg: HybridConfig, *, dtype: torch.dtype, device: torch.device, tp_rank: int = 0, tp_size: int = 1,
                 seed: int = 42, init_std: float = 0.02, max_position: Optional[int] = None, **_unused: Any) -> None:
        if tp_size != 1:
            raise NotImplementedError("the hybrid decoder runs on one rank (no tensor-parallel sharding of its layers yet)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise TypeError(f"hybrid decoder: dtype {dtype} (bfloat16 or float32)")
        self.cfg, self.dtype, self.device = cfg, dtype, device
        self.tp_rank, self.tp_size = tp_rank, tp_size
        self.max_position = int(max_position or cfg.max_position)
        g = torch.Generator(device=device)
        g.manual_seed(seed)

        def w(*shape, std=init_std):  # seeded weights until a checkpoint is loaded
            return (torch.randn(shape, generator=g, device=device, dtype=torch.float32) * std).to(dtype)

        W = cfg.hidden_size
        self.pre_norm = cfg.residual == "pre_norm_depth"
        self.parallel = cfg.residual == "parallel_shift"
        self.conv_stream = cfg.residual == "pre_norm_conv"
        self.embed_norm = self.head = self.pair_table = self.loop_step = None
        self.embed = w(cfg.vocab_size, W, std=1.0)
        self.final_norm = w(W, std=0.1)
        self.layers: List[_Layer] = []
        tables: Dict[tuple, torch.Tensor] = {}

        def f32(*shape, std=init_std, mean=0.0):  # what the kernels read as fp32: norm offsets, per-column scales, biases, rates
            return mean + torch.randn(shape, generator=g, device=device, dtype=torch.float32) * std

        def plain_table(dims, base):
            key = ("plain", dims, base)
            if key not in tables:
                tables[key] = plain_rotary_table(dims, base, self.max_position, device)
            return tables[key]

        for spec in cfg.layers:
            L = _Layer(spec)
            H, d, dv = spec.heads, spec.dim, spec.vdim
            L.norm1 = w(W, std=0.1)
            if self.parallel:
                L.norm1, L.ls1, L.ls2 = f32(W, std=0.1), f32(W, std=0.2, mean=1.0), f32(W, std=0.2, mean=1.0)
                L.shift = f32(W, std=0.2, mean=0.5) if cfg.token_shift else None
            if spec.kind == "parallel":
                a, b = spec.left, spec.right
                G, Gs, N = a.kv_heads, b.kv_heads, b.dim
                n_left, inner = (H + G) * d + G * dv, b.heads * b.vdim
                # one input projection: q | k | v of the attention, then z | x | B | C | dt of the state-space layer
                L.w_in = w(n_left + 2 * inner + 2 * Gs * N + b.heads, W, std=W ** -0.5)
                L.in_bias = f32(n_left, std=0.1)
                L.pb = f32(H, std=1.0, mean=-2.0)
                L.cos_sin = plain_table(a.rot_dims, a.rot_base) if a.rot_dims else None
                L.taps = w(inner + 2 * Gs * N, b.conv, std=b.conv ** -0.5)
                L.conv_b = w(inner + 2 * Gs * N, std=0.1)
                L.dt_bias, L.rate, L.skip = f32(b.heads, std=0.5), -torch.exp(f32(b.heads, std=0.5)), f32(b.heads, std=0.5, mean=1.0)
                L.out_norm = f32(inner, std=0.1, mean=1.0)
                # one output projection over the row [attention heads | state-space channels]
                L.o = w(W, H * dv + inner, std=(H * dv + inner) ** -0.5)
                L.out_bias = f32(W, std=0.1)
            elif spec.kind == "mamba1":
                inner, N, dr = spec.vdim, spec.dim, spec.dt_rank
                L.w_in = w(2 * inner, W, std=W ** -0.5)           # x | z
                L.taps = w(inner, spec.conv, std=spec.conv ** -0.5)
                L.conv_b = w(inner, std=0.1)
                L.w_x = w(dr + 2 * N, inner, std=inner ** -0.5)   # dt | B | C
                L.w_dt = w(inner, dr, std=dr ** -0.5)
                L.dt_bias, L.skip = f32(inner, std=0.5, mean=-2.0), f32(inner, std=0.3, mean=1.0)
                L.rate = -torch.exp(f32(inner, N, std=0.5))       # A = -exp(A_log)
                L.o = w(W, inner, std=inner ** -0.5)
            elif spec.kind == "sink_attention":
                G = spec.kv_heads
                L.w_in = w(H * d + G * d + G * dv, W, std=W ** -0.5)  # q | k | v
                L.o = w(W, H * dv, std=(H * dv) ** -0.5)
                L.sink = f32(H, std=1.0)
                if spec.rot_dims:
                    key = ("wave", spec.rot_dims, spec.rot_base, spec.rot_scaling)
                    if key not in tables:
                        tables[key] = wavelength_scaled_rotary_table(spec.rot_dims, spec.rot_base, dict(spec.rot_scaling) if spec.rot_scaling else None,
                                                                     self.max_position, device)
                    L.cos_sin = tables[key]
            elif spec.kind == "latent_attention":
                r, R = spec.rot_dim, spec.kv_rank
                L.w_in = w(H * (d + r) + (0 if spec.kv_from is not None else R + r) + (H * dv if spec.out_gate else 0), W, std=W ** -0.5)
                L.uk_t = w(H, R, d, std=R ** -0.5)   # W_uk per head, transposed: q_abs = q_unrotated @ uk_t[h]^T
                L.uv = w(H, dv, R, std=R ** -0.5)
                L.o = w(W, H * dv, std=(H * dv) ** -0.5)
                L.c_norm = None if spec.kv_from is not None else (1.0 + w(R, std=0.1).float()).to(dtype)
                L.sink = f32(H, std=1.0) if spec.sink else None
                if spec.interleaved or self.conv_stream:
                    L.cos_sin = plain_table(spec.rot_dims, spec.rot_base)
                else:
                    key = (spec.rot_dims, spec.rot_base, spec.rot_scaling)
                    if key not in tables:
                        tables[key] = rotary_table(spec, self.max_position, device)
                    L.cos_sin = tables[key]
            elif spec.kind == "lightning":
                L.w_in = w(2 * H * d + 2 * H * dv, W, std=W ** -0.5)  # q | k | v | gate
                L.o = w(W, H * dv, std=(H * dv) ** -0.5)
                L.out_norm = (1.0 + w(H * dv, std=0.1).float()).to(dtype)
                L.decay = torch.tensor(spec.decay, dtype=torch.float32, device=device)
            elif spec.kind == "attention":
                G = spec.kv_heads
                L.w_in = w(H * d + G * d + G * dv + H, W, std=W ** -0.5)  # q | k | v | one gate per head
                L.o = w(W, H * dv, std=(H * dv) ** -0.5)
                L.talk = torch.eye(H, dtype=torch.float32, device=device) + w(H, H, std=0.2).float()
                L.lam = w(1, std=0.3)
            else:  # delta, channel_delta
                G, C = spec.kv_heads, 2 * spec.kv_heads * d + H * dv
                tail = spec.decay_rank + spec.gate_rank if spec.kind == "channel_delta" else H + H * dv
                L.w_in = w(C + H + tail, W, std=W ** -0.5)  # q | k | v | beta | decay input | gate input
                L.taps = w(C, spec.conv, std=spec.conv ** -0.5)
                n_decay = H * d if spec.kind == "channel_delta" else H
                L.rate = -torch.exp(w(H, std=0.5).float())  # -exp(A_log)
                L.dt_bias = w(n_decay, std=0.5).float()
                if spec.kind == "channel_delta":
                    L.a2 = w(H * d, spec.decay_rank, std=spec.decay_rank ** -0.5)
                    L.g2 = w(H * dv, spec.gate_rank, std=spec.gate_rank ** -0.5)
                L.out_norm = (1.0 + w(dv, std=0.1).float()).to(dtype)
                L.o = w(W, H * dv, std=(H * dv) ** -0.5)
            m = spec.mlp
            if isinstance(m, MoeSpec):
                L.norm2 = w(W, std=0.1)
                L.router = w(m.experts, W, std=W ** -0.5)
                L.bias = None if m.pick == "sigmoid_input" else w(m.experts, std=0.01)
                L.up = w(m.experts, (2 if m.gated else 1) * m.ff, W, std=W ** -0.5)  # gated: every expert's gate rows, then its up rows
                L.down = w(m.experts, W, m.ff, std=m.ff ** -0.5)
            elif isinstance(m, DenseFfSpec):
                L.norm2 = None if self.parallel else w(W, std=0.1)
                L.up = w((2 if m.act == "silu_gate" else 1) * m.ff, W, std=W ** -0.5)  # silu_gate: the gate rows, then the up rows
                L.down = w(W, m.ff, std=m.ff ** -0.5)
                L.act = torch.tensor([0.3, -0.4] if m.act == "xielu" else [1.0, 0.3, 0.1, 0.01], dtype=torch.float32, device=device)
            if isinstance(m, MoeSpec) and m.shared_ff:
                L.sh_up = w(2 * m.shared_ff, W, std=W ** -0.5)
                L.sh_down = w(W, m.shared_ff, std=m.shared_ff ** -0.5)
            if self.conv_stream:
                L.norm1, L.norm2 = (1.0 + L.norm1.float()).to(dtype), None if L.norm2 is None else (1.0 + L.norm2.float()).to(dtype)
                if cfg.conv_taps:
                    L.canon1 = w(W, cfg.conv_taps, std=0.3)
                    L.canon2 = w(W, cfg.conv_taps, std=0.3) if m is not None else None
            if self.pre_norm:
                L.norm1, L.norm2 = (1.0 + L.norm1.float()).to(dtype), None if L.norm2 is None else (1.0 + L.norm2.float()).to(dtype)
                c = torch.full((len(self.layers) + 2,), 0.1, dtype=torch.float32, device=device)
                c[-1] = 1.0
                L.depth_w = c
            self.layers.append(L)
        if self.pre_norm:
            self.final_norm = (1.0 + self.final_norm.float()).to(dtype)
            self.embed_norm = (1.0 + w(W, std=0.1).float()).to(dtype)
            self.head = w(cfg.vocab_size, W, std=W ** -0.5)
        if self.conv_stream:
            self.final_norm = (1.0 + self.final_norm.float()).to(dtype)
            self.head = w(cfg.vocab_size, W, std=W ** -0.5)
            if cfg.loop is not None:
                self.loop_step = f32(cfg.loop[2], W, std=0.3)
        if self.parallel:
            self.final_norm = f32(W, std=0.1)
            self.head = w(cfg.vocab_size, W, std=W ** -0.5)
            if cfg.pair_embed is not None:
                self.pair_table = w(cfg.pair_embed[0] + 1, W, std=1.0)
            self._derive()

    # ------------------------------------------------------------------ weights
    def _derive(self) -> None:
        """What the kernels read that is a function of loaded tensors: a pair layer's output bias as it enters the residual sum
        (the attention's projection bias times the attention's scale times the layer scale of the mixer)."""
        for L in self.layers:
            if L.spec.kind == "parallel":
                L.sum_bias = (L.out_bias * L.spec.left_scale * L.ls1).contiguous()

    def _tensors(self):
        yield self.embed
        yield self.final_norm
        for t in (self.embed_norm, self.head, self.pair_table, self.loop_step):
            if t is not None:
                yield t
        for L in self.layers:
            for k in ("w_in", "o", "norm1", "norm2", "uk_t", "uv", "c_norm", "out_norm", "router", "bias", "up", "down", "talk", "lam",
                      "taps", "rate", "dt_bias", "a2", "g2", "act", "depth_w", "sink", "ls1", "ls2", "shift", "in_bias", "out_bias", "pb",
                      "skip", "conv_b", "canon1", "canon2", "w_x", "w_dt", "sh_up", "sh_down"):
                t = getattr(L, k)
                if t is not None:
                    yield t

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self._tensors())

    def streamed_bytes_per_step(self) -> int:
        return self.weight_bytes()

    def load_state(self, state: Dict[str, torch.Tensor]) -> None:
        """Overwrite the seeded weights with a checkpoint's tensors (checkpoint names: 'embed', 'final.norm',
        'l<i>.norm1', 'l<i>.mix.<name>', 'l<i>.mlp.e<j>.up' ...), merging what one launch reads together: q | dkv, q | k | v | g,
        the experts of a layer stacked, W_uk split per head and transposed."""
        cfg = self.cfg

        def put(dst: torch.Tensor, src: torch.Tensor) -> None:
            if tuple(dst.shape) != tuple(src.shape):
                raise ValueError(f"checkpoint tensor of shape {tuple(src.shape)} where the config implies {tuple(dst.shape)}")
            dst.copy_(src.to(device=self.device, dtype=torch.float32))  # rounds to the destination's dtype (fp32 tensors stay fp32)

        put(self.embed, state["embed"])
        put(self.final_norm, state["final.norm"])
        if self.pre_norm:
            put(self.embed_norm, state["embed.norm"])
            put(self.head, state["head"])
        if self.parallel:
            put(self.head, state["head"])
            if self.pair_table is not None:
                put(self.pair_table, state["bigram"])
        if self.conv_stream:
            put(self.head, state["head"])
            if self.loop_step is not None:
                put(self.loop_step, state["loop.step"])
        for i, L in enumerate(self.layers):
            s, p = L.spec, f"l{i}.mix."
            H, d, dv = s.heads, s.dim, s.vdim
            put(L.norm1, state[f"l{i}.norm1"])
            if L.canon1 is not None:
                put(L.canon1, state[f"l{i}.canon1"])
            if L.canon2 is not None:
                put(L.canon2, state[f"l{i}.canon2"])
            if L.depth_w is not None:
                put(L.depth_w, state[f"l{i}.dwa"])
            if self.parallel:
                put(L.ls1, state[f"l{i}.ls1"])
                if s.mlp is not None:
                    put(L.ls2, state[f"l{i}.ls2"])
                if L.shift is not None:
                    put(L.shift, state[f"l{i}.shift"])
            if L.sink is not None:
                put(L.sink, state[p + "sink"])
            if s.kind == "parallel":
                a, b = p + "left.", p + "right."
                put(L.w_in, torch.cat([state[a + "q"], state[a + "k"], state[a + "v"], state[b + "in"]], dim=0))
                put(L.in_bias, torch.cat([state[a + "q.b"], state[a + "k.b"], state[a + "v.b"]], dim=0))
                put(L.pb, state[a + "pb"])
                put(L.taps, state[b + "conv"])
                put(L.conv_b, state[b + "conv.b"])
                put(L.dt_bias, state[b + "dt_bias"])
                put(L.rate, -torch.exp(state[b + "A_log"].to(torch.float32)))
                put(L.skip, state[b + "D"])
                put(L.out_norm, state[b + "norm"])
                put(L.o, torch.cat([state[a + "o"], state[b + "o"]], dim=1))
                put(L.out_bias, state[a + "o.b"])
            elif s.kind == "mamba1":
                put(L.w_in, state[p + "in"])
                put(L.taps, state[p + "conv"])
                put(L.conv_b, state[p + "conv.b"])
                put(L.w_x, state[p + "x"])
                put(L.w_dt, state[p + "dt"])
                put(L.dt_bias, state[p + "dt.b"])
                put(L.rate, -torch.exp(state[p + "A_log"].to(torch.float32)))
                put(L.skip, state[p + "D"])
            elif s.kind == "sink_attention":
                put(L.w_in, torch.cat([state[p + "q"], state[p + "k"], state[p + "v"]], dim=0))
            elif s.kind == "attention":
                put(L.w_in, torch.cat([state[p + "q"], state[p + "k"], state[p + "v"], state[p + "g"]], dim=0))
                put(L.talk, state[p + "talk"])
                put(L.lam, state[p + "vmix"].reshape(1) if (p + "vmix") in state else torch.zeros(1))
            elif s.kind in ("delta", "channel_delta"):
                tail = [state[p + "a1"], state[p + "g1"]] if s.kind == "channel_delta" else [state[p + "a"], state[p + "g"]]
                put(L.w_in, torch.cat([state[p + "q"], state[p + "k"], state[p + "v"], state[p + "b"]] + tail, dim=0))
                put(L.taps, torch.cat([state[p + "q.conv"], state[p + "k.conv"], state[p + "v.conv"]], dim=0))
                put(L.rate, -torch.exp(state[p + "A_log"].to(torch.float32)))
                put(L.dt_bias, state[p + "dt_bias"])
                put(L.out_norm, state[p + "norm"])
                if s.kind == "channel_delta":
                    put(L.a2, state[p + "a2"])
                    put(L.g2, state[p + "g2"])
            elif s.kind == "latent_attention":
                parts = [state[p + "q"]] + ([] if s.kv_from is not None else [state[p + "dkv"]]) + ([state[p + "g"]] if s.out_gate else [])
                put(L.w_in, torch.cat(parts, dim=0))
                put(L.uk_t, state[p + "uk"].view(H, d, s.kv_rank).transpose(1, 2).contiguous())
                put(L.uv, state[p + "uv"].view(H, dv, s.kv_rank))
                if s.kv_from is None:
                    put(L.c_norm, state[p + "dkv.norm"])
            else:
                put(L.w_in, torch.cat([state[p + "q"], state[p + "k"], state[p + "v"], state[p + "g"]], dim=0))
                put(L.out_norm, state[p + "norm"])
            if s.kind != "parallel":
                put(L.o, state[p + "o"])
            if s.mlp is None and f"l{i}.norm2" in state and not self.pre_norm and not self.parallel and not self.conv_stream:  # no feed-forward, but a second norm
                L.norm2 = torch.empty_like(L.norm1)
                put(L.norm2, state[f"l{i}.norm2"])
            if isinstance(s.mlp, DenseFfSpec) and s.mlp.act == "silu_gate":
                q = f"l{i}.mlp."
                put(L.norm2, state[f"l{i}.norm2"])
                put(L.up, torch.cat([state[q + "gate"], state[q + "up"]], dim=0))
                put(L.down, state[q + "down"])
            elif isinstance(s.mlp, DenseFfSpec):
                q = f"l{i}.mlp."
                if L.norm2 is not None:
                    put(L.norm2, state[f"l{i}.norm2"])
                put(L.up, state[q + "up"])
                put(L.down, state[q + "down"])
                put(L.act, state[q + "act"])
            elif isinstance(s.mlp, MoeSpec) and s.mlp.gated:
                q = f"l{i}.mlp."
                put(L.norm2, state[f"l{i}.norm2"])
                put(L.router, state[q + "router"])
                if s.mlp.pick == "sigmoid_input":
                    L.bias = None
                    if s.mlp.shared_ff:
                        put(L.sh_up, torch.cat([state[q + "shared.gate"], state[q + "shared.up"]], dim=0))
                        put(L.sh_down, state[q + "shared.down"])
                else:
                    put(L.bias, state[q + "router.b"])
                put(L.up, torch.stack([torch.cat([state[f"{q}e{e}.gate"], state[f"{q}e{e}.up"]], dim=0) for e in range(s.mlp.experts)]))
                put(L.down, torch.stack([state[f"{q}e{e}.down"] for e in range(s.mlp.experts)]))
            elif s.mlp is not None:
                q = f"l{i}.mlp."
                put(L.norm2, state[f"l{i}.norm2"])
                put(L.router, state[q + "router"])
                if (q + "correction") in state:
                    put(L.bias, state[q + "correction"])
                else:
                    L.bias = None
                put(L.up, torch.stack([state[f"{q}e{e}.up"] for e in range(s.mlp.experts)]))
                put(L.down, torch.stack([state[f"{q}e{e}.down"] for e in range(s.mlp.experts)]))
        self._derive()

    def export_state(self) -> Dict[str, torch.Tensor]:
        """The inverse of load_state (checkpoint names, host tensors): what tests and tools hand to an independent implementation."""
        out = {"embed": self.embed, "final.norm": self.final_norm}
        if self.pre_norm:
            out["embed.norm"], out["head"] = self.embed_norm, self.head
        if self.parallel:
            out["head"] = self.head
            if self.pair_table is not None:
                out["bigram"] = self.pair_table
        if self.conv_stream:
            out["head"] = self.head
            if self.loop_step is not None:
                out["loop.step"] = self.loop_step
        for i, L in enumerate(self.layers):
            s, p = L.spec, f"l{i}.mix."
            H, d, dv = s.heads, s.dim, s.vdim
            out[f"l{i}.norm1"] = L.norm1
            if L.canon1 is not None:
                out[f"l{i}.canon1"] = L.canon1
            if L.canon2 is not None:
                out[f"l{i}.canon2"] = L.canon2
            if L.depth_w is not None:
                out[f"l{i}.dwa"] = L.depth_w
            if self.parallel:
                out[f"l{i}.ls1"] = L.ls1
                if s.mlp is not None:
                    out[f"l{i}.ls2"] = L.ls2
                if L.shift is not None:
                    out[f"l{i}.shift"] = L.shift
            if L.sink is not None:
                out[p + "sink"] = L.sink
            if s.kind == "parallel":
                a, b = p + "left.", p + "right."
                G, sp = s.left.kv_heads, s.right
                cuts = [H * d, G * d, G * dv]
                out[a + "q"], out[a + "k"], out[a + "v"], out[b + "in"] = torch.split(L.w_in, cuts + [L.w_in.shape[0] - sum(cuts)], dim=0)
                out[a + "q.b"], out[a + "k.b"], out[a + "v.b"] = torch.split(L.in_bias, cuts, dim=0)
                out[a + "pb"], out[b + "conv"], out[b + "conv.b"], out[b + "dt_bias"] = L.pb, L.taps, L.conv_b, L.dt_bias
                out[b + "A_log"], out[b + "D"], out[b + "norm"] = torch.log(-L.rate), L.skip, L.out_norm
                out[a + "o"], out[b + "o"] = L.o[:, : H * dv], L.o[:, H * dv:]
                out[a + "o.b"] = L.out_bias
            elif s.kind == "mamba1":
                out[p + "in"], out[p + "conv"], out[p + "conv.b"], out[p + "x"], out[p + "dt"] = L.w_in, L.taps, L.conv_b, L.w_x, L.w_dt
                out[p + "dt.b"], out[p + "A_log"], out[p + "D"] = L.dt_bias, torch.log(-L.rate), L.skip
            elif s.kind == "sink_attention":
                out[p + "q"], out[p + "k"], out[p + "v"] = torch.split(L.w_in, [H * d, s.kv_heads * d, s.kv_heads * dv], dim=0)
            elif s.kind == "attention":
                cuts = [H * d, s.kv_heads * d, s.kv_heads * dv, H]
                out[p + "q"], out[p + "k"], out[p + "v"], out[p + "g"] = torch.split(L.w_in, cuts, dim=0)
                out[p + "talk"], out[p + "vmix"] = L.talk, L.lam.reshape(())
            elif s.kind in ("delta", "channel_delta"):
                G, ch = s.kv_heads, s.kind == "channel_delta"
                cuts = [G * d, G * d, H * dv, H] + ([s.decay_rank, s.gate_rank] if ch else [H, H * dv])
                names = ["q", "k", "v", "b"] + (["a1", "g1"] if ch else ["a", "g"])
                for n, t in zip(names, torch.split(L.w_in, cuts, dim=0)):
                    out[p + n] = t
                out[p + "q.conv"], out[p + "k.conv"], out[p + "v.conv"] = torch.split(L.taps, cuts[:3], dim=0)
                out[p + "A_log"], out[p + "dt_bias"], out[p + "norm"] = torch.log(-L.rate), L.dt_bias, L.out_norm
                if ch:
                    out[p + "a2"], out[p + "g2"] = L.a2, L.g2
            elif s.kind == "latent_attention":
                nq = H * (d + s.rot_dim)
                out[p + "q"] = L.w_in[:nq]
                if s.kv_from is None:
                    out[p + "dkv"], out[p + "dkv.norm"] = L.w_in[nq: nq + s.kv_rank + s.rot_dim], L.c_norm
                if s.out_gate:
                    out[p + "g"] = L.w_in[L.w_in.shape[0] - H * dv:]
                out[p + "uk"] = L.uk_t.transpose(1, 2).reshape(H * d, s.kv_rank)
                out[p + "uv"] = L.uv.reshape(H * dv, s.kv_rank)
            else:
                a, b = H * d, H * dv
                out[p + "q"], out[p + "k"], out[p + "v"], out[p + "g"] = L.w_in[:a], L.w_in[a:2 * a], L.w_in[2 * a:2 * a + b], L.w_in[2 * a + b:]
                out[p + "norm"] = L.out_norm
            if s.kind != "parallel":
                out[p + "o"] = L.o
            if s.mlp is None and L.norm2 is not None:
                out[f"l{i}.norm2"] = L.norm2
            if isinstance(s.mlp, DenseFfSpec) and s.mlp.act == "silu_gate":
                q = f"l{i}.mlp."
                out[f"l{i}.norm2"], out[q + "gate"], out[q + "up"], out[q + "down"] = L.norm2, L.up[: s.mlp.ff], L.up[s.mlp.ff:], L.down
            elif isinstance(s.mlp, DenseFfSpec):
                q = f"l{i}.mlp."
                out[q + "up"], out[q + "down"], out[q + "act"] = L.up, L.down, L.act
                if L.norm2 is not None:
                    out[f"l{i}.norm2"] = L.norm2
            elif isinstance(s.mlp, MoeSpec) and s.mlp.gated:
                q = f"l{i}.mlp."
                out[f"l{i}.norm2"], out[q + "router"] = L.norm2, L.router
                if s.mlp.pick == "sigmoid_input":
                    if s.mlp.shared_ff:
                        out[q + "shared.gate"], out[q + "shared.up"] = L.sh_up[: s.mlp.shared_ff], L.sh_up[s.mlp.shared_ff:]
                        out[q + "shared.down"] = L.sh_down
                else:
                    out[q + "router.b"] = L.bias
                for e in range(s.mlp.experts):
                    out[f"{q}e{e}.gate"], out[f"{q}e{e}.up"], out[f"{q}e{e}.down"] = L.up[e, : s.mlp.ff], L.up[e, s.mlp.ff:], L.down[e]
            elif s.mlp is not None:
                q = f"l{i}.mlp."
                out[f"l{i}.norm2"], out[q + "router"] = L.norm2, L.router
                if L.bias is not None:
                    out[q + "correction"] = L.bias
                for e in range(s.mlp.experts):
                    out[f"{q}e{e}.up"], out[f"{q}e{e}.down"] = L.up[e], L.down[e]
        return {k: v.detach().to("cpu").contiguous() for k, v in out.items()}

    def tune_gemms(self, batch_sizes, mode: str = "heuristic", log=None, prefill_tokens=()) -> List[dict]:
        return []  # the library's heuristic pick; the grouped products have one kernel

    # ------------------------------------------------------------------ forward
    def _latent(self, i: int, L: _Layer, h: torch.Tensor, ctx: Any, batch: Any) -> torch.Tensor:
        s, md, kv = L.spec, batch.attn_metadata, ctx.kv_cache
        T, H, d, r, R, dv = h.shape[0], s.heads, s.dim, s.rot_dim, s.kv_rank, s.vdim
        proj = mixops.linear(h, L.w_in)
        q_abs = torch.empty((T, H, R + r), dtype=torch.float32, device=h.device)
        rows = kv.latent_rows(i)
        own = s.kv_from is None
        mixops.latent_prep(proj, q_abs, rows if own else None, batch.out_loc if own else None, batch.positions, L.cos_sin,
                           L.c_norm, self.cfg.rms_norm_eps, H, d, r, R, interleaved=s.interleaved)
        mixops.gemm_nt(q_abs, proj, L.uk_t, T, R, d, lda=proj.stride(0), ldb=d, ldc=H * (R + r), groups=H, a_gs=d + r,
                       b_gs=R * d, c_gs=R + r)
        o_lat = torch.empty((T, H, R), dtype=torch.float32, device=h.device)
        # few query rows per request (decode, short portions): cut the keys into ranges so that the launch fills the chip
        splits = mixops.latent_attn_splits(md.batch, T, H, md.max_seqlen_k) if md.max_seqlen_q <= 16 else 1
        mixops.latent_attn(o_lat, q_abs, rows, ctx.page_table, md.req_rows, md.seq_lens, md.cu_seqlens_q, md.batch, R, s.scale,
                           splits=splits, sink=L.sink)
        # with an output gate the heads' values stay fp32 until the gate has multiplied them: one rounding on the way into W_o
        o = torch.empty((T, H * dv), dtype=torch.float32 if s.out_gate else self.dtype, device=h.device)
        mixops.gemm_nt(o, o_lat, L.uv, T, dv, R, lda=H * R, ldb=R, ldc=H * dv, groups=H, a_gs=R, b_gs=dv * R, c_gs=dv)
        if s.out_gate:
            g_off = L.w_in.shape[0] - H * dv
            o = mixops.sigmoid_gate(o, proj[:, g_off:])
        return mixops.linear(o, L.o)

    def _mamba(self, i: int, L: _Layer, h: torch.Tensor, ctx: Any, batch: Any) -> torch.Tensor:
        """Selective scan: in-projection, causal convolution + SiLU with the request's conv state, the two-step step-size projection,
        the recurrence on the request's fp32 state (gated by silu(z) in the same launch), output projection."""
        s, md, kv = L.spec, batch.attn_metadata, ctx.kv_cache
        inner, N, dr = s.vdim, s.dim, s.dt_rank
        proj = mixops.linear(h, L.w_in)
        x = mixops.short_conv(proj, inner, L.taps, kv.conv_state(i), md.cu_seqlens_q, md.seq_lens, md.req_rows, md.batch, unit_heads=0,
                              scaled_heads=0, d=1, bias=L.conv_b, model_dtype=True)
        dbc = mixops.linear(x, L.w_x)
        dt_in = mixops.linear(dbc[:, :dr], L.w_dt)
        y = mixops.selective_scan(x, proj[:, inner:], dt_in, dbc[:, dr:], L.rate, L.dt_bias, L.skip, kv.state(i), md.cu_seqlens_q, md.seq_lens,
                                  md.req_rows, md.batch, chunks=getattr(md, "scan_chunks", None))
        return mixops.linear(y, L.o)

    def _sink_attention(self, i: int, L: _Layer, h: torch.Tensor, ctx: Any, batch: Any) -> torch.Tensor:
        """Grouped attention over a window with a sink: projections, rotation of q and k and unit-RMS values into the cache rows, scores /
        softmax / weighted values in one launch, output projection."""
        s, md, kv = L.spec, batch.attn_metadata, ctx.kv_cache
        T, H, G, d, dv = h.shape[0], s.heads, s.kv_heads, s.dim, s.vdim
        proj = mixops.linear(h, L.w_in)
        kc, vc = kv.kv_rows(i)
        q = mixops.qk_prep(proj, None, kc, vc, batch.out_loc, batch.positions, L.cos_sin, self.cfg.rms_norm_eps, H, G, d, dv,
                           interleaved=False, unit=False, unit_v=s.v_norm)
        o = torch.empty((T, H * dv), dtype=self.dtype, device=h.device)
        splits = mixops.sink_attn_splits(md.batch, T, H, G, s.window, md.max_seqlen_k) if md.max_seqlen_q <= 16 else 1
        mixops.sink_attn(o, q, kc, vc, ctx.page_table, md.req_rows, md.seq_lens, md.cu_seqlens_q, md.batch, H, G, d, dv, s.scale, s.window,
                         L.sink if s.sink else None, splits=splits)
        return mixops.linear(o, L.o)

    def _gated_ff(self, h: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
        return mixops.linear(mixops.silu_mul(mixops.linear(h, up)), down)

    def _input_weighted_experts(self, L: _Layer, h: torch.Tensor) -> torch.Tensor:
        """-> [T, top, W]: every chosen expert's output on score * h (the score is inside the expert's input, so the caller adds the
        rows as they are)."""
        m, (T, W) = L.spec.mlp, h.shape
        # few tokens (decode, short portions): logits, choice and the scaled rows leave one launch; many tokens: every token re-reading
        # the router matrix costs more than the launches it saves, so the logits come from the product kernel
        if T <= self.ROUTE_FUSE_MAX_TOKENS:
            ids, _, hs = mixops.route_scale(h, L.router, m.top)
        else:
            ids, wts = mixops.route_sigmoid(h, L.router, m.top)
            hs = mixops.scale_rows(h, wts)
        seg, perm = mixops.moe_sort(ids, m.experts)
        n = T * m.top
        gu = torch.empty((n, 2 * m.ff), dtype=self.dtype, device=h.device)
        mixops.gemm_nt(gu, hs, L.up, n, 2 * m.ff, W, lda=W, ldb=W, ldc=2 * m.ff, groups=m.experts, b_gs=2 * m.ff * W, seg=seg, a_rows=perm, a_div=1)
        act = mixops.silu_mul(gu)
        y = torch.empty((T, m.top, W), dtype=self.dtype, device=h.device)
        mixops.gemm_nt(y, act, L.down, n, W, m.ff, lda=m.ff, ldb=m.ff, ldc=W, groups=m.experts, b_gs=W * m.ff, seg=seg, c_rows=perm)
        return y

    def _forward_conv(self, ctx: Any, batch: Any, layer_outputs: Optional[list]) -> torch.Tensor:
        """The pre-norm stream with grouped norms, input convolutions and a looped run of layers -> the final-normed rows [tokens, W].
        One `norm_conv` launch closes a sublayer (residual sum with the multiplier, the loop's step vector) and opens the next (norm,
        input convolution); the convolutions' new state rows are staged and committed after the last layer."""
        cfg, eps, md, kv = self.cfg, self.cfg.rms_norm_eps, batch.attn_metadata, ctx.kv_cache
        T, W, dev, bs = batch.input_ids.shape[0], cfg.hidden_size, self.device, batch.attn_metadata.batch
        runs, n, mult, groups = cfg.runs, cfg.conv_taps, cfg.residual_mult, cfg.norm_groups
        req = dict(cu_q=md.cu_seqlens_q, seq_lens=md.seq_lens, req_rows=md.req_rows, batch=bs)
        staging = torch.empty((len(runs), 2, bs, n - 1, W), dtype=torch.float32, device=dev) if n > 1 else None
        x = mixops.embed_scaled(self.embed, batch.input_ids, 1.0)

        def open_sublayer(x_in, parts, add, weight, taps, run, sub):
            """-> (x after the sum, the sublayer's input rows in the model dtype)."""
            h = torch.empty((T, W), dtype=self.dtype, device=dev)
            x_out = torch.empty((T, W), dtype=torch.float32, device=dev) if parts or add is not None else None
            conv = dict(taps=taps, state=kv.conv_in_state(run, sub), staging=staging[run, sub], **req) if taps is not None and n > 1 else dict(taps=taps)
            mixops.norm_conv(x_in, weight, eps, groups, h, parts=parts, mult=mult, add=add, x_out=x_out, **conv)
            return (x_in if x_out is None else x_out), h

        pending: tuple = ()
        for run, (i, pass_no) in enumerate(runs):
            L = self.layers[i]
            add = self.loop_step[pass_no] if pass_no is not None else None
            x, h = open_sublayer(x, pending, add, L.norm1, L.canon1, run, 0)
            if layer_outputs is not None and run > 0:
                layer_outputs.append(x - add if add is not None else x.clone())
            kind = L.spec.kind
            if kind == "latent_attention":
                y = self._latent(run, L, h, ctx, batch)
            elif kind == "mamba1":
                y = self._mamba(run, L, h, ctx, batch)
            elif kind == "sink_attention":
                y = self._sink_attention(run, L, h, ctx, batch)
            else:
                raise NotImplementedError(f"mixer {kind!r} in a looped pre-norm stack")
            m = L.spec.mlp
            if m is None:
                pending = (y,)
                continue
            x, h = open_sublayer(x, (y,), None, L.norm2, L.canon2, run, 1)
            if isinstance(m, DenseFfSpec):
                pending = (self._gated_ff(h, L.up, L.down),)
            else:
                pending = (self._input_weighted_experts(L, h),) + ((self._gated_ff(h, L.sh_up, L.sh_down),) if m.shared_ff else ())
        x, hf = open_sublayer(x, pending, None, self.final_norm, None, 0, 0)
        if layer_outputs is not None and runs:
            layer_outputs.append(x.clone())
        if staging is not None:
            mixops.commit_rows(kv.conv_in_states.view(2 * len(runs), -1, (n - 1) * W), staging.view(2 * len(runs), bs, (n - 1) * W), md.req_rows, bs,
                               md.cu_seqlens_q)
        return hf

    def _lightning(self, i: int, L: _Layer, h: torch.Tensor, ctx: Any, batch: Any) -> torch.Tensor:
        s, md = L.spec, batch.attn_metadata
        T, H, d, dv = h.shape[0], s.heads, s.dim, s.vdim
        proj = mixops.linear(h, L.w_in)
        o = torch.empty((T, H * dv), dtype=torch.float32, device=h.device)
        mixops.lightning(o, proj, ctx.kv_cache.state(i), L.decay, md.cu_seqlens_q, md.seq_lens, md.req_rows, md.batch,
                         chunks=getattr(md, "chunks", None))
        gated = mixops.gated_norm(o, proj[:, 2 * H * d + H * dv:], L.out_norm, self.cfg.rms_norm_eps)
        return mixops.linear(gated, L.o)

    def _experts(self, L: _Layer, h: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        """-> per-choice outputs [T, top, W] of the experts `ids` chose; the weighted sum over choices is the caller's norm's."""
        m, (T, W) = L.spec.mlp, h.shape
        seg, perm = mixops.moe_sort(ids, m.experts)
        n = T * m.top
        act = torch.empty((n, m.ff), dtype=self.dtype, device=h.device)
        mixops.gemm_nt(act, h, L.up, n, m.ff, W, lda=W, ldb=W, ldc=m.ff, groups=m.experts, b_gs=m.ff * W, seg=seg, a_rows=perm,
                       a_div=m.top, act=mixops.ACT_RELU2)
        y = torch.empty((T, m.top, W), dtype=self.dtype, device=h.device)
        mixops.gemm_nt(y, act, L.down, n, W, m.ff, lda=m.ff, ldb=m.ff, ldc=W, groups=m.experts, b_gs=W * m.ff, seg=seg, c_rows=perm)
        return y

    def _attention(self, i: int, L: _Layer, h: torch.Tensor, ctx: Any, batch: Any, shared: Dict[str, Any]) -> torch.Tensor:
        """Windowed attention with mixed heads: projections, cache rows (values blended with the first value-mixing layer's),
        scores / softmax / gate in one launch, output projection."""
        s, md, kv = L.spec, batch.attn_metadata, ctx.kv_cache
        T, H, G, d, dv = h.shape[0], s.heads, s.kv_heads, s.dim, s.vdim
        proj = mixops.linear(h, L.w_in)
        k_off, v_off, g_off = H * d, H * d + G * d, H * d + G * d + G * dv
        first = shared.get("v_first") if s.v_mix else None
        kc, vc = kv.kv_rows(i)
        mixops.kv_store(kc, vc, batch.out_loc, proj, k_off, v_off, v_first=first, lam=L.lam if first is not None else None)
        if s.v_mix and first is None:
            shared["v_first"] = proj[:, v_off: v_off + G * dv]
        o = torch.empty((T, H * dv), dtype=self.dtype, device=h.device)
        mixops.window_attn(o, proj, g_off, kc, vc, ctx.page_table, md.req_rows, md.seq_lens, md.cu_seqlens_q, md.batch, H, G, d, dv,
                           s.window, s.scale, L.talk, splits=mixops.window_attn_splits(md.batch, T, s.window, md.max_seqlen_k))
        return mixops.linear(o, L.o)

    def _delta(self, i: int, L: _Layer, h: torch.Tensor, ctx: Any, batch: Any) -> torch.Tensor:
        """Gated delta rule: projections, short convolution (+ unit vectors) with the request's conv state, the recurrence on
        the request's fp32 state, per-head gated norm, output projection."""
        s, md, kv = L.spec, batch.attn_metadata, ctx.kv_cache
        T, H, G, d, dv = h.shape[0], s.heads, s.kv_heads, s.dim, s.vdim
        C = 2 * G * d + H * dv
        proj = mixops.linear(h, L.w_in)
        qkv = mixops.short_conv(proj, C, L.taps, kv.conv_state(i), md.cu_seqlens_q, md.seq_lens, md.req_rows, md.batch,
                                unit_heads=2 * G, scaled_heads=G, d=d)
        b_raw = proj[:, C: C + H]
        if s.kind == "channel_delta":
            a_raw = mixops.linear(proj[:, C + H: C + H + s.decay_rank], L.a2)
            gate = mixops.linear(proj[:, C + H + s.decay_rank: C + H + s.decay_rank + s.gate_rank], L.g2)
            act = mixops.GATE_SIGMOID
        else:
            a_raw, gate, act = proj[:, C + H: C + 2 * H], proj[:, C + 2 * H: C + 2 * H + H * dv], mixops.GATE_SILU
        o = torch.empty((T, H * dv), dtype=torch.float32, device=h.device)
        mixops.delta_rule(o, qkv, kv.state(i), b_raw, a_raw, s.kind == "channel_delta", L.rate, L.dt_bias, md.cu_seqlens_q, md.seq_lens,
                          md.req_rows, md.batch, G, chunks=getattr(md, "delta_chunks", None))
        return mixops.linear(mixops.head_gated_norm(o, gate, L.out_norm, self.cfg.rms_norm_eps, H, dv, act), L.o)

    def _gated_experts(self, L: _Layer, h: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        """-> per-choice outputs [T, top, W] of experts W_down (silu(W_gate h) * (W_up h)); the weighted sum is the caller's."""
        m, (T, W) = L.spec.mlp, h.shape
        seg, perm = mixops.moe_sort(ids, m.experts)
        n = T * m.top
        gu = torch.empty((n, 2 * m.ff), dtype=self.dtype, device=h.device)
        mixops.gemm_nt(gu, h, L.up, n, 2 * m.ff, W, lda=W, ldb=W, ldc=2 * m.ff, groups=m.experts, b_gs=2 * m.ff * W, seg=seg,
                       a_rows=perm, a_div=m.top)
        act = mixops.silu_mul(gu)
        y = torch.empty((T, m.top, W), dtype=self.dtype, device=h.device)
        mixops.gemm_nt(y, act, L.down, n, W, m.ff, lda=m.ff, ldb=m.ff, ldc=W, groups=m.experts, b_gs=W * m.ff, seg=seg, c_rows=perm)
        return y

    def _pair(self, i: int, L: _Layer, g: torch.Tensor, ctx: Any, batch: Any) -> torch.Tensor:
        """Sigmoid attention and a state-space layer on the same input: one input projection, the two mixers' kernels writing
        their (scaled) outputs side by side into one row, one output projection."""
        s, md, kv, eps = L.spec, batch.attn_metadata, ctx.kv_cache, self.cfg.rms_norm_eps
        a, b = s.left, s.right
        T, H, G, d, dv = g.shape[0], a.heads, a.kv_heads, a.dim, a.vdim
        Hs, Gs, N, P = b.heads, b.kv_heads, b.dim, b.vdim
        n_left, inner, C = (H + G) * d + G * dv, Hs * P, Hs * P + 2 * Gs * N
        proj = mixops.linear(g, L.w_in)
        cat = torch.empty((T, H * dv + inner), dtype=self.dtype, device=g.device)
        # left: q / k prepared (bias, rotation, unit RMS), k and v into the cache rows, weights without normalisation over keys
        kc, vc = kv.kv_rows(i)
        q = mixops.qk_prep(proj, L.in_bias, kc, vc, batch.out_loc, batch.positions, L.cos_sin, eps, H, G, d, dv,
                           interleaved=a.interleaved, unit=True)
        mixops.sigmoid_attn(cat[:, : H * dv], q, kc, vc, ctx.page_table, md.req_rows, md.seq_lens, md.cu_seqlens_q, md.batch, H, G, d, dv,
                            a.scale, a.softcap, L.pb, out_scale=s.left_scale,
                            splits=mixops.sigmoid_attn_splits(md.batch, T, H, G, md.max_seqlen_k) if md.max_seqlen_q <= 16 else 1)
        # right: proj[:, n_left:] = z | x B C | dt
        z, xbc_raw, dt_raw = proj[:, n_left: n_left + inner], proj[:, n_left + inner: n_left + inner + C], proj[:, n_left + inner + C:]
        xbc = mixops.short_conv(xbc_raw, C, L.taps, kv.conv_state(i), md.cu_seqlens_q, md.seq_lens, md.req_rows, md.batch,
                                unit_heads=0, scaled_heads=0, d=1, bias=L.conv_b)
        y = torch.empty((T, inner), dtype=torch.float32, device=g.device)
        mixops.ssd(y, xbc, dt_raw, kv.state(i), L.rate, L.dt_bias, L.skip, md.cu_seqlens_q, md.seq_lens, md.req_rows, md.batch, Gs,
                   chunks=getattr(md, "ssd_chunks", None))
        mixops.gate_group_norm(cat[:, H * dv:], y, z, L.out_norm, eps, b.norm_groups, out_scale=s.right_scale)
        return mixops.linear(cat, L.o)

    def _forward_parallel(self, ctx: Any, batch: Any, layer_outputs: Optional[list]) -> torch.Tensor:
        """One norm per layer, token-shifted mixer and feed-forward side by side -> the final-normed rows [tokens, W]."""
        cfg, eps, md, kv = self.cfg, self.cfg.rms_norm_eps, batch.attn_metadata, ctx.kv_cache
        T, W, n, dev, bs = batch.input_ids.shape[0], cfg.hidden_size, len(self.layers), self.device, batch.attn_metadata.batch
        req = dict(positions=batch.positions, cu_q=md.cu_seqlens_q, req_rows=md.req_rows, batch=bs)
        pe = cfg.pair_embed
        x = mixops.embed_scaled(self.embed, batch.input_ids, cfg.embed_scale, pair=self.pair_table, buckets=pe[0] if pe else 0,
                                mul_prev=pe[1] if pe else 0, mul_cur=pe[2] if pe else 0, prev_tok=kv.prev_token if pe else None, **req)
        staging = torch.empty((n, bs, W), dtype=torch.float32, device=dev) if cfg.token_shift else None
        hf = torch.empty((T, W), dtype=self.dtype, device=dev)

        def open_layer(i: int, x_in: torch.Tensor, parts=(), bias=None, x_out=None):
            """Closes the layer before (its parts summed onto x_in -> x_out) and opens layer i: -> (h, g)."""
            if i == n:
                mixops.shift_norm(x_in, self.final_norm, eps, dtype=self.dtype, w_offset=1.0, parts=parts, bias=bias, x_out=x_out, h_out=hf)
                return hf, hf
            L = self.layers[i]
            h = torch.empty((T, W), dtype=self.dtype, device=dev) if L.spec.mlp is not None or L.shift is None else None
            if L.shift is None:
                mixops.shift_norm(x_in, L.norm1, eps, dtype=self.dtype, w_offset=1.0, parts=parts, bias=bias, x_out=x_out, h_out=h)
                return h, h
            g = torch.empty((T, W), dtype=self.dtype, device=dev)
            mixops.shift_norm(x_in, L.norm1, eps, dtype=self.dtype, w_offset=1.0, parts=parts, bias=bias, x_out=x_out, h_out=h, g_out=g,
                              shift=L.shift, state=kv.shift_state(i), staging=staging[i], **req)
            return h, g

        h, g = open_layer(0, x)
        for i, L in enumerate(self.layers):
            y = self._pair(i, L, g, ctx, batch) if L.spec.kind == "parallel" else self._latent(i, L, g, ctx, batch)
            parts = [(y, L.ls1)]
            if L.spec.mlp is not None:
                parts.append((mixops.linear(mixops.xielu(mixops.linear(h, L.up), L.act), L.down), L.ls2))
            x_next = torch.empty((T, W), dtype=torch.float32, device=dev)
            h, g = open_layer(i + 1, x, parts, L.sum_bias, x_next)
            x = x_next
            if layer_outputs is not None:
                layer_outputs.append(x.clone())
        if cfg.token_shift or pe:
            mixops.commit_rows(kv.shift_states if cfg.token_shift else None, staging, md.req_rows, bs, md.cu_seqlens_q,
                               prev_tok=kv.prev_token if pe else None, ids=batch.input_ids if pe else None)
        return hf

    def _forward_pre_norm(self, ctx: Any, batch: Any, layer_outputs: Optional[list]) -> torch.Tensor:
        """The pre-norm, depth-averaged stream -> the final-normed rows [tokens, W] in the model dtype."""
        cfg, eps = self.cfg, self.cfg.rms_norm_eps
        T, W, n = batch.input_ids.shape[0], cfg.hidden_size, len(self.layers)
        dev = self.device
        hist = torch.empty((n + 1, T, W), dtype=torch.float32, device=dev)  # X_0 .. X_n: what every layer's average reads
        mixops.embed_norm(self.embed, batch.input_ids, self.embed_norm, eps, hist[0])
        x = hist[0]
        h = torch.empty((T, W), dtype=self.dtype, device=dev)
        mid = torch.empty((T, W), dtype=torch.float32, device=dev)
        mixops.prenorm(x, weight=self.layers[0].norm1 if n else self.final_norm, h_out=h, eps=eps)
        shared: Dict[str, Any] = {}
        for i, L in enumerate(self.layers):
            kind, m = L.spec.kind, L.spec.mlp
            if kind == "attention":
                y = self._attention(i, L, h, ctx, batch, shared)
            elif kind in ("delta", "channel_delta"):
                y = self._delta(i, L, h, ctx, batch)
            else:
                raise NotImplementedError(f"mixer {kind!r} in a pre-norm stack")
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            x_next = torch.empty((T, W), dtype=torch.float32, device=dev)
            if m is None:
                mixops.prenorm(x, y=y, sum_out=hist[i + 1], history=hist, depth_w=L.depth_w, x_out=x_next, weight=nxt, h_out=h, eps=eps)
            else:
                if isinstance(m, DenseFfSpec):
                    mixops.prenorm(x, y=y, sum_out=mid, weight=L.norm2, h_out=h, eps=eps)
                    f, gate = mixops.linear(mixops.poly_act(mixops.linear(h, L.up), L.act, eps), L.down), None
                else:
                    fuse = T <= self.ROUTE_FUSE_MAX_TOKENS
                    picks = mixops.prenorm(x, y=y, sum_out=mid, weight=L.norm2, h_out=h, eps=eps,
                                           route=(L.router, L.bias, m.top) if fuse else None)
                    if not fuse:
                        picks = mixops.route_top(h, L.router, L.bias, m.top)
                    f, gate = self._gated_experts(L, h, picks[0]), picks[1]
                mixops.prenorm(mid, y=f, gate=gate, sum_out=hist[i + 1], history=hist, depth_w=L.depth_w, x_out=x_next, weight=nxt,
                               h_out=h, eps=eps)
            x = x_next
            if layer_outputs is not None:
                layer_outputs.append(x.clone())
        return h

    def forward(self, ctx: Any, batch: Any, logits_out: Optional[torch.Tensor] = None, layer_outputs: Optional[list] = None) -> torch.Tensor:
        """-> logits [rows, vocab] in the model dtype: at `batch.logit_rows` (token indices) when set, else at every request's
        last token (prefill) or at every token (decode)."""
        cfg = self.cfg
        eps, alpha = cfg.rms_norm_eps, cfg.postln_alpha
        if self.pre_norm or self.parallel or self.conv_stream:
            hf = self._forward_pre_norm(ctx, batch, layer_outputs) if self.pre_norm else \
                self._forward_parallel(ctx, batch, layer_outputs) if self.parallel else self._forward_conv(ctx, batch, layer_outputs)
            rows = getattr(batch, "logit_rows", None)
            if rows is None and batch.is_prefill:
                rows = batch.attn_metadata.get_last_indices(batch.size)
            if rows is not None:
                hf = hf.index_select(0, rows.to(torch.int64))
            if logits_out is not None and logits_out.shape == (hf.shape[0], cfg.vocab_size) and logits_out.dtype == self.dtype:
                logits = mixops.linear(hf, self.head, out=logits_out)
            else:
                logits = mixops.linear(hf, self.head)
            return mixops.softcap(logits, cfg.logit_softcap) if cfg.logit_softcap > 0.0 else logits
        x, h = mixops.embed(self.embed, batch.input_ids)
        for i, L in enumerate(self.layers):
            y = self._latent(i, L, h, ctx, batch) if L.spec.kind == "latent_attention" else self._lightning(i, L, h, ctx, batch)
            m = L.spec.mlp
            # Few tokens (decode, short portions): the norm that closes the mixer's sum also routes its output -- router logits,
            # choice and weights leave the same launch.  Many tokens: every token re-reading the router weights costs more than
            # the launches it saves, so the logits come from the product kernel (weights reused across a 128-token tile).
            fuse = m is not None and h.shape[0] <= self.ROUTE_FUSE_MAX_TOKENS
            picks = mixops.postnorm(x, L.norm1, eps, y=y, alpha=alpha, x_out=x, h_out=h,
                                    route=(L.router, L.bias, m.top, m.groups, m.keep) if fuse else None)
            if m is not None and not fuse:
                picks = mixops.route(h, L.router, L.bias, m.top, m.groups, m.keep)
            if m is not None:
                y = self._experts(L, h, picks[0])
                mixops.postnorm(x, L.norm2, eps, y=y, gate=picks[1], alpha=alpha, x_out=x, h_out=h)
            elif L.norm2 is not None:
                mixops.postnorm(x, L.norm2, eps, alpha=alpha, x_out=x, h_out=h)
            if layer_outputs is not None:
                layer_outputs.append(x.clone())
        rows = getattr(batch, "logit_rows", None)
        if rows is None and batch.is_prefill:
            rows = batch.attn_metadata.get_last_indices(batch.size)
        if rows is not None:
            x = x.index_select(0, rows.to(torch.int64))
        hf = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        mixops.postnorm(x, self.final_norm, eps, h_out=hf)
        if logits_out is not None and logits_out.shape == (hf.shape[0], cfg.vocab_size) and logits_out.dtype == self.dtype:
            return mixops.linear(hf, self.embed, out=logits_out)
        return mixops.linear(hf, self.embed)

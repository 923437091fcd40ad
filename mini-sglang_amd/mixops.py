"""torch-facing wrappers of the sequence-mixing kernels (include/msgl_mix.h, csrc/seqmix.hip, csrc/mix_delta.hip).

Same rules as ops.py: device tensors only, no CPU fallback, pointers + sizes + the current stream go straight to
the C ABI.  `linear` is the projection seam of the hybrid models: the library GEMM (bf16, or fp32 in the library's
true 32-bit mode) and, for shapes the library has no solution for, the grouped kernel of this file.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib, ops
from ._lib import check_mix, mix_lib

ACT_NONE, ACT_RELU2 = 0, 1


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return _lib.BF16
    if t.dtype == torch.float32:
        return _lib.F32
    raise TypeError(f"expected a bf16 or fp32 tensor, got {t.dtype}")


def _dev(*ts: Optional[torch.Tensor]) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("mini_sglang_amd mixops run on the HIP device only (got a CPU tensor)")


def _i32(t: torch.Tensor) -> torch.Tensor:
    assert t.dtype == torch.int32 and t.is_contiguous(), (t.dtype, t.stride())
    return t


def _p(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


def embed(table: torch.Tensor, ids: torch.Tensor):
    """-> (fp32 rows, the same rows in the table's dtype)."""
    _dev(table, ids)
    assert table.dim() == 2 and table.is_contiguous()
    T, W = ids.shape[0], table.shape[1]
    x32 = torch.empty((T, W), dtype=torch.float32, device=table.device)
    h = torch.empty((T, W), dtype=table.dtype, device=table.device)
    check_mix(mix_lib().msgl_mix_embed(x32.data_ptr(), h.data_ptr(), table.data_ptr(), _i32(ids).data_ptr(), T, W,
                                       _code(table), _stream()), "embed")
    return x32, h


def postnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, *, y: Optional[torch.Tensor] = None,
             gate: Optional[torch.Tensor] = None, alpha: float = 1.0, x_out: Optional[torch.Tensor] = None,
             h_out: Optional[torch.Tensor] = None, route=None):
    """s = alpha x + sum_p gate[:, p] y[:, p];  out = rms_unit(s) * (1 + weight) -> x_out (fp32) and / or h_out (weight's dtype).
    y: [rows, W] or [rows, parts, W].  route = (router [E, W], bias [E] | None, top, groups, keep): the normed rows are routed in
    the same launch -> returns (expert ids int32 [rows, top], weights fp32 [rows, top]), else None."""
    _dev(x, weight, y, gate, x_out, h_out)
    rows, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous() and weight.shape == (W,) and weight.is_contiguous()
    parts = 0
    if y is not None:
        assert y.is_contiguous() and y.dtype == weight.dtype and y.shape[0] == rows and y.shape[-1] == W
        parts = 1 if y.dim() == 2 else y.shape[1]
    if gate is not None:
        assert gate.dtype == torch.float32 and gate.is_contiguous() and gate.numel() == rows * parts
    for o, dt in ((x_out, torch.float32), (h_out, weight.dtype)):
        assert o is None or (o.shape == (rows, W) and o.is_contiguous() and o.dtype == dt)
    router = bias = ids = wts = None
    E = top = groups = keep = 0
    if route is not None:
        router, bias, top, groups, keep = route
        _dev(router, bias)
        E = router.shape[0]
        assert router.shape == (E, W) and router.is_contiguous() and router.dtype == weight.dtype
        assert bias is None or (bias.dtype == weight.dtype and bias.shape == (E,) and bias.is_contiguous())
        ids = torch.empty((rows, top), dtype=torch.int32, device=x.device)
        wts = torch.empty((rows, top), dtype=torch.float32, device=x.device)
    if rows:
        check_mix(mix_lib().msgl_mix_postnorm(x.data_ptr(), _p(x_out), _p(h_out), _p(y), parts, _p(gate), weight.data_ptr(),
                                              float(alpha), float(eps), rows, W, _code(weight), _p(router), _p(bias), E, top, groups,
                                              keep, _p(ids), _p(wts), _stream()), "postnorm")
    return None if route is None else (ids, wts)


def latent_prep(proj: torch.Tensor, q_abs: torch.Tensor, cache: Optional[torch.Tensor], out_loc: Optional[torch.Tensor],
                positions: torch.Tensor, cos_sin: torch.Tensor, c_norm_w: Optional[torch.Tensor], eps: float, H: int, d: int,
                r: int, R: int, interleaved: bool = False) -> None:
    """Rotates the query parts into q_abs[:, :, R:]; with `cache`, norms + rotates + stores this layer's own latent rows.
    interleaved: entries (2i, 2i + 1) of a rotated part form pair i instead of (i, i + half)."""
    _dev(proj, q_abs, cache, out_loc, positions, cos_sin, c_norm_w)
    T = proj.shape[0]
    has_kv = cache is not None
    assert proj.dim() == 2 and proj.stride(1) == 1
    assert q_abs.dtype == torch.float32 and q_abs.is_contiguous() and q_abs.shape == (T, H, R + r)
    assert cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.dim() == 2
    if has_kv:
        assert cache.is_contiguous() and cache.shape[1] == R + r and cache.dtype == proj.dtype
        assert c_norm_w.dtype == proj.dtype and c_norm_w.shape == (R,) and out_loc.shape[0] == T
    check_mix(mix_lib().msgl_mix_latent_prep(
        proj.data_ptr(), proj.stride(0), q_abs.data_ptr(), _p(cache), _p(None if out_loc is None else _i32(out_loc)),
        _i32(positions).data_ptr(), cos_sin.data_ptr(), _p(c_norm_w), float(eps), T, H, d, r, cos_sin.shape[1], R, int(has_kv),
        int(interleaved), _code(proj), _stream()), "latent_prep")


def latent_attn_splits(batch: int, total_q: int, H: int, max_keys: int) -> int:
    """Key ranges per request for a step with few query rows: enough workgroups to fill the chip, at least 256 keys each (measured: 64-key ranges double the launch's time -- every
    range pays the query fragments, a partial row and its share of the merge).
    A function of static sizes only (batch, rows, the LONGEST possible key count), so a captured graph keeps its grid."""
    hb = min(H, 64)
    blocks = (-(-total_q // (64 // hb)) + batch) * -(-H // hb)
    return max(1, min(1024 // max(blocks, 1), max_keys // 256, 64))


def latent_attn(out: torch.Tensor, q_abs: torch.Tensor, cache: torch.Tensor, table: torch.Tensor, req_rows: torch.Tensor,
                seq_lens: torch.Tensor, cu_q: torch.Tensor, batch: int, dv: int, scale: float, splits: int = 1,
                sink: Optional[torch.Tensor] = None) -> None:
    """sink (fp32 [H]): one more term exp(sink[h]) in every softmax denominator of head h, with no key and no value."""
    _dev(out, q_abs, cache, table, req_rows, seq_lens, cu_q, sink)
    assert sink is None or (sink.dtype == torch.float32 and sink.is_contiguous() and sink.shape == (q_abs.shape[1],))
    T, H, dk = q_abs.shape
    assert q_abs.dtype == torch.float32 and q_abs.is_contiguous() and out.dtype == torch.float32 and out.is_contiguous()
    assert out.shape == (T, H, dv) and cache.is_contiguous() and cache.shape[1] == dk
    assert table.dtype == torch.int32 and table.stride(1) == 1
    assert req_rows.numel() >= batch and seq_lens.numel() >= batch and cu_q.numel() >= batch + 1
    ws = None
    if splits > 1:
        ws = torch.empty(mix_lib().msgl_mix_latent_attn_workspace_floats(T, H, dv, splits), dtype=torch.float32, device=out.device)
    check_mix(mix_lib().msgl_mix_latent_attn(
        out.data_ptr(), q_abs.data_ptr(), cache.data_ptr(), table.data_ptr(), table.stride(0), _i32(req_rows).data_ptr(),
        _i32(seq_lens).data_ptr(), _i32(cu_q).data_ptr(), batch, T, H, dk, dv, float(scale), _p(sink), _code(cache), splits, _p(ws),
        _stream()), "latent_attn")


def lightning(out: torch.Tensor, qkv: torch.Tensor, state: torch.Tensor, decay: torch.Tensor, cu_q: torch.Tensor,
              seq_lens: torch.Tensor, slots: torch.Tensor, batch: int, chunks=None) -> None:
    """state: fp32 [slots, H, d, dv]; qkv rows = [q H*d | k H*d | v H*dv | anything].  chunks = (items int32 [n, 3], item_first
    int32 [batch + 1], n) cuts long portions into pieces that run in parallel (see include/msgl_mix.h)."""
    _dev(out, qkv, state, decay, cu_q, seq_lens, slots)
    _, H, d, dv = state.shape
    assert state.dtype == torch.float32 and state.is_contiguous() and decay.dtype == torch.float32 and decay.shape == (H,)
    assert out.dtype == torch.float32 and out.is_contiguous() and out.shape == (qkv.shape[0], H * dv) and qkv.stride(1) == 1
    items = first = scratch = None
    n_items = 0
    if chunks is not None:
        items, first, n_items = chunks
        _dev(items, first)
        assert items.numel() == 3 * n_items and first.numel() == batch + 1
        scratch = torch.empty((n_items, H, d, dv), dtype=torch.float32, device=out.device)
    check_mix(mix_lib().msgl_mix_lightning(
        out.data_ptr(), qkv.data_ptr(), qkv.stride(0), state.data_ptr(), decay.data_ptr(), _i32(cu_q).data_ptr(),
        _i32(seq_lens).data_ptr(), _i32(slots).data_ptr(), batch, H, d, dv, _code(qkv), n_items,
        _p(None if items is None else _i32(items)), _p(None if first is None else _i32(first)), _p(scratch), _stream()), "lightning")


def gated_norm(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    _dev(o, gate, weight)
    rows, N = o.shape
    assert o.dtype == torch.float32 and o.is_contiguous() and gate.shape == (rows, N) and gate.stride(1) == 1
    assert weight.dtype == gate.dtype and weight.shape == (N,) and weight.is_contiguous()
    out = torch.empty((rows, N), dtype=gate.dtype, device=o.device)
    check_mix(mix_lib().msgl_mix_gated_norm(out.data_ptr(), o.data_ptr(), gate.data_ptr(), gate.stride(0), weight.data_ptr(),
                                            float(eps), rows, N, _code(gate), _stream()), "gated_norm")
    return out


def route(h: torch.Tensor, router: torch.Tensor, bias: Optional[torch.Tensor], top: int, groups: int, keep: int):
    """-> (expert ids int32 [T, top], weights fp32 [T, top]).  Router logits in fp32 (fp32 accumulation over the token's copy in
    the model dtype: 16-bit products are exact in fp32), then softmax, corrected group-limited choice and weights in one pass."""
    _dev(h, router, bias)
    T, W = h.shape
    E = router.shape[0]
    assert h.is_contiguous() and router.is_contiguous() and router.shape == (E, W) and router.dtype == h.dtype
    assert bias is None or (bias.dtype == h.dtype and bias.shape == (E,) and bias.is_contiguous())
    z = torch.empty((T, E), dtype=torch.float32, device=h.device)
    gemm_nt(z, h, router, T, E, W, lda=W, ldb=W, ldc=E)
    ids = torch.empty((T, top), dtype=torch.int32, device=h.device)
    wts = torch.empty((T, top), dtype=torch.float32, device=h.device)
    check_mix(mix_lib().msgl_mix_route(ids.data_ptr(), wts.data_ptr(), z.data_ptr(), _p(bias), T, E, top, groups, keep, _code(h),
                                       _stream()), "route")
    return ids, wts


def moe_sort(ids: torch.Tensor, experts: int):
    """-> (segment offsets int32 [E + 1], permutation int32 [T * top])."""
    _dev(ids)
    n = ids.numel()
    seg = torch.empty(2 * experts + 1, dtype=torch.int32, device=ids.device)  # offsets, then the per-expert counts (scratch)
    perm = torch.empty(max(n, 1), dtype=torch.int32, device=ids.device)
    check_mix(mix_lib().msgl_mix_moe_sort(seg.data_ptr(), perm.data_ptr(), seg[experts + 1:].data_ptr(), _i32(ids).data_ptr(), n,
                                          experts, _stream()), "moe_sort")
    return seg[: experts + 1], perm


def gemm_nt(C: torch.Tensor, A: torch.Tensor, B: torch.Tensor, M: int, N: int, K: int, *, lda: int, ldb: int, ldc: int,
            groups: int = 1, a_gs: int = 0, b_gs: int = 0, c_gs: int = 0, seg: Optional[torch.Tensor] = None,
            a_rows: Optional[torch.Tensor] = None, a_div: int = 1, c_rows: Optional[torch.Tensor] = None,
            act: int = ACT_NONE) -> None:
    """The grouped / segmented / gathered product of csrc/seqmix.hip; the caller states every stride (elements)."""
    _dev(C, A, B, seg, a_rows, c_rows)
    check_mix(mix_lib().msgl_mix_gemm_nt(
        C.data_ptr(), A.data_ptr(), B.data_ptr(), M, N, K, lda, ldb, ldc, groups, a_gs, b_gs, c_gs, _p(seg), _p(a_rows), a_div,
        _p(c_rows), act, _code(A), _code(B), _code(C), _stream()), "gemm_nt")


_NO_LIBRARY_SOLUTION: set = set()


def linear(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M, N] = x[M, K] w[N, K]^T, fp32 accumulation, output in x's dtype."""
    _dev(x, w)
    assert x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1] and x.dtype == w.dtype
    assert x.stride(1) == 1 and w.stride(1) == 1
    M, K = x.shape
    N = w.shape[0]
    if out is None:
        out = torch.empty((M, N), dtype=x.dtype, device=x.device)
    if M == 0:
        return out
    key = (M, N, K, x.stride(0), w.stride(0), out.stride(0), x.dtype)
    if key not in _NO_LIBRARY_SOLUTION:
        try:
            if x.dtype == torch.float32:
                ws = ops.gemm_workspace(x.device)
                _lib.check_gemm(_lib.gemm_lib().msgl_gemm_nt(
                    out.data_ptr(), x.data_ptr(), w.data_ptr(), M, N, K, x.stride(0), w.stride(0), out.stride(0), _lib.F32,
                    ws.data_ptr(), ws.numel(), _stream()), "gemm_nt (fp32)")
                return out
            return ops.linear(x, w, out=out)
        except _lib.MsglError:
            _NO_LIBRARY_SOLUTION.add(key)
    gemm_nt(out, x, w, M, N, K, lda=x.stride(0), ldb=w.stride(0), ldc=out.stride(0))
    return out


# ------------------------------------------------------------------ pre-norm hybrid decoders (csrc/mix_delta.hip)
GATE_SIGMOID, GATE_SILU = 0, 1


def embed_norm(table: torch.Tensor, ids: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> torch.Tensor:
    """out (fp32 [T, W]) = the embedding rows divided by their root mean square, times `weight`."""
    _dev(table, ids, weight, out)
    T, W = ids.shape[0], table.shape[1]
    assert table.is_contiguous() and weight.dtype == table.dtype and weight.shape == (W,) and weight.is_contiguous()
    assert out.dtype == torch.float32 and out.is_contiguous() and out.shape == (T, W)
    check_mix(mix_lib().msgl_mix_embed_norm(out.data_ptr(), table.data_ptr(), _i32(ids).data_ptr(), weight.data_ptr(), float(eps), T, W,
                                            _code(table), _stream()), "embed_norm")
    return out


def prenorm(x: torch.Tensor, *, y: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
            sum_out: Optional[torch.Tensor] = None, history: Optional[torch.Tensor] = None, depth_w: Optional[torch.Tensor] = None,
            x_out: Optional[torch.Tensor] = None, weight: Optional[torch.Tensor] = None, h_out: Optional[torch.Tensor] = None,
            eps: float = 1e-6, route=None, dtype: Optional[torch.dtype] = None):
    """s = x + sum_p gate[:, p] y[:, p] -> sum_out;  with depth_w (fp32 [n]) the row that goes on is
    sum_{j < n - 1} depth_w[j] history[j] + depth_w[n - 1] s -> x_out (history: fp32 [>= n - 1, rows, W]; sum_out may be
    history[n - 1]);  weight: h_out = rms_unit(row) * weight in the weight's dtype.  route = (router [E, W], bias [E] | None, top):
    the normed rows are routed in the same launch -> (expert ids int32 [rows, top], softmax weights fp32 [rows, top])."""
    _dev(x, y, gate, sum_out, history, depth_w, x_out, weight, h_out)
    rows, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    parts = 0
    if y is not None:
        assert y.is_contiguous() and y.shape[0] == rows and y.shape[-1] == W
        parts = 1 if y.dim() == 2 else y.shape[1]
    t = weight if weight is not None else y
    assert t is not None and (y is None or weight is None or y.dtype == weight.dtype)
    if gate is not None:
        assert gate.dtype == torch.float32 and gate.is_contiguous() and gate.numel() == rows * parts
    for o in (sum_out, x_out):
        assert o is None or (o.shape == (rows, W) and o.is_contiguous() and o.dtype == torch.float32)
    n_mix = 0
    if depth_w is not None:
        n_mix = depth_w.numel()
        assert depth_w.dtype == torch.float32 and depth_w.is_contiguous() and x_out is not None
        assert n_mix == 1 or (history is not None and history.dtype == torch.float32 and history.is_contiguous()
                              and history.shape[0] >= n_mix - 1 and history.shape[1:] == (rows, W))
    if weight is not None:
        assert weight.shape == (W,) and weight.is_contiguous() and h_out is not None
        assert h_out.shape == (rows, W) and h_out.is_contiguous() and h_out.dtype == weight.dtype
    router = bias = ids = wts = None
    E = top = 0
    if route is not None:
        router, bias, top = route
        _dev(router, bias)
        E = router.shape[0]
        assert router.shape == (E, W) and router.is_contiguous() and router.dtype == weight.dtype
        assert bias is None or (bias.dtype == weight.dtype and bias.shape == (E,) and bias.is_contiguous())
        ids = torch.empty((rows, top), dtype=torch.int32, device=x.device)
        wts = torch.empty((rows, top), dtype=torch.float32, device=x.device)
    if rows:
        check_mix(mix_lib().msgl_mix_prenorm(
            x.data_ptr(), _p(y), parts, _p(gate), _p(sum_out), _p(history), 0 if history is None else history.stride(0), _p(depth_w),
            n_mix, _p(x_out), _p(weight), _p(h_out), float(eps), rows, W, _code(t), _p(router), _p(bias), E, top, _p(ids), _p(wts),
            _stream()), "prenorm")
    return None if route is None else (ids, wts)


def poly_act(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """coef[0] N(z) + coef[1] N(z^2) + coef[2] N(z^3) + coef[3] per row (N = divide by the row's root mean square)."""
    _dev(z, coef)
    rows, N = z.shape
    assert z.stride(1) == 1 and coef.dtype == torch.float32 and coef.numel() == 4 and coef.is_contiguous()
    out = torch.empty((rows, N), dtype=z.dtype, device=z.device)
    check_mix(mix_lib().msgl_mix_poly_act(out.data_ptr(), z.data_ptr(), z.stride(0), coef.data_ptr(), float(eps), rows, N, _code(z),
                                          _stream()), "poly_act")
    return out


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """rows [gate | up] of 2 N -> silu(gate) * up, rows of N."""
    _dev(gate_up)
    rows, N2 = gate_up.shape
    assert gate_up.is_contiguous() and N2 % 2 == 0
    out = torch.empty((rows, N2 // 2), dtype=gate_up.dtype, device=gate_up.device)
    check_mix(mix_lib().msgl_mix_silu_mul(out.data_ptr(), gate_up.data_ptr(), rows, N2 // 2, _code(gate_up), _stream()), "silu_mul")
    return out


def route_top(h: torch.Tensor, router: torch.Tensor, bias: Optional[torch.Tensor], top: int):
    """-> (expert ids int32 [T, top], weights fp32 [T, top]): fp32 logits (product kernel, fp32 accumulation) + bias, the `top`
    largest win, weights = softmax over the winners."""
    _dev(h, router, bias)
    T, W = h.shape
    E = router.shape[0]
    assert h.is_contiguous() and router.is_contiguous() and router.shape == (E, W) and router.dtype == h.dtype
    assert bias is None or (bias.dtype == h.dtype and bias.shape == (E,) and bias.is_contiguous())
    z = torch.empty((T, E), dtype=torch.float32, device=h.device)
    gemm_nt(z, h, router, T, E, W, lda=W, ldb=W, ldc=E)
    ids = torch.empty((T, top), dtype=torch.int32, device=h.device)
    wts = torch.empty((T, top), dtype=torch.float32, device=h.device)
    check_mix(mix_lib().msgl_mix_route_top(ids.data_ptr(), wts.data_ptr(), z.data_ptr(), _p(bias), T, E, top, _code(h), _stream()),
              "route_top")
    return ids, wts


def kv_store(k_cache: torch.Tensor, v_cache: torch.Tensor, out_loc: torch.Tensor, src: torch.Tensor, k_off: int, v_off: int,
             v_first: Optional[torch.Tensor] = None, lam: Optional[torch.Tensor] = None) -> None:
    """k = src[:, k_off : +nk], v = src[:, v_off : +nv] -> the cache rows at out_loc; v blended with v_first by `lam` when given."""
    _dev(k_cache, v_cache, out_loc, src, v_first, lam)
    T = src.shape[0]
    nk, nv = k_cache.shape[1], v_cache.shape[1]
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == src.dtype == v_cache.dtype
    assert src.stride(1) == 1 and out_loc.shape[0] == T
    if v_first is not None:
        assert v_first.dtype == src.dtype and v_first.stride(1) == 1 and v_first.shape == (T, nv) and lam.dtype == src.dtype
    check_mix(mix_lib().msgl_mix_kv_store(
        k_cache.data_ptr(), v_cache.data_ptr(), _i32(out_loc).data_ptr(), src.data_ptr(), src.stride(0), k_off, v_off, nk, nv,
        _p(v_first), 0 if v_first is None else v_first.stride(0), _p(lam), T, _code(src), _stream()), "kv_store")


def window_attn_splits(batch: int, total_q: int, window: int, max_keys: int) -> int:
    """Key ranges per token for a step with few query tokens: enough workgroups to fill the chip, at least two 64-key tiles each.
    A function of static sizes only (rows, the window or the LONGEST possible key count), so a captured graph keeps its grid."""
    if total_q >= 8 * batch and total_q >= 256:
        return 1
    keys = min(window, max_keys) if window > 0 else max_keys
    return max(1, min(512 // max(total_q, 1), keys // 128, 32))


def window_attn(out: torch.Tensor, src: torch.Tensor, g_off: int, k_cache: torch.Tensor, v_cache: torch.Tensor, table: torch.Tensor,
                req_rows: torch.Tensor, seq_lens: torch.Tensor, cu_q: torch.Tensor, batch: int, H: int, G: int, d: int, dv: int,
                window: int, scale: float, talk: torch.Tensor, splits: int = 1) -> None:
    """Sliding-window attention with the heads' scores mixed by `talk` (fp32 [H, H]) and a sigmoid gate per head (src[:, g_off + h]);
    q = src[:, : H * d].  out: [T, H * dv] in the model dtype.  splits > 1: the visible keys of every token in that many ranges
    (partial results merged by a second launch), for steps with few query tokens."""
    _dev(out, src, k_cache, v_cache, table, req_rows, seq_lens, cu_q, talk)
    T = src.shape[0]
    assert src.stride(1) == 1 and out.is_contiguous() and out.shape == (T, H * dv) and out.dtype == src.dtype
    assert k_cache.is_contiguous() and k_cache.shape[1] == G * d and v_cache.is_contiguous() and v_cache.shape[1] == G * dv
    assert k_cache.dtype == src.dtype == v_cache.dtype and talk.dtype == torch.float32 and talk.is_contiguous() and talk.shape == (H, H)
    assert table.dtype == torch.int32 and table.stride(1) == 1
    assert req_rows.numel() >= batch and seq_lens.numel() >= batch and cu_q.numel() >= batch + 1
    ws = None
    if splits > 1:
        ws = torch.empty(mix_lib().msgl_mix_window_attn_workspace_floats(T, H, dv, splits), dtype=torch.float32, device=out.device)
    check_mix(mix_lib().msgl_mix_window_attn(
        out.data_ptr(), src.data_ptr(), src.stride(0), g_off, k_cache.data_ptr(), v_cache.data_ptr(), table.data_ptr(), table.stride(0),
        _i32(req_rows).data_ptr(), _i32(seq_lens).data_ptr(), _i32(cu_q).data_ptr(), batch, T, H, G, d, dv, window, float(scale),
        talk.data_ptr(), _code(src), splits, _p(ws), _stream()), "window_attn")


def short_conv(src: torch.Tensor, C: int, taps: torch.Tensor, state: Optional[torch.Tensor], cu_q: torch.Tensor, seq_lens: torch.Tensor,
               slots: torch.Tensor, batch: int, unit_heads: int, scaled_heads: int, d: int, bias: Optional[torch.Tensor] = None,
               model_dtype: bool = False) -> torch.Tensor:
    """Causal per-channel convolution + SiLU of src[:, :C] (taps [C, n]; state [slots, n - 1, C] carries the inputs before the
    portion and is moved on), unit vectors for the first `unit_heads` groups of d channels -> fp32 [T, C] (model_dtype: in src's
    dtype instead, for a result that feeds a projection)."""
    _dev(src, taps, state, cu_q, seq_lens, slots, bias)
    T, n = src.shape[0], taps.shape[1]
    assert bias is None or (bias.dtype == src.dtype and bias.shape == (C,) and bias.is_contiguous())
    assert src.stride(1) == 1 and taps.is_contiguous() and taps.shape[0] == C and taps.dtype == src.dtype
    assert n == 1 or (state.is_contiguous() and state.dtype == src.dtype and state.shape[1:] == (n - 1, C))
    out = torch.empty((T, C), dtype=src.dtype if model_dtype else torch.float32, device=src.device)
    check_mix(mix_lib().msgl_mix_short_conv(
        0 if model_dtype else out.data_ptr(), out.data_ptr() if model_dtype else 0, src.data_ptr(), src.stride(0), taps.data_ptr(), _p(bias), _p(state), _i32(cu_q).data_ptr(), _i32(seq_lens).data_ptr(),
        _i32(slots).data_ptr(), batch, T, C, n, unit_heads, scaled_heads, d, _code(src), _stream()), "short_conv")
    return out


def delta_rule(out: torch.Tensor, qkv: torch.Tensor, state: torch.Tensor, b_raw: torch.Tensor, a_raw: torch.Tensor, per_channel: bool,
               rate: torch.Tensor, dt_bias: torch.Tensor, cu_q: torch.Tensor, seq_lens: torch.Tensor, slots: torch.Tensor, batch: int,
               G: int, chunks=None) -> None:
    """state: fp32 [slots, H, d, dv]; qkv: fp32 rows [q G*d | k G*d | v H*dv]; b_raw [T, H], a_raw [T, H] or [T, H*d] in the model
    dtype (views with a row stride are fine); rate = -exp(A_log) and dt_bias in fp32.  chunks = (items int32 [n, 3], item_first
    int32 [batch + 1], n) cuts long portions into pieces that run in parallel (see include/msgl_mix.h)."""
    _dev(out, qkv, state, b_raw, a_raw, rate, dt_bias, cu_q, seq_lens, slots)
    _, H, d, dv = state.shape
    T = qkv.shape[0]
    na = H * d if per_channel else H
    assert state.dtype == torch.float32 and state.is_contiguous() and qkv.dtype == torch.float32 and qkv.is_contiguous()
    assert qkv.shape == (T, 2 * G * d + H * dv) and out.dtype == torch.float32 and out.is_contiguous() and out.shape == (T, H * dv)
    assert b_raw.stride(1) == 1 and a_raw.stride(1) == 1 and b_raw.shape == (T, H) and a_raw.shape == (T, na) and a_raw.dtype == b_raw.dtype
    assert rate.dtype == torch.float32 and rate.shape == (H,) and dt_bias.dtype == torch.float32 and dt_bias.shape == (na,)
    items = first = scratch = None
    n_items = 0
    if chunks is not None:
        items, first, n_items = chunks
        _dev(items, first)
        assert items.numel() == 3 * n_items and first.numel() == batch + 1
        scratch = torch.empty(n_items * H * d * (2 * dv + d), dtype=torch.float32, device=out.device)
    check_mix(mix_lib().msgl_mix_delta_rule(
        out.data_ptr(), qkv.data_ptr(), state.data_ptr(), b_raw.data_ptr(), b_raw.stride(0), a_raw.data_ptr(), a_raw.stride(0),
        int(per_channel), rate.data_ptr(), dt_bias.data_ptr(), _i32(cu_q).data_ptr(), _i32(seq_lens).data_ptr(), _i32(slots).data_ptr(),
        batch, H, G, d, dv, _code(b_raw), n_items, _p(None if items is None else _i32(items)),
        _p(None if first is None else _i32(first)), _p(scratch), _stream()), "delta_rule")


def head_gated_norm(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float, H: int, dv: int, gate_act: int) -> torch.Tensor:
    """Per head: o / rms(o) * weight[dv] * act(gate) -> [rows, H * dv] in the gate's dtype."""
    _dev(o, gate, weight)
    rows = o.shape[0]
    assert o.dtype == torch.float32 and o.is_contiguous() and o.shape == (rows, H * dv) and gate.shape == (rows, H * dv)
    assert gate.stride(1) == 1 and weight.dtype == gate.dtype and weight.shape == (dv,) and weight.is_contiguous()
    out = torch.empty((rows, H * dv), dtype=gate.dtype, device=o.device)
    check_mix(mix_lib().msgl_mix_head_gated_norm(out.data_ptr(), o.data_ptr(), gate.data_ptr(), gate.stride(0), weight.data_ptr(),
                                                 float(eps), rows, H, dv, gate_act, _code(gate), _stream()), "head_gated_norm")
    return out


# ------------------------------------------------------------------ parallel-residual hybrid decoders (csrc/mix_par.hip)
def _f32(t: Optional[torch.Tensor], n: int) -> Optional[torch.Tensor]:
    assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.shape == (n,)), (None if t is None else (t.dtype, t.shape))
    return t


def embed_scaled(table: torch.Tensor, ids: torch.Tensor, scale: float, out: Optional[torch.Tensor] = None, *, pair: Optional[torch.Tensor] = None,
                 buckets: int = 0, mul_prev: int = 0, mul_cur: int = 0, positions: Optional[torch.Tensor] = None,
                 cu_q: Optional[torch.Tensor] = None, req_rows: Optional[torch.Tensor] = None, batch: int = 0,
                 prev_tok: Optional[torch.Tensor] = None) -> torch.Tensor:
    """-> fp32 [T, W] = scale * table[id] + pair[(previous id * mul_prev + id * mul_cur) mod buckets] (pair row `buckets` at position
    0; the id before a portion's first token: prev_tok[req_rows[b]], int32)."""
    _dev(table, ids, pair, positions, cu_q, req_rows, prev_tok)
    T, W = ids.shape[0], table.shape[1]
    assert table.is_contiguous() and (pair is None or (pair.is_contiguous() and pair.dtype == table.dtype and pair.shape == (buckets + 1, W)))
    if out is None:
        out = torch.empty((T, W), dtype=torch.float32, device=table.device)
    assert out.dtype == torch.float32 and out.is_contiguous() and out.shape == (T, W)
    check_mix(mix_lib().msgl_mix_embed_scaled(
        out.data_ptr(), table.data_ptr(), _p(pair), _i32(ids).data_ptr(), _p(positions), _p(cu_q), _p(req_rows), batch, _p(prev_tok),
        float(scale), buckets, mul_prev, mul_cur, T, W, _code(table), _stream()), "embed_scaled")
    return out


def shift_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, *, dtype: torch.dtype, w_offset: float = 0.0, parts=(), bias: Optional[torch.Tensor] = None,
               x_out: Optional[torch.Tensor] = None, h_out: Optional[torch.Tensor] = None, g_out: Optional[torch.Tensor] = None,
               shift: Optional[torch.Tensor] = None, state: Optional[torch.Tensor] = None, staging: Optional[torch.Tensor] = None,
               positions: Optional[torch.Tensor] = None, cu_q: Optional[torch.Tensor] = None, req_rows: Optional[torch.Tensor] = None,
               batch: int = 0) -> None:
    """row = x + bias + sum over parts (y, v) of v * y -> x_out (fp32; a buffer other than x);  h = rms_unit(row) * (weight + w_offset) -> h_out;
    with `shift`: g = h + (h of the token before - h) * shift -> g_out (the token before a portion: state[req_rows[b]], fp32; the
    last h of request b -> staging[b]).  weight, shift, bias and the v of a part: fp32 [W]; y: [rows, W] views in `dtype`."""
    rows, W = x.shape
    _dev(x, weight, bias, x_out, h_out, g_out, shift, state, staging, positions, cu_q, req_rows)
    assert x.dtype == torch.float32 and x.is_contiguous() and len(parts) <= 2
    _f32(weight, W), _f32(bias, W), _f32(shift, W)
    ys = []
    for y, v in parts:
        _dev(y, v)
        assert y.dtype == dtype and y.shape == (rows, W) and y.stride(1) == 1
        ys.append((y.data_ptr(), y.stride(0), _p(_f32(v, W))))
    ys += [(0, 0, 0)] * (2 - len(ys))
    for o, dt in ((x_out, torch.float32), (h_out, dtype), (g_out, dtype)):
        assert o is None or (o.shape == (rows, W) and o.is_contiguous() and o.dtype == dt)
    if shift is not None:
        assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1] == W
        assert staging.dtype == torch.float32 and staging.is_contiguous() and staging.shape == (batch, W)
    if rows:
        check_mix(mix_lib().msgl_mix_shift_norm(
            x.data_ptr(), _p(x_out), ys[0][0], ys[0][1], ys[0][2], ys[1][0], ys[1][1], ys[1][2], _p(bias), weight.data_ptr(), float(w_offset), _p(shift),
            _p(h_out), _p(g_out), _p(state), _p(staging), _p(positions), _p(cu_q), _p(req_rows), batch, float(eps), rows, W,
            _lib.BF16 if dtype == torch.bfloat16 else _lib.F32, _stream()), "shift_norm")


def commit_rows(dst: Optional[torch.Tensor], src: Optional[torch.Tensor], slots: torch.Tensor, batch: int, cu_q: torch.Tensor,
                prev_tok: Optional[torch.Tensor] = None, ids: Optional[torch.Tensor] = None) -> None:
    """dst[l, slots[b]] = src[l, b] (fp32 [L, rows, W] <- [L, batch, W]); prev_tok[slots[b]] = the last id of request b."""
    _dev(dst, src, slots, cu_q, prev_tok, ids)
    L = W = 0
    if dst is not None:
        L, _, W = dst.shape
        assert dst.dtype == torch.float32 and dst.is_contiguous() and src.dtype == torch.float32 and src.is_contiguous()
        assert src.shape == (L, batch, W)
    check_mix(mix_lib().msgl_mix_commit_rows(_p(dst), 0 if dst is None else dst.stride(0), _p(src), 0 if src is None else src.stride(0), L,
                                             _i32(slots).data_ptr(), batch, W, _p(prev_tok), _p(ids), _i32(cu_q).data_ptr(), _stream()),
              "commit_rows")


def qk_prep(proj: torch.Tensor, bias: Optional[torch.Tensor], k_cache: torch.Tensor, v_cache: torch.Tensor, out_loc: torch.Tensor,
            positions: torch.Tensor, cos_sin: Optional[torch.Tensor], eps: float, H: int, G: int, d: int, dv: int, *, interleaved: bool,
            unit: bool, unit_v: bool = False) -> torch.Tensor:
    """Projection rows [q | k | v | ...] (+ fp32 bias) -> rotated (and unit-RMS) q as fp32 [T, H * d]; k, v into the cache rows
    (unit_v: every value head divided by its root mean square first)."""
    _dev(proj, bias, k_cache, v_cache, out_loc, positions, cos_sin)
    T = proj.shape[0]
    n = (H + G) * d + G * dv
    assert proj.stride(1) == 1 and proj.shape[1] >= n and (bias is None or _f32(bias, n) is not None)
    assert k_cache.is_contiguous() and k_cache.shape[1] == G * d and v_cache.is_contiguous() and v_cache.shape[1] == G * dv
    assert k_cache.dtype == proj.dtype == v_cache.dtype and out_loc.shape[0] == T
    rd = 0
    if cos_sin is not None:
        assert cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.dim() == 2
        rd = cos_sin.shape[1]
    q = torch.empty((T, H * d), dtype=torch.float32, device=proj.device)
    check_mix(mix_lib().msgl_mix_qk_prep(
        proj.data_ptr(), proj.stride(0), _p(bias), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), _i32(out_loc).data_ptr(),
        _i32(positions).data_ptr(), _p(cos_sin), rd, int(interleaved), int(unit) | (2 if unit_v else 0), float(eps), T, H, G, d, dv, _code(proj), _stream()),
        "qk_prep")
    return q


def sigmoid_attn_splits(batch: int, total_q: int, H: int, G: int, max_keys: int) -> int:
    """Key ranges per request for a step with few query rows: enough workgroups to fill the chip, at least 256 keys each.  A
    function of static sizes only (batch, rows, the LONGEST possible key count), so a captured graph keeps its grid."""
    rep = H // G
    hb = 1
    while hb * 2 <= min(rep, 64):
        hb *= 2
    blocks = (-(-total_q // (64 // hb)) + batch) * G * -(-rep // hb)
    return max(1, min(1024 // max(blocks, 1), max_keys // 256, 64))


def sigmoid_attn(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, table: torch.Tensor, req_rows: torch.Tensor,
                 seq_lens: torch.Tensor, cu_q: torch.Tensor, batch: int, H: int, G: int, d: int, dv: int, scale: float, softcap: float,
                 pb: Optional[torch.Tensor], out_scale: float = 1.0, splits: int = 1) -> None:
    """out[:, : H * dv] (a view with a row stride is fine) = out_scale * sum over visible keys of sigmoid(cap(scale q.k) + pb[h]) v."""
    _dev(out, q, k_cache, v_cache, table, req_rows, seq_lens, cu_q, pb)
    T = q.shape[0]
    assert q.dtype == torch.float32 and q.is_contiguous() and q.shape == (T, H * d)
    assert out.shape == (T, H * dv) and out.stride(1) == 1 and out.dtype == k_cache.dtype == v_cache.dtype
    assert k_cache.is_contiguous() and k_cache.shape[1] == G * d and v_cache.is_contiguous() and v_cache.shape[1] == G * dv
    assert table.dtype == torch.int32 and table.stride(1) == 1 and (pb is None or _f32(pb, H) is not None)
    assert req_rows.numel() >= batch and seq_lens.numel() >= batch and cu_q.numel() >= batch + 1
    ws = None
    if splits > 1:
        ws = torch.empty(mix_lib().msgl_mix_sigmoid_attn_workspace_floats(T, H, dv, splits), dtype=torch.float32, device=out.device)
    check_mix(mix_lib().msgl_mix_sigmoid_attn(
        out.data_ptr(), out.stride(0), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), table.data_ptr(), table.stride(0),
        _i32(req_rows).data_ptr(), _i32(seq_lens).data_ptr(), _i32(cu_q).data_ptr(), batch, T, H, G, d, dv, float(scale), float(softcap),
        _p(pb), float(out_scale), _code(k_cache), splits, _p(ws), _stream()), "sigmoid_attn")


def ssd(out: torch.Tensor, xbc: torch.Tensor, dt_raw: torch.Tensor, state: torch.Tensor, rate: torch.Tensor, dt_bias: torch.Tensor,
        D: torch.Tensor, cu_q: torch.Tensor, seq_lens: torch.Tensor, slots: torch.Tensor, batch: int, G: int, chunks=None) -> None:
    """state: fp32 [slots, H, N, P]; xbc: fp32 rows [x H*P | B G*N | C G*N]; dt_raw [T, H] in the model dtype (a view with a row
    stride is fine); rate = -exp(A_log), dt_bias, D in fp32 [H].  chunks = (items int32 [n, 3], item_first int32 [batch + 1], n)
    cuts long portions into pieces that run in parallel."""
    _dev(out, xbc, dt_raw, state, rate, dt_bias, D, cu_q, seq_lens, slots)
    _, H, N, P = state.shape
    T = xbc.shape[0]
    assert state.dtype == torch.float32 and state.is_contiguous() and xbc.dtype == torch.float32 and xbc.stride(1) == 1
    assert xbc.shape[1] == H * P + 2 * G * N and out.dtype == torch.float32 and out.is_contiguous() and out.shape == (T, H * P)
    assert dt_raw.shape == (T, H) and dt_raw.stride(1) == 1
    _f32(rate, H), _f32(dt_bias, H), _f32(D, H)
    items = first = scratch = None
    n_items = 0
    if chunks is not None:
        items, first, n_items = chunks
        _dev(items, first)
        assert items.numel() == 3 * n_items and first.numel() == batch + 1
        scratch = torch.empty(n_items * H * (N * P + 1), dtype=torch.float32, device=out.device)
    check_mix(mix_lib().msgl_mix_ssd(
        out.data_ptr(), xbc.data_ptr(), xbc.stride(0), dt_raw.data_ptr(), dt_raw.stride(0), state.data_ptr(), rate.data_ptr(),
        dt_bias.data_ptr(), D.data_ptr(), _i32(cu_q).data_ptr(), _i32(seq_lens).data_ptr(), _i32(slots).data_ptr(), batch, H, G, N, P,
        _code(dt_raw), n_items, _p(None if items is None else _i32(items)), _p(None if first is None else _i32(first)), _p(scratch),
        _stream()), "ssd")


def gate_group_norm(out: torch.Tensor, y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, eps: float, groups: int,
                    out_scale: float = 1.0) -> None:
    """out (a [rows, N] view, model dtype) = rms_unit per group of (y * silu(z)) * weight * out_scale; y fp32, z a view in out's dtype."""
    _dev(out, y, z, weight)
    rows, N = y.shape
    assert y.dtype == torch.float32 and y.is_contiguous() and z.shape == (rows, N) and z.stride(1) == 1 and z.dtype == out.dtype
    assert out.shape == (rows, N) and out.stride(1) == 1 and _f32(weight, N) is not None
    check_mix(mix_lib().msgl_mix_gate_group_norm(out.data_ptr(), out.stride(0), y.data_ptr(), z.data_ptr(), z.stride(0), weight.data_ptr(),
                                                 float(eps), rows, N, groups, float(out_scale), _code(z), _stream()), "gate_group_norm")


def xielu(z: torch.Tensor, pq: torch.Tensor) -> torch.Tensor:
    """z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2;  pq = (p, q) fp32 on the device."""
    _dev(z, pq)
    rows, N = z.shape
    assert z.stride(1) == 1 and _f32(pq, 2) is not None
    out = torch.empty((rows, N), dtype=z.dtype, device=z.device)
    check_mix(mix_lib().msgl_mix_xielu(out.data_ptr(), z.data_ptr(), z.stride(0), pq.data_ptr(), rows, N, _code(z), _stream()), "xielu")
    return out


# ------------------------------------------------------------------ looped pre-norm hybrid decoders (csrc/mix_scan.hip)
def norm_conv(x: torch.Tensor, weight: torch.Tensor, eps: float, groups: int, h_out: torch.Tensor, *, parts=(), mult: float = 1.0,
              add: Optional[torch.Tensor] = None, x_out: Optional[torch.Tensor] = None, taps: Optional[torch.Tensor] = None,
              state: Optional[torch.Tensor] = None, staging: Optional[torch.Tensor] = None, cu_q: Optional[torch.Tensor] = None,
              seq_lens: Optional[torch.Tensor] = None, req_rows: Optional[torch.Tensor] = None, batch: int = 0) -> None:
    """row = x + mult * (sum of the parts' rows) + add -> x_out (fp32, a buffer other than x);  h = row normed in `groups` equal parts,
    times weight;  h_out = h + sum_j taps[:, j] * h of the token (n - 1 - j) before (taps [W, n] in h_out's dtype; the tokens before a
    portion: state[req_rows[b]], fp32 [rows, n - 1, W]; every request's new state rows -> staging[b], fp32 [batch, n - 1, W]).
    parts: up to two tensors [rows, W] or [rows, p, W] in h_out's dtype; add: fp32 [W]."""
    rows, W = x.shape
    _dev(x, weight, h_out, add, x_out, taps, state, staging, cu_q, seq_lens, req_rows)
    dt = h_out.dtype
    assert x.dtype == torch.float32 and x.is_contiguous() and weight.dtype == dt and weight.shape == (W,) and weight.is_contiguous()
    assert h_out.shape == (rows, W) and h_out.is_contiguous() and len(parts) <= 2 and W % groups == 0
    _f32(add, W)
    assert x_out is None or (x_out.dtype == torch.float32 and x_out.is_contiguous() and x_out.shape == (rows, W) and x_out.data_ptr() != x.data_ptr())
    ys = []
    for y in parts:
        _dev(y)
        assert y.dtype == dt and y.is_contiguous() and y.shape[0] == rows and y.shape[-1] == W and y.dim() in (2, 3)
        ys.append((y.data_ptr(), 1 if y.dim() == 2 else y.shape[1]))
    ys += [(0, 0)] * (2 - len(ys))
    n = 1
    if taps is not None:
        n = taps.shape[1]
        assert taps.dtype == dt and taps.is_contiguous() and taps.shape == (W, n)
    if n > 1:
        assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (n - 1, W)
        assert staging.dtype == torch.float32 and staging.is_contiguous() and staging.shape == (batch, n - 1, W)
        assert cu_q.numel() >= batch + 1 and seq_lens.numel() >= batch and req_rows.numel() >= batch
    if rows:
        check_mix(mix_lib().msgl_mix_norm_conv(
            x.data_ptr(), _p(x_out), ys[0][0], ys[0][1], ys[1][0], ys[1][1], float(mult), _p(add), weight.data_ptr(), groups, float(eps),
            _p(taps), n, _p(state) if n > 1 else 0, _p(staging) if n > 1 else 0, h_out.data_ptr(),
            _p(None if cu_q is None or n == 1 else _i32(cu_q)), _p(None if n == 1 else _i32(seq_lens)), _p(None if n == 1 else _i32(req_rows)),
            batch, rows, W, _code(h_out), _stream()), "norm_conv")


def selective_scan(x: torch.Tensor, z: torch.Tensor, dt_in: torch.Tensor, bc: torch.Tensor, A: torch.Tensor, dt_bias: torch.Tensor,
                   D: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor, seq_lens: torch.Tensor, slots: torch.Tensor, batch: int,
                   chunks=None) -> torch.Tensor:
    """state: fp32 [slots, C, N]; x, z, dt_in: [T, C] in the model dtype (views with a row stride are fine); bc: [T, 2 N] = B | C;
    A = -exp(A_log) fp32 [C, N]; dt_bias, D fp32 [C] -> y * silu(z), [T, C] in the model dtype.  chunks = (items int32 [n, 3],
    item_first int32 [batch + 1], n) cuts long portions into pieces that run in parallel."""
    _dev(x, z, dt_in, bc, A, dt_bias, D, state, cu_q, seq_lens, slots)
    _, C, N = state.shape
    T = x.shape[0]
    assert state.dtype == torch.float32 and state.is_contiguous() and A.dtype == torch.float32 and A.is_contiguous() and A.shape == (C, N)
    for t in (x, z, dt_in):
        assert t.shape == (T, C) and t.stride(1) == 1 and t.dtype == x.dtype
    assert bc.shape == (T, 2 * N) and bc.stride(1) == 1 and bc.dtype == x.dtype
    _f32(dt_bias, C), _f32(D, C)
    out = torch.empty((T, C), dtype=x.dtype, device=x.device)
    items = first = scratch = None
    n_items = 0
    if chunks is not None:
        items, first, n_items = chunks
        _dev(items, first)
        assert items.numel() == 3 * n_items and first.numel() == batch + 1
        scratch = torch.empty(n_items * C * (N + 1), dtype=torch.float32, device=x.device)
    check_mix(mix_lib().msgl_mix_selective_scan(
        out.data_ptr(), x.data_ptr(), x.stride(0), z.data_ptr(), z.stride(0), dt_in.data_ptr(), dt_in.stride(0), bc.data_ptr(), bc.stride(0),
        A.data_ptr(), dt_bias.data_ptr(), D.data_ptr(), state.data_ptr(), _i32(cu_q).data_ptr(), _i32(seq_lens).data_ptr(),
        _i32(slots).data_ptr(), batch, C, N, _code(x), n_items, _p(None if items is None else _i32(items)),
        _p(None if first is None else _i32(first)), _p(scratch), _stream()), "selective_scan")
    return out


def sink_attn_splits(batch: int, total_q: int, H: int, G: int, window: int, max_keys: int) -> int:
    """Key ranges per request for a step with few query rows: enough workgroups to fill the chip, at least 256 keys each.  A
    function of static sizes only (batch, rows, the window or the LONGEST possible key count), so a captured graph keeps its grid."""
    rep = H // G
    hb = 1
    while hb * 2 <= min(rep, 64):
        hb *= 2
    blocks = (-(-total_q // (64 // hb)) + batch) * G * -(-rep // hb)
    keys = min(window, max_keys) if window > 0 else max_keys
    return max(1, min(1024 // max(blocks, 1), keys // 256, 64))


def sink_attn(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, table: torch.Tensor, req_rows: torch.Tensor,
              seq_lens: torch.Tensor, cu_q: torch.Tensor, batch: int, H: int, G: int, d: int, dv: int, scale: float, window: int,
              sink: Optional[torch.Tensor], splits: int = 1) -> None:
    """out[:, : H * dv] = softmax attention over the last `window` keys (0: all earlier keys) with exp(sink[h]) as one more term of
    the denominator (sink fp32 [H] or None)."""
    _dev(out, q, k_cache, v_cache, table, req_rows, seq_lens, cu_q, sink)
    T = q.shape[0]
    assert q.dtype == torch.float32 and q.is_contiguous() and q.shape == (T, H * d)
    assert out.shape == (T, H * dv) and out.stride(1) == 1 and out.dtype == k_cache.dtype == v_cache.dtype
    assert k_cache.is_contiguous() and k_cache.shape[1] == G * d and v_cache.is_contiguous() and v_cache.shape[1] == G * dv
    assert table.dtype == torch.int32 and table.stride(1) == 1 and (sink is None or _f32(sink, H) is not None)
    assert req_rows.numel() >= batch and seq_lens.numel() >= batch and cu_q.numel() >= batch + 1
    ws = None
    if splits > 1:
        ws = torch.empty(mix_lib().msgl_mix_sink_attn_workspace_floats(T, H, dv, splits), dtype=torch.float32, device=out.device)
    check_mix(mix_lib().msgl_mix_sink_attn(
        out.data_ptr(), out.stride(0), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), table.data_ptr(), table.stride(0),
        _i32(req_rows).data_ptr(), _i32(seq_lens).data_ptr(), _i32(cu_q).data_ptr(), batch, T, H, G, d, dv, float(scale), int(window),
        _p(sink), _code(k_cache), splits, _p(ws), _stream()), "sink_attn")


def route_sigmoid(h: torch.Tensor, router: torch.Tensor, top: int):
    """-> (expert ids int32 [T, top], weights fp32 [T, top]): fp32 logits (product kernel, fp32 accumulation), the `top` largest
    win, the weight of a choice is the sigmoid of its logit."""
    _dev(h, router)
    T, W = h.shape
    E = router.shape[0]
    assert h.is_contiguous() and router.is_contiguous() and router.shape == (E, W) and router.dtype == h.dtype
    z = torch.empty((T, E), dtype=torch.float32, device=h.device)
    gemm_nt(z, h, router, T, E, W, lda=W, ldb=W, ldc=E)
    ids = torch.empty((T, top), dtype=torch.int32, device=h.device)
    wts = torch.empty((T, top), dtype=torch.float32, device=h.device)
    check_mix(mix_lib().msgl_mix_route_sigmoid(ids.data_ptr(), wts.data_ptr(), z.data_ptr(), T, E, top, _stream()), "route_sigmoid")
    return ids, wts


def scale_rows(h: torch.Tensor, wts: torch.Tensor) -> torch.Tensor:
    """-> [T * top, W]: row t * top + k = wts[t, k] * h[t]."""
    _dev(h, wts)
    T, W = h.shape
    top = wts.shape[1]
    assert h.is_contiguous() and wts.dtype == torch.float32 and wts.is_contiguous() and wts.shape == (T, top)
    out = torch.empty((T * top, W), dtype=h.dtype, device=h.device)
    check_mix(mix_lib().msgl_mix_scale_rows(out.data_ptr(), h.data_ptr(), wts.data_ptr(), T, top, W, _code(h), _stream()), "scale_rows")
    return out


def route_scale(h: torch.Tensor, router: torch.Tensor, top: int):
    """route_sigmoid and scale_rows in one launch, a workgroup per token (steps with few tokens) -> (ids, weights, scaled rows)."""
    _dev(h, router)
    T, W = h.shape
    E = router.shape[0]
    assert h.is_contiguous() and router.is_contiguous() and router.shape == (E, W) and router.dtype == h.dtype
    ids = torch.empty((T, top), dtype=torch.int32, device=h.device)
    wts = torch.empty((T, top), dtype=torch.float32, device=h.device)
    out = torch.empty((T * top, W), dtype=h.dtype, device=h.device)
    check_mix(mix_lib().msgl_mix_route_scale(ids.data_ptr(), wts.data_ptr(), out.data_ptr(), h.data_ptr(), router.data_ptr(), T, E, top, W,
                                             _code(h), _stream()), "route_scale")
    return ids, wts, out


def sigmoid_gate(o: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """-> o * sigmoid(g) in g's dtype; o fp32 [rows, N], g a [rows, N] view with a row stride."""
    _dev(o, g)
    rows, N = o.shape
    assert o.dtype == torch.float32 and o.is_contiguous() and g.shape == (rows, N) and g.stride(1) == 1
    out = torch.empty((rows, N), dtype=g.dtype, device=o.device)
    check_mix(mix_lib().msgl_mix_sigmoid_gate(out.data_ptr(), o.data_ptr(), g.data_ptr(), g.stride(0), rows, N, _code(g), _stream()),
              "sigmoid_gate")
    return out


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap * tanh(x / cap) in place."""
    _dev(x)
    assert x.dim() == 2 and x.stride(1) == 1
    if x.shape[0] == 0:
        return x
    check_mix(mix_lib().msgl_mix_softcap(x.data_ptr(), x.stride(0), x.shape[0], x.shape[1], float(cap), _code(x), _stream()), "softcap")
    return x

"""KV pool behind the reference's KV-cache interface (P/kvcache/base.py:10-37; the pool it replaces: P/kvcache/mha_pool.py:10-68).

One HBM allocation for the process lifetime, sized for 288 GB parts:
    pool[2 (k|v), num_layers, num_pages, page_size, local_kv_heads, head_dim]
One layer's K (or V) is therefore a contiguous slab of token rows, a token's row is local_kv_heads x 256 B
(2048 B at TP1 ... 256 B at TP8), slots are token-granular indices into that slab, and the extra last page is
the dummy target of padded graph rows (P/engine/engine.py:57-63, 89-98).  Only the stand-alone driver of this
repository (engine.py) builds this class; behind the plugin the reference's own MHAKVCache object is used and
its `store_kv` is what gets rebound.
"""
from __future__ import annotations

import torch

from . import ops


def heads_per_rank(total: int, ranks: int, replicate: bool = False) -> int:
    """How many of `total` heads (or MLP columns) one of `ranks` tensor-parallel ranks owns.  With replicate=True a
    group larger than the head count keeps one head per rank, shared by ranks // total neighbours (KV heads at
    tp > Hkv).  Same arithmetic as the reference's sharding helper (P/utils/misc.py:20-26)."""
    if replicate and ranks > total:
        if ranks % total:
            raise ValueError(f"cannot replicate {total} heads over {ranks} ranks (not a multiple)")
        return 1
    if total % ranks:
        raise ValueError(f"cannot split {total} evenly over {ranks} ranks")
    return total // ranks


class MHAKVCache:
    def __init__(self, num_kv_heads: int, num_layers: int, head_dim: int, num_pages: int, page_size: int,
                 dtype: torch.dtype, device: torch.device, tp_size: int = 1) -> None:
        heads = heads_per_rank(num_kv_heads, tp_size, replicate=True)
        slots = num_pages * page_size
        self.pool = torch.empty((2, num_layers, num_pages, page_size, heads, head_dim), device=device, dtype=dtype)
        self._layers = num_layers
        self._tok_shape = (slots, heads, head_dim)   # [slot, head, dim] view of one layer
        self._row_shape = (slots, heads * head_dim)  # [slot, row] view of one layer

    # the reference's accessors ([num_pages, page_size, heads, dim] per layer)
    def k_cache(self, index: int) -> torch.Tensor:
        return self.pool[0, index]

    def v_cache(self, index: int) -> torch.Tensor:
        return self.pool[1, index]

    # token-row views used by the kernels
    def k_rows(self, index: int) -> torch.Tensor:
        return self.pool[0, index].view(self._row_shape)

    def v_rows(self, index: int) -> torch.Tensor:
        return self.pool[1, index].view(self._row_shape)

    def k_tokens(self, index: int) -> torch.Tensor:
        return self.pool[0, index].view(self._tok_shape)

    def v_tokens(self, index: int) -> torch.Tensor:
        return self.pool[1, index].view(self._tok_shape)

    def store_kv(self, k: torch.Tensor, v: torch.Tensor, out_loc: torch.Tensor, layer_id: int) -> None:
        ops.store_kv(self.k_rows(layer_id), self.v_rows(layer_id), out_loc,
                     k.view(k.shape[0], -1), v.view(v.shape[0], -1))

    @property
    def device(self) -> torch.device:
        return self.pool.device

    @property
    def dtype(self) -> torch.dtype:
        return self.pool.dtype

    @property
    def num_layers(self) -> int:
        return self._layers


def create_kvcache_pool(model_config, num_pages: int, page_size: int, dtype: torch.dtype, device: torch.device,
                        tp_size: int = 1, state_rows: int = 0):
    """P/kvcache/__init__.py:27-44; a configuration that lists its layers one by one (`layers` of specs) gets the per-layer
    HybridCache with `state_rows` recurrent-state slots."""
    if hasattr(model_config, "layers"):
        # a configuration with a repeated run of layers lists one spec per layer RUN (`cache_layers`): every pass has its own rows
        return HybridCache(getattr(model_config, "cache_layers", model_config.layers), num_pages, page_size, state_rows, dtype, device,
                           shift_width=model_config.hidden_size if getattr(model_config, "token_shift", False) else 0,
                           prev_token=getattr(model_config, "pair_embed", None) is not None,
                           conv_in=(getattr(model_config, "conv_taps", 0), model_config.hidden_size))
    return MHAKVCache(num_kv_heads=model_config.num_kv_heads, num_pages=num_pages, page_size=page_size,
                      num_layers=model_config.num_layers, head_dim=model_config.head_dim, device=device,
                      dtype=dtype, tp_size=tp_size)


class HybridCache:
    """Per-layer memory of a model that mixes latent-attention layers with linear-recurrence layers.

    * a latent-attention layer that owns its keys caches ONE row per token, shared by all heads: `latent_rows(layer)` is
      `[num_pages * page_size, kv_rank + rot_dim]` in the model dtype, indexed by the same token slots of the global page
      table as the MHA pool (the extra last page is the dummy target of padded rows); a layer that borrows another layer's
      keys has no rows of its own and is handed the owner's;
    * a linear-recurrence layer keeps one fp32 state `[heads, dim, vdim]` per running request: `state(layer)` is
      `[state_rows, heads, dim, vdim]`, indexed by the request's page-table row, so a row that is handed to a new request
      brings its state slot with it (the kernel starts a request whose first token is at position 0 from zero).
    * a key/value attention layer (`attention`) caches per token its keys `[kv_heads * dim]` and its (blended) values
      `[kv_heads * vdim]` in the model dtype: `kv_rows(layer)` = two tensors indexed by the same token slots;
    * a delta-rule layer (`delta`, `channel_delta`) keeps the fp32 state `[heads, dim, vdim]` like a lightning layer and,
      beside it, the last `conv - 1` inputs of its short convolution: `conv_state(layer)` is `[state_rows, conv - 1,
      channels]` in the model dtype, channels = 2 * kv_heads * dim + heads * vdim, same row index.
    * a `parallel` layer (sigmoid attention beside a state-space layer) has both: `kv_rows(layer)` for the attention's keys and
      values, `state(layer)` = fp32 `[state_rows, heads, state, vdim]` and `conv_state(layer)` = `[state_rows, conv - 1, heads *
      vdim + 2 * groups * state]` for the state-space layer;
    * a model whose mixers read a blend of a token's normed row and the previous token's (`shift_width` > 0) keeps, per layer and
      request, the last normed row in fp32: `shift_state(layer)` is `[state_rows, width]` (all layers: `shift_states`);
    * a model whose embedding depends on the previous token (`prev_token`) keeps each request's last token id: `prev_token`,
      int32 `[state_rows]`.
    * a windowed attention layer with a sink (`sink_attention`) caches keys and (normed) values like `attention`: every token stays
      cached, the window is applied when reading;
    * a selective-scan layer (`mamba1`) keeps the fp32 state `[state_rows, inner, state]` and the last `conv - 1` inputs of its
      convolution, `conv_state(layer)` = `[state_rows, conv - 1, inner]` in the model dtype;
    * a model with a causal convolution of `taps` in front of every sublayer (`conv_in` = (taps, width)) keeps, per layer, sublayer and
      request, the last `taps - 1` normed rows in fp32: `conv_in_state(layer, sub)` is `[state_rows, taps - 1, width]` (all of them:
      `conv_in_states`, `[layers, 2, state_rows, taps - 1, width]`).
    Layers may differ in every size, so each gets its own allocation.  Every per-request row is indexed by the request's
    page-table row and needs no clearing: a request whose first token is at position 0 never reads what the row held.
    """

    def __init__(self, layers, num_pages: int, page_size: int, state_rows: int, dtype: torch.dtype, device: torch.device,
                 shift_width: int = 0, prev_token: bool = False, conv_in=(0, 0)) -> None:
        self._latent, self._state, self._owner, self._kv, self._conv = {}, {}, {}, {}, {}
        slots = num_pages * page_size
        taps_in, width_in = conv_in
        self.conv_in_states = torch.zeros((len(layers), 2, state_rows, taps_in - 1, width_in), dtype=torch.float32, device=device) \
            if taps_in > 1 else None
        self.shift_states = torch.zeros((len(layers), state_rows, shift_width), dtype=torch.float32, device=device) if shift_width else None
        self.prev_token = torch.zeros((state_rows,), dtype=torch.int32, device=device) if prev_token else None
        for i, spec in enumerate(layers):
            if spec.kind == "parallel":
                a, b = spec.left, spec.right
                self._kv[i] = (torch.zeros((slots, a.kv_heads * a.dim), dtype=dtype, device=device),
                               torch.zeros((slots, a.kv_heads * a.vdim), dtype=dtype, device=device))
                self._state[i] = torch.zeros((state_rows, b.heads, b.dim, b.vdim), dtype=torch.float32, device=device)
                if b.conv > 1:
                    self._conv[i] = torch.zeros((state_rows, b.conv - 1, b.heads * b.vdim + 2 * b.kv_heads * b.dim), dtype=dtype, device=device)
            elif spec.kind == "latent_attention":
                if spec.kv_from is None:
                    self._latent[i] = torch.zeros((slots, spec.kv_rank + spec.rot_dim), dtype=dtype, device=device)
                self._owner[i] = i if spec.kv_from is None else spec.kv_from
            elif spec.kind == "lightning":
                self._state[i] = torch.zeros((state_rows, spec.heads, spec.dim, spec.vdim), dtype=torch.float32, device=device)
            elif spec.kind in ("attention", "sink_attention"):
                self._kv[i] = (torch.zeros((slots, spec.kv_heads * spec.dim), dtype=dtype, device=device),
                               torch.zeros((slots, spec.kv_heads * spec.vdim), dtype=dtype, device=device))
            elif spec.kind == "mamba1":
                self._state[i] = torch.zeros((state_rows, spec.vdim, spec.dim), dtype=torch.float32, device=device)
                if spec.conv > 1:
                    self._conv[i] = torch.zeros((state_rows, spec.conv - 1, spec.vdim), dtype=dtype, device=device)
            elif spec.kind in ("delta", "channel_delta"):
                self._state[i] = torch.zeros((state_rows, spec.heads, spec.dim, spec.vdim), dtype=torch.float32, device=device)
                if spec.conv > 1:
                    channels = 2 * spec.kv_heads * spec.dim + spec.heads * spec.vdim
                    self._conv[i] = torch.zeros((state_rows, spec.conv - 1, channels), dtype=dtype, device=device)
            else:
                raise ValueError(f"layer {i}: no cache layout for mixer {spec.kind!r}")
        for i, j in self._owner.items():
            if j not in self._latent:
                raise ValueError(f"layer {i} borrows the keys of layer {j}, which caches none")
        self._dtype, self._device, self._layers = dtype, device, len(layers)

    def latent_rows(self, layer: int) -> torch.Tensor:
        return self._latent[self._owner[layer]]

    def owns_latent(self, layer: int) -> bool:
        return layer in self._latent

    def state(self, layer: int) -> torch.Tensor:
        return self._state[layer]

    def kv_rows(self, layer: int):
        """(keys [slots, kv_heads * dim], values [slots, kv_heads * vdim]) of a key/value attention layer."""
        return self._kv[layer]

    def conv_state(self, layer: int):
        """[state_rows, conv - 1, channels] of a delta-rule or state-space layer, or None when its convolution has one tap."""
        return self._conv.get(layer)

    def conv_in_state(self, layer: int, sub: int) -> torch.Tensor:
        """fp32 [state_rows, taps - 1, width]: every request's last normed rows in front of sublayer `sub` (0 mixer, 1 feed-forward)."""
        return self.conv_in_states[layer, sub]

    def shift_state(self, layer: int) -> torch.Tensor:
        """fp32 [state_rows, width]: every request's last normed row of this layer."""
        return self.shift_states[layer]

    @staticmethod
    def bytes_per_page(layers, page_size: int, dtype: torch.dtype) -> int:
        es = torch.empty((), dtype=dtype).element_size()
        per_token = sum(s.kv_rank + s.rot_dim for s in layers if s.kind == "latent_attention" and s.kv_from is None)
        per_token += sum(s.kv_heads * (s.dim + s.vdim) for s in layers if s.kind in ("attention", "sink_attention"))
        per_token += sum(s.left.kv_heads * (s.left.dim + s.left.vdim) for s in layers if s.kind == "parallel")
        return per_token * es * page_size

    @staticmethod
    def state_bytes(layers, state_rows: int, dtype: torch.dtype = torch.bfloat16, shift_width: int = 0, conv_in=(0, 0)) -> int:
        es = torch.empty((), dtype=dtype).element_size()
        taps_in, width_in = conv_in
        total = sum(4 * s.heads * s.dim * s.vdim * state_rows for s in layers if s.kind in ("lightning", "delta", "channel_delta"))
        total += sum(es * (s.conv - 1) * (2 * s.kv_heads * s.dim + s.heads * s.vdim) * state_rows
                     for s in layers if s.kind in ("delta", "channel_delta"))
        for s in (x.right for x in layers if x.kind == "parallel"):
            total += (4 * s.heads * s.dim * s.vdim + es * (s.conv - 1) * (s.heads * s.vdim + 2 * s.kv_heads * s.dim)) * state_rows
        total += sum((4 * s.vdim * s.dim + es * (s.conv - 1) * s.vdim) * state_rows for s in layers if s.kind == "mamba1")
        total += 4 * 2 * max(taps_in - 1, 0) * width_in * len(layers) * state_rows
        return total + 4 * shift_width * len(layers) * state_rows

    @property
    def device(self) -> torch.device:
        return self._device

    @property
    def dtype(self) -> torch.dtype:
        return self._dtype

    @property
    def num_layers(self) -> int:
        return self._layers

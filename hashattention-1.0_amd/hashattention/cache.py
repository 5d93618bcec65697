"""A KV cache for `transformers` models that appends in place.

The reference's patched layer calls `past_key_value.update(...)` and attends over what it returns
(hashattention/hashattention_llama.py:573-576).  With the library's `DynamicCache` that call is
`torch.cat([self.keys, key_states], dim=-2)`: every decode step copies the whole cache of the layer - at 131072 cached
tokens and batch 4, 2 x 1.07 GB per layer per token in front of a sparse attention step that reads 40 MB.
`PreallocatedCache` is a `DynamicCache` whose layers keep capacity ahead of their length and copy only the new tokens;
`update` returns `[:, :, :length]` views of the buffers, which the kernels of this package read through their strides.
Everything else (`get_seq_length`, mask sizes, `crop`, beam reordering, offloading) behaves as for `DynamicCache`.

    cache = PreallocatedCache(capacity=prompt_len + max_new_tokens)
    out = model.generate(**inputs, past_key_values=cache, max_new_tokens=...)

A caller who passes a plain `DynamicCache` (or none, so that `generate` makes one) needs to do nothing: the converted
attention modules turn their layer of it into a `PreallocatedLayer` in place at the first decode step (`adopt_dynamic_layer`).

`StaticCache` works with the patched layers as well (they take the number of valid tokens from the cache, not from the
shape of the returned tensors), at the price of one device-to-host read of its length per layer and step.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from transformers.cache_utils import Cache, DynamicCache, DynamicLayer


class PreallocatedLayer(DynamicLayer):
    """`DynamicLayer` over buffers [batch, kv_heads, capacity, head_dim] that grow geometrically; `keys` / `values` are
    views of the first `length` tokens.  Assigning to `keys` / `values` (cropping, batch selection, offloading - whatever
    the base classes do by assignment) adopts the assigned tensor as the new buffer."""

    default_capacity = 0
    growth = 2.0
    min_growth = 0
    max_growth = None   # most tokens of room added at a time (None: no bound, the geometric growth alone)

    def __init__(self, capacity: Optional[int] = None, **kwargs):
        self._kbuf = self._vbuf = None
        self._len = 0
        self.epoch = 0
        super().__init__()
        self.epoch = 0      # counts assignments to `keys` from here on: contents replaced from outside (beam reordering, batch selection)
        self.capacity_hint = int(self.default_capacity if capacity is None else capacity)

    # -- keys / values as views of the buffers
    @property
    def keys(self):
        return None if self._kbuf is None else self._kbuf[:, :, :self._len]

    @keys.setter
    def keys(self, t):
        self.epoch += 1
        self._kbuf = t
        self._len = 0 if t is None or t.dim() < 3 else int(t.shape[-2])
        if t is not None and t.dim() < 3:
            self._kbuf = None

    @property
    def values(self):
        return None if self._vbuf is None else self._vbuf[:, :, :self._len]

    @values.setter
    def values(self, t):
        self._vbuf = None if t is None or t.dim() < 3 else t

    def lazy_initialization(self, key_states: torch.Tensor, value_states: torch.Tensor) -> None:
        self.dtype, self.device = key_states.dtype, key_states.device
        self.is_initialized = True

    def _reserve(self, key_states: torch.Tensor, value_states: torch.Tensor, need: int) -> None:
        have = 0 if self._kbuf is None else self._kbuf.shape[-2]
        if self._kbuf is not None and self._vbuf is not None and need <= have and self._kbuf.device == key_states.device:
            return
        grown = int(have * self.growth)
        if self.max_growth is not None:
            grown = min(grown, have + self.max_growth)
        cap = max(need, self.capacity_hint, grown, have + self.min_growth if have else 0)
        b, h, _, dk = key_states.shape
        kbuf = torch.empty(b, h, cap, dk, dtype=key_states.dtype, device=key_states.device)
        vbuf = torch.empty(b, h, cap, value_states.shape[-1], dtype=value_states.dtype, device=value_states.device)
        if self._len:
            kbuf[:, :, :self._len].copy_(self._kbuf[:, :, :self._len])
            vbuf[:, :, :self._len].copy_(self._vbuf[:, :, :self._len])
        self._kbuf, self._vbuf = kbuf, vbuf

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, *args, **kwargs) -> Tuple[torch.Tensor, torch.Tensor]:
        if not self.is_initialized:
            self.lazy_initialization(key_states, value_states)
        t = key_states.shape[-2]
        n = self._len
        self._reserve(key_states, value_states, n + t)
        self._kbuf[:, :, n:n + t].copy_(key_states)
        self._vbuf[:, :, n:n + t].copy_(value_states)
        self._len = n + t
        return self._kbuf[:, :, :self._len], self._vbuf[:, :, :self._len]

    def append_slots(self, like: torch.Tensor, batch: int, heads: int, head_dim: int, t: int = 1):
        """Room for `t` more tokens that a kernel writes itself: returns (key buffer, value buffer, position of the first new
        token) with the buffers [batch, heads, capacity, head_dim] of `like`'s dtype and device, and counts the tokens as
        cached.  The caller fills positions [pos, pos + t) of both buffers on the current stream."""
        if not self.is_initialized:
            self.dtype, self.device = like.dtype, like.device
            self.is_initialized = True
        n = self._len
        have = 0 if self._kbuf is None else self._kbuf.shape[-2]
        if self._kbuf is None or n + t > have or self._kbuf.device != like.device:
            shape = torch.empty(batch, heads, 0, head_dim, dtype=like.dtype, device=like.device)
            self._reserve(shape, shape, n + t)
        self._len = n + t
        return self._kbuf, self._vbuf, n

    def get_seq_length(self) -> int:
        return self._len if self._kbuf is not None else 0

    def crop(self, tokens_to_remove: int) -> None:
        """Forget the last `tokens_to_remove` tokens (a negative count, as the base class takes it; a positive value is the
        length to keep, the base class's legacy meaning).  The buffers stay."""
        if tokens_to_remove > 0:
            self._len = min(self._len, tokens_to_remove)
        else:
            self._len = max(self._len + tokens_to_remove, 0)

    def reset(self) -> None:
        self._len = 0

    @property
    def capacity(self) -> int:
        return 0 if self._kbuf is None else int(self._kbuf.shape[-2])


def adopt_dynamic_layer(layer) -> bool:
    """Turn a plain `DynamicLayer` that already holds tokens into a `PreallocatedLayer` IN PLACE: same object, same tensors
    (they become its buffers, full to the brim, so the next append allocates a larger buffer once), same behaviour
    towards the cache that owns it - but later appends copy only the new tokens.  This is how a cache that `generate` created
    on its own (`DynamicCache`, one `torch.cat` of the layer's whole cache per token) is taken over by the converted attention
    modules.  Only the exact class is taken: sliding-window, quantized or static layers keep their own logic.  Returns
    whether the layer is a `PreallocatedLayer` afterwards."""
    if isinstance(layer, PreallocatedLayer):
        return True
    if type(layer) is not DynamicLayer or not getattr(layer, "is_initialized", False):
        return False
    k, v = layer.__dict__.get("keys"), layer.__dict__.get("values")
    if not isinstance(k, torch.Tensor) or not isinstance(v, torch.Tensor) or k.dim() != 4 or v.dim() != 4 or k.shape[-2] == 0:
        return False
    del layer.__dict__["keys"], layer.__dict__["values"]       # the names are properties of the new class
    layer.__class__ = PreallocatedLayer
    layer._kbuf, layer._vbuf, layer._len = k, v, int(k.shape[-2])
    layer.capacity_hint = 0
    # nobody said how long this cache will get: a quarter more room at a time, 256 to 8192 tokens - a prompt of 131072 tokens must
    # not reserve 32768 more per layer for an answer of a few hundred, and copying the layer once per 8192 appended tokens costs
    # nothing that shows
    layer.growth, layer.min_growth, layer.max_growth = 1.25, 256, 8192
    layer.epoch = 0
    return True


class PreallocatedCache(DynamicCache):
    """`DynamicCache` of `PreallocatedLayer`s.  `capacity`: tokens to reserve per layer at its first update (prompt plus the
    tokens to generate, if known); a layer that outgrows it doubles."""

    def __init__(self, capacity: int = 0, num_layers: Optional[int] = None):
        layer_cls = type("PreallocatedLayer", (PreallocatedLayer,), {"default_capacity": int(capacity)})
        if num_layers is None:
            Cache.__init__(self, layer_class_to_replicate=layer_cls)
        else:
            Cache.__init__(self, layers=[layer_cls() for _ in range(num_layers)])
        self.capacity = int(capacity)

"""Model-side half of the drop-in: the hash module `USA` and the logic shared by the patched Llama and
Mistral attention layers.  Mirrors the reference's module API
(hashattention/hashattention_llama.py:87-226 `USA`, :229-631 `LlamaAttention_heavy_hitter`, :633-725 helpers)
with the decode branch running on the HIP kernels through `decode.HashDecodeLayer`.

What differs from the reference on purpose
  * the decode branch never builds dense [b, H, q, S] score/mask tensors and never re-hashes cached keys:
    key codes live in a per-layer bit-cache that is extended as the KV cache grows (the reference keeps
    `past_key_signatures = None`, hashattention_llama.py:407-408);
  * ties at the top-k boundary go to the lowest token index (the reference's `sort` at :430 is unstable);
  * softmax and the value product are fp32 throughout (the reference rounds probabilities to the query
    dtype at :613);
  * the LSH baseline (`lth_num_layers == 0`, :75-84, :130-139) and `CENTER` normalisation (:163-167) hash inputs that
    depend on a statistic over ALL cached keys (their largest norm; their mean and deviation), so a key's code changes
    as the cache grows: in these two modes the bit-cache is rebuilt at every step, as the reference re-hashes every
    step, and only selection and attention keep their speed;
  * the training side - soft mode (`hard=False`: tanh / sigmoid, :174-176, 197-198), `train_step` (:304-316) and the train
    branch of `usa_local_compute` (:356-371) - is differentiable torch code batched over heads (one baddbmm per MLP layer
    instead of a Python loop over heads); the recall statistic (:372-398) runs on the selection kernel.
"""
from __future__ import annotations

import math
import os
import weakref
from typing import List, Optional, Tuple

import torch
from torch import nn

from . import _ops
from .cache import PreallocatedLayer, adopt_dynamic_layer
from .decode import HashDecodeLayer

DECODE_MAX_Q_LEN = 128   # reference: `if q_len > 128 or self.train_usa` routes to the original forward (:529)
DEFAULT_USA_CFG = {"lth_int_dim": 128, "lth_final_dim": 32, "lth_thold": 0}     # reference :68-72


def memory_efficient_softmax(x: torch.Tensor, dim: int) -> torch.Tensor:
    """Max-subtracted softmax in the input's dtype (reference :37-44; its `use_softmax_maxtrick` switch).  The kernels of
    this build always subtract the running maximum; the function is kept for callers of the module API."""
    e = torch.exp(x - x.amax(dim=dim, keepdim=True))
    return e / e.sum(dim=dim, keepdim=True)


class SignSTE(torch.autograd.Function):
    """sign(x) whose gradient is that of tanh(x) (reference :51-63)."""

    @staticmethod
    def forward(ctx, x):
        ctx.save_for_backward(x)
        return torch.sign(x)

    @staticmethod
    def backward(ctx, grad_output):
        (x,) = ctx.saved_tensors
        return grad_output * (1 - torch.tanh(x).square())


def ste_sign(x: torch.Tensor) -> torch.Tensor:
    return SignSTE.apply(x)


# last attention mask examined, as ONE tuple so that a reader never sees parts of two examinations: (weak reference,
# (version, length, batch, rows), the `_StepMask` it became or None when it changes nothing)
_MASK_PROBE = [(None, None, None)]
_FUSED_ROWS = 8


class _StepMask:
    """The additive attention mask of one forward pass in the forms the kernels take; one object serves all layers of the
    pass.  `prefix`: int32 [b] on the device when the mask of a single-token step blocks exactly the first prefix[b] tokens of
    every sequence and nothing else (a left-padded batch) - the fused launch takes that; else None.  `rows()`: fp32
    [b, q, S]; `table()`: fp32 [b, S] of a single-token step."""
    __slots__ = ("_m", "b", "q_len", "S", "prefix", "_rows")

    def __init__(self, m, b, q_len, S, prefix):
        self._m, self.b, self.q_len, self.S, self.prefix, self._rows = m, b, q_len, S, prefix, None

    def rows(self) -> torch.Tensor:
        if self._rows is None:
            m = self._m
            if m.dtype == torch.bool:
                m = torch.zeros(m.shape, dtype=torch.float32, device=m.device).masked_fill_(torch.logical_not(m), float("-inf"))
            self._rows = m.float().expand(self.b, self.q_len, self.S).contiguous()
            self._m = None
        return self._rows

    def table(self) -> torch.Tensor:
        return self.rows()[:, 0]

LSH_PAD = 3     # zero coordinates after the lifted one: the encode kernels take input widths that are multiples of 4


def lift_to_sphere(x: torch.Tensor, pad: int = 0) -> torch.Tensor:
    """[b, heads, s, d] -> [b, heads, s, d + 1 + pad]: the coordinate sqrt(M^2 - |x|^2) that gives every vector of a head
    the same length M = (largest norm in that head) + 1e-3, so that sign random projections rank by inner product;
    `pad` zeros follow.  Arithmetic as the reference's `IpToCS` (:75-84) per head: the norm in the input's dtype, M^2 in
    double rounded to fp32, the difference rounded to the input's dtype before relu and sqrt."""
    norm = torch.linalg.vector_norm(x, dim=-1, keepdim=True)
    big = norm.amax(dim=(0, 2), keepdim=True).double() + 1e-3
    gap = ((big * big).float() - norm.square().float()).to(x.dtype)
    parts = [x, torch.sqrt(torch.relu(gap))]
    if pad:
        parts.append(x.new_zeros(*x.shape[:-1], pad))
    return torch.cat(parts, dim=-1)


class IpToCS(nn.Module):
    """First stage of an LSH-baseline head (reference :75-84): x [..., s, d] of ONE head -> [..., s, d + 1]."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        flat = x.reshape(1, 1, -1, x.shape[-1])
        return lift_to_sphere(flat).reshape(*x.shape[:-1], x.shape[-1] + 1)


class USA(nn.Module):
    """Per-head learned hash: `num_heads` independent MLPs for keys and for queries.

    Same constructor, parameter names and state-dict keys as the reference
    ("learning_to_hash_transformation_{k,q}.{head}.{0,2,4}.{weight,bias}", hashattention_llama.py:99-128),
    so reference checkpoints load unchanged.
    """

    def __init__(self, num_heads: int, head_dim: int, usa_params: dict = DEFAULT_USA_CFG):
        super().__init__()
        self.head_dim = head_dim
        self.num_heads = num_heads
        self.int_dim = usa_params["lth_int_dim"]
        self.lth_final_dim = usa_params["lth_final_dim"]
        self.lth_thold = usa_params["lth_thold"]
        self.num_layers = usa_params.get("lth_num_layers", 3)   # the Mistral variant has no such key (mistral:566-570)
        if self.num_layers not in (0, 1, 2, 3):
            raise NotImplementedError("lth_num_layers must be 0 (LSH baseline), 1, 2 or 3")
        if self.lth_final_dim not in (32, 64):
            raise NotImplementedError("lth_final_dim must be 32 or 64: codes are packed in one or two 32-bit words")
        self.center = bool(os.environ.get("CENTER", 0))      # as the reference reads it (:34, :98): any non-empty value is on

        def mlp():
            if self.num_layers == 3:
                return nn.Sequential(nn.Linear(head_dim, self.int_dim), nn.SiLU(), nn.Linear(self.int_dim, self.int_dim),
                                     nn.SiLU(), nn.Linear(self.int_dim, self.lth_final_dim))
            if self.num_layers == 2:
                return nn.Sequential(nn.Linear(head_dim, self.int_dim), nn.SiLU(), nn.Linear(self.int_dim, self.lth_final_dim))
            return nn.Sequential(nn.Linear(head_dim, self.lth_final_dim))

        if self.num_layers == 0:
            # LSH baseline (:130-139): one random projection of the lifted vector per head, shared by keys and queries
            # (the same modules under three names, so a state dict holds each tensor under all three prefixes)
            print("Implementing LSH for baseline")
            self.learning_to_hash_transformation = nn.ModuleList(
                [nn.Sequential(IpToCS(), nn.Linear(head_dim + 1, self.lth_final_dim)) for _ in range(num_heads)])
            for seq in self.learning_to_hash_transformation:
                nn.init.normal_(seq[1].weight)
            self.learning_to_hash_transformation_k = self.learning_to_hash_transformation
            self.learning_to_hash_transformation_q = self.learning_to_hash_transformation
            return
        self.learning_to_hash_transformation_k = nn.ModuleList([mlp() for _ in range(num_heads)])
        self.learning_to_hash_transformation_q = nn.ModuleList([mlp() for _ in range(num_heads)])

    # -- weights in the form the kernels take
    def layers(self, side: str) -> List[List[Tuple[torch.Tensor, torch.Tensor]]]:
        mods = self.learning_to_hash_transformation_k if side == "k" else self.learning_to_hash_transformation_q
        return [[(m.weight, m.bias) for m in seq if isinstance(m, nn.Linear)] for seq in mods]

    @property
    def kernel_num_layers(self) -> int:
        """Linear layers per head as the encode kernels count them (the LSH baseline is one layer on the lifted input)."""
        return max(1, self.num_layers)

    def kernel_layers(self, side: str) -> List[List[Tuple[torch.Tensor, torch.Tensor]]]:
        """`layers(side)` in the shape the kernels take: the LSH projection gets zero columns for the padding
        coordinates of `hash_inputs`."""
        heads = self.layers(side)
        if self.num_layers != 0:
            return heads
        return [[(torch.nn.functional.pad(w, (0, LSH_PAD)), b) for (w, b) in h] for h in heads]

    @property
    def rehash_every_step(self) -> bool:
        """True when a key's code depends on the other cached keys (LSH lift, CENTER statistics): no code can be kept."""
        return self.center or self.num_layers == 0

    def hash_inputs(self, K: torch.Tensor, Q: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """What the encode kernels are fed in hard mode for keys K [b, Hx, S, d] (Hx = KV heads or query heads) and
        queries Q [b, H, t, d]: unchanged for the learned hashes; with CENTER, both standardised per head with the mean
        and deviation of that head's keys over batch and positions (:163-167); for the LSH baseline, both lifted
        (`lift_to_sphere`, each with its own largest norm) and zero-padded to a width the kernels take."""
        if self.center:
            rep = Q.shape[1] // K.shape[1]
            mean, std = K.mean(dim=(0, 2), keepdim=True), K.std(dim=(0, 2), keepdim=True)
            K = (K - mean) / (std + 1e-6)
            Q = (Q - mean.repeat_interleave(rep, dim=1)) / (std.repeat_interleave(rep, dim=1) + 1e-6)
        if self.num_layers == 0:
            K, Q = lift_to_sphere(K, LSH_PAD), lift_to_sphere(Q, LSH_PAD)
        return K, Q

    @property
    def dtype(self) -> torch.dtype:
        return self.learning_to_hash_transformation_k[0][-1].weight.dtype

    @property
    def arith(self) -> int:
        """A module kept in bf16 computes with bf16 roundings after every layer; anything else in fp32."""
        return _ops.HA_ARITH_BF16 if self.dtype == torch.bfloat16 else _ops.HA_ARITH_F32

    def _stacked(self, side: str) -> List[Tuple[torch.Tensor, torch.Tensor]]:
        """Per layer (W [heads, out, in], b [heads, out]) stacked from the per-head modules; gradients reach the modules."""
        heads = self.layers(side)
        return [(torch.stack([h[l][0] for h in heads]), torch.stack([h[l][1] for h in heads])) for l in range(len(heads[0]))]

    def _soft_logits(self, vectors: torch.Tensor, side: str) -> torch.Tensor:
        """[b, heads, s, d] -> MLP outputs [b, heads, s, D], all heads in one baddbmm per layer (differentiable)."""
        b, a, s, d = vectors.shape
        if a != self.num_heads:
            raise ValueError(f"expected {self.num_heads} heads, got {a}")
        if self.num_layers == 0:
            vectors = lift_to_sphere(vectors)
        x = vectors.transpose(0, 1).reshape(a, b * s, -1)
        stacked = self._stacked(side)
        for l, (w, bias) in enumerate(stacked):
            x = torch.baddbmm(bias.unsqueeze(1), x, w.transpose(1, 2))
            if l + 1 < len(stacked):
                x = torch.nn.functional.silu(x)
        return x.view(a, b, s, -1).transpose(0, 1)

    def _embed(self, vectors: torch.Tensor, side: str, hard: bool, prepared: bool = False):
        """hard: (signs of the logits, packed codes) from the encode kernel; soft: (tanh of the logits, None).
        `prepared`: the vectors already went through `hash_inputs`."""
        if not hard:
            return torch.tanh(self._soft_logits(vectors.to(self.dtype), side)), None
        if self.num_layers == 0 and not prepared:
            vectors = lift_to_sphere(vectors, LSH_PAD)
        b, a, s, d = vectors.shape
        if a != self.num_heads:
            raise ValueError(f"expected {self.num_heads} heads, got {a}")
        w = self._packed_weights(side, vectors.device)
        codes = torch.empty(b, a, s, self.lth_final_dim // 32, dtype=torch.int32, device=vectors.device)
        logits = _ops.encode_pack(vectors, w, self.kernel_num_layers, self.int_dim, self.lth_final_dim, codes,
                                  arith=self.arith, want_logits=True)
        return torch.sign(logits), codes

    def invalidate_packed(self) -> None:
        """Forget the packed copies of the weights.  They are rebuilt whenever a parameter's version counter or storage
        changes; an update that bypasses the counter (`p.data.add_(...)`, an EMA or optimizer writing through `.data`) must
        be followed by this call.  Loading a state dict, `train()` / `eval()` and `train_step` call it themselves."""
        self.__dict__.pop("_packed", None)

    def train(self, mode: bool = True):
        self.invalidate_packed()
        return super().train(mode)

    def _load_from_state_dict(self, *args, **kwargs):
        self.invalidate_packed()
        return super()._load_from_state_dict(*args, **kwargs)

    def _packed_weights(self, side: str, device) -> torch.Tensor:
        """The side's weights in the kernels' blob form, repacked only when a parameter changed (tensor versions) or moved."""
        params = [t for head in self.layers(side) for wb in head for t in wb]
        key = (str(device),) + tuple((t.data_ptr(), t._version, t.dtype) for t in params)
        cache = self.__dict__.setdefault("_packed", {})
        hit = cache.get(side)
        if hit is None or hit[0] != key:
            hit = (key, _ops.pack_usa_weights(self.kernel_layers(side), device))
            cache[side] = hit
        return hit[1]

    def k_embedding(self, vectors: torch.Tensor, hard: bool = False) -> torch.Tensor:
        """[b, heads, s, d] -> embeddings [b, heads, s, D] in fp32: signs (hard) or tanh (soft) (reference :204-214)."""
        return self._embed(vectors, "k", hard)[0].float()

    def q_embedding(self, vectors: torch.Tensor, hard: bool = False) -> torch.Tensor:
        return self._embed(vectors, "q", hard)[0].float()

    def forward(self, K: torch.Tensor, Q: torch.Tensor, hard: bool = False):
        """hard: span[b, h, t, s] = <sign q_t, sign k_s> = D - 2 * Hamming, non-causal entries at finfo.min; soft (the
        default, differentiable): sigmoid(<tanh q_t, tanh k_s> - lth_thold), non-causal entries 0.  Returns
        (span, K embeddings) as the reference (:151-200).  The decode path does not call it."""
        b, a, s, _ = K.shape
        t = Q.shape[2]
        causal = torch.tril(torch.ones(t, s, device=K.device), diagonal=s - t).bool()
        if not hard:
            if self.center:     # per head: keys and queries standardised with the statistics of the keys (:163-167)
                mean = K.mean(dim=(0, 2), keepdim=True)
                std = K.std(dim=(0, 2), keepdim=True)
                K, Q = (K - mean) / (std + 1e-6), (Q - mean) / (std + 1e-6)
            kt, _ = self._embed(K, "k", False)
            qt, _ = self._embed(Q, "q", False)
            span = torch.matmul(qt, kt.transpose(2, 3))
            span = torch.where(causal, span, torch.full([], torch.finfo(span.dtype).min, dtype=span.dtype, device=K.device))
            return torch.sigmoid(span - self.lth_thold), kt
        Kh, Qh = self.hash_inputs(K, Q)
        ksign, kcodes = self._embed(Kh.contiguous(), "k", True, prepared=True)
        _, qcodes = self._embed(Qh.contiguous(), "q", True, prepared=True)
        D = self.lth_final_dim
        # the t query tokens of a head are t "query heads" of its code head: one scoring launch for all of them
        # (the launch takes up to 65535 of them: longer chunks go in slices of tokens)
        t_slice = max(1, 65535 // a)
        ham = torch.cat([_ops.hamming_score(kcodes, qcodes[:, :, t0:t0 + t_slice].reshape(b, -1, qcodes.shape[-1]), s)
                         .view(b, a, -1, s) for t0 in range(0, t, t_slice)], dim=2)
        span = (D - 2 * ham.to(torch.int32)).to(K.dtype)
        span = torch.where(causal, span, torch.full([], torch.finfo(span.dtype).min, dtype=span.dtype, device=K.device))
        return span, ksign.to(K.dtype)


class HeavyHitterMixin:
    """State and decode branch shared by `LlamaAttention_heavy_hitter` and `MistralAttention_heavy_hitter`.

    The host class provides q_proj/k_proj/v_proj/o_proj, `config`, `layer_idx`, `head_dim` and the rotary
    helper `_apply_rope(q, k, cos, sin)`.
    """

    def _init_heavy_hitter(self, config):
        self.num_heads = config.num_attention_heads
        self.num_key_value_heads = config.num_key_value_heads
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.hidden_size = config.hidden_size
        self.init_budget = config.init_budget
        self.heavy_budget = config.heavy_budget
        self.recent_budget = config.recent_budget
        self.usa_retrieve_depth = getattr(config, "usa_retrieve_depth", 0)
        self.usa_eval_mode = getattr(config, "usa_eval_mode", "simple")
        self.usa_module = None
        self.usa_module_dtype = None
        self.past_key_signatures = None      # kept for API parity; the bit-cache lives in self._hash_layer
        self.use_softmax_maxtrick = False
        self.collect_stats = False
        self.train_usa = False
        self.tr_loss_func = None
        self.tr_optimizer = None
        self.overlaps = {}
        self.last_train_loss = None
        self.print_offloading_flag = False
        # KV cache to host memory beyond this many tokens (reference :286, :495-511: 24000, sized for 80 GB parts).  Off by
        # default here: 288 GB of HBM hold the caches this path is built for; set a length to get the reference's policy.
        self.offloading_length = None
        self.flash_forward = None
        self._hash_layer: Optional[HashDecodeLayer] = None
        self._cache_ref = None       # weak reference to the KV cache object whose keys the bit-cache was made from
        self._cache_id = None
        # single-token steps of a bf16 model on a cache that appends in place (cache.PreallocatedCache) take `_fast_decode`:
        # five launches for the whole module instead of ~25 library calls; set False to keep every step on the general path
        self.adopt_cache = True     # a plain DynamicLayer of the caller's cache is turned into one that appends in place
        self.fast_decode = True
        self.fast_layer = True      # ... and the decoder layer around this module as well (`fast_decoder_layer_forward`)

    def __repr__(self):
        return (f"{super().__repr__()}\nSparsification Setting(topk:{self.heavy_budget}  edge:{self.init_budget, self.recent_budget} "
                f"\n eval_mode:{self.usa_eval_mode} stats:{self.collect_stats}\n Istraining:{self.train_usa} )")

    def _reset_state(self):
        """A new example starts (reference :298-301): drop the cached codes."""
        self.past_key_signatures = None
        self.print_offloading_flag = False
        self._cache_ref = self._cache_id = None
        if self._hash_layer is not None:
            self._hash_layer.reset()

    # ---- KV offload policy (reference :495-511), on the installed cache classes (`cache.layers[i].keys / .values`)
    def _cache_layer(self, cache):
        if cache is None or not hasattr(cache, "layers") or len(cache.layers) <= self.layer_idx:
            return None
        layer = cache.layers[self.layer_idx]
        return layer if getattr(layer, "keys", None) is not None else None

    def ensure_gpu(self, cache, device):
        layer = self._cache_layer(cache)
        if layer is not None and not layer.keys.is_cuda:
            known = self._holds_known_keys(cache)
            layer.keys, layer.values = layer.keys.to(device), layer.values.to(device)
            if known:
                self._note_key_storage(cache)       # moved by this layer itself: the same contents

    def offload_if_necessary_cpu(self, cache):
        layer = self._cache_layer(cache)
        if layer is None or self.offloading_length is None or layer.keys.shape[2] < self.offloading_length:
            return
        if not self.print_offloading_flag and self.layer_idx == 0:
            print("OFFLOADING ENABLED >>")
            self.print_offloading_flag = True
        layer.keys, layer.values = layer.keys.cpu(), layer.values.cpu()

    # ---- bit-cache plumbing
    def _cache_len(self, cache) -> int:
        """Tokens this layer already holds in `cache` (0 for no cache or a layer not yet written)."""
        if cache is None:
            return 0
        if hasattr(cache, "get_seq_length"):
            try:
                return int(cache.get_seq_length(self.layer_idx))
            except (IndexError, KeyError):
                return 0
        layer = self._cache_layer(cache)
        return 0 if layer is None else int(layer.keys.shape[-2])

    def _key_storage(self, cache):
        """What identifies the contents this layer's cache holds between two forward passes: the tensor object its layer
        keeps the keys in (`DynamicLayer` and `StaticLayer` replace that object whenever they reorder, select or repeat batch
        entries), or, for a `PreallocatedLayer`, the layer and its count of outside assignments (its buffer is also replaced
        when it grows, with the same contents)."""
        if cache is None or not hasattr(cache, "layers") or len(cache.layers) <= self.layer_idx:
            return None
        layer = cache.layers[self.layer_idx]
        if isinstance(layer, PreallocatedLayer):
            return ("preallocated", id(layer), layer.epoch)
        keys = getattr(layer, "keys", None)
        return keys if isinstance(keys, torch.Tensor) else None

    def _note_key_storage(self, cache) -> None:
        """Remember the key storage as this forward pass leaves it (`_holds_known_keys` at the next pass)."""
        held = self._key_storage(cache)
        self.__dict__["_keys_seen"] = weakref.ref(held) if isinstance(held, torch.Tensor) else held

    def _holds_known_keys(self, cache) -> bool:
        seen = self.__dict__.get("_keys_seen")
        if seen is None:
            return False
        now = self._key_storage(cache)
        return now is not None and ((seen() is now) if isinstance(seen, weakref.ref) else seen == now)

    def _sync_bit_cache(self, cache) -> None:
        """Keep the bit-cache in step with the KV cache before a forward pass appends to it.  The reference is stateless
        here (`past_key_signatures` stays None, :407-408, every key is re-hashed every step), so a caller may start a new
        prompt without `reset_usa`: codes are kept only while the SAME cache object still holds at least the tokens they
        were made from, in the storage this layer last saw.  Another cache object drops them all, and so does a cache whose
        batch entries were reordered, selected or repeated between two passes (beam search); a cache that was rewound
        keeps the codes of its prefix when its storage is still the same (`PreallocatedCache.crop`; the library's
        `DynamicCache.crop` leaves a new tensor behind and is hashed afresh)."""
        if cache is None:
            same = False
        elif self._cache_ref is not None:
            same = self._cache_ref() is cache
        else:
            same = self._cache_id is not None and self._cache_id == id(cache)
        if not same:
            self._cache_ref, self._cache_id = None, (id(cache) if cache is not None else None)
            try:
                self._cache_ref = weakref.ref(cache) if cache is not None else None
            except TypeError:           # a cache class without weak references: object identities are compared instead
                pass
        hl = self._hash_layer
        if hl is None:
            return
        if same and hl.n_cached > 0 and not self._holds_known_keys(cache):
            same = False        # same cache object, other contents: beam search reordered it, or rows were selected or repeated
        if not same:
            hl.reset()
        else:
            hl.n_cached = min(hl.n_cached, self._cache_len(cache))

    def _ensure_hash_layer(self, batch: int, seq_len: int, device) -> HashDecodeLayer:
        if self.usa_module is None:
            raise RuntimeError("convert_usa() must attach a USA module before the decode branch runs")
        hl = self._hash_layer
        if hl is None:
            usa = self.usa_module
            hl = HashDecodeLayer(usa.kernel_layers("k"), usa.kernel_layers("q"), self.num_heads, self.num_key_value_heads,
                                 self.head_dim, usa.kernel_num_layers, usa.int_dim, usa.lth_final_dim, self.init_budget, self.recent_budget,
                                 self.heavy_budget, self.usa_eval_mode, self.usa_retrieve_depth, usa.arith, device)
            self._hash_layer = hl
        if hl.B != batch or hl.S_cap < seq_len:
            keep = hl.codes[:, :, :hl.n_cached].clone() if (hl.B == batch and hl.n_cached > 0) else None
            n = hl.n_cached if keep is not None else 0
            hl.allocate(batch, max(2 * hl.S_cap if hl.B == batch else 0, seq_len + 1024))
            if keep is not None:
                hl.codes[:, :, :n] = keep
                hl.n_cached = n
        return hl

    def _hash_inputs(self, key_states, query_states):
        """The tensors the encode kernels read for these keys [b, Hkv, S, d] and queries [b, H, q, d]: the states
        themselves for a learned hash; their standardised / lifted form (`USA.hash_inputs`, computed in the hash
        module's dtype as the reference casts, :406) when codes depend on the whole cache."""
        usa = self.usa_module
        if usa is None or not usa.rehash_every_step:
            return key_states, query_states
        kh, qh = usa.hash_inputs(key_states.to(usa.dtype), query_states.to(usa.dtype))
        return kh.contiguous(), qh.contiguous()

    def _additive_mask(self, attention_mask, b: int, q_len: int, S: int):
        """The reference adds `attention_mask` [b, 1, q, S] to the scores before the keep-mask and the softmax (:593-598).
        Returns it as a `_StepMask`, or None when it changes nothing for any row's causal part (the kernels apply the
        causal structure themselves), which is the case for every unpadded batch.  A boolean mask (True = attend) is
        accepted as well.  Deciding costs one device-to-host read per forward pass, not per layer, and the fp32 form is
        made once per pass: the layers of a model are handed the same tensor object."""
        if attention_mask is None:
            return None
        if attention_mask.dim() != 4 or attention_mask.shape[1] != 1 or attention_mask.shape[2] != q_len \
                or attention_mask.shape[3] < S or attention_mask.shape[0] not in (1, b):
            raise ValueError(f"Attention mask should be of size {(b, 1, q_len, S)}, but is {tuple(attention_mask.size())}")
        key = (attention_mask._version, S, b, q_len)
        last = _MASK_PROBE[0]
        if last[0] is not None and last[0]() is attention_mask and last[1] == key:
            return last[2]
        m = attention_mask[:, 0, :, :S]
        if m.dtype != torch.bool and not m.is_floating_point():
            m = m.float()
        if m.dtype == torch.bool:
            blocked = torch.logical_not(m)
            hard = blocked
        else:
            blocked = m != 0
            hard = (m == torch.finfo(m.dtype).min) | (m == float("-inf"))      # what the library writes for "do not attend"
        if q_len == 1:
            # a left-padded batch: per sequence a prefix is blocked for good, nothing else
            row = blocked[:, 0]
            n = row.sum(-1)
            is_prefix = (row == (torch.arange(S, device=m.device)[None, :] < n[:, None])).all() & (hard[:, 0] == row).all()
            matters, is_prefix = torch.stack([row.any(), is_prefix]).tolist()
            prefix = n.to(torch.int32).expand(b).contiguous() if (matters and is_prefix) else None
        else:
            causal = torch.tril(torch.ones(q_len, S, dtype=torch.bool, device=m.device), diagonal=S - q_len)
            matters, prefix = bool((blocked & causal).any().item()), None
        step_mask = _StepMask(m, b, q_len, S, prefix) if matters else None
        _MASK_PROBE[0] = (weakref.ref(attention_mask), key, step_mask)
        return step_mask

    def _sparse_attention(self, query_states, key_states, value_states, attention_mask=None):
        """query [b, H, q, d] (q <= 128), key/value [b, Hkv, S, d] holding the whole cache including the new tokens.
        Returns [b, H, q, d].  Row i attends as query at absolute position S - q + i (reference :423-428)."""
        b, H, q_len, d = query_states.shape
        S = key_states.shape[2]
        amask = self._additive_mask(attention_mask, b, q_len, S)
        hl = self._ensure_hash_layer(b, S, query_states.device)
        key_hash, query_hash = self._hash_inputs(key_states, query_states)
        if hl.n_cached > S - q_len or self.usa_module.rehash_every_step:
            hl.reset()                       # the cache was rewound (new prompt without reset_usa), or no code can be kept
        if hl.n_cached < S - q_len:          # keys cached by a prefill (or by dense steps): encode them in bulk
            lo = hl.n_cached
            bulk = key_hash[:, :, lo:S - q_len]
            hl.encode_keys_bulk(bulk, pos0=lo)
            hl.n_cached = S - q_len
        out = torch.empty(b, H, q_len, d, dtype=query_states.dtype, device=query_states.device)
        # the reference takes the heavy budget from the full key length for every query row (:431-434)
        heavy = hl.heavy_count(S)
        heavy_abs = 0.0 if heavy == 0 else heavy + 0.5       # > 1: an absolute count for the kernels
        if q_len == 1:
            saved = hl.heavy_budget
            hl.heavy_budget = heavy_abs
            try:
                hl.step(query_states, key_states, value_states, S, out[:, :, 0],
                        hash_inputs=None if key_hash is key_states else (key_hash, query_hash),
                        attn_mask=amask)
            finally:
                hl.heavy_budget = saved
            return out
        # a chunk of q_len rows: the new keys join the bit-cache, then every row of every sequence is one batch entry of ONE
        # selection and ONE attention launch - the codes and K/V of its sequence, its own query code and its own length
        # S - q_len + i + 1 (reference :423-428)
        hl.encode_keys(key_hash[:, :, S - q_len:S], pos0=S - q_len)
        hl.n_cached = S
        return hl.chunk_step(query_states, key_states, value_states, S, out, heavy_abs,
                             q_hash=None if query_hash is query_states else query_hash,
                             attn_mask=None if amask is None else amask.rows())

    # ---- the single-token step as five launches
    def _fused_qkv_weight(self) -> torch.Tensor:
        """The q, k and v projection weights stacked as one [H d + 2 Hkv d, hidden] matrix (a copy, rebuilt when one of the
        three parameters was replaced or updated in place through its version counter; after a write through `.data`
        delete `self._qkv_fused`)."""
        ws = (self.q_proj.weight, self.k_proj.weight, self.v_proj.weight)
        key = tuple((w.data_ptr(), w._version, w.dtype, w.device) for w in ws)
        hit = self.__dict__.get("_qkv_fused")
        if hit is None or hit[0] != key:
            hit = (key, torch.cat([w.detach() for w in ws], dim=0).contiguous())
            self.__dict__["_qkv_fused"] = hit
        return hit[1]

    def _weight_tiles(self, name: str, weights, glu: bool = False) -> torch.Tensor:
        """The tiled copy (`ha_pack_weight_tiles`) of the given weights stacked row-wise, which `ha_linear_tiled` reads for
        batches of 9 to 32 sequences; kept under `name`, rebuilt like `_fused_qkv_weight`."""
        key = tuple((w.data_ptr(), w._version, w.dtype, w.device) for w in weights)
        hit = self.__dict__.get(name)
        if hit is None or hit[0] != key:
            stacked = weights[0].detach() if len(weights) == 1 else torch.cat([w.detach() for w in weights], dim=0)
            hit = (key, _ops.pack_weight_tiles(stacked, glu=glu))
            self.__dict__[name] = hit
        return hit[1]

    def _takes_tiled_projections(self, b: int, hidden: int) -> bool:
        return b > _FUSED_ROWS and _ops.linear_tiled_applies(b, max(hidden, self.num_heads * self.head_dim))

    def _fast_decode_slot(self, hidden_states, position_embeddings, attention_mask, cache):
        """(This layer's `PreallocatedLayer` of `cache`, the additive mask as a `_StepMask` or None when it changes nothing)
        when the step can take `_fast_decode`, else None: one new token per sequence, inference, bf16 hidden states and
        projections without biases, 128-wide heads, a learned hash whose codes can be cached, no KV offloading, and a cache
        whose layers append in place."""
        if not self.fast_decode or torch.is_grad_enabled() or self.train_usa or self.offloading_length is not None:
            return None
        b, q_len, hidden = hidden_states.shape
        if q_len != 1 or hidden % 32 or self.head_dim != 128 or hidden_states.dtype != torch.bfloat16 \
                or not hidden_states.is_contiguous() or position_embeddings is None:
            return None
        own = self._modules     # plain nn.Linear projections only: a wrapper around one (an adapter) has a forward of its own
        if any(type(own.get(n)) is not nn.Linear for n in ("q_proj", "k_proj", "v_proj", "o_proj")):
            return None
        if any(own[n].bias is not None for n in ("q_proj", "k_proj", "v_proj", "o_proj")) or self.q_proj.weight.dtype != torch.bfloat16:
            return None
        if self.q_proj.weight.device != hidden_states.device:       # a model spread over devices: its own hooks move the inputs
            return None
        usa = self.usa_module
        if usa is None or usa.rehash_every_step or getattr(cache, "offloading", False):
            return None
        layers = getattr(cache, "layers", None)
        if layers is None:
            return None
        if len(layers) <= self.layer_idx:
            make = getattr(cache, "layer_class_to_replicate", None)
            if make is None or not (isinstance(make, type) and issubclass(make, PreallocatedLayer)):
                return None
            while len(layers) <= self.layer_idx:
                layers.append(make())
        slot = layers[self.layer_idx]
        if not isinstance(slot, PreallocatedLayer):
            return None
        kb = slot._kbuf
        if kb is not None and (kb.shape[0] != b or kb.shape[1] != self.num_key_value_heads or kb.shape[3] != 128
                               or kb.dtype != torch.bfloat16 or kb.device != hidden_states.device or slot._vbuf is None
                               or slot._vbuf.stride() != kb.stride()):
            return None
        cos, sin = position_embeddings
        if cos.dtype != torch.bfloat16 or cos.shape[-1] != 128 or cos.shape[-2] != 1 or cos.shape[0] not in (1, b) or cos.dim() != 3 \
                or cos.stride(-1) != 1 or sin.stride() != cos.stride():
            return None
        S = slot.get_seq_length() + 1
        return slot, self._additive_mask(attention_mask, b, 1, S)

    def _fast_decode(self, hidden_states, position_embeddings, slot, norm=None, residual=None, amask=None):
        """The decode branch (reference :551-625) for one new token per sequence in five launches: fused QKV projection
        (ha_linear_skinny; the library's GEMM on the stacked weight for more than 16 sequences), rotary embedding + in-place cache append + both hashes (ha_rope_encode_step_cos_sin), distance
        histograms, selection fused into the gather attention, output projection.  For the decoder layer around it
        (`fast_decoder_layer_forward`): `norm` = (weight, eps) of an RMSNorm applied to hidden_states inside the QKV projection,
        `residual` [b, hidden] added inside the output projection."""
        b, _, hidden = hidden_states.shape
        H, Hkv, d = self.num_heads, self.num_key_value_heads, self.head_dim
        dev = hidden_states.device
        sc = self.__dict__.get("_fast_scratch")
        if sc is None or sc["qkv"].shape[0] != b or sc["qkv"].device != dev:
            sc = dict(qkv=torch.empty(b, (H + 2 * Hkv) * d, dtype=torch.bfloat16, device=dev),
                      q=torch.empty(b, H, d, dtype=torch.bfloat16, device=dev),
                      attn=torch.empty(b, H, d, dtype=torch.bfloat16, device=dev))
            self.__dict__["_fast_scratch"] = sc
        tiled = self._takes_tiled_projections(b, hidden)
        if tiled:                               # 9 to 32 sequences: the matrix cores on a tiled copy of the stacked weight
            _ops._linear_tiled_unchecked(hidden_states[:, 0, :], self._weight_tiles("_qkv_tiles", (self.q_proj.weight, self.k_proj.weight,
                                                                                                 self.v_proj.weight)),
                                         sc["qkv"].shape[1], sc["qkv"])
        elif b > _ops.LINEAR_SKINNY_MAX_ROWS:   # more sequences than the projection kernels take: the library's GEMM, still one call
            torch.mm(hidden_states[:, 0, :], self._fused_qkv_weight().t(), out=sc["qkv"])
        elif norm is None:
            _ops._linear_skinny_unchecked(hidden_states[:, 0, :], self._fused_qkv_weight(), sc["qkv"])
        else:
            _ops._linear_skinny_unchecked(hidden_states[:, 0, :], self._fused_qkv_weight(), sc["qkv"], norm_weight=norm[0], eps=norm[1])
        kbuf, vbuf, pos = slot.append_slots(hidden_states, b, Hkv, d, 1)
        S = pos + 1
        hl = self._ensure_hash_layer(b, S, dev)
        if hl.n_cached > pos:
            hl.reset()                       # the cache was rewound
        if hl.n_cached < pos:                # keys cached by a prefill: hashed in bulk, once
            hl.encode_keys_bulk(kbuf[:, :, hl.n_cached:pos], pos0=hl.n_cached)
        cos, sin = position_embeddings
        _ops.rope_encode_step_cos_sin(sc["qkv"], H, Hkv, pos, cos[:, 0, :], sin[:, 0, :], sc["q"], kbuf, vbuf, hl.wk, hl.wq, hl.num_layers,
                                      hl.int_dim, hl.final_dim, hl.codes, hl.qcodes, arith=hl.arith)
        hl.n_cached = S
        heavy = hl.heavy_count(S)
        saved = hl.heavy_budget
        hl.heavy_budget = 0.0 if heavy == 0 else heavy + 0.5
        try:
            # a mask that matters (reference :593-598): the prefix of a left-padded batch goes into the fused launch; any other
            # takes the selection into memory and the masked gather
            hl._select_attend(sc["q"], kbuf, vbuf, S, sc["attn"], None, attn_mask=amask)
        finally:
            hl.heavy_budget = saved
        out = torch.empty(b, 1, hidden, dtype=torch.bfloat16, device=dev)
        if tiled:
            _ops._linear_tiled_unchecked(sc["attn"].view(b, H * d), self._weight_tiles("_o_tiles", (self.o_proj.weight,)), hidden,
                                         out.view(b, hidden), residual=residual)
        elif b > _ops.LINEAR_SKINNY_MAX_ROWS:
            torch.mm(sc["attn"].view(b, H * d), self.o_proj.weight.t(), out=out.view(b, hidden))
            if residual is not None:
                out.view(b, hidden).add_(residual)      # the projection's rounding, then the addition's
        else:
            _ops._linear_skinny_unchecked(sc["attn"].view(b, H * d), self.o_proj.weight, out.view(b, hidden), residual=residual)
        return out, None

    def _adopt_cache_layer(self, cache) -> None:
        """Before a decode step: this layer's part of a cache that `generate` (or the caller) created as a plain `DynamicCache`
        becomes a `PreallocatedLayer` in place (`cache.adopt_dynamic_layer`), so that neither this step nor any later one
        re-copies the layer's cache - and single-token steps can take the few-launch paths.  Not for offloaded caches, whose
        owner moves the tensors around."""
        if not self.adopt_cache or cache is None or getattr(cache, "offloading", False) or self.offloading_length is not None:
            return
        layers = getattr(cache, "layers", None)
        if layers is not None and len(layers) > self.layer_idx and not isinstance(layers[self.layer_idx], PreallocatedLayer):
            known = self._holds_known_keys(cache)
            if adopt_dynamic_layer(layers[self.layer_idx]) and known:
                self._note_key_storage(cache)       # the same contents under their new description

    def _heavy_hitter_forward(self, hidden_states, position_embeddings, attention_mask, cache, **kwargs):
        bsz, q_len, _ = hidden_states.shape
        self.ensure_gpu(cache, hidden_states.device)
        if q_len <= DECODE_MAX_Q_LEN and not self.train_usa:
            self._adopt_cache_layer(cache)
        self._sync_bit_cache(cache)
        if q_len == 1 and not kwargs.get("output_attentions"):
            slot = self._fast_decode_slot(hidden_states, position_embeddings, attention_mask, cache)
            if slot is not None:
                ret = self._fast_decode(hidden_states, position_embeddings, slot[0], amask=slot[1])
                self._note_key_storage(cache)
                return ret
        if q_len > DECODE_MAX_Q_LEN or self.train_usa:
            # prefill, and every step while the hash is being trained: the original dense forward (reference :529-550);
            # its keys are hashed lazily at the first decode step
            ret = self.flash_forward(hidden_states=hidden_states, position_embeddings=position_embeddings,
                                     attention_mask=attention_mask, past_key_values=cache, **kwargs)
            if self.collect_stats or self.train_usa:
                self.usa_local_compute(hidden_states, attention_mask, None, cache, position_embeddings)
            self.offload_if_necessary_cpu(cache)
            self._note_key_storage(cache)
            return ret
        if kwargs.get("output_attentions"):
            # the reference returns the weights of its dense product (:615-631); the gather attention never forms them
            raise NotImplementedError("output_attentions=True: the sparse decode branch does not materialise attention weights")
        hidden_shape = (bsz, q_len, -1, self.head_dim)
        query_states = self.q_proj(hidden_states).view(hidden_shape).transpose(1, 2)
        key_states = self.k_proj(hidden_states).view(hidden_shape).transpose(1, 2)
        value_states = self.v_proj(hidden_states).view(hidden_shape).transpose(1, 2)
        if position_embeddings is None:
            raise ValueError("position_embeddings (cos, sin) are required")
        cos, sin = position_embeddings
        query_states, key_states = self._apply_rope(query_states, key_states, cos, sin)
        if cache is not None:
            key_states, value_states = cache.update(key_states, value_states, self.layer_idx)
            # the tokens the cache holds, from the cache and not from the shape of what it returns: a cache that keeps capacity
            # ahead of its length (`StaticCache`; `cache.PreallocatedCache` returns views of the right length already) hands out
            # its whole buffer
            S = self._cache_len(cache)
            if 0 < S < key_states.shape[2]:
                key_states, value_states = key_states[:, :, :S], value_states[:, :, :S]
        if key_states.stride(-1) != 1 or value_states.stride() != key_states.stride():
            key_states, value_states = key_states.contiguous(), value_states.contiguous()
        attn = self._sparse_attention(query_states.contiguous(), key_states, value_states, attention_mask)
        attn = attn.transpose(1, 2).reshape(bsz, q_len, -1).contiguous()
        out = self.o_proj(attn)
        self.offload_if_necessary_cpu(cache)
        self._note_key_storage(cache)
        return out, None

    # ---- reference API kept for callers; outside the accelerated path
    def compute_mask_multi(self, key_states, query_states):
        """Boolean keep-mask [b, H, q, S] (reference :401-446), materialised from the kernels' index lists.
        key_states is the repeat_kv'd key tensor as in the reference; only its first KV copy per group is read."""
        b, H, q_len, d = query_states.shape
        S = key_states.shape[2]
        kv = key_states[:, ::self.num_key_value_groups].contiguous() if key_states.shape[1] == H else key_states
        hl = self._ensure_hash_layer(b, S, query_states.device)
        kv, query_hash = self._hash_inputs(kv, query_states)
        hl.reset()
        hl.encode_keys(kv, pos0=0)
        hl.n_cached = S
        # one spare column collects the unused tail of every index list
        mask = torch.zeros(b, H, q_len, S + 1, dtype=torch.bool, device=query_states.device)
        heavy = hl.heavy_count(S)
        saved = hl.heavy_budget
        hl.heavy_budget = 0.0 if heavy == 0 else heavy + 0.5
        try:
            ar = torch.arange(hl.idx_cap, device=mask.device)
            for i in range(q_len):
                s_i = S - q_len + i + 1
                hl.encode_query(query_hash[:, :, i:i + 1].contiguous())
                hl.select(s_i, None)
                valid = ar[None, None, :] < hl.counts[:, :, None]
                where = torch.where(valid, hl.idx.long(), torch.full_like(hl.idx, S, dtype=torch.long))
                mask[:, :, i].scatter_(2, where, True)
        finally:
            hl.heavy_budget = saved
            hl.reset()      # these codes belong to the keys handed in, not to a KV cache: the next decode step hashes afresh
        mask = mask[..., :S]
        return mask

    def compute_mask(self, key_states, query_states):
        assert query_states.shape[-2] == 1
        return self.compute_mask_multi(key_states, query_states)

    @torch.inference_mode(False)
    def train_step(self, K, Q, target, target_mask):
        """One optimizer step of the hash module on this layer's keys and queries (reference :304-316): soft scores of
        Q [b, H, q, d] against K [b, H, S, d] (KV heads already repeated), entries outside `target_mask` zeroed, the
        installed loss against `target`, backward, optimizer step.  The loss is kept in `last_train_loss`."""
        if self.tr_loss_func is None or self.tr_optimizer is None:
            raise RuntimeError("set_train_usa_mode(model, loss_func, optimizer) must install a loss and an optimizer first")
        with torch.enable_grad():
            K, Q, target = K.clone(), Q.clone(), target.clone()      # tensors of their own for the backward pass
            span, _ = self.usa_module(K, Q)
            span = span.masked_fill(torch.logical_not(target_mask), 0)
            loss = self.tr_loss_func(span, target)
            self.tr_optimizer.zero_grad()
            loss.backward()
            self.tr_optimizer.step()
        self.last_train_loss = loss.detach()
        if self._hash_layer is not None:       # the packed weights and the cached codes belong to the old parameters
            self._hash_layer = None
        self.usa_module.invalidate_packed()
        if self.layer_idx == 5:
            print(self.layer_idx, K.shape[2], "Train Loss:", loss.item(), flush=True)

    def usa_local_compute(self, hidden_states, attention_mask=None, position_ids=None, past_key_value=None,
                          position_embeddings=None):
        """Recall statistic of the hash ranking (reference :319-398, eval branch): whenever the cache length is a multiple
        of 1024, for every query row of this chunk, which fraction of its 32 highest true attention logits among the
        candidates [init, pos - recent] is inside the S // 16 candidates of smallest Hamming distance.  Accumulated per
        cache length in `self.overlaps[S] = [sum, sum of squares, count, mean, std]` as the reference does.

        The hash side runs on the selection kernel: all rows of the chunk in one ha_select call against the same codes
        (batch stride 0), each row with its own length.  Ties of the hash score go to the lowest index (the reference's
        torch.topk leaves them open); rows with fewer than 32 candidates count only real candidates as targets."""
        cache = past_key_value
        if cache is None or len(cache.layers) <= self.layer_idx:
            return
        keys = cache.layers[self.layer_idx].keys                        # [b, Hkv, S, d], the chunk's keys already appended
        if keys is None or keys.shape[-2] % 1024 != 0:
            return
        bsz, q_len, _ = hidden_states.shape
        S = keys.shape[-2]
        H, d = self.num_heads, self.head_dim
        shape = (bsz, q_len, -1, d)
        q = self.q_proj(hidden_states).view(shape).transpose(1, 2)
        k_new = self.k_proj(hidden_states).view(shape).transpose(1, 2)
        cos, sin = position_embeddings
        q, _ = self._apply_rope(q, k_new, cos, sin)
        q = q.contiguous()
        keys = keys if keys.stride(-1) == 1 else keys.contiguous()
        dev = q.device
        if self.train_usa:
            # train branch (:356-371): per row, the 32 highest true logits among the candidates [init, pos - recent] are the
            # positives; the hash module takes one optimizer step on them.  Logits in fp32 (the reference: model dtype).
            kk = keys.repeat_interleave(self.num_key_value_groups, dim=1)                       # [b, H, S, d]
            w = torch.matmul(q.float(), kk.float().transpose(2, 3)) / math.sqrt(d)
            cand = torch.tril(torch.ones(q_len, S, device=dev), diagonal=S - q_len - self.recent_budget).bool()
            cand[:, :self.init_budget] = False
            w.masked_fill_(torch.logical_not(cand), torch.finfo(w.dtype).min)
            target = torch.zeros(w.shape, dtype=self.usa_module.dtype, device=dev)
            target.scatter_(-1, torch.topk(w, k=32, dim=-1).indices, 1.0)
            del w
            self.train_step(kk.to(self.usa_module.dtype), q.to(self.usa_module.dtype), target, cand)
            return

        # ---- hash side: codes of all keys and of every query row, one selection per row
        hl = self._ensure_hash_layer(bsz, S, dev)
        key_hash, query_hash = self._hash_inputs(keys, q)
        kc = torch.zeros(bsz, hl.Hc, S, hl.W, dtype=torch.int32, device=dev)
        _ops.encode_pack(key_hash, hl.wk, hl.num_layers, hl.int_dim, hl.final_dim, kc, 0, None, hl.arith)
        qc = torch.zeros(bsz, H, q_len, hl.W, dtype=torch.int32, device=dev)
        _ops.encode_pack(query_hash, hl.wq, hl.num_layers, hl.int_dim, hl.final_dim, qc, 0, None, hl.arith)
        n_pred = S // 16
        if n_pred < 2:                                  # a heavy budget <= 1 would be read as a fraction
            return
        cap = min(S, self.init_budget + self.recent_budget + n_pred)
        lens = torch.arange(S - q_len + 1, S + 1, dtype=torch.int32, device=dev)      # row i sees keys [0, S - q_len + i]
        ws = _ops.workspace(_ops.select_workspace_bytes(q_len, H, hl.Hc, hl.W, S), dev)
        idx = torch.empty(q_len, H, cap, dtype=torch.int32, device=dev)
        cnt = torch.empty(q_len, H, dtype=torch.int32, device=dev)
        scale = 1.0 / math.sqrt(d)
        top_true = 32
        ratios = []
        for b in range(bsz):
            _ops.select(kc[b:b + 1].expand(q_len, -1, -1, -1), qc[b].transpose(0, 1).contiguous(), S, lens, self.init_budget,
                        self.recent_budget, float(n_pred) + 0.5, idx, cnt, ws)
            # lists are ascending; everything past the count becomes a sentinel so that a binary search can test membership
            pos = torch.arange(cap, device=dev)
            lists = torch.where(pos[None, None, :] < cnt[:, :, None], idx, torch.full_like(idx, 2 ** 31 - 1))
            # ---- true side (reference :357-366): logits of the candidates, top 32
            kk = keys[b].repeat_interleave(self.num_key_value_groups, dim=0).float()             # [H, S, d]
            logits = torch.matmul(q[b].float(), kk.transpose(1, 2)) * scale                       # [H, q_len, S]
            j = torch.arange(S, device=dev)
            cand = (j[None, :] >= self.init_budget) & (j[None, :] <= (lens[:, None] - 1 - self.recent_budget))   # [q_len, S]
            logits = logits.masked_fill(~cand[None], float("-inf"))
            kt = min(top_true, S)
            top = torch.topk(logits, kt, dim=-1)
            tgt = top.indices.transpose(0, 1).contiguous().to(torch.int32)                       # [q_len, H, kt]
            real = torch.isfinite(top.values).transpose(0, 1)
            where = torch.searchsorted(lists, tgt).clamp_(max=cap - 1)
            hit = (torch.gather(lists, 2, where) == tgt) & real
            ratios.append(hit.sum(-1).float() / top_true)                                         # [q_len, H]
        r = torch.stack(ratios)                                                                  # [b, q_len, H]
        st = self.overlaps.setdefault(S, [0, 0, 0, 0, 0])                                        # sum, sqsum, ct, mean, std
        st[0] += r.sum().item()
        st[1] += torch.square(r).sum().item()
        st[2] += r.numel()
        st[3] = st[0] / st[2]
        st[4] = math.sqrt(max(st[1] / st[2] - st[3] ** 2, 0.0))
        self.last_overlap_ratio = r.permute(0, 2, 1)                                             # [b, H, q_len], for tests


# ------------------------------------------------------------------------------------------ the decoder layer around it

def _stacked_gate_up(attn, mlp) -> torch.Tensor:
    """gate_proj and up_proj weights as one [2 F, hidden] matrix (gate rows, then up rows: what the projection kernel's
    SwiGLU form reads); a copy, kept on the attention module and rebuilt when a parameter was replaced or updated in place
    through its version counter."""
    ws = (mlp.gate_proj.weight, mlp.up_proj.weight)
    key = tuple((w.data_ptr(), w._version, w.dtype, w.device) for w in ws)
    hit = attn.__dict__.get("_gate_up_fused")
    if hit is None or hit[0] != key:
        hit = (key, torch.cat([w.detach() for w in ws], dim=0).contiguous())
        attn.__dict__["_gate_up_fused"] = hit
    return hit[1]


def _layer_modules(layer):
    """(mlp, input norm, post-attention norm, gate, up, down) of a decoder layer of the Llama shape - RMSNorm, attention,
    residual, RMSNorm, SiLU-gated MLP of plain nn.Linear projections without biases, residual - or False.  Looked up once
    and again whenever one of these modules is no longer the object that was looked at (an adapter library replaces
    projections by wrappers with a forward of their own; such a layer keeps the library's path)."""
    seen = layer.__dict__.get("_fast_seen")
    own = layer._modules
    mlp = own.get("mlp")
    sub = mlp._modules if mlp is not None else {}
    now = (mlp, own.get("input_layernorm"), own.get("post_attention_layernorm"), sub.get("gate_proj"), sub.get("up_proj"), sub.get("down_proj"))
    if seen is not None and all(a is b for a, b in zip(seen[0], now)):
        return seen[1]
    n1, n2, lin = now[1], now[2], now[3:]
    act = getattr(mlp, "act_fn", None)      # nn.SiLU, or the class transformers keeps under "silu"
    ok = mlp is not None and n1 is not None and n2 is not None and all(type(m) is nn.Linear and m.bias is None for m in lin) \
        and (isinstance(act, nn.SiLU) or type(act).__name__ == "SiLUActivation") \
        and all(getattr(n, "weight", None) is not None and hasattr(n, "variance_epsilon") and "RMSNorm" in type(n).__name__ for n in (n1, n2))
    layer.__dict__["_fast_seen"] = (now, now if ok else False)
    return now if ok else False


FUSED_LAYER_MAX_ROWS = _FUSED_ROWS     # sequences for which the projection kernel takes the norm in front and SwiGLU behind


def _layer_takes_fast_path(layer, hidden_states):
    """The layer's modules (`_layer_modules`) when a single-token step can run as a handful of launches - seven for up to 8
    sequences, twelve calls above: bf16 weights, for the seven-launch form hidden states of at most 16384 elements (the
    projection kernel's fused forms), and no forward hook on a module that this path would not call (activation capture,
    adapters that wrap a forward); else False."""
    if hidden_states.shape[1] != 1:
        return False
    mods = _layer_modules(layer)
    if not mods:
        return False
    if layer.self_attn._forward_hooks or layer.self_attn._forward_pre_hooks:
        return False
    for m in mods:
        if m._forward_hooks or m._forward_pre_hooks:
            return False
    gate, down = mods[3], mods[5]
    if gate.in_features > 16384 and hidden_states.shape[0] <= FUSED_LAYER_MAX_ROWS:    # the norm-in-front form keeps a row of hidden states in registers
        return False
    bf16 = torch.bfloat16
    if gate.weight.dtype != bf16 or mods[4].weight.dtype != bf16 or down.weight.dtype != bf16 or mods[1].weight.dtype != bf16 \
            or mods[2].weight.dtype != bf16:
        return False
    return mods


def fast_decoder_layer_forward(layer, hidden_states, attention_mask=None, position_ids=None, past_key_values=None, use_cache=False,
                               position_embeddings=None, **kwargs):
    """`forward` of a transformers decoder layer whose attention module was converted.  A single-token step that the attention
    module takes in five launches (`_fast_decode_slot`) runs the WHOLE layer in seven for up to 8 sequences: input RMSNorm
    inside the QKV projection, the attention step, residual inside the output projection, post-attention RMSNorm in front of
    and SwiGLU behind the stacked gate/up projection, residual inside the down projection (the launches of
    `LlamaShapedDecoder`) - instead of the ~25 library calls of the layer's own forward, which at these sizes are bound by
    the host.  Larger batches take nine to twelve calls (below).  Everything else goes to the layer's own forward.  The fused
    forms round where the modules they replace round, so outputs differ from the layer's own by the bf16 rounding of other
    summation orders only."""
    attn = layer.self_attn
    cache = past_key_values if past_key_values is not None else kwargs.get("past_key_value")
    mods = getattr(attn, "fast_layer", False) and not kwargs.get("output_attentions") and _layer_takes_fast_path(layer, hidden_states)
    if mods:
        attn.ensure_gpu(cache, hidden_states.device)
        if not attn.train_usa:
            attn._adopt_cache_layer(cache)
        attn._sync_bit_cache(cache)
        slot = attn._fast_decode_slot(hidden_states, position_embeddings, attention_mask, cache)
        if slot is not None and hidden_states.shape[0] > FUSED_LAYER_MAX_ROWS:
            # more sequences than the fused forms take: the same layer in nine to twelve calls - each RMSNorm one launch with the
            # module's two roundings, the attention step (the first residual inside its output projection), gate/up with SwiGLU
            # (9 to 32 sequences: one launch on a tiled copy of the stacked weight; above: the library's GEMM and ha_swiglu), the
            # down projection (9 to 16 sequences: from tiles, the second residual inside; above: the library's GEMM and an
            # addition) - instead of the library layer's ~26
            b, _, hidden = hidden_states.shape
            mlp, n1, n2, gate, _, down = mods
            h = torch.empty_like(hidden_states)
            _ops.rmsnorm(hidden_states[:, 0, :], n1.weight, float(n1.variance_epsilon), h[:, 0, :])
            x1, _ = attn._fast_decode(h, position_embeddings, slot[0], residual=hidden_states[:, 0, :], amask=slot[1])
            attn._note_key_storage(cache)
            _ops.rmsnorm(x1[:, 0, :], n2.weight, float(n2.variance_epsilon), h[:, 0, :])
            act = attn.__dict__.get("_fast_act")
            if act is None or act.shape[0] != b or act.shape[1] != gate.out_features or act.device != hidden_states.device:
                act = torch.empty(b, gate.out_features, dtype=torch.bfloat16, device=hidden_states.device)
                attn.__dict__["_fast_act"] = act
            if attn._takes_tiled_projections(b, hidden):    # 9 to 32 sequences: gate/up on the matrix cores, SwiGLU inside
                _ops._linear_tiled_unchecked(h[:, 0, :], attn._weight_tiles("_gate_up_tiles", (mlp.gate_proj.weight, mlp.up_proj.weight),
                                                                            glu=True), 2 * gate.out_features, act, swiglu=True)
            else:
                _ops.swiglu(torch.mm(h[:, 0, :], _stacked_gate_up(attn, mlp).t()), act)
            if b <= _ops.LINEAR_SKINNY_MAX_ROWS and attn._takes_tiled_projections(b, hidden):
                out = torch.empty_like(x1)      # the down projection with its residual inside, x requested next to the tiles
                _ops._linear_tiled_unchecked(act, attn._weight_tiles("_down_tiles", (down.weight,)), hidden, out[:, 0, :],
                                             residual=x1[:, 0, :])
                return out
            return x1 + torch.mm(act, down.weight.t()).view(b, 1, hidden)
        if slot is not None:
            b = hidden_states.shape[0]
            mlp, n1, n2, gate, _, down = mods
            x1, _ = attn._fast_decode(hidden_states, position_embeddings, slot[0], norm=(n1.weight, float(n1.variance_epsilon)),
                                      residual=hidden_states[:, 0, :], amask=slot[1])
            attn._note_key_storage(cache)
            act = attn.__dict__.get("_fast_act")
            if act is None or act.shape[0] != b or act.shape[1] != gate.out_features or act.device != hidden_states.device:
                act = torch.empty(b, gate.out_features, dtype=torch.bfloat16, device=hidden_states.device)
                attn.__dict__["_fast_act"] = act
            x1_rows = x1[:, 0, :]
            _ops._linear_skinny_unchecked(x1_rows, _stacked_gate_up(attn, mlp), act, norm_weight=n2.weight, eps=float(n2.variance_epsilon),
                                          swiglu=True)
            out = torch.empty_like(x1)
            _ops._linear_skinny_unchecked(act, down.weight, out[:, 0, :], residual=x1_rows)
            return out
    return layer._hf_forward(hidden_states, attention_mask=attention_mask, position_ids=position_ids, past_key_values=past_key_values,
                             use_cache=use_cache, position_embeddings=position_embeddings, **kwargs)


def install_fast_layers(model):
    """Route the decoder layers that hold a converted attention module through `fast_decoder_layer_forward`."""
    import types
    for layer in model.modules():
        attn = getattr(layer, "self_attn", None)
        if isinstance(attn, HeavyHitterMixin) and "_hf_forward" not in layer.__dict__ and hasattr(layer, "mlp"):
            layer.__dict__["_hf_forward"] = layer.forward
            layer.forward = types.MethodType(fast_decoder_layer_forward, layer)
    return model


# ------------------------------------------------------------------------------------------ module-patch helpers

def _head_dim_of(config) -> int:
    """Width of an attention head; the kernels are built for 128 (Llama-3.x 8B / 70B, Mistral-7B: the models the reference's
    checkpoints are for) and say so before anything is patched rather than at the first decode step."""
    head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
    if head_dim != 128:
        raise NotImplementedError(f"the HIP attention kernels of this build are written for 128-wide heads; this model has head_dim={head_dim}")
    return head_dim


def build_usa_modules(config, path, force_num_layers=None) -> nn.ModuleList:
    """Body of `load_usa` (reference :633-646): one USA per decoder layer, optionally loaded from a state dict.
    `force_num_layers`: the depth of the hash MLP when the family's reference ignores `config.lth_num_layers` (Mistral)."""
    cfg = {"lth_int_dim": config.lth_init_dim, "lth_final_dim": config.lth_final_dim, "lth_thold": config.lth_thold,
           "lth_num_layers": force_num_layers if force_num_layers is not None else config.lth_num_layers}
    head_dim = _head_dim_of(config)
    mods = nn.ModuleList([USA(config.num_attention_heads, head_dim, cfg) for _ in range(config.num_hidden_layers)])
    if path is not None:
        # checkpoints are plain state dicts of tensors: load them without executing anything from the file
        mods.load_state_dict(torch.load(path, map_location="cpu", weights_only=True))
    if not torch.cuda.is_available():
        raise RuntimeError("load_usa() returns the modules on the GPU (reference :646) and no GPU is visible; "
                           "this build has no CPU path")
    _ops.load_library()
    return mods.cuda()


def convert_modules(model, config, usa_modules, collect_stats, train_usa, original_cls, patched_cls):
    """Body of `convert_usa` (reference :650-667): replace every `original_cls` by `patched_cls` in place."""
    _head_dim_of(config)
    for name, module in reversed(model._modules.items()):
        if len(list(module.children())) > 0:
            model._modules[name] = convert_modules(module, config, usa_modules, collect_stats, train_usa,
                                                   original_cls, patched_cls)
        if isinstance(module, original_cls):
            device = next(module.parameters()).device
            new_module = patched_cls(config, module.layer_idx).bfloat16().to(device)
            new_module.load_state_dict(module.state_dict())
            new_module.usa_module = usa_modules[module.layer_idx]
            new_module.usa_module_dtype = usa_modules[module.layer_idx].dtype
            new_module.flash_forward = module.forward
            new_module.collect_stats = collect_stats
            new_module.train_usa = train_usa
            model._modules[name] = new_module
    return model


def walk(model, patched_cls, fn):
    for name, module in reversed(model._modules.items()):
        if len(list(module.children())) > 0:
            model._modules[name] = walk(module, patched_cls, fn)
        if isinstance(module, patched_cls):
            fn(module)
    return model

"""Host logic of the patched layer that needs no GPU: how the attention mask of a forward pass is examined - what the reference
adds to the scores before its softmax (hashattention_llama.py:593-598) - and in which form it is handed to the kernels; which
decoder layers take the few-launch step."""
import torch

from hashattention import _patched


def _layer():
    return _patched.HeavyHitterMixin.__new__(_patched.HeavyHitterMixin)


def _additive(keep: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    """The library's float form of a keep-mask: 0 where a token may be attended, the most negative value elsewhere."""
    return torch.zeros(keep.shape, dtype=dtype).masked_fill_(~keep, torch.finfo(dtype).min)


def test_a_mask_that_blocks_nothing_is_dropped():
    layer, b, S = _layer(), 3, 40
    assert layer._additive_mask(None, b, 1, S) is None
    keep = torch.ones(b, 1, 1, S, dtype=torch.bool)
    assert layer._additive_mask(keep, b, 1, S) is None
    assert layer._additive_mask(_additive(keep, torch.bfloat16), b, 1, S) is None
    # a chunk of rows: what the mask blocks beyond the causal edge changes nothing, the kernels apply that edge themselves
    causal = torch.tril(torch.ones(5, S, dtype=torch.bool), diagonal=S - 5)[None, None].expand(b, 1, 5, S)
    assert layer._additive_mask(causal, b, 5, S) is None
    # longer than the cache (a buffer with room ahead): only the first S columns count
    wide = torch.ones(b, 1, 1, S + 9, dtype=torch.bool)
    wide[..., S:] = False
    assert layer._additive_mask(wide, b, 1, S) is None


def test_left_padding_is_recognised_as_one_number_per_sequence():
    layer, b, S = _layer(), 3, 40
    keep = torch.ones(b, 1, 1, S, dtype=torch.bool)
    keep[1, ..., :7] = False
    keep[2, ..., :39] = False
    for mask in (keep, _additive(keep), _additive(keep, torch.bfloat16), _additive(keep, torch.float16),
                 torch.zeros(b, 1, 1, S).masked_fill_(~keep, float("-inf"))):
        sm = layer._additive_mask(mask, b, 1, S)
        assert sm is not None and sm.prefix is not None and sm.prefix.dtype == torch.int32 and sm.prefix.tolist() == [0, 7, 39]
        table = sm.table()
        assert table.shape == (b, S) and table.dtype == torch.float32
        assert torch.equal(table == 0, keep[:, 0, 0]) and bool((table[~keep[:, 0, 0]] <= -6e4).all())
    # one mask row shared by the batch
    one = torch.ones(1, 1, 1, S, dtype=torch.bool)
    one[..., :4] = False
    sm = layer._additive_mask(one, b, 1, S)
    assert sm.prefix.tolist() == [4, 4, 4] and sm.table().shape == (b, S)


def test_other_masks_keep_their_table():
    layer, b, S = _layer(), 2, 40
    hole = torch.ones(b, 1, 1, S, dtype=torch.bool)
    hole[0, ..., 10:13] = False                                    # not a prefix
    sm = layer._additive_mask(hole, b, 1, S)
    assert sm is not None and sm.prefix is None and torch.equal(sm.table() == 0, hole[:, 0, 0])
    bias = torch.zeros(b, 1, 1, S)
    bias[1, ..., :5] = -2.5                                        # a prefix, but of finite terms: they are added, not dropped
    sm = layer._additive_mask(bias, b, 1, S)
    assert sm is not None and sm.prefix is None and torch.equal(sm.table(), bias[:, 0, 0])
    mixed = _additive(torch.ones(b, 1, 1, S, dtype=torch.bool))
    mixed[0, ..., :3] = torch.finfo(torch.float32).min
    mixed[0, ..., 3] = -1.0
    sm = layer._additive_mask(mixed, b, 1, S)
    assert sm.prefix is None
    # a chunk of rows with padding: the fp32 rows, no prefix form
    keep = torch.tril(torch.ones(4, S, dtype=torch.bool), diagonal=S - 4)[None, None].repeat(b, 1, 1, 1)
    keep[1, ..., :6] = False
    sm = layer._additive_mask(keep, b, 4, S)
    assert sm is not None and sm.prefix is None and sm.rows().shape == (b, 4, S) and bool((sm.rows()[1, :, :6] == float("-inf")).all())


def test_one_examination_serves_every_layer_of_a_pass_and_a_changed_mask_is_examined_again():
    a, c, b, S = _layer(), _layer(), 2, 30
    keep = torch.ones(b, 1, 1, S, dtype=torch.bool)
    keep[0, ..., :5] = False
    first = a._additive_mask(keep, b, 1, S)
    assert c._additive_mask(keep, b, 1, S) is first and first.rows() is first.rows()      # the fp32 form is made once
    keep[0, ..., :9] = False                                       # written in place: the tensor's version moved
    again = c._additive_mask(keep, b, 1, S)
    assert again is not first and again.prefix.tolist() == [9, 0]
    assert a._additive_mask(keep, b, 1, S - 1) is not again         # another length: examined again
    other = keep.clone()
    assert a._additive_mask(other, b, 1, S) is not again


def test_a_mask_of_the_wrong_shape_is_refused():
    import pytest
    layer = _layer()
    with pytest.raises(ValueError, match="Attention mask should be of size"):
        layer._additive_mask(torch.ones(2, 1, 1, 10, dtype=torch.bool), 2, 1, 12)
    with pytest.raises(ValueError):
        layer._additive_mask(torch.ones(3, 1, 1, 12, dtype=torch.bool), 2, 1, 12)


def _decoder_layer(**kw):
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaDecoderLayer
    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=1, num_attention_heads=2, num_key_value_heads=1,
                      head_dim=128, vocab_size=64, **kw)
    return LlamaDecoderLayer(cfg, 0).bfloat16()


def test_which_decoder_layers_take_the_few_launch_step():
    # the whole-layer step reads weights directly: it is for layers of the Llama shape made of plain modules, and steps aside for
    # anything that wants a say (wrappers around a projection, hooks, biases, another activation)
    layer = _decoder_layer()
    x = torch.zeros(2, 1, 256, dtype=torch.bfloat16)
    mods = _patched._layer_modules(layer)
    assert mods and mods[0] is layer.mlp and mods[3] is layer.mlp.gate_proj and mods[5] is layer.mlp.down_proj
    assert _patched._layer_takes_fast_path(layer, x) is mods
    assert _patched._layer_takes_fast_path(layer, torch.zeros(2, 3, 256, dtype=torch.bfloat16)) is False      # a chunk of tokens
    assert _patched._layer_takes_fast_path(layer, torch.zeros(40, 1, 256, dtype=torch.bfloat16)) is mods      # any number of sequences

    class Wrapped(torch.nn.Module):
        def __init__(self, inner):
            super().__init__()
            self.inner = inner

        def forward(self, t):
            return self.inner(t) + 1

    plain = layer.mlp.up_proj
    layer.mlp.up_proj = Wrapped(plain)
    assert _patched._layer_modules(layer) is False and _patched._layer_takes_fast_path(layer, x) is False
    layer.mlp.up_proj = plain                                       # the wrapper is gone: the step comes back
    assert _patched._layer_takes_fast_path(layer, x)
    handle = layer.mlp.down_proj.register_forward_hook(lambda m, a, o: None)
    assert _patched._layer_takes_fast_path(layer, x) is False
    handle.remove()
    assert _patched._layer_takes_fast_path(layer, x)
    handle = layer.self_attn.register_forward_pre_hook(lambda m, a: None)
    assert _patched._layer_takes_fast_path(layer, x) is False
    handle.remove()
    assert _patched._layer_takes_fast_path(layer.float(), x) is False       # fp32 weights
    assert _patched._layer_modules(_decoder_layer(mlp_bias=True)) is False
    assert _patched._layer_modules(_decoder_layer(hidden_act="gelu")) is False


class _Codes:
    """Stands in for the hash layer: what `_sync_bit_cache` reads and writes."""

    def __init__(self, n):
        self.n_cached, self.resets = n, 0

    def reset(self):
        self.n_cached, self.resets = 0, self.resets + 1


def _attn(n_cached):
    layer = _layer()
    layer.layer_idx, layer._cache_ref, layer._cache_id, layer._hash_layer = 0, None, None, _Codes(n_cached)
    return layer


def test_codes_follow_the_cache_they_were_made_from():
    # the reference re-hashes every key at every step (hashattention_llama.py:407-408), so nothing a caller does to the cache
    # between two passes may leave codes of other contents behind: another cache object, reordered or selected batch entries
    # (beam search), a rewound cache
    from transformers import DynamicCache
    from hashattention.cache import PreallocatedCache
    k = torch.zeros(3, 1, 6, 4)
    for make in (DynamicCache, lambda: PreallocatedCache(capacity=16)):
        cache = make()
        cache.update(k, k, 0)
        attn = _attn(0)
        attn._sync_bit_cache(cache)                  # first sight of this cache
        attn._hash_layer.n_cached = 6                # ... the pass hashes its keys and notes where they lie
        attn._note_key_storage(cache)
        attn._sync_bit_cache(cache)
        assert attn._hash_layer.n_cached == 6 and attn._hash_layer.resets == 1      # untouched cache: codes kept
        cache.update(k[:, :, :1], k[:, :, :1], 0)    # the cache's own append (a new tensor for DynamicCache): seen by the pass
        attn._hash_layer.n_cached = 7
        attn._note_key_storage(cache)
        attn._sync_bit_cache(cache)
        assert attn._hash_layer.n_cached == 7
        cache.reorder_cache(torch.tensor([2, 0, 1]))     # beam search moved batch entries
        attn._sync_bit_cache(cache)
        assert attn._hash_layer.n_cached == 0 and attn._hash_layer.resets == 2
        attn._hash_layer.n_cached = 7
        attn._note_key_storage(cache)
        cache.crop(4)                                # rewound: the in-place cache keeps the codes of its prefix, the library's
        attn._sync_bit_cache(cache)                  # leaves a new tensor behind and is hashed afresh
        assert attn._hash_layer.n_cached == (4 if isinstance(cache, PreallocatedCache) else 0)
        other = make()
        other.update(k, k, 0)
        attn._hash_layer.n_cached = 4
        attn._sync_bit_cache(other)                  # another cache object: nothing is kept
        assert attn._hash_layer.n_cached == 0
        attn._sync_bit_cache(None)
        assert attn._hash_layer.n_cached == 0

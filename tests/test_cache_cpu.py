"""Host logic of `hashattention.cache` on CPU tensors (no kernel involved): a PreallocatedLayer must behave as the DynamicLayer
it replaces - same keys / values after every update, crop, batch selection and reordering - while appending in place."""
import torch
from transformers import DynamicCache

from hashattention.cache import PreallocatedCache, PreallocatedLayer, adopt_dynamic_layer


def _states(g, b, h, t, d=8):
    return torch.randn(b, h, t, d, generator=g), torch.randn(b, h, t, d, generator=g)


def test_updates_match_dynamic_cache_and_append_in_place():
    g = torch.Generator().manual_seed(0)
    ref, got = DynamicCache(), PreallocatedCache(capacity=16)
    ptr = None
    for step, t in enumerate([5, 1, 1, 3, 1]):                    # 11 tokens: inside the reserved 16
        for layer in range(2):
            k, v = _states(g, 2, 3, t)
            rk, rv = ref.update(k, v, layer)
            gk, gv = got.update(k, v, layer)
            assert torch.equal(gk, rk) and torch.equal(gv, rv)
            assert gk.shape == rk.shape and gk.stride(-1) == 1
        if ptr is None:
            ptr = got.layers[0]._kbuf.data_ptr()
        assert got.layers[0]._kbuf.data_ptr() == ptr              # never reallocated
        assert got.get_seq_length() == ref.get_seq_length() and got.get_seq_length(1) == ref.get_seq_length(1)
    layer = got.layers[0]
    assert isinstance(layer, PreallocatedLayer) and layer.capacity == 16 and layer.keys.shape[2] == 11
    assert layer.get_mask_sizes(1) == ref.layers[0].get_mask_sizes(1)
    # outgrowing the reservation doubles the buffer and keeps the content
    k, v = _states(g, 2, 3, 9)
    rk, _ = ref.update(k, v, 0)
    gk, _ = got.update(k, v, 0)
    assert torch.equal(gk, rk) and layer.capacity == 32 and layer._kbuf.data_ptr() != ptr


def test_crop_selection_reordering_and_adoption():
    g = torch.Generator().manual_seed(1)
    ref, got = DynamicCache(), PreallocatedCache()
    for layer in range(2):
        k, v = _states(g, 4, 2, 7)
        ref.update(k, v, layer)
        got.update(k, v, layer)
    ref.crop(-2)
    got.crop(-2)
    assert got.get_seq_length() == 5 and torch.equal(got.layers[1].keys, ref.layers[1].keys)
    k, v = _states(g, 4, 2, 1)                                     # appending after a crop overwrites the cropped slots
    assert torch.equal(got.update(k, v, 0)[0], ref.update(k, v, 0)[0])
    idx = torch.tensor([2, 0])
    ref.batch_select_indices(idx)
    got.batch_select_indices(idx)
    assert torch.equal(got.layers[0].keys, ref.layers[0].keys) and torch.equal(got.layers[0].values, ref.layers[0].values)
    ref.batch_repeat_interleave(2)
    got.batch_repeat_interleave(2)
    assert torch.equal(got.layers[0].keys, ref.layers[0].keys) and got.layers[0].keys.shape[0] == 4
    beam = torch.tensor([1, 1, 3, 0])
    ref.reorder_cache(beam)
    got.reorder_cache(beam)
    assert torch.equal(got.layers[0].values, ref.layers[0].values)
    k, v = _states(g, 4, 2, 2)                                     # and the adopted tensors keep growing
    assert torch.equal(got.update(k, v, 0)[0], ref.update(k, v, 0)[0])
    got.layers[0].reset()
    assert got.layers[0].get_seq_length() == 0 and got.get_seq_length(1) == 5


def test_append_slots_reserves_room_a_kernel_fills():
    layer = PreallocatedLayer(capacity=4)
    like = torch.zeros(1, dtype=torch.float32)
    kb, vb, pos = layer.append_slots(like, batch=2, heads=3, head_dim=8)
    assert pos == 0 and kb.shape == (2, 3, 4, 8) and layer.get_seq_length() == 1 and layer.keys.shape[2] == 1
    kb[:, :, 0] = 1.0
    vb[:, :, 0] = 2.0
    for want in (1, 2, 3):
        assert layer.append_slots(like, 2, 3, 8)[2] == want
    kb2, _, pos = layer.append_slots(like, 2, 3, 8)                # the fifth token does not fit four slots
    assert pos == 4 and layer.capacity == 8 and kb2.data_ptr() != kb.data_ptr()
    assert (layer.keys[:, :, 0] == 1.0).all() and (layer.values[:, :, 0] == 2.0).all()


def test_epoch_counts_outside_assignments_only():
    # the patched layers keep their codes while `epoch` stands still: growth and appends leave it, reordering bumps it
    cache = PreallocatedCache(capacity=2)
    g = torch.Generator().manual_seed(3)
    for _ in range(5):                                             # outgrows the capacity twice
        cache.update(*_states(g, 2, 2, 1), 0)
    layer = cache.layers[0]
    assert layer.epoch == 0 and layer.capacity >= 5
    layer.append_slots(torch.zeros(1), 2, 2, 8)
    layer.crop(-1)
    assert layer.epoch == 0
    cache.reorder_cache(torch.tensor([1, 0]))
    assert layer.epoch == 1
    cache.batch_repeat_interleave(2)
    assert layer.epoch == 2 and layer.keys.shape[0] == 4


def test_models_with_other_head_widths_are_refused_before_anything_is_patched():
    # the kernels are built for 128-wide heads: say so at load_usa / convert_usa, not at the first decode step
    import pytest
    from transformers import LlamaConfig, LlamaForCausalLM
    from hashattention import hashattention_llama as hl
    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=1, num_attention_heads=4, num_key_value_heads=2,
                      head_dim=64, vocab_size=64)
    for k, v in dict(lth_init_dim=128, lth_final_dim=32, lth_thold=0, lth_num_layers=3, init_budget=8, heavy_budget=0.125,
                     recent_budget=8, usa_retrieve_depth=6, usa_eval_mode="simple").items():
        setattr(cfg, k, v)
    with pytest.raises(NotImplementedError, match="128-wide heads"):
        hl.load_usa(cfg, None)
    model = LlamaForCausalLM(cfg)
    before = type(model.model.layers[0].self_attn)
    with pytest.raises(NotImplementedError, match="128-wide heads"):
        hl.convert_usa(model, cfg, [None], collect_stats=False, train_usa=False)
    assert type(model.model.layers[0].self_attn) is before


def test_a_dynamic_layer_is_adopted_in_place():
    from transformers.cache_utils import DynamicLayer, DynamicSlidingWindowLayer
    g = torch.Generator().manual_seed(4)
    ref, got = DynamicCache(), DynamicCache()
    for t in (6, 1):
        k, v = _states(g, 2, 2, t)
        ref.update(k, v, 0)
        got.update(k, v, 0)
    layer = got.layers[0]
    assert type(layer) is DynamicLayer and adopt_dynamic_layer(layer) and got.layers[0] is layer
    assert isinstance(layer, PreallocatedLayer) and layer.get_seq_length() == 7 and layer.capacity == 7 and layer.epoch == 0
    assert "keys" not in layer.__dict__ and torch.equal(layer.keys, ref.layers[0].keys)
    for t in (1, 1, 3):                                            # grows by a quarter (at least 256 tokens), then appends in place
        k, v = _states(g, 2, 2, t)
        a, b = got.update(k, v, 0)
        c, d = ref.update(k, v, 0)
        assert torch.equal(a, c) and torch.equal(b, d)
    assert layer.capacity == 7 + 256 and got.get_seq_length() == 12
    ptr = layer._kbuf.data_ptr()
    got.update(*_states(g, 2, 2, 1), 0)
    assert layer._kbuf.data_ptr() == ptr
    # a long prompt: the room added at a time is bounded (8192 tokens), not a quarter of the prompt
    long = DynamicCache()
    long.update(torch.zeros(1, 1, 100000, 4), torch.zeros(1, 1, 100000, 4), 0)
    assert adopt_dynamic_layer(long.layers[0])
    long.update(torch.zeros(1, 1, 1, 4), torch.zeros(1, 1, 1, 4), 0)
    assert long.layers[0].capacity == 100000 + 8192 and long.get_seq_length() == 100001
    # other layer kinds, and layers that hold nothing yet, are left alone
    assert not adopt_dynamic_layer(DynamicLayer()) and not adopt_dynamic_layer(DynamicSlidingWindowLayer(sliding_window=4))
    assert adopt_dynamic_layer(layer)                              # already one

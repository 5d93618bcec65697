"""`hashattention.cache.PreallocatedCache` - a DynamicCache whose layers append in place - and `StaticCache` under the patched
layers: same logits and tokens as with the library's DynamicCache (whose update re-copies the whole cache every step)."""
import pytest
import torch
from transformers import DynamicCache, LlamaConfig, LlamaForCausalLM, StaticCache

from hashattention import hashattention_llama as hl
from hashattention.cache import PreallocatedCache, PreallocatedLayer
from tests.test_gpu_model_api import _config

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _model(fast_decode=False, adopt_cache=False, **usa_cfg):
    torch.manual_seed(0)
    cfg = _config(LlamaConfig)
    for k, v in usa_cfg.items():
        setattr(cfg, k, v)
    model = LlamaForCausalLM(cfg).bfloat16().to(DEV)
    usa = hl.load_usa(cfg, None)
    model = hl.convert_usa(model, cfg, usa, collect_stats=False, train_usa=False)
    for layer in model.model.layers:        # the five-launch single-token path has a test of its own below
        layer.self_attn.fast_decode = fast_decode
        layer.self_attn.adopt_cache = adopt_cache       # off: a DynamicCache stays what the library made it
    return cfg, model


def _decode(model, ids, cache, steps):
    outs = []
    with torch.no_grad():
        n0 = ids.shape[1] - sum(steps)
        o = model(ids[:, :n0], past_key_values=cache, use_cache=True)
        outs.append(o.logits[:, -1].float())
        pos = n0
        for n in steps:
            o = model(ids[:, pos:pos + n], past_key_values=cache, use_cache=True)
            outs.append(o.logits.float())
            pos += n
    return outs


def test_preallocated_cache_gives_the_logits_of_dynamic_cache_and_never_recopies():
    print("\n[case] PreallocatedCache vs DynamicCache", flush=True)
    cfg, model = _model()
    ids = torch.randint(0, cfg.vocab_size, (2, 300), generator=torch.Generator().manual_seed(1)).to(DEV)
    steps = [1, 1, 7, 1, 1]
    want = _decode(model, ids, DynamicCache(), steps)
    hl.reset_usa(model)
    cache = PreallocatedCache(capacity=512)
    got = _decode(model, ids, cache, steps)
    for g, w in zip(got, want):
        assert torch.equal(g, w)
    layer = cache.layers[0]
    assert isinstance(layer, PreallocatedLayer) and layer.capacity == 512 and cache.get_seq_length() == 300
    assert layer.keys.shape[2] == 300 and layer.keys.data_ptr() == layer._kbuf.data_ptr()
    # the buffer never moved: appends were in place
    ptr = layer._kbuf.data_ptr()
    with torch.no_grad():
        model(ids[:, :1], past_key_values=cache, use_cache=True)
    assert layer._kbuf.data_ptr() == ptr and cache.get_seq_length() == 301
    # outgrowing the capacity doubles it and keeps the content
    small = PreallocatedCache(capacity=0)
    hl.reset_usa(model)
    got2 = _decode(model, ids, small, steps)
    for g, w in zip(got2, want):
        assert torch.equal(g, w)
    assert small.layers[0].capacity >= 300
    # cropping forgets tokens without touching the buffer; the bit-cache follows (same cache object, shorter)
    cache.crop(-2)
    assert cache.get_seq_length() == 299 and cache.layers[1].keys.shape[2] == 299


def test_generate_with_a_preallocated_cache_gives_the_same_tokens():
    print("\n[case] generate() with PreallocatedCache", flush=True)
    cfg, model = _model()
    ids = torch.randint(0, cfg.vocab_size, (2, 140), generator=torch.Generator().manual_seed(2)).to(DEV)
    kw = dict(max_new_tokens=12, do_sample=False, pad_token_id=0)
    want = model.generate(ids, past_key_values=DynamicCache(), **kw)
    hl.reset_usa(model)
    got = model.generate(ids, past_key_values=PreallocatedCache(capacity=160), **kw)
    assert torch.equal(got, want)


def test_static_cache_under_the_patched_layers():
    # StaticCache.update returns its whole buffer: the layer must take the number of valid tokens from the cache
    print("\n[case] StaticCache under the patched layers", flush=True)
    cfg, model = _model()
    ids = torch.randint(0, cfg.vocab_size, (2, 200), generator=torch.Generator().manual_seed(3)).to(DEV)
    steps = [1, 1, 1]
    want = _decode(model, ids, DynamicCache(), steps)
    hl.reset_usa(model)
    got = _decode(model, ids, StaticCache(config=cfg, max_cache_len=256), steps)
    for g, w in zip(got[1:], want[1:]):             # decode steps (the prefill's dense attention sees a padded buffer either way)
        assert (g - w).abs().max().item() < 2e-2, (g - w).abs().max().item()


@pytest.mark.parametrize("whole_layer", [False, True])
def test_single_token_steps_in_five_launches_match_the_general_path(whole_layer):
    # on a PreallocatedCache a bf16 model's single-token steps run as fused QKV projection, rotary + in-place append + hashes,
    # histograms, select-attend, output projection; the general path (library projections, torch rotary embedding,
    # cache.update) must give the same logits up to bf16 rounding of different summation orders, and the same greedy tokens.
    # whole_layer: the decoder layer around the attention module in the same style (norms and residuals inside the
    # projections, stacked gate/up projection with SwiGLU behind it): seven launches per layer
    print(f"\n[case] five-launch single-token path vs general path, whole layer: {whole_layer}", flush=True)
    # the whole-layer path keeps the roundings of the modules it replaces (two per RMSNorm, the projection's before a residual is
    # added), so queries, keys and with them the selected tokens are those of the general path
    cfg, model = _model(fast_decode=False)
    for layer in model.model.layers:
        layer.self_attn.fast_layer = whole_layer
    ids = torch.randint(0, cfg.vocab_size, (3, 260), generator=torch.Generator().manual_seed(4)).to(DEV)
    steps = [1, 1, 1, 6, 1, 1]                  # single tokens, a chunk (general path), single tokens again
    want = _decode(model, ids, PreallocatedCache(capacity=300), steps)
    hl.reset_usa(model)
    for layer in model.model.layers:
        layer.self_attn.fast_decode = True
        assert "_fast_scratch" not in layer.self_attn.__dict__
    cache = PreallocatedCache(capacity=300)
    got = _decode(model, ids, cache, steps)
    assert all("_fast_scratch" in layer.self_attn.__dict__ for layer in model.model.layers), "the fast path was not taken"
    assert all(("_fast_act" in layer.self_attn.__dict__) == whole_layer for layer in model.model.layers)
    assert cache.get_seq_length() == 260 and cache.layers[0].keys.shape[2] == 260
    worst = max((g - w).abs().max().item() for g, w in zip(got, want))
    scale = max(w.abs().max().item() for w in want)
    print(f"max-abs logit difference {worst:.3e} (largest logit {scale:.2f})", flush=True)
    assert worst <= 3e-2 * max(scale, 1.0)
    # the keys the fused launch rotated and appended equal the ones torch rotated, bit for bit (same roundings)
    ref_cache = PreallocatedCache(capacity=300)
    for layer in model.model.layers:
        layer.self_attn.fast_decode = False
    hl.reset_usa(model)
    with torch.no_grad():
        model(ids[:, :200], past_key_values=ref_cache, use_cache=True)
        model(ids[:, 200:201], past_key_values=ref_cache, use_cache=True)
    fast_cache = PreallocatedCache(capacity=300)
    for layer in model.model.layers:
        layer.self_attn.fast_decode = True
    hl.reset_usa(model)
    with torch.no_grad():
        model(ids[:, :200], past_key_values=fast_cache, use_cache=True)
        model(ids[:, 200:201], past_key_values=fast_cache, use_cache=True)
    k_ref, k_fast = ref_cache.layers[0].keys[:, :, 200], fast_cache.layers[0].keys[:, :, 200]
    v_ref, v_fast = ref_cache.layers[0].values[:, :, 200], fast_cache.layers[0].values[:, :, 200]
    # layer 0 sees the same hidden states on both paths; its projections differ by summation order only
    assert (k_ref.float() - k_fast.float()).abs().max().item() <= 2e-2 and (v_ref.float() - v_fast.float()).abs().max().item() <= 2e-2
    # greedy generation: same tokens
    kw = dict(max_new_tokens=10, do_sample=False, pad_token_id=0)
    hl.reset_usa(model)
    fast_tokens = model.generate(ids[:, :150], past_key_values=PreallocatedCache(capacity=200), **kw)
    for layer in model.model.layers:
        layer.self_attn.fast_decode = False
    hl.reset_usa(model)
    slow_tokens = model.generate(ids[:, :150], past_key_values=PreallocatedCache(capacity=200), **kw)
    assert torch.equal(fast_tokens, slow_tokens)


def test_rope_encode_step_with_cos_sin_tables_matches_torch_bit_for_bit():
    # ha_rope_encode_step_cos_sin against transformers' apply_rotary_pos_emb on the same bf16 rows (products and sum rounded
    # alike), the in-place cache append, and the two hashes against ha_encode_step on the rotated rows
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    from hashattention import _ops
    from hashattention.synthetic import make_usa_weights
    from tests.parity_util import small_workload
    print("\n[case] ha_rope_encode_step_cos_sin", flush=True)
    B, H, Hkv, cap, pos = 3, 8, 2, 40, 17
    g = torch.Generator().manual_seed(8)
    w = small_workload(batch=B, seq_lens=[cap] * B, n_q_heads=H, n_kv_heads=Hkv, n_code_heads=Hkv, seed=5)
    usa = make_usa_weights(w)
    wk, wq = _ops.pack_usa_weights(usa.k, DEV), _ops.pack_usa_weights(usa.q, DEV)
    qkv = torch.randn(B, (H + 2 * Hkv) * 128, generator=g).bfloat16().to(DEV)
    ang = torch.rand(B, 64, generator=g) * 6.28
    cos = torch.cat([ang.cos(), ang.cos()], -1).bfloat16().to(DEV)          # [B, 128], as rotary_emb builds them
    sin = torch.cat([ang.sin(), ang.sin()], -1).bfloat16().to(DEV)
    kc = torch.full((B, Hkv, cap, 128), 7.0, dtype=torch.bfloat16, device=DEV)
    vc = torch.full((B, Hkv, cap, 128), 7.0, dtype=torch.bfloat16, device=DEV)
    q_out = torch.empty(B, H, 128, dtype=torch.bfloat16, device=DEV)
    kcodes = torch.zeros(B, Hkv, cap, 1, dtype=torch.int32, device=DEV)
    qcodes = torch.zeros(B, H, 1, 1, dtype=torch.int32, device=DEV)
    _ops.rope_encode_step_cos_sin(qkv, H, Hkv, pos, cos, sin, q_out, kc, vc, wk, wq, 3, 128, 32, kcodes, qcodes)
    q = qkv[:, :H * 128].view(B, 1, H, 128).transpose(1, 2)
    k = qkv[:, H * 128:(H + Hkv) * 128].view(B, 1, Hkv, 128).transpose(1, 2)
    v = qkv[:, (H + Hkv) * 128:].view(B, Hkv, 128)
    q_ref, k_ref = apply_rotary_pos_emb(q, k, cos[:, None, :], sin[:, None, :])
    assert torch.equal(q_out, q_ref[:, :, 0]) and torch.equal(kc[:, :, pos], k_ref[:, :, 0]) and torch.equal(vc[:, :, pos], v)
    untouched = torch.ones(cap, dtype=torch.bool)
    untouched[pos] = False
    assert (kc[:, :, untouched] == 7.0).all() and (vc[:, :, untouched] == 7.0).all()
    kcodes2 = torch.zeros_like(kcodes)
    qcodes2 = torch.zeros_like(qcodes)
    _ops.encode_step(k_ref.contiguous(), q_ref[:, :, 0].contiguous(), wk, wq, 3, 128, 32, kcodes2, qcodes2, pos0=pos)
    assert torch.equal(kcodes, kcodes2) and torch.equal(qcodes, qcodes2)
    # one table row shared by the batch (stride 0)
    q_out2 = torch.empty_like(q_out)
    _ops.rope_encode_step_cos_sin(qkv, H, Hkv, pos + 1, cos[:1], sin[:1], q_out2, kc, vc, wk, wq, 3, 128, 32, kcodes, qcodes)
    q_ref2, _ = apply_rotary_pos_emb(q, k, cos[:1, None, :], sin[:1, None, :])
    assert torch.equal(q_out2, q_ref2[:, :, 0])


def test_mistral_takes_the_five_launch_step_too():
    from transformers import MistralConfig, MistralForCausalLM
    from hashattention import hashattention_mistral as hm
    print("\n[case] five-launch single-token path and whole-layer path, Mistral", flush=True)
    torch.manual_seed(0)
    cfg = _config(MistralConfig, sliding_window=None)
    model = MistralForCausalLM(cfg).bfloat16().to(DEV)
    model = hm.convert_usa(model, cfg, hm.load_usa(cfg, None), collect_stats=False, train_usa=False)
    ids = torch.randint(0, cfg.vocab_size, (2, 220), generator=torch.Generator().manual_seed(6)).to(DEV)
    steps = [1, 1, 1]
    for layer in model.model.layers:
        layer.self_attn.fast_decode = False
    want = _decode(model, ids, PreallocatedCache(capacity=256), steps)
    hm.reset_usa(model)
    for layer in model.model.layers:
        layer.self_attn.fast_decode = True
    got = _decode(model, ids, PreallocatedCache(capacity=256), steps)
    assert all("_fast_scratch" in layer.self_attn.__dict__ and "_fast_act" in layer.self_attn.__dict__ for layer in model.model.layers)
    worst = max((g - w).abs().max().item() for g, w in zip(got, want))
    scale = max(w.abs().max().item() for w in want)
    assert worst <= 3e-2 * max(scale, 1.0), (worst, scale)


@pytest.mark.parametrize("kind", ["dynamic", "preallocated", "preallocated_fast"])
def test_reordering_the_cache_between_steps_drops_the_stale_codes(kind):
    # beam search permutes, selects and repeats batch entries of the cache between two steps (`Cache.reorder_cache`): the codes
    # the layers keep for the cached keys then belong to other rows.  The reference re-hashes every key at every step; here the
    # layers notice that the cache's key storage is no longer the one they left and hash the cache afresh.
    print(f"\n[case] cache reordered between steps, {kind}", flush=True)
    cfg, model = _model(fast_decode=kind.endswith("fast"))
    make = (lambda: DynamicCache()) if kind == "dynamic" else (lambda: PreallocatedCache(capacity=400))
    ids = torch.randint(0, cfg.vocab_size, (3, 264), generator=torch.Generator().manual_seed(5)).to(DEV)
    perm = torch.tensor([2, 0, 0], device=DEV)          # a permutation with a repeat, as beams do
    with torch.no_grad():
        # the run to compare with: the reordered batch from the start
        want_cache = make()
        model(ids[perm, :260], past_key_values=want_cache, use_cache=True)
        want = [model(ids[perm, 260 + i:261 + i], past_key_values=want_cache, use_cache=True).logits.float() for i in range(4)]
        hl.reset_usa(model)
        cache = make()
        model(ids[:, :260], past_key_values=cache, use_cache=True)
        for i in range(2):                              # two steps in the original order fill the bit-cache
            model(ids[:, 260 + i:261 + i], past_key_values=cache, use_cache=True)
        cache.crop(-2)
        cache.reorder_cache(perm)
        got = [model(ids[perm, 260 + i:261 + i], past_key_values=cache, use_cache=True).logits.float() for i in range(4)]
    for g, w in zip(got, want):
        assert torch.equal(g, w), (g - w).abs().max().item()


@pytest.mark.parametrize("kind", ["dynamic", "preallocated_fast"])
def test_beam_search_gives_the_tokens_of_a_run_that_rehashes_every_step(kind):
    # generate() with beams reorders the cache at every step.  The run to compare with forgets its codes before every forward
    # pass (`reset_usa`), which is what the reference does by construction (it hashes every cached key at every step).
    print(f"\n[case] beam search, {kind}", flush=True)
    cfg, model = _model(fast_decode=kind.endswith("fast"))
    make = (lambda: DynamicCache()) if kind == "dynamic" else (lambda: PreallocatedCache(capacity=256))
    ids = torch.randint(0, cfg.vocab_size, (2, 150), generator=torch.Generator().manual_seed(6)).to(DEV)
    kw = dict(max_new_tokens=10, do_sample=False, num_beams=3, pad_token_id=0)
    def forget(module, args):
        hl.reset_usa(module)            # (a pre-hook's return value would replace the arguments)

    hook = model.register_forward_pre_hook(forget)
    try:
        want = model.generate(ids, past_key_values=make(), **kw)
    finally:
        hook.remove()
    hl.reset_usa(model)
    got = model.generate(ids, past_key_values=make(), **kw)
    assert torch.equal(got, want)


def test_hooks_on_the_layers_modules_keep_the_librarys_decoder_layer():
    # the whole-layer path calls neither `mlp.forward` nor the norms: a forward hook on one of them must keep firing
    print("\n[case] forward hook on the MLP of a converted layer", flush=True)
    cfg, model = _model(fast_decode=True)
    ids = torch.randint(0, cfg.vocab_size, (2, 150), generator=torch.Generator().manual_seed(7)).to(DEV)
    cache = PreallocatedCache(capacity=200)
    seen = []
    hook = model.model.layers[1].mlp.register_forward_hook(lambda m, a, o: seen.append(o.shape))
    with torch.no_grad():
        model(ids[:, :140], past_key_values=cache, use_cache=True)
        model(ids[:, 140:141], past_key_values=cache, use_cache=True)
    assert len(seen) == 2 and seen[1] == (2, 1, cfg.hidden_size)
    assert "_fast_act" in model.model.layers[0].self_attn.__dict__ and "_fast_act" not in model.model.layers[1].self_attn.__dict__
    hook.remove()
    with torch.no_grad():
        model(ids[:, 141:142], past_key_values=cache, use_cache=True)
    assert len(seen) == 2 and "_fast_act" in model.model.layers[1].self_attn.__dict__


def test_ops_launch_on_torchs_current_stream():
    # the binding takes the current stream's raw handle from torch without building a Stream object per launch
    from hashattention import _ops
    t = torch.zeros(1, device=DEV)
    assert (_ops._stream(t) or 0) == torch.cuda.current_stream(DEV).cuda_stream
    side = torch.cuda.Stream(device=DEV)
    with torch.cuda.stream(side):
        assert _ops._stream(t) == side.cuda_stream
    assert (_ops._stream(t) or 0) == torch.cuda.current_stream(DEV).cuda_stream


@pytest.mark.parametrize("fast", [False, True])
def test_a_cache_that_generate_made_itself_is_taken_over_in_place(fast):
    # nothing but `model.generate(ids)`, as the reference's README runs it: transformers creates a DynamicCache, whose layers
    # re-copy their whole cache per token; at the first decode step every converted attention module turns its layer of that
    # cache into one that appends in place (same object, same tensors).  Same tokens as with the library's own layers.
    print(f"\n[case] DynamicCache adopted in place, few-launch steps: {fast}", flush=True)
    cfg, model = _model(fast_decode=fast, adopt_cache=False)
    ids = torch.randint(0, cfg.vocab_size, (2, 150), generator=torch.Generator().manual_seed(8)).to(DEV)
    kw = dict(max_new_tokens=12, do_sample=False, pad_token_id=0, return_dict_in_generate=True)
    want = model.generate(ids, **kw)
    from transformers.cache_utils import DynamicLayer
    assert all(type(l) is DynamicLayer for l in want.past_key_values.layers)
    for layer in model.model.layers:
        layer.self_attn.adopt_cache = True
    hl.reset_usa(model)
    got = model.generate(ids, **kw)
    assert torch.equal(got.sequences, want.sequences)
    cache = got.past_key_values
    assert type(cache) is DynamicCache and all(isinstance(l, PreallocatedLayer) for l in cache.layers)
    assert cache.get_seq_length() == 150 + 12 - 1 and cache.layers[0].capacity > cache.get_seq_length()
    # (the few-launch steps differ from the general path by bf16 roundings of other summation orders)
    close = (lambda x, y: torch.equal(x, y)) if not fast else (lambda x, y: (x.float() - y.float()).abs().max().item() <= 3e-2)
    assert close(cache.layers[1].keys, want.past_key_values.layers[1].keys)
    # the caller's own DynamicCache, continued over two calls, cropped and reordered in between
    own = DynamicCache()
    with torch.no_grad():
        model(ids[:, :140], past_key_values=own, use_cache=True)
        a = model(ids[:, 140:141], past_key_values=own, use_cache=True).logits
        assert isinstance(own.layers[0], PreallocatedLayer)
        ptr = own.layers[0]._kbuf.data_ptr()
        model(ids[:, 141:142], past_key_values=own, use_cache=True)
        assert own.layers[0]._kbuf.data_ptr() == ptr            # appended in place
        own.crop(-1)
        own.reorder_cache(torch.tensor([1, 0], device=DEV))
        b = model(ids[[1, 0], 141:142], past_key_values=own, use_cache=True).logits
    ref = DynamicCache()
    for layer in model.model.layers:
        layer.self_attn.adopt_cache = False
    hl.reset_usa(model)
    with torch.no_grad():
        model(ids[:, :140], past_key_values=ref, use_cache=True)
        a_ref = model(ids[:, 140:141], past_key_values=ref, use_cache=True).logits
        ref.reorder_cache(torch.tensor([1, 0], device=DEV))
        b_ref = model(ids[[1, 0], 141:142], past_key_values=ref, use_cache=True).logits
    assert close(a, a_ref) and close(b, b_ref)


def test_a_left_padded_batch_takes_the_few_launch_steps_too():
    # batched generation pads prompts on the left: the attention mask then matters (reference :593-598 adds it before the
    # softmax), the step keeps its few launches and attends through the masked gather; against the general path
    print("\n[case] left-padded batch through the few-launch steps", flush=True)
    cfg, model = _model(fast_decode=False)
    g = torch.Generator().manual_seed(9)
    ids = torch.randint(1, cfg.vocab_size, (3, 200), generator=g).to(DEV)
    am = torch.ones(3, 200, dtype=torch.long, device=DEV)
    am[1, :37] = 0
    am[2, :150] = 0
    kw = dict(max_new_tokens=10, do_sample=False, pad_token_id=0, attention_mask=am)
    want = model.generate(ids, past_key_values=PreallocatedCache(capacity=256), **kw)
    hl.reset_usa(model)
    for layer in model.model.layers:
        layer.self_attn.fast_decode = True
    got = model.generate(ids, past_key_values=PreallocatedCache(capacity=256), **kw)
    assert all("_fast_act" in layer.self_attn.__dict__ for layer in model.model.layers), "the few-launch step was not taken"
    assert torch.equal(got, want)
    with torch.no_grad():                       # one step's logits
        outs = []
        for fast in (False, True):
            hl.reset_usa(model)
            for layer in model.model.layers:
                layer.self_attn.fast_decode = fast
            cache = PreallocatedCache(capacity=256)
            model(ids[:, :199], attention_mask=am[:, :199], past_key_values=cache, use_cache=True)
            outs.append(model(ids[:, 199:], attention_mask=am, past_key_values=cache, use_cache=True).logits.float())
    assert (outs[0] - outs[1]).abs().max().item() <= 3e-2 * max(1.0, outs[0].abs().max().item())


def test_whole_layer_step_with_an_mlp_wider_than_the_row_streaming_kernel_takes():
    # intermediate size above 16384 (Llama-3.1-70B has 28672): the down projection's rows are too long for the row-streaming
    # form of the projection kernel and take its matrix-core form; the layer still runs in seven launches
    print("\n[case] whole-layer step, intermediate size 16512", flush=True)
    torch.manual_seed(0)
    cfg = _config(LlamaConfig)
    cfg.intermediate_size = 16512
    model = LlamaForCausalLM(cfg).bfloat16().to(DEV)
    model = hl.convert_usa(model, cfg, hl.load_usa(cfg, None), collect_stats=False, train_usa=False)
    ids = torch.randint(0, cfg.vocab_size, (2, 203), generator=torch.Generator().manual_seed(11)).to(DEV)
    outs = []
    for fast in (False, True):
        hl.reset_usa(model)
        for layer in model.model.layers:
            layer.self_attn.fast_decode = fast
        outs.append(_decode(model, ids, PreallocatedCache(capacity=256), [1, 1, 1]))
    assert all("_fast_act" in layer.self_attn.__dict__ for layer in model.model.layers)
    worst = max((g - w).abs().max().item() for g, w in zip(outs[1], outs[0]))
    scale = max(w.abs().max().item() for w in outs[0])
    assert worst <= 3e-2 * max(scale, 1.0), (worst, scale)


@pytest.mark.parametrize("shape", ["three_per_kv", "yarn", "heads_narrower_than_hidden"])
def test_few_launch_steps_on_other_model_shapes(shape):
    # 6 query heads on 2 KV heads (Llama-3.2-3B has 24 on 8); a rotary embedding that scales its cos/sin (yarn: the step takes
    # the tables the model hands over): the seven-launch layer against the general path
    print(f"\n[case] whole-layer step, {shape}", flush=True)
    torch.manual_seed(0)
    if shape == "three_per_kv":
        cfg = _config(LlamaConfig, hidden_size=768, num_attention_heads=6)
    elif shape == "heads_narrower_than_hidden":     # Mistral-Nemo: 32 heads of 128 on a hidden size of 5120
        cfg = _config(LlamaConfig, hidden_size=640)
    else:
        cfg = _config(LlamaConfig, rope_parameters=dict(rope_type="yarn", factor=4.0, original_max_position_embeddings=1024,
                                                        rope_theta=10000.0))
    model = LlamaForCausalLM(cfg).bfloat16().to(DEV)
    model = hl.convert_usa(model, cfg, hl.load_usa(cfg, None), collect_stats=False, train_usa=False)
    ids = torch.randint(0, cfg.vocab_size, (3, 230), generator=torch.Generator().manual_seed(12)).to(DEV)
    outs = []
    for fast in (False, True):
        hl.reset_usa(model)
        for layer in model.model.layers:
            layer.self_attn.fast_decode = fast
        outs.append(_decode(model, ids, PreallocatedCache(capacity=256), [1, 1, 4, 1]))
    assert all("_fast_act" in layer.self_attn.__dict__ for layer in model.model.layers)
    worst = max((g - w).abs().max().item() for g, w in zip(outs[1], outs[0]))
    scale = max(w.abs().max().item() for w in outs[0])
    assert worst <= 3e-2 * max(scale, 1.0), (worst, scale)


@pytest.mark.parametrize("batch,whole_layer", [(18, False), (18, True), (12, True), (12, False), (9, True), (40, True)])
def test_few_call_steps_with_more_sequences_than_the_fused_projections_take(batch, whole_layer):
    # 18 sequences: the attention module keeps its five-call step (the library's GEMM on the stacked QKV weight and on the
    # output projection, the rotary/append/hash launch, histograms, select-attend).  The decoder layer around it: the library's
    # own, or (whole_layer, the default) twelve calls - one launch per RMSNorm with the module's roundings, one GEMM on the
    # stacked gate/up weight, one SwiGLU launch.  12 sequences: the same with the projection kernel's matrix-core form inside
    # the attention step.
    print(f"\n[case] few-call steps, {batch} sequences, whole layer: {whole_layer}", flush=True)
    cfg, model = _model(fast_decode=False)
    ids = torch.randint(0, cfg.vocab_size, (batch, 140), generator=torch.Generator().manual_seed(13)).to(DEV)
    outs = []
    for fast in (False, True):
        hl.reset_usa(model)
        for layer in model.model.layers:
            layer.self_attn.fast_decode = fast
            layer.self_attn.fast_layer = whole_layer
            layer.self_attn.__dict__.pop("_fast_scratch", None)
        outs.append(_decode(model, ids, PreallocatedCache(capacity=160), [1, 1, 3, 1]))
    assert all("_fast_scratch" in layer.self_attn.__dict__ and ("_fast_act" in layer.self_attn.__dict__) == whole_layer
               for layer in model.model.layers)
    worst = max((g - w).abs().max().item() for g, w in zip(outs[1], outs[0]))
    scale = max(w.abs().max().item() for w in outs[0])
    assert worst <= 3e-2 * max(scale, 1.0), (worst, scale)


def test_a_wrapper_around_a_projection_keeps_its_say():
    # adapter libraries replace nn.Linear projections by wrappers with a forward of their own: the few-launch steps read
    # weights directly, so they step aside for such a module (its output must show in the logits) and come back when it is gone
    print("\n[case] projections wrapped after convert_usa", flush=True)

    class Shifted(torch.nn.Module):
        def __init__(self, base):
            super().__init__()
            self.base_layer = base
            self.weight, self.bias = base.weight, base.bias       # as adapter wrappers expose them

        def forward(self, x):
            return self.base_layer(x) + 0.5

    cfg, model = _model(fast_decode=True)
    ids = torch.randint(0, cfg.vocab_size, (2, 180), generator=torch.Generator().manual_seed(12)).to(DEV)

    def step_logits():
        hl.reset_usa(model)
        cache = PreallocatedCache(capacity=256)
        with torch.no_grad():
            model(ids[:, :179], past_key_values=cache, use_cache=True)
            return model(ids[:, 179:], past_key_values=cache, use_cache=True).logits.float()

    plain = step_logits()
    for where, name in ((model.model.layers[0].mlp, "down_proj"), (model.model.layers[1].self_attn, "q_proj")):
        base = getattr(where, name)
        setattr(where, name, Shifted(base))
        for layer in model.model.layers:
            layer.self_attn.fast_decode = True
        got = step_logits()
        for layer in model.model.layers:
            layer.self_attn.fast_decode = False
        want = step_logits()
        assert (got - want).abs().max().item() <= 3e-2 * max(1.0, want.abs().max().item()), name
        assert (got - plain).abs().max().item() > 10 * (got - want).abs().max().item(), name      # the wrapper was heard
        setattr(where, name, base)
    for layer in model.model.layers:
        layer.self_attn.fast_decode = True
        layer.self_attn.__dict__.pop("_fast_act", None)
    again = step_logits()
    assert all("_fast_act" in layer.self_attn.__dict__ for layer in model.model.layers)
    assert (again - plain).abs().max().item() <= 3e-2 * max(1.0, plain.abs().max().item())

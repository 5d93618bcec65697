"""The drop-in boundary on a GPU: `load_usa` / `convert_usa` / `reset_usa` on tiny random-init Llama and Mistral
models, prefill through the original forward and decode steps through the HIP path, against the same model on
the CPU whose attention layers run the oracle's restatement of the reference decode branch
(hashattention/hashattention_llama.py:551-631).  fp32 everywhere so the comparison is tight."""
import copy
import types

import pytest
import torch
from transformers import DynamicCache, LlamaConfig, LlamaForCausalLM, MistralConfig, MistralForCausalLM

from hashattention import hashattention_llama as hl
from hashattention import hashattention_mistral as hm
from oracle import hashattn_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

USA_CFG = dict(lth_init_dim=128, lth_final_dim=32, lth_thold=0, lth_num_layers=3, init_budget=8, heavy_budget=0.125,
               recent_budget=8, usa_retrieve_depth=6, usa_eval_mode="simple")


def _config(cls, **kw):
    shape = dict(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                 head_dim=128, vocab_size=512, max_position_embeddings=4096)
    shape.update(kw)
    cfg = cls(**shape)
    for k, v in USA_CFG.items():
        setattr(cfg, k, v)
    return cfg


def _oracle_forward(layer, usa, cfg, apply_rope, **variant):
    """CPU restatement of the reference's patched forward, bound to an unpatched attention layer.  `variant`: center=True
    or lsh=True for the hash variants whose inputs depend on the whole cache."""
    orig = layer.forward
    k_heads = [[(m.weight.detach().float().cpu(), m.bias.detach().float().cpu()) for m in seq if isinstance(m, torch.nn.Linear)]
               for seq in usa.learning_to_hash_transformation_k]
    q_heads = [[(m.weight.detach().float().cpu(), m.bias.detach().float().cpu()) for m in seq if isinstance(m, torch.nn.Linear)]
               for seq in usa.learning_to_hash_transformation_q]

    def forward(self, hidden_states, position_embeddings=None, attention_mask=None, past_key_values=None, **kwargs):
        b, q_len, _ = hidden_states.shape
        if q_len > 128:
            return orig(hidden_states=hidden_states, position_embeddings=position_embeddings, attention_mask=attention_mask,
                        past_key_values=past_key_values, **kwargs)
        shape = (b, q_len, -1, self.head_dim)
        q = self.q_proj(hidden_states).view(shape).transpose(1, 2)
        k = self.k_proj(hidden_states).view(shape).transpose(1, 2)
        v = self.v_proj(hidden_states).view(shape).transpose(1, 2)
        cos, sin = position_embeddings
        q, k = apply_rope(q, k, cos, sin)
        k, v = past_key_values.update(k, v, self.layer_idx)
        add = attention_mask            # added to the scores (reference :593-598); the library may hand it over as booleans
        if add is not None:
            add = add[..., :k.shape[2]]
            if add.dtype == torch.bool:
                add = torch.zeros(add.shape, dtype=q.dtype).masked_fill_(~add, float("-inf"))
        out, _ = orc.reference_decode_attention(q, k, v, k_heads, q_heads, cfg.init_budget, cfg.recent_budget, cfg.heavy_budget,
                                                attention_mask=add, **variant)
        return self.o_proj(out.transpose(1, 2).reshape(b, q_len, -1)), None

    layer.forward = types.MethodType(forward, layer)


def _run(model, ids, steps, make_cache=DynamicCache):
    cache = make_cache()
    outs = []
    with torch.no_grad():
        o = model(ids[:, :-sum(steps)], past_key_values=cache, use_cache=True)
        outs.append(o.logits[:, -1].float().cpu())
        pos = ids.shape[1] - sum(steps)
        for n in steps:
            o = model(ids[:, pos:pos + n], past_key_values=cache, use_cache=True)
            outs.append(o.logits.float().cpu())
            pos += n
    return outs


@pytest.mark.parametrize("family", ["llama", "mistral", "llama_3_per_kv", "llama_bias_yarn"])
def test_patched_model_matches_reference_semantics(family):
    print(f"\n[case] model api {family}", flush=True)
    torch.manual_seed(0)
    if family == "llama":
        cfg, model_cls, api = _config(LlamaConfig), LlamaForCausalLM, hl
    elif family == "llama_3_per_kv":    # three query heads per KV head (Llama-3.2-3B: 24 on 8)
        cfg, model_cls, api = _config(LlamaConfig, hidden_size=768, num_attention_heads=6), LlamaForCausalLM, hl
        family = "llama"
    elif family == "llama_bias_yarn":   # projections with biases, cos/sin scaled by the rotary embedding (yarn's attention factor)
        cfg = _config(LlamaConfig, attention_bias=True, mlp_bias=True,
                      rope_parameters=dict(rope_type="yarn", factor=4.0, original_max_position_embeddings=1024, rope_theta=10000.0))
        model_cls, api, family = LlamaForCausalLM, hl, "llama"
    else:
        cfg, model_cls, api = _config(MistralConfig, sliding_window=None), MistralForCausalLM, hm
    model = model_cls(cfg).bfloat16().float()           # bf16-representable weights: convert_usa's bf16 cast is then lossless
    ref = copy.deepcopy(model)

    usa = api.load_usa(cfg, None)                        # random-init hash modules, on the GPU
    assert next(usa.parameters()).is_cuda
    model = api.convert_usa(model.to(DEV), cfg, usa, collect_stats=False, train_usa=False)
    patched = model.model.layers[0].self_attn
    assert type(patched).__name__.endswith("_heavy_hitter") and patched.q_proj.weight.dtype == torch.bfloat16
    model = model.float()                                # the reference converts to bf16; compare in fp32 instead

    rope = __import__(f"transformers.models.{family}.modeling_{family}", fromlist=["apply_rotary_pos_emb"]).apply_rotary_pos_emb
    for li, layer in enumerate(ref.model.layers):
        _oracle_forward(layer.self_attn, usa[li], cfg, rope)

    ids = torch.randint(0, cfg.vocab_size, (2, 200 + 1 + 1 + 5 + 1), generator=torch.Generator().manual_seed(1))
    steps = [1, 1, 5, 1]                                 # single-token steps and one 5-token chunk (q_len <= 128 branch)
    got = _run(model, ids.to(DEV), steps)
    want = _run(ref, ids, steps)
    for g, w in zip(got, want):
        assert g.shape == w.shape
        err = (g - w).abs().max().item()
        assert err < 2e-3, err

    # a new prompt after reset_usa starts from an empty bit-cache
    api.reset_usa(model)
    assert model.model.layers[0].self_attn._hash_layer.n_cached == 0
    got2 = _run(model, ids.to(DEV), steps)
    for g, g2 in zip(got, got2):
        assert torch.equal(g, g2)


def test_mistral_sliding_window_cache():
    # A Mistral configuration with a sliding window: the library's cache (what `generate` builds from the configuration) keeps
    # the last window - 1 tokens only, so every decode step sees a window whose first token moved.  The reference's patched
    # forward attends to whatever the cache returns (hashattention_mistral.py has no sliding-window logic of its own); so does
    # this one, re-hashing the window each step.
    print("\n[case] model api mistral, sliding-window cache", flush=True)
    torch.manual_seed(0)
    cfg = _config(MistralConfig, sliding_window=48)
    model = MistralForCausalLM(cfg).bfloat16().float()
    ref = copy.deepcopy(model)
    usa = hm.load_usa(cfg, None)
    model = hm.convert_usa(model.to(DEV), cfg, usa, collect_stats=False, train_usa=False).float()
    rope = __import__("transformers.models.mistral.modeling_mistral", fromlist=["apply_rotary_pos_emb"]).apply_rotary_pos_emb
    for li, layer in enumerate(ref.model.layers):
        _oracle_forward(layer.self_attn, usa[li], cfg, rope)
    ids = torch.randint(0, cfg.vocab_size, (2, 150 + 1 + 1 + 3 + 1 + 1), generator=torch.Generator().manual_seed(4))
    steps = [1, 1, 3, 1, 1]
    seen = []

    def make():
        seen.append(DynamicCache(config=cfg))
        return seen[-1]
    got = _run(model, ids.to(DEV), steps, make)
    assert type(seen[0].layers[0]).__name__ == "DynamicSlidingWindowLayer" and seen[0].layers[0].keys.shape[2] == 47
    want = _run(ref, ids, steps, make)
    for g, w in zip(got, want):
        assert g.shape == w.shape
        err = (g - w).abs().max().item()
        print(f"  step rows {tuple(g.shape)}: max err {err:.2e}", flush=True)
        assert err < 2e-3, err
    # the same through generate, which builds that cache itself
    out = model.generate(ids[:, :150].to(DEV), max_new_tokens=6, do_sample=False, pad_token_id=0)
    assert out.shape == (2, 156)


def test_usa_forward_and_mask_api():
    # USA.forward / k_embedding and compute_mask_multi keep the reference's shapes and meaning
    print("\n[case] USA.forward / compute_mask_multi", flush=True)
    torch.manual_seed(3)
    cfg = _config(LlamaConfig)
    usa = hl.load_usa(cfg, None)[0]
    K = torch.randn(1, 2, 300, 128, device=DEV).repeat_interleave(2, dim=1)   # repeat_kv'd keys, as the reference passes them
    Q = torch.randn(1, 4, 3, 128, device=DEV)
    span, ksign = usa(K, Q, hard=True)
    k_heads = [[(m.weight.detach().cpu(), m.bias.detach().cpu()) for m in seq if isinstance(m, torch.nn.Linear)]
               for seq in usa.learning_to_hash_transformation_k]
    q_heads = [[(m.weight.detach().cpu(), m.bias.detach().cpu()) for m in seq if isinstance(m, torch.nn.Linear)]
               for seq in usa.learning_to_hash_transformation_q]
    span_ref, ksign_ref = orc.usa_forward_hard(K.cpu(), Q.cpu(), k_heads, q_heads)
    assert torch.equal(span.cpu(), span_ref) and torch.equal(ksign.cpu(), ksign_ref)
    assert torch.equal(usa.k_embedding(K, hard=True).cpu(), ksign_ref)
    with torch.no_grad():
        soft, ktanh = usa(K, Q, hard=False)                   # soft mode: probabilities, zero beyond the causal edge
    soft_ref, ktanh_ref = orc.usa_forward_soft(K.cpu(), Q.cpu(), k_heads, q_heads, cfg.lth_thold)
    assert (soft.cpu() - soft_ref).abs().max().item() < 1e-5 and (ktanh.cpu() - ktanh_ref).abs().max().item() < 1e-5

    layer = hl.LlamaAttention_heavy_hitter(cfg, 0).to(DEV)
    layer.usa_module = usa
    mask = layer.compute_mask_multi(K, Q)
    mask_ref = orc.compute_mask_multi(span_ref, cfg.init_budget, cfg.recent_budget, cfg.heavy_budget)
    assert torch.equal(mask.cpu(), mask_ref)


def test_usa_forward_with_more_query_rows_than_one_scoring_launch_takes():
    # heads * query tokens beyond 65535 (the scoring launch's limit of query "heads"): USA.forward slices the tokens; also a
    # parameter changed through .data (no version bump) followed by invalidate_packed() must reach the kernels
    print("\n[case] USA.forward with 4 x 16500 query rows; invalidate_packed", flush=True)
    torch.manual_seed(5)
    cfg = _config(LlamaConfig)
    usa = hl.load_usa(cfg, None)[0]
    t, s = 16500, 16600
    K = torch.randn(1, 4, s, 128, device=DEV)
    Q = torch.randn(1, 4, t, 128, device=DEV)
    span, _ = usa(K, Q, hard=True)
    assert span.shape == (1, 4, t, s)
    lo = 16384 - 3                                      # rows on both sides of the slice boundary (65535 // 4 = 16383)
    small, _ = usa(K, Q[:, :, lo:lo + 6].contiguous(), hard=True)
    rows = torch.arange(lo, lo + 6)
    causal = torch.arange(s)[None, :] <= (rows[:, None] + s - t)
    # the short call's causal edge sits at other columns: compare the columns both calls score
    both = causal & (torch.arange(s)[None, :] <= (torch.arange(6)[:, None] + s - 6))
    assert torch.equal(span[0, :, lo:lo + 6].cpu()[:, both], small[0].cpu()[:, both])
    before = usa.k_embedding(K[:, :, :64].contiguous(), hard=True).clone()
    with torch.no_grad():
        for seq in usa.learning_to_hash_transformation_k:
            seq[-1].weight.data.neg_()
            seq[-1].bias.data.neg_()
    usa.invalidate_packed()
    after = usa.k_embedding(K[:, :, :64].contiguous(), hard=True)
    assert torch.equal(after, -before)


def test_recall_statistic_matches_the_oracle():
    # collect_stats=True: after a 1024-token prefill every layer holds the recall of its hash ranking (reference :319-398);
    # layer 0 is compared row by row with the oracle on the same queries and keys
    print("\n[case] recall statistic (collect_stats)", flush=True)
    torch.manual_seed(4)
    cfg = _config(LlamaConfig)
    model = LlamaForCausalLM(cfg).bfloat16().float()
    usa = hl.load_usa(cfg, None)
    model = hl.convert_usa(model.to(DEV), cfg, usa, collect_stats=True, train_usa=False).float()
    attn = model.model.layers[0].self_attn
    seen = {}

    def grab(mod, args, kwargs):
        seen["h"] = kwargs["hidden_states"] if "hidden_states" in kwargs else args[0]
        seen["pe"] = kwargs["position_embeddings"]
    hook = attn.register_forward_pre_hook(grab, with_kwargs=True)
    ids = torch.randint(0, cfg.vocab_size, (1, 1024), generator=torch.Generator().manual_seed(2)).to(DEV)
    cache = DynamicCache()
    with torch.no_grad():
        model(ids, past_key_values=cache, use_cache=True)
    hook.remove()
    assert list(attn.overlaps) == [1024] and attn.overlaps[1024][2] == 4 * 1024
    got = attn.last_overlap_ratio.cpu()                                                      # [1, H, q_len]
    rope = __import__("transformers.models.llama.modeling_llama", fromlist=["apply_rotary_pos_emb"]).apply_rotary_pos_emb
    with torch.no_grad():
        q = attn.q_proj(seen["h"]).view(1, 1024, 4, 128).transpose(1, 2)
        q, _ = rope(q, q, *seen["pe"])
    keys = cache.layers[0].keys
    lin = lambda seqs: [[(m.weight.detach().float().cpu(), m.bias.detach().float().cpu()) for m in s if isinstance(m, torch.nn.Linear)]
                        for s in seqs]
    rows = slice(1024 - 96, 1024)                                                            # the oracle is a Python loop: the last 96 rows
    want = orc.recall_overlap(q[:, :, rows].float().cpu(), keys.float().cpu(), lin(usa[0].learning_to_hash_transformation_k),
                              lin(usa[0].learning_to_hash_transformation_q), cfg.init_budget, cfg.recent_budget)
    diff = (got[:, :, rows] - want).abs()
    # a near tie between the 32nd and 33rd true logit may flip with the summation order of the GPU matmul: 1/32 on few rows
    assert diff.max().item() <= 1 / 32 + 1e-6 and (diff > 0).float().mean().item() < 0.05, (diff.max().item(), (diff > 0).float().mean().item())
    assert 0.0 < attn.overlaps[1024][3] <= 1.0
    hl.print_stats(model)


def _greedy(model, prompt, n_new, cache=None):
    """Greedy continuation with a cache of its own (as `generate` makes one per call) unless one is handed in."""
    cache = DynamicCache() if cache is None else cache
    toks = []
    with torch.no_grad():
        logits = model(prompt, past_key_values=cache, use_cache=True).logits[:, -1]
        for _ in range(n_new):
            nxt = logits.argmax(-1, keepdim=True)
            toks.append(nxt)
            logits = model(nxt, past_key_values=cache, use_cache=True).logits[:, -1]
    return torch.cat(toks, dim=1).cpu(), logits.float().cpu()


def test_a_new_prompt_needs_no_reset_usa():
    # The reference keeps no hash state between calls (past_key_signatures stays None, hashattention_llama.py:407-408), and
    # its README never calls reset_usa between prompts.  The bit-cache must therefore notice a new prompt by itself: a
    # longer prompt after a shorter one (the stale codes of the first would otherwise stay in front), a shorter one after a
    # longer one, a short prompt that goes through the q_len <= 128 branch, and a cache object that is rewound and reused.
    print("\n[case] prompts back to back without reset_usa", flush=True)
    torch.manual_seed(0)
    cfg = _config(LlamaConfig)
    model = LlamaForCausalLM(cfg).bfloat16().float()
    usa = hl.load_usa(cfg, None)
    model = hl.convert_usa(model.to(DEV), cfg, usa, collect_stats=False, train_usa=False).float()
    g = torch.Generator().manual_seed(9)
    prompts = [torch.randint(0, cfg.vocab_size, (2, n), generator=g).to(DEV) for n in (200, 500, 150, 60, 300)]
    want = []
    for p in prompts:                              # every prompt from a clean state
        hl.reset_usa(model)
        want.append(_greedy(model, p, 10))
    hl.reset_usa(model)
    for p, (toks, logits) in zip(prompts, want):   # the same prompts back to back, no reset in between
        got_toks, got_logits = _greedy(model, p, 10)
        assert torch.equal(got_toks, toks)
        assert (got_logits - logits).abs().max().item() < 1e-4
    # one cache object, rewound to a prefix and continued with other tokens: the codes of the prefix stay valid, the rest
    # is hashed again
    hl.reset_usa(model)
    cache = DynamicCache()
    _greedy(model, prompts[1], 6, cache)
    assert model.model.layers[0].self_attn._hash_layer.n_cached == 500 + 6
    cache.crop(-106)                                       # drop the last 106 tokens: 400 are left
    tail = prompts[4][:, :150]
    got = _greedy(model, tail, 5, cache)
    assert model.model.layers[0].self_attn._hash_layer.n_cached == 400 + 150 + 5
    hl.reset_usa(model)
    ref = _greedy(model, torch.cat([prompts[1][:, :400], tail], dim=1), 5)
    assert torch.equal(got[0], ref[0])
    assert (got[1] - ref[1]).abs().max().item() < 2e-2      # the prefill was chunked differently (500 | 150 against 550 at once)


def test_attention_weights_are_refused_on_the_decode_branch():
    # the reference returns the weights of its dense product when asked (hashattention_llama.py:615-631); the gather attention
    # never forms them, and says so instead of returning None
    print("\n[case] output_attentions on the decode branch", flush=True)
    torch.manual_seed(0)
    cfg = _config(LlamaConfig)
    model = LlamaForCausalLM(cfg).bfloat16().to(DEV)
    model = hl.convert_usa(model, cfg, hl.load_usa(cfg, None), collect_stats=False, train_usa=False)
    attn = model.model.layers[0].self_attn
    hidden = torch.randn(1, 1, cfg.hidden_size, device=DEV, dtype=torch.bfloat16)
    cos = torch.ones(1, 1, 128, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        out, weights = attn(hidden, position_embeddings=(cos, torch.zeros_like(cos)), past_key_values=DynamicCache())
        assert out.shape == hidden.shape and weights is None
        with pytest.raises(NotImplementedError, match="attention weights"):
            attn(hidden, position_embeddings=(cos, torch.zeros_like(cos)), past_key_values=DynamicCache(), output_attentions=True)

"""Additive masks on the gather attention (ha_sparse_decode_masked): by token position - the `attention_mask` the reference's
patched layer adds before its softmax (hashattention_llama.py:593-598), i.e. the padding of a batch - and by place in the
list - the `Mask` argument of the reference's fwd_sparse kernel (efficiency/kernels/sparse.py:14, 46-58, 190-212).  Kernel
against the oracle, then a left-padded batch through a patched model against the oracle-driven model."""
import copy

import numpy as np
import pytest
import torch
from transformers import DynamicCache, LlamaConfig, LlamaForCausalLM

from hashattention import _ops
from hashattention import hashattention_llama as hl
from oracle import hashattn_oracle as orc
from tests.test_gpu_model_api import _config

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 2e-2), (torch.float16, 2e-2), (torch.float32, 2e-5)])
@pytest.mark.parametrize("by_slot", [False, True])
def test_masked_gather_attention_matches_the_oracle(dtype, tol, by_slot):
    print(f"\n[case] masked gather attention {dtype} by_slot={by_slot}", flush=True)
    g = torch.Generator().manual_seed(11 + int(by_slot))
    B, H, Hkv, S, cap = 3, 4, 2, 5000, 3000          # lists long enough to be split over several workgroups
    q = torch.randn(B, H, 128, generator=g).to(dtype)
    k = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
    v = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
    counts = torch.tensor([[cap, 1700, 1, 37], [5, cap, 600, 2999], [0, 64, 65, 2048]], dtype=torch.int32)
    idx = torch.zeros(B, H, cap, dtype=torch.int32)
    for b in range(B):
        for h in range(H):
            n = int(counts[b, h])
            idx[b, h, :n] = torch.sort(torch.randperm(S, generator=g)[:n]).values.to(torch.int32)
    n_mask = cap if by_slot else S
    mask = torch.randn(B, n_mask, generator=g) * 2.0
    mask[torch.rand(B, n_mask, generator=g) < 0.3] = float("-inf")
    mask[1, :] = torch.where(torch.rand(n_mask, generator=g) < 0.5, torch.tensor(torch.finfo(torch.bfloat16).min), torch.tensor(0.0))
    if by_slot:
        mask[0, :40] = float("-inf")                     # row (0, 3) with 37 entries: everything removed
    else:
        mask[0, idx[0, 3, :37].long()] = float("-inf")
    out = torch.empty(B, H, 128, dtype=dtype, device=DEV)
    ws = _ops.workspace(_ops.sparse_decode_workspace_bytes(B, H, cap), DEV)
    _ops.sparse_decode(q.to(DEV), k.to(DEV), v.to(DEV), idx.to(DEV), counts.to(DEV), 1 / 128 ** 0.5, out, ws,
                       mask=mask.to(DEV), mask_by_slot=by_slot)
    torch.cuda.synchronize()
    got = out.float().cpu()
    worst = 0.0
    for b in range(B):
        for h in range(H):
            n = int(counts[b, h])
            ii = idx[b, h, :n].long()
            terms = mask[b, :n] if by_slot else mask[b, ii]
            if n == 0 or not torch.isfinite(terms).any() or (terms <= torch.finfo(torch.bfloat16).min).all():
                # nothing left (or everything at the most negative value, where the reference's softmax is uniform over
                # noise): only the fully removed rows are checked, they are defined as zero
                if n == 0 or not torch.isfinite(terms).any():
                    assert (got[b, h] == 0).all(), (b, h)
                continue
            want = orc.sparse_attend(q[b, h], k[b, h // 2], v[b, h // 2], ii.numpy(), 1 / 128 ** 0.5, slot_mask=terms)
            worst = max(worst, (got[b, h] - want).abs().max().item())
    print(f"  max abs error {worst:.2e}", flush=True)
    assert worst <= tol
    # a mask of zeros is the unmasked kernel, bit for bit; a constant mask changes nothing but round-off
    out0 = torch.empty_like(out)
    out1 = torch.empty_like(out)
    zeros = torch.zeros(1, n_mask, device=DEV).expand(B, n_mask)          # one row shared by the batch: stride 0
    _ops.sparse_decode(q.to(DEV), k.to(DEV), v.to(DEV), idx.to(DEV), counts.to(DEV), 1 / 128 ** 0.5, out0, ws)
    _ops.sparse_decode(q.to(DEV), k.to(DEV), v.to(DEV), idx.to(DEV), counts.to(DEV), 1 / 128 ** 0.5, out1, ws, mask=zeros,
                       mask_by_slot=by_slot)
    torch.cuda.synchronize()
    assert torch.equal(out0, out1)
    _ops.sparse_decode(q.to(DEV), k.to(DEV), v.to(DEV), idx.to(DEV), counts.to(DEV), 1 / 128 ** 0.5, out1, ws,
                       mask=torch.full((B, n_mask), 3.25, device=DEV), mask_by_slot=by_slot)
    torch.cuda.synchronize()
    assert (out0.float() - out1.float()).abs().max().item() <= tol


def _oracle_forward_masked(layer, usa, cfg, apply_rope):
    import types
    orig = layer.forward
    heads = lambda mods: [[(m.weight.detach().float().cpu(), m.bias.detach().float().cpu()) for m in seq if isinstance(m, torch.nn.Linear)]
                          for seq in mods]
    k_heads, q_heads = heads(usa.learning_to_hash_transformation_k), heads(usa.learning_to_hash_transformation_q)

    def forward(self, hidden_states, position_embeddings=None, attention_mask=None, past_key_values=None, **kwargs):
        b, q_len, _ = hidden_states.shape
        if q_len > 128:
            return orig(hidden_states=hidden_states, position_embeddings=position_embeddings, attention_mask=attention_mask,
                        past_key_values=past_key_values, **kwargs)
        shape = (b, q_len, -1, self.head_dim)
        q = self.q_proj(hidden_states).view(shape).transpose(1, 2)
        k = self.k_proj(hidden_states).view(shape).transpose(1, 2)
        v = self.v_proj(hidden_states).view(shape).transpose(1, 2)
        q, k = apply_rope(q, k, *position_embeddings)
        k, v = past_key_values.update(k, v, self.layer_idx)
        am = attention_mask
        if am is not None and am.dtype == torch.bool:      # the additive form the reference's eager path receives
            am = torch.zeros(am.shape).masked_fill(~am, torch.finfo(torch.float32).min)
        out, _ = orc.reference_decode_attention(q, k, v, k_heads, q_heads, cfg.init_budget, cfg.recent_budget, cfg.heavy_budget,
                                                attention_mask=None if am is None else am[..., :k.shape[2]])
        return self.o_proj(out.transpose(1, 2).reshape(b, q_len, -1)), None

    layer.forward = types.MethodType(forward, layer)


def _run(model, ids, am, steps):
    cache = DynamicCache()
    outs = []
    with torch.no_grad():
        pos = ids.shape[1] - sum(steps)
        o = model(ids[:, :pos], attention_mask=am[:, :pos], past_key_values=cache, use_cache=True)
        outs.append(o.logits[:, -1].float().cpu())
        for n in steps:
            o = model(ids[:, pos:pos + n], attention_mask=am[:, :pos + n], past_key_values=cache, use_cache=True)
            outs.append(o.logits.float().cpu())
            pos += n
    return outs


def test_left_padded_batch_through_the_patched_model():
    print("\n[case] patched model, left-padded batch", flush=True)
    torch.manual_seed(7)
    cfg = _config(LlamaConfig)
    model = LlamaForCausalLM(cfg).bfloat16().float()
    ref = copy.deepcopy(model)
    usa = hl.load_usa(cfg, None)
    model = hl.convert_usa(model.to(DEV), cfg, usa, collect_stats=False, train_usa=False).float()
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    for li, layer in enumerate(ref.model.layers):
        _oracle_forward_masked(layer.self_attn, usa[li], cfg, apply_rotary_pos_emb)
    T = 200 + 1 + 1 + 5 + 1
    ids = torch.randint(0, cfg.vocab_size, (2, T), generator=torch.Generator().manual_seed(3))
    am = torch.ones(2, T, dtype=torch.long)
    am[1, :45] = 0                                    # sequence 1 starts with 45 padding tokens
    steps = [1, 1, 5, 1]
    got = _run(model, ids.to(DEV), am.to(DEV), steps)
    want = _run(ref, ids, am, steps)
    for a, b in zip(got, want):
        err = (a - b).abs().max().item()
        print(f"  max |logit difference| {err:.2e}", flush=True)
        assert a.shape == b.shape and err < 2e-3, err
    # the mask matters: without it the padded sequence's logits differ, the unpadded one's do not
    hl.reset_usa(model)
    plain = _run(model, ids.to(DEV), torch.ones_like(am).to(DEV), steps)
    assert (plain[-1][1] - got[-1][1]).abs().max().item() > 1e-3
    assert (plain[-1][0] - got[-1][0]).abs().max().item() < 1e-4


def test_generate_with_a_left_padded_batch():
    """`model.generate` end to end (greedy): prefill of 150 tokens through the original forward, then single-token steps
    through the HIP path with the padding mask, against the oracle-driven model on the CPU: the same tokens."""
    print("\n[case] generate, left-padded batch", flush=True)
    torch.manual_seed(8)
    cfg = _config(LlamaConfig)
    cfg.pad_token_id = 0
    model = LlamaForCausalLM(cfg).bfloat16().float()
    ref = copy.deepcopy(model)
    usa = hl.load_usa(cfg, None)
    model = hl.convert_usa(model.to(DEV), cfg, usa, collect_stats=False, train_usa=False).float()
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    for li, layer in enumerate(ref.model.layers):
        _oracle_forward_masked(layer.self_attn, usa[li], cfg, apply_rotary_pos_emb)
    ids = torch.randint(1, cfg.vocab_size, (2, 150), generator=torch.Generator().manual_seed(4))
    am = torch.ones(2, 150, dtype=torch.long)
    am[0, :23] = 0
    ids[0, :23] = 0
    kw = dict(max_new_tokens=6, do_sample=False, use_cache=True, pad_token_id=0)
    with torch.no_grad():
        got = model.generate(input_ids=ids.to(DEV), attention_mask=am.to(DEV), **kw).cpu()
        want = ref.generate(input_ids=ids, attention_mask=am, **kw)
    print("  new tokens:", got[:, 150:].tolist(), flush=True)
    assert got.shape == (2, 156) and torch.equal(got, want)
    assert model.model.layers[0].self_attn._hash_layer.n_cached == 155      # the last token is sampled, not fed back

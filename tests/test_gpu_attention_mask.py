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


@pytest.mark.parametrize("fused", [False, True])
def test_left_padded_batch_through_the_patched_model(fused, monkeypatch):
    # fused: batches of 32 and more (sequence, head) rows take the fused select-attend launch, which is handed the padding as one
    # number per sequence; here the threshold is lowered so that the tiny model takes it (and the call is counted)
    print(f"\n[case] patched model, left-padded batch, fused launch: {fused}", flush=True)
    from hashattention import decode
    seen = []
    if fused:
        allocate, launch = decode.HashDecodeLayer.allocate, _ops.sparse_decode_fused

        def allocate_low(self, *a, **kw):
            self.fused_min_rows = 1
            return allocate(self, *a, **kw)

        def launch_counted(*a, **kw):
            seen.append(kw.get("masked_prefix"))
            return launch(*a, **kw)
        monkeypatch.setattr(decode.HashDecodeLayer, "allocate", allocate_low)
        monkeypatch.setattr(_ops, "sparse_decode_fused", launch_counted)
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
    if fused:       # three single-token steps of two layers went through the fused launch with the prefix [0, 45]
        assert len(seen) == 6 and all(p is not None and p.tolist() == [0, 45] for p in seen), seen
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


@pytest.mark.parametrize("case", ["ragged", "uniform_split_rows", "wide_codes"])
def test_fused_launch_with_a_masked_prefix_matches_the_oracle(case):
    # the mask of a left-padded batch inside the fused select-attend launch (ha_sparse_decode_fused_prefix_masked): the tokens in
    # front of masked_prefix[b] stay selected and counted - the selection does not see the mask, hashattention_llama.py:593-598 -
    # and add nothing to the softmax.  Against the oracle's gather attention with -inf on those entries, and against
    # ha_select + ha_sparse_decode_masked with the same mask as a table.
    from oracle import c_oracle
    from hashattention.synthetic import make_problem
    from tests.parity_util import ATOL, oracle_codes, small_workload, to_i32
    print(f"\n[case] fused launch, masked prefix: {case}", flush=True)
    if case == "ragged":         # prefixes: none, inside the sink window, into the candidates, all but the last token, everything
        w = small_workload(batch=5, seq_lens=[1500, 1111, 3000, 700, 900], heavy_budget=0.125, seed=41)
        prefix, ragged = [0, 9, 1200, 699, 900], True
    elif case == "uniform_split_rows":   # long equal rows (cut into pieces), lengths given on the host
        w = small_workload(batch=2, seq_lens=[20000, 20000], n_q_heads=4, n_kv_heads=2, n_code_heads=4, heavy_budget=1 / 16, seed=42,
                           dtype=torch.float16)
        prefix, ragged = [4097, 15], False
    else:                        # 64-bit codes
        w = small_workload(batch=3, seq_lens=[5000, 2500, 4000], lth_num_layers=2, lth_final_dim=64, heavy_budget=0.25, seed=43,
                           dtype=torch.float32)
        prefix, ragged = [100, 0, 3990], True
    p = make_problem(w)
    B, H, Hc, S, W = w.batch, w.n_q_heads, w.n_code_heads, w.max_seq_len, w.code_words
    _, _, kc64, qc64 = oracle_codes(p)
    kc_np, qc_np, seq_np = to_i32(kc64), to_i32(qc64), p.seq_lens.numpy()
    kcodes, qcodes = torch.from_numpy(kc_np).to(DEV), torch.from_numpy(qc_np).to(DEV)
    q3, k, v = p.q[:, :, 0, :].contiguous().to(DEV), p.k.to(DEV), p.v.to(DEV)
    seq = p.seq_lens.to(DEV) if ragged else None
    assert _ops.fused_applies(B, H, Hc, W, S, w.init_budget, w.recent_budget, w.heavy_budget)
    cap = max(w.n_selected(s) for s in w.seq_lens)
    idx_ref, counts_ref = c_oracle.select(kc_np, qc_np, seq_np, w.init_budget, w.recent_budget, w.heavy_budget, cap, mode=0, depth=0)
    pre = torch.tensor(prefix, dtype=torch.int32, device=DEV)
    sm = 1 / 128 ** 0.5
    ws = _ops.workspace(_ops.select_workspace_bytes(B, H, Hc, W, S), DEV)
    ws4 = _ops.workspace(_ops.sparse_decode_fused_workspace_bytes(B, H, Hc, S), DEV)
    outs = []
    for ready in (True, False):
        if not ready and not _ops.fused_local_thresholds(B, Hc, S):
            continue
        counts = torch.full((B, H), -5, dtype=torch.int32, device=DEV)
        out = torch.empty(B, H, 128, dtype=w.dtype, device=DEV)
        if ready:
            _ops.select_prepare(kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, counts, ws)
        else:
            _ops.select_histogram(kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, ws)
        _ops.sparse_decode_fused(q3, k, v, kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, ws, sm, out, ws4,
                                 thresholds_ready=ready, out_counts=counts, masked_prefix=pre)
        torch.cuda.synchronize()
        assert np.array_equal(counts.cpu().numpy(), counts_ref), "the mask must not change what is selected"
        outs.append(out)
    if len(outs) == 2:
        assert torch.equal(outs[0], outs[1])
    got = outs[0].float().cpu()
    worst = 0.0
    G = H // w.n_kv_heads
    for b in range(B):
        for h in range(H):
            n = int(counts_ref[b, h])
            ii = torch.from_numpy(idx_ref[b, h, :n].astype(np.int64))
            terms = torch.where(ii < prefix[b], torch.tensor(float("-inf")), torch.tensor(0.0))
            if n == 0 or not torch.isfinite(terms).any():
                assert (got[b, h] == 0).all(), (b, h)
                continue
            want = orc.sparse_attend(p.q[b, h, 0], p.k[b, h // G], p.v[b, h // G], ii.numpy(), sm, slot_mask=terms)
            worst = max(worst, (got[b, h] - want).abs().max().item())
    print(f"  max abs error {worst:.2e}", flush=True)
    assert worst <= ATOL[w.dtype]
    # the same mask as a table through the two-launch path
    idx = torch.full((B, H, cap), -1, dtype=torch.int32, device=DEV)
    counts = torch.zeros(B, H, dtype=torch.int32, device=DEV)
    _ops.select(kcodes, qcodes, S, p.seq_lens.to(DEV), w.init_budget, w.recent_budget, w.heavy_budget, idx, counts, ws)
    table = torch.zeros(B, S, device=DEV)
    for b in range(B):
        table[b, :prefix[b]] = float("-inf")
    out2 = torch.empty_like(outs[0])
    _ops.sparse_decode(q3, k, v, idx, counts, sm, out2, _ops.workspace(_ops.sparse_decode_workspace_bytes(B, H, cap), DEV), mask=table)
    torch.cuda.synchronize()
    same = (out2.float() - outs[0].float()).abs().max().item()
    assert same <= (1e-5 if w.dtype == torch.float32 else 1e-2), same
    # a prefix of zero everywhere is the plain fused launch, bit for bit
    out3, out4 = torch.empty_like(out2), torch.empty_like(out2)
    _ops.select_prepare(kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, counts, ws)
    _ops.sparse_decode_fused(q3, k, v, kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, ws, sm, out3, ws4)
    _ops.sparse_decode_fused(q3, k, v, kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, ws, sm, out4, ws4,
                             masked_prefix=torch.zeros(B, dtype=torch.int32, device=DEV))
    torch.cuda.synchronize()
    assert torch.equal(out3, out4)

"""End-to-end decode steps through HashDecodeLayer (bit-cache append -> select -> attend) against the oracle's
restatement of the reference layer (dense scores, every key re-hashed, stable sort, masked fp32 softmax)."""
import numpy as np
import pytest
import torch

from hashattention import _ops
from hashattention.decode import HashDecodeLayer
from hashattention.synthetic import make_problem
from oracle import hashattn_oracle as orc
from tests.parity_util import small_workload

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _layer(w, p, **kw):
    return HashDecodeLayer(p.usa.k, p.usa.q, w.n_q_heads, w.n_kv_heads, w.head_dim, w.lth_num_layers, w.lth_int_dim,
                           w.lth_final_dim, w.init_budget, w.recent_budget, w.heavy_budget, device=DEV, **kw)


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("hc", [2, 8])
def test_three_decode_steps_match_reference_layer(hc, fused):
    # fp32 end to end: the step output equals the reference layer's masked dense attention on the same cache, through the
    # fused select-attend launch and through ha_select + ha_sparse_decode
    print(f"\n[case] decode layer Hc={hc} fused={fused}", flush=True)
    w = small_workload(batch=2, seq_lens=[900, 900], n_code_heads=hc, dtype=torch.float32, seed=17)
    p = make_problem(w)
    S = w.max_seq_len
    k, v = p.k.to(DEV), p.v.to(DEV)
    layer = _layer(w, p)
    layer.allocate(w.batch, S)
    layer.use_fused = fused
    layer.fused_ok = _ops.fused_applies(w.batch, w.n_q_heads, hc, w.code_words, S, w.init_budget, w.recent_budget, w.heavy_budget)
    assert layer.fused_ok             # small batches default to the two-launch path: force the fused one here
    s0 = S - 3
    layer.encode_keys(k[:, :, :s0])
    layer.n_cached = s0
    g = torch.Generator().manual_seed(5)
    for step in range(3):
        s = s0 + step + 1
        q = torch.randn(w.batch, w.n_q_heads, 1, w.head_dim, generator=g)
        out = torch.empty(w.batch, w.n_q_heads, w.head_dim, device=DEV)
        layer.step(q.to(DEV), k, v, s, out)
        if fused:           # the fused step keeps its lists in LDS: write them out for the comparison below
            layer.select(s, None)
        ref, mask = orc.reference_decode_attention(q, p.k[:, :, :s], p.v[:, :, :s], p.usa.k, p.usa.q, w.init_budget,
                                                   w.recent_budget, w.heavy_budget)
        # selected sets must be identical (codes may differ only at |logit| ~ 0, which would show up here)
        idx = layer.idx.cpu().numpy()
        cnt = layer.counts.cpu().numpy()
        for b in range(w.batch):
            for h in range(w.n_q_heads):
                got = np.zeros(s, dtype=bool)
                got[idx[b, h, :cnt[b, h]]] = True
                assert np.array_equal(got, mask[b, h, 0].numpy()), (step, b, h)
        err = (out.cpu() - ref[:, :, 0]).abs().max().item()
        assert err < 2e-5, err


def test_step_refuses_a_gap_in_the_bit_cache():
    w = small_workload(batch=1, seq_lens=[200], seed=3)
    p = make_problem(w)
    layer = _layer(w, p)
    layer.allocate(1, 200)
    out = torch.empty(1, w.n_q_heads, 128, dtype=w.dtype, device=DEV)
    with pytest.raises(RuntimeError):
        layer.step(p.q.to(DEV), p.k.to(DEV), p.v.to(DEV), 200, out)   # nothing cached yet, one token appended


def test_cpu_tensors_are_refused():
    with pytest.raises(ValueError):
        _ops.hamming_score(torch.zeros(1, 1, 4, 1, dtype=torch.int32), torch.zeros(1, 1, 1, dtype=torch.int32), 4)


@pytest.mark.parametrize("fused", [True, False])
def test_step_replayed_from_a_hip_graph_matches_eager(fused):
    # the step allocates nothing and reads its lengths from arguments, so it can be captured; every replay, with eager
    # work and synchronisations in between, must reproduce the eager output bit for bit
    print(f"\n[case] graph replay fused={fused}", flush=True)
    w = small_workload(batch=8, seq_lens=[3000] * 8, n_q_heads=32, n_kv_heads=8, n_code_heads=8, seed=23)
    p = make_problem(w)
    S = w.max_seq_len
    k, v, q = p.k.to(DEV), p.v.to(DEV), p.q.to(DEV)
    layer = _layer(w, p)
    layer.allocate(w.batch, S)
    layer.use_fused = fused
    assert layer.fused_ok
    layer.encode_keys(k[:, :, :S - 1])
    out = torch.empty(w.batch, w.n_q_heads, w.head_dim, dtype=w.dtype, device=DEV)

    def step():
        layer.n_cached = S - 1
        layer.step(q, k, v, S, out)

    step()
    want = out.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for i in range(4):
        out.zero_()
        layer.counts.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), i
        scratch = torch.randn(1 << 20, device=DEV).sum().item()     # unrelated eager work between replays
        assert scratch == scratch


@pytest.mark.parametrize("hc", [2, 8])
@pytest.mark.parametrize("batch,T,masked", [(3, 7, False), (2, 5, True), (1, 128, False)])
def test_chunk_of_tokens_in_one_selection_and_one_attention_launch(batch, T, masked, hc):
    # a chunk of T new tokens per sequence (hashattention_llama.py:423-428): row i of every sequence attends with its own
    # causal windows and budget.  All B * T rows go through ONE ha_select_rows and ONE ha_sparse_decode_rows call; output
    # and kept sets against the reference layer's dense restatement (causal + optional padding mask added to the scores)
    print(f"\n[case] chunk step B={batch} T={T} masked={masked} Hc={hc}", flush=True)
    S = 700
    w = small_workload(batch=batch, seq_lens=[S] * batch, n_code_heads=hc, dtype=torch.float32, seed=31 + T)
    p = make_problem(w)
    k, v = p.k.to(DEV), p.v.to(DEV)
    layer = _layer(w, p)
    layer.allocate(batch, S)
    layer.encode_keys(k)
    layer.n_cached = S
    q = torch.randn(batch, w.n_q_heads, T, w.head_dim, generator=torch.Generator().manual_seed(9))
    add = torch.zeros(batch, 1, T, S)
    rows = torch.arange(T).view(T, 1) + S - T
    add.masked_fill_((torch.arange(S).view(1, S) > rows).view(1, 1, T, S), torch.finfo(torch.float32).min)
    amask = None
    if masked:                      # left padding of different lengths, as transformers hands it to the layer
        for b in range(batch):
            add[b, :, :, :3 + 2 * b] = torch.finfo(torch.float32).min
        amask = add[:, 0].contiguous().to(DEV)
    out = torch.empty(batch, w.n_q_heads, T, w.head_dim, device=DEV)
    for rep in range(2):            # the second call reuses the buffers of the first
        heavy = layer.heavy_count(S)            # the reference sizes every row's budget by the cache length (:431-434)
        layer.chunk_step(q.to(DEV), k, v, S, out, 0.0 if heavy == 0 else heavy + 0.5, attn_mask=amask)
        ref, mask = orc.reference_decode_attention(q, p.k, p.v, p.usa.k, p.usa.q, w.init_budget, w.recent_budget, w.heavy_budget,
                                                   attention_mask=add)
        idx = layer._chunk["idx"].cpu().numpy()
        cnt = layer._chunk["cnt"].cpu().numpy()
        causal = (add[0, 0] == 0) if not masked else (torch.arange(S).view(1, S) <= rows)
        for b in range(batch):
            for i in range(T):
                for h in range(w.n_q_heads):
                    got = np.zeros(S, dtype=bool)
                    got[idx[b * T + i, h, :cnt[b * T + i, h]]] = True
                    assert np.array_equal(got, (mask[b, h, i] & causal[i]).numpy()), (b, i, h)
        err = (out.cpu() - ref).abs().max().item()
        assert err < 2e-5, err


def test_chunk_buffers_follow_the_batch_shape_at_constant_row_count():
    # (B, T) = (2, 4) then (4, 2): the same number of rows, but the query codes [B, H, T, W] and the row lengths are shaped by
    # B and T separately - buffers kept from the first shape must not serve the second
    print("\n[case] chunk step (B, T) = (2, 4) then (4, 2)", flush=True)
    S = 600
    w4 = small_workload(batch=4, seq_lens=[S] * 4, dtype=torch.float32, seed=77)
    p4 = make_problem(w4)
    layer = _layer(w4, p4)
    for (B, T) in ((2, 4), (4, 2), (2, 4)):
        k, v = p4.k[:B].to(DEV), p4.v[:B].to(DEV)
        layer.allocate(B, S)
        layer.encode_keys(k)
        layer.n_cached = S
        q = torch.randn(B, w4.n_q_heads, T, w4.head_dim, generator=torch.Generator().manual_seed(B * 10 + T))
        out = torch.empty(B, w4.n_q_heads, T, w4.head_dim, device=DEV)
        heavy = layer.heavy_count(S)
        layer.chunk_step(q.to(DEV), k, v, S, out, heavy + 0.5)
        add = torch.zeros(B, 1, T, S)
        rows = torch.arange(T).view(T, 1) + S - T
        add.masked_fill_((torch.arange(S).view(1, S) > rows).view(1, 1, T, S), torch.finfo(torch.float32).min)
        ref, _ = orc.reference_decode_attention(q, p4.k[:B], p4.v[:B], p4.usa.k, p4.usa.q, w4.init_budget, w4.recent_budget,
                                                w4.heavy_budget, attention_mask=add)
        assert layer._chunk["qc"].shape[:3] == (B, w4.n_q_heads, T)
        err = (out.cpu() - ref).abs().max().item()
        assert err < 2e-5, (B, T, err)

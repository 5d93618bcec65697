"""Attention over a cache addressed through a token -> slot table (`ha_sparse_decode_paged`, `ha_sparse_decode_fused_paged`):
the `Req_to_tokens` indirection of the reference's sparse flash-decode (efficiency/kernels/flash_fwd_sparse.py:396-470, table
built at efficiency/kernels/torchatt.py:165).  Oracle: the gather attention on the cache the table describes,
K[b, h, j] = pool[table[b, j], h] (oracle.rows_through_slot_table).  The paged launches add the same rows in the same order
as the unpaged ones on that cache, so the two outputs must also agree bit for bit."""
import math

import numpy as np
import pytest
import torch

from hashattention import _ops
from hashattention.synthetic import make_problem, make_problem_on_device, named_workload
from oracle import c_oracle
from oracle import hashattn_oracle as orc
from tests.parity_util import ATOL, oracle_codes, small_workload, to_i32

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _scatter_into_pool(k, v, seq_lens, spare, g, device=None):
    """Logical caches k, v [B, Hkv, S, d] -> (pool_k, pool_v [n_slots, Hkv, d], table int32 [B, S]) with the tokens of all
    sequences scattered over the pool by one random permutation; table entries past a sequence's length point at slot 0."""
    B, Hkv, S, d = k.shape
    n_slots = B * S + spare
    perm = torch.randperm(n_slots, generator=g)[:B * S].view(B, S).to(torch.int32)
    table = torch.zeros(B, S, dtype=torch.int32)
    for b in range(B):
        table[b, :seq_lens[b]] = perm[b, :seq_lens[b]]
    dev = device or k.device
    pool_k = torch.randn(n_slots, Hkv, d, generator=g).to(k.dtype).to(dev)      # unused slots hold noise, not zeros
    pool_v = torch.randn(n_slots, Hkv, d, generator=g).to(k.dtype).to(dev)
    tab = table.to(dev).long()
    for b in range(B):
        n = int(seq_lens[b])
        pool_k[tab[b, :n]] = k[b, :, :n].to(dev).transpose(0, 1)
        pool_v[tab[b, :n]] = v[b, :, :n].to(dev).transpose(0, 1)
    return pool_k, pool_v, table


def _pool_views(pool, B):
    """[n_slots, Hkv, d] -> the [B, Hkv, n_slots, d] view the ABI takes: batch stride 0, token-major rows."""
    n, Hkv, d = pool.shape
    return pool.view(1, n, Hkv, d).permute(0, 2, 1, 3).expand(B, Hkv, n, d)


CASES = [
    dict(name="ragged_bf16", batch=3, seq_lens=[1500, 1111, 40], dtype=torch.bfloat16),
    dict(name="split_rows_fp16", batch=1, seq_lens=[6000], n_q_heads=8, n_kv_heads=2, n_code_heads=2, dtype=torch.float16,
         heavy_budget=0.25),
    dict(name="fp32_two_word_codes", batch=2, seq_lens=[2100, 2100], dtype=torch.float32, lth_num_layers=2, lth_final_dim=64),
    dict(name="many_rows_equal_lengths", batch=8, seq_lens=[3000] * 8, n_q_heads=32, n_kv_heads=8, n_code_heads=8, dtype=torch.bfloat16,
         init_budget=128, recent_budget=128, heavy_budget=1 / 8),
    dict(name="no_windows_mha", batch=2, seq_lens=[4096, 4096], n_q_heads=8, n_kv_heads=8, n_code_heads=8, dtype=torch.float16,
         init_budget=0, recent_budget=0, heavy_budget=128.0),
    dict(name="windows_only", batch=2, seq_lens=[100, 31], dtype=torch.bfloat16),
]


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_paged_launches_equal_the_unpaged_ones_on_the_cache_the_table_describes(case):
    print(f"\n[case] paged cache {case['name']}", flush=True)
    w = small_workload(**{**case, "seed": 41})
    p = make_problem(w)
    B, H, Hkv, Hc, S, W = w.batch, w.n_q_heads, w.n_kv_heads, w.n_code_heads, w.max_seq_len, w.code_words
    g = torch.Generator().manual_seed(99)
    pool_k, pool_v, table = _scatter_into_pool(p.k, p.v, w.seq_lens, spare=777, g=g, device=DEV)
    # the oracle's view of the table reproduces the logical cache
    for b in range(B):
        n = w.seq_lens[b]
        assert torch.equal(orc.rows_through_slot_table(pool_k.cpu(), table)[b, :, :n], p.k[b, :, :n])
    kp, vp = _pool_views(pool_k, B), _pool_views(pool_v, B)
    assert (B == 1 or kp.stride(0) == 0) and kp.stride(2) == Hkv * 128
    slots = table.to(DEV)
    _, _, kc64, qc64 = oracle_codes(p)
    kc_np, qc_np = to_i32(kc64), to_i32(qc64)
    kcodes, qcodes = torch.from_numpy(kc_np).to(DEV), torch.from_numpy(qc_np).to(DEV)
    seq_np = p.seq_lens.numpy()
    seq = p.seq_lens.to(DEV)
    q3, k, v = p.q[:, :, 0].contiguous().to(DEV), p.k.to(DEV), p.v.to(DEV)
    scale = 1 / math.sqrt(128)
    cap = max(max(w.n_selected(s) for s in w.seq_lens), 1)
    idx = torch.zeros(B, H, cap, dtype=torch.int32, device=DEV)
    counts = torch.zeros(B, H, dtype=torch.int32, device=DEV)
    ws_s = _ops.workspace(_ops.select_workspace_bytes(B, H, Hc, W, S), DEV)
    _ops.select(kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, idx, counts, ws_s)
    idx_ref, cnt_ref = c_oracle.select(kc_np, qc_np, seq_np, w.init_budget, w.recent_budget, w.heavy_budget, cap)
    assert np.array_equal(counts.cpu().numpy(), cnt_ref)
    ref = c_oracle.sparse_attend(p.q[:, :, 0], orc.rows_through_slot_table(pool_k.cpu(), table),
                                 orc.rows_through_slot_table(pool_v.cpu(), table), idx_ref, cnt_ref, scale)
    ws_a = _ops.workspace(_ops.sparse_decode_workspace_bytes(B, H, cap), DEV)

    # ---- list-fed
    plain, paged = torch.empty(B, H, 128, dtype=w.dtype, device=DEV), torch.empty(B, H, 128, dtype=w.dtype, device=DEV)
    _ops.sparse_decode(q3, k, v, idx, counts, scale, plain, ws_a)
    _ops.sparse_decode(q3, kp, vp, idx, counts, scale, paged, ws_a, slots=slots)
    torch.cuda.synchronize()
    err = np.abs(paged.float().cpu().numpy() - ref).max()
    assert err <= ATOL[w.dtype], err
    assert torch.equal(paged, plain), "list-fed: the paged launch differs from the unpaged one"

    # ---- list-fed with masks: by token position (the table must not touch the mask's index) and by place in the list
    for by_slot in (False, True):
        n_mask = cap if by_slot else S
        mask = (torch.randn(B, n_mask, generator=g) * 2).to(DEV)
        mask[torch.rand(B, n_mask, generator=g).to(DEV) < 0.2] = float("-inf")
        a, b2 = torch.empty_like(plain), torch.empty_like(plain)
        _ops.sparse_decode(q3, k, v, idx, counts, scale, a, ws_a, mask=mask, mask_by_slot=by_slot)
        _ops.sparse_decode(q3, kp, vp, idx, counts, scale, b2, ws_a, mask=mask, mask_by_slot=by_slot, slots=slots)
        assert torch.equal(a, b2), f"masked (by_slot={by_slot}): the paged launch differs from the unpaged one"

    # ---- selection fused into the launch
    if not _ops.fused_applies(B, H, Hc, W, S, w.init_budget, w.recent_budget, w.heavy_budget):
        return
    ws_f = _ops.workspace(_ops.sparse_decode_fused_workspace_bytes(B, H, Hc, S), DEV)
    for lens in ((seq, None) if len(set(w.seq_lens)) == 1 else (seq,)):
        for local in ((True, False) if _ops.fused_local_thresholds(B, Hc, S) else (False,)):
            cnt_a = torch.full((B, H), -1, dtype=torch.int32, device=DEV)
            cnt_b = torch.full((B, H), -1, dtype=torch.int32, device=DEV)
            fa, fb = torch.empty_like(plain), torch.empty_like(plain)
            if local:
                _ops.select_histogram(kcodes, qcodes, S, lens, w.init_budget, w.recent_budget, ws_s)
            else:
                _ops.select_prepare(kcodes, qcodes, S, lens, w.init_budget, w.recent_budget, w.heavy_budget, cnt_a, ws_s)
                cnt_b.copy_(cnt_a)
            kw = dict(thresholds_ready=not local)
            _ops.sparse_decode_fused(q3, k, v, kcodes, qcodes, S, lens, w.init_budget, w.recent_budget, w.heavy_budget, ws_s, scale, fa,
                                     ws_f, out_counts=cnt_a if local else None, **kw)
            _ops.sparse_decode_fused(q3, kp, vp, kcodes, qcodes, S, lens, w.init_budget, w.recent_budget, w.heavy_budget, ws_s, scale, fb,
                                     ws_f, out_counts=cnt_b if local else None, slots=slots, **kw)
            torch.cuda.synchronize()
            assert np.array_equal(cnt_b.cpu().numpy(), cnt_ref)
            errf = np.abs(fb.float().cpu().numpy() - ref).max()
            assert errf <= ATOL[w.dtype], (errf, local, lens is None)
            assert torch.equal(fa, fb), f"fused (local thresholds {local}, lengths on the host {lens is None}): paged differs from unpaged"
            fb2 = torch.empty_like(fb)      # a second call: nothing of the first may linger
            _ops.sparse_decode_fused(q3, kp, vp, kcodes, qcodes, S, lens, w.init_budget, w.recent_budget, w.heavy_budget, ws_s, scale, fb2,
                                     ws_f, out_counts=cnt_b if local else None, slots=slots, **kw)
            assert torch.equal(fb, fb2)


def test_chunk_rows_share_the_table_of_their_sequence():
    # rows_per_sequence > 1: the T rows of a sequence read one table row and one pool view
    print("\n[case] paged cache, chunk of rows", flush=True)
    B, T, H, Hkv, S, cap = 2, 3, 4, 2, 900, 200
    g = torch.Generator().manual_seed(5)
    k, v = torch.randn(B, Hkv, S, 128, generator=g).bfloat16(), torch.randn(B, Hkv, S, 128, generator=g).bfloat16()
    q = torch.randn(B * T, H, 128, generator=g).bfloat16()
    pool_k, pool_v, table = _scatter_into_pool(k, v, [S] * B, spare=50, g=g, device=DEV)
    idx = torch.stack([torch.stack([torch.sort(torch.randperm(S, generator=g)[:cap]).values for _ in range(H)]) for _ in range(B * T)]).to(torch.int32)
    counts = torch.randint(1, cap + 1, (B * T, H), generator=g, dtype=torch.int32)
    ws = _ops.workspace(_ops.sparse_decode_workspace_bytes(B * T, H, cap), DEV)
    a, b2 = torch.empty(B * T, H, 128, dtype=torch.bfloat16, device=DEV), torch.empty(B * T, H, 128, dtype=torch.bfloat16, device=DEV)
    _ops.sparse_decode_rows(q.to(DEV), k.to(DEV), v.to(DEV), T, idx.to(DEV), counts.to(DEV), 0.09, a, ws)
    _ops.sparse_decode(q.to(DEV), _pool_views(pool_k, B), _pool_views(pool_v, B), idx.to(DEV), counts.to(DEV), 0.09, b2, ws,
                       slots=table.to(DEV), rows_per_sequence=T)
    assert torch.equal(a, b2)
    ref = c_oracle.sparse_attend(q, k.repeat_interleave(T, dim=0), v.repeat_interleave(T, dim=0), idx.numpy(), counts.numpy(), 0.09)
    assert np.abs(b2.float().cpu().numpy() - ref).max() <= 2e-2


def test_the_prototypes_identity_table_and_pool_layout():
    # torchatt.py:148-165: k, v [B * N, H, D] fp16, req_to_tokens = arange(B * N).reshape(B, N), MHA, topk lists in score order
    print("\n[case] paged cache, the prototype's identity table", flush=True)
    B, N, H, D, topk = 4, 2048, 32, 128, 64
    g = torch.Generator().manual_seed(165)
    q = torch.empty(B, H, D).normal_(mean=0.1, std=0.2, generator=g).half()
    k = torch.empty(B * N, H, D).normal_(mean=0.1, std=0.2, generator=g).half()
    v = torch.empty(B * N, H, D).normal_(mean=0.1, std=10.0, generator=g).half()
    req_to_tokens = torch.arange(B * N, dtype=torch.int64).reshape(B, N)
    idx = torch.stack([torch.stack([torch.randperm(N, generator=g)[:topk] for _ in range(H)]) for _ in range(B)]).to(torch.int32)
    counts = torch.full((B, H), topk, dtype=torch.int32)
    out = torch.empty(B, H, D, dtype=torch.float16, device=DEV)
    ws = _ops.workspace(_ops.sparse_decode_workspace_bytes(B, H, topk), DEV)
    kd, vd = k.to(DEV), v.to(DEV)
    _ops.sparse_decode(q.to(DEV), _pool_views(kd, B), _pool_views(vd, B), idx.to(DEV), counts.to(DEV), 1 / math.sqrt(D), out, ws,
                       slots=req_to_tokens.to(torch.int32).to(DEV))
    ref = c_oracle.sparse_attend(q, orc.rows_through_slot_table(k, req_to_tokens), orc.rows_through_slot_table(v, req_to_tokens),
                                 idx.numpy(), counts.numpy(), 1 / math.sqrt(D))
    err = np.abs(out.float().cpu().numpy() - ref).max()
    print(f"max-abs error {err:.3e} (reference atol 1e-2)", flush=True)
    assert err <= 1e-2


def test_slot_table_arguments_are_validated():
    lib = _ops.load_library()
    t = torch.zeros(1 << 16, dtype=torch.uint8, device=DEV)
    p = t.data_ptr()
    import ctypes as C
    args = [p, 512, 128, p, p, _ops.HA_BF16, 0, 128, 256, 1, 1, 4, 2, p, 300, p, C.c_float(0.1), None, 0, 0, 0]
    tail = [p, p, 1 << 16, None]
    assert lib.ha_sparse_decode_paged(*args, None, 0, 100, *tail) == -1              # table missing
    assert lib.ha_sparse_decode_paged(*args, p, -1, 100, *tail) == -2                # negative stride
    assert lib.ha_sparse_decode_paged(*args, p, 0, 0, *tail) == -2                   # empty pool
    assert lib.ha_sparse_decode_paged(*args, p + 2, 0, 100, *tail) == -4             # misaligned table


@pytest.mark.parametrize("name", ["config2"])
def test_full_size_permuted_pool(name):
    # the headline shape with every token of every sequence at a random slot of one pool: fused and list-fed launches through
    # the table against the same launches on the contiguous cache (bit for bit), and the table-free output against the oracle
    # is covered by test_gpu_fullsize
    print(f"\n[case] paged cache at full size {name}", flush=True)
    w = named_workload(name)
    p = make_problem_on_device(w, DEV)
    B, H, Hkv, Hc, S, W = w.batch, w.n_q_heads, w.n_kv_heads, w.n_code_heads, w.max_seq_len, w.code_words
    from hashattention.decode import HashDecodeLayer
    layer = HashDecodeLayer(p.usa.k, p.usa.q, H, Hkv, 128, w.lth_num_layers, w.lth_int_dim, w.lth_final_dim, w.init_budget,
                            w.recent_budget, w.heavy_budget, device=DEV)
    layer.allocate(B, S)
    layer.encode_keys(p.k, use_mfma=True)
    layer.n_cached = S - 1
    out = torch.empty(B, H, 128, dtype=w.dtype, device=DEV)
    layer.step(p.q, p.k, p.v, S, out)                       # fused, contiguous cache
    g = torch.Generator(device=DEV).manual_seed(7)
    n_slots = B * S
    perm = torch.randperm(n_slots, generator=g, device=DEV).view(B, S)
    pool_k = torch.empty(n_slots, Hkv, 128, dtype=w.dtype, device=DEV)
    pool_v = torch.empty(n_slots, Hkv, 128, dtype=w.dtype, device=DEV)
    for b in range(B):
        pool_k[perm[b]] = p.k[b].transpose(0, 1)
        pool_v[perm[b]] = p.v[b].transpose(0, 1)
    slots = perm.to(torch.int32)
    kp, vp = _pool_views(pool_k, B), _pool_views(pool_v, B)
    q3 = p.q[:, :, 0]
    paged = torch.empty_like(out)
    _ops.sparse_decode_fused(q3, kp, vp, layer.codes, layer.qcodes.view(B, H, W), S, None, w.init_budget, w.recent_budget,
                             w.heavy_budget, layer.ws_select, layer.sm_scale, paged, layer.ws_fused,
                             thresholds_ready=not layer.local_thresholds, out_counts=layer.counts, slots=slots)
    torch.cuda.synchronize()
    assert torch.equal(paged, out), (paged.float() - out.float()).abs().max().item()
    layer.select(S, None)
    a, b2 = torch.empty_like(out), torch.empty_like(out)
    layer.attend(q3, p.k, p.v, a)
    _ops.sparse_decode(q3, kp, vp, layer.idx, layer.counts, layer.sm_scale, b2, layer.ws_attend, slots=slots)
    assert torch.equal(a, b2)
    assert (a.float() - out.float()).abs().max().item() <= 1e-2

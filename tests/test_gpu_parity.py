"""GPU parity: every stage of the HIP decode path, called through the C ABI, against the oracle.

Integer stages (codes from given logits' signs, Hamming distances, selected index lists, counts) must be
bit-exact; attention outputs within 2e-2 max-abs for bf16/fp16 and 2e-5 for fp32 of the double-precision
oracle.  Sizes are chosen so the oracle finishes in seconds.
"""
import numpy as np
import pytest
import torch

from hashattention import _ops
from tests.parity_util import run_decode_case, small_workload

pytestmark = pytest.mark.gpu


def _announce(name):
    print(f"\n[case] {name}", flush=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_small_decode_all_stages(dtype):
    _announce(f"small {dtype}")
    run_decode_case(small_workload(dtype=dtype), verbose=True)


def test_one_code_head_per_query_head():
    # reference-exact layout: every query head has its own K hash MLP (hashattention_llama.py:642)
    _announce("Hc == H")
    run_decode_case(small_workload(n_code_heads=8, seed=11), verbose=True)


@pytest.mark.parametrize("gq", [1, 2, 4, 8])
def test_group_sizes(gq):
    _announce(f"H/Hc = {gq}")
    run_decode_case(small_workload(n_q_heads=8, n_kv_heads=8 // gq, n_code_heads=8 // gq, seed=20 + gq), verbose=True)


def test_three_query_heads_per_kv_head():
    # 24 query heads on 8 KV heads (Llama-3.2-3B's ratio) in the reference's layout, one K hash MLP per query head: the gather
    # reads K/V through a group of three.  A code head shared by three query heads is refused, not mis-read.
    _announce("H/Hkv = 3, Hc == H")
    run_decode_case(small_workload(n_q_heads=6, n_kv_heads=2, n_code_heads=6, seed=31), verbose=True)
    run_decode_case(small_workload(batch=3, seq_lens=[9000, 4100, 77], n_q_heads=12, n_kv_heads=4, n_code_heads=12, seed=32))
    # wider groups than the dense kernel's eight slots: two passes over the KV head (12 = 8 + 4; 16 = 8 + 8, Llama-3.1-405B's ratio)
    run_decode_case(small_workload(n_q_heads=12, n_kv_heads=1, n_code_heads=12, seed=33))
    run_decode_case(small_workload(batch=2, seq_lens=[3000, 0], n_q_heads=32, n_kv_heads=2, n_code_heads=32, seed=34))
    dev = "cuda:0"
    kc = torch.zeros(1, 2, 256, 1, dtype=torch.int32, device=dev)
    qc = torch.zeros(1, 6, 1, 1, dtype=torch.int32, device=dev)
    ws = _ops.workspace(1 << 20, dev)
    with pytest.raises(_ops.HashAttnError, match="must be 1, 2, 4 or 8"):
        _ops.select(kc, qc, 256, torch.tensor([256], dtype=torch.int32, device=dev), 4, 4, 0.125,
                    torch.zeros(1, 6, 64, dtype=torch.int32, device=dev), torch.zeros(1, 6, dtype=torch.int32, device=dev), ws)


def test_64bit_codes_ragged():
    # 2-layer MLP, 64-bit codes (two words), ragged batch: the configs[4] shape in small
    _announce("W=2 ragged")
    w = small_workload(batch=3, seq_lens=[2300, 700, 1025], lth_num_layers=2, lth_final_dim=64, heavy_budget=1.0 / 16, seed=3)
    run_decode_case(w, verbose=True)


def test_one_layer_mlp():
    _announce("1-layer MLP")
    run_decode_case(small_workload(lth_num_layers=1, seed=5), verbose=True)


@pytest.mark.parametrize("seq_lens", [[1], [5, 31], [32, 33], [40, 64], [1024, 1023, 1025], [2048, 4097]])
def test_short_and_boundary_lengths(seq_lens):
    # init = recent = 16: lengths below, at and just above init + recent; chunk boundaries of the select kernels
    _announce(f"lengths {seq_lens}")
    run_decode_case(small_workload(batch=len(seq_lens), seq_lens=seq_lens, seed=100 + seq_lens[0]), verbose=True)


@pytest.mark.parametrize("heavy", [0.0, 0.5, 1.0, 40.0, 100000.0])
def test_heavy_budget_forms(heavy):
    # fraction of the length, 1.0 (fraction: everything), absolute count, absolute count above the candidates
    _announce(f"heavy_budget {heavy}")
    run_decode_case(small_workload(heavy_budget=heavy, seed=31), verbose=True)


@pytest.mark.parametrize("init,recent", [(0, 0), (0, 16), (16, 0), (128, 128)])
def test_window_forms(init, recent):
    _announce(f"init {init} recent {recent}")
    run_decode_case(small_workload(init_budget=init, recent_budget=recent, seed=41), verbose=True)


@pytest.mark.parametrize("depth", [0, 2, 40])
def test_threshold_mode(depth):
    # usa_eval_mode != 'simple': every candidate within the distance threshold, all ties (hashattention_llama.py:439-443)
    _announce(f"threshold depth {depth}")
    run_decode_case(small_workload(seed=51), mode="threshold", depth=depth, verbose=True)


def test_index_capacity_is_respected():
    # a list shorter than the selection: nothing is written past idx_cap, the count still reports the full size
    _announce("idx_cap clamp")
    from hashattention import _ops
    from oracle import c_oracle
    from tests.parity_util import oracle_codes, to_i32
    from hashattention.synthetic import make_problem
    w = small_workload(seed=61)
    p = make_problem(w)
    _, _, kc64, qc64 = oracle_codes(p)
    kc_np, qc_np = to_i32(kc64), to_i32(qc64)
    dev = "cuda:0"
    cap = 100
    guard = 64
    idx = torch.full((w.batch, w.n_q_heads, cap + guard), -7, dtype=torch.int32, device=dev)
    view = idx[:, :, :cap]
    # the ABI takes a contiguous [B, H, idx_cap] block: emulate a tight buffer followed by guard words
    tight = torch.full((w.batch * w.n_q_heads * cap + guard,), -7, dtype=torch.int32, device=dev)
    out_idx = tight[: w.batch * w.n_q_heads * cap].view(w.batch, w.n_q_heads, cap)
    counts = torch.zeros(w.batch, w.n_q_heads, dtype=torch.int32, device=dev)
    ws = _ops.workspace(_ops.select_workspace_bytes(w.batch, w.n_q_heads, w.n_code_heads, 1, w.max_seq_len), dev)
    _ops.select(torch.from_numpy(kc_np).to(dev), torch.from_numpy(qc_np).to(dev), w.max_seq_len, p.seq_lens.to(dev),
                w.init_budget, w.recent_budget, w.heavy_budget, out_idx, counts, ws)
    ref_idx, ref_counts = c_oracle.select(kc_np, qc_np, p.seq_lens.numpy(), w.init_budget, w.recent_budget, w.heavy_budget, cap)
    assert np.array_equal(counts.cpu().numpy(), ref_counts) and ref_counts.max() > cap
    assert np.array_equal(out_idx.cpu().numpy(), ref_idx)
    assert (tight[-guard:] == -7).all()
    del view


def test_config0_shape_fp32():
    # configs[0]: B=1, S=4096, 32 q heads / 8 KV heads, one K hash MLP per query head, fp32, heavy 0.25
    _announce("config0")
    from hashattention.synthetic import named_workload
    r = run_decode_case(named_workload("config0"), verbose=True)
    assert r["n_selected"] == 1280


ALGOS = {"histogram": 1, "sampled": 2, "sampled_exact_rows": 3}


@pytest.mark.parametrize("algo", list(ALGOS))
@pytest.mark.parametrize("case", ["plain", "ragged64", "threshold", "short", "big_budget", "gq1", "long"])
def test_every_select_algorithm_gives_the_same_lists(algo, case):
    # the three ways of finding the threshold (exact histogram, sampled guess, the guess's in-kernel exact path)
    # against the same oracle; "long" makes the sample a true subsample (more than 4096 candidates per row)
    _announce(f"select algo {algo} / {case}")
    kw = dict(check_encode=False, check_dense=False, algo=ALGOS[algo], verbose=True)
    if case == "plain":
        run_decode_case(small_workload(seed=201), **kw)
    elif case == "ragged64":
        run_decode_case(small_workload(batch=3, seq_lens=[2300, 700, 1025], lth_num_layers=2, lth_final_dim=64, seed=202), **kw)
    elif case == "threshold":
        run_decode_case(small_workload(seed=203), mode="threshold", depth=1, **kw)
    elif case == "short":
        run_decode_case(small_workload(batch=4, seq_lens=[1, 31, 33, 40], seed=204), **kw)
    elif case == "big_budget":      # more than half of the candidates kept: candidate segments overflow, rows go exact
        run_decode_case(small_workload(heavy_budget=0.7, seed=205), **kw)
    elif case == "gq1":
        run_decode_case(small_workload(n_code_heads=8, seed=206), **kw)
    else:
        run_decode_case(small_workload(batch=2, seq_lens=[20000, 9000], n_q_heads=4, n_kv_heads=1, n_code_heads=1,
                                       heavy_budget=1 / 32, seed=207), **kw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fused_path_equals_two_launch_path_on_unsplit_rows(dtype):
    # 512 rows: neither path splits a row; the LDS list holds the same tokens as ha_select's list (in another fixed order),
    # so the outputs agree to fp32 summation order (fp32 caches) or one rounding of the output (bf16)
    _announce(f"fused vs two-launch, unsplit rows, {dtype}")
    from hashattention import _ops
    from hashattention.synthetic import make_problem
    from tests.parity_util import oracle_codes, to_i32
    import math
    w = small_workload(batch=16, seq_lens=[3000 + 37 * i for i in range(16)], n_q_heads=32, n_kv_heads=8, n_code_heads=8,
                       init_budget=16, recent_budget=16, heavy_budget=1 / 16, seed=401, dtype=dtype)
    p = make_problem(w)
    _, _, kc64, qc64 = oracle_codes(p)
    dev = "cuda:0"
    B, H, Hc, S, d = w.batch, w.n_q_heads, w.n_code_heads, w.max_seq_len, w.head_dim
    kc, qc = torch.from_numpy(to_i32(kc64)).to(dev), torch.from_numpy(to_i32(qc64)).to(dev)
    q3, k, v, seq = p.q[:, :, 0, :].contiguous().to(dev), p.k.to(dev), p.v.to(dev), p.seq_lens.to(dev)
    cap = max(w.n_selected(s) for s in w.seq_lens)
    idx = torch.empty(B, H, cap, dtype=torch.int32, device=dev)
    counts = torch.empty(B, H, dtype=torch.int32, device=dev)
    ws = _ops.workspace(_ops.select_workspace_bytes(B, H, Hc, 1, S), dev)
    wa = _ops.workspace(_ops.sparse_decode_workspace_bytes(B, H, cap), dev)
    wf = _ops.workspace(_ops.sparse_decode_fused_workspace_bytes(B, H, Hc, S), dev)
    out_a, out_b = torch.empty(B, H, d, dtype=w.dtype, device=dev), torch.empty(B, H, d, dtype=w.dtype, device=dev)
    sm = 1.0 / math.sqrt(d)
    _ops.select(kc, qc, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, idx, counts, ws)
    _ops.sparse_decode(q3, k, v, idx, counts, sm, out_a, wa)
    counts2 = torch.empty_like(counts)
    _ops.select_prepare(kc, qc, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, counts2, ws)
    _ops.sparse_decode_fused(q3, k, v, kc, qc, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, ws, sm, out_b, wf)
    assert torch.equal(counts, counts2)
    diff = (out_a.float() - out_b.float()).abs().max().item()
    assert diff <= (5e-6 if dtype == torch.float32 else 8e-3), diff
    # and a second call gives the same bits: the order inside the list is fixed
    out_c = torch.empty_like(out_b)
    _ops.sparse_decode_fused(q3, k, v, kc, qc, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, ws, sm, out_c, wf)
    assert torch.equal(out_b, out_c)


def _random_workload(rng, i):
    H, Hkv = [(8, 2), (4, 4), (8, 8), (16, 2), (32, 8), (4, 1)][rng.integers(6)]
    Hc = [Hkv, H][rng.integers(2)]
    B = int(rng.integers(1, 10))
    top = int(rng.choice([40, 700, 3000, 9000, 20000]))
    if rng.integers(2):
        lens = [int(rng.integers(max(1, top // 8), top + 1)) for _ in range(B)]
    else:
        lens = [int(rng.integers(max(1, top // 2), top + 1))] * B
    wide = bool(rng.integers(2))
    heavy = float(rng.choice([0.0, 1.0 / 32, 0.125, 0.5, 1.0, 37.0, 300.0]))
    return small_workload(name=f"random{i}", batch=B, seq_lens=lens, n_q_heads=H, n_kv_heads=Hkv, n_code_heads=Hc,
                          lth_num_layers=2 if wide else 3, lth_final_dim=64 if wide else 32,
                          init_budget=int(rng.choice([0, 4, 16, 128])), recent_budget=int(rng.choice([0, 1, 16, 128])),
                          heavy_budget=heavy, dtype=[torch.bfloat16, torch.float16, torch.float32][rng.integers(3)], seed=100 + i)


@pytest.mark.parametrize("block", range(8))
def test_random_shapes_every_stage_against_the_oracle(block):
    # seeded sweep over batch sizes, head layouts, ragged and equal lengths, code widths, budgets and dtypes: every
    # stage of every case against the oracle, the fused launch with its in-kernel plan included
    rng = np.random.default_rng(2024 + block)
    for i in range(8):
        w = _random_workload(rng, block * 8 + i)
        print(f"\n[case] {w.name}: B={w.batch} H={w.n_q_heads}/{w.n_kv_heads}/{w.n_code_heads} S={w.seq_lens} bits={w.lth_final_dim} "
              f"init={w.init_budget} recent={w.recent_budget} heavy={w.heavy_budget} {w.dtype}", flush=True)
        run_decode_case(w, check_encode=False, check_dense=False)


@pytest.mark.parametrize("heavy,fused", [(8000.5, True), (8001.5, False)])
def test_largest_list_of_the_fused_path(heavy, fused):
    # the fused launch keeps a row's list in LDS, 8192 entries at most: a selection of exactly that size goes through it
    # (every stage against the oracle, as in the other cases), one entry more is refused by it and served by the list path
    print(f"\n[case] list of {int(heavy) + 192} entries", flush=True)
    w = small_workload(batch=2, seq_lens=[30000, 30000], n_q_heads=4, n_kv_heads=2, n_code_heads=2, init_budget=100, recent_budget=92,
                       heavy_budget=heavy, seed=91)
    assert bool(_ops.fused_applies(2, 4, 2, 1, 30000, 100, 92, heavy)) == fused
    rep = run_decode_case(w, check_encode=False, check_dense=False, verbose=True)
    assert rep["n_selected"] == int(heavy) + 192 and ("fused_err" in rep) == fused


@pytest.mark.parametrize("batch,heads", [(140, 1), (130, 2)])
def test_ragged_batch_larger_than_the_in_kernel_plan(batch, heads):
    # the fused launch plans ragged batches of up to 128 sequences inside the kernel; beyond that every row keeps the
    # pieces the host sized for the longest sequence (with one head per sequence the rows are cut into pieces, with two
    # they are not).  Every stage against the oracle.
    print(f"\n[case] ragged batch of {batch} sequences, {heads} head(s)", flush=True)
    rng = np.random.default_rng(5 + batch)
    lens = [int(x) for x in rng.integers(700, 5000, batch)]
    lens[3], lens[7] = 17, 4999                      # one shorter than its windows, one at the top
    w = small_workload(batch=batch, seq_lens=lens, n_q_heads=heads, n_kv_heads=1, n_code_heads=1, init_budget=16, recent_budget=24,
                       heavy_budget=0.05, seed=93)
    rep = run_decode_case(w, check_encode=False, check_dense=False, verbose=True)
    assert "fused_err" in rep


@pytest.mark.parametrize("lens,heads,bits,heavy", [([70000, 70000], (8, 2, 2), 32, 1.0 / 32), ([131072], (4, 4, 4), 64, 0.002),
                                                    ([52000, 90000, 33000], (8, 8, 8), 32, 1500.0), ([200000], (16, 4, 4), 32, 7000.0)])
def test_long_rows_cut_into_pieces_of_equal_work(lens, heads, bits, heavy):
    # few long rows: the fused launch cuts every row into pieces whose boundaries follow the selected rows and the chunks to
    # scan (every workgroup of a row derives them from the row's chunk prefixes), with the lengths on the host (one workgroup
    # per CU, scan codes requested a round ahead) and on the device (in-kernel plan).  Every stage against the oracle.
    print(f"\n[case] long rows {lens} heads={heads} bits={bits} heavy={heavy}", flush=True)
    w = small_workload(name="long", batch=len(lens), seq_lens=lens, n_q_heads=heads[0], n_kv_heads=heads[1], n_code_heads=heads[2],
                       lth_num_layers=2 if bits == 64 else 3, lth_final_dim=bits, init_budget=128, recent_budget=16,
                       heavy_budget=heavy, dtype=torch.bfloat16, seed=77)
    rep = run_decode_case(w, check_encode=False, check_dense=False, verbose=True)
    assert "fused_err" in rep


@pytest.mark.parametrize("batch,heads,lens,dtype", [(16, (32, 8, 8), "uniform", torch.bfloat16), (16, (32, 8, 16), "ragged", torch.bfloat16),
                                                     (64, (8, 4, 4), "ragged", torch.float16), (40, (16, 2, 2), "short", torch.bfloat16)])
def test_grids_of_512_rows_and_more(batch, heads, lens, dtype):
    # 512 and more (sequence, head) rows: more fused workgroups than the device holds at once (two per CU), query heads that
    # share a code head and scan the same codes side by side.  Equal lengths (on the host and on the device), ragged lengths
    # (in-kernel plan), rows shorter than their windows.  Every stage against the oracle.
    print(f"\n[case] many rows: B={batch} heads={heads} lengths {lens} {dtype}", flush=True)
    rng = np.random.default_rng(batch + heads[0])
    if lens == "uniform":
        seq_lens = [9000] * batch
    elif lens == "ragged":
        seq_lens = [int(x) for x in rng.integers(1500, 9000, batch)]
    else:
        seq_lens = [int(x) for x in rng.integers(1, 1300, batch)]
        seq_lens[0], seq_lens[1] = 1, 40
    w = small_workload(name="many_rows", batch=batch, seq_lens=seq_lens, n_q_heads=heads[0], n_kv_heads=heads[1], n_code_heads=heads[2],
                       init_budget=32, recent_budget=48, heavy_budget=1.0 / 16, dtype=dtype, seed=101)
    assert batch * heads[0] >= 512
    rep = run_decode_case(w, check_encode=False, check_dense=False, verbose=True)
    assert "fused_err" in rep


@pytest.mark.parametrize("tokens,heads", [(1 << 20, (2, 1, 1)), (300001, (4, 2, 2)), (1 << 19, (8, 8, 8))])
def test_rows_of_many_chunks_through_the_fused_path(tokens, heads):
    # rows of more than 256 chunks (few code heads: chunks of 1024 tokens, up to 1024 of them here): a fused workgroup keeps only
    # the chunk prefixes of its own piece in LDS, pieces hold at most 256 chunks, thresholds come from ha_select_prepare (more
    # than 64 chunks).  With 8 code heads the same length has 256 chunks and the whole row's prefixes fit.  Every stage against
    # the oracle.
    print(f"\n[case] row of {tokens} tokens, heads {heads}", flush=True)
    w = small_workload(name="many_chunks", batch=1, seq_lens=[tokens], n_q_heads=heads[0], n_kv_heads=heads[1], n_code_heads=heads[2],
                       init_budget=64, recent_budget=64, heavy_budget=4000.0, dtype=torch.bfloat16, seed=17)
    assert _ops.fused_applies(1, heads[0], heads[2], 1, tokens, 64, 64, 4000.0)
    rep = run_decode_case(w, check_encode=False, check_dense=False, verbose=True)
    assert "fused_err" in rep

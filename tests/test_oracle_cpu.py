"""Pins of the CPU oracle that need no fixture: known-answer patterns of the reference's own self-tests,
closed forms, invariants and brute force on tiny inputs, chosen so that a plausible slip (a wrong bit order, an
off-by-one window, a dropped term, a transposed operand) fails at least one of them."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle
from oracle import hashattn_oracle as orc


# ---------------------------------------------------------------- popcount / Hamming
def test_popcount_known_answers_like_the_reference_selftest():
    # efficiency/kernels/bit_count_uint32.py:36-58: seed 42, shape (10, 20, 30), against bin(x).count('1')
    torch.manual_seed(42)
    x = torch.randint(0, 2 ** 32 - 1, (10, 20, 30), dtype=torch.int64)
    want = torch.tensor([bin(v).count("1") for v in x.reshape(-1).tolist()]).reshape(x.shape)
    assert torch.equal(orc.popcount_u32(x), want)
    # the C oracle: distance to an all-zero query code is the popcount
    kc = x.reshape(10, 20, 30, 1).numpy().astype(np.uint32)
    ham = c_oracle.hamming(kc, np.zeros((10, 20, 1), dtype=np.uint32), [30] * 10)
    assert np.array_equal(ham, want.numpy().astype(np.uint8))
    # 64-bit codes as two words (bit_count_long.py:36-58: randint below 2**63)
    y = torch.randint(0, 2 ** 63 - 1, (6, 5, 30), dtype=torch.int64)
    want64 = np.array([bin(v).count("1") for v in y.reshape(-1).tolist()]).reshape(6, 5, 30)
    two = np.stack([(y.numpy() & 0xFFFFFFFF), (y.numpy() >> 32)], axis=-1).astype(np.uint32)
    assert np.array_equal(c_oracle.hamming(two, np.zeros((6, 5, 2), dtype=np.uint32), [30] * 6), want64.astype(np.uint8))
    assert torch.equal(orc.hamming(torch.zeros(6, 5, 2, dtype=torch.int64), torch.from_numpy(two.astype(np.int64))),
                       torch.from_numpy(want64))


def test_pack_bit_order_and_span_identity():
    # bit i = (logit_i > 0), least significant bit = dim 0 (efficiency/kernels/torchatt.py:55-56, 159)
    lg = -torch.ones(1, 64)
    lg[0, 0] = 1.0
    lg[0, 33] = 2.0
    assert orc.pack_codes(lg).tolist() == [[1, 2]]
    assert orc.pack_codes(torch.ones(3, 32)).tolist() == [[0xFFFFFFFF]] * 3
    assert orc.pack_codes(torch.zeros(3, 32)).tolist() == [[0]] * 3            # sign(0) = 0 -> relu -> bit 0
    # permuting output dims permutes bits
    g = torch.Generator().manual_seed(0)
    x = torch.randn(50, 32, generator=g)
    perm = torch.randperm(32, generator=g)
    a, b = orc.pack_codes(x)[:, 0], orc.pack_codes(x[:, perm])[:, 0]
    for i in range(32):
        assert torch.equal((b >> i) & 1, (a >> perm[i]) & 1)
    # span = <sign q, sign k> = D - 2 * Hamming when no logit is exactly zero (hashattention_llama.py:180-187)
    q, k = torch.randn(7, 32, generator=g), torch.randn(11, 32, generator=g)
    span = torch.sign(q) @ torch.sign(k).T
    ham = orc.popcount_u32(orc.pack_codes(q)[:, None, 0] ^ orc.pack_codes(k)[None, :, 0])
    assert torch.equal(span, (32 - 2 * ham).float())
    # ... and differs exactly by the zero coordinates otherwise: the +-1/0 and the bit formulation part ways
    q[0, 5] = 0.0
    span0 = torch.sign(q[0]) @ torch.sign(k).T
    ham0 = orc.popcount_u32(orc.pack_codes(q[:1])[:, None, 0] ^ orc.pack_codes(k)[None, :, 0])[0]
    assert torch.equal(span0 + (-torch.sign(k[:, 5])), (32 - 2 * ham0).float())    # bit 0 acts as sign -1


# ---------------------------------------------------------------- hash MLP
def test_usa_mlp_closed_form_and_c_encode():
    g = torch.Generator().manual_seed(1)
    layers = [(torch.randn(8, 4, generator=g), torch.randn(8, generator=g)), (torch.randn(32, 8, generator=g), torch.randn(32, generator=g))]
    x = torch.randn(5, 4, generator=g)
    want = torch.empty(5, 32)
    for r in range(5):
        h = [sum(x[r, k] * layers[0][0][o, k] for k in range(4)) + layers[0][1][o] for o in range(8)]
        h = [v / (1 + math.exp(-v)) for v in h]                                    # SiLU
        for o in range(32):
            want[r, o] = sum(h[k] * layers[1][0][o, k] for k in range(8)) + layers[1][1][o]
    got = orc.usa_mlp(x, layers)
    assert torch.allclose(got, want, atol=1e-5)
    lg, codes = c_oracle.encode(x.numpy(), [(W.numpy(), b.numpy()) for W, b in layers])
    assert np.abs(lg - want.numpy()).max() < 1e-5
    assert np.array_equal(codes[:, 0], orc.pack_codes(want).numpy().astype(np.uint32)[:, 0])
    # all-zero weights and a positive bias: every bit set
    z = [(torch.zeros(32, 4), torch.ones(32))]
    assert (c_oracle.encode(x.numpy(), [(z[0][0].numpy(), z[0][1].numpy())])[1] == 0xFFFFFFFF).all()
    # head i of the MLP list reads input head i // rep
    heads = [[(torch.eye(32, 4) * (i + 1), torch.zeros(32))] for i in range(4)]
    xin = torch.randn(1, 2, 3, 4, generator=g)
    out = orc.usa_logits(xin, heads)
    for i in range(4):
        assert torch.allclose(out[0, i, :, :4], xin[0, i // 2] * (i + 1))


# ---------------------------------------------------------------- selection
def _brute(ham_row, S, init, recent, k):
    lo, hi = min(init, S), max(min(init, S), S - recent)
    cand = sorted(range(lo, hi), key=lambda j: (ham_row[j], j))[:min(k, hi - lo)]
    return sorted(set(range(lo)) | set(cand) | set(range(hi, S)))


@pytest.mark.parametrize("S,init,recent,hb", [(1, 4, 4, 0.5), (8, 4, 4, 0.5), (9, 4, 4, 0.5), (40, 4, 6, 0.25), (40, 0, 0, 0.1),
                                               (40, 0, 5, 7.0), (40, 3, 0, 1.0), (200, 16, 16, 0.03125), (64, 50, 60, 0.5),
                                               (33, 1, 1, 100.0), (50, 2, 2, 0.0)])
def test_selection_three_ways(S, init, recent, hb):
    g = torch.Generator().manual_seed(S * 7 + init)
    H = 3
    kc = torch.randint(0, 2 ** 32, (1, H, S, 1), generator=g, dtype=torch.int64)
    qc = torch.randint(0, 2 ** 32, (1, H, 1), generator=g, dtype=torch.int64)
    ham = orc.hamming(qc, kc)[0]                                                   # [H, S]
    k = orc.heavy_count(S, hb)
    want = [_brute(ham[h].tolist(), S, init, recent, k) for h in range(H)]
    assert orc.select_indices(ham, S, init, recent, hb) == want
    idx, cnt = c_oracle.select(kc.numpy().astype(np.uint32), qc.numpy().astype(np.uint32), [S], init, recent, hb, S)
    assert [idx[0, h, :cnt[0, h]].tolist() for h in range(H)] == want
    assert np.array_equal(orc.select_indices_np(ham.numpy(), S, init, recent, hb), np.array(want))
    # the reference's mask construction (tril / masked_fill / sort / scatter) on span = 32 - 2 * ham, query row q = 1
    span = (32 - 2 * ham).float()[None, :, None, :]
    mask = orc.compute_mask_multi(span, init, recent, hb)[0, :, 0]
    assert torch.equal(mask, orc.mask_from_indices(want, S))
    # an unstable sort may pick other members of the tie bucket, never another count or another score multiset
    mask_u = orc.compute_mask_multi(span, init, recent, hb, stable=False)[0, :, 0]
    assert orc.tie_invariant_equal(mask, mask_u, span[0, :, 0])


def test_heavy_count_truncation():
    # int(k * heavy_budget) in double arithmetic; > 1.0 means an absolute count (hashattention_llama.py:431-434)
    assert orc.heavy_count(4096, 0.25) == 1024 and orc.heavy_count(65536, 1 / 32) == 2048
    assert orc.heavy_count(7, 0.3) == 2 and orc.heavy_count(10, 0.29) == 2 and orc.heavy_count(100, 0.07) == 7
    assert orc.heavy_count(50, 1.0) == 50 and orc.heavy_count(50, 2.5) == 2 and orc.heavy_count(50, 1.5) == 1


@pytest.mark.parametrize("depth", [0, 1, 3, 40])
def test_threshold_mode(depth):
    # every candidate with span >= max(top - 2*depth, k-th value), all ties kept (hashattention_llama.py:439-443)
    g = torch.Generator().manual_seed(depth)
    S, init, recent, hb = 120, 5, 7, 0.1
    kc = torch.randint(0, 2 ** 32, (1, 2, S, 1), generator=g, dtype=torch.int64)
    qc = torch.randint(0, 2 ** 32, (1, 2, 1), generator=g, dtype=torch.int64)
    ham = orc.hamming(qc, kc)[0]
    span = (32 - 2 * ham).float()[None, :, None, :]
    mask = orc.compute_mask_multi(span, init, recent, hb, mode="thold", retrieve_depth=depth)[0, :, 0]
    sel = orc.select_indices(ham, S, init, recent, hb, mode="thold", retrieve_depth=depth)
    assert torch.equal(mask, orc.mask_from_indices(sel, S))
    idx, cnt = c_oracle.select(kc.numpy().astype(np.uint32), qc.numpy().astype(np.uint32), [S], init, recent, hb, S, mode=1, depth=depth)
    assert [idx[0, h, :cnt[0, h]].tolist() for h in range(2)] == sel
    for h in range(2):
        cand = list(range(init, S - recent))
        ds = sorted(ham[h, j].item() for j in cand)
        th = min(ds[0] + depth, ds[orc.heavy_count(S, hb) - 1])
        assert sorted(set(sel[h]) - set(range(init)) - set(range(S - recent, S))) == [j for j in cand if ham[h, j] <= th]


# ---------------------------------------------------------------- attention
def test_attention_special_cases():
    g = torch.Generator().manual_seed(2)
    b, H, Hkv, S, d = 2, 4, 2, 37, 16
    Q, K, V = torch.randn(b, H, 1, d, generator=g), torch.randn(b, Hkv, S, d, generator=g), torch.randn(b, Hkv, S, d, generator=g)
    Kr, Vr = orc.repeat_kv(K, 2), orc.repeat_kv(V, 2)
    assert torch.equal(Kr[:, 1], K[:, 0]) and torch.equal(Kr[:, 2], K[:, 1])      # repeat_interleave, not tile
    # an all-True mask is plain attention
    full = orc.masked_decode_attention(Q, Kr, Vr, torch.ones(b, H, 1, S, dtype=torch.bool))
    assert torch.allclose(full, F.scaled_dot_product_attention(Q, Kr, Vr), atol=1e-6)
    assert torch.allclose(full, orc.dense_attention(Q, Kr, Vr), atol=1e-6)
    # a masked row equals gather-only attention over the kept indices, and the C oracle agrees
    mask = torch.rand(b, H, 1, S, generator=g) < 0.3
    mask[..., 0] = True
    dense = orc.masked_decode_attention(Q, Kr, Vr, mask)
    idx = np.full((b, H, S), -1, dtype=np.int32)
    cnt = np.zeros((b, H), dtype=np.int32)
    for bb in range(b):
        for h in range(H):
            ii = mask[bb, h, 0].nonzero()[:, 0]
            idx[bb, h, :len(ii)] = ii.numpy()
            cnt[bb, h] = len(ii)
            o = orc.sparse_attend(Q[bb, h, 0], K[bb, h // 2], V[bb, h // 2], ii, 1 / math.sqrt(d))
            assert torch.allclose(o, dense[bb, h, 0], atol=1e-6)
    co = c_oracle.sparse_attend(Q[:, :, 0], K, V, idx, cnt, 1 / math.sqrt(d))
    assert np.abs(co - dense[:, :, 0].numpy()).max() < 1e-6
    cd = c_oracle.dense_attend(Q[:, :, 0], K, V, [S, S - 5], 1 / math.sqrt(d))
    assert np.abs(cd[0] - full[0, :, 0].numpy()).max() < 1e-6
    short = orc.dense_attention(Q[1:], Kr[1:, :, :S - 5], Vr[1:, :, :S - 5])
    assert np.abs(cd[1] - short[0, :, 0].numpy()).max() < 1e-6
    # split-K merge is exact log-sum-exp algebra
    q, k, v = Q[0, 0, 0], K[0, 0], V[0, 0]
    whole = orc.sparse_attend(q, k, v, range(S), 0.25)
    parts, lses = [], []
    for lo, hi in ((0, 10), (10, 11), (11, S)):
        a = (k[lo:hi] @ q) * 0.25
        parts.append(torch.softmax(a, 0) @ v[lo:hi])
        lses.append(torch.logsumexp(a, 0))
    assert torch.allclose(orc.merge_splits(torch.stack(parts), torch.stack(lses)), whole, atol=1e-6)


def test_rope_is_a_rotation_of_half_pairs():
    g = torch.Generator().manual_seed(3)
    d, t = 8, 5
    q, k = torch.randn(1, 2, t, d, generator=g), torch.randn(1, 1, t, d, generator=g)
    ang = torch.randn(1, t, d // 2, generator=g)
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1), torch.cat([ang.sin(), ang.sin()], -1)
    qe, ke = orc.apply_rotary_pos_emb(q, k, cos, sin)
    zq = torch.complex(q[..., :d // 2], q[..., d // 2:]) * torch.polar(torch.ones_like(ang), ang).unsqueeze(1)
    assert torch.allclose(qe, torch.cat([zq.real, zq.imag], -1), atol=1e-6)
    assert torch.allclose(qe.norm(dim=-1), q.norm(dim=-1), atol=1e-5) and torch.allclose(ke.norm(dim=-1), k.norm(dim=-1), atol=1e-5)


def test_reference_decode_attention_is_consistent_with_its_stages():
    from hashattention.synthetic import make_problem
    from tests.parity_util import small_workload
    w = small_workload(batch=1, seq_lens=[300], dtype=torch.float32, n_code_heads=8)
    p = make_problem(w)
    out, mask = orc.reference_decode_attention(p.q, p.k, p.v, p.usa.k, p.usa.q, w.init_budget, w.recent_budget, w.heavy_budget)
    kc = orc.pack_codes(orc.usa_logits(orc.repeat_kv(p.k, 4), p.usa.k))
    qc = orc.pack_codes(orc.usa_logits(p.q, p.usa.q))[:, :, 0]
    sel = orc.select_indices(orc.hamming(qc, kc)[0], 300, w.init_budget, w.recent_budget, w.heavy_budget)
    assert torch.equal(mask[0, :, 0], orc.mask_from_indices(sel, 300))
    for h in range(w.n_q_heads):
        o = orc.sparse_attend(p.q[0, h, 0], p.k[0, h // 4], p.v[0, h // 4], sel[h], 1 / math.sqrt(128))
        assert torch.allclose(o, out[0, h, 0], atol=1e-5)


def test_recall_overlap_is_pinned_by_its_special_cases_and_a_verbatim_restatement():
    # (1) when S // 16 covers every candidate the statistic is min(32, #candidates) / 32 whatever the hashes say;
    # (2) the dense formulation written as the reference writes it (masked logits, two torch.topk, scatter, product:
    #     hashattention_llama.py:357-386) must lie between the canonical value with the boundary ties of the hash score
    #     all left out and all taken in - torch.topk is free to pick any of them
    import math
    from hashattention.synthetic import make_usa_weights, Workload
    g = torch.Generator().manual_seed(11)
    w = Workload("t", 1, [96], n_q_heads=4, n_kv_heads=2, n_code_heads=4, lth_int_dim=32, seed=2)
    usa = make_usa_weights(w)
    S, q_len, init, recent = 96, 40, 4, 6
    k = torch.randn(1, 2, S, 128, generator=g)
    q = torch.randn(1, 4, q_len, 128, generator=g)
    got = orc.recall_overlap(q, k, usa.k, usa.q, init, recent, top_true=3)                  # S // 16 = 6 predictions
    # verbatim restatement
    kk = orc.repeat_kv(k, 2)
    logits = torch.matmul(q, kk.transpose(2, 3)) / math.sqrt(128)
    keep = torch.tril(torch.ones(q_len, S), diagonal=S - q_len - recent).bool()
    keep[:, :init] = False
    logits = logits.masked_fill(~keep, torch.finfo(logits.dtype).min)
    target = torch.zeros_like(logits)
    target.scatter_(-1, torch.topk(logits, 3, dim=-1).indices, 1.0)
    span, _ = orc.usa_forward_hard(kk, q, usa.k, usa.q)
    span = span.masked_fill(~keep, torch.finfo(span.dtype).min)
    pred = torch.zeros_like(span)
    pred.scatter_(-1, torch.topk(span, S // 16, dim=-1).indices, 1.0)
    verbatim = (pred * target).sum(-1) / target.sum(-1)
    # bounds from the threshold value of the hash score
    thr = torch.topk(span, S // 16, dim=-1).values[..., -1:]
    lower = ((span > thr).float() * target).sum(-1) / 3
    upper = ((span >= thr).float() * target).sum(-1) / 3
    rows = keep.sum(-1) >= S // 16                                                          # rows whose candidates fill the prediction
    assert rows.any()
    assert ((verbatim >= lower - 1e-6) & (verbatim <= upper + 1e-6))[..., rows].all()
    assert ((got >= lower - 1e-6) & (got <= upper + 1e-6))[..., rows].all()
    assert (upper - lower)[..., rows].abs().max() <= 1.0 and (got[..., rows] > 0).any()
    # special case: predictions cover all candidates
    few = orc.recall_overlap(q, k, usa.k, usa.q, init, S - q_len - 5, top_true=3)            # at most ~ q_len candidates... per row i: i + 2
    ncand = torch.clamp(torch.arange(q_len) + S - q_len - (S - q_len - 5) - init + 1, min=0)
    full = ncand <= S // 16
    want = torch.clamp(ncand, max=3).float() / 3
    assert torch.allclose(few[0, :, full], want[full].expand(4, -1))


def test_additive_masks_of_the_oracle():
    """`attention_mask` of the dense formulation (hashattention_llama.py:593-598) and the slot mask of the gather formulation
    (sparse.py:207), pinned by what the mathematics fixes: -inf removes an entry (equals attending without it), a constant
    changes nothing, the dense form equals torch's scaled_dot_product_attention with the summed masks, and the two
    formulations agree when the slot mask is the position mask gathered through the list."""
    g = torch.Generator().manual_seed(5)
    b, H, S, d = 2, 3, 50, 16
    Q, K, V = torch.randn(b, H, 1, d, generator=g), torch.randn(b, H, S, d, generator=g), torch.randn(b, H, S, d, generator=g)
    keep = torch.rand(b, H, 1, S, generator=g) < 0.6
    keep[..., 0] = True
    am = torch.randn(b, 1, 1, S, generator=g)
    am[:, :, :, 5:9] = float("-inf")
    out = orc.masked_decode_attention(Q, K, V, keep, am)
    sdpa = torch.nn.functional.scaled_dot_product_attention(Q, K, V, attn_mask=am.expand(b, H, 1, S).masked_fill(~keep, float("-inf")))
    assert (out - sdpa).abs().max().item() < 1e-5
    # the gather formulation with the position mask gathered through the list
    for bi in range(b):
        for h in range(H):
            idx = torch.nonzero(keep[bi, h, 0]).flatten()
            got = orc.sparse_attend(Q[bi, h, 0], K[bi, h], V[bi, h], idx.numpy(), 1 / d ** 0.5, slot_mask=am[bi, 0, 0, idx])
            assert (got - out[bi, h, 0]).abs().max().item() < 1e-5
            # -inf on a slot == the list without that slot; a constant shift == no mask
            live = torch.isfinite(am[bi, 0, 0, idx])
            short = orc.sparse_attend(Q[bi, h, 0], K[bi, h], V[bi, h], idx[live].numpy(), 1 / d ** 0.5, slot_mask=am[bi, 0, 0, idx[live]])
            assert (short - got).abs().max().item() < 1e-6
            plain = orc.sparse_attend(Q[bi, h, 0], K[bi, h], V[bi, h], idx.numpy(), 1 / d ** 0.5)
            shifted = orc.sparse_attend(Q[bi, h, 0], K[bi, h], V[bi, h], idx.numpy(), 1 / d ** 0.5, slot_mask=torch.full((len(idx),), 1.5))
            assert (plain - shifted).abs().max().item() < 1e-6
            assert (plain - got).abs().max().item() > 1e-3          # and the random mask does change the result


def test_rows_through_slot_table_against_loops_and_the_prototypes_identity_table():
    # `K[Req_to_tokens[b, idx] * stride_kbs + kv_head * stride_kh]` (flash_fwd_sparse.py:466-474) written as explicit loops, and
    # the table the prototype builds (torchatt.py:165, arange(B * N).reshape(B, N)), under which the pool IS the token-major
    # cache that torch_fwd_sparse views as K.view(B, -1, H, D) (sparse.py:196-203): the two reference files must agree
    g = torch.Generator().manual_seed(12)
    B, N, H, D, spare = 3, 17, 2, 4, 5
    pool = torch.randn(B * N + spare, H, D, generator=g)
    table = torch.randperm(B * N + spare, generator=g)[:B * N].view(B, N)
    got = orc.rows_through_slot_table(pool, table)
    assert got.shape == (B, H, N, D)
    for b in range(B):
        for h in range(H):
            for j in range(N):
                assert torch.equal(got[b, h, j], pool[int(table[b, j]), h])
    flat = pool[:B * N]
    identity = torch.arange(B * N).reshape(B, N)
    assert torch.equal(orc.rows_through_slot_table(flat, identity), flat.view(B, N, H, D).permute(0, 2, 1, 3))
    # a transposed table (a plausible mistake: [S, B]) does not reproduce the loops
    assert not torch.equal(orc.rows_through_slot_table(pool, table.t().contiguous().view(B, N)), got)

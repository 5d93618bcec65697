"""The reference prototype's own self-checks, with its recipes, layouts and calling conventions, through the HIP path.

(a) `test_fwd_sparse` (efficiency/kernels/sparse.py:217-254): B=32, N=2048, MHA H=32, D=128, 128 list entries per row in
    `randperm` order (NOT sorted), fp16 N(0.1, 0.2), K/V allocated token-major [B*N, H, D] and handed over as strided
    [B, H, N, D] views, `Mask` zero and random; checked against `torch_fwd_sparse`'s restatement (oracle.sparse_attend)
    at the reference's atol 1e-3.
(b) `test_flash_correctness` (efficiency/kernels/torchatt.py:143-165, 208-262): V ~ N(0.1, 10), hash weights [H, D, D]
    applied as x @ W with [H, 1, D] biases (one set for keys and queries), k = N / 32, no sink or recent window, index
    lists fed in ascending order, in `topk` order (by score) and rebuilt in LDS by the fused launch; atol 1e-2 as there.
    The prototype's MLP runs in fp16; here the fp16 rows go through the fp32 arithmetic of the encode kernel and the
    oracle follows that (fp16 arithmetic of cuBLAS is not reproducible on a CPU), so codes are compared with the
    fp32 oracle and everything behind the codes is exact.
The list order is free: the output depends on it only through the order of fp32 additions.
"""
import math

import numpy as np
import pytest
import torch

from hashattention import _ops
from oracle import c_oracle
from oracle import hashattn_oracle as orc
from tests.parity_util import compare_codes, to_i32

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _token_major(B, N, H, D, mean, std, g, dtype=torch.float16):
    """A [B*N, H, D] allocation as the prototype makes it, and its [B, H, N, D] strided view (no copy)."""
    flat = torch.empty(B * N, H, D).normal_(mean=mean, std=std, generator=g).to(dtype)
    return flat, flat.view(B, N, H, D).permute(0, 2, 1, 3)


@pytest.mark.parametrize("random_mask", [False, True])
def test_fwd_sparse_recipe_token_major_unsorted_lists(random_mask):
    print(f"\n[case] sparse.py test_fwd_sparse recipe, random_mask={random_mask}", flush=True)
    B, N, H, D, HEAVY = 32, 2048, 32, 128, 128
    g = torch.Generator().manual_seed(217)
    q = torch.empty(B, H, D).normal_(mean=0.1, std=0.2, generator=g).half()
    k_flat, k_view = _token_major(B, N, H, D, 0.1, 0.2, g)
    v_flat, v_view = _token_major(B, N, H, D, 0.1, 0.2, g)
    heavy = torch.stack([torch.stack([torch.randperm(N, generator=g)[:HEAVY] for _ in range(H)]) for _ in range(B)]).to(torch.int32)
    counts = torch.full((B, H), HEAVY, dtype=torch.int32)
    mask = torch.zeros(B, HEAVY)
    if random_mask:
        mask = torch.randn(B, HEAVY, generator=g).half().float()        # the prototype's Mask is fp16
    kd, vd = k_flat.to(DEV).view(B, N, H, D).permute(0, 2, 1, 3), v_flat.to(DEV).view(B, N, H, D).permute(0, 2, 1, 3)
    assert kd.stride() == (N * H * D, D, H * D, 1)                       # token-major: rows of one head are H * D apart
    out = torch.empty(B, H, D, dtype=torch.float16, device=DEV)
    ws = _ops.workspace(_ops.sparse_decode_workspace_bytes(B, H, HEAVY), DEV)
    scale = 1.0 / math.sqrt(D)
    _ops.sparse_decode(q.to(DEV), kd, vd, heavy.to(DEV), counts.to(DEV), scale, out, ws, mask=mask.to(DEV), mask_by_slot=True)
    torch.cuda.synchronize()
    got = out.float().cpu()
    want = torch.stack([torch.stack([orc.sparse_attend(q[b, h], k_view[b, h], v_view[b, h], heavy[b, h].numpy(), scale, mask[b])
                                     for h in range(H)]) for b in range(B)])
    err = (got - want).abs().max().item()
    print(f"max-abs error {err:.3e} (reference atol 1e-3)", flush=True)
    assert err <= 1e-3
    if not random_mask:       # Mask == 0 is fwd_sparse_no_mask: the unmasked launch must give the same bits
        out2 = torch.empty_like(out)
        _ops.sparse_decode(q.to(DEV), kd, vd, heavy.to(DEV), counts.to(DEV), scale, out2, ws)
        assert torch.equal(out, out2)
        ref = c_oracle.sparse_attend(q, k_view, v_view, heavy.numpy(), counts.numpy(), scale)
        assert np.abs(got.numpy() - ref).max() <= 1e-3


def _prototype_hash_layers(H, D, g):
    """The prototype's hash weights: [H, D, D], [H, D, D], [H, D, 32] N(0, 0.1) used as x @ W, biases [H, 1, .] N(0, 0.1),
    fp16 values (torchatt.py:153-158).  Returned per head as nn.Linear-style (W [out, in], b [out]) in fp32."""
    ws = [torch.empty(H, D, n).normal_(mean=0, std=0.1, generator=g).half() for n in (D, D, 32)]
    bs = [torch.empty(H, 1, n).normal_(mean=0, std=0.1, generator=g).half() for n in (D, D, 32)]
    return [[(ws[l][h].float().t().contiguous(), bs[l][h, 0].float().contiguous()) for l in range(3)] for h in range(H)]


@pytest.mark.parametrize("B,N", [(2, 4096), (1, 16384)])
def test_flash_correctness_recipe_encode_select_attend(B, N):
    print(f"\n[case] torchatt.py test_flash_correctness recipe B={B} N={N}", flush=True)
    H, D = 32, 128
    topk = N // 32
    g = torch.Generator().manual_seed(208 + B)
    q = torch.empty(B, H, D).normal_(mean=0.1, std=0.2, generator=g).half()
    k_flat, k_view = _token_major(B, N, H, D, 0.1, 0.2, g)
    v_flat, v_view = _token_major(B, N, H, D, 0.1, 10.0, g)
    layers = _prototype_hash_layers(H, D, g)          # "keys and queries use separate usa_modules. But for timing using the same"
    kd = k_flat.to(DEV).view(B, N, H, D).permute(0, 2, 1, 3)
    vd = v_flat.to(DEV).view(B, N, H, D).permute(0, 2, 1, 3)
    qd = q.to(DEV)
    scale = 1.0 / math.sqrt(D)

    # ---- key_labels / query_label (torchatt.py:183-184, 55-56): bit i = (logit_i > 0), least significant bit = dim 0
    wts = _ops.pack_usa_weights(layers, DEV)
    kcodes = torch.zeros(B, H, N, 1, dtype=torch.int32, device=DEV)
    qcodes = torch.zeros(B, H, 1, 1, dtype=torch.int32, device=DEV)
    _ops.encode_pack(kd, wts, 3, D, 32, kcodes)                           # strided token-major rows, one MLP per head
    _ops.encode_pack(qd.unsqueeze(2), wts, 3, D, 32, qcodes)
    kl = orc.usa_logits(k_view.float(), layers)
    ql = orc.usa_logits(q.float().unsqueeze(2), layers)
    kc_np, qc_np = to_i32(orc.pack_codes(kl)), to_i32(orc.pack_codes(ql)[:, :, 0, :])
    nk = compare_codes("key labels", kcodes.cpu().numpy().view(np.uint32), kc_np.view(np.uint32), kl.numpy())
    nq = compare_codes("query labels", qcodes.cpu().numpy().view(np.uint32)[:, :, 0], qc_np.view(np.uint32), ql[:, :, 0].numpy())
    print(f"sign bits differing where |logit| < 1e-4: keys {nk}, queries {nq}", flush=True)
    # the labels as the prototype holds them: sum(bits * 2**arange(32)) as int64 [H, B, N]
    power = 2 ** torch.arange(32, dtype=torch.int64)
    labels = ((kl > 0).long() * power).sum(-1).permute(1, 0, 2)
    assert np.array_equal(labels.numpy().astype(np.uint32), kc_np.view(np.uint32)[..., 0].transpose(1, 0, 2))

    # ---- from the oracle's codes on: match / count / topk (torchatt.py:58-67) = the topk smallest Hamming distances
    kc, qc = torch.from_numpy(kc_np).to(DEV), torch.from_numpy(qc_np).to(DEV)
    seq = np.full(B, N, dtype=np.int32)
    idx = torch.full((B, H, topk), -1, dtype=torch.int32, device=DEV)
    counts = torch.zeros(B, H, dtype=torch.int32, device=DEV)
    ws_s = _ops.workspace(_ops.select_workspace_bytes(B, H, H, 1, N), DEV)
    _ops.select(kc, qc, N, None, 0, 0, float(topk), idx, counts, ws_s)     # no sink, no recent window, absolute budget
    idx_ref, counts_ref = c_oracle.select(kc_np, qc_np, seq, 0, 0, float(topk), topk)
    assert np.array_equal(counts.cpu().numpy(), counts_ref) and (counts_ref == topk).all()
    assert np.array_equal(idx.cpu().numpy(), idx_ref)
    # against torch.topk on the prototype's count = popcount(~(q ^ k)) over 64 bits: same multiset of kept counts
    ham = c_oracle.hamming(kc_np, qc_np, seq).astype(np.int64)
    count = torch.from_numpy(64 - ham)                                      # 32 upper ones + (32 - distance)
    top = torch.topk(count, topk, dim=-1)
    kept = np.take_along_axis(64 - ham, idx_ref.astype(np.int64), axis=-1)
    assert np.array_equal(np.sort(kept, -1), np.sort(top.values.numpy(), -1))

    ref = c_oracle.sparse_attend(q, k_view, v_view, idx_ref, counts_ref, scale)
    ws_a = _ops.workspace(_ops.sparse_decode_workspace_bytes(B, H, topk), DEV)

    def attend(lists):
        out = torch.empty(B, H, D, dtype=torch.float16, device=DEV)
        _ops.sparse_decode(qd, kd, vd, lists, counts, scale, out, ws_a)
        torch.cuda.synchronize()
        return out.float().cpu().numpy()

    err_sorted = np.abs(attend(idx) - ref).max()
    # the same tokens in topk order (best score first, ties by index): the list order only changes the order of additions
    order = np.lexsort((idx_ref, np.take_along_axis(ham, idx_ref.astype(np.int64), axis=-1)), axis=-1)
    by_score = np.take_along_axis(idx_ref, order, axis=-1)
    err_topk = np.abs(attend(torch.from_numpy(np.ascontiguousarray(by_score)).to(DEV)) - ref).max()
    # torch.topk's own lists (its choice among the tied tokens): against the oracle on those lists
    own = top.indices.to(torch.int32)
    err_own = np.abs(attend(own.to(DEV)) - c_oracle.sparse_attend(q, k_view, v_view, own.numpy(), counts_ref, scale)).max()
    print(f"max-abs error: ascending lists {err_sorted:.3e}, topk order {err_topk:.3e}, torch.topk's lists {err_own:.3e} "
          "(reference atol 1e-2)", flush=True)
    assert max(err_sorted, err_topk, err_own) <= 1e-2

    # ---- the fused launch: histograms, thresholds in the launch, list rebuilt in LDS from the codes
    assert _ops.fused_applies(B, H, H, 1, N, 0, 0, float(topk))
    out_f = torch.empty(B, H, D, dtype=torch.float16, device=DEV)
    cnt_f = torch.zeros(B, H, dtype=torch.int32, device=DEV)
    ws_f = _ops.workspace(_ops.sparse_decode_fused_workspace_bytes(B, H, H, N), DEV)
    if _ops.fused_local_thresholds(B, H, N):
        _ops.select_histogram(kc, qc, N, None, 0, 0, ws_s)
        _ops.sparse_decode_fused(qd, kd, vd, kc, qc, N, None, 0, 0, float(topk), ws_s, scale, out_f, ws_f,
                                 thresholds_ready=False, out_counts=cnt_f)
    else:
        _ops.select_prepare(kc, qc, N, None, 0, 0, float(topk), cnt_f, ws_s)
        _ops.sparse_decode_fused(qd, kd, vd, kc, qc, N, None, 0, 0, float(topk), ws_s, scale, out_f, ws_f)
    torch.cuda.synchronize()
    assert np.array_equal(cnt_f.cpu().numpy(), counts_ref)
    err_fused = np.abs(out_f.float().cpu().numpy() - ref).max()
    print(f"max-abs error of the fused launch {err_fused:.3e}", flush=True)
    assert err_fused <= 1e-2

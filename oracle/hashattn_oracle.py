"""CPU restatement of HashAttention's sparse decode path.  TEST INFRASTRUCTURE ONLY.

This module is the checker the HIP kernels are compared with.  Nothing in the
shipped package imports it: only the tests, the smoke run and the benchmark's
CPU-baseline leg may.  Every function names the lines of the reference
(`/root/reference`, xAlg-ai/HashAttention-1.0) whose behaviour it restates.

Stages
  usa_mlp / usa_logits      hash MLP of one head / all heads       hashattention/hashattention_llama.py:99-128, 159-169
  usa_forward_hard          ternary sign, span = <sign q, sign k>  hashattention_llama.py:151-200, 51-55
  standardise_by_keys       CENTER: (x - mean_k) / (std_k + 1e-6) per head      hashattention_llama.py:163-167
  lift_one_head             LSH baseline: extra coordinate sqrt(M^2 - |x|^2)     hashattention_llama.py:75-84, 130-139
  pack_codes                bit i = logit_i > 0, LSB = dim 0       efficiency/kernels/torchatt.py:55-56, 159, 183-184
  hamming                   popcount(q ^ k)                        efficiency/kernels/bit_count_uint32.py:4-12, torchatt.py:58-62
  compute_mask_multi        sink | recent | top-k heavy mask       hashattention_llama.py:401-446
  select_indices            the same selection as index lists (canonical lowest-index tie-break)
  masked_decode_attention   dense QK^T, mask, fp32 softmax, AV     hashattention_llama.py:578-623
  sparse_attend             gather-only attention                  efficiency/kernels/sparse.py:190-214
  merge_splits              split-K log-sum-exp merge              efficiency/kernels/flash_fwd_sparse.py:451-508, 535-553
  repeat_kv / rotate_half / apply_rotary_pos_emb   textbook restatements of the `transformers`
                            helpers the reference imports (hashattention_llama.py:18); the reference
                            holds no test at that boundary: parity unpinned there.
  reference_decode_attention  the whole emulated layer-step (used as the timed CPU baseline)
  usa_forward_soft          tanh embeddings, sigmoid(span - thold)  hashattention_llama.py:151-200 (hard=False)
  recall_targets            true-logit top-32 target + candidate mask of the train branch  hashattention_llama.py:356-371
  weighted_bce / train_step the training script's loss and one optimizer step  train_hashattention.py:88-95, hashattention_llama.py:304-316

Tie-break.  The reference sorts with `span.sort(descending=True)` without
`stable=True` (hashattention_llama.py:430), so which of the equal-score tokens
fill the last places is implementation-defined.  This oracle fixes the
canonical rule "lowest index first" (`stable=True`); `tie_invariant_equal`
compares two masks up to that freedom.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F

# --------------------------------------------------------------------------- hash MLP


def usa_mlp(x: torch.Tensor, layers: Sequence[Tuple[torch.Tensor, torch.Tensor]]) -> torch.Tensor:
    """`nn.Sequential(Linear, SiLU, Linear, SiLU, Linear)` of one head (1-3 Linear layers).

    reference: hashattention_llama.py:99-128 (module construction), :168-169 (application).
    """
    h = x
    for i, (W, b) in enumerate(layers):
        h = F.linear(h, W.to(h.dtype), b.to(h.dtype))
        if i + 1 < len(layers):
            h = F.silu(h)
    return h


def usa_logits(x: torch.Tensor, heads: Sequence[Sequence[Tuple[torch.Tensor, torch.Tensor]]]) -> torch.Tensor:
    """Per-head MLP over x [b, n_in_heads, t, d] -> logits [b, n_heads, t, D].

    Head i of the MLP list reads input head i // (n_heads / n_in_heads): with one K MLP per
    query head the reference feeds it `repeat_kv`'d keys (hashattention_llama.py:578, 605, 159-169),
    i.e. KV head i // group.
    """
    b, n_in, t, _ = x.shape
    n_heads = len(heads)
    rep = n_heads // n_in
    outs = [usa_mlp(x[:, i // rep], heads[i]) for i in range(n_heads)]
    return torch.stack(outs, dim=1)


def standardise_by_keys(K: torch.Tensor, Q: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """CENTER switch of `USA.forward` (hashattention_llama.py:163-167): inside the loop over heads, the keys of head i
    (all batch entries, all positions) give a mean and an unbiased deviation per feature; keys AND queries of that head
    are shifted and scaled with them, `1e-6` added to the deviation.  K, Q [b, H, s|t, d] with equal head counts."""
    Ko, Qo = torch.empty_like(K), torch.empty_like(Q)
    for i in range(K.shape[1]):
        k = K[:, i]
        flat = k.reshape(-1, k.shape[-1])
        mu, sd = flat.mean(dim=0), flat.std(dim=0)
        Ko[:, i] = (k - mu) / (sd + 1e-6)
        Qo[:, i] = (Q[:, i] - mu) / (sd + 1e-6)
    return Ko, Qo


def lift_one_head(x: torch.Tensor) -> torch.Tensor:
    """`IpToCS` (hashattention_llama.py:75-84), the first stage of every head of the LSH baseline (:130-139): with
    M = (largest norm among ALL vectors handed in) + 1e-3, append sqrt(max(M^2 - |x|^2, 0)), so that every lifted vector
    has norm M and the angle between lifted vectors orders them by inner product.  M is a Python float (double), as
    `.item()` makes it in the reference."""
    lengths = torch.linalg.vector_norm(x, dim=-1, keepdim=True)
    M = float(lengths.max()) + 1e-3
    return torch.cat([x, torch.sqrt(torch.clamp_min(M ** 2 - lengths ** 2, 0))], dim=-1)


def lift_heads(X: torch.Tensor) -> torch.Tensor:
    """The lift applied head by head, as the per-head `Sequential(IpToCS(), Linear)` sees its slice X[:, i]."""
    return torch.stack([lift_one_head(X[:, i]) for i in range(X.shape[1])], dim=1)


def usa_forward_hard(K: torch.Tensor, Q: torch.Tensor, k_heads, q_heads, center: bool = False,
                     lsh: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """`USA.forward(K, Q, hard=True)`: span[b,h,t,s] = sum_i sign(q)_i sign(k)_i, non-causal -> finfo.min.

    reference: hashattention_llama.py:151-200.  K, Q are [b, H, s|t, d] (K already repeat_kv'd).
    torch.sign maps 0 to 0 (:55), so an exactly-zero logit contributes nothing to the span.
    `center`: the CENTER switch (:163-167); `lsh`: heads are `[(W [D, d + 1], b)]` applied to lifted vectors (:130-139).
    """
    if center:
        K, Q = standardise_by_keys(K, Q)
    if lsh:
        K, Q = lift_heads(K), lift_heads(Q)
    kl = usa_logits(K, k_heads)
    ql = usa_logits(Q, q_heads)
    ks, qs = torch.sign(kl), torch.sign(ql)
    span = torch.einsum("bhtd,bhsd->bhts", qs, ks)
    t, s = Q.shape[-2], K.shape[-2]
    causal = torch.tril(torch.ones(t, s), diagonal=s - t).bool()
    span = torch.where(causal, span, torch.full([], torch.finfo(span.dtype).min, dtype=span.dtype))
    return span, ks


def pack_codes(logits: torch.Tensor) -> torch.Tensor:
    """logits [..., D] (D multiple of 32) -> int64 tensor [..., D/32] holding uint32 words.

    bit i of the code = (logit_i > 0) (`relu(sign(x))`), least significant bit = output dim 0
    (`power = 2**arange(32)`): efficiency/kernels/torchatt.py:55-56, 159, 183-184.
    """
    D = logits.shape[-1]
    assert D % 32 == 0
    bits = (logits > 0).to(torch.int64).reshape(*logits.shape[:-1], D // 32, 32)
    power = (2 ** torch.arange(32, dtype=torch.int64))
    return (bits * power).sum(dim=-1)


def popcount_u32(x: torch.Tensor) -> torch.Tensor:
    """Element-wise population count of uint32 values held in an int64 tensor (SWAR).

    reference: `__popc` kernel, efficiency/kernels/bit_count_uint32.py:4-12.
    """
    x = x & 0xFFFFFFFF
    x = x - ((x >> 1) & 0x55555555)
    x = (x & 0x33333333) + ((x >> 2) & 0x33333333)
    x = (x + (x >> 4)) & 0x0F0F0F0F
    return ((x * 0x01010101) & 0xFFFFFFFF) >> 24


def hamming(qcodes: torch.Tensor, kcodes: torch.Tensor) -> torch.Tensor:
    """qcodes [B, H, W], kcodes [B, Hc, S, W] (uint32 words in int64) -> Hamming distance [B, H, S].

    Query head h is scored against code head h // (H / Hc).  The reference prototype ranks by
    popcount(~(q ^ k)) (torchatt.py:58-66), which is monotone decreasing in this distance, and
    the model path by span = D - 2 * hamming (hashattention_llama.py:180-187).
    """
    B, H, W = qcodes.shape
    Hc = kcodes.shape[1]
    kc = kcodes.repeat_interleave(H // Hc, dim=1)
    x = qcodes[:, :, None, :] ^ kc
    return popcount_u32(x).sum(dim=-1)


# --------------------------------------------------------------------------- selection


def heavy_count(seq_len: int, heavy_budget: float) -> int:
    """reference: hashattention_llama.py:431-434 (fraction of the current length, or absolute if > 1)."""
    return int(heavy_budget) if heavy_budget > 1.0 else int(seq_len * heavy_budget)


def compute_mask_multi(span: torch.Tensor, init_budget: int, recent_budget: int, heavy_budget: float,
                       mode: str = "simple", retrieve_depth: float = 0.0, stable: bool = True) -> torch.Tensor:
    """Keep-mask [b, H, q, S] from span scores [b, H, q, S]; restates hashattention_llama.py:423-446.

    `stable=True` is the canonical lowest-index tie-break; `stable=False` reproduces the
    reference call verbatim (implementation-defined order among ties).
    """
    span = span.clone()
    q, k = span.shape[-2], span.shape[-1]
    chr_mask = torch.tril(torch.ones(q, k), diagonal=k - q - recent_budget).bool()
    chr_mask[:, :init_budget] = False
    span.masked_fill_(~chr_mask, torch.finfo(span.dtype).min)
    mask = torch.zeros_like(span).bool()
    mask[:, :, :, :] = torch.tril(torch.ones(q, k), diagonal=k - q).bool()
    mask = mask * (~chr_mask)
    values, indices = span.sort(dim=-1, descending=True, stable=stable)
    hb = heavy_count(k, heavy_budget)
    if mode == "simple":
        mask.scatter_(3, indices[:, :, :, :hb], True)
    else:
        depth_thold = values[:, :, :, :1] - 2 * retrieve_depth
        num_thold = values[:, :, :, hb - 1:hb]
        mask.masked_fill_(span >= torch.maximum(depth_thold, num_thold), True)
    return mask


def select_indices(ham: torch.Tensor, seq_len: int, init_budget: int, recent_budget: int, heavy_budget: float,
                   mode: str = "simple", retrieve_depth: int = 0) -> List[List[int]]:
    """Index-set formulation of the q_len == 1 selection for one sequence.

    ham: Hamming distances [H, >=seq_len]; returns one ascending list per head:
    sink [0, init) | the k_eff = min(heavy, #candidates) candidates of [init, seq_len - recent)
    with the smallest distance (ties: lowest index) | recent [seq_len - recent, seq_len).
    Derived independently of `compute_mask_multi` (no tril/scatter) so each checks the other.
    """
    out = []
    lo, hi = min(init_budget, seq_len), max(min(init_budget, seq_len), seq_len - recent_budget)
    kk = min(heavy_count(seq_len, heavy_budget), hi - lo)
    for h in range(ham.shape[0]):
        cand = list(range(lo, hi))
        row = ham[h].tolist()
        if mode == "simple":
            heavy = sorted(sorted(cand, key=lambda j: (row[j], j))[:kk])
        elif cand and kk > 0:
            order = sorted(row[j] for j in cand)
            thold = min(order[0] + int(math.floor(retrieve_depth)), order[kk - 1])
            heavy = [j for j in cand if row[j] <= thold]
        else:
            heavy = []
        out.append(list(range(0, lo)) + heavy + list(range(hi, seq_len)))
    return out


def select_indices_np(ham: np.ndarray, seq_len: int, init_budget: int, recent_budget: int,
                      heavy_budget: float) -> np.ndarray:
    """Vectorised `select_indices` ('simple' mode) for full-size rows: [H, n_sel] int32, ascending."""
    lo, hi = min(init_budget, seq_len), max(min(init_budget, seq_len), seq_len - recent_budget)
    kk = min(heavy_count(seq_len, heavy_budget), hi - lo)
    H = ham.shape[0]
    cand = ham[:, lo:hi].astype(np.int64)
    order = np.argsort(cand, axis=1, kind="stable")[:, :kk] + lo
    order.sort(axis=1)
    sink = np.broadcast_to(np.arange(0, lo), (H, lo))
    recent = np.broadcast_to(np.arange(hi, seq_len), (H, seq_len - hi))
    return np.concatenate([sink, order, recent], axis=1).astype(np.int32)


def mask_from_indices(idx: Sequence[Sequence[int]], seq_len: int) -> torch.Tensor:
    m = torch.zeros(len(idx), seq_len, dtype=torch.bool)
    for h, row in enumerate(idx):
        m[h, torch.as_tensor(list(row), dtype=torch.long)] = True
    return m


def tie_invariant_equal(mask_a: torch.Tensor, mask_b: torch.Tensor, score: torch.Tensor) -> bool:
    """True when two keep-masks [.., S] agree up to the choice among equal scores.

    For every row: same number kept, and the kept multiset of scores is identical.
    """
    if mask_a.shape != mask_b.shape or not torch.equal(mask_a.sum(-1), mask_b.sum(-1)):
        return False
    big = score.max().item() + 1
    sa = torch.where(mask_a, score, torch.full_like(score, big)).sort(dim=-1).values
    sb = torch.where(mask_b, score, torch.full_like(score, big)).sort(dim=-1).values
    return torch.equal(sa, sb)


# --------------------------------------------------------------------------- attention


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[b, Hkv, s, d] -> [b, Hkv * n_rep, s, d], each KV head repeated n_rep times in place
    (= repeat_interleave on dim 1); third-party `transformers` helper used at hashattention_llama.py:578-579."""
    return x.repeat_interleave(n_rep, dim=1)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    return torch.cat((-x[..., d:], x[..., :d]), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin):
    """Rotate-half RoPE (third-party helper used at hashattention_llama.py:571); cos/sin [b, t, d]."""
    cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    return q * cos + rotate_half(q) * sin, k * cos + rotate_half(k) * sin


def masked_decode_attention(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, mask: torch.Tensor,
                            attention_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Dense scores, (+ the additive attention mask,) keep-mask to finfo.min, softmax in fp32 cast back to Q's dtype, times V.

    reference: hashattention_llama.py:585, 593-598 (`attn_weights + attention_mask`, [b, 1, q, S]), 606, 613, 615.
    Q [b,H,q,d]; K,V [b,H,S,d]; mask [b,H,q,S].
    """
    w = torch.matmul(Q, K.transpose(2, 3)) / math.sqrt(Q.shape[-1])
    if attention_mask is not None:
        assert attention_mask.shape == (Q.shape[0], 1, Q.shape[2], K.shape[2])
        w = w + attention_mask
    w = w.masked_fill(~mask, torch.finfo(w.dtype).min)
    w = F.softmax(w, dim=-1, dtype=torch.float32).to(Q.dtype)
    return torch.matmul(w, V)


def sparse_attend(q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, idx: Sequence[int], sm_scale: float,
                  slot_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One (batch, head): softmax(q . K[idx] * scale + slot_mask) @ V[idx] in fp32.

    reference: `torch_fwd_sparse`, efficiency/kernels/sparse.py:190-214 (fp32 softmax; `att_value += Mask[b]`, :207, one
    term per place in the list).  q [d]; K, V [S, d]; slot_mask [len(idx)] or None.
    """
    ii = torch.as_tensor(np.asarray(idx), dtype=torch.long)
    k, v = K[ii].float(), V[ii].float()
    a = (k @ q.float()) * sm_scale
    if slot_mask is not None:
        a = a + slot_mask[:len(ii)].float()
    p = torch.softmax(a, dim=0)
    return p @ v


def rows_through_slot_table(pool: torch.Tensor, req_to_tokens: torch.Tensor) -> torch.Tensor:
    """The cache a token -> slot table describes: pool [n_slots, Hkv, d] (K or V as the sparse flash-decode holds it), table
    [B, S] -> [B, Hkv, S, d] with out[b, h, j] = pool[table[b, j], h].

    reference: `k_loc = Req_to_tokens[cur_batch, topk_token_indices]; off_k = k_loc * stride_kbs + cur_kv_head * stride_kh`,
    efficiency/kernels/flash_fwd_sparse.py:466-474 (the table built at efficiency/kernels/torchatt.py:165).
    """
    return pool[req_to_tokens.long()].permute(0, 2, 1, 3)


def merge_splits(part_o: torch.Tensor, part_lse: torch.Tensor) -> torch.Tensor:
    """Merge per-split normalised outputs [n, d] with their log-sum-exp [n] into one output [d].

    reference: stage-2 epilogue and stage-3 loop, efficiency/kernels/flash_fwd_sparse.py:496-508, 535-553.
    """
    m = part_lse.max()
    w = torch.exp(part_lse - m)
    return (w[:, None] * part_o).sum(0) / w.sum()


def dense_attention(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor) -> torch.Tensor:
    """`torch_attention_naive`, efficiency/kernels/torchatt.py:17-30, without its final transpose."""
    w = torch.matmul(Q, K.transpose(2, 3)) / math.sqrt(Q.shape[-1])
    w = F.softmax(w, dim=-1, dtype=torch.float32).to(Q.dtype)
    return torch.matmul(w, V)


def reference_decode_attention(Q, K, V, k_heads, q_heads, init_budget, recent_budget, heavy_budget,
                               mode="simple", retrieve_depth=0.0, stable=True, usa_dtype=None, center=False, lsh=False,
                               attention_mask=None):
    """The reference's emulated decode step between RoPE/cache update and o_proj.

    reference: hashattention_llama.py:578-623 with compute_mask_multi :401-446: repeat K/V over the
    group, dense QK^T, re-hash every key, full sort, masked fp32 softmax, AV.
    Q [b,H,q,d]; K,V [b,Hkv,S,d].  Returns (attn_output [b,H,q,d], keep mask [b,H,q,S]).
    `center` / `lsh` (one K head per query head): the hash reads standardised / lifted vectors, as `usa_forward_hard`.
    `attention_mask` [b, 1, q, S]: added to the scores before the keep-mask (:593-598); the selection does not see it.
    """
    H, Hkv = Q.shape[1], K.shape[1]
    Kr, Vr = repeat_kv(K, H // Hkv), repeat_kv(V, H // Hkv)
    ud = usa_dtype or Q.dtype
    # the K MLP list has either one entry per query head or one per KV head
    Kin = Kr if len(k_heads) == H else K
    Kin, Qin = Kin.to(ud), Q.to(ud)
    if center or lsh:
        assert len(k_heads) == H
        if center:
            Kin, Qin = standardise_by_keys(Kin, Qin)
        if lsh:
            Kin, Qin = lift_heads(Kin), lift_heads(Qin)
    kl = usa_logits(Kin, k_heads)
    if kl.shape[1] != H:
        kl = repeat_kv(kl, H // kl.shape[1])
    ql = usa_logits(Qin, q_heads)
    span = torch.einsum("bhtd,bhsd->bhts", torch.sign(ql), torch.sign(kl))
    t, s = Q.shape[-2], K.shape[-2]
    causal = torch.tril(torch.ones(t, s), diagonal=s - t).bool()
    span = torch.where(causal, span, torch.full([], torch.finfo(span.dtype).min, dtype=span.dtype))
    mask = compute_mask_multi(span, init_budget, recent_budget, heavy_budget, mode, retrieve_depth, stable)
    return masked_decode_attention(Q, Kr, Vr, mask, attention_mask), mask


def recall_overlap(q: torch.Tensor, k: torch.Tensor, k_heads, q_heads, init_budget: int, recent_budget: int,
                   top_true: int = 32) -> torch.Tensor:
    """The recall statistic of the reference's `usa_local_compute` (hashattention_llama.py:357-386): for every query row,
    the fraction of its `top_true` highest-scoring candidate keys (true attention logits) that are among the S // 16
    candidates of highest hash score.  q [b, H, q_len, d] are the last q_len positions of the S cached keys k
    [b, Hkv, S, d]; candidates of row i are j in [init, i + S - q_len - recent].  Returns [b, H, q_len] float.

    Two points where the reference is not fully specified are fixed here: ties of the hash score are broken by lowest
    index (its torch.topk leaves them open), and rows with fewer than `top_true` candidates count only real
    candidates as targets (its top-k would pad the target with masked positions) while still dividing by `top_true`.
    """
    b, H, q_len, d = q.shape
    S = k.shape[2]
    kk = repeat_kv(k.float(), H // k.shape[1])
    logits = torch.matmul(q.float(), kk.transpose(2, 3)) / math.sqrt(d)                     # :358
    cand = torch.tril(torch.ones(q_len, S), diagonal=S - q_len - recent_budget).bool()      # :360
    cand[:, :init_budget] = False                                                            # :361
    span, _ = usa_forward_hard(kk, q.float(), k_heads if len(k_heads) == H else [k_heads[h // (H // len(k_heads))] for h in range(H)],
                               q_heads)
    out = torch.zeros(b, H, q_len)
    n_pred = S // 16                                                                         # :375
    for i in range(q_len):
        js = torch.nonzero(cand[i]).flatten()
        if js.numel() == 0:
            continue
        for bb in range(b):
            for h in range(H):
                lg = logits[bb, h, i, js]
                true_top = js[torch.topk(lg, min(top_true, js.numel())).indices]
                sp = span[bb, h, i, js]
                order = sorted(range(js.numel()), key=lambda t: (-float(sp[t]), int(js[t])))[:n_pred]
                pred = set(int(js[t]) for t in order)
                out[bb, h, i] = sum(1 for j in true_top.tolist() if j in pred) / float(top_true)
    return out


# --------------------------------------------------------------------------- training side

def usa_forward_soft(K: torch.Tensor, Q: torch.Tensor, k_heads, q_heads, thold: float = 0.0, center: bool = False,
                     lsh: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """`USA.forward(K, Q, hard=False)`: tanh of both embeddings, span = <tanh q, tanh k>, non-causal entries set to
    finfo.min, then sigmoid(span - thold) (so non-causal entries come out as exactly 0).  Returns (scores, tanh K).

    reference: hashattention_llama.py:151-200 (:174-176 tanh, :184-185 baddbmm, :190-194 causal fill, :196-197 sigmoid).
    Differentiable: built from torch ops on whatever tensors the head lists hold.  `center`, `lsh` as in `usa_forward_hard`.
    """
    if center:
        K, Q = standardise_by_keys(K, Q)
    if lsh:
        K, Q = lift_heads(K), lift_heads(Q)
    kt = torch.tanh(usa_logits(K, k_heads))
    qt = torch.tanh(usa_logits(Q, q_heads))
    span = torch.einsum("bhtd,bhsd->bhts", qt, kt)
    t, s = Q.shape[-2], K.shape[-2]
    causal = torch.tril(torch.ones(t, s), diagonal=s - t).bool()
    span = torch.where(causal, span, torch.full([], torch.finfo(span.dtype).min, dtype=span.dtype))
    return torch.sigmoid(span - thold), kt


def recall_targets(q: torch.Tensor, k: torch.Tensor, init_budget: int, recent_budget: int, top_true: int = 32):
    """What the train branch of `usa_local_compute` hands to `train_step` (hashattention_llama.py:356-371): the candidate
    mask [q_len, S] (causal, minus the recent window, minus the sink) and the 0/1 target [b, H, q_len, S] marking each
    row's `top_true` highest true logits q.k/sqrt(d) after non-candidates were set to finfo.min.  q [b, H, q_len, d] are
    the rotated queries of the last q_len positions, k [b, Hkv, S, d] the cached keys."""
    b, H, q_len, d = q.shape
    S = k.shape[2]
    kk = repeat_kv(k, H // k.shape[1])
    w = torch.matmul(q, kk.transpose(2, 3)) / math.sqrt(d)                                    # :358
    cand = torch.tril(torch.ones(q_len, S), diagonal=S - q_len - recent_budget).bool()        # :360
    cand[:, :init_budget] = False                                                              # :361
    w = w.masked_fill(torch.logical_not(cand), torch.finfo(w.dtype).min)                       # :363
    idx = torch.topk(w, k=top_true, dim=-1).indices                                            # :365
    target = torch.zeros_like(w)
    target.scatter_(-1, idx, 1.0)                                                              # :366-368
    return target, cand


def weighted_bce(alpha: float, beta: float):
    """The loss the training script installs (train_hashattention.py:88-95): binary cross entropy with positives weighted
    by S * beta + alpha, mean over all entries."""
    def loss(yhat: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
        w = y.shape[-1] * beta + alpha
        weight = y * (w - 1) + torch.ones_like(y)
        return F.binary_cross_entropy(yhat.reshape(-1), y.reshape(-1), weight=weight.reshape(-1))
    return loss


def train_step(K, Q, target, target_mask, k_heads, q_heads, loss_fn, optimizer, thold: float = 0.0) -> float:
    """One `train_step` (hashattention_llama.py:304-316): soft scores, entries outside `target_mask` zeroed, loss against
    the target, zero_grad / backward / step.  The head lists must hold the leaf tensors the optimizer updates.
    Returns the loss before the update."""
    span, _ = usa_forward_soft(K.clone(), Q.clone(), k_heads, q_heads, thold)
    span = span.masked_fill(torch.logical_not(target_mask), 0)
    loss = loss_fn(span, target.clone())
    optimizer.zero_grad()
    loss.backward()
    optimizer.step()
    return float(loss.item())

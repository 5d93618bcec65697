"""Shared driver of the GPU parity checks: runs the HIP path through the C ABI and compares every
stage with the oracle on the same seeded inputs.  Used by tests/test_gpu_*.py and by smoke()."""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

from hashattention import _ops
from hashattention.synthetic import Problem, Workload, make_problem
from oracle import c_oracle
from oracle import hashattn_oracle as orc

# attention output tolerances (max-abs).  bf16/fp16: the bar of the target (2e-2 against fp32 math);
# fp32: accumulation-order noise only.
ATOL = {torch.bfloat16: 2e-2, torch.float16: 2e-2, torch.float32: 2e-5}
# a sign bit may differ from the oracle only where the oracle's logit is this close to zero
LOGIT_EPS = 1e-4


def small_workload(**kw) -> Workload:
    base = dict(name="small", batch=2, seq_lens=[1500, 1111], n_q_heads=8, n_kv_heads=2, n_code_heads=2,
                init_budget=16, recent_budget=16, heavy_budget=0.125, dtype=torch.bfloat16, seed=7)
    base.update(kw)
    return Workload(**base)


def oracle_codes(p: Problem):
    """(k logits [B,Hc,S,D], q logits [B,H,1,D], kcodes int64 [B,Hc,S,W], qcodes int64 [B,H,W]) by the torch oracle."""
    kl = orc.usa_logits(p.k.float(), p.usa.k)
    ql = orc.usa_logits(p.q.float(), p.usa.q)
    return kl, ql, orc.pack_codes(kl), orc.pack_codes(ql)[:, :, 0, :]


def to_i32(codes_i64: torch.Tensor) -> torch.Tensor:
    """uint32 words held in int64 -> the int32 bit pattern torch can keep on the GPU."""
    return codes_i64.to(torch.int64).numpy().astype(np.uint32).view(np.int32).copy()


def compare_codes(name, got_u32: np.ndarray, want_u32: np.ndarray, logits: np.ndarray, valid: Optional[np.ndarray] = None):
    """Bits may differ only where |oracle logit| < LOGIT_EPS.  Returns the number of differing bits."""
    diff = got_u32 ^ want_u32                                     # [..., W]
    if valid is not None:
        diff = diff * valid[..., None].astype(np.uint32)
    if not diff.any():
        return 0
    W = diff.shape[-1]
    bits = ((diff[..., :, None] >> np.arange(32, dtype=np.uint32)) & 1).reshape(*diff.shape[:-1], W * 32).astype(bool)
    bad = bits & (np.abs(logits) >= LOGIT_EPS)
    assert not bad.any(), f"{name}: {int(bad.sum())} sign bits differ where |logit| >= {LOGIT_EPS}"
    return int(bits.sum())


def run_decode_case(w: Workload, check_encode: bool = True, mode: str = "simple", depth: int = 0,
                    idx_cap: Optional[int] = None, check_dense: bool = True, verbose: bool = False, dev="cuda:0",
                    algo: int = _ops.HA_SELECT_ALGO_AUTO):
    """encode -> hamming -> select -> sparse attend (+ dense) on the GPU, each stage against the oracle."""
    p = make_problem(w)
    B, H, Hkv, Hc, d, S, W = w.batch, w.n_q_heads, w.n_kv_heads, w.n_code_heads, w.head_dim, w.max_seq_len, w.code_words
    kl, ql, kc64, qc64 = oracle_codes(p)
    kc_np, qc_np = to_i32(kc64), to_i32(qc64)
    seq_np = p.seq_lens.numpy()
    valid = (np.arange(S)[None, :] < seq_np[:, None])              # [B, S]

    q3 = p.q[:, :, 0, :].contiguous().to(dev)
    k, v = p.k.to(dev), p.v.to(dev)
    seq = p.seq_lens.to(dev)
    report = {}

    # ---- encode (exact fp32 arithmetic) against the torch oracle
    if check_encode:
        wk = _ops.pack_usa_weights(p.usa.k, dev)
        wq = _ops.pack_usa_weights(p.usa.q, dev)
        kcodes_gpu = torch.zeros(B, Hc, S, W, dtype=torch.int32, device=dev)
        qcodes_gpu = torch.zeros(B, H, 1, W, dtype=torch.int32, device=dev)
        klog = _ops.encode_pack(k, wk, w.lth_num_layers, w.lth_int_dim, w.lth_final_dim, kcodes_gpu, want_logits=True)
        qlog = _ops.encode_pack(q3.unsqueeze(2), wq, w.lth_num_layers, w.lth_int_dim, w.lth_final_dim, qcodes_gpu,
                                want_logits=True)
        torch.cuda.synchronize()
        vmask = np.broadcast_to(valid[:, None, :], (B, Hc, S))
        kerr = (klog.cpu() - kl).abs()[torch.from_numpy(vmask.copy())].max().item()
        qerr = (qlog.cpu() - ql).abs().max().item()
        assert kerr < 2e-4 and qerr < 2e-4, f"logit error k={kerr} q={qerr}"
        nk = compare_codes("k codes", kcodes_gpu.cpu().numpy().view(np.uint32), kc_np.view(np.uint32), kl.numpy(), vmask)
        nq = compare_codes("q codes", qcodes_gpu.cpu().numpy().view(np.uint32)[:, :, 0], qc_np.view(np.uint32), ql[:, :, 0].numpy())
        report.update(k_logit_err=kerr, q_logit_err=qerr, k_bits_flipped=nk, q_bits_flipped=nq)

    # ---- from here on feed the ORACLE codes so every later stage is exact
    kcodes = torch.from_numpy(kc_np).to(dev)
    qcodes = torch.from_numpy(qc_np).to(dev)

    ham = _ops.hamming_score(kcodes, qcodes, S, seq).cpu().numpy()
    ham_ref = c_oracle.hamming(kc_np, qc_np, seq_np)
    assert np.array_equal(ham, ham_ref), "hamming scores differ"

    n_sel_max = max(w.n_selected(s) for s in w.seq_lens)
    cap = idx_cap if idx_cap is not None else (S if mode != "simple" else max(n_sel_max, 1))   # a list buffer needs one entry
    idx = torch.full((B, H, cap), -1, dtype=torch.int32, device=dev)
    counts = torch.zeros(B, H, dtype=torch.int32, device=dev)
    ws = _ops.workspace(_ops.select_workspace_bytes(B, H, Hc, W, S), dev)
    m = _ops.HA_SELECT_SIMPLE if mode == "simple" else _ops.HA_SELECT_THRESHOLD
    _ops.select(kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, idx, counts, ws, mode=m, depth=depth,
                algo=algo)
    idx_ref, counts_ref = c_oracle.select(kc_np, qc_np, seq_np, w.init_budget, w.recent_budget, w.heavy_budget, cap,
                                          mode=0 if mode == "simple" else 1, depth=depth)
    idx_np, counts_np = idx.cpu().numpy(), counts.cpu().numpy()
    assert np.array_equal(counts_np, counts_ref), f"selected counts differ: {counts_np} vs {counts_ref}"
    assert np.array_equal(idx_np, idx_ref), "selected indices differ"
    report.update(n_selected=int(counts_np.max()))

    # ---- gather-attend against the double-precision C oracle on the same index lists
    sm_scale = 1.0 / math.sqrt(d)
    out = torch.empty(B, H, d, dtype=w.dtype, device=dev)
    ws2 = _ops.workspace(_ops.sparse_decode_workspace_bytes(B, H, cap), dev)
    _ops.sparse_decode(q3, k, v, idx, counts, sm_scale, out, ws2)
    ref = c_oracle.sparse_attend(p.q[:, :, 0, :], p.k, p.v, idx_ref, counts_ref, sm_scale)
    err = float(np.abs(out.float().cpu().numpy() - ref).max())
    assert err <= ATOL[w.dtype], f"sparse attend max-abs error {err} > {ATOL[w.dtype]}"
    report.update(sparse_err=err)

    # ---- the same attention as window partial + heavy-only launch
    win = torch.empty(B, H, 130, dtype=torch.float32, device=dev)
    out2 = torch.empty_like(out)
    _ops.window_partial(q3, k, v, S, seq, w.init_budget, w.recent_budget, sm_scale, win)
    _ops.sparse_decode_heavy(q3, k, v, idx, counts, sm_scale, out2, ws2, win, w.init_budget, w.recent_budget, S, seq)
    err2 = float(np.abs(out2.float().cpu().numpy() - ref).max())
    assert err2 <= ATOL[w.dtype], f"window + heavy attend max-abs error {err2} > {ATOL[w.dtype]}"
    report.update(split_window_err=err2)

    # ---- selection fused into the attend launch: thresholds from ha_select_prepare, list rebuilt in LDS from the codes
    if mode == "simple" and _ops.fused_applies(B, H, Hc, W, S, w.init_budget, w.recent_budget, w.heavy_budget):
        counts3 = torch.full((B, H), -5, dtype=torch.int32, device=dev)
        out3 = torch.empty_like(out)
        ws4 = _ops.workspace(_ops.sparse_decode_fused_workspace_bytes(B, H, Hc, S), dev)
        _ops.select_prepare(kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, counts3, ws)
        _ops.sparse_decode_fused(q3, k, v, kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, ws, sm_scale,
                                 out3, ws4)
        assert np.array_equal(counts3.cpu().numpy(), counts_ref), "fused path: counts differ"
        err3 = float(np.abs(out3.float().cpu().numpy() - ref).max())
        assert err3 <= ATOL[w.dtype], f"fused select+attend max-abs error {err3} > {ATOL[w.dtype]}"
        same = float((out3.float() - out.float()).abs().max().item())
        # the two paths add the same rows in different orders: accumulation-order noise in fp32, one rounding of the output in bf16/fp16
        assert same <= (1e-5 if w.dtype == torch.float32 else 1e-2), f"fused vs two-launch output differ by {same}"
        report.update(fused_err=err3, fused_vs_unfused=same)
        if len(set(w.seq_lens)) == 1:      # equal lengths given on the host (no length array): the same pieces, the same output
            out5 = torch.empty_like(out)
            _ops.sparse_decode_fused(q3, k, v, kcodes, qcodes, S, None, w.init_budget, w.recent_budget, w.heavy_budget, ws, sm_scale,
                                     out5, ws4)
            err5 = float(np.abs(out5.float().cpu().numpy() - ref).max())
            assert err5 <= ATOL[w.dtype], f"fused select+attend (lengths on the host) max-abs error {err5} > {ATOL[w.dtype]}"
        if _ops.fused_local_thresholds(B, Hc, S):       # thresholds derived inside the attention launch: same output bit for bit
            counts4 = torch.full((B, H), -5, dtype=torch.int32, device=dev)
            out4 = torch.empty_like(out)
            ws5 = _ops.workspace(_ops.select_workspace_bytes(B, H, Hc, W, S), dev)
            _ops.select_histogram(kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, ws5)
            _ops.sparse_decode_fused(q3, k, v, kcodes, qcodes, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, ws5, sm_scale,
                                     out4, ws4, thresholds_ready=False, out_counts=counts4)
            assert np.array_equal(counts4.cpu().numpy(), counts_ref), "fused path, local thresholds: counts differ"
            assert torch.equal(out4, out3), "fused path: local thresholds change the output"

    if check_dense:
        outd = torch.empty(B, H, d, dtype=w.dtype, device=dev)
        ws3 = _ops.workspace(_ops.dense_decode_workspace_bytes(B, H, S), dev)
        _ops.dense_decode(q3, k, v, S, seq, sm_scale, outd, ws3)
        refd = c_oracle.dense_attend(p.q[:, :, 0, :], p.k, p.v, seq_np, sm_scale)
        errd = float(np.abs(outd.float().cpu().numpy() - refd).max())
        assert errd <= ATOL[w.dtype], f"dense attend max-abs error {errd} > {ATOL[w.dtype]}"
        report.update(dense_err=errd)
    if verbose:
        print(w.name, report, flush=True)
    return report

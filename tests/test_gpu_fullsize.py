"""The benchmark configurations at their full sizes.  Codes are made on the GPU (MFMA encoder), copied back, and
the CPU oracle recomputes selection and attention from those same codes: index lists bit for bit, outputs within
2e-2 (bf16).  Size-independent properties on top: ascending lists, exact counts, windows present, and the
selected tokens' distances never exceed those of any unselected candidate."""
import math

import numpy as np
import pytest
import torch

from hashattention import _ops
from hashattention.decode import HashDecodeLayer
from hashattention.synthetic import Workload, make_problem_on_device, named_workload
from oracle import c_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _long_rows(name):
    # rows of more than 262144 tokens: more chunks than the attention launch derives thresholds for by itself, so the step is
    # encode, ha_select_prepare, ha_sparse_decode_fused on ready thresholds; an absolute heavy budget keeps a row's list in LDS
    if name == "long_million":      # one sequence of a million tokens, the 8B head layout
        return Workload(name, batch=1, seq_lens=[1_000_000], heavy_budget=4000.0)
    lens = [300_000, 300_000] if name == "long_uniform" else [300_000, 277_123]
    return Workload(name, batch=2, seq_lens=lens, n_q_heads=16, n_kv_heads=4, n_code_heads=4, heavy_budget=4000.0)


@pytest.mark.parametrize("name", ["config1", "config2", "config3", "config4", "long_uniform", "long_ragged", "long_million"])
def test_full_size_configuration(name):
    print(f"\n[case] full size {name}", flush=True)
    w = _long_rows(name) if name.startswith("long") else named_workload(name)
    p = make_problem_on_device(w, DEV)
    B, H, Hkv, S, W = w.batch, w.n_q_heads, w.n_kv_heads, w.max_seq_len, w.code_words
    layer = HashDecodeLayer(p.usa.k, p.usa.q, H, Hkv, 128, w.lth_num_layers, w.lth_int_dim, w.lth_final_dim, w.init_budget,
                            w.recent_budget, w.heavy_budget, device=DEV)
    layer.allocate(B, S)
    layer.encode_keys(p.k, use_mfma=True)
    ragged = len(set(w.seq_lens)) > 1
    seq = p.seq_lens if ragged else None
    if name.startswith("long"):
        assert layer.use_fused and layer.fused_ok and not layer.local_thresholds
    out = torch.empty(B, H, 128, dtype=w.dtype, device=DEV)
    if ragged:
        layer.step(p.q, p.k, p.v, S, out, seq_lens=seq)
    else:
        layer.n_cached = S - 1
        layer.step(p.q, p.k, p.v, S, out)
    if layer.use_fused and layer.fused_ok:      # the step's fused launch keeps its lists in LDS: write them out for the index checks
        layer.select(S, seq)
    torch.cuda.synchronize()

    kc = layer.codes.cpu().numpy()
    qc = layer.qcodes.view(B, H, W).cpu().numpy()
    seq_np = np.array(w.seq_lens, dtype=np.int32)
    idx, cnt = layer.idx.cpu().numpy(), layer.counts.cpu().numpy()
    ref_idx, ref_cnt = c_oracle.select(kc, qc, seq_np, w.init_budget, w.recent_budget, w.heavy_budget, layer.idx_cap)
    assert np.array_equal(cnt, ref_cnt)
    for b in range(B):
        assert (cnt[b] == w.n_selected(w.seq_lens[b])).all()
        n = cnt[b, 0]
        assert np.array_equal(idx[b, :, :n], ref_idx[b, :, :n]), b
        assert (np.diff(idx[b, :, :n], axis=1) > 0).all()
        assert (idx[b, :, :w.init_budget] == np.arange(w.init_budget)).all()
        assert (idx[b, :, n - w.recent_budget:n] == np.arange(w.seq_lens[b] - w.recent_budget, w.seq_lens[b])).all()
    # distances of the selected candidates are all <= those of the unselected ones (one row per sequence)
    ham = c_oracle.hamming(kc, qc, seq_np)
    for b in range(B):
        s, n = w.seq_lens[b], cnt[b, 5]
        sel = np.zeros(s, dtype=bool)
        sel[idx[b, 5, :n]] = True
        cand = np.zeros(s, dtype=bool)
        cand[w.init_budget:s - w.recent_budget] = True
        assert ham[b, 5, :s][sel & cand].max() <= ham[b, 5, :s][~sel & cand].min()

    ref = c_oracle.sparse_attend(p.q[:, :, 0].cpu(), p.k.cpu(), p.v.cpu(), ref_idx, ref_cnt, 1 / math.sqrt(128))
    err = np.abs(out.float().cpu().numpy() - ref).max()
    print(f"  n_selected {cnt.min()}..{cnt.max()}, sparse max-abs error {err:.2e}", flush=True)
    assert err <= 2e-2
    if name in ("config2", "config3", "config4"):
        # the fused launch with a masked prefix per sequence (the mask of a left-padded batch, hashattention_llama.py:593-598):
        # sequences without one keep the plain launch's output bit for bit; for the others a list entry at -inf is a list
        # without that entry, which the oracle attends to
        prefix = [0 if b % 2 == 0 else 1000 + 37 * b for b in range(B)]
        out_m = torch.empty_like(out)
        layer.select_prepare(S, seq)
        layer.attend_fused(p.q[:, :, 0], p.k, p.v, out_m, S, seq, masked_prefix=torch.tensor(prefix, dtype=torch.int32, device=DEV))
        torch.cuda.synchronize()
        assert torch.equal(out_m[0::2], out[0::2])
        idx_m, cnt_m = np.zeros_like(ref_idx), ref_cnt.copy()
        for b in range(B):
            for h in range(H):
                n = ref_cnt[b, h]
                skip = int(np.searchsorted(ref_idx[b, h, :n], prefix[b]))
                idx_m[b, h, :n - skip] = ref_idx[b, h, skip:n]
                cnt_m[b, h] = n - skip
        assert (cnt_m[1::2] < ref_cnt[1::2]).all()
        ref_m = c_oracle.sparse_attend(p.q[:, :, 0].cpu(), p.k.cpu(), p.v.cpu(), idx_m, cnt_m, 1 / math.sqrt(128))
        err_m = np.abs(out_m.float().cpu().numpy() - ref_m).max()
        print(f"  masked prefix: sparse max-abs error {err_m:.2e}", flush=True)
        assert err_m <= 2e-2
    if name != "config2":       # dense baseline against the oracle too (config2: 4 GB of K/V through a scalar loop is slow)
        outd = torch.empty_like(out)
        ws = _ops.workspace(_ops.dense_decode_workspace_bytes(B, H, S), DEV)
        _ops.dense_decode(p.q[:, :, 0], p.k, p.v, S, seq, 1 / math.sqrt(128), outd, ws)
        refd = c_oracle.dense_attend(p.q[:, :, 0].cpu(), p.k.cpu(), p.v.cpu(), seq_np, 1 / math.sqrt(128))
        errd = np.abs(outd.float().cpu().numpy() - refd).max()
        print(f"  dense max-abs error {errd:.2e}", flush=True)
        assert errd <= 2e-2


@pytest.mark.parametrize("name,n_seq", [("config1", 1), ("config3", 1), ("config4", 2)])
def test_full_length_fp32_encoders_against_the_oracle(name, n_seq):
    # the fp32 hash of every cached key of whole sequences at the benchmark lengths (32K, 128K, ragged with 64-bit codes),
    # by the exact scalar kernel and by the fp32 matrix-core kernel, against the torch fp32 oracle on the CPU: a sign bit may
    # differ only where the oracle's |logit| < 1e-4
    from oracle import hashattn_oracle as orc
    from tests.parity_util import compare_codes
    print(f"\n[case] full-length fp32 encoders {name}", flush=True)
    w = named_workload(name)
    p = make_problem_on_device(w, DEV)
    S, W, Hc = w.max_seq_len, w.code_words, w.n_code_heads
    k = p.k[:n_seq]
    wk = _ops.pack_usa_weights(p.usa.k, DEV)
    exact = torch.zeros(n_seq, Hc, S, W, dtype=torch.int32, device=DEV)
    mfma = torch.zeros(n_seq, Hc, S, W, dtype=torch.int32, device=DEV)
    _ops.encode_pack(k, wk, w.lth_num_layers, w.lth_int_dim, w.lth_final_dim, exact)
    _ops.encode_pack_prefill_f32(k, wk, w.lth_num_layers, w.lth_int_dim, w.lth_final_dim, mfma)
    torch.cuda.synchronize()
    k_cpu = k.float().cpu()
    for b in range(n_seq):
        kl = orc.usa_logits(k_cpu[b:b + 1], p.usa.k)                        # [1, Hc, S, D]
        want = orc.pack_codes(kl).numpy().astype(np.uint32)
        valid = np.zeros((1, Hc, S), dtype=bool)
        valid[:, :, :w.seq_lens[b]] = True
        n_exact = compare_codes("exact kernel", exact[b:b + 1].cpu().numpy().view(np.uint32), want, kl.numpy(), valid)
        n_mfma = compare_codes("fp32 mfma kernel", mfma[b:b + 1].cpu().numpy().view(np.uint32), want, kl.numpy(), valid)
        print(f"  sequence {b}: {w.seq_lens[b]} tokens x {Hc} heads x {w.lth_final_dim} bits, differing from the oracle: "
              f"exact {n_exact}, mfma {n_mfma}", flush=True)

"""What the bf16 hash path costs downstream.  A hash module kept in bf16 (bf16 MFMA bulk encoder for the cached keys, the scalar
kernel in bf16 arithmetic for the query) flips some sign bits against the fp32 module of the same weights; this test measures
what those flips do to the selection and to the attention output on the configs[1] workload (B=1, 32768 tokens, 1/8 heavy):
the share of each row's heavy set that both code sets select, and the distance of the attention output from the oracle's
output on the fp32 codes.  The bounds are three times what this workload shows."""
import math

import numpy as np
import pytest
import torch

from hashattention import _ops
from hashattention.synthetic import make_problem_on_device, named_workload
from oracle import c_oracle
from oracle import hashattn_oracle as orc
from tests.parity_util import to_i32

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_bf16_codes_select_nearly_the_same_tokens_on_config1():
    print("\n[case] bf16 codes against fp32 codes, config1", flush=True)
    w = named_workload("config1")
    p = make_problem_on_device(w, DEV)
    B, H, Hkv, Hc, S, W = w.batch, w.n_q_heads, w.n_kv_heads, w.n_code_heads, w.max_seq_len, w.code_words
    bf = lambda heads: [[(Wt.to(torch.bfloat16), b.to(torch.bfloat16)) for Wt, b in layers] for layers in heads]
    k_cpu, q_cpu = p.k.cpu(), p.q.cpu()
    # fp32 module: the oracle's codes
    kl, ql = orc.usa_logits(k_cpu.float(), p.usa.k), orc.usa_logits(q_cpu.float(), p.usa.q)
    kc32, qc32 = to_i32(orc.pack_codes(kl)), to_i32(orc.pack_codes(ql)[:, :, 0, :])
    # bf16 module of the same weights: MFMA bulk encoder for the keys, scalar kernel in bf16 arithmetic for the query
    kc16 = torch.zeros(B, Hc, S, W, dtype=torch.int32, device=DEV)
    qc16 = torch.zeros(B, H, 1, W, dtype=torch.int32, device=DEV)
    _ops.encode_pack_prefill(p.k, _ops.pack_usa_weights_bf16(bf(p.usa.k), DEV), w.lth_num_layers, w.lth_int_dim, w.lth_final_dim, kc16)
    _ops.encode_pack(p.q, _ops.pack_usa_weights(bf(p.usa.q), DEV), w.lth_num_layers, w.lth_int_dim, w.lth_final_dim, qc16,
                     arith=_ops.HA_ARITH_BF16)
    torch.cuda.synchronize()
    flips_k = int(np.unpackbits((kc16.cpu().numpy().view(np.uint32) ^ kc32.view(np.uint32)).view(np.uint8)).sum()) / (B * Hc * S * 32 * W)
    flips_q = int(np.unpackbits((qc16.cpu().numpy().view(np.uint32)[:, :, 0] ^ qc32.view(np.uint32)).view(np.uint8)).sum()) / (B * H * 32 * W)
    print(f"  sign bits differing from the fp32 module: keys {flips_k:.3e}, queries {flips_q:.3e}", flush=True)

    seq = np.array(w.seq_lens, dtype=np.int32)
    cap = w.n_selected(S)
    idx32, cnt32 = c_oracle.select(kc32, qc32, seq, w.init_budget, w.recent_budget, w.heavy_budget, cap)
    idx = torch.zeros(B, H, cap, dtype=torch.int32, device=DEV)
    cnt = torch.zeros(B, H, dtype=torch.int32, device=DEV)
    ws = _ops.workspace(_ops.select_workspace_bytes(B, H, Hc, W, S), DEV)
    _ops.select(kc16, qc16.view(B, H, W), S, None, w.init_budget, w.recent_budget, w.heavy_budget, idx, cnt, ws)
    idx16 = idx.cpu().numpy()
    assert np.array_equal(cnt.cpu().numpy(), cnt32)
    n_heavy = cap - w.init_budget - w.recent_budget
    common = np.array([[len(np.intersect1d(idx16[b, h, :cap], idx32[b, h, :cap])) - (cap - n_heavy) for h in range(H)] for b in range(B)])
    share = common / n_heavy
    print(f"  share of a row's {n_heavy} heavy tokens selected under both code sets: min {share.min():.4f}, mean {share.mean():.4f}", flush=True)

    scale = 1 / math.sqrt(128)
    out = torch.empty(B, H, 128, dtype=w.dtype, device=DEV)
    wsa = _ops.workspace(_ops.sparse_decode_workspace_bytes(B, H, cap), DEV)
    _ops.sparse_decode(p.q[:, :, 0], p.k, p.v, idx, cnt, scale, out, wsa)
    ref32 = c_oracle.sparse_attend(q_cpu[:, :, 0], k_cpu, p.v.cpu(), idx32, cnt32, scale)
    ref16 = c_oracle.sparse_attend(q_cpu[:, :, 0], k_cpu, p.v.cpu(), idx16, cnt32, scale)
    got = out.float().cpu().numpy()
    d_codes = float(np.abs(ref16 - ref32).max())          # what the other selection does to the exact output
    d_total = float(np.abs(got - ref32).max())            # the bf16-code path end to end against the fp32-code oracle
    print(f"  attention output max-abs: selection alone {d_codes:.3e}, bf16-code path against the fp32-code oracle {d_total:.3e}", flush=True)
    assert np.abs(got - ref16).max() <= 2e-2               # the kernel on its own lists
    # observed on this workload: 1.5e-3 of the key bits and 1 of the 1024 query bits differ; a row keeps 97.6 % of its heavy set
    # on average (70 % in the row whose query bit flipped: every distance of that row moves by one, and with it the
    # membership of its tie bucket); the output moves by 4.3e-2 (N(0,1) values: other tokens, another average) - which is
    # the distance between a bf16 and an fp32 hash MODULE, not a kernel error: against the oracle on its own lists the kernel
    # is within 2e-2 above.  Bounds: three times the observed figures.
    assert flips_k < 4.5e-3 and flips_q < 3e-3
    assert share.mean() > 1 - 3 * (1 - 0.9755) and share.min() > 1 - 3 * (1 - 0.70)
    assert d_total < 3 * 4.4e-2

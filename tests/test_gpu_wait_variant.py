"""The fused attention launch waits for the codes it staged through LDS with a hand-counted `s_waitcnt vmcnt(8)`.  That is
correct only while at least eight loads of the wave are younger than the staged requests and no store of the wave is
outstanding in between.  The library's twin built with -DHASHATTN_STAGE_WAIT_ALL waits for everything instead; if the counted
wait ever lets codes (or slot translations) be read before they arrived, the two builds disagree on some shape of this
sweep.  Same bits demanded, with and without a token -> slot table."""
import ctypes as C

import numpy as np
import pytest
import torch

from hashattention import _ops
from hashattention.synthetic import make_problem
from tests.parity_util import oracle_codes, to_i32
from tests.test_gpu_parity import _random_workload

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class _use_library:
    def __init__(self, lib):
        self.lib = lib

    def __enter__(self):
        self.saved, _ops._lib = _ops._lib, self.lib

    def __exit__(self, *a):
        _ops._lib = self.saved


@pytest.mark.parametrize("block", range(4))
def test_counted_wait_and_full_wait_give_the_same_bits(block):
    main = _ops.load_library()
    twin = _ops.load_wait_all_variant()
    assert twin is not main and twin.ha_version() == main.ha_version()
    rng = np.random.default_rng(2024 + block)
    ran = 0
    for i in range(16):
        w = _random_workload(rng, block * 16 + i)
        B, H, Hkv, Hc, S, W = w.batch, w.n_q_heads, w.n_kv_heads, w.n_code_heads, w.max_seq_len, w.code_words
        if not _ops.fused_applies(B, H, Hc, W, S, w.init_budget, w.recent_budget, w.heavy_budget):
            continue
        print(f"\n[case] {w.name}: B={B} H={H}/{Hkv}/{Hc} S={w.seq_lens} bits={w.lth_final_dim} heavy={w.heavy_budget} {w.dtype}", flush=True)
        p = make_problem(w)
        _, _, kc64, qc64 = oracle_codes(p)
        kc, qc = torch.from_numpy(to_i32(kc64)).to(DEV), torch.from_numpy(to_i32(qc64)).to(DEV)
        q3, k, v, seq = p.q[:, :, 0].contiguous().to(DEV), p.k.to(DEV), p.v.to(DEV), p.seq_lens.to(DEV)
        ws_s = _ops.workspace(_ops.select_workspace_bytes(B, H, Hc, W, S), DEV)
        ws_f = _ops.workspace(_ops.sparse_decode_fused_workspace_bytes(B, H, Hc, S), DEV)
        local = _ops.fused_local_thresholds(B, Hc, S)
        cnt = torch.zeros(B, H, dtype=torch.int32, device=DEV)
        if local:
            _ops.select_histogram(kc, qc, S, seq, w.init_budget, w.recent_budget, ws_s)
        else:
            _ops.select_prepare(kc, qc, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, cnt, ws_s)
        slots = torch.stack([torch.randperm(S, generator=torch.Generator().manual_seed(b)) for b in range(B)]).to(torch.int32).to(DEV)
        kperm, vperm = torch.empty_like(k), torch.empty_like(v)
        for b in range(B):
            kperm[b, :, slots[b].long()] = k[b]
            vperm[b, :, slots[b].long()] = v[b]
        outs = []
        for lib in (main, twin):
            with _use_library(lib):
                a, b2 = torch.empty(B, H, 128, dtype=w.dtype, device=DEV), torch.empty(B, H, 128, dtype=w.dtype, device=DEV)
                kw = dict(thresholds_ready=not local, out_counts=cnt if local else None)
                _ops.sparse_decode_fused(q3, k, v, kc, qc, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, ws_s, 0.088, a, ws_f, **kw)
                _ops.sparse_decode_fused(q3, kperm, vperm, kc, qc, S, seq, w.init_budget, w.recent_budget, w.heavy_budget, ws_s, 0.088, b2,
                                         ws_f, slots=slots, **kw)
                torch.cuda.synchronize()
                outs.append((a, b2))
        assert torch.equal(outs[0][0], outs[1][0]), "plain cache: the counted wait and the full wait disagree"
        assert torch.equal(outs[0][1], outs[1][1]), "slot table: the counted wait and the full wait disagree"
        assert torch.equal(outs[0][0], outs[0][1]), "slot table: output differs from the plain cache it describes"
        ran += 1
    assert ran >= 8

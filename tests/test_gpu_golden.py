"""GPU against the committed configs[0] fixture (tests/golden/config0.npz): the integer stages bit for bit from the
stored codes, the fp32 outputs to 2e-5, and the GPU's own exact encoder up to sign bits of ~0 logits."""
import math
import os

import numpy as np
import pytest
import torch

from hashattention import _ops
from hashattention.synthetic import make_problem, named_workload

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config0.npz"))


def test_config0_golden():
    print("\n[case] config0 golden", flush=True)
    w = named_workload("config0")
    p = make_problem(w)
    kcodes = torch.from_numpy(G["kcodes"].view(np.int32)).to(DEV)            # [1, 32, 4096, 1]
    qcodes = torch.from_numpy(G["qcodes"].view(np.int32)[:, :, 0]).contiguous().to(DEV)
    idx = torch.full((1, 32, 1280), -1, dtype=torch.int32, device=DEV)
    counts = torch.zeros(1, 32, dtype=torch.int32, device=DEV)
    ws = _ops.workspace(_ops.select_workspace_bytes(1, 32, 32, 1, 4096), DEV)
    _ops.select(kcodes, qcodes, 4096, None, w.init_budget, w.recent_budget, w.heavy_budget, idx, counts, ws)
    assert np.array_equal(counts.cpu().numpy()[0], G["n_selected"])
    mask = np.zeros((32, 4096), dtype=bool)
    ii = idx.cpu().numpy()[0]
    assert (np.diff(ii, axis=1) > 0).all()                                   # ascending, no duplicates
    for h in range(32):
        mask[h, ii[h]] = True
    assert np.array_equal(np.packbits(mask, axis=-1), G["mask"])

    q3, k, v = p.q[:, :, 0].contiguous().to(DEV), p.k.to(DEV), p.v.to(DEV)
    out = torch.empty(1, 32, 128, device=DEV)
    ws2 = _ops.workspace(_ops.sparse_decode_workspace_bytes(1, 32, 1280), DEV)
    _ops.sparse_decode(q3, k, v, idx, counts, 1 / math.sqrt(128), out, ws2)
    assert np.abs(out.cpu().numpy()[0] - G["out"]).max() < 2e-5

    # the GPU's exact encoder: one K hash MLP per query head reading KV head h // 4
    wk = _ops.pack_usa_weights(p.usa.k, DEV)
    mine = torch.zeros(1, 32, 4096, 1, dtype=torch.int32, device=DEV)
    lg = _ops.encode_pack(k, wk, 3, 128, 32, mine, want_logits=True)
    diff = mine.cpu().numpy().view(np.uint32) ^ G["kcodes"]
    nflip = int(np.unpackbits(diff.view(np.uint8)).sum())
    print("  sign bits differing from the fixture:", nflip, "of", diff.size * 32, flush=True)
    assert nflip <= int(G["near_zero_logits"][0])
    if nflip:
        bits = ((diff[..., None] >> np.arange(32, dtype=np.uint32)) & 1).astype(bool)[:, :, :, 0, :]
        assert (np.abs(lg.cpu().numpy())[bits] < 1e-4).all()

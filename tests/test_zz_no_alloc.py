"""ha_select_static: the selection entry point that allocates nothing (its scratch is a device array built into the
library).  Through the C ABI, against ha_select with a caller-owned workspace: index lists and counts bit for bit, on two
calls in a row of which the second is smaller (the shared scratch still holds the first call's contents), then a larger
one again; no device memory is allocated by the calls; a shape whose scratch does not fit is refused."""
import numpy as np
import pytest
import torch

from hashattention import _ops
from oracle import c_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(B, H, Hc, W, lens, init, recent, heavy, mode, depth, seed):
    g = torch.Generator().manual_seed(seed)
    S = max(lens)
    kc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, Hc, S, W), generator=g, dtype=torch.int64).to(torch.int32).to(DEV)
    qc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, W), generator=g, dtype=torch.int64).to(torch.int32).to(DEV)
    if W == 1:      # few distinct distances would make every row's tie bucket huge with random codes; bias codes towards the query
        near = torch.rand(B, Hc, S, 1, generator=g).to(DEV) < 0.05
        flips = torch.randint(0, 2 ** 8, (B, Hc, S, 1), generator=g, dtype=torch.int64).to(torch.int32).to(DEV)
        kc = torch.where(near, qc.view(B, Hc, H // Hc, W)[:, :, :1] ^ flips, kc)
    seq = torch.tensor(lens, dtype=torch.int32, device=DEV)
    cap = S if mode != _ops.HA_SELECT_SIMPLE else max(1, min(S, init + recent + (int(heavy) if heavy > 1 else int(S * heavy))))
    return kc, qc, S, seq, cap


def _both(B, H, Hc, W, lens, init=16, recent=16, heavy=0.125, mode=_ops.HA_SELECT_SIMPLE, depth=0, seed=0, check_oracle=True):
    kc, qc, S, seq, cap = _case(B, H, Hc, W, lens, init, recent, heavy, mode, depth, seed)
    idx_a = torch.full((B, H, cap), -1, dtype=torch.int32, device=DEV)
    idx_b = torch.full((B, H, cap), -1, dtype=torch.int32, device=DEV)
    cnt_a = torch.zeros(B, H, dtype=torch.int32, device=DEV)
    cnt_b = torch.zeros(B, H, dtype=torch.int32, device=DEV)
    ws = _ops.workspace(_ops.select_workspace_bytes(B, H, Hc, W, S), DEV)
    _ops.select(kc, qc, S, seq, init, recent, heavy, idx_a, cnt_a, ws, mode=mode, depth=depth)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(DEV)["allocation.all.allocated"], torch.cuda.mem_get_info()[0]
    _ops.select_static(kc, qc, S, seq, init, recent, heavy, idx_b, cnt_b, mode=mode, depth=depth)
    torch.cuda.synchronize()
    after = torch.cuda.memory_stats(DEV)["allocation.all.allocated"], torch.cuda.mem_get_info()[0]
    assert torch.equal(cnt_a, cnt_b), (cnt_a, cnt_b)
    assert torch.equal(idx_a, idx_b)
    assert int(cnt_a.max()) > 0
    if check_oracle:        # and against the oracle directly, not only through ha_select
        ref_idx, ref_cnt = c_oracle.select(kc.cpu().numpy(), qc.cpu().numpy(), np.array(lens, dtype=np.int32), init, recent, heavy, cap,
                                           mode=0 if mode == _ops.HA_SELECT_SIMPLE else 1, depth=depth)
        assert np.array_equal(cnt_b.cpu().numpy(), ref_cnt) and np.array_equal(idx_b.cpu().numpy(), ref_idx)
    return before, after


def test_select_static_matches_select_on_calls_in_a_row():
    print("\n[case] ha_select_static vs ha_select", flush=True)
    lib = _ops.load_library()
    assert lib.ha_select_static_max_bytes() == 8 << 20
    _both(4, 8, 2, 1, [20000, 9000, 4097, 12345], seed=1)                       # first call on this GPU: resolves the array
    before, after = _both(2, 8, 2, 1, [3000, 1500], seed=2)                     # smaller, right behind it
    assert before == after, "ha_select_static changed the allocator's state or the free device memory"
    _both(1, 4, 4, 1, [700], init=4, recent=4, heavy=50.0, seed=3)             # smaller still, absolute budget
    _both(3, 8, 4, 2, [9000, 2000, 30000], heavy=1.0 / 16, seed=4)              # larger again, 64-bit codes
    _both(2, 8, 2, 1, [5000, 2500], mode=_ops.HA_SELECT_THRESHOLD, depth=2, seed=5)
    _both(2, 8, 2, 1, [100, 20], seed=6)                                        # rows that are all window
    _both(16, 32, 8, 1, [65536] * 16, init=128, recent=128, heavy=1.0 / 32, seed=7, check_oracle=False)   # the headline shape: 1.2 MB of scratch


def test_select_static_refuses_what_does_not_fit():
    print("\n[case] ha_select_static: size limit", flush=True)
    B, H, Hc, W, S = 64, 32, 8, 2, 131072              # 64 * 32 rows * 32 chunks * 65 levels * 4 bytes = 17 MB
    kc = torch.zeros(1, Hc, S, W, dtype=torch.int32, device=DEV).expand(B, -1, -1, -1)
    qc = torch.zeros(B, H, W, dtype=torch.int32, device=DEV)
    idx = torch.zeros(B, H, 16, dtype=torch.int32, device=DEV)
    cnt = torch.full((B, H), -7, dtype=torch.int32, device=DEV)
    with pytest.raises(_ops.HashAttnError) as e:
        _ops.select_static(kc, qc, S, None, 4, 4, 0.01, idx, cnt)
    assert e.value.status == -5 and "ha_select_static" in str(e.value) and "ha_select_workspace_bytes" in str(e.value)
    torch.cuda.synchronize()
    assert (cnt == -7).all()                            # refused before anything was launched

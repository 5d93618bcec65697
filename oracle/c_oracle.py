"""numpy-facing loader of the C oracle (oracle/hashattn_oracle.c).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhashattn_oracle.so")
_lib = None


def build() -> str:
    subprocess.run(["gcc", "-O2", "-fopenmp", "-shared", "-fPIC", "-o", LIB_PATH,
                    os.path.join(_HERE, "hashattn_oracle.c"), "-lm"], check=True)
    return LIB_PATH


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _u32(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32) if a.dtype == np.int32 else a.astype(np.uint32)


def hamming(kcodes, qcodes, seq_lens) -> np.ndarray:
    """kcodes [B,Hc,S,W], qcodes [B,H,W] (uint32/int32), seq_lens [B] -> uint8 [B,H,S] (255 beyond seq_len)."""
    kc, qc = _u32(kcodes), _u32(qcodes)
    B, Hc, S, W = kc.shape
    H = qc.shape[1]
    sl = np.ascontiguousarray(seq_lens, dtype=np.int32)
    out = np.full((B, H, S), 255, dtype=np.uint8)
    lib().orc_hamming(_p(kc), _p(qc), B, H, Hc, C.c_int64(S), W, _p(sl), _p(out))
    return out


def select(kcodes, qcodes, seq_lens, init, recent, heavy_budget, idx_cap, mode=0, depth=0):
    """-> (idx int32 [B,H,idx_cap] ascending, padded with -1; counts int32 [B,H])."""
    kc, qc = _u32(kcodes), _u32(qcodes)
    B, Hc, S, W = kc.shape
    H = qc.shape[1]
    sl = np.ascontiguousarray(seq_lens, dtype=np.int32)
    idx = np.full((B, H, idx_cap), -1, dtype=np.int32)
    counts = np.zeros((B, H), dtype=np.int32)
    lib().orc_select(_p(kc), _p(qc), B, H, Hc, C.c_int64(S), W, _p(sl), int(init), int(recent), C.c_double(heavy_budget),
                     int(mode), int(depth), _p(idx), C.c_int64(idx_cap), _p(counts))
    return idx, counts


def encode(x, layers):
    """x fp32 [n, in]; layers [(W [out,in], b [out])] numpy fp32 -> (logits [n, D], codes uint32 [n, D/32])."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    n = x.shape[0]
    Ws = [np.ascontiguousarray(W, dtype=np.float32) for W, _ in layers]
    bs = [np.ascontiguousarray(b, dtype=np.float32) for _, b in layers]
    dims = np.array([Ws[0].shape[1]] + [W.shape[0] for W in Ws], dtype=np.int32)
    D = int(dims[-1])
    logits = np.empty((n, D), dtype=np.float32)
    codes = np.empty((n, D // 32), dtype=np.uint32)
    Wp = (C.c_void_p * len(Ws))(*[W.ctypes.data for W in Ws])
    bp = (C.c_void_p * len(bs))(*[b.ctypes.data for b in bs])
    lib().orc_encode(_p(x), C.c_int64(n), len(Ws), _p(dims), Wp, bp, _p(logits), _p(codes))
    return logits, codes


_DT = {"float32": 0, "bfloat16": 1, "float16": 2}


def _raw(t):
    """torch tensor -> (numpy view of raw storage, dtype code)."""
    import torch
    t = t.detach().contiguous().cpu()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy(), 1
    if t.dtype == torch.float16:
        return t.view(torch.int16).numpy(), 2
    return t.float().numpy(), 0


def sparse_attend(q, k, v, idx, counts, sm_scale) -> np.ndarray:
    """q [B,H,d], k/v [B,Hkv,S,d] torch tensors; idx [B,H,cap], counts [B,H] numpy -> fp32 [B,H,d]."""
    qa, dt = _raw(q)
    ka, _ = _raw(k)
    va, _ = _raw(v)
    B, H, d = q.shape
    Hkv, S = k.shape[1], k.shape[2]
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    counts = np.ascontiguousarray(counts, dtype=np.int32)
    out = np.empty((B, H, d), dtype=np.float32)
    lib().orc_sparse_attend(_p(qa), _p(ka), _p(va), dt, B, H, Hkv, C.c_int64(S), d, _p(idx), C.c_int64(idx.shape[2]),
                            _p(counts), C.c_double(sm_scale), _p(out))
    return out


def dense_attend(q, k, v, seq_lens, sm_scale) -> np.ndarray:
    qa, dt = _raw(q)
    ka, _ = _raw(k)
    va, _ = _raw(v)
    B, H, d = q.shape
    Hkv, S = k.shape[1], k.shape[2]
    sl = np.ascontiguousarray(seq_lens, dtype=np.int32)
    out = np.empty((B, H, d), dtype=np.float32)
    lib().orc_dense_attend(_p(qa), _p(ka), _p(va), dt, B, H, Hkv, C.c_int64(S), d, _p(sl), C.c_double(sm_scale), _p(out))
    return out

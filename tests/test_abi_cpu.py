"""Host-side checks of the C ABI that need no GPU: the library loads, exports every function the header declares,
sizes its workspaces sensibly and validates arguments before it touches HIP (so a bad call is refused with the
same status on any machine).  No kernel is launched here."""
import ctypes as C
import os
import re

import pytest
import torch

from hashattention import _ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hashattn.h")

HA_ERR_NULL, HA_ERR_SHAPE, HA_ERR_DTYPE, HA_ERR_ALIGN, HA_ERR_WS, HA_ERR_NODEV = -1, -2, -3, -4, -5, -6


@pytest.fixture(scope="module")
def lib():
    return _ops.load_library()


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ha_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    names = _declared_functions()
    assert {"ha_version", "ha_encode_pack", "ha_encode_step", "ha_encode_pack_prefill", "ha_hamming_score", "ha_select",
            "ha_sparse_decode", "ha_dense_decode", "ha_select_workspace_bytes", "ha_sparse_decode_workspace_bytes",
            "ha_dense_decode_workspace_bytes", "ha_usa_packed_floats", "ha_status_string", "ha_last_error_string",
            "ha_device_count"} <= set(names)
    for n in names:
        assert hasattr(lib, n), n
    assert lib.ha_version() == 202
    assert lib.ha_status_string(0) == b"ok" and lib.ha_status_string(HA_ERR_WS) == b"workspace missing or too small"


def test_packed_weight_sizes(lib):
    assert lib.ha_usa_packed_floats(3, 128, 128, 32) == 128 * 128 + 128 + 128 * 128 + 128 + 128 * 32 + 32 == 37152
    assert lib.ha_usa_packed_floats(2, 128, 128, 64) == 24768
    assert lib.ha_usa_packed_floats(1, 128, 128, 32) == 128 * 32 + 32
    assert lib.ha_usa_packed_floats(0, 128, 128, 32) == 0
    W = torch.arange(6.0).reshape(2, 3)
    blob = _ops.pack_usa_weights([[(W, torch.tensor([7.0, 8.0]))]])
    assert blob.tolist() == [[0, 3, 1, 4, 2, 5, 7, 8]]          # W^T [in][out], then the bias
    assert _ops.pack_usa_weights_bf16([[(W, torch.tensor([7.0, 8.0]))]]).float().tolist() == [[0, 1, 2, 3, 4, 5, 7, 8]]


def test_workspace_sizes(lib):
    assert lib.ha_select_workspace_bytes(0, 32, 8, 1, 100) == 0 and lib.ha_select_workspace_bytes(1, 32, 8, 3, 100) == 0
    small = lib.ha_select_workspace_bytes(1, 32, 8, 1, 4096)
    big = lib.ha_select_workspace_bytes(16, 32, 8, 1, 65536)
    assert 0 < small < big < 128 << 20
    assert lib.ha_select_workspace_bytes(16, 32, 8, 2, 65536) >= big
    assert 0 < lib.ha_sparse_decode_workspace_bytes(16, 32, 2304) < 64 << 20
    assert 0 < lib.ha_dense_decode_workspace_bytes(16, 32, 65536) < 256 << 20


def _buf(n=4096):
    return (C.c_char * n)()


def _aligned(buf, a=256):
    addr = C.addressof(buf)
    return C.c_void_p((addr + a - 1) // a * a)


def test_arguments_are_validated_before_any_device_work(lib):
    """Host buffers stand in for device pointers: every call below must be refused during validation."""
    b = _buf(1 << 16)
    p = _aligned(b)
    odd = C.c_void_p(p.value + 2)
    null = None
    # select
    args = dict(kcodes=p, sb=1024, sh=1024, q=p, B=1, H=4, Hc=2, W=1, S=1000, sl=null, init=4, rec=4, hb=C.c_double(0.25),
                mode=0, depth=0, algo=0, idx=p, cap=300, cnt=p, ws=p, wsb=1 << 16, st=null)

    def select(**kw):
        a = {**args, **kw}
        return lib.ha_select(a["kcodes"], a["sb"], a["sh"], a["q"], a["B"], a["H"], a["Hc"], a["W"], a["S"], a["sl"], a["init"], a["rec"],
                             a["hb"], a["mode"], a["depth"], a["algo"], a["idx"], a["cap"], a["cnt"], a["ws"], a["wsb"], a["st"])

    assert select(kcodes=null) == HA_ERR_NULL and b"NULL" in lib.ha_last_error_string()
    assert select(idx=null) == HA_ERR_NULL
    assert select(W=3) == HA_ERR_SHAPE
    assert select(Hc=3) == HA_ERR_SHAPE                        # H not a multiple of Hc
    assert select(H=32, Hc=2) == HA_ERR_SHAPE                  # 16 query heads per code head
    assert select(sh=999) == HA_ERR_SHAPE                      # row stride shorter than the sequence
    assert select(init=-1) == HA_ERR_SHAPE and select(hb=C.c_double(-0.5)) == HA_ERR_SHAPE and select(mode=7) == HA_ERR_SHAPE
    assert select(cap=0) == HA_ERR_SHAPE and select(algo=9) == HA_ERR_SHAPE
    assert select(kcodes=odd) == HA_ERR_ALIGN
    assert select(ws=null) == HA_ERR_WS and select(wsb=16) == HA_ERR_WS
    assert select(ws=C.c_void_p(p.value + 64)) == HA_ERR_ALIGN

    # sparse / dense decode
    def sparse(**kw):
        a = dict(q=p, qsb=512, qsh=128, k=p, v=p, dt=_ops.HA_BF16, sb=128000, sh=128000, ss=128, B=1, H=4, Hkv=2, idx=p, cap=300,
                 cnt=p, sc=C.c_float(0.088), out=p, ws=p, wsb=1 << 16, st=null)
        a.update(kw)
        return lib.ha_sparse_decode(a["q"], a["qsb"], a["qsh"], a["k"], a["v"], a["dt"], a["sb"], a["sh"], a["ss"], a["B"], a["H"], a["Hkv"],
                                    a["idx"], a["cap"], a["cnt"], a["sc"], a["out"], a["ws"], a["wsb"], a["st"])

    assert sparse(v=null) == HA_ERR_NULL and sparse(idx=null) == HA_ERR_NULL
    assert sparse(dt=9) == HA_ERR_DTYPE
    assert sparse(Hkv=3) == HA_ERR_SHAPE and sparse(ss=64) == HA_ERR_SHAPE
    assert sparse(k=odd) == HA_ERR_ALIGN and sparse(ss=132) == HA_ERR_ALIGN     # rows would not stay 16-byte aligned
    assert sparse(wsb=8) == HA_ERR_WS

    def masked(**kw):
        a = dict(mask=p, msb=400, mlen=400, slot=0, cap=300, Hkv=2, wsb=1 << 16)
        a.update(kw)
        return lib.ha_sparse_decode_masked(p, 512, 128, p, p, _ops.HA_BF16, 128000, 128000, 128, 1, 4, a["Hkv"], p, a["cap"], p,
                                           C.c_float(0.088), a["mask"], a["msb"], a["mlen"], a["slot"], p, p, a["wsb"], null)

    assert masked(mask=null) == HA_ERR_NULL
    assert masked(mlen=0) == HA_ERR_SHAPE and masked(msb=-1) == HA_ERR_SHAPE and masked(slot=2) == HA_ERR_SHAPE
    assert masked(slot=1, mlen=299) == HA_ERR_SHAPE              # a mask by list slot must cover the whole list
    assert masked(mask=odd) == HA_ERR_ALIGN
    assert masked(Hkv=3) == HA_ERR_SHAPE and masked(wsb=8) == HA_ERR_WS      # the checks of ha_sparse_decode apply
    assert masked() == HA_ERR_NODEV and masked(slot=1) == HA_ERR_NODEV

    def paged(**kw):        # the list-fed attention through a token -> slot table
        a = dict(tab=p, tsb=1000, n=5000, mask=null, rps=1, B=2, Hkv=2)
        a.update(kw)
        return lib.ha_sparse_decode_paged(p, 512, 128, p, p, _ops.HA_BF16, 0, 128, 256, a["B"], a["rps"], 4, a["Hkv"], p, 300, p,
                                          C.c_float(0.088), a["mask"], 400, 400, 0, a["tab"], a["tsb"], a["n"], p, p, 1 << 16, null)

    assert paged(tab=null) == HA_ERR_NULL and paged(tsb=-1) == HA_ERR_SHAPE and paged(n=0) == HA_ERR_SHAPE
    assert paged(tab=odd) == HA_ERR_ALIGN and paged(rps=3) == HA_ERR_SHAPE and paged(Hkv=3) == HA_ERR_SHAPE
    assert paged() == HA_ERR_NODEV and paged(mask=p) == HA_ERR_NODEV and paged(B=4, rps=2) == HA_ERR_NODEV
    assert lib.ha_dense_decode(p, 512, 128, p, p, _ops.HA_F32, 128000, 128000, 128, 1, 4, 2, 0, null, C.c_float(0.1), p, p, 1 << 16,
                               null) == HA_ERR_SHAPE           # max_seq_len must be positive

    # encoders
    def enc(**kw):
        a = dict(x=p, dt=_ops.HA_BF16, sb=1280, sh=1280, st_=128, B=1, xh=2, nh=4, T=10, w=p, nl=3, hd=128, idim=128, fd=32, ar=0,
                 codes=p, csb=64, csh=16, pos0=0, pd=null, lg=null, st=null)
        a.update(kw)
        return lib.ha_encode_pack(a["x"], a["dt"], a["sb"], a["sh"], a["st_"], a["B"], a["xh"], a["nh"], a["T"], a["w"], a["nl"], a["hd"],
                                  a["idim"], a["fd"], a["ar"], a["codes"], a["csb"], a["csh"], a["pos0"], a["pd"], a["lg"], a["st"])

    assert enc(w=null) == HA_ERR_NULL

    def enc_cached(**kw):
        a = dict(k=p, ss=128, q=p, lens=p, H=4, hd=128, dt=_ops.HA_BF16)
        a.update(kw)
        return lib.ha_encode_step_cached(a["k"], 128000, 64000, a["ss"], a["q"], 512, 128, a["dt"], 1, 2, 2, a["H"], a["lens"], p, p, 3,
                                         a["hd"], 128, 32, 0, p, 4000, 1000, p, null)

    assert enc_cached(k=null) == HA_ERR_NULL and enc_cached(lens=null) == HA_ERR_NULL and enc_cached(q=null) == HA_ERR_NULL
    assert enc_cached(ss=64) == HA_ERR_SHAPE and enc_cached(H=0) == HA_ERR_SHAPE and enc_cached(dt=7) == HA_ERR_DTYPE
    assert enc_cached() == HA_ERR_NODEV
    assert enc(fd=48) == HA_ERR_SHAPE and enc(nl=4) == HA_ERR_SHAPE and enc(nh=3) == HA_ERR_SHAPE and enc(hd=300) == HA_ERR_SHAPE
    assert enc(dt=5) == HA_ERR_DTYPE and enc(ar=2) == HA_ERR_DTYPE
    # positions given by the host must lie inside the row of the code buffer (16 tokens between heads here); positions
    # read from device memory are the kernel's to skip
    assert enc(pos0=7) == HA_ERR_SHAPE and b"code row" in lib.ha_last_error_string()
    assert enc(pos0=6) == HA_ERR_NODEV and enc(pos0=7, pd=p) == HA_ERR_NODEV
    assert lib.ha_encode_pack_prefill(p, 1280, 1280, 128, 1, 2, 4, 10, p, 3, 128, 128, 32, p, 64, 16, 7, null, null) == HA_ERR_SHAPE
    assert lib.ha_encode_pack_prefill(p, 1280, 1280, 128, 1, 2, 4, 10, p, 3, 128, 128, 32, p, 64, 16, 6, null, null) == HA_ERR_NODEV
    assert lib.ha_encode_pack_prefill(p, 1280, 1280, 128, 1, 2, 4, 10, p, 3, 128, 64, 32, p, 64, 16, 0, null, null) == HA_ERR_SHAPE
    assert lib.ha_encode_pack_prefill(odd, 1280, 1280, 128, 1, 2, 4, 10, p, 3, 128, 128, 32, p, 64, 16, 0, null, null) == HA_ERR_ALIGN
    assert lib.ha_hamming_score(p, 1024, 1024, p, 1, 4, 2, 1, 1000, null, null, null) == HA_ERR_NULL

    # fused select-attend
    def prep(**kw):
        a = {**args, **kw}
        return lib.ha_select_prepare(a["kcodes"], a["sb"], a["sh"], a["q"], a["B"], a["H"], a["Hc"], a["W"], a["S"], a["sl"], a["init"],
                                     a["rec"], a["hb"], a["mode"], a["depth"], a["cnt"], a["ws"], a["wsb"], a["st"])

    assert prep(cnt=null) == HA_ERR_NULL and prep(W=3) == HA_ERR_SHAPE and prep(wsb=16) == HA_ERR_WS
    assert lib.ha_sparse_decode_fused_applies(1, 4, 2, 1, 1000, 4, 4, C.c_double(0.25), 0) == 1
    assert lib.ha_sparse_decode_fused_applies(1, 4, 2, 1, 1000, 4, 4, C.c_double(0.25), 1) == 0          # threshold mode
    assert lib.ha_sparse_decode_fused_applies(1, 4, 2, 1, 100000, 4, 4, C.c_double(0.25), 0) == 0        # 25 008 entries > 8192
    assert lib.ha_sparse_decode_fused_applies(1, 8, 8, 1, 1 << 22, 4, 4, C.c_double(4000.0), 0) == 1     # any length: the list is what counts
    assert lib.ha_sparse_decode_fused_workspace_bytes(1, 4, 2, 1000) > 0
    assert lib.ha_sparse_decode_fused_local_thresholds(1, 2, 1000) == 1 and lib.ha_sparse_decode_fused_local_thresholds(1, 2, 1 << 20) == 0
    assert lib.ha_select_histogram(p, 1024, 1024, null, 1, 4, 2, 1, 1000, null, 4, 4, p, 1 << 20, null) == HA_ERR_NULL

    def fused(**kw):
        a = dict(q=p, qsb=512, qsh=128, k=p, v=p, dt=_ops.HA_BF16, sb=128000, sh=128000, ss=128, kc=p, csb=1024, csh=1024, qc=p, B=1, H=4,
                 Hkv=2, Hc=2, W=1, S=1000, sl=null, init=4, rec=4, hb=C.c_double(0.25), sws=p, swsb=1 << 20, tr=1, oc=null,
                 sc=C.c_float(0.088), out=p, ws=p, wsb=1 << 20, st=null)
        a.update(kw)
        return lib.ha_sparse_decode_fused(a["q"], a["qsb"], a["qsh"], a["k"], a["v"], a["dt"], a["sb"], a["sh"], a["ss"], a["kc"], a["csb"],
                                          a["csh"], a["qc"], a["B"], a["H"], a["Hkv"], a["Hc"], a["W"], a["S"], a["sl"], a["init"], a["rec"],
                                          a["hb"], a["sws"], a["swsb"], a["tr"], a["oc"], a["sc"], a["out"], a["ws"], a["wsb"], a["st"])

    assert fused(kc=null) == HA_ERR_NULL and fused(sws=null) == HA_ERR_NULL and fused(dt=9) == HA_ERR_DTYPE
    assert fused(Hc=3) == HA_ERR_SHAPE and fused(csh=999) == HA_ERR_SHAPE and fused(hb=C.c_double(0.9), S=60000, csb=60000, csh=60000) == HA_ERR_SHAPE
    assert fused(swsb=16) == HA_ERR_WS and fused(wsb=16) == HA_ERR_WS and fused(k=odd) == HA_ERR_ALIGN

    def fused_paged(**kw):
        a = dict(tab=p, tsb=1000, n=5000, Hc=2)
        a.update(kw)
        return lib.ha_sparse_decode_fused_paged(p, 512, 128, p, p, _ops.HA_BF16, 0, 128, 256, p, 1024, 1024, p, 1, 4, 2, a["Hc"], 1, 1000, null,
                                                4, 4, C.c_double(0.25), p, 1 << 20, 1, null, a["tab"], a["tsb"], a["n"], C.c_float(0.088), p,
                                                p, 1 << 20, null)

    assert fused_paged(tab=null) == HA_ERR_NULL and fused_paged(n=1 << 40) == HA_ERR_SHAPE and fused_paged(tab=odd) == HA_ERR_ALIGN
    assert fused_paged(Hc=3) == HA_ERR_SHAPE and fused_paged() == HA_ERR_NODEV

    # decoder plumbing
    def rope(**kw):
        a = dict(qkv=p, sb=768, dt=_ops.HA_BF16, B=1, H=4, Hkv=1, pos=5, pd=null, f=p, q=p, k=p, v=p, ksb=12800, ksh=12800, kss=128,
                 cl=100, st=null)
        a.update(kw)
        return lib.ha_rope_append(a["qkv"], a["sb"], a["dt"], a["B"], a["H"], a["Hkv"], a["pos"], a["pd"], a["f"], a["q"], a["k"], a["v"],
                                  a["ksb"], a["ksh"], a["kss"], a["cl"], a["st"])

    assert rope(f=null) == HA_ERR_NULL and rope(dt=7) == HA_ERR_DTYPE
    assert rope(sb=512) == HA_ERR_SHAPE and rope(pos=100) == HA_ERR_SHAPE and rope(pos=-1) == HA_ERR_SHAPE and rope(kss=64) == HA_ERR_SHAPE
    import ctypes as _C
    lib.ha_rope_encode_step.restype = _C.c_int
    i64 = _C.c_int64

    def rope_enc(**kw):
        a = dict(qkv=p, sb=i64(48 * 128), dt=_ops.HA_BF16, B=1, H=32, Hkv=8, Hc=8, pos=3, pd=null, f=p, q=p, k=p, v=p, ksb=i64(8 * 100 * 128),
                 ksh=i64(100 * 128), kss=i64(128), cl=i64(100), wk=p, wq=p, nl=3, hd=128, idim=128, fd=32, ar=0, kc=p, csb=i64(800), csh=i64(100),
                 qc=p, st=null)
        a.update(kw)
        return lib.ha_rope_encode_step(*[a[k] for k in ("qkv", "sb", "dt", "B", "H", "Hkv", "Hc", "pos", "pd", "f", "q", "k", "v", "ksb", "ksh",
                                                        "kss", "cl", "wk", "wq", "nl", "hd", "idim", "fd", "ar", "kc", "csb", "csh", "qc", "st")])

    assert rope_enc(f=null) == HA_ERR_NULL and rope_enc(qc=null) == HA_ERR_NULL and rope_enc(dt=7) == HA_ERR_DTYPE
    assert rope_enc(hd=64) == HA_ERR_SHAPE and rope_enc(pos=100) == HA_ERR_SHAPE and rope_enc(sb=i64(512)) == HA_ERR_SHAPE
    assert rope_enc(fd=48) == HA_ERR_SHAPE and rope_enc(Hc=3) == HA_ERR_SHAPE
    lin = lambda **kw: lib.ha_linear_skinny(*[{**dict(x=p, xs=4096, w=p, ws=4096, r=null, rs=0, o=p, os=4096, M=4, N=4096, K=4096, st=null), **kw}[k]
                                              for k in ("x", "xs", "w", "ws", "r", "rs", "o", "os", "M", "N", "K", "st")])
    assert lin(w=null) == HA_ERR_NULL and lin(M=17) == HA_ERR_SHAPE and lin(K=100) == HA_ERR_SHAPE and lin(ws=100) == HA_ERR_SHAPE
    assert lin(x=odd) == HA_ERR_ALIGN and lin(xs=4100) == HA_ERR_ALIGN and lin(r=p, rs=10) == HA_ERR_SHAPE
    linf = lambda **kw: lib.ha_linear_skinny_fused(*[{**dict(x=p, xs=4096, w=p, ws=4096, r=null, rs=0, g=p, eps=C.c_float(1e-5), act=1, o=p, os=4096,
                                                            M=4, N=4096, K=4096, st=null), **kw}[k]
                                                     for k in ("x", "xs", "w", "ws", "r", "rs", "g", "eps", "act", "o", "os", "M", "N", "K", "st")])
    assert linf(act=5) == HA_ERR_SHAPE and linf(N=4095) == HA_ERR_SHAPE and linf(r=p, rs=4096) == HA_ERR_SHAPE      # SwiGLU: even rows, no residual
    assert linf(M=9) == HA_ERR_SHAPE and linf(K=32768, xs=32768, ws=32768) == HA_ERR_SHAPE and linf(g=odd) == HA_ERR_ALIGN
    assert linf(os=1000) == HA_ERR_SHAPE and linf(eps=C.c_float(-1.0)) == HA_ERR_ALIGN
    # tiled projections, the RMSNorm launch, the fused launch with a masked prefix
    assert lib.ha_weight_tiles_elems(6144, 4096, 0) == 6144 * 4096 and lib.ha_weight_tiles_elems(100, 64, 0) == 112 * 64
    assert lib.ha_weight_tiles_elems(2 * 100, 64, 1) == 13 * 16 * 64            # 100 columns: 13 tiles of 8 gate + 8 up rows
    assert lib.ha_weight_tiles_elems(64, 100, 0) == 0 and lib.ha_weight_tiles_elems(7, 64, 1) == 0 and lib.ha_weight_tiles_elems(0, 64, 0) == 0
    pack = lambda **kw: lib.ha_pack_weight_tiles(*[{**dict(w=p, ws=4096, N=64, K=4096, glu=0, t=p, st=null), **kw}[k]
                                                   for k in ("w", "ws", "N", "K", "glu", "t", "st")])
    assert pack(t=null) == HA_ERR_NULL and pack(K=100) == HA_ERR_SHAPE and pack(ws=64) == HA_ERR_SHAPE and pack(N=7, glu=1) == HA_ERR_SHAPE
    assert pack(w=odd) == HA_ERR_ALIGN and pack(glu=2) == HA_ERR_SHAPE
    lint = lambda **kw: lib.ha_linear_tiled(*[{**dict(x=p, xs=4096, t=p, r=null, rs=0, act=0, o=p, os=4096, M=16, N=4096, K=4096, st=null), **kw}[k]
                                              for k in ("x", "xs", "t", "r", "rs", "act", "o", "os", "M", "N", "K", "st")])
    assert lint(t=null) == HA_ERR_NULL and lint(M=33) == HA_ERR_SHAPE and lint(K=100) == HA_ERR_SHAPE and lint(x=odd) == HA_ERR_ALIGN
    assert lint(M=17, K=8192, xs=8192) == HA_ERR_SHAPE          # more than 16 rows: up to 4096 inputs
    assert lint(K=16384, xs=16384, act=1, N=4096) == HA_ERR_SHAPE    # rows too long for registers: no activation
    assert lint(act=1, r=p, rs=4096) == HA_ERR_SHAPE and lint(act=1, N=4095) == HA_ERR_SHAPE and lint(os=100) == HA_ERR_SHAPE
    assert lint(r=p, rs=10) == HA_ERR_SHAPE and lint(act=3) == HA_ERR_SHAPE
    norm = lambda **kw: lib.ha_rmsnorm(*[{**dict(x=p, xs=4096, w=p, dt=_ops.HA_BF16, M=4, K=4096, eps=C.c_float(1e-5), o=p, os=4096, st=null), **kw}[k]
                                         for k in ("x", "xs", "w", "dt", "M", "K", "eps", "o", "os", "st")])
    assert norm(w=null) == HA_ERR_NULL and norm(dt=9) == HA_ERR_DTYPE and norm(xs=100) == HA_ERR_SHAPE and norm(M=0) == HA_ERR_SHAPE
    assert norm(eps=C.c_float(-1.0)) == HA_ERR_SHAPE
    lib.ha_sparse_decode_fused_prefix_masked.restype = _C.c_int
    fpm = lambda pre: lib.ha_sparse_decode_fused_prefix_masked(p, i64(4096), i64(128), p, p, _ops.HA_BF16, i64(8 * 1000 * 128), i64(1000 * 128), i64(128),
                                                               p, i64(8000), i64(1000), p, 1, 32, 8, 8, 1, 1000, null, 4, 4, C.c_double(0.25),
                                                               p, C.c_size_t(1 << 16), 1, null, pre, C.c_float(0.1), p, p, C.c_size_t(1 << 16), null)
    assert fpm(null) == HA_ERR_NULL and fpm(odd) == HA_ERR_ALIGN
    assert lib.ha_swiglu(null, 64, _ops.HA_BF16, 1, 32, p, null) == HA_ERR_NULL
    assert lib.ha_swiglu(p, 63, _ops.HA_BF16, 1, 32, p, null) == HA_ERR_SHAPE and lib.ha_swiglu(p, 64, 9, 1, 32, p, null) == HA_ERR_DTYPE


@pytest.mark.skipif(torch.cuda.is_available(), reason="this check is about a machine without a GPU")
def test_no_device_is_a_status_not_a_crash(lib):
    b = _buf(1 << 16)
    p = _aligned(b)
    assert lib.ha_device_count() == 0
    st = lib.ha_hamming_score(p, 1024, 1024, p, 1, 4, 2, 1, 1000, None, p, None)
    assert st == HA_ERR_NODEV and b"no HIP device" in lib.ha_last_error_string()
    with pytest.raises(ValueError):                            # the Python layer refuses CPU tensors outright
        _ops.hamming_score(torch.zeros(1, 1, 4, 1, dtype=torch.int32), torch.zeros(1, 1, 1, dtype=torch.int32), 4)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_ops, "_lib", None)
    monkeypatch.setattr(_ops, "lib_path", lambda: str(tmp_path / "libhashattn.so"))
    with pytest.raises(ImportError):
        _ops.load_library()


def test_module_api_helpers_of_the_reference_are_present():
    """Small pieces of the reference's module surface that need no kernel: `ste_sign` (sign forward, tanh-derivative
    backward, hashattention_llama.py:51-66), `memory_efficient_softmax` (:37-44), `DEFAULT_USA_CFG` (:68-72)."""
    import torch
    from hashattention import hashattention_llama as hl, hashattention_mistral as hm
    x = torch.tensor([-2.0, -0.0, 0.0, 0.3, 5.0], requires_grad=True)
    y = hl.ste_sign(x)
    assert y.tolist() == [-1.0, 0.0, 0.0, 1.0, 1.0]
    (y * torch.arange(1.0, 6.0)).sum().backward()
    assert torch.allclose(x.grad, torch.arange(1.0, 6.0) * (1 - torch.tanh(x.detach()) ** 2))
    z = torch.randn(3, 7) * 30
    assert torch.allclose(hl.memory_efficient_softmax(z, dim=-1), torch.softmax(z, dim=-1), atol=1e-6)
    assert hl.DEFAULT_USA_CFG == {"lth_int_dim": 128, "lth_final_dim": 32, "lth_thold": 0}
    for api in (hl, hm):
        for name in ("USA", "load_usa", "convert_usa", "reset_usa", "set_train_usa_mode", "set_eval_usa_mode", "print_stats"):
            assert callable(getattr(api, name))

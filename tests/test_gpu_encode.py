"""GPU checks of the hash-MLP encoders.

fp32 arithmetic (ha_encode_pack, HA_ARITH_F32) is covered stage by stage in test_gpu_parity.  Here:
  - the bf16-arithmetic scalar kernel against torch running the same MLP in bf16 on the CPU;
  - the MFMA prefill encoder against the bf16 scalar kernel (same arithmetic, different summation order);
  - appending to the bit-cache at an offset / per-sequence offsets leaves the other positions untouched.
bf16 rounding makes a different summation order flip a rounding now and then, so these two are judged on
the bit-agreement rate, not exactness; the fp32 path is the bit-exact one.
"""
import numpy as np
import pytest
import torch

from hashattention import _ops
from hashattention.synthetic import make_problem
from oracle import hashattn_oracle as orc
from tests.parity_util import small_workload

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _bits_differing(a: torch.Tensor, b: torch.Tensor) -> int:
    x = (a.cpu().numpy().view(np.uint32) ^ b.cpu().numpy().view(np.uint32))
    return int(np.unpackbits(x.view(np.uint8)).sum())


def _bf16_layers(heads):
    return [[(W.to(torch.bfloat16), b.to(torch.bfloat16)) for W, b in layers] for layers in heads]


@pytest.mark.parametrize("layers,final", [(3, 32), (2, 64), (1, 32), (3, 64), (2, 32), (1, 64)])
def test_bf16_arith_and_mfma_agree(layers, final):
    print(f"\n[case] encoders layers={layers} final={final}", flush=True)
    w = small_workload(batch=2, seq_lens=[3000, 1700], lth_num_layers=layers, lth_final_dim=final, seed=70 + layers)
    p = make_problem(w)
    B, Hc, S, W = w.batch, w.n_code_heads, w.max_seq_len, w.code_words
    k = p.k.to(DEV)
    kb = _bf16_layers(p.usa.k)
    # torch bf16 on the CPU: the arithmetic a hash module kept in bf16 performs
    want = orc.pack_codes(orc.usa_logits(p.k, kb).float())
    want_i32 = torch.from_numpy(want.numpy().astype(np.uint32).view(np.int32).copy())

    wk32 = _ops.pack_usa_weights(kb, DEV)             # bf16 values, exactly representable in the fp32 blob
    wk16 = _ops.pack_usa_weights_bf16(kb, DEV)
    c_scalar = torch.zeros(B, Hc, S, W, dtype=torch.int32, device=DEV)
    c_mfma = torch.full((B, Hc, S, W), -1, dtype=torch.int32, device=DEV)
    _ops.encode_pack(k, wk32, layers, w.lth_int_dim, final, c_scalar, arith=_ops.HA_ARITH_BF16)
    _ops.encode_pack_prefill(k, wk16, layers, w.lth_int_dim, final, c_mfma)
    torch.cuda.synchronize()
    total = B * Hc * S * final
    d_ref = _bits_differing(c_scalar, want_i32) / total
    d_mfma = _bits_differing(c_mfma, c_scalar) / total
    print(f"  bits differing: scalar-bf16 vs torch-bf16 {d_ref:.2e}, mfma vs scalar-bf16 {d_mfma:.2e}", flush=True)
    # observed over the six shapes: at most 1.2e-3 against torch's bf16 arithmetic (another summation order inside every
    # Linear), at most one bit of 384 000 between the two kernels; bounds at three times that
    assert d_ref < 3.5e-3
    assert d_mfma < 1e-5


def test_mfma_tail_and_offsets():
    # T not a multiple of the 512-token tile nor of 32; append at pos0 and at per-sequence offsets
    print("\n[case] mfma tails/offsets", flush=True)
    w = small_workload(batch=2, seq_lens=[777, 777], seed=81)
    p = make_problem(w)
    kb = _bf16_layers(p.usa.k)
    k = p.k.to(DEV)
    wk16 = _ops.pack_usa_weights_bf16(kb, DEV)
    wk32 = _ops.pack_usa_weights(kb, DEV)
    B, Hc, S, W = w.batch, w.n_code_heads, w.max_seq_len, 1
    cap = S + 300
    for enc in ("mfma", "scalar"):
        full = torch.full((B, Hc, cap, W), 12345, dtype=torch.int32, device=DEV)
        part = torch.full((B, Hc, cap, W), 12345, dtype=torch.int32, device=DEV)
        pos = torch.tensor([100, 250], dtype=torch.int32, device=DEV)
        if enc == "mfma":
            _ops.encode_pack_prefill(k, wk16, 3, 128, 32, full, pos0=0)
            _ops.encode_pack_prefill(k[:, :, 5:600], wk16, 3, 128, 32, part, pos_dev=pos)
        else:
            _ops.encode_pack(k, wk32, 3, 128, 32, full, pos0=0, arith=_ops.HA_ARITH_BF16)
            _ops.encode_pack(k[:, :, 5:600], wk32, 3, 128, 32, part, pos_dev=pos, arith=_ops.HA_ARITH_BF16)
        torch.cuda.synchronize()
        assert (full[:, :, S:] == 12345).all(), enc
        for b, p0 in enumerate([100, 250]):
            assert torch.equal(part[b, :, p0:p0 + 595], full[b, :, 5:600]), enc
            assert (part[b, :, :p0] == 12345).all() and (part[b, :, p0 + 595:] == 12345).all(), enc


def test_exact_zero_logit_gives_bit_zero():
    # bit = (logit > 0): an exactly-zero logit packs as 0 (efficiency/kernels/torchatt.py:55, relu(sign(0)) = 0)
    W1 = torch.zeros(32, 128)
    b1 = torch.zeros(32)
    b1[::2] = 1.0
    b1[1::4] = -1.0          # dims 3, 7, 11, ... stay exactly 0
    x = torch.randn(1, 1, 9, 128, device=DEV)
    codes = torch.zeros(1, 1, 9, 1, dtype=torch.int32, device=DEV)
    _ops.encode_pack(x, _ops.pack_usa_weights([[(W1, b1)]], DEV), 1, 128, 32, codes)
    want = sum(1 << i for i in range(0, 32, 2))
    assert (codes.cpu().numpy().view(np.uint32) == want).all()


def test_encode_step_equals_two_encode_packs():
    # the single-launch step encode (new key + query) writes exactly what two separate launches write
    print("\n[case] encode_step", flush=True)
    for ragged in (False, True):
        w = small_workload(batch=5, seq_lens=[300] * 5, n_q_heads=8, n_kv_heads=2, n_code_heads=2, seed=91)
        p = make_problem(w)
        k, q = p.k.to(DEV), p.q.to(DEV)
        wk, wq = _ops.pack_usa_weights(p.usa.k, DEV), _ops.pack_usa_weights(p.usa.q, DEV)
        a = torch.full((5, 2, 304, 1), 7, dtype=torch.int32, device=DEV)
        b = a.clone()
        qa = torch.zeros(5, 8, 1, 1, dtype=torch.int32, device=DEV)
        qb = torch.zeros(5, 8, 1, dtype=torch.int32, device=DEV)
        if ragged:
            pos = torch.tensor([299, 10, 0, 150, 298], dtype=torch.int32, device=DEV)
            newk = torch.gather(k, 2, pos.view(-1, 1, 1, 1).expand(-1, 2, 1, 128).long())
            _ops.encode_pack(newk, wk, 3, 128, 32, a, pos_dev=pos)
            _ops.encode_step(newk, q[:, :, 0, :], wk, wq, 3, 128, 32, b, qb, pos_dev=pos)
        else:
            _ops.encode_pack(k[:, :, 299:300], wk, 3, 128, 32, a, pos0=299)
            _ops.encode_step(k[:, :, 299:300], q[:, :, 0, :], wk, wq, 3, 128, 32, b, qb, pos0=299)
        _ops.encode_pack(q, wq, 3, 128, 32, qa)
        torch.cuda.synchronize()
        assert torch.equal(a, b) and torch.equal(qa.view(5, 8, 1), qb)
        assert int((a != 7).sum()) == 5 * 2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_encode_step_cached_reads_the_new_keys_in_place(dtype):
    # lengths on the device: the key of sequence b is read from cache row seq_lens[b] - 1; the same bits as a gather of those
    # rows followed by ha_encode_step, and nothing else in the bit-cache is touched.  A length of 0 writes nothing.
    print(f"\n[case] encode_step_cached {dtype}", flush=True)
    g = torch.Generator().manual_seed(31)
    B, H, Hkv, Hc, cap, W = 5, 8, 2, 4, 300, 1
    w = small_workload(batch=1, seq_lens=[64], seed=33)
    p = make_problem(w)
    k_layers = (p.usa.k * 4)[:Hc]
    q_layers = (p.usa.q * 4)[:H]
    wk, wq = _ops.pack_usa_weights(k_layers, DEV), _ops.pack_usa_weights(q_layers, DEV)
    k_cache = torch.randn(B, Hkv, cap, 128, generator=g).to(dtype).to(DEV)
    q3 = torch.randn(B, H, 128, generator=g).to(dtype).to(DEV)
    lens = torch.tensor([300, 1, 0, 137, 42], dtype=torch.int32, device=DEV)
    arith = _ops.HA_ARITH_BF16 if dtype == torch.bfloat16 else _ops.HA_ARITH_F32
    got = torch.full((B, Hc, cap, W), 777, dtype=torch.int32, device=DEV)
    got_q = torch.zeros(B, H, W, dtype=torch.int32, device=DEV)
    _ops.encode_step_cached(k_cache, q3, wk, wq, 3, 128, 32, got, got_q, lens, arith=arith)
    want = torch.full((B, Hc, cap, W), 777, dtype=torch.int32, device=DEV)
    want_q = torch.zeros(B, H, W, dtype=torch.int32, device=DEV)
    live = [0, 1, 3, 4]
    pos = (lens - 1).clamp(min=0)
    newk = torch.gather(k_cache, 2, pos.view(-1, 1, 1, 1).expand(-1, Hkv, 1, 128).long())
    _ops.encode_step(newk, q3, wk, wq, 3, 128, 32, want, want_q, pos_dev=pos.to(torch.int32), arith=arith)
    torch.cuda.synchronize()
    assert torch.equal(got_q, want_q)
    assert torch.equal(got[live], want[live])
    assert (got[2] == 777).all()                                   # the empty sequence wrote nothing
    touched = (got != 777).sum().item()
    assert touched <= len(live) * Hc * W and touched >= len(live) * Hc * W - 2       # a code may happen to equal the filler


@pytest.mark.parametrize("int_dim,layers", [(256, 3), (200, 3), (64, 2), (256, 2)])
def test_generic_mlp_widths_against_the_oracle(int_dim, layers):
    # hidden widths other than 128: layers wider than 128 outputs stream their weights instead of parking them in
    # registers, widths that are not multiples of 16 keep the plain weight layout.  fp32 logits against torch, codes exact
    # wherever a logit is not within round-off of zero
    print(f"\n[case] hash MLP with hidden width {int_dim}, {layers} layers", flush=True)
    g = torch.Generator().manual_seed(int_dim + layers)
    B, Hx, Hn, T, D = 2, 2, 4, 37, 32
    dims = [(128, int_dim), (int_dim, int_dim), (int_dim, D)] if layers == 3 else [(128, int_dim), (int_dim, D)]
    heads = [[(torch.randn(o, i, generator=g) * i ** -0.5, torch.randn(o, generator=g) * 0.05) for i, o in dims] for _ in range(Hn)]
    x = torch.randn(B, Hx, T, 128, generator=g)
    want = orc.usa_logits(x, heads)                                      # [B, Hn, T, D]
    w = _ops.pack_usa_weights(heads, DEV)
    codes = torch.zeros(B, Hn, T, 1, dtype=torch.int32, device=DEV)
    got = _ops.encode_pack(x.to(DEV), w, layers, int_dim, D, codes, want_logits=True).cpu()
    torch.cuda.synchronize()
    err = (got - want).abs().max().item()
    print(f"  max |logit difference| {err:.2e}", flush=True)
    assert err < 1e-4
    want_codes = orc.pack_codes(want).numpy().astype(np.uint32)
    diff = codes.cpu().numpy().view(np.uint32) ^ want_codes
    bits = ((diff[..., 0, None] >> np.arange(32, dtype=np.uint32)) & 1).astype(bool)
    assert (np.abs(want.numpy())[bits] < 1e-4).all()


@pytest.mark.parametrize("B", [3, 20, 60])
def test_encode_step_rows_per_workgroup(B):
    # 3, 20 and 60 sequences: the step's encode launch runs one, two and four rows per workgroup; codes of the new keys and
    # of the queries against the oracle (bits may differ only where a logit is within round-off of zero)
    print(f"\n[case] encode_step, {B} sequences", flush=True)
    from tests.parity_util import compare_codes
    g = torch.Generator().manual_seed(50 + B)
    H, Hkv, Hc = 8, 2, 2
    w = small_workload(batch=1, seq_lens=[64], seed=51)
    p = make_problem(w)
    k_layers, q_layers = (p.usa.k * 4)[:Hc], (p.usa.q * 4)[:H]
    wk, wq = _ops.pack_usa_weights(k_layers, DEV), _ops.pack_usa_weights(q_layers, DEV)
    k_new = torch.randn(B, Hkv, 1, 128, generator=g)
    q = torch.randn(B, H, 1, 128, generator=g)
    kcodes = torch.zeros(B, Hc, 8, 1, dtype=torch.int32, device=DEV)
    qcodes = torch.zeros(B, H, 1, dtype=torch.int32, device=DEV)
    _ops.encode_step(k_new.to(DEV), q[:, :, 0].to(DEV), wk, wq, 3, 128, 32, kcodes, qcodes, pos0=5)
    torch.cuda.synchronize()
    kl, ql = orc.usa_logits(k_new, k_layers), orc.usa_logits(q, q_layers)
    want_k = orc.pack_codes(kl).numpy().astype(np.uint32)            # [B, Hc, 1, 1]
    want_q = orc.pack_codes(ql).numpy().astype(np.uint32)            # [B, H, 1, 1]
    nk = compare_codes("new keys", kcodes[:, :, 5:6].cpu().numpy().view(np.uint32), want_k, kl.numpy())
    nq = compare_codes("queries", qcodes.view(B, H, 1, 1).cpu().numpy().view(np.uint32), want_q, ql.numpy())
    print(f"  bits differing at near-zero logits: keys {nk}, queries {nq}", flush=True)
    assert (kcodes[:, :, :5] == 0).all() and (kcodes[:, :, 6:] == 0).all()


def test_device_side_positions_outside_the_cache_write_nothing():
    # Positions read from device memory cannot be checked on the host.  A sequence whose position lies outside its cache
    # row must leave caches and bit-cache untouched (it would otherwise land in a neighbouring head's row or beyond the
    # buffer); the sequences inside are written as usual.  Every kernel exits normally.
    print("\n[case] device-side positions beyond the cache", flush=True)
    w = small_workload(batch=4, seq_lens=[64] * 4, seed=31)
    p = make_problem(w)
    B, H, Hkv, Hc, d, cap = 4, w.n_q_heads, w.n_kv_heads, w.n_code_heads, 128, 40
    wk, wq = _ops.pack_usa_weights(p.usa.k, DEV), _ops.pack_usa_weights(p.usa.q, DEV)
    g = torch.Generator(device=DEV).manual_seed(2)
    qkv = torch.randn(B, (H + 2 * Hkv) * d, generator=g, device=DEV).to(torch.bfloat16)
    inv_freq = (1.0 / (500000.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV)
    pos = torch.tensor([7, cap, -3, 100000], dtype=torch.int32, device=DEV)       # inside, one past the end, negative, far out

    def buffers():
        kc = torch.full((B, Hkv, cap, d), 7.0, dtype=torch.bfloat16, device=DEV)
        return kc, kc.clone(), torch.full((B, Hc, cap, 1), 12345, dtype=torch.int32, device=DEV)
    k1, v1, c1 = buffers()
    q1 = torch.zeros(B, H, d, dtype=torch.bfloat16, device=DEV)
    qc1 = torch.zeros(B, H, 1, dtype=torch.int32, device=DEV)
    _ops.rope_encode_step(qkv, H, Hkv, 0, inv_freq, q1, k1, v1, wk, wq, 3, 128, 32, c1, qc1, pos_dev=pos)
    # the same launch for the first sequence alone, at its host-side position: what "written as usual" means
    k2, v2, c2 = buffers()
    q2 = torch.zeros(1, H, d, dtype=torch.bfloat16, device=DEV)
    qc2 = torch.zeros(1, H, 1, dtype=torch.int32, device=DEV)
    _ops.rope_encode_step(qkv[:1], H, Hkv, 7, inv_freq, q2, k2[:1], v2[:1], wk, wq, 3, 128, 32, c2[:1], qc2)
    torch.cuda.synchronize()
    assert torch.equal(k1[0], k2[0]) and torch.equal(v1[0], v2[0]) and torch.equal(c1[0], c2[0]) and torch.equal(qc1[0], qc2[0])
    assert (k1[1:] == 7.0).all() and (v1[1:] == 7.0).all() and (c1[1:] == 12345).all()
    # the two-launch form: ha_rope_append and ha_encode_step with the same positions
    k3, v3, c3 = buffers()
    q3 = torch.zeros(B, H, d, dtype=torch.bfloat16, device=DEV)
    qc3 = torch.zeros(B, H, 1, dtype=torch.int32, device=DEV)
    _ops.rope_append(qkv, H, Hkv, 0, inv_freq, q3, k3, v3, pos)
    knew = torch.randn(B, Hkv, 1, d, generator=g, device=DEV).to(torch.bfloat16)
    _ops.encode_step(knew, q3, wk, wq, 3, 128, 32, c3, qc3, pos_dev=pos)
    torch.cuda.synchronize()
    assert torch.equal(k3[0], k2[0]) and torch.equal(v3[0], v2[0]) and torch.equal(q3, q1)
    assert (k3[1:] == 7.0).all() and (v3[1:] == 7.0).all() and (c3[1:] == 12345).all()
    assert (c3[0, :, :7] == 12345).all() and (c3[0, :, 8:] == 12345).all() and (c3[0, :, 7] != 12345).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("layers,final,code_heads", [(3, 32, 8), (3, 64, 2), (2, 32, 2), (2, 64, 8), (1, 32, 2), (1, 64, 2)])
def test_fp32_mfma_bulk_encoder_against_the_oracle(layers, final, code_heads, dtype):
    # the fp32 matrix-core encoder is judged by the rule of the exact kernel: a sign bit may differ from the torch fp32
    # oracle only where the oracle's |logit| < 1e-4; against the exact kernel itself only a handful of bits may differ
    print(f"\n[case] fp32 mfma encoder layers={layers} final={final} Hc={code_heads} {dtype}", flush=True)
    from tests.parity_util import compare_codes
    w = small_workload(batch=2, seq_lens=[1900, 1333], lth_num_layers=layers, lth_final_dim=final, n_code_heads=code_heads,
                       dtype=dtype, seed=90 + layers + final)
    p = make_problem(w)
    B, Hc, S, W = w.batch, w.n_code_heads, w.max_seq_len, w.code_words
    k = p.k.to(DEV)
    wk = _ops.pack_usa_weights(p.usa.k, DEV)
    kl = orc.usa_logits(p.k.float(), p.usa.k)
    want = orc.pack_codes(kl).numpy().astype(np.uint32)
    c_mfma = torch.full((B, Hc, S + 7, W), -1, dtype=torch.int32, device=DEV)
    c_exact = torch.full((B, Hc, S + 7, W), -1, dtype=torch.int32, device=DEV)
    _ops.encode_pack_prefill_f32(k, wk, layers, w.lth_int_dim, final, c_mfma)
    _ops.encode_pack(k, wk, layers, w.lth_int_dim, final, c_exact)
    torch.cuda.synchronize()
    got = c_mfma.cpu().numpy().view(np.uint32)
    assert (got[:, :, S:] == 0xFFFFFFFF).all()                       # nothing written beyond the T rows
    n = compare_codes("fp32 mfma", got[:, :, :S], want, kl.numpy())
    d = _bits_differing(c_mfma[:, :, :S], c_exact[:, :, :S])
    print(f"  bits differing: vs oracle {n}, vs exact kernel {d} of {B * Hc * S * final}", flush=True)
    assert d <= 1e-5 * B * Hc * S * final + 2


def test_fp32_mfma_tail_and_offsets():
    # T not a multiple of the 256-token tile nor of 32; append at pos0 and at per-sequence offsets; strided rows
    print("\n[case] fp32 mfma tails/offsets", flush=True)
    w = small_workload(batch=2, seq_lens=[777, 777], seed=83)
    p = make_problem(w)
    k = p.k.to(DEV)
    wk = _ops.pack_usa_weights(p.usa.k, DEV)
    B, Hc, S = w.batch, w.n_code_heads, w.max_seq_len
    cap = S + 300
    outs = {}
    for enc in ("mfma", "exact"):
        f = _ops.encode_pack_prefill_f32 if enc == "mfma" else _ops.encode_pack
        full = torch.full((B, Hc, cap, 1), 12345, dtype=torch.int32, device=DEV)
        part = torch.full((B, Hc, cap, 1), 12345, dtype=torch.int32, device=DEV)
        pos = torch.tensor([100, 250], dtype=torch.int32, device=DEV)
        f(k, wk, 3, 128, 32, full, pos0=0)
        f(k[:, :, 5:600], wk, 3, 128, 32, part, pos_dev=pos)
        torch.cuda.synchronize()
        outs[enc] = (full.cpu(), part.cpu())
    full, part = outs["mfma"]
    assert (full[:, :, S:] == 12345).all()
    for b, p0 in enumerate((100, 250)):
        assert (part[b, :, :p0] == 12345).all() and (part[b, :, p0 + 595:] == 12345).all()
        assert _bits_differing(part[b, :, p0:p0 + 595], full[b, :, 5:600]) == 0
    assert _bits_differing(full[:, :, :S], outs["exact"][0][:, :, :S]) <= 2
    # a position from device memory that lies beyond the row writes nothing
    small = torch.full((B, Hc, 64, 1), 777, dtype=torch.int32, device=DEV)
    _ops.encode_pack_prefill_f32(k[:, :, :40], wk, 3, 128, 32, small, pos_dev=torch.tensor([30, 64], dtype=torch.int32, device=DEV))
    torch.cuda.synchronize()
    assert (small[1] == 777).all() and (small[0, :, :30] == 777).all() and (small[0, :, 30:] != 777).any()

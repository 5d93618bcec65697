"""The decoder-step harness (RMSNorm, fused QKV, rotate-half RoPE, in-place cache append, sparse attention,
SwiGLU, lm_head) against a `transformers` Llama of the same weights whose attention layers were converted with
`convert_usa`: both run the HIP attention, so this checks the plumbing around it.  fp32, tight tolerance."""
import pytest
import torch
from transformers import DynamicCache, LlamaConfig, LlamaForCausalLM, MistralConfig, MistralForCausalLM

from hashattention import _ops
from hashattention import hashattention_llama as hl
from hashattention import hashattention_mistral as hm
from hashattention.decoder import LlamaShapedDecoder
from hashattention.synthetic import UsaWeights

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _linears(seqs):
    return [[(m.weight.detach().float().cpu(), m.bias.detach().float().cpu()) for m in seq if isinstance(m, torch.nn.Linear)]
            for seq in seqs]


def test_decoder_step_matches_converted_llama():
    print("\n[case] decoder step vs converted Llama", flush=True)
    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                      head_dim=128, vocab_size=512, max_position_embeddings=4096, rope_theta=500000.0, rms_norm_eps=1e-5)
    usa_cfg = dict(lth_init_dim=128, lth_final_dim=32, lth_thold=0, lth_num_layers=3, init_budget=8, heavy_budget=0.125,
                   recent_budget=8, usa_retrieve_depth=6, usa_eval_mode="simple")
    for k, v in usa_cfg.items():
        setattr(cfg, k, v)
    model = LlamaForCausalLM(cfg).bfloat16().float()
    usa = hl.load_usa(cfg, None)
    model = hl.convert_usa(model.to(DEV), cfg, usa, collect_stats=False, train_usa=False).float()

    B, S0, steps = 2, 300, 3
    ids = torch.randint(0, cfg.vocab_size, (B, S0 + steps), generator=torch.Generator().manual_seed(1)).to(DEV)
    cache = DynamicCache()
    want = []
    with torch.no_grad():
        model(ids[:, :S0], past_key_values=cache, use_cache=True)        # q_len > 128: dense prefill
        keys = [cache.layers[l].keys.clone() for l in range(2)]
        values = [cache.layers[l].values.clone() for l in range(2)]
        for t in range(steps):
            want.append(model(ids[:, S0 + t:S0 + t + 1], past_key_values=cache, use_cache=True).logits[:, 0].float().cpu())

    dec = LlamaShapedDecoder(n_layers=2, hidden=512, ffn=1024, n_heads=4, n_kv_heads=2, head_dim=128, vocab=512,
                             rope_theta=500000.0, rms_eps=1e-5, n_code_heads=4, lth_num_layers=3, lth_int_dim=128,
                             lth_final_dim=32, init_budget=8, recent_budget=8, heavy_budget=0.125, dtype=torch.float32, device=DEV)
    dec.load_hf_llama(model)
    weights = [UsaWeights(k=_linears(u.learning_to_hash_transformation_k), q=_linears(u.learning_to_hash_transformation_q))
               for u in usa]
    dec.allocate(B, 512, weights)
    dec.load_cache(keys, values)
    with torch.no_grad():
        for t in range(steps):
            got = dec.decode_step(ids[:, S0 + t]).float().cpu()
            err = (got - want[t]).abs().max().item()
            print(f"step {t}: max-abs logit difference {err:.2e}", flush=True)
            assert err < 2e-3, err
    assert dec.seq_len == S0 + steps


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_rope_append_and_swiglu_against_torch(dtype):
    # the two plumbing kernels alone, against transformers' rotate-half formula and F.silu, host position and per-sequence positions
    print(f"\n[case] rope_append / swiglu {dtype}", flush=True)
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    from hashattention import _ops
    g = torch.Generator(device=DEV).manual_seed(5)
    B, H, Hkv, d, cap = 3, 8, 2, 128, 40
    qkv_full = torch.randn(B, (H + 2 * Hkv) * d + 64, generator=g, device=DEV).to(dtype)     # a row stride wider than the payload
    qkv = qkv_full[:, :(H + 2 * Hkv) * d]
    inv_freq = (1.0 / (500000.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV)
    for pos_dev in (None, torch.tensor([7, 0, 39], dtype=torch.int32, device=DEV)):
        k_cache = torch.zeros(B, Hkv, cap, d, dtype=dtype, device=DEV)
        v_cache = torch.zeros_like(k_cache)
        q_out = torch.empty(B, H, d, dtype=dtype, device=DEV)
        _ops.rope_append(qkv, H, Hkv, 11, inv_freq, q_out, k_cache, v_cache, pos_dev)
        pos = pos_dev.long() if pos_dev is not None else torch.full((B,), 11, device=DEV)
        ang = pos[:, None].float() * inv_freq[None, :]
        cos, sin = torch.cat([ang.cos(), ang.cos()], -1).to(dtype), torch.cat([ang.sin(), ang.sin()], -1).to(dtype)
        q = qkv[:, :H * d].view(B, H, 1, d).float()
        k = qkv[:, H * d:(H + Hkv) * d].view(B, Hkv, 1, d).float()
        qr, kr = apply_rotary_pos_emb(q, k, cos.float()[:, None, :], sin.float()[:, None, :])       # [B, 1, d] tables, fp32 math
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert (q_out.float() - qr[:, :, 0]).abs().max().item() <= tol
        want_k = torch.zeros_like(k_cache, dtype=torch.float32)
        want_v = torch.zeros_like(want_k)
        for b in range(B):
            want_k[b, :, pos[b]] = kr[b, :, 0]
            want_v[b, :, pos[b]] = qkv[b, (H + Hkv) * d:].view(Hkv, d).float()
        assert (k_cache.float() - want_k).abs().max().item() <= tol           # also: nothing written at any other position
        assert torch.equal(v_cache.float(), want_v)
    F_ = 1000
    gu = torch.randn(B, 2 * F_, generator=g, device=DEV).to(dtype)
    out = torch.empty(B, F_, dtype=dtype, device=DEV)
    _ops.swiglu(gu, out)
    want = torch.nn.functional.silu(gu[:, :F_]) * gu[:, F_:]
    assert (out.float() - want.float()).abs().max().item() <= (1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("M,N,K", [(4, 4096, 4096), (1, 1000, 512), (16, 6144, 4096), (4, 4096, 14336), (3, 20, 64), (4, 128256, 1024),
                                   (8, 4100, 4096), (5, 333, 8192), (7, 50, 14336), (2, 4096, 16416), (12, 77, 96),
                                   (4, 8192, 28672)])       # the last one: the down projection of a 70B model (rows too long for the row-streaming form)
def test_linear_skinny_against_fp32_matmul(M, N, K):
    # bf16 inputs, fp32 accumulation: against the fp32 product of the same bf16 values, one bf16 rounding of the result apart
    print(f"\n[case] linear_skinny {M}x{N}x{K}", flush=True)
    from hashattention import _ops
    g = torch.Generator(device=DEV).manual_seed(M * 7 + N)
    x = torch.randn(M, K, generator=g, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g, device=DEV) * K ** -0.5).to(torch.bfloat16)
    res = torch.randn(M, N, generator=g, device=DEV).to(torch.bfloat16)
    want = x.float() @ w.float().t()
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    _ops.linear_skinny(x, w, out)
    assert (out.float() - want).abs().max().item() <= 2e-2 * max(1.0, want.abs().max().item())
    assert torch.equal(out, want.to(torch.bfloat16)) or (out.float() - want.to(torch.bfloat16).float()).abs().max().item() <= 2 ** -6
    _ops.linear_skinny(x, w, out, residual=res)
    want2 = want + res.float()
    assert (out.float() - want2).abs().max().item() <= 2e-2 * max(1.0, want2.abs().max().item())
    # strided views (a slice of a wider buffer) for x and out
    xw = torch.zeros(M, K + 64, dtype=torch.bfloat16, device=DEV)
    xw[:, :K] = x
    ow = torch.zeros(M, N + 8, dtype=torch.bfloat16, device=DEV)
    _ops.linear_skinny(xw[:, :K], w, ow[:, :N])
    assert (ow[:, :N].float() - want).abs().max().item() <= 2e-2 * max(1.0, want.abs().max().item()) and (ow[:, N:] == 0).all()


def test_bf16_decoder_step_with_and_without_the_skinny_projections():
    # the bf16 step routes three projections through ha_linear_skinny; with the library GEMMs instead the logits agree to bf16 noise
    print("\n[case] bf16 decoder step, skinny projections on/off", flush=True)
    dec = LlamaShapedDecoder(n_layers=2, hidden=512, ffn=1024, n_heads=4, n_kv_heads=2, head_dim=128, vocab=512, n_code_heads=2,
                             init_budget=8, recent_budget=8, heavy_budget=0.125, dtype=torch.bfloat16, device=DEV, seed=3)
    dec.allocate(2, 400)
    dec.fill_cache_synthetic(300)
    tokens = torch.tensor([5, 17], device=DEV)
    with torch.no_grad():
        a = dec.decode_step(tokens, advance=False).float()
        dec.fuse_rope = False                       # ha_rope_append + ha_encode_step instead of the one launch: the same bits
        assert torch.equal(dec.decode_step(tokens, advance=False).float(), a)
        dec.fuse_rope = True
        dec.skinny_all = False                      # library GEMMs for the down projection and the lm_head
        c = dec.decode_step(tokens, advance=False).float()
        dec.use_skinny = False
        b = dec.decode_step(tokens, advance=False).float()
    assert torch.isfinite(a).all()
    assert (a - b).abs().max().item() <= 0.05 * max(1.0, b.abs().max().item())
    assert (c - b).abs().max().item() <= 0.05 * max(1.0, b.abs().max().item())


def test_bf16_decoder_step_of_a_dozen_sequences_on_tiled_weights():
    # 9 to 16 sequences: QKV, output and gate/up projections on the matrix cores from tiled copies of the weights (residual and
    # SwiGLU inside), RMSNorm as one launch; against the same step through the library's GEMMs, and through graph replay
    print("\n[case] bf16 decoder step, 12 sequences, tiled projections on/off", flush=True)
    dec = LlamaShapedDecoder(n_layers=2, hidden=512, ffn=1024, n_heads=4, n_kv_heads=2, head_dim=128, vocab=512, n_code_heads=2,
                             init_budget=8, recent_budget=8, heavy_budget=0.125, dtype=torch.bfloat16, device=DEV, seed=5)
    dec.allocate(12, 400)
    dec.fill_cache_synthetic(300)
    assert dec._tiled() and "w13_t" in dec.layers[0]
    tokens = torch.arange(12, device=DEV) * 7 + 3
    with torch.no_grad():
        a = dec.decode_step(tokens, advance=False).float()
        dec.use_skinny = False
        assert not dec._tiled()
        b = dec.decode_step(tokens, advance=False).float()
        dec.use_skinny = True
        got = dec.generate(tokens, 5)
        dec.seq_len -= 5
        for hl in dec.hash:
            hl.n_cached -= 5
        want = dec.generate(tokens, 5, use_graph=False)
    assert torch.isfinite(a).all()
    assert (a - b).abs().max().item() <= 0.05 * max(1.0, b.abs().max().item())
    assert torch.equal(got, want)


def test_decoder_step_on_the_fused_attention_path_matches_the_two_launch_path():
    # 32 (sequence, head) rows: every layer takes ha_select_histogram + ha_sparse_decode_fused; the same step through
    # ha_select + ha_sparse_decode must agree to bf16 noise, and the index lists the fused path never writes stay usable
    print("\n[case] bf16 decoder step, fused attention path on/off", flush=True)
    dec = LlamaShapedDecoder(n_layers=2, hidden=512, ffn=1024, n_heads=8, n_kv_heads=2, head_dim=128, vocab=512, n_code_heads=2,
                             init_budget=8, recent_budget=8, heavy_budget=0.125, dtype=torch.bfloat16, device=DEV, seed=4)
    dec.allocate(4, 3000)
    dec.fill_cache_synthetic(2500)
    assert all(hl.fused_ok for hl in dec.hash)
    tokens = torch.tensor([5, 17, 40, 3], device=DEV)
    with torch.no_grad():
        a = dec.decode_step(tokens, advance=False).float()
        hl0 = dec.hash[0]
        out = torch.empty(4, 8, 128, dtype=torch.bfloat16, device=DEV)
        hl0.attend(dec.q_rot, dec.k_cache[0], dec.v_cache[0], out)          # lists never selected: zero-filled, in bounds
        for hl in dec.hash:
            hl.use_fused = False
        b = dec.decode_step(tokens, advance=False).float()
    torch.cuda.synchronize()
    assert torch.isfinite(a).all()
    assert (a - b).abs().max().item() <= 0.05 * max(1.0, b.abs().max().item())


@pytest.mark.parametrize("M,N,K", [(4, 6144, 4096), (1, 512, 1024), (8, 1000, 4096), (3, 96, 8192), (4, 200, 16384), (5, 64, 64),
                                   (4, 10240, 8192), (2, 9000, 4096)])      # the last two: row counts chosen for whole rounds
def test_linear_skinny_with_rmsnorm_in_front(M, N, K):
    # against the RMSNorm module of transformers (and of the reference's harness, efficiency/model.py:314-319: the normalised
    # row is rounded to the input type, then multiplied by the weight and rounded again), followed by the fp32 product
    print(f"\n[case] linear_skinny + RMSNorm {M}x{N}x{K}", flush=True)
    from transformers.models.llama.modeling_llama import LlamaRMSNorm
    from hashattention import _ops
    g = torch.Generator(device=DEV).manual_seed(M + N + K)
    x = (torch.randn(M, K, generator=g, device=DEV) * 3).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g, device=DEV) * K ** -0.5).to(torch.bfloat16)
    gamma = (1 + 0.2 * torch.randn(K, generator=g, device=DEV)).to(torch.bfloat16)
    res = torch.randn(M, N, generator=g, device=DEV).to(torch.bfloat16)
    norm = LlamaRMSNorm(K, eps=1e-5).to(DEV, torch.bfloat16)
    with torch.no_grad():
        norm.weight.copy_(gamma)
        h = norm(x)
    want = h.float() @ w.float().t()
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    _ops.linear_skinny(x, w, out, norm_weight=gamma, eps=1e-5)
    assert (out.float() - want).abs().max().item() <= 2e-2 * max(1.0, want.abs().max().item())
    _ops.linear_skinny(x, w, out, residual=res, norm_weight=gamma, eps=1e-5)
    want2 = want + res.float()
    assert (out.float() - want2).abs().max().item() <= 2e-2 * max(1.0, want2.abs().max().item())
    # the normalised rows themselves: an identity weight returns them
    if K <= 1024:
        eye = torch.eye(K, dtype=torch.bfloat16, device=DEV)
        hn = torch.empty(M, K, dtype=torch.bfloat16, device=DEV)
        _ops.linear_skinny(x, eye, hn, norm_weight=gamma, eps=1e-5)
        assert (hn.float() - h.float()).abs().max().item() <= 2 ** -6 * max(1.0, h.float().abs().max().item())
        # the same two roundings: equal bit for bit, but for an element whose first rounding sits on a tie that the last
        # digit of the row's mean square (summed in another order) decides
        assert (hn != h).float().mean().item() <= 1e-3, (hn != h).float().mean().item()


@pytest.mark.parametrize("M,F,K", [(4, 14336, 4096), (1, 100, 512), (8, 777, 4096), (2, 48, 8192), (4, 40, 64), (4, 28672, 8192)])
def test_linear_skinny_with_swiglu_behind(M, F, K):
    # against the unfused pair: ha_linear_skinny into a bf16 gate/up buffer, then ha_swiglu - same roundings, same sums
    print(f"\n[case] linear_skinny + SwiGLU {M}x{F}x{K}", flush=True)
    from hashattention import _ops
    g = torch.Generator(device=DEV).manual_seed(M + F + K)
    x = torch.randn(M, K, generator=g, device=DEV).to(torch.bfloat16)
    w = (torch.randn(2 * F, K, generator=g, device=DEV) * K ** -0.5).to(torch.bfloat16)
    gamma = (1 + 0.2 * torch.randn(K, generator=g, device=DEV)).to(torch.bfloat16)
    for norm in (None, gamma):
        gu = torch.empty(M, 2 * F, dtype=torch.bfloat16, device=DEV)
        _ops.linear_skinny(x, w, gu, norm_weight=norm, eps=1e-5)
        want = torch.empty(M, F, dtype=torch.bfloat16, device=DEV)
        _ops.swiglu(gu, want)
        out = torch.full((M, F + 8), 7.0, dtype=torch.bfloat16, device=DEV)
        _ops.linear_skinny(x, w, out[:, :F], norm_weight=norm, eps=1e-5, swiglu=True)
        assert (out[:, F:] == 7.0).all()
        # the two kernels group the rows of W differently, so a sum can differ in its last bf16 digit
        ref = torch.nn.functional.silu(gu[:, :F].float()) * gu[:, F:].float()
        assert (out[:, :F].float() - ref).abs().max().item() <= 2e-2 * max(1.0, ref.abs().max().item())
        assert (out[:, :F].float() - want.float()).abs().max().item() <= 2 ** -6 * max(1.0, want.float().abs().max().item())


@pytest.mark.parametrize("dtype,B", [(torch.float32, 5), (torch.bfloat16, 5), (torch.float16, 5), (torch.bfloat16, 40), (torch.float32, 100)])
@pytest.mark.parametrize("code_heads", ["kv", "q"])
def test_rope_encode_step_equals_rope_append_then_encode_step(dtype, B, code_heads):
    # one launch against the two it replaces: rotated query, both caches and both code buffers bit for bit.  5, 40 and 100
    # sequences: one, two and four rows per workgroup of the encode launch
    print(f"\n[case] rope_encode_step {dtype} B={B} code heads per {code_heads} head", flush=True)
    from hashattention import _ops
    from hashattention.synthetic import layer_dims
    g = torch.Generator(device=DEV).manual_seed(11)
    gc = torch.Generator().manual_seed(12)
    H, Hkv, d, cap = 8, 2, 128, 50
    Hc = Hkv if code_heads == "kv" else H
    heads = lambda n: [[(torch.randn(fo, fi, generator=gc) * fi ** -0.5, torch.randn(fo, generator=gc) * 0.01)
                        for fi, fo in layer_dims(d, 128, 32, 3)] for _ in range(n)]
    wk, wq = _ops.pack_usa_weights(heads(Hc), DEV), _ops.pack_usa_weights(heads(H), DEV)
    qkv = torch.randn(B, (H + 2 * Hkv) * d + 32, generator=g, device=DEV).to(dtype)[:, :(H + 2 * Hkv) * d]
    inv_freq = (1.0 / (500000.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV)
    some = torch.tensor([3, 49, 0, 21, 8] + [int(x) for x in torch.randint(0, cap, (B - 5,), generator=gc)], dtype=torch.int32, device=DEV)
    for pos, pos_dev in ((17, None), (0, some)):
        outs = []
        for fused in (False, True):
            k_cache = torch.zeros(B, Hkv, cap, d, dtype=dtype, device=DEV)
            v_cache = torch.zeros_like(k_cache)
            q_out = torch.zeros(B, H, d, dtype=dtype, device=DEV)
            kcodes = torch.zeros(B, Hc, cap, 1, dtype=torch.int32, device=DEV)
            qcodes = torch.zeros(B, H, 1, dtype=torch.int32, device=DEV)
            if fused:
                _ops.rope_encode_step(qkv, H, Hkv, pos, inv_freq, q_out, k_cache, v_cache, wk, wq, 3, 128, 32, kcodes, qcodes, pos_dev)
            else:
                _ops.rope_append(qkv, H, Hkv, pos, inv_freq, q_out, k_cache, v_cache, pos_dev)
                p = pos_dev.long() if pos_dev is not None else torch.full((B,), pos, device=DEV)
                k_new = torch.gather(k_cache, 2, p.view(B, 1, 1, 1).expand(B, Hkv, 1, d))
                _ops.encode_step(k_new, q_out, wk, wq, 3, 128, 32, kcodes, qcodes, pos0=pos, pos_dev=pos_dev)
            outs.append((q_out, k_cache, v_cache, kcodes, qcodes))
        for a, b in zip(*outs):
            assert torch.equal(a, b)
        assert outs[1][3].ne(0).any() and outs[1][1].ne(0).any()


@pytest.mark.parametrize("n_heads,batch", [(8, 4), (4, 2)])
def test_generate_replays_one_graph_for_successive_tokens(n_heads, batch):
    # positions on the device: one captured graph serves every token.  Against the same steps launched one by one with the
    # position on the host (8 heads x 4 sequences: the fused attention launch; 4 x 2: the list-fed launches)
    print(f"\n[case] decoder generate, graph replay per token, H={n_heads} B={batch}", flush=True)
    mk = lambda: LlamaShapedDecoder(n_layers=2, hidden=512, ffn=1024, n_heads=n_heads, n_kv_heads=2, head_dim=128, vocab=512,
                                    n_code_heads=2, init_budget=8, recent_budget=8, heavy_budget=0.125, dtype=torch.bfloat16,
                                    device=DEV, seed=6)
    n_new, ctx = 12, 1500
    first = torch.arange(3, 3 + batch, device=DEV)
    decs = [mk() for _ in range(3)]
    for dec in decs:
        dec.allocate(batch, 2000)
        dec.fill_cache_synthetic(ctx, seed=1)
    assert all(hl.fused_ok for hl in decs[0].hash) == (n_heads * batch >= 32)
    with torch.no_grad():
        host, tok = [], first
        first_logits = None
        for _ in range(n_new):
            logits = decs[0].decode_step(tok)
            first_logits = logits.float().clone() if first_logits is None else first_logits
            tok = logits.argmax(-1)
            host.append(tok)
        host = torch.stack(host, dim=1)
        graph = decs[1].generate(first, n_new, use_graph=True)
        eager = decs[2].generate(first, n_new, use_graph=False)
    torch.cuda.synchronize()
    assert graph.shape == (batch, n_new) and decs[1].seq_len == ctx + n_new and decs[1].hash[0].n_cached == ctx + n_new
    assert torch.equal(graph, eager)                       # the replayed graph and the same launches made eagerly: the same bits
    for l in range(2):                                     # the caches and the bit-caches grew identically
        assert torch.equal(decs[1].k_cache[l], decs[2].k_cache[l]) and torch.equal(decs[1].hash[l].codes, decs[2].hash[l].codes)
    # positions on the host: the rows are cut into other pieces, so the attention output may differ in its last bit
    same = (graph == host).float().mean().item()
    print(f"  tokens equal to the host-position loop: {same:.3f}", flush=True)
    assert torch.equal(graph[:, 0], host[:, 0]) and same >= 0.9
    assert torch.equal(decs[0].k_cache[0][:, :, :ctx + 1], decs[1].k_cache[0][:, :, :ctx + 1])
    with pytest.raises(ValueError):
        decs[1].generate(first, 2000)
    # a sampler in place of the arg-max: the reference's `sample` (arg-max of the probabilities) gives the greedy tokens again;
    # a top-k sampler with its own generator runs through the same captured graph
    more = decs[1].generate(graph[:, -1], 4)
    with torch.no_grad():
        again = decs[2].generate(eager[:, -1], 4, use_graph=False, sampler=lambda lg: torch.softmax(lg.float(), -1).argmax(-1))
    assert torch.equal(more, again)
    g = torch.Generator(device=DEV).manual_seed(0)

    def top_k(lg, k=5):
        v, i = torch.topk(lg.float(), k, dim=-1)
        return i.gather(-1, torch.multinomial(torch.softmax(v, -1), 1, generator=g))[:, 0]

    sampled = decs[1].generate(more[:, -1], 6, sampler=top_k)
    assert sampled.shape == (batch, 6) and int(sampled.min()) >= 0 and int(sampled.max()) < 512


@pytest.mark.parametrize("family", ["llama", "mistral", "llama3_rope"])
def test_decoder_from_hf_prefill_and_generate_match_the_patched_model(family):
    # the serving path end to end: a transformers Llama (or Mistral: the same decoder shape) + hash modules ->
    # LlamaShapedDecoder.from_hf, prefill by the model itself, greedy generation by graph replay; against `generate` of the
    # same model patched with convert_usa
    print(f"\n[case] decoder from_hf + prefill_from_hf + generate vs patched model.generate, {family}", flush=True)
    torch.manual_seed(2)
    shape = dict(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                 head_dim=128, vocab_size=512, max_position_embeddings=4096, rope_theta=500000.0, rms_norm_eps=1e-5)
    if family == "llama":
        cfg, LlamaForCausalLM, hl = LlamaConfig(**shape), globals()["LlamaForCausalLM"], globals()["hl"]
    elif family == "llama3_rope":   # Llama-3.1's frequency scaling: the decoder takes the model's own (scaled) frequencies
        del shape["rope_theta"]
        cfg = LlamaConfig(rope_parameters=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                               original_max_position_embeddings=64, rope_theta=500000.0), **shape)
        LlamaForCausalLM, hl = globals()["LlamaForCausalLM"], globals()["hl"]
    else:
        cfg, LlamaForCausalLM, hl = MistralConfig(sliding_window=None, **shape), MistralForCausalLM, hm
    for k, v in dict(lth_init_dim=128, lth_final_dim=32, lth_thold=0, lth_num_layers=3, init_budget=8, heavy_budget=0.125,
                     recent_budget=8, usa_retrieve_depth=6, usa_eval_mode="simple").items():
        setattr(cfg, k, v)
    model = LlamaForCausalLM(cfg).bfloat16().float()
    if family == "llama3_rope":
        assert model.model.rotary_emb.rope_type == "llama3"
    usa = hl.load_usa(cfg, None)
    model = hl.convert_usa(model.to(DEV), cfg, usa, collect_stats=False, train_usa=False).float()
    B, S0, n_new = 2, 200, 8
    ids = torch.randint(1, cfg.vocab_size, (B, S0), generator=torch.Generator().manual_seed(5)).to(DEV)
    with torch.no_grad():
        want = model.generate(input_ids=ids, max_new_tokens=n_new, do_sample=False, use_cache=True, pad_token_id=0)[:, S0:].cpu()
    hl.reset_usa(model)
    dec = LlamaShapedDecoder.from_hf(model, usa, batch=B, cache_len=256, dtype=torch.float32, device=DEV)
    assert dec.Hc == 4 and dec.budgets == (8, 8, 0.125) and dec.embed.shape == (512, 512)
    with torch.no_grad():
        first = dec.prefill_from_hf(model, ids)
        rest = dec.generate(first, n_new - 1)
    got = torch.cat([first[:, None], rest], dim=1).cpu()
    print("  tokens:", got.tolist(), flush=True)
    assert torch.equal(got, want)
    assert dec.seq_len == S0 + n_new - 1


@pytest.mark.parametrize("M,N,K,form", [(16, 6144, 4096, "plain"), (12, 4096, 4096, "residual"), (16, 2 * 14336, 4096, "glu"),
                                        (9, 1000, 64, "plain"), (1, 40, 32, "residual"), (16, 2 * 100, 1536, "glu"),
                                        (13, 4096, 8192, "residual"), (4, 520, 2080, "plain"),
                                        (32, 6144, 4096, "plain"), (17, 4096, 4096, "residual"), (24, 2 * 14336, 4096, "glu"),
                                        (29, 300, 96, "residual"), (20, 2 * 72, 2048, "glu"),
                                        (16, 4096, 14336, "residual"), (10, 100, 8224, "plain"), (3, 4096, 28672, "residual")])
def test_linear_tiled_against_fp32_matmul(M, N, K, form):
    # the matrix-core projection on a tiled copy of the weights (ha_pack_weight_tiles, ha_linear_tiled) against the product in fp32
    # with the roundings of the modules it stands for: the projection's output rounded to bf16 before a residual is added;
    # SwiGLU on rounded gate and up values.  Shapes: whole and ragged tile rows, one to thirty-two rows of x, K from one k-step to
    # the 8192 inputs a workgroup holds and beyond (x requested next to the tiles), a K that leaves waves without work
    print(f"\n[case] ha_linear_tiled M={M} N={N} K={K} {form}", flush=True)
    g = torch.Generator(device=DEV).manual_seed(N + K + M)
    x = torch.randn(M, K, generator=g, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g, device=DEV) * K ** -0.5).to(torch.bfloat16)
    tiles = _ops.pack_weight_tiles(w, glu=form == "glu")
    y = x.float() @ w.float().t()
    if form == "glu":
        gate, up = y[:, :N // 2].bfloat16().float(), y[:, N // 2:].bfloat16().float()
        want = torch.nn.functional.silu(gate).bfloat16().float() * up
        out = torch.full((M, N // 2), 7.0, dtype=torch.bfloat16, device=DEV)
        _ops.linear_tiled(x, tiles, N, out, swiglu=True)
    elif form == "residual":
        res = torch.randn(M, N, generator=g, device=DEV).to(torch.bfloat16)
        want = y.bfloat16().float() + res.float()
        out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
        _ops.linear_tiled(x, tiles, N, out, residual=res)
    else:
        want = y
        out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
        _ops.linear_tiled(x, tiles, N, out)
    torch.cuda.synchronize()
    # bf16 output: half a unit in the last place of the largest value, plus a rounding of gate / up / product that may fall the other way
    tol = 2.0 ** -8 * max(1.0, want.abs().max().item()) * (3 if form != "plain" else 1)
    err = (out.float() - want).abs().max().item()
    assert err <= tol, (err, tol)
    # the same rows with a stride of their own, written into a wider buffer
    xs = torch.zeros(M, K + 64, dtype=torch.bfloat16, device=DEV)[:, :K]
    xs.copy_(x)
    wide = torch.full((M, out.shape[1] + 24), 7.0, dtype=torch.bfloat16, device=DEV)
    if form == "glu":
        _ops.linear_tiled(xs, tiles, N, wide[:, :out.shape[1]], swiglu=True)
    elif form == "residual":
        _ops.linear_tiled(xs, tiles, N, wide[:, :out.shape[1]], residual=res)
    else:
        _ops.linear_tiled(xs, tiles, N, wide[:, :out.shape[1]])
    torch.cuda.synchronize()
    assert torch.equal(wide[:, :out.shape[1]], out) and bool((wide[:, out.shape[1]:] == 7.0).all())


@pytest.mark.parametrize("dtype,M,K", [(torch.bfloat16, 12, 4096), (torch.bfloat16, 3, 5120), (torch.float16, 5, 1024),
                                       (torch.float32, 4, 768), (torch.bfloat16, 2, 100), (torch.bfloat16, 2, 14336)])
def test_rmsnorm_launch_rounds_as_the_module_it_replaces(dtype, M, K):
    # ha_rmsnorm against transformers' LlamaRMSNorm in the same dtype: the normalised row rounded to the element type, then the
    # product with the weight rounded again.  The sum of squares is added in another order, so a rounding may fall the other way
    # for a few elements: one unit in the last place at most, in fewer than one element of a thousand.
    from transformers.models.llama.modeling_llama import LlamaRMSNorm
    print(f"\n[case] ha_rmsnorm {dtype} {M}x{K}", flush=True)
    g = torch.Generator(device=DEV).manual_seed(K + M)
    x = (torch.randn(M, K, generator=g, device=DEV) * 3).to(dtype)
    mod = LlamaRMSNorm(K, eps=1e-5).to(DEV, dtype)
    mod.weight.data = (1 + 0.3 * torch.randn(K, generator=g, device=DEV)).to(dtype)
    want = mod(x)
    xs = torch.empty(M, K + 8, dtype=dtype, device=DEV)[:, :K]      # rows with a stride of their own
    xs.copy_(x)
    for src in (x, xs):
        out = torch.full((M, K), 7.0, dtype=dtype, device=DEV)
        _ops.rmsnorm(src, mod.weight, 1e-5, out)
        torch.cuda.synchronize()
        if dtype == torch.float32:
            assert (out - want).abs().max().item() <= 1e-5 * want.abs().max().item()
            continue
        differ = out != want
        assert differ.float().mean().item() <= 1e-3, differ.float().mean().item()
        ulp = (out.view(torch.int16).int() - want.view(torch.int16).int()).abs()
        assert int(ulp.max()) <= 1


@pytest.mark.parametrize("what", ["attention_bias", "mlp_bias", "yarn", "dynamic"])
def test_decoder_from_hf_refuses_what_its_launches_do_not_express(what):
    print(f"\n[case] decoder from_hf refuses {what}", flush=True)
    shape = dict(hidden_size=512, intermediate_size=1024, num_hidden_layers=1, num_attention_heads=4, num_key_value_heads=2,
                 head_dim=128, vocab_size=512, max_position_embeddings=4096)
    if what == "yarn":
        shape["rope_parameters"] = dict(rope_type="yarn", factor=4.0, original_max_position_embeddings=1024, rope_theta=10000.0)
    elif what == "dynamic":
        shape["rope_parameters"] = dict(rope_type="dynamic", factor=2.0, rope_theta=10000.0)
    else:
        shape[what] = True
    cfg = LlamaConfig(**shape)
    for k, v in dict(lth_init_dim=128, lth_final_dim=32, lth_thold=0, lth_num_layers=3, init_budget=8, heavy_budget=0.125,
                     recent_budget=8, usa_retrieve_depth=6, usa_eval_mode="simple").items():
        setattr(cfg, k, v)
    model = LlamaForCausalLM(cfg).bfloat16().to(DEV)
    with pytest.raises(NotImplementedError):
        LlamaShapedDecoder.from_hf(model, hl.load_usa(cfg, None), batch=1, cache_len=64, dtype=torch.float32, device=DEV)
    # the patched model takes all of these: biases through the modules, the rotary embedding through the model's own cos/sin
    model = hl.convert_usa(model, cfg, hl.load_usa(cfg, None), collect_stats=False, train_usa=False)
    ids = torch.randint(1, 512, (2, 150), generator=torch.Generator().manual_seed(6)).to(DEV)
    out = model.generate(ids, max_new_tokens=4, do_sample=False, pad_token_id=0)
    assert out.shape == (2, 154)


def test_ragged_prompts_through_the_decoder_generation_loop():
    # prompts of different lengths, right-padded: every sequence continues at its own length (positions and lengths on the
    # device).  Against the same prompts run one by one, unpadded.
    print("\n[case] decoder generate, ragged prompts", flush=True)
    torch.manual_seed(4)
    cfg = LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                      head_dim=128, vocab_size=512, max_position_embeddings=4096, rope_theta=500000.0, rms_norm_eps=1e-5)
    for k, v in dict(lth_init_dim=128, lth_final_dim=32, lth_thold=0, lth_num_layers=3, init_budget=8, heavy_budget=0.125,
                     recent_budget=8, usa_retrieve_depth=6, usa_eval_mode="simple").items():
        setattr(cfg, k, v)
    model = LlamaForCausalLM(cfg).float().to(DEV)
    usa = hl.load_usa(cfg, None).float()
    lens, S0, n_new = [200, 141, 173], 200, 6
    ids = torch.randint(1, cfg.vocab_size, (3, S0), generator=torch.Generator().manual_seed(6)).to(DEV)
    am = (torch.arange(S0)[None, :] < torch.tensor(lens)[:, None]).long().to(DEV)
    dec = LlamaShapedDecoder.from_hf(model, usa, batch=3, cache_len=256, dtype=torch.float32, device=DEV)
    with torch.no_grad():
        first = dec.prefill_from_hf(model, ids, am)
        assert dec.lengths == lens and dec.seq_len == 200
        with pytest.raises(RuntimeError):
            dec.decode_step(first)
        rest = dec.generate(first, n_new)
    got = torch.cat([first[:, None], rest], dim=1).cpu()
    assert dec.lengths == [n + n_new for n in lens]
    one = LlamaShapedDecoder.from_hf(model, usa, batch=1, cache_len=256, dtype=torch.float32, device=DEV)
    for b, n in enumerate(lens):
        with torch.no_grad():
            f = one.prefill_from_hf(model, ids[b:b + 1, :n])
            r = one.generate(f, n_new)
        want = torch.cat([f[:, None], r], dim=1).cpu()[0]
        print(f"  sequence {b} ({n} tokens): {got[b].tolist()}", flush=True)
        assert torch.equal(got[b], want), (b, got[b], want)
    with pytest.raises(ValueError):
        dec.prefill_from_hf(model, ids, torch.flip(am, dims=[1]))            # left padding is not a ragged batch


def test_full_width_decoder_step_at_131072_tokens():
    # The shape the decode throughput is quoted on, two layers deep: hidden 4096, ffn 14336, 32 query / 8 KV heads, four
    # sequences with 131071 cached tokens each, bf16.  (1) the step on the fused select-attend launch against the same step
    # on ha_select + ha_sparse_decode; (2) the last layer's attention output against the double-precision oracle on the index
    # lists the oracle's own selection makes from that layer's codes.
    import math
    import numpy as np
    from oracle import c_oracle
    print("\n[case] full-width decoder step, B=4, context 131072", flush=True)
    B, S = 4, 131072
    dec = LlamaShapedDecoder(n_layers=2, hidden=4096, ffn=14336, n_heads=32, n_kv_heads=8, head_dim=128, vocab=32000, n_code_heads=8,
                             init_budget=128, recent_budget=128, heavy_budget=1.0 / 32, dtype=torch.bfloat16, device=DEV, seed=11)
    dec.allocate(B, S)
    dec.fill_cache_synthetic(S - 1)
    tokens = torch.tensor([3, 1415, 9265, 31999], device=DEV)
    assert all(h.use_fused and h.fused_ok for h in dec.hash)
    last = dec.hash[-1]

    def snapshot():
        # what the last layer's attention launch read and wrote in the step just made (the new token's row included)
        return dict(q=dec.q_rot.cpu(), out=dec.attn_out.float().cpu().numpy(),
                    kc=last.codes[:, :, :S].cpu().numpy().view(np.uint32), qc=last.qcodes.view(B, 32, 1).cpu().numpy().view(np.uint32),
                    k_new=dec.k_cache[-1][:, :, S - 1].cpu(), v_new=dec.v_cache[-1][:, :, S - 1].cpu())

    with torch.no_grad():
        fused = dec.decode_step(tokens, advance=False).float().clone()
        snap_fused = snapshot()
        for h in dec.hash:
            h.use_fused = False
        lists = dec.decode_step(tokens, advance=False).float()
        snap_lists = snapshot()
    assert torch.isfinite(fused).all()
    scale = max(1.0, fused.abs().max().item())
    err = (fused - lists).abs().max().item()
    print(f"  logits: fused launch vs index lists in memory, max-abs {err:.2e} (largest logit {scale:.2f})", flush=True)
    assert err <= 3e-2 * scale, err
    seq = np.full(B, S, dtype=np.int32)
    cap = 128 + 128 + S // 32
    k_cpu, v_cpu = dec.k_cache[-1][:, :, :S].cpu(), dec.v_cache[-1][:, :, :S].cpu()
    for name, snap in (("fused launch", snap_fused), ("lists in memory", snap_lists)):
        # the layer's input differs by bf16 noise between the two steps (the first layer's attention adds its rows in another
        # order), so each step is checked against the oracle on ITS query, codes and new row
        k_cpu[:, :, S - 1], v_cpu[:, :, S - 1] = snap["k_new"], snap["v_new"]
        ref_idx, ref_cnt = c_oracle.select(snap["kc"], snap["qc"], seq, 128, 128, 1.0 / 32, cap)
        assert (ref_cnt == cap).all()
        if name == "lists in memory":
            assert np.array_equal(last.counts.cpu().numpy(), ref_cnt) and np.array_equal(last.idx.cpu().numpy()[:, :, :cap], ref_idx)
        ref = c_oracle.sparse_attend(snap["q"], k_cpu, v_cpu, ref_idx, ref_cnt, 1 / math.sqrt(128))
        aerr = np.abs(snap["out"] - ref).max()
        print(f"  last layer's attention output ({name}) vs the oracle: max-abs {aerr:.2e}", flush=True)
        assert aerr <= 2e-2

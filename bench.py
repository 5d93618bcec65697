#!/usr/bin/env python3
"""Benchmark of the HashAttention sparse decode step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config config2]

A step is one pass of the hot path over one batch of synthetic input for a single attention layer:
hash-encode of the new key and the query, Hamming select over the bit-cache, gather-only attention.
The workload is the configuration the metric is quoted on (config2: Llama-3.1-8B attention shape,
batch 16, 64K context, 32x sparse); K/V and the bit-cache are resident in HBM before timing starts.
Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (os.path.join(ROOT, "hashattention-1.0_amd"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBPS = 8000.0   # MI355X HBM3E, published peak

TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "decode_step_config2_hbm_traffic.md")


def measured_traffic(workload_name, fused, code_heads):
    """HBM bytes per launch of the step's attention kernel as the two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE, each
    scaled on a 1 GiB copy) measured them: read from the tracked summary, which names the commit it was measured at in
    lines of the form `traffic_bytes[config2, fused, code_heads=8] = 588.6e6 (commit abc1234)`.  None when the summary
    has no line for this workload."""
    import re
    try:
        text = open(TRAFFIC_SUMMARY).read()
    except OSError:
        return None
    key = re.escape(f"traffic_bytes[{workload_name}, {'fused' if fused else 'lists'}, code_heads={code_heads}]")
    m = re.search(key + r"\s*=\s*([0-9.eE+]+)\s*\(commit ([0-9a-f]{7,40})\)", text)
    return {"bytes": float(m.group(1)), "commit": m.group(2)} if m else None


def algorithmic_bytes(w, n_sel_rows):
    """Algorithmic HBM bytes of one layer-step, per stage.  n_sel_rows = sum over (b, h) of selected tokens."""
    d, H, B = w.head_dim, w.n_q_heads, w.batch
    eb = 2 if str(w.dtype) != "torch.float32" else 4
    tokens = sum(w.seq_lens)
    score = w.n_code_heads * tokens * 4 * w.code_words                  # every cached code read once
    select = n_sel_rows * 4                                             # index lists written
    gather = n_sel_rows * (2 * d * eb) + n_sel_rows * 4 + B * H * d * eb * 2   # K+V rows, index read, q read + out write
    dense = w.n_kv_heads * tokens * 2 * d * eb
    return dict(score=score, select=select, gather=gather, dense=dense)


def time_gpu(fn, steps, warmup, torch):
    """Average ms per call over `steps` back-to-back calls, HIP events on the stream the kernels run on."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def time_rotating(fns, steps, warmup, torch):
    """`time_gpu` over a rotation: call i runs fns[i % len(fns)], so consecutive launches work on different inputs."""
    it = [0]

    def fn():
        fns[it[0] % len(fns)]()
        it[0] += 1
    return time_gpu(fn, steps, warmup, torch)


def capture_graph(fn, torch):
    """fn() captured in a HIP graph (after one eager pass on a side stream, as capture wants it)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g


def cpu_baseline(w, torch, budget_s=12.0):
    """The oracle's restatement of the reference decode step (dense QK^T, every key re-hashed, full sort, masked
    fp32 softmax) timed on the host, one sequence of the workload at a time until `budget_s` seconds are spent,
    then scaled linearly to the batch."""
    from hashattention.synthetic import Workload, make_problem
    from oracle import hashattn_oracle as orc
    times = []
    t_start = time.perf_counter()
    for b in range(w.batch):
        w1 = Workload(**{**w.__dict__, "name": w.name + "-cpu", "batch": 1, "seq_lens": [w.seq_lens[b]], "seed": w.seed + b})
        p = make_problem(w1)
        q, k, v = p.q.float(), p.k.float(), p.v.float()
        if b == 0:     # warm-up on a prefix (thread pools, allocator)
            orc.reference_decode_attention(q, k[:, :, :4096], v[:, :, :4096], p.usa.k, p.usa.q, w.init_budget,
                                           w.recent_budget, w.heavy_budget)
        t0 = time.perf_counter()
        orc.reference_decode_attention(q, k, v, p.usa.k, p.usa.q, w.init_budget, w.recent_budget, w.heavy_budget)
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_start > budget_s:
            break
    per_seq = sum(times) / len(times)
    tokens = sum(w.seq_lens[:len(times)]) / len(times)
    scale = sum(w.seq_lens) / tokens          # linear in cached tokens (ragged batches)
    return {"value": per_seq * 1e6 * scale, "unit": "us/layer", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{len(times)} of {w.batch} sequences (fp32, torch CPU, {os.cpu_count()} logical cpus, "
                      f"{torch.get_num_threads()} torch threads), {sum(times):.2f} s measured, scaled x{scale:.2f} by cached tokens"}


def cpu_sparse_stages(w, torch):
    """The same stages as the GPU step (codes cached, encode the new token, select, gather-attend), run by the C oracle
    (OpenMP) on the host for the first sequence of the workload and scaled linearly by cached tokens to the batch.  The
    codes of the cached keys are made beforehand, un-timed, as on the GPU."""
    import numpy as np
    from hashattention.synthetic import Workload, make_problem
    from oracle import c_oracle, hashattn_oracle as orc
    w1 = Workload(**{**w.__dict__, "name": w.name + "-cpu", "batch": 1, "seq_lens": [w.seq_lens[0]], "seed": w.seed})
    p = make_problem(w1)
    S, H, Hkv, d = w1.seq_lens[0], w.n_q_heads, w.n_kv_heads, w.head_dim
    Hc, W = len(p.usa.k), w.lth_final_dim // 32
    np_layers = lambda head: [(Wt.numpy(), b.numpy()) for Wt, b in head]
    kf = p.k.float()
    kcodes = np.empty((1, Hc, S, W), dtype=np.uint32)
    for hc in range(Hc):
        kcodes[0, hc] = c_oracle.encode(kf[0, hc * Hkv // Hc].numpy(), np_layers(p.usa.k[hc]))[1]
    t0 = time.perf_counter()
    qcodes = np.empty((1, H, W), dtype=np.uint32)
    for hc in range(Hc):        # the new key's code (already in kcodes: timed for the work, result identical)
        c_oracle.encode(kf[0, hc * Hkv // Hc, S - 1:S].numpy(), np_layers(p.usa.k[hc]))
    for h in range(H):
        qcodes[0, h] = c_oracle.encode(p.q[0, h].float().numpy(), np_layers(p.usa.q[h]))[1][0]
    t1 = time.perf_counter()
    cap = min(S, w.init_budget + w.recent_budget + orc.heavy_count(S, w.heavy_budget))
    idx, counts = c_oracle.select(kcodes, qcodes, [S], w.init_budget, w.recent_budget, w.heavy_budget, cap)
    t2 = time.perf_counter()
    c_oracle.sparse_attend(p.q[:, :, 0], p.k, p.v, idx, counts, 1.0 / math.sqrt(d))
    t3 = time.perf_counter()
    scale = sum(w.seq_lens) / S
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count()))
    enc, sel, att = (t1 - t0) * 1e6 * w.batch, (t2 - t1) * 1e6 * scale, (t3 - t2) * 1e6 * scale
    return {"value": enc + sel + att, "unit": "us/layer", "cores": threads, "kind": "port",
            "stages_us": {"encode_new_k_and_q": enc, "score_select_full_sort": sel, "gather_attend": att},
            "sample": f"sequence 0 of {w.batch} ({S} tokens, C oracle with OpenMP, {threads} threads), {t3 - t0:.2f} s measured; "
                      f"encode scaled x{w.batch} by sequences, select and attend x{scale:.2f} by cached tokens"}


def traffic_probe(torch, device, attend_fns):
    """For `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`: a plain copy of known size three times, then the step's
    attention launch three times on every input set in turn.  The copy gives the scale of the counter (bytes per reported KiB)."""
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device=device).random_(0, 255)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    for _ in range(3):
        for fn in attend_fns:
            fn()
    torch.cuda.synchronize()
    print(json.dumps({"probe": f"copy 1 GiB x3 (runtime copy kernel), then the step's sparse_attend launch x3 on each of {len(attend_fns)} input sets in turn"}))


def decoder_bench(args, torch):
    """--config config3: the whole 32-layer Llama-3.1-8B-shaped decoder step (random-init weights, synthetic cache of
    131072 tokens per sequence, batch 4) with the sparse attention step in every layer; decode tokens/s."""
    from hashattention import _ops
    from hashattention.decoder import LlamaShapedDecoder
    from hashattention.synthetic import named_workload
    w = named_workload("config3")
    B, S = w.batch, w.max_seq_len
    dev = "cuda:0"
    dec = LlamaShapedDecoder(n_layers=args.layers, n_code_heads=w.n_code_heads, init_budget=w.init_budget,
                             recent_budget=w.recent_budget, heavy_budget=w.heavy_budget, dtype=torch.bfloat16, device=dev)
    dec.allocate(B, S)
    t0 = time.perf_counter()
    ms_prefill_encode = dec.fill_cache_synthetic(S - 1)
    fill_s = time.perf_counter() - t0
    tokens = torch.randint(0, dec.vocab, (B,), device=dev)
    logits = [None]

    def step(dense=False):
        with torch.no_grad():
            logits[0] = dec.decode_step(tokens, advance=False, dense=dense)

    def graphed(fn):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        return g

    ms_eager = time_gpu(step, args.steps, args.warmup, torch)
    eager_logits = logits[0].clone()
    g = graphed(step)
    ms_graph = time_gpu(g.replay, args.steps, args.warmup, torch)
    graph_ok = bool(torch.equal(logits[0], eager_logits))
    ms_step = min(ms_eager, ms_graph)
    gd = graphed(lambda: step(dense=True))
    ms_dense = time_gpu(gd.replay, max(5, args.steps // 8), 2, torch)
    # the attention step of one layer alone, at this shape
    hl0 = dec.hash[0]
    q = torch.randn(B, dec.H, 1, dec.d, device=dev).to(torch.bfloat16)
    out = torch.empty(B, dec.H, dec.d, dtype=torch.bfloat16, device=dev)

    def layer_step():
        hl0.n_cached = S - 1
        hl0.step(q, dec.k_cache[0], dec.v_cache[0], S, out)

    ms_layer = time_gpu(layer_step, args.steps, args.warmup, torch)
    # the layer's attention launch alone: the fused launch replays on the histograms and query codes the step left
    # behind; the two-launch path's gather reads the index lists its selection wrote
    fused0 = hl0.use_fused and hl0.fused_ok and not hl0.overlap_windows
    if fused0:
        attend_alone = lambda: hl0.attend_fused(q[:, :, 0, :], dec.k_cache[0], dec.v_cache[0], out, S, None)
    else:
        attend_alone = lambda: hl0.attend(q[:, :, 0, :], dec.k_cache[0], dec.v_cache[0], out)
    ms_attend = time_gpu(attend_alone, args.steps, args.warmup, torch)
    n_sel_rows = int(hl0.counts.sum().item())
    # the generation loop proper: greedy tokens at advancing positions, one captured graph replayed per token with the
    # position on the device (the last `n_gen` slots of the synthetic cache are written again by the generated tokens)
    n_gen = max(8, min(args.steps, S - 2))
    def rewind():
        dec.seq_len = S - 1 - n_gen
        for hl in dec.hash:
            hl.n_cached = dec.seq_len
    with torch.no_grad():
        rewind()
        dec.generate(tokens, 4)                       # capture + a few replays
        rewind()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        gen_tokens = dec.generate(tokens, n_gen)
        e1.record()
        torch.cuda.synchronize()
    ms_gen = e0.elapsed_time(e1) / n_gen
    ab = algorithmic_bytes(w, n_sel_rows)
    n_params = sum(t.numel() for p in dec.layers for t in p.values()) + dec.lm_head.numel()
    step_bytes = 2 * n_params + dec.L * (ab["score"] + ab["select"] + ab["gather"])
    res = {
        "metric": "decode_tokens_per_s", "value": B / (min(ms_step, ms_gen) * 1e-3), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": min(ms_step, ms_gen),
        "step_launch": {"value_is": "generation_loop" if ms_gen <= ms_step else ("graph" if ms_graph <= ms_eager else "eager"),
                        "hip_graph_replay_ms": ms_graph, "eager_launches_from_python_ms": ms_eager, "generation_loop_ms": ms_gen},
        "graph_replay_matches_eager": graph_ok,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"config3: {dec.L}-layer Llama-3.1-8B-shaped decoder step, B={B} context={S} H={dec.H} Hkv={dec.Hkv} "
                               f"d={dec.d} hidden={dec.hidden} ffn={dec.ffn} vocab={dec.vocab} code_heads={dec.Hc} "
                               f"init={w.init_budget} recent={w.recent_budget} heavy={w.heavy_budget:g} n_sel={n_sel_rows // (B * dec.H)}"},
        "generation_loop": {"tokens_per_sequence": n_gen, "ms_per_token_step": ms_gen, "tokens_per_s": B / (ms_gen * 1e-3),
                            "how": "greedy, positions on the device, one HIP graph replayed per token + arg-max",
                            "distinct_tokens": int(gen_tokens.unique().numel())},
        "dense_attention_step_ms": ms_dense, "speedup_vs_dense_attention": ms_dense / min(ms_step, ms_gen),
        "dense_tokens_per_s": B / (ms_dense * 1e-3),
        "attention_step_us_per_layer": ms_layer * 1e3, "attention_share_of_step": dec.L * ms_layer / min(ms_step, ms_gen),
        "prefill_encode_ms_per_layer": ms_prefill_encode,
        "prefill_encode_tflops": 2 * B * dec.Hc * (S - 1) * (128 * 128 * 2 + 128 * 32) / (ms_prefill_encode * 1e-3) / 1e12,
        "cache_fill_seconds": fill_s,
        "hbm_gbps_step": step_bytes / (ms_step * 1e-3) / 1e9, "hbm_frac_step": step_bytes / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "roofline": {"kernel": "sparse_attend_kernel (selection fused)" if fused0 else "sparse_attend_kernel", "bound": "hbm", "achieved": ab["gather"] / (ms_attend * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": ab["gather"] / (ms_attend * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                     "traffic": None, "algorithmic_bytes": ab["gather"], "us": ms_attend * 1e3},
    }
    return res


def hf_path_bench(args, torch):
    """--config config3 --hf-path: the drop-in path itself.  A random-init `transformers` Llama of Llama-3.1-8B width with
    `--layers` decoder layers goes through `load_usa(config, None)` + `convert_usa` (the reference's own call sequence,
    README.md:37-55), its KV cache is filled directly with 131071 synthetic tokens per sequence (batch 4), and single-token
    forward passes are timed - with `hashattention.cache.PreallocatedCache` (appends in place) and with the library's
    `DynamicCache` (re-copies the layer's whole cache every step) - next to `LlamaShapedDecoder.from_hf` of the same model.
    Per-layer figures are the slope between a model of `--layers` layers and one of half as many (embedding, final norm and
    lm_head cancel)."""
    from transformers import DynamicCache, LlamaConfig, LlamaForCausalLM
    from hashattention import hashattention_llama as hl
    from hashattention.cache import PreallocatedCache
    from hashattention.decoder import LlamaShapedDecoder
    from hashattention.synthetic import named_workload
    shape = args.config if args.config in ("config2", "config3") else "config3"     # config2: 16 sequences of 65536 tokens
    w = named_workload(shape)
    B, S = (args.batch or w.batch), w.max_seq_len
    dev = "cuda:0"
    steps, warm = max(8, min(args.steps, 64)), 3

    def build(L):
        cfg = LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=L, num_attention_heads=32, num_key_value_heads=8,
                          head_dim=128, vocab_size=128256, max_position_embeddings=S + 4096, rope_theta=500000.0, rms_norm_eps=1e-5)
        for k, v in dict(lth_init_dim=128, lth_final_dim=32, lth_thold=0, lth_num_layers=3, init_budget=w.init_budget,
                         heavy_budget=w.heavy_budget, recent_budget=w.recent_budget, usa_retrieve_depth=0, usa_eval_mode="simple").items():
            setattr(cfg, k, v)
        torch.manual_seed(0)
        with torch.device(dev):
            model = LlamaForCausalLM(cfg).bfloat16()
        usa = hl.load_usa(cfg, None)
        return cfg, hl.convert_usa(model, cfg, usa, collect_stats=False, train_usa=False).eval(), usa

    def fill(cache, L, n):
        g = torch.Generator(device=dev).manual_seed(1)
        for l in range(L):
            k = torch.randn(B, 8, n, 128, generator=g, device=dev, dtype=torch.bfloat16)
            v = torch.randn(B, 8, n, 128, generator=g, device=dev, dtype=torch.bfloat16)
            cache.update(k, v, l)
            del k, v

    def time_tokens(model, cache, n_steps, n_warm, padded=False):
        ids = torch.randint(0, 128256, (B, 1), device=dev)

        def one():
            am = None
            if padded:      # a left-padded batch, as batched generation makes them: five padding tokens in front of sequence 0
                am = torch.ones(B, cache.get_seq_length() + 1, dtype=torch.long, device=dev)
                am[0, :5] = 0
            model(ids, attention_mask=am, past_key_values=cache, use_cache=True)
        with torch.no_grad():
            for _ in range(n_warm):                      # the first pass hashes the 131071 cached keys of every layer
                one()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            e0.record()
            for _ in range(n_steps):
                one()
            e1.record()
            host_ms = (time.perf_counter() - t0) * 1e3 / n_steps     # time to issue a step from Python (no wait inside)
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n_steps, host_ms

    out = {}
    L_full = max(2, args.layers if args.layers != 32 else 4)
    for L in (L_full // 2, L_full):
        cfg, model, usa = build(L)
        cache = PreallocatedCache(capacity=S + 256, num_layers=L)
        fill(cache, L, S - 1 - warm)
        ms_pre, host_pre = time_tokens(model, cache, steps, warm)
        # the same steps on a left-padded batch (the padding mask inside the fused launch)
        cache.crop(-(steps + warm))
        ms_padded, _ = time_tokens(model, cache, steps, warm, padded=True)
        # the same with only the attention module in few launches (the decoder layer around it through the library's own forward)
        for lyr in model.model.layers:
            lyr.self_attn.fast_layer = False
        cache.crop(-(steps + warm))
        ms_attn_fast, _ = time_tokens(model, cache, steps, warm)
        for lyr in model.model.layers:
            lyr.self_attn.fast_layer = True
        # the attention module of one layer alone, at a fixed length: hidden states in, attention output out
        layer = model.model.layers[0].self_attn
        h = torch.randn(B, 1, 4096, device=dev, dtype=torch.bfloat16)
        with torch.no_grad():
            n_now = cache.get_seq_length()
            pos = torch.full((B, 1), n_now, device=dev, dtype=torch.long)
            pe = model.model.rotary_emb(h, pos)

            def attn_only():
                layer(hidden_states=h, position_embeddings=pe, attention_mask=None, past_key_values=cache)
                cache.layers[0].crop(-1)
            ms_attn = time_gpu(attn_only, steps, warm, torch)
        del cache
        hl.reset_usa(model)
        # a cache that the caller (or `generate`) created as the library's DynamicCache: taken over in place at the first decode
        # step (the default), and left to the library (one torch.cat of every layer's whole cache per token)
        dyn = DynamicCache()
        fill(dyn, L, S - 1 - warm)
        ms_adopted, _ = time_tokens(model, dyn, steps, warm)
        del dyn
        hl.reset_usa(model)
        torch.cuda.empty_cache()
        for lyr in model.model.layers:
            lyr.self_attn.adopt_cache = False
        dyn = DynamicCache()
        fill(dyn, L, S - 1 - 2)
        ms_dyn, _ = time_tokens(model, dyn, 4, 2)
        del dyn
        hl.reset_usa(model)
        torch.cuda.empty_cache()
        dec = LlamaShapedDecoder.from_hf(model, usa, batch=B, cache_len=S + 256)
        dec.fill_cache_synthetic(S - 1)
        tok = torch.randint(0, 128256, (B,), device=dev)
        with torch.no_grad():
            dec.generate(tok, 4)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            dec.generate(tok, steps)
            e1.record()
            torch.cuda.synchronize()
        ms_dec = e0.elapsed_time(e1) / steps
        out[L] = dict(patched_preallocated_ms=ms_pre, patched_preallocated_host_issue_ms=host_pre, patched_left_padded_batch_ms=ms_padded,
                      patched_preallocated_attention_module_only_ms=ms_attn_fast, patched_dynamic_cache_adopted_ms=ms_adopted,
                      patched_dynamic_cache_ms=ms_dyn,
                      decoder_generate_ms=ms_dec, patched_attention_module_us=ms_attn * 1e3)
        del dec, model, usa
        torch.cuda.empty_cache()
    lo, hi = out[L_full // 2], out[L_full]
    dL = L_full - L_full // 2
    per_layer = {k.replace("_ms", "_us_per_layer"): (hi[k] - lo[k]) / dL * 1e3 for k in hi if k.endswith("_ms")}
    res = {
        "metric": "decode_ms_per_token_patched_transformers_model", "value": hi["patched_preallocated_ms"], "unit": "ms/token-step",
        "n_gpus": 1, "steps": steps, "warmup": warm, "ms_per_step": hi["patched_preallocated_ms"], "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{shape} through the drop-in API: transformers Llama (hidden 4096, ffn 14336, 32/8 heads, vocab 128256), "
                               f"{L_full} layers, load_usa(config, None) + convert_usa, B={B} context={S}, one key-side hash MLP per query "
                               f"head (fp32 modules), init={w.init_budget} recent={w.recent_budget} heavy={w.heavy_budget:g}"},
        "layers": {str(k): v for k, v in out.items()},
        "per_layer_slope": per_layer,
        "how": "single-token forward passes of the patched model, eager launches from Python, HIP events around the timed passes "
               "(patched_preallocated: whole decoder layers in seven launches each; ..._attention_module_only: the attention module in five "
               "launches inside the library's own decoder layer; patched_left_padded_batch: the seven-launch steps with an attention mask that "
               "blocks five padding tokens in front of sequence 0, handed to the fused launch as one number per sequence; patched_dynamic_cache_adopted: the caller hands over a plain DynamicCache, "
               "whose layers the attention modules turn into in-place ones at the first decode step; patched_dynamic_cache: the same "
               "with that switched off, torch.cat per layer and token); "
               "per-layer = difference between the two layer counts; decoder = LlamaShapedDecoder.from_hf(...).generate (one HIP graph "
               "replayed per token); patched_attention_module = self_attn.forward of one layer alone at a fixed length",
    }
    return res


class InputSet:
    """One attention layer's worth of inputs and state: its own Q/K/V, hash weights, bit-cache, workspaces and output."""

    def __init__(self, w, args, dev, torch, seed_offset, code_heads=None):
        from hashattention.decode import HashDecodeLayer
        from hashattention.synthetic import Workload, make_problem_on_device, make_usa_weights
        self.w = Workload(**{**w.__dict__, "seed": w.seed + seed_offset})
        self.p = make_problem_on_device(self.w, dev)
        self.torch, self.dev = torch, dev
        self.ragged = len(set(w.seq_lens)) > 1
        self.seq_lens = self.p.seq_lens if self.ragged else None
        self.S = w.max_seq_len
        self.q3 = self.p.q[:, :, 0, :]
        self.layer = self.make_layer(self.p.usa, args)
        self.out = torch.empty(w.batch, w.n_q_heads, w.head_dim, dtype=w.dtype, device=dev)

    def make_layer(self, usa, args):
        from hashattention.decode import HashDecodeLayer
        w, torch = self.w, self.torch
        layer = HashDecodeLayer(usa.k, usa.q, w.n_q_heads, w.n_kv_heads, w.head_dim, w.lth_num_layers, w.lth_int_dim, w.lth_final_dim,
                                w.init_budget, w.recent_budget, w.heavy_budget, device=self.dev)
        if args.fused_min_rows is not None:
            layer.fused_min_rows = args.fused_min_rows
        layer.allocate(w.batch, self.S)
        layer.select_algo = args.select_algo
        layer.overlap_windows = args.overlap_windows
        layer.use_fused = not args.two_launch
        # prefill: codes of every cached key (un-timed, as in the reference protocol: efficiency/kernels/torchatt.py:183-184)
        layer.encode_keys(self.p.k, use_mfma=(w.dtype == torch.bfloat16 and not args.exact_encode))
        torch.cuda.synchronize()
        layer.n_cached = self.S - 1             # the step re-encodes the newest key, as a real decode step does
        return layer

    def other_code_heads(self, n_code_heads, args):
        """A second layer over the same K/V with `n_code_heads` key-side hash MLPs (its own weights and bit-cache)."""
        from hashattention.synthetic import Workload, make_usa_weights
        w2 = Workload(**{**self.w.__dict__, "n_code_heads": n_code_heads})
        twin = object.__new__(InputSet)
        twin.__dict__.update(self.__dict__)
        twin.w = w2
        twin.layer = twin.make_layer(make_usa_weights(w2), args)
        twin.out = self.torch.empty_like(self.out)
        return twin

    # the launches that are timed
    def step(self):
        if self.ragged:
            self.layer.step(self.p.q, self.p.k, self.p.v, self.S, self.out, seq_lens=self.seq_lens)
        else:
            self.layer.n_cached = self.S - 1
            self.layer.step(self.p.q, self.p.k, self.p.v, self.S, self.out)

    def encode_only(self):
        from hashattention import _ops
        l, S = self.layer, self.S
        _ops.encode_step(self.p.k[:, :, S - 1:S], self.q3, l.wk, l.wq, l.num_layers, l.int_dim, l.final_dim, l.codes, l.qcodes, pos0=S - 1)

    def select(self):
        self.layer.select(self.S, self.seq_lens)

    def select_prepare(self):
        self.layer.select_prepare(self.S, self.seq_lens)

    def attend_fused(self):
        self.layer.attend_fused(self.q3, self.p.k, self.p.v, self.out, self.S, self.seq_lens)

    def attend_lists(self):
        self.layer.attend(self.q3, self.p.k, self.p.v, self.out)

    def attend_fused_paged(self):
        """The fused launch reading the same cache through a token -> slot table that maps every token to its own row."""
        from hashattention import _ops
        l, w = self.layer, self.w
        if not hasattr(self, "slots"):
            self.slots = self.torch.arange(self.S, dtype=self.torch.int32, device=self.dev).repeat(w.batch, 1)
        _ops.sparse_decode_fused(self.q3, self.p.k, self.p.v, l.codes, l.qcodes.view(w.batch, w.n_q_heads, l.W), self.S, self.seq_lens,
                                 l.init_budget, l.recent_budget, l.heavy_budget, l.ws_select, l.sm_scale, self.out, l.ws_fused,
                                 thresholds_ready=not l.local_thresholds, out_counts=l.counts, slots=self.slots)

    def attend_lists_paged(self):
        from hashattention import _ops
        l = self.layer
        if not hasattr(self, "slots"):
            self.slots = self.torch.arange(self.S, dtype=self.torch.int32, device=self.dev).repeat(self.w.batch, 1)
        _ops.sparse_decode(self.q3, self.p.k, self.p.v, l.idx, l.counts, l.sm_scale, self.out, l.ws_attend, slots=self.slots)


def first_step_probe(s, args, torch):
    """The first decode step after a prefill, per layer, with one key-side hash MLP per query head (the reference's layout):
    every cached key is hashed in bulk (`encode_keys_bulk`: bf16 MFMA for a hash module kept in bf16, fp32 MFMA for one kept
    in fp32) and one decode step follows.  Milliseconds per layer, HIP events; the fp32 module's scalar-kernel time is measured
    on one sequence's keys and scaled to the batch."""
    from hashattention import _ops
    from hashattention.decode import HashDecodeLayer
    from hashattention.synthetic import make_usa_weights
    w, S = s.w, s.S
    usa = make_usa_weights(w)
    out = {"code_heads": w.n_code_heads, "cached_tokens": S - 1, "sequences": w.batch}
    for name, arith in (("bf16_module", _ops.HA_ARITH_BF16), ("fp32_module", _ops.HA_ARITH_F32)):
        layer = HashDecodeLayer(usa.k, usa.q, w.n_q_heads, w.n_kv_heads, w.head_dim, w.lth_num_layers, w.lth_int_dim, w.lth_final_dim,
                                w.init_budget, w.recent_budget, w.heavy_budget, arith=arith, device=s.dev)
        layer.allocate(w.batch, S)

        def first():
            layer.encode_keys_bulk(s.p.k[:, :, :S - 1])
            layer.n_cached = S - 1
            layer.step(s.p.q, s.p.k, s.p.v, S, s.out)

        def bulk():
            layer.encode_keys_bulk(s.p.k[:, :, :S - 1])

        out[name + "_ms"] = time_gpu(first, 3, 1, torch)
        out[name + "_bulk_hash_ms"] = time_gpu(bulk, 3, 1, torch)
        if arith == _ops.HA_ARITH_F32:
            def scalar():
                _ops.encode_pack(s.p.k[:1, :, :S - 1], layer.wk, layer.num_layers, layer.int_dim, layer.final_dim, layer.codes, 0, None, arith)
            out["fp32_module_scalar_kernel_bulk_hash_ms"] = time_gpu(scalar, 1, 1, torch) * w.batch
        del layer
    flop = w.batch * w.n_code_heads * (S - 1) * 2 * (w.head_dim * w.lth_int_dim + (w.lth_num_layers - 2) * w.lth_int_dim ** 2
                                                      + w.lth_int_dim * w.lth_final_dim)
    out["bulk_hash_tflops"] = {k[:-len("_bulk_hash_ms")]: flop / (out[k] * 1e-3) / 1e12 for k in list(out) if k.endswith("_bulk_hash_ms")}
    return out


def chunk_steps_probe(s, args, torch):
    """Chunked decode (1 < q_len <= 128 new tokens per sequence, the reference's `compute_mask_multi` branch with one causal
    window per query row, hashattention_llama.py:423-428): the chunk's rows become batch entries of ONE selection and ONE attention
    launch.  Microseconds per chunk and layer for 8 and 64 rows per sequence, and the gather's share of the HBM roofline
    (516 bytes per selected (row, head, token))."""
    from hashattention.decode import HashDecodeLayer
    from hashattention.synthetic import make_usa_weights
    w, S = s.w, s.S
    usa = make_usa_weights(w)
    layer = HashDecodeLayer(usa.k, usa.q, w.n_q_heads, w.n_kv_heads, w.head_dim, w.lth_num_layers, w.lth_int_dim, w.lth_final_dim,
                            w.init_budget, w.recent_budget, w.heavy_budget, device=s.dev)
    layer.allocate(w.batch, S)
    layer.encode_keys_bulk(s.p.k[:, :, :S])
    layer.n_cached = S
    heavy = layer.heavy_count(S)
    out = {"sequences": w.batch, "cached_tokens": S}
    for T in (8, 64):
        q = torch.randn(w.batch, w.n_q_heads, T, w.head_dim, device=s.dev).to(s.p.k.dtype)
        o = torch.empty_like(q)
        run = lambda: layer.chunk_step(q, s.p.k, s.p.v, S, o, heavy + 0.5)
        ms = time_gpu(run, 3, 1, torch)
        n_sel = int(layer._chunk["cnt"].sum().item())
        out[f"rows_{T}"] = {"us_per_chunk": ms * 1e3, "us_per_row": ms * 1e3 / T, "selected_row_head_tokens": n_sel,
                            "gather_hbm_frac_of_whole_chunk_step": n_sel * 516 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
        layer._chunk = None
        del q, o
    del layer
    torch.cuda.empty_cache()
    return out


def brief_layer_bench(name, args, torch, dev, n_sets=2):
    """One of the other named configurations, timed like the headline one but without its side legs: the step over a rotation
    of `n_sets` input sets (eager launches and a graph replay), its attention launch alone, its scoring launch alone, and the
    dense flash-decode on the same inputs."""
    from hashattention import _ops
    from hashattention.synthetic import named_workload
    w = named_workload(name)
    sets = [InputSet(w, args, dev, torch, 101 * i) for i in range(n_sets)]
    s0, layer = sets[0], sets[0].layer
    B, H, S = w.batch, w.n_q_heads, w.max_seq_len
    fused = layer.use_fused and layer.fused_ok and not layer.overlap_windows
    steps, warmup = max(20, args.steps // 2), max(3, args.warmup // 2)
    rot = lambda n: [getattr(s, n) for s in sets]
    ms_eager, ms_graph, graph_ok = time_step(sets, steps, warmup, torch)
    ms_step = min(ms_eager, ms_graph)
    ms_prepare = time_rotating(rot("select_prepare"), steps, warmup, torch) if fused else None
    for s in sets:
        s.step()
        if not fused:
            s.select()
    ms_attend = time_rotating(rot("attend_fused" if fused else "attend_lists"), steps, warmup, torch)
    out_dense = torch.empty_like(s0.out)
    ws_dense = _ops.workspace(_ops.dense_decode_workspace_bytes(B, H, S), dev)
    dense = [(lambda s=s: _ops.dense_decode(s.q3, s.p.k, s.p.v, S, s.seq_lens, layer.sm_scale, out_dense, ws_dense)) for s in sets]
    ms_dense = time_rotating(dense, max(6, steps // 4), 2, torch)
    s0.step()
    if fused:
        s0.select()
    n_sel_rows = int(layer.counts.sum().item())
    ab = algorithmic_bytes(w, n_sel_rows)
    step_bytes = ab["score"] + ab["gather"] + (0 if fused else ab["select"])
    res = {"workload": f"{w.name}: B={B} S={'ragged ' + str(min(w.seq_lens)) + '..' + str(S) if s0.ragged else S} code_heads={w.n_code_heads} "
                       f"code_bits={w.lth_final_dim} heavy={w.heavy_budget:g} n_sel={n_sel_rows // (B * H)}",
           "us_per_layer": ms_step * 1e3, "hip_graph_replay_us": ms_graph * 1e3, "eager_launches_from_python_us": ms_eager * 1e3,
           "graph_replay_matches_eager": graph_ok, "input_sets": n_sets, "steps": steps,
           "hbm_frac_step": step_bytes / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
           "speedup_vs_dense": ms_dense / ms_step, "dense_flash_decode_us": ms_dense * 1e3,
           "dense_hbm_frac": ab["dense"] / (ms_dense * 1e-3) / 1e9 / HBM_PEAK_GBPS,
           "roofline": {"kernel": "sparse_attend_kernel (selection fused)" if fused else "sparse_attend_kernel", "bound": "hbm",
                        "frac": ab["gather"] / (ms_attend * 1e-3) / 1e9 / HBM_PEAK_GBPS, "us": ms_attend * 1e3, "algorithmic_bytes": ab["gather"]}}
    if fused:
        res["score_roofline"] = {"kernel": "select_hist_kernel" + ("" if layer.local_thresholds else " + select_threshold_kernel"),
                                 "frac": ab["score"] / (ms_prepare * 1e-3) / 1e9 / HBM_PEAK_GBPS, "us": ms_prepare * 1e3,
                                 "algorithmic_bytes": ab["score"]}
    del sets, dense
    torch.cuda.empty_cache()
    return res


def time_step(sets, steps, warmup, torch):
    """The whole step over a rotation of input sets: eager launches and one HIP graph holding one pass over all sets,
    replayed.  Returns (ms eager, ms graph, graph replay reproduces the eager outputs)."""
    fns = [s.step for s in sets]
    ms_eager = time_rotating(fns, steps, warmup, torch)
    torch.cuda.synchronize()
    ref = [s.out.clone() for s in sets]

    def one_pass():
        for f in fns:
            f()
    graph = capture_graph(one_pass, torch)
    replays = max(1, (steps + len(sets) - 1) // len(sets))
    ms_graph = time_gpu(graph.replay, replays, max(1, warmup // len(sets)), torch) / len(sets)
    ok = all(bool(torch.equal(s.out, r)) for s, r in zip(sets, ref))
    return ms_eager, ms_graph, ok


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="config2")
    ap.add_argument("--batch", type=int, default=None, help="override the number of sequences of a uniform configuration (a variant, not the named workload)")
    ap.add_argument("--code-heads", type=int, default=None, help="key-side hash MLPs per layer: 8 (one per KV head, the named workloads) or 32 "
                    "(one per query head, as the reference's load_usa builds them); a variant, not the named workload")
    ap.add_argument("--input-sets", type=int, default=4, help="independent (Q, K, V, codes, weights) sets the timed launches rotate over, "
                    "so that consecutive launches never touch the same rows (as consecutive layers of a model)")
    ap.add_argument("--no-code-heads-32", action="store_true", help="skip the extra timing of the one-code-per-query-head layout")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true", help="config2 only: skip config1 / config3 / config4, the decoder step and "
                    "the patched transformers model that the default run appends to its line")
    ap.add_argument("--no-first-step", action="store_true", help="skip timing the first decode step after a prefill (bulk hash of all cached keys)")
    ap.add_argument("--exact-encode", action="store_true", help="fill the bit-cache with the fp32 kernel instead of MFMA")
    ap.add_argument("--select-algo", type=int, default=0, help="0 auto, 1 histogram, 2 sampled (ha_select algo)")
    ap.add_argument("--fused-min-rows", type=int, default=None, help="take the fused select-attend path from this many (sequence, head) rows on")
    ap.add_argument("--two-launch", action="store_true", help="ha_select + ha_sparse_decode instead of the fused select-attend path")
    ap.add_argument("--overlap-windows", action="store_true", help="attend to sink|recent on a second stream (ha_window_partial)")
    ap.add_argument("--layers", type=int, default=32, help="decoder layers of the config3 whole-step workload")
    ap.add_argument("--layer-only", action="store_true", help="config3: time one attention layer-step instead of the whole decoder")
    ap.add_argument("--hf-path", action="store_true", help="config3: time a transformers Llama patched with convert_usa (the drop-in path) "
                    "next to LlamaShapedDecoder; --layers sets the layer count (default 4)")
    ap.add_argument("--traffic-probe", action="store_true", help="run the launches the HBM-traffic counters are read from, then exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the sparse decode path shards by (sequence, KV head) with no exchange, "
              "and this build neither launches nor measures more than one GPU. Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    from hashattention import _ops
    from hashattention.synthetic import named_workload

    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the HashAttention path has no CPU fallback", file=sys.stderr)
        sys.exit(2)
    _ops.load_library()
    if args.config in ("config2", "config3") and args.hf_path:
        print(json.dumps(hf_path_bench(args, torch)))
        return
    if args.config == "config3" and not args.layer_only:
        print(json.dumps(decoder_bench(args, torch)))
        return
    dev = "cuda:0"
    w = named_workload(args.config)
    if args.batch is not None:
        if len(set(w.seq_lens)) > 1:
            sys.exit("--batch applies to configurations whose sequences have one length")
        w.batch, w.seq_lens, w.name = args.batch, [w.seq_lens[0]] * args.batch, f"{w.name} with batch {args.batch}"
    if args.code_heads is not None and args.code_heads != w.n_code_heads:
        w.n_code_heads, w.name = args.code_heads, f"{w.name} with {args.code_heads} code heads"
    n_sets = max(1, args.input_sets)
    sets = [InputSet(w, args, dev, torch, 101 * i) for i in range(n_sets)]
    s0 = sets[0]
    layer = s0.layer
    B, H, Hkv, d, S = w.batch, w.n_q_heads, w.n_kv_heads, w.head_dim, w.max_seq_len
    ragged = s0.ragged
    fused = layer.use_fused and layer.fused_ok and not layer.overlap_windows
    rot = lambda name: [getattr(s, name) for s in sets]

    if args.traffic_probe:
        for s in sets:
            s.step()
        traffic_probe(torch, dev, rot("attend_fused") if fused else rot("attend_lists"))
        return
    ms_step_eager, ms_step_graph, graph_ok = time_step(sets, args.steps, args.warmup, torch)
    ms_step = min(ms_step_graph, ms_step_eager)
    # the same step replayed on ONE input set, as earlier versions of this benchmark timed it: the rows it gathers (604 MB)
    # are the same in every launch, so part of them can still sit in the 256 MB memory-side cache
    ms_single_eager, ms_single_graph, _ = time_step(sets[:1], args.steps, args.warmup, torch)
    ms_encode = time_rotating(rot("encode_only"), args.steps, args.warmup, torch)
    ms_select = time_rotating(rot("select"), args.steps, args.warmup, torch)
    ms_window = 0.0
    if layer.overlap_windows:      # the dominant kernel as the step launches it: heavy tokens only, window partial merged
        p = s0.p
        _ops.window_partial(s0.q3, p.k, p.v, S, s0.seq_lens, w.init_budget, w.recent_budget, layer.sm_scale, layer.win)
        ms_attend = time_gpu(lambda: _ops.sparse_decode_heavy(s0.q3, p.k, p.v, layer.idx, layer.counts, layer.sm_scale, s0.out,
                                                              layer.ws_attend, layer.win, w.init_budget, w.recent_budget, S,
                                                              s0.seq_lens), args.steps, args.warmup, torch)
        ms_window = time_gpu(lambda: _ops.window_partial(s0.q3, p.k, p.v, S, s0.seq_lens, w.init_budget, w.recent_budget,
                                                         layer.sm_scale, layer.win), args.steps, args.warmup, torch)
    elif fused:    # the step's dominant launch: list rebuilt from the codes in LDS + gather-attend
        for s in sets:
            s.select()                         # leaves the lists for the comparison below
        ms_attend_lists = time_rotating(rot("attend_lists"), args.steps, args.warmup, torch)
        ms_prepare = time_rotating(rot("select_prepare"), args.steps, args.warmup, torch)
        ms_attend = time_rotating(rot("attend_fused"), args.steps, args.warmup, torch)
        ms_attend_single = time_gpu(s0.attend_fused, args.steps, args.warmup, torch)
        # the same launches through a token -> slot table (identity: every token at its own row), timed right behind the plain
        # ones; outputs must be the same bits
        try:
            ref_out = s0.out.clone()
            s0.attend_fused_paged()
            paged_ok = bool(torch.equal(s0.out, ref_out))
            ms_attend_paged = time_rotating(rot("attend_fused_paged"), args.steps, args.warmup, torch)
            ms_lists_paged = time_rotating(rot("attend_lists_paged"), args.steps, args.warmup, torch)
            paged = {"select_attend_fused_us": ms_attend_paged * 1e3, "vs_unpaged": ms_attend_paged / ms_attend,
                     "two_launch_attend_us": ms_lists_paged * 1e3, "two_launch_vs_unpaged": ms_lists_paged / ms_attend_lists,
                     "same_bits_as_unpaged": paged_ok,
                     "how": "ha_sparse_decode_fused_paged / ha_sparse_decode_paged with slot_of_token[b, j] = j on the same cache"}
        except Exception as e:      # noqa: BLE001 - a side leg: reported in place of its figures
            paged = {"error": f"{type(e).__name__}: {e}"}
    else:
        ms_attend = time_rotating(rot("attend_lists"), args.steps, args.warmup, torch)
    out_dense = torch.empty_like(s0.out)
    ws_dense = _ops.workspace(_ops.dense_decode_workspace_bytes(B, H, S), dev)
    dense = [(lambda s=s: _ops.dense_decode(s.q3, s.p.k, s.p.v, S, s.seq_lens, layer.sm_scale, out_dense, ws_dense)) for s in sets]
    ms_dense = time_rotating(dense, max(10, args.steps // 4), max(2, args.warmup // 4), torch)
    dense[0]()

    s0.step()
    if fused:
        s0.select()
    n_sel_rows = int(layer.counts.sum().item())
    ab = algorithmic_bytes(w, n_sel_rows)
    eb = 2 if w.dtype != torch.float32 else 4
    if layer.overlap_windows:      # bytes of the heavy-only launch: its rows, their indices, q, out and the window partial
        n_win_rows = sum(H * (min(w.init_budget, s) + s - max(s - w.recent_budget, min(w.init_budget, s))) for s in w.seq_lens)
        attend_bytes = (n_sel_rows - n_win_rows) * (2 * d * eb + 4) + B * H * (2 * d * eb + 130 * 4)
    else:
        attend_bytes = ab["gather"]
    # algorithmic bytes of the step: codes read once, rows gathered; the index lists travel through memory on the two-launch path only
    sparse_bytes = ab["score"] + ab["gather"] + (0 if fused else ab["select"])
    err = (s0.out.float() - out_dense.float()).abs().max().item()   # informational: sparse vs dense output distance
    traffic = measured_traffic(args.config, bool(fused), w.n_code_heads) if args.batch is None else None

    def roofline_obj(kernel, nbytes, ms, **extra):
        gbps = nbytes / (ms * 1e-3) / 1e9
        return {"kernel": kernel, "bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS,
                "algorithmic_bytes": nbytes, "us": ms * 1e3, **extra}

    res = {
        "metric": "sparse_decode_us_per_layer",
        "value": ms_step * 1e3,
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "step_launch": {"value_is": "graph" if ms_step_graph <= ms_step_eager else "eager",
                        "hip_graph_replay_us": ms_step_graph * 1e3, "eager_launches_from_python_us": ms_step_eager * 1e3,
                        "input_sets": n_sets,
                        "how": f"launches rotate over {n_sets} independent input sets (own Q, K, V, hash weights, bit-cache): no launch "
                               "touches the rows of the launch before it"},
        "single_set": {"us_per_layer": min(ms_single_eager, ms_single_graph) * 1e3, "hip_graph_replay_us": ms_single_graph * 1e3,
                       "eager_launches_from_python_us": ms_single_eager * 1e3,
                       "how": "the same step replayed on one input set (every launch gathers the same rows)"},
        "graph_replay_matches_eager": graph_ok,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if w.dtype == torch.bfloat16 else str(w.dtype).replace("torch.", ""),
        "data": "synthetic",
        "config": {"workload": f"{w.name}: B={B} S={'ragged ' + str(min(w.seq_lens)) + '..' + str(S) if ragged else S} "
                               f"H={H} Hkv={Hkv} d={d} code_heads={w.n_code_heads} code_bits={w.lth_final_dim} "
                               f"init={w.init_budget} recent={w.recent_budget} heavy={w.heavy_budget:g} "
                               f"n_sel={n_sel_rows // (B * H)}"},
        "path": ("ha_encode_step + ha_select_histogram + ha_sparse_decode_fused (thresholds in the attention launch)"
                 if layer.local_thresholds else "ha_encode_step + ha_select_prepare + ha_sparse_decode_fused") if fused else
                "ha_encode_step + ha_select + " + ("ha_window_partial + ha_sparse_decode_heavy" if layer.overlap_windows else "ha_sparse_decode"),
        "stages_us": {"encode_new_k_and_q": ms_encode * 1e3,
                      **({"select_prepare": ms_prepare * 1e3, "select_attend_fused": ms_attend * 1e3,
                          "select_attend_fused_single_set": ms_attend_single * 1e3,
                          "two_launch_select": ms_select * 1e3, "two_launch_attend": ms_attend_lists * 1e3} if fused else
                         {"score_select": ms_select * 1e3, "gather_attend": ms_attend * 1e3}),
                      "window_partial_second_stream": ms_window * 1e3, "dense_flash_decode": ms_dense * 1e3},
        "hbm_gbps_step": sparse_bytes / (ms_step * 1e-3) / 1e9,
        "hbm_frac_step": sparse_bytes / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "speedup_vs_dense": ms_dense / ms_step,
        "dense_hbm_gbps": ab["dense"] / (ms_dense * 1e-3) / 1e9,
        "tokens_per_s_layer": B / (ms_step * 1e-3),
        "sparse_vs_dense_max_abs": err,
        **({"paged_cache_identity_table": paged} if fused else {}),
        # the scoring stream (XOR + popcount over every cached code, histogrammed on the fly) as its own launch
        **({"score_roofline": roofline_obj("select_hist_kernel", ab["score"], ms_prepare)} if fused and layer.local_thresholds else {}),
        "roofline": roofline_obj("sparse_attend_kernel (selection fused)" if fused else "sparse_attend_kernel", attend_bytes, ms_attend,
                                 traffic=traffic["bytes"] if traffic else None,
                                 traffic_measured_at_commit=traffic["commit"] if traffic else None),
    }
    # the layout the reference's load_usa builds (one key-side hash MLP per QUERY head, hashattention_llama.py:642): four
    # times the codes, no code shared inside a KV group; same K/V, rotation and timing protocol
    if w.n_code_heads != H and not args.no_code_heads_32 and args.batch is None and fused:
        twins = [s.other_code_heads(H, args) for s in sets]
        t_eager, t_graph, t_ok = time_step(twins, args.steps, args.warmup, torch)
        t_fused = twins[0].layer.use_fused and twins[0].layer.fused_ok
        t_prepare = time_rotating([t.select_prepare for t in twins], args.steps, args.warmup, torch)
        t_attend = time_rotating([t.attend_fused if t_fused else t.attend_lists for t in twins], args.steps, args.warmup, torch)
        t_step = min(t_eager, t_graph)
        ab2 = algorithmic_bytes(twins[0].w, n_sel_rows)
        bytes2 = ab2["score"] + ab2["gather"] + (0 if t_fused else ab2["select"])
        res["code_heads_per_query_head"] = {
            "code_heads": H, "us_per_layer": t_step * 1e3, "hip_graph_replay_us": t_graph * 1e3, "eager_launches_from_python_us": t_eager * 1e3,
            "graph_replay_matches_eager": t_ok, "hbm_gbps_step": bytes2 / (t_step * 1e-3) / 1e9,
            "hbm_frac_step": bytes2 / (t_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, "speedup_vs_dense": ms_dense / t_step,
            "score_roofline": roofline_obj("select_hist_kernel", ab2["score"], t_prepare),
            "roofline": roofline_obj("sparse_attend_kernel (selection fused)" if t_fused else "sparse_attend_kernel", ab2["gather"], t_attend)}
        if not args.no_first_step:
            res["first_step_after_prefill"] = first_step_probe(twins[0], args, torch)
            res["chunked_decode"] = chunk_steps_probe(sets[0], args, torch)
        del twins
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(w, torch)
        res["cpu_sparse_port"] = cpu_sparse_stages(w, torch)
    # the other named configurations, the 32-layer decoder step and the patched transformers model, in the same run
    if args.config == "config2" and args.batch is None and args.code_heads is None and not args.two_launch and not args.no_other_configs:
        del sets, s0, layer, dense
        torch.cuda.empty_cache()
        t0 = time.perf_counter()

        def leg(name, fn):
            """A side leg must never take the headline figures down with it: a failure is reported in its place."""
            try:
                res[name] = fn()
            except Exception as e:      # noqa: BLE001 - reported, not swallowed
                res[name] = {"error": f"{type(e).__name__}: {e}"}
            torch.cuda.empty_cache()

        leg("other_configs", lambda: {name: brief_layer_bench(name, args, torch, dev) for name in ("config1", "config3", "config4")})
        sub = argparse.Namespace(**{**vars(args), "steps": max(10, args.steps // 10), "warmup": 2})

        def decoder_leg():
            d = decoder_bench(sub, torch)
            return {"tokens_per_s": d["value"], "ms_per_step": d["ms_per_step"],
                                  "generation_loop_ms": d["generation_loop"]["ms_per_token_step"],
                                  "hip_graph_replay_ms": d["step_launch"]["hip_graph_replay_ms"],
                                  "eager_launches_from_python_ms": d["step_launch"]["eager_launches_from_python_ms"],
                                  "dense_attention_step_ms": d["dense_attention_step_ms"], "speedup_vs_dense_attention": d["speedup_vs_dense_attention"],
                                  "attention_step_us_per_layer": d["attention_step_us_per_layer"], "hbm_frac_step": d["hbm_frac_step"],
                                  "prefill_encode_ms_per_layer": d["prefill_encode_ms_per_layer"], "prefill_encode_tflops": d["prefill_encode_tflops"],
                                  "graph_replay_matches_eager": d["graph_replay_matches_eager"], "workload": d["config"]["workload"],
                                  "steps": sub.steps}

        def hf_leg():
            h = hf_path_bench(argparse.Namespace(**{**vars(args), "steps": 16, "layers": 4, "config": "config3"}), torch)
            return {"workload": h["config"]["workload"], "ms_per_token_step": h["value"], "layers": h["layers"],
                    "per_layer_slope": h["per_layer_slope"], "how": h["how"]}

        leg("decoder_config3", decoder_leg)
        leg("patched_transformers_model_config3", hf_leg)
        res["other_legs_seconds"] = time.perf_counter() - t0
    print(json.dumps(res))


if __name__ == "__main__":
    main()

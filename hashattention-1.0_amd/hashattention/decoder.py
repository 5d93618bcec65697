"""A Llama-shaped decoder step around the sparse attention op: the tokens/s harness of the 32-layer workload.

The reference measures end-to-end decode throughput with a gpt-fast fork (efficiency/generate.py:386-434,
efficiency/model.py:98-345: RMSNorm, rotary embedding, SwiGLU feed-forward, static KV cache).  That fork is not
runnable as shipped and drives Double-Sparsity labels, not hashes; this module is the same decoder shape with
the HashAttention step in every layer.  Outside attention, for up to 8 sequences of bf16, every projection is the
row-streaming kernel: QKV with its RMSNorm folded in, gate/up with its RMSNorm in front and SwiGLU behind, lm_head with
the final norm in front (`ha_linear_skinny_fused`), output and down projection with the residual folded in
(`ha_linear_skinny`); RoPE + cache append is one launch (`ha_rope_append`).  Other dtypes and batches take library calls
(`F.rms_norm`, hipBLASLt) plus `ha_swiglu`.  The point is to time the whole step, and to check the plumbing around the op
(rotate-half RoPE, grouped KV heads, cache append) against `transformers`.

Caches are preallocated `[B, Hkv, S_cap, d]` per layer; a step writes the new key/value in place, so there is no
per-step concatenation.
"""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn.functional as F

from . import _ops
from .decode import HashDecodeLayer
from .synthetic import UsaWeights, layer_dims


class LlamaShapedDecoder:
    def __init__(self, n_layers=32, hidden=4096, ffn=14336, n_heads=32, n_kv_heads=8, head_dim=128, vocab=128256,
                 rope_theta=500000.0, rms_eps=1e-5, n_code_heads=8, lth_num_layers=3, lth_int_dim=128, lth_final_dim=32,
                 init_budget=128, recent_budget=128, heavy_budget=1.0 / 32, dtype=torch.bfloat16, device="cuda:0", seed=0,
                 random_init=True):
        self.L, self.hidden, self.ffn, self.H, self.Hkv, self.d, self.vocab = n_layers, hidden, ffn, n_heads, n_kv_heads, head_dim, vocab
        self.theta, self.eps, self.dtype, self.device = rope_theta, rms_eps, dtype, torch.device(device)
        self.Hc = n_code_heads
        self.use_skinny = True   # ha_linear_skinny for the projections (bf16, batch <= 8) ...
        self.skinny_all = True   # ... including the down projection and the lm_head (False: library GEMMs for these two)
        self.tile_few_rows = True     # batches of up to 8: output and down projection from tiled copies of their weights
        self.fuse_rope = True    # ha_rope_encode_step instead of ha_rope_append + ha_encode_step
        self.usa_shape = (lth_num_layers, lth_int_dim, lth_final_dim)
        self.budgets = (init_budget, recent_budget, heavy_budget)
        g = torch.Generator(device=device).manual_seed(seed)

        def w(*shape, fan_in):
            if not random_init:                    # the weights come from a model (`from_hf`): no 16 GB of noise first
                return torch.empty(0, dtype=dtype, device=device)
            return (torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * fan_in ** -0.5).to(dtype)

        q_out, kv_out = n_heads * head_dim, n_kv_heads * head_dim
        self.embed = w(vocab, hidden, fan_in=1.0)
        self.lm_head = w(vocab, hidden, fan_in=hidden)                     # [out, in] as nn.Linear
        self.final_norm = torch.ones(hidden, dtype=dtype, device=device)
        self.layers = []
        for _ in range(n_layers):
            self.layers.append(dict(
                attn_norm=torch.ones(hidden, dtype=dtype, device=device), ffn_norm=torch.ones(hidden, dtype=dtype, device=device),
                wqkv=w(q_out + 2 * kv_out, hidden, fan_in=hidden), wo=w(hidden, q_out, fan_in=q_out),
                w13=w(2 * ffn, hidden, fan_in=hidden), w2=w(hidden, ffn, fan_in=ffn)))
        self.hash: List[HashDecodeLayer] = []
        self.k_cache: List[torch.Tensor] = []
        self.v_cache: List[torch.Tensor] = []
        self.B = self.S_cap = self.seq_len = 0
        self.lengths = None      # per-sequence lengths of a ragged batch (host list); None: every sequence holds seq_len tokens
        self._gen_graph = self._gen_logits = None
        inv = 1.0 / (rope_theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32, device=device) / head_dim))
        self.inv_freq = inv

    # ------------------------------------------------------------------ setup
    def random_usa(self, seed: int) -> UsaWeights:
        g = torch.Generator().manual_seed(seed)
        nl, idim, fdim = self.usa_shape
        out = UsaWeights()
        for side, n in (("k", self.Hc), ("q", self.H)):
            heads = []
            for _ in range(n):
                heads.append([(torch.randn(fo, fi, generator=g) * fi ** -0.5, torch.randn(fo, generator=g) * 0.01)
                              for fi, fo in layer_dims(self.d, idim, fdim, nl)])
            setattr(out, side, heads)
        return out

    def allocate(self, B: int, S_cap: int, usa_per_layer: Optional[List[UsaWeights]] = None) -> None:
        self.B, self.S_cap, self.seq_len, self.lengths = B, S_cap, 0, None
        nl, idim, fdim = self.usa_shape
        init, recent, heavy = self.budgets
        arith = _ops.HA_ARITH_BF16 if self.dtype == torch.bfloat16 else _ops.HA_ARITH_F32
        self.k_cache, self.v_cache, self.hash = [], [], []
        for l in range(self.L):
            self.k_cache.append(torch.zeros(B, self.Hkv, S_cap, self.d, dtype=self.dtype, device=self.device))
            self.v_cache.append(torch.zeros(B, self.Hkv, S_cap, self.d, dtype=self.dtype, device=self.device))
            usa = usa_per_layer[l] if usa_per_layer is not None else self.random_usa(1000 + l)
            hl = HashDecodeLayer(usa.k, usa.q, self.H, self.Hkv, self.d, nl, idim, fdim, init, recent, heavy, arith=arith,
                                 device=self.device)
            hl.allocate(B, S_cap)
            self.hash.append(hl)
        self.attn_out = torch.empty(B, self.H, self.d, dtype=self.dtype, device=self.device)
        self.q_rot = torch.empty(B, self.H, self.d, dtype=self.dtype, device=self.device)
        self.ffn_act = torch.empty(B, self.ffn, dtype=self.dtype, device=self.device)
        self.qkv = torch.empty(B, (self.H + 2 * self.Hkv) * self.d, dtype=self.dtype, device=self.device)
        self.x_attn = [torch.empty(B, self.hidden, dtype=self.dtype, device=self.device) for _ in range(2)]
        self.gate_up = torch.empty(B, 2 * self.ffn, dtype=self.dtype, device=self.device)
        self.logits = torch.empty(B, self.vocab, dtype=self.dtype, device=self.device)
        # a step whose position lives on the device (`decode_step(..., device_pos=True)`, `generate`): token, position and
        # length of every sequence
        self.tok_dev = torch.zeros(B, dtype=torch.int64, device=self.device)
        self.pos_dev = torch.zeros(B, dtype=torch.int32, device=self.device)
        self.len_dev = torch.ones(B, dtype=torch.int32, device=self.device)
        self._gen_graph = self._gen_logits = None
        self.ws_dense = _ops.workspace(_ops.dense_decode_workspace_bytes(B, self.H, S_cap), self.device)
        self._pack_tiles()

    def _tiled(self) -> bool:
        """9 to 32 sequences of a bf16 model: the projections whose inputs fit (QKV, output, gate/up) run on the matrix cores
        from tiled copies of their weights (`ha_linear_tiled`)."""
        B = getattr(self, "B", 0)
        return self.use_skinny and self.dtype == torch.bfloat16 and B > 8 and _ops.linear_tiled_applies(B, max(self.hidden, self.H * self.d))

    def _pack_tiles(self) -> None:
        """(Re)make the tiled copies for the batch this decoder was allocated for; dropped when they do not apply."""
        few = self.use_skinny and self.dtype == torch.bfloat16 and 0 < getattr(self, "B", 0) <= 8 and self.tile_few_rows
        for p in self.layers:
            for name in ("wqkv_t", "wo_t", "w13_t", "w2_t"):
                p.pop(name, None)
            if "wqkv" not in p:
                continue
            if self._tiled():
                p["wqkv_t"] = _ops.pack_weight_tiles(p["wqkv"])
                p["wo_t"] = _ops.pack_weight_tiles(p["wo"])
                p["w13_t"] = _ops.pack_weight_tiles(p["w13"], glu=True)
                if self.B <= 16:        # with its residual inside: ahead of the library's GEMM plus an addition up to 16 rows
                    p["w2_t"] = _ops.pack_weight_tiles(p["w2"])
            elif few:
                # up to 8 sequences: the two projections that carry no norm run from tiled copies as well (4 sequences, launched
                # alone: output projection 8.5 us against 9.3 for the row-streaming kernel, down projection 21.8 against 23.8)
                if self.H * self.d <= _ops.LINEAR_TILED_MAX_K:
                    p["wo_t"] = _ops.pack_weight_tiles(p["wo"])
                p["w2_t"] = _ops.pack_weight_tiles(p["w2"])

    def fill_cache_synthetic(self, seq_len: int, seed: int = 0) -> float:
        """Put `seq_len` synthetic tokens (N(0,1) keys/values) in every layer's cache and hash all keys with the MFMA
        encoder.  Returns the milliseconds the hashing of one layer took (HIP events)."""
        g = torch.Generator(device=self.device).manual_seed(seed)
        ms = []
        for l in range(self.L):
            for b in range(self.B):
                self.k_cache[l][b, :, :seq_len] = torch.randn(self.Hkv, seq_len, self.d, generator=g, device=self.device).to(self.dtype)
                self.v_cache[l][b, :, :seq_len] = torch.randn(self.Hkv, seq_len, self.d, generator=g, device=self.device).to(self.dtype)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            self.hash[l].encode_keys(self.k_cache[l][:, :, :seq_len], pos0=0,
                                     use_mfma=self.dtype == torch.bfloat16 and self.hash[l].wk_bf16 is not None)
            e1.record()
            torch.cuda.synchronize()
            ms.append(e0.elapsed_time(e1))
            self.hash[l].n_cached = seq_len
        self.seq_len = seq_len
        return sum(ms) / len(ms)

    def load_cache(self, keys: List[torch.Tensor], values: List[torch.Tensor], lengths: Optional[List[int]] = None) -> None:
        """Take over a prefilled cache: per layer keys/values [B, Hkv, S, d] (rotary already applied to the keys).
        `lengths`: tokens of every sequence when the batch is ragged (right-padded to S); what lies beyond a sequence's
        length is never read and is overwritten as the sequence grows.  A ragged batch decodes through `generate` only."""
        S = keys[0].shape[2]
        if lengths is not None:
            lengths = [int(n) for n in lengths]
            if len(lengths) != self.B or min(lengths) < 1 or max(lengths) > S:
                raise ValueError(f"lengths must be {self.B} values in 1..{S}")
            if len(set(lengths)) == 1:       # equal lengths after all: a uniform batch of that length
                keys, values = [k[:, :, :lengths[0]] for k in keys], [v[:, :, :lengths[0]] for v in values]
                S, lengths = lengths[0], None
        for l in range(self.L):
            self.k_cache[l][:, :, :S] = keys[l]
            self.v_cache[l][:, :, :S] = values[l]
            # as the patched layer hashes a prefilled cache: on the matrix cores, in the arithmetic of the hash module
            self.hash[l].encode_keys_bulk(self.k_cache[l][:, :, :S], pos0=0)
            self.hash[l].n_cached = S
        self.seq_len = S if lengths is None else max(lengths)
        self.lengths = lengths

    # ------------------------------------------------------------------ one decode step
    def decode_step(self, tokens: torch.Tensor, advance: bool = True, dense: bool = False, device_pos: bool = False) -> torch.Tensor:
        """tokens [B] int64 -> logits [B, vocab].  The new token sits at position `seq_len`; with advance=False the
        step can be replayed (HIP graph) at a fixed context length.  dense=True attends to the whole cache with the
        dense flash-decode kernel instead (the baseline the sparse step is compared with).
        device_pos=True: the position is read from `pos_dev` / `len_dev` on the device instead (every kernel of the step
        takes it from there and sizes its work for the cache capacity), so ONE captured graph serves successive tokens;
        `generate` drives it.  bf16 with 128-wide heads, sparse attention only; `seq_len` is left alone.

        Per layer (bf16, up to 8 sequences): QKV projection with its RMSNorm folded in, ha_rope_append, the attention
        step, output projection with the residual folded in, gate/up projection with its RMSNorm and SwiGLU folded in,
        down projection with the residual folded in.  Other dtypes and batches: the same steps as library calls plus
        ha_rmsnorm and ha_swiglu."""
        B, H, Hkv, d = self.B, self.H, self.Hkv, self.d
        if self.lengths is not None and not device_pos:
            raise RuntimeError("a ragged batch keeps its positions on the device: use generate()")
        pos = self.seq_len
        S = pos + 1
        x = self.embed[tokens]                                            # [B, hidden]
        # the row-streaming kernel against the library GEMM at B = 4: QKV 11.3 us (19.3), output projection 9.5 (19.1),
        # gate/up 40.9 (59.8), down projection 24.7 (25.1), lm_head 174.8 (184.7)
        skinny = self.use_skinny and self.dtype == torch.bfloat16 and B <= 8
        # 16-bit models outside the fused forms keep their roundings: the norm's two (ha_rmsnorm), the projection's own before a
        # residual is added (efficiency/model.py:314-319, :190-191); fp32 has none to keep
        lowp = self.dtype != torch.float32

        def norm(t, weight):
            if not lowp:
                return F.rms_norm(t, (self.hidden,), weight, self.eps)
            out = torch.empty_like(t)
            _ops.rmsnorm(t, weight, self.eps, out)
            return out
        tiled = self._tiled() and "wqkv_t" in self.layers[0]
        for l, p in enumerate(self.layers):
            if skinny:      # RMSNorm rides in the projection that consumes it
                qkv = _ops.linear_skinny(x, p["wqkv"], self.qkv, norm_weight=p["attn_norm"], eps=self.eps)
            elif tiled:
                qkv = _ops.linear_tiled(norm(x, p["attn_norm"]), p["wqkv_t"], self.qkv.shape[1], self.qkv)
            else:
                qkv = F.linear(norm(x, p["attn_norm"]), p["wqkv"])
            hl = self.hash[l]
            if device_pos:
                if dense or d != 128:
                    raise RuntimeError("device_pos steps run the sparse attention on 128-wide heads")
                _ops.rope_encode_step(qkv, H, Hkv, 0, self.inv_freq, self.q_rot, self.k_cache[l], self.v_cache[l], hl.wk, hl.wq,
                                      hl.num_layers, hl.int_dim, hl.final_dim, hl.codes, hl.qcodes, pos_dev=self.pos_dev, arith=hl.arith)
                hl._select_attend(self.q_rot, self.k_cache[l], self.v_cache[l], self.S_cap, self.attn_out, self.len_dev)
            elif dense:
                _ops.rope_append(qkv, H, Hkv, pos, self.inv_freq, self.q_rot, self.k_cache[l], self.v_cache[l])
                _ops.dense_decode(self.q_rot, self.k_cache[l], self.v_cache[l], S, None, hl.sm_scale, self.attn_out, self.ws_dense)
            elif self.fuse_rope and d == 128:
                hl.n_cached = pos       # rotary embedding, cache append and both hashes in one launch
                hl.step_from_qkv(qkv, pos, self.inv_freq, self.q_rot, self.k_cache[l], self.v_cache[l], self.attn_out)
            else:
                _ops.rope_append(qkv, H, Hkv, pos, self.inv_freq, self.q_rot, self.k_cache[l], self.v_cache[l])
                hl.n_cached = pos
                hl.step(self.q_rot.unsqueeze(2), self.k_cache[l], self.v_cache[l], S, self.attn_out)
            if skinny:
                # x lives in one of two buffers from here on (the down projection below adds in place)
                xo = self.x_attn[0 if self.skinny_all else (l + 1) % 2]
                if "wo_t" in p:
                    x = _ops.linear_tiled(self.attn_out.view(B, H * d), p["wo_t"], self.hidden, xo, residual=x)
                else:
                    x = _ops.linear_skinny(self.attn_out.view(B, H * d), p["wo"], xo, residual=x)
                # RMSNorm in front, SwiGLU behind: the gate/up projection writes the activated [B, ffn] directly
                _ops.linear_skinny(x, p["w13"], self.ffn_act, norm_weight=p["ffn_norm"], eps=self.eps, swiglu=True)
            elif tiled:     # residual inside the output projection, SwiGLU inside the gate/up projection
                x = _ops.linear_tiled(self.attn_out.view(B, H * d), p["wo_t"], self.hidden, self.x_attn[0], residual=x)
                _ops.linear_tiled(norm(x, p["ffn_norm"]), p["w13_t"], 2 * self.ffn, self.ffn_act, swiglu=True)
            else:
                if lowp:
                    x = x + F.linear(self.attn_out.view(B, H * d), p["wo"])
                else:
                    x = x.addmm_(self.attn_out.view(B, H * d), p["wo"].t())
                _ops.swiglu(F.linear(norm(x, p["ffn_norm"]), p["w13"]), self.ffn_act)
            if skinny and self.skinny_all and "w2_t" in p:
                x = _ops.linear_tiled(self.ffn_act, p["w2_t"], self.hidden, self.x_attn[1], residual=x)
            elif skinny and self.skinny_all:
                x = _ops.linear_skinny(self.ffn_act, p["w2"], self.x_attn[1], residual=x)
            elif tiled and "w2_t" in p:
                x = _ops.linear_tiled(self.ffn_act, p["w2_t"], self.hidden, self.x_attn[1], residual=x)
            elif lowp and not skinny:
                x = x + F.linear(self.ffn_act, p["w2"])
            else:
                x = x.addmm_(self.ffn_act, p["w2"].t())      # in place: the out-of-place form first copies x into its result
        if advance and not device_pos:
            self.seq_len = S
        if skinny and self.skinny_all:
            return _ops.linear_skinny(x, self.lm_head, self.logits, norm_weight=self.final_norm, eps=self.eps)
        return F.linear(norm(x, self.final_norm), self.lm_head)

    # ------------------------------------------------------------------ greedy generation, one graph for all tokens
    def generate(self, tokens: torch.Tensor, n_new: int, use_graph: bool = True, sampler=None) -> torch.Tensor:
        """Greedy decoding: `tokens` [B] are fed at position `seq_len`, then each step's arg-max, `n_new` steps in all;
        returns the [B, n_new] tokens produced.  `sampler`: a function logits [B, vocab] -> tokens [B] (int64, on the device,
        without a host synchronisation if the loop is to stay free of them) in place of the arg-max, which is what the
        reference's `sample` takes (efficiency/generate.py:44-49).  The protocol of the reference's harness (efficiency/generate.py:68-96,
        `decode_n_tokens`, its step compiled at :340-348): the step is captured ONCE as a HIP graph whose kernels read the position
        from device memory, and replayed per token; between replays only the arg-max and the position increment are
        launched, and nothing waits for the host."""
        B = self.B
        if tokens.shape != (B,):
            raise ValueError(f"tokens must be [{B}]")
        if self.seq_len + n_new > self.S_cap:
            raise ValueError(f"{n_new} more tokens do not fit the cache ({self.seq_len} of {self.S_cap} used)")
        self.tok_dev.copy_(tokens)
        if self.lengths is None:
            self.pos_dev.fill_(self.seq_len)
        else:       # ragged: every sequence continues at its own length
            self.pos_dev.copy_(torch.tensor(self.lengths, dtype=torch.int32))
        torch.add(self.pos_dev, 1, out=self.len_dev)
        out = torch.empty(B, n_new, dtype=torch.int64, device=self.device)
        step = lambda: self.decode_step(self.tok_dev, device_pos=True)
        if use_graph:
            if self._gen_graph is None:     # captured once per allocation: the buffers it names do not change
                # two eager passes on a side stream, as graph capture wants them; they write the slots of the current
                # position, which the first replay writes again with the same values
                side, main = torch.cuda.Stream(device=self.device), torch.cuda.current_stream(self.device)
                side.wait_stream(main)
                with torch.cuda.stream(side):
                    step()
                    step()
                main.wait_stream(side)
                self._gen_graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(self._gen_graph):
                    self._gen_logits = step()      # the graph's own output buffer: every replay leaves its logits there
            run = self._gen_graph.replay
        else:
            def run():
                self._gen_logits = step()
        for i in range(n_new):
            run()
            if sampler is None:
                torch.argmax(self._gen_logits, dim=-1, out=self.tok_dev)
            else:
                self.tok_dev.copy_(sampler(self._gen_logits).reshape(B))
            out[:, i].copy_(self.tok_dev)
            self.pos_dev.add_(1)
            self.len_dev.add_(1)
        self.seq_len += n_new
        if self.lengths is not None:
            self.lengths = [n + n_new for n in self.lengths]
        for hl in self.hash:
            hl.n_cached = self.seq_len
        return out

    # ------------------------------------------------------------------ weights from a transformers Llama
    @classmethod
    def from_hf(cls, model, usa_modules, batch: int, cache_len: int, dtype=torch.bfloat16, device="cuda:0") -> "LlamaShapedDecoder":
        """The decoder for a `transformers` LlamaForCausalLM and the hash modules `load_usa` returned for it (one `USA` per
        layer): same weights, budgets from the model's config (`init_budget`, `heavy_budget`, `recent_budget`, as
        `convert_usa` reads them), caches for `batch` sequences of up to `cache_len` tokens.  Follow with
        `prefill_from_hf` and `generate`."""
        cfg, usa0 = model.config, usa_modules[0]
        if usa0.rehash_every_step:
            raise NotImplementedError("the LSH baseline and CENTER re-hash the whole cache every step: use the patched layer")
        # what this decoder's launches do not express is refused here rather than dropped in silence
        if getattr(cfg, "attention_bias", False) or getattr(cfg, "mlp_bias", False):
            raise NotImplementedError("projections with biases: use the patched model (convert_usa), which calls the modules")
        rot = model.model.rotary_emb
        if float(getattr(rot, "attention_scaling", 1.0)) != 1.0 or getattr(rot, "rope_type", "default") in ("dynamic", "longrope"):
            raise NotImplementedError(f"rotary embedding of type {getattr(rot, 'rope_type', '?')!r} (scaled cos/sin, or frequencies that "
                                      "change with the length): use the patched model, which takes the model's own cos/sin")
        if getattr(cfg, "hidden_act", "silu") != "silu":
            raise NotImplementedError(f"hidden_act={cfg.hidden_act!r}: the gate/up launch applies SiLU")
        head_dim = getattr(cfg, "head_dim", None) or cfg.hidden_size // cfg.num_attention_heads
        dec = cls(n_layers=cfg.num_hidden_layers, hidden=cfg.hidden_size, ffn=cfg.intermediate_size, n_heads=cfg.num_attention_heads,
                  n_kv_heads=cfg.num_key_value_heads, head_dim=head_dim, vocab=cfg.vocab_size, rms_eps=cfg.rms_norm_eps,
                  n_code_heads=usa0.num_heads, lth_num_layers=usa0.num_layers, lth_int_dim=usa0.int_dim, lth_final_dim=usa0.lth_final_dim,
                  init_budget=cfg.init_budget, recent_budget=cfg.recent_budget, heavy_budget=cfg.heavy_budget, dtype=dtype,
                  device=device, random_init=False)
        dec.load_hf_llama(model)
        lin = lambda seqs: [[(m.weight.detach().float().cpu(), m.bias.detach().float().cpu()) for m in seq if isinstance(m, torch.nn.Linear)]
                            for seq in seqs]
        dec.allocate(batch, cache_len, [UsaWeights(k=lin(u.learning_to_hash_transformation_k), q=lin(u.learning_to_hash_transformation_q))
                                        for u in usa_modules])
        return dec

    def prefill_from_hf(self, model, input_ids: torch.Tensor, attention_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Prefill with the `transformers` model itself (its dense attention: the reference's `q_len > 128` branch,
        hashattention_llama.py:529-550), take over its KV cache and hash the keys.  input_ids [B, S]; prompts of different
        lengths are RIGHT-padded and described by attention_mask [B, S] (ones, then zeros): every sequence then continues
        at its own length.  Returns the first generated token of every sequence [B] (greedy)."""
        from transformers import DynamicCache
        if input_ids.shape[0] != self.B or input_ids.shape[1] + 1 > self.S_cap:
            raise ValueError(f"prompts must be [{self.B}, < {self.S_cap}]")
        lengths = None
        if attention_mask is not None:
            am = attention_mask.to(torch.long).cpu()
            lengths = am.sum(dim=1).tolist()
            ramp = torch.arange(am.shape[1])[None, :] < am.sum(dim=1, keepdim=True)
            if not torch.equal(am.bool(), ramp) or min(lengths) < 1:
                raise ValueError("attention_mask must be ones followed by zeros in every row (right padding), at least one token each")
            attention_mask = attention_mask.to(self.device)
        cache = DynamicCache()
        with torch.no_grad():
            logits = model(input_ids.to(self.device), attention_mask=attention_mask, past_key_values=cache, use_cache=True).logits
        if lengths is None:
            last = logits[:, -1]
        else:
            last = logits[torch.arange(self.B, device=logits.device), torch.tensor(lengths, device=logits.device) - 1]
        self.load_cache([cache.layers[l].keys.to(self.dtype) for l in range(self.L)],
                        [cache.layers[l].values.to(self.dtype) for l in range(self.L)], lengths)
        return last.argmax(-1)

    def load_hf_llama(self, model) -> None:
        """Copy the weights of a `transformers` LlamaForCausalLM of the same shape (used by the plumbing test)."""
        sd = model.state_dict()
        self._gen_graph = self._gen_logits = None       # a captured generation step names the old weight buffers
        cast = lambda t: t.detach().to(self.device, self.dtype)
        self.embed = cast(sd["model.embed_tokens.weight"])
        self.lm_head = cast(sd["lm_head.weight"])
        self.final_norm = cast(sd["model.norm.weight"])
        # the model's own rotary frequencies: a buffer, so a dtype round trip of the model (`.bfloat16().float()`) has
        # rounded them, and the cache it filled was rotated with the rounded values
        self.inv_freq = model.model.rotary_emb.inv_freq.detach().to(self.device, torch.float32)
        for l, p in enumerate(self.layers):
            pre = f"model.layers.{l}."
            p["attn_norm"] = cast(sd[pre + "input_layernorm.weight"])
            p["ffn_norm"] = cast(sd[pre + "post_attention_layernorm.weight"])
            p["wqkv"] = torch.cat([cast(sd[pre + f"self_attn.{n}_proj.weight"]) for n in "qkv"], dim=0)
            p["wo"] = cast(sd[pre + "self_attn.o_proj.weight"])
            p["w13"] = torch.cat([cast(sd[pre + "mlp.gate_proj.weight"]), cast(sd[pre + "mlp.up_proj.weight"])], dim=0)
            p["w2"] = cast(sd[pre + "mlp.down_proj.weight"])
        if getattr(self, "B", 0):
            self._pack_tiles()

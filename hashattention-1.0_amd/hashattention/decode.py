"""Per-layer state and launch sequence of the sparse decode step.

`HashDecodeLayer` owns what the reference's patched attention layer recomputes from scratch every step
(hashattention/hashattention_llama.py:401-446, 578-615): the packed hash-MLP weights and the bit-cache of
key codes, plus the index lists and workspaces of the kernels.  One decode step is

    windows  attention over sink | recent, second stream    (ha_window_partial, overlaps the next two)
    encode   code of the new key -> bit-cache, query codes  (ha_encode_step, one launch)
    select   Hamming histograms per 4096-token chunk        (ha_select_histogram; ha_select_prepare adds the
                                                               per-row thresholds for rows of more than 64 chunks)
    attend   threshold per row, index list rebuilt in LDS   (ha_sparse_decode_fused)
             from the codes, gather-only attention over it
or, for threshold mode and lists above 8192 entries, ha_select (histogram, threshold, ordered compaction into
memory) + ha_sparse_decode (ha_sparse_decode_heavy merged with the window partial when overlap_windows is on).

All buffers are allocated once per (batch, capacity) and reused: the step itself allocates nothing.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from . import _ops


class HashDecodeLayer:
    def __init__(self, k_layers, q_layers, n_q_heads: int, n_kv_heads: int, head_dim: int, num_layers: int, int_dim: int,
                 final_dim: int, init_budget: int, recent_budget: int, heavy_budget: float, eval_mode: str = "simple",
                 retrieve_depth: float = 0, arith: int = _ops.HA_ARITH_F32, device="cuda:0"):
        """k_layers / q_layers: per head, the list of (W [out,in], b [out]) of its hash MLP.  len(k_layers) is the
        number of code heads: n_q_heads (one K MLP per query head, as the reference builds it) or n_kv_heads."""
        self.H, self.Hkv, self.d = n_q_heads, n_kv_heads, head_dim
        self.Hc = len(k_layers)
        if self.Hc not in (n_q_heads, n_kv_heads) and n_q_heads % self.Hc != 0:
            raise ValueError("number of K hash MLPs must divide the number of query heads")
        self.num_layers, self.int_dim, self.final_dim = num_layers, int_dim, final_dim
        self.W = final_dim // 32
        self.init_budget, self.recent_budget, self.heavy_budget = int(init_budget), int(recent_budget), float(heavy_budget)
        self.mode = _ops.HA_SELECT_SIMPLE if eval_mode == "simple" else _ops.HA_SELECT_THRESHOLD
        self.depth = int(math.floor(retrieve_depth))
        self.arith = arith
        self.select_algo = _ops.HA_SELECT_ALGO_AUTO
        # attend to sink | recent on a second stream while the selection runs.  Off by default: at 64K-token rows the
        # windows are already served from L2 to the heads of a group and the fork/join costs more than it hides.
        self.overlap_windows = False
        # rebuild the index list in LDS inside the attend launch instead of writing it to memory (simple mode, lists of
        # up to 8192 entries; decided per allocation)
        self.use_fused = True
        self.fused_min_rows = 32
        self.device = torch.device(device)
        self.wk = _ops.pack_usa_weights(k_layers, self.device)
        self.wq = _ops.pack_usa_weights(q_layers, self.device)
        self.wk_bf16 = None
        if head_dim == 128 and int_dim == 128 and k_layers[0][0][0].shape[1] == 128:
            self.wk_bf16 = _ops.pack_usa_weights_bf16(k_layers, self.device)
        self.sm_scale = 1.0 / math.sqrt(head_dim)
        self.B = self.S_cap = 0
        self.n_cached = 0          # tokens of every sequence already in the bit-cache (uniform batches)

    # ------------------------------------------------------------------ buffers
    def heavy_count(self, s: int) -> int:
        hb = self.heavy_budget
        return int(hb) if hb > 1.0 else int(s * hb)

    def index_capacity(self, s_max: int) -> int:
        if self.mode != _ops.HA_SELECT_SIMPLE:
            return s_max                                    # threshold mode keeps all ties: no a-priori bound
        return min(s_max, self.init_budget + self.recent_budget + self.heavy_count(s_max))

    def allocate(self, B: int, S_cap: int) -> None:
        """(Re)allocate the bit-cache and scratch for batch B and at least S_cap cached tokens (rounded up to whole groups of
        64: the selection kernels read four codes per 128-bit load only from rows that hold whole groups of four, and fall
        back to single loads otherwise - a third slower at 16 x 65536 tokens)."""
        dev = self.device
        S_cap = -(-int(S_cap) // 64) * 64
        self.B, self.S_cap = B, S_cap
        self.codes = torch.zeros(B, self.Hc, S_cap, self.W, dtype=torch.int32, device=dev)
        self.qcodes = torch.zeros(B, self.H, 1, self.W, dtype=torch.int32, device=dev)
        self.idx_cap = self.index_capacity(S_cap)
        # zero-filled: the fused path never writes the lists, and a gather over lists that were never selected must
        # stay inside the cache
        self.idx = torch.zeros(B, self.H, self.idx_cap, dtype=torch.int32, device=dev)
        self.counts = torch.zeros(B, self.H, dtype=torch.int32, device=dev)
        self.ws_select = _ops.workspace(_ops.select_workspace_bytes(B, self.H, self.Hc, self.W, S_cap), dev)
        self.ws_attend = _ops.workspace(_ops.sparse_decode_workspace_bytes(B, self.H, self.idx_cap), dev)
        # measured: with the thresholds derived in the attention launch the fused path is ahead from 32 rows on (a row
        # is then cut into up to 8 pieces: 39.2 against 45 us at B = 1, 32K tokens; 84.1 against 86.5 us at B = 4, 128K)
        self.fused_ok = B * self.H >= self.fused_min_rows and _ops.fused_applies(B, self.H, self.Hc, self.W, S_cap, self.init_budget,
                                                                 self.recent_budget, self.heavy_budget, self.mode)
        # rows of up to 64 chunks: the attention launch derives the thresholds itself, the step is three launches
        self.local_thresholds = _ops.fused_local_thresholds(B, self.Hc, S_cap)
        self.ws_fused = _ops.workspace(_ops.sparse_decode_fused_workspace_bytes(B, self.H, self.Hc, S_cap), dev)
        self.win = torch.empty(B, self.H, 130, dtype=torch.float32, device=dev)
        self.side_stream = torch.cuda.Stream(device=dev)
        self.n_cached = 0
        self._chunk = None          # the chunk buffers are shaped by the batch

    def reset(self) -> None:
        """Forget the cached codes (a new prompt starts); buffers are kept."""
        self.n_cached = 0

    # ------------------------------------------------------------------ stages
    def encode_keys(self, k: torch.Tensor, pos0: int = 0, pos_dev: Optional[torch.Tensor] = None, use_mfma: bool = False) -> None:
        """k [B, Hkv, T, d]: codes of T keys per sequence into bit-cache positions pos0.. (or pos_dev[b]..)."""
        if use_mfma:
            if self.wk_bf16 is None or k.dtype != torch.bfloat16:
                raise ValueError("the MFMA encoder needs bf16 keys and 128-wide MLP layers")
            _ops.encode_pack_prefill(k, self.wk_bf16, self.num_layers, self.int_dim, self.final_dim, self.codes, pos0, pos_dev)
        else:
            _ops.encode_pack(k, self.wk, self.num_layers, self.int_dim, self.final_dim, self.codes, pos0, pos_dev, self.arith)

    # from this many keys per sequence on, a bulk encode goes to the matrix cores (below, the latency-built kernel wins)
    BULK_MIN_TOKENS = 256

    def encode_keys_bulk(self, k: torch.Tensor, pos0: int = 0, pos_dev: Optional[torch.Tensor] = None) -> None:
        """`encode_keys` for the keys a prefill left behind: on the matrix cores in the arithmetic of the hash module -
        bf16 MFMA for a module kept in bf16 (bf16 keys), fp32 MFMA for a module kept in fp32 - when the MLP is 128 wide
        throughout; the scalar kernel otherwise and for a handful of keys."""
        wide = self.wk_bf16 is not None and k.shape[2] >= self.BULK_MIN_TOKENS     # 128-wide layers: the MFMA shapes
        if wide and self.arith == _ops.HA_ARITH_BF16 and k.dtype == torch.bfloat16:
            _ops.encode_pack_prefill(k, self.wk_bf16, self.num_layers, self.int_dim, self.final_dim, self.codes, pos0, pos_dev)
        elif wide and self.arith == _ops.HA_ARITH_F32:
            _ops.encode_pack_prefill_f32(k, self.wk, self.num_layers, self.int_dim, self.final_dim, self.codes, pos0, pos_dev)
        else:
            _ops.encode_pack(k, self.wk, self.num_layers, self.int_dim, self.final_dim, self.codes, pos0, pos_dev, self.arith)

    def encode_query(self, q: torch.Tensor) -> None:
        """q [B, H, 1, d] -> self.qcodes."""
        _ops.encode_pack(q, self.wq, self.num_layers, self.int_dim, self.final_dim, self.qcodes, 0, None, self.arith)

    def select(self, max_seq_len: int, seq_lens: Optional[torch.Tensor]) -> None:
        _ops.select(self.codes, self.qcodes.view(self.B, self.H, self.W), max_seq_len, seq_lens, self.init_budget,
                    self.recent_budget, self.heavy_budget, self.idx, self.counts, self.ws_select, self.mode, self.depth,
                    self.select_algo)

    def select_prepare(self, max_seq_len: int, seq_lens: Optional[torch.Tensor]) -> None:
        if self.local_thresholds:
            _ops.select_histogram(self.codes, self.qcodes.view(self.B, self.H, self.W), max_seq_len, seq_lens, self.init_budget,
                                  self.recent_budget, self.ws_select)
            return
        _ops.select_prepare(self.codes, self.qcodes.view(self.B, self.H, self.W), max_seq_len, seq_lens, self.init_budget,
                            self.recent_budget, self.heavy_budget, self.counts, self.ws_select, self.mode, self.depth)

    def attend_fused(self, q3: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, max_seq_len: int,
                     seq_lens: Optional[torch.Tensor], masked_prefix: Optional[torch.Tensor] = None) -> None:
        _ops.sparse_decode_fused(q3, k, v, self.codes, self.qcodes.view(self.B, self.H, self.W), max_seq_len, seq_lens,
                                 self.init_budget, self.recent_budget, self.heavy_budget, self.ws_select, self.sm_scale, out,
                                 self.ws_fused, thresholds_ready=not self.local_thresholds, out_counts=self.counts,
                                 masked_prefix=masked_prefix)

    def attend(self, q3: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor,
               attn_mask: Optional[torch.Tensor] = None) -> None:
        _ops.sparse_decode(q3, k, v, self.idx, self.counts, self.sm_scale, out, self.ws_attend, mask=attn_mask)

    # ------------------------------------------------------------------ one decode step
    def step(self, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, seq_len: int, out: torch.Tensor,
             seq_lens: Optional[torch.Tensor] = None, n_new: int = 1,
             hash_inputs: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
             attn_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """q [B, H, 1, d]; k_cache/v_cache [B, Hkv, >=seq_len, d] already holding the new token(s) at the end.

        Uniform batches: the last `n_new` tokens (positions seq_len - n_new ..) are encoded and appended to the
        bit-cache; everything before must already be there (`encode_keys` at prefill).  Ragged batches pass
        `seq_lens` (int32 [B], lengths including the new token) and `seq_len` = their maximum.
        `hash_inputs` = (keys [B, Hkv, >=seq_len, d'], queries [B, H, 1, d']): what the hash MLPs read when that is not the
        cache and the query themselves (standardised or lifted vectors; uniform batches only).
        `attn_mask` fp32 [B, >= seq_len]: added to the scaled score of the token at each position before the softmax (the
        padding mask of a batch); the selection does not see it.  Takes the list-fed attention launch.
        """
        q3 = q[:, :, 0, :]
        k_hash, q_hash3 = (k_cache, q3) if hash_inputs is None else (hash_inputs[0], hash_inputs[1][:, :, 0, :])
        if hash_inputs is not None and seq_lens is not None:
            raise ValueError("hash_inputs are supported for uniform batches only")
        main = torch.cuda.current_stream(self.device)
        if self.overlap_windows:
            # fork: the sink and recent windows need no selection, so their share of the attention runs on a second
            # stream under the (latency-bound) encode and select launches; joined before the heavy tokens are attended
            self.side_stream.wait_stream(main)
            with torch.cuda.stream(self.side_stream):
                _ops.window_partial(q3, k_cache, v_cache, seq_len, seq_lens, self.init_budget, self.recent_budget,
                                    self.sm_scale, self.win)
        if seq_lens is None:
            if self.n_cached + n_new != seq_len:
                raise RuntimeError(f"bit-cache holds {self.n_cached} tokens, step at length {seq_len} appends {n_new}")
            if n_new > 1:       # a short multi-token append: older tokens first, the newest rides with the query
                self.encode_keys(k_hash[:, :, seq_len - n_new:seq_len - 1], pos0=seq_len - n_new)
            _ops.encode_step(k_hash[:, :, seq_len - 1:seq_len], q_hash3, self.wk, self.wq, self.num_layers, self.int_dim,
                             self.final_dim, self.codes, self.qcodes, pos0=seq_len - 1, arith=self.arith)
            self.n_cached = seq_len
        else:
            # ragged: the new key of sequence b sits at seq_lens[b] - 1 and is read from the cache in place
            _ops.encode_step_cached(k_cache, q3, self.wk, self.wq, self.num_layers, self.int_dim, self.final_dim, self.codes,
                                    self.qcodes, seq_lens, arith=self.arith)
        return self._select_attend(q3, k_cache, v_cache, seq_len, out, seq_lens, main, attn_mask)

    def _select_attend(self, q3, k_cache, v_cache, seq_len, out, seq_lens, main=None, attn_mask=None):
        """attn_mask: fp32 [B, >= seq_len] added to the scores, or an object that describes the mask of a left-padded batch -
        `.prefix` int32 [B] (tokens below it are blocked) and `.table()` for the fp32 form: the fused launch takes the
        prefix, every other path the table."""
        if attn_mask is not None and not torch.is_tensor(attn_mask):
            if attn_mask.prefix is not None and self.use_fused and self.fused_ok and not self.overlap_windows:
                self.select_prepare(seq_len, seq_lens)
                self.attend_fused(q3, k_cache, v_cache, out, seq_len, seq_lens, masked_prefix=attn_mask.prefix)
                return out
            attn_mask = attn_mask.table()
        if attn_mask is not None:
            if self.overlap_windows:
                raise RuntimeError("an attention mask is not supported together with the second-stream window partial")
            if attn_mask.dim() != 2 or attn_mask.shape[0] != self.B or attn_mask.shape[1] < seq_len:
                raise ValueError(f"attn_mask must be [B={self.B}, >= {seq_len}], got {tuple(attn_mask.shape)}")
            self.select(seq_len, seq_lens)
            self.attend(q3, k_cache, v_cache, out, attn_mask)
            return out
        if self.use_fused and self.fused_ok and not self.overlap_windows:
            self.select_prepare(seq_len, seq_lens)
            self.attend_fused(q3, k_cache, v_cache, out, seq_len, seq_lens)
            return out
        self.select(seq_len, seq_lens)
        if self.overlap_windows:
            main.wait_stream(self.side_stream)
            _ops.sparse_decode_heavy(q3, k_cache, v_cache, self.idx, self.counts, self.sm_scale, out, self.ws_attend, self.win,
                                     self.init_budget, self.recent_budget, seq_len, seq_lens)
        else:
            self.attend(q3, k_cache, v_cache, out)
        return out

    # ------------------------------------------------------------------ a chunk of several new tokens per sequence
    def _chunk_buffers(self, n_rows: int, cap: int, s_max: int, dtype: torch.dtype):
        """Lists, counts, query codes, output rows and workspaces of `chunk_step`, kept between calls and grown when a
        chunk needs more."""
        key = (self.B, n_rows, dtype)      # the query codes [B, H, T, W] and the row lengths depend on B and T separately
        cb = getattr(self, "_chunk", None)
        if cb is None or cb["key"] != key or cb["cap"] < cap or cb["s_max"] < s_max:
            dev = self.device
            cap_a, s_a = max(cap, cb["cap"] if cb and cb["key"] == key else 0), max(s_max, self.S_cap)
            cb = dict(key=key, cap=cap_a, s_max=s_a,
                      qc=torch.zeros(self.B, self.H, n_rows // self.B, self.W, dtype=torch.int32, device=dev),
                      qc_rows=torch.zeros(n_rows, self.H, self.W, dtype=torch.int32, device=dev),
                      idx=torch.zeros(n_rows, self.H, cap_a, dtype=torch.int32, device=dev),
                      cnt=torch.zeros(n_rows, self.H, dtype=torch.int32, device=dev),
                      out=torch.empty(n_rows, self.H, self.d, dtype=dtype, device=dev),
                      q_rows=torch.empty(n_rows, self.H, self.d, dtype=dtype, device=dev),
                      lens=torch.zeros(n_rows, dtype=torch.int32, device=dev),
                      ramp=torch.arange(n_rows, dtype=torch.int32, device=dev) % (n_rows // self.B),
                      ws_s=_ops.workspace(_ops.select_workspace_bytes(n_rows, self.H, self.Hc, self.W, s_a), dev),
                      ws_a=_ops.workspace(_ops.sparse_decode_workspace_bytes(n_rows, self.H, cap_a), dev))
            self._chunk = cb
        return cb

    def chunk_step(self, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, seq_len: int, out: torch.Tensor,
                   heavy_budget: float, q_hash: Optional[torch.Tensor] = None, attn_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """q [B, H, T, d]: T new query tokens per sequence (1 < T <= 128) whose keys are already in the caches and in the
        bit-cache (`encode_keys`); row i attends as the query at position seq_len - T + i with its own causal windows
        (hashattention_llama.py:423-428).  Three launches for the whole batch: the query codes, ONE selection and ONE
        attention over the B * T rows (`ha_select_rows`, `ha_sparse_decode_rows`).  out [B, H, T, d].
        `q_hash`: what the query-side hash MLPs read when that is not q itself; attn_mask fp32 [B, T, >= seq_len]."""
        B, H, T, d = q.shape
        S = seq_len
        n_rows = B * T
        cap = S if self.mode != _ops.HA_SELECT_SIMPLE else max(1, min(S, self.init_budget + self.recent_budget + self.heavy_count(S)))
        cb = self._chunk_buffers(n_rows, cap, S, q.dtype)
        qh = q if q_hash is None else q_hash
        _ops.encode_pack(qh, self.wq, self.num_layers, self.int_dim, self.final_dim, cb["qc"], 0, None, self.arith)
        cb["qc_rows"].view(B, T, H, self.W).copy_(cb["qc"].transpose(1, 2))
        cb["q_rows"].view(B, T, H, d).copy_(q.transpose(1, 2))
        torch.add(cb["ramp"], S - T + 1, out=cb["lens"])                    # row (b, i) sees keys [0, S - T + i]
        _ops.select_rows(self.codes, cb["qc_rows"], T, S, cb["lens"], self.init_budget, self.recent_budget, heavy_budget,
                         cb["idx"], cb["cnt"], cb["ws_s"], self.mode, self.depth)
        mask = None if attn_mask is None else attn_mask.reshape(n_rows, attn_mask.shape[-1])
        _ops.sparse_decode_rows(cb["q_rows"], k_cache, v_cache, T, cb["idx"], cb["cnt"], self.sm_scale, cb["out"], cb["ws_a"], mask=mask)
        out.copy_(cb["out"].view(B, T, H, d).transpose(1, 2))
        return out

    def step_from_qkv(self, qkv: torch.Tensor, pos: int, inv_freq: torch.Tensor, q_rot: torch.Tensor, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """The decode step of a uniform batch straight from the fused QKV projection of the new token, qkv [B, (H + 2 Hkv) * 128]:
        rotary embedding at position `pos`, cache append, hashing of the new key and of the query in ONE launch
        (ha_rope_encode_step), then selection and attention as in `step`.  q_rot [B, H, 128] receives the rotated query."""
        if self.overlap_windows:
            raise RuntimeError("step_from_qkv does not run the second-stream window partial: use rope_append + step")
        if self.n_cached != pos:
            raise RuntimeError(f"bit-cache holds {self.n_cached} tokens, the new token sits at position {pos}")
        _ops.rope_encode_step(qkv, self.H, self.Hkv, pos, inv_freq, q_rot, k_cache, v_cache, self.wk, self.wq, self.num_layers,
                              self.int_dim, self.final_dim, self.codes, self.qcodes, arith=self.arith)
        self.n_cached = pos + 1
        return self._select_attend(q_rot, k_cache, v_cache, pos + 1, out, None)

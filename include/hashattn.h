/*
 * hashattn.h - C ABI of the MI355X (gfx950) HashAttention sparse-decode library.
 *
 * The reference (xAlg-ai/HashAttention-1.0) has no FFI: its boundary is the Python module API
 * `load_usa` / `convert_usa` (hashattention/hashattention_llama.py:633-667) whose patched attention
 * layer runs the decode branch (:551-631) in eager PyTorch.  This header is what the patched layer
 * of this build binds through ctypes instead; each entry names the reference code it replaces.
 *
 * Conventions
 *   - every function returns HA_OK (0) or a negative ha_status; nothing throws or aborts;
 *   - arguments are validated before the first HIP call, so bad arguments are reported
 *     identically with or without a GPU; ha_last_error_string() holds the detail (thread-local);
 *   - all pointers are device pointers unless named host_*; `stream` is a hipStream_t (NULL = the
 *     null stream); calls are stream-ordered, never synchronise, never allocate: the caller owns
 *     every buffer including workspaces (sized by the *_workspace_bytes functions);
 *   - strides are in ELEMENTS of the tensor's type; the innermost dimension is contiguous;
 *   - head_dim is 128; codes are W = 1 or 2 uint32 words per token (32- or 64-bit hashes);
 *   - dtype codes: HA_F32, HA_BF16, HA_F16.
 */
#ifndef HASHATTN_H
#define HASHATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HA_VERSION 202 /* 0.2.2: + ha_sparse_decode_fused_prefix_masked, ha_rmsnorm, ha_linear_tiled (+ ha_pack_weight_tiles); the dense baseline and the window partial take any number of query heads per KV head; 0.2.1: ha_linear_skinny[_fused] round as the modules they replace (two roundings per RMSNorm, the product's before a residual); 0.2.0: + ha_sparse_decode_paged, ha_sparse_decode_fused_paged, ha_rope_encode_step_cos_sin */

typedef enum ha_status {
    HA_OK = 0,
    HA_ERR_NULL_POINTER = -1,
    HA_ERR_BAD_SHAPE = -2,      /* a size, head count, word count or budget outside what the kernels support */
    HA_ERR_BAD_DTYPE = -3,
    HA_ERR_MISALIGNED = -4,     /* pointer or stride not aligned for 128-bit row loads */
    HA_ERR_WORKSPACE = -5,      /* workspace missing or smaller than *_workspace_bytes() */
    HA_ERR_NO_DEVICE = -6,      /* no HIP device visible to this process */
    HA_ERR_HIP = -7             /* a HIP runtime call or kernel launch failed */
} ha_status;

#define HA_F32 0
#define HA_BF16 1
#define HA_F16 2

#define HA_ARITH_F32 0  /* hash MLP in fp32 FMA chains (module kept in fp32) */
#define HA_ARITH_BF16 1 /* activations rounded to bf16 after every Linear and SiLU (module kept in bf16) */

#define HA_SELECT_SIMPLE 0    /* usa_eval_mode == 'simple': exactly k_eff heavy tokens */
#define HA_SELECT_THRESHOLD 1 /* otherwise: every candidate within the distance threshold, ties included */

/* How ha_select finds the threshold; every choice returns the same lists. */
#define HA_SELECT_ALGO_AUTO 0              /* the library's choice (currently the histogram method) */
#define HA_SELECT_ALGO_HISTOGRAM 1         /* two passes over the codes: exact histogram, then compaction */
#define HA_SELECT_ALGO_SAMPLED 2           /* sampled upper bound of the threshold, one filtering pass, exact finish */
#define HA_SELECT_ALGO_SAMPLED_EXACT_ROWS 3 /* diagnostic: as SAMPLED with every row sent through its in-kernel exact path */

int ha_version(void);
const char *ha_status_string(int status);
const char *ha_last_error_string(void);
/* number of HIP devices visible (0 without a GPU); never fails */
int ha_device_count(void);

/* ---------------------------------------------------------------------------------------------
 * Hash-MLP weights.  One head's MLP is 1-3 Linear layers head_dim -> int_dim (-> int_dim) ->
 * final_dim with SiLU between them (USA.__init__, hashattention_llama.py:99-128).  The kernels read
 * a packed fp32 blob per head, 16-byte aligned: for each layer the weights, then bias [out].  A layer
 * with a multiple of 16 inputs stores W transposed with its inputs in groups of four, [in / 4][out][4]:
 * W[o][k] sits at ((k / 4) * out + o) * 4 + k % 4, so that the lanes of a wave (consecutive outputs) fetch
 * consecutive 16-byte pieces; any other layer stores plain W^T [in][out] (W[o][k] at k * out + o).
 * ha_usa_packed_floats() is the blob length of ONE head; heads are concatenated.
 * Limits: head_dim, int_dim <= 256 and multiples of 4; final_dim in {32, 64}.
 */
int64_t ha_usa_packed_floats(int n_layers, int head_dim, int int_dim, int final_dim);

/*
 * Encode rows through the per-head hash MLP and pack sign bits: bit i of a code = (logit_i > 0),
 * least significant bit = output dim 0.  Replaces USA.k_embedding / q_embedding and the MLP +
 * sign of USA.forward (hashattention_llama.py:159-173, 204-226) and the bit packing of
 * efficiency/kernels/torchatt.py:55-56, 159, 183-184.
 *
 *   x        [B, x_heads, T, head_dim] of x_dtype, strides x_stride_{b,h,t}
 *   weights  packed blob of n_heads heads; MLP head i reads x head i / (n_heads / x_heads)
 *   codes    [B, n_heads, ., W] uint32, strides c_stride_{b,h} in words; token t of sequence b is
 *            written at position pos0 + t, or pos_dev[b] + t when pos_dev (int32 [B]) is given:
 *            this is the append into the per-layer bit-cache; a position taken from pos_dev that lies outside the row
 *            (negative, or beyond the c_stride_h / W tokens a row spans) is written nowhere
 *   logits   optional fp32 [B, n_heads, T, final_dim] contiguous (tests, diagnostics); may be NULL
 */
int ha_encode_pack(const void *x, int x_dtype, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t,
                   int B, int x_heads, int n_heads, int T,
                   const float *weights, int n_layers, int head_dim, int int_dim, int final_dim, int arith,
                   uint32_t *codes, int64_t c_stride_b, int64_t c_stride_h, int pos0, const int32_t *pos_dev,
                   float *logits, void *stream);

/*
 * The encode of one decode step in a single launch: the newest key of every sequence is appended to
 * the bit-cache (as ha_encode_pack with T = 1) and the query codes are written to qcodes [B, H, W].
 * Replaces the q_embedding / k_embedding pair of the cached branch of compute_mask_multi
 * (hashattention_llama.py:411-414).
 *   k_new [B, Hkv, 1, head_dim], q [B, H, head_dim] (strides q_stride_{b,h}), both of x_dtype
 *   weights_k: Hc heads, weights_q: H heads (packed as for ha_encode_pack)
 */
int ha_encode_step(const void *k_new, int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_t,
                   const void *q, int64_t q_stride_b, int64_t q_stride_h, int x_dtype,
                   int B, int Hkv, int Hc, int H, int T_new,
                   const float *weights_k, const float *weights_q,
                   int n_layers, int head_dim, int int_dim, int final_dim, int arith,
                   uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, int pos0, const int32_t *pos_dev,
                   uint32_t *qcodes, void *stream);

/*
 * ha_encode_step for a batch whose lengths live on the device: the newest key of sequence b is read from the
 * cache itself, row seq_lens[b] - 1 of k_cache [B, Hkv, ., head_dim] (strides k_stride_{b,h,s}), and its code is
 * written to the same position of the bit-cache; no host-side gather of the new rows.  A sequence of length 0
 * writes nothing.  Same reference lines as ha_encode_step (hashattention_llama.py:411-414).
 */
int ha_encode_step_cached(const void *k_cache, int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s,
                          const void *q, int64_t q_stride_b, int64_t q_stride_h, int x_dtype,
                          int B, int Hkv, int Hc, int H, const int32_t *seq_lens,
                          const float *weights_k, const float *weights_q,
                          int n_layers, int head_dim, int int_dim, int final_dim, int arith,
                          uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, uint32_t *qcodes, void *stream);

/*
 * Bulk (prefill) encode on the matrix cores: the same mapping as ha_encode_pack in HA_ARITH_BF16
 * arithmetic, computed as three chained bf16 MFMA GEMMs per 128-token tile.  x must be bf16,
 * head_dim == int_dim == 128.  `weights_bf16` is the blob of ha_usa_packed_floats() elements per
 * head converted to bf16 in the NATIVE nn.Linear orientation: per layer W [out][in], then bias [out].
 * Replaces the un-timed prefill encode of efficiency/kernels/torchatt.py:183-184.
 */
int ha_encode_pack_prefill(const void *x, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t,
                           int B, int x_heads, int n_heads, int T,
                           const void *weights_bf16, int n_layers, int head_dim, int int_dim, int final_dim,
                           uint32_t *codes, int64_t c_stride_b, int64_t c_stride_h, int pos0, const int32_t *pos_dev,
                           void *stream);

/*
 * Bulk (prefill) encode for hash modules kept in fp32 (what load_usa returns, hashattention_llama.py:640-646; the layer
 * casts the keys to the module's dtype, :406): the mapping of ha_encode_pack in HA_ARITH_F32, computed as chained fp32
 * MFMA GEMMs per 256-token tile.  x of x_dtype (bf16 / fp16 rows are widened exactly), head_dim == int_dim == 128,
 * `weights` the same packed fp32 blob ha_encode_pack reads.  The matrix core sums in its own order, so a sign bit can
 * differ from ha_encode_pack's where the logit is within fp32 rounding of zero.  Replaces the same un-timed prefill
 * encode (efficiency/kernels/torchatt.py:183-184) as ha_encode_pack_prefill.
 */
int ha_encode_pack_prefill_f32(const void *x, int x_dtype, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t,
                               int B, int x_heads, int n_heads, int T,
                               const float *weights, int n_layers, int head_dim, int int_dim, int final_dim,
                               uint32_t *codes, int64_t c_stride_b, int64_t c_stride_h, int pos0, const int32_t *pos_dev,
                               void *stream);

/*
 * Hamming distance of every cached code to the query code: scores[b, h, j] =
 * popcount(kcodes[b, h / (H/Hc), j] ^ qcodes[b, h]) for j < seq_len[b] (any number of query heads per code head:
 * the t query tokens of USA.forward are t * H "heads").  Diagnostic/test entry;
 * ha_select fuses this.  Replaces efficiency/kernels/bit_count_uint32.py:4-33, bit_count_long.py:4-33
 * and the xor of torchatt.py:58 (span = final_dim - 2 * distance, hashattention_llama.py:180-187).
 *   kcodes [B, Hc, ., W] strides kc_stride_{b,h} words; qcodes [B, H, W] contiguous;
 *   seq_lens int32 [B] or NULL (all = max_seq_len); scores uint8 [B, H, max_seq_len] contiguous.
 */
int ha_hamming_score(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes,
                     int B, int H, int Hc, int W, int max_seq_len, const int32_t *seq_lens,
                     uint8_t *scores, void *stream);

/*
 * Token selection for one decode query per sequence.  For sequence length S: candidates are
 * j in [init, S - recent); k_eff = min(heavy, #candidates) with heavy = (heavy_budget > 1) ?
 * (int)heavy_budget : (int)(S * heavy_budget); the k_eff candidates of smallest Hamming distance
 * (ties: lowest index) are kept together with the sink [0, init) and recent [S - recent, S)
 * windows.  HA_SELECT_THRESHOLD keeps every candidate with distance <=
 * min(d_min + depth, d_(k_eff)) instead.  Replaces compute_mask_multi / compute_mask
 * (hashattention_llama.py:401-493; the sort at :430) and torch.topk of torchatt.py:46, 66.
 *
 *   out_idx    int32 [B, H, idx_cap]: ascending token indices; nothing is written past idx_cap
 *   out_counts int32 [B, H]: number selected (the true count, even if it exceeds idx_cap)
 *   workspace  ha_select_workspace_bytes(...) bytes, 256-byte aligned
 * H / Hc (query heads that share one code head) must be 1, 2, 4 or 8, else HA_ERR_BAD_SHAPE; the reference keeps one
 * key-side hash per query head, Hc = H (hashattention_llama.py:642).  The attention entry points take any whole
 * number of query heads per KV head.
 * kc_stride_b may be 0: every batch entry then reads the same codes, i.e. B queries (each with its own row of
 * qcodes and its own seq_lens[b]) against one sequence - the rows of a multi-token chunk
 * (hashattention_llama.py:423-428) or of the recall statistic (:319-398) in one call.
 */
size_t ha_select_workspace_bytes(int B, int H, int Hc, int W, int max_seq_len);
int ha_select(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes,
              int B, int H, int Hc, int W, int max_seq_len, const int32_t *seq_lens,
              int init_budget, int recent_budget, double heavy_budget, int mode, int depth, int algo,
              int32_t *out_idx, int64_t idx_cap, int32_t *out_counts,
              void *workspace, size_t workspace_bytes, void *stream);

/*
 * ha_select and ha_sparse_decode for a chunk of several new tokens per sequence (hashattention_llama.py:423-428: the
 * decode branch takes up to 128 query tokens, each with its own causal windows and budget).  The B batch entries are
 * rows: rows_per_sequence consecutive ones belong to one sequence, i.e. entry n reads the codes (the K/V cache) of
 * sequence n / rows_per_sequence - kc_stride_b and kv_stride_b are strides between SEQUENCES - and has its own query
 * (qcodes [B, H, W], q [B, H, 128]), its own length seq_lens[n] (required), index list, count, output row and, for the
 * attention, its own mask row (mask may be NULL; by token position, as ha_sparse_decode_masked with mask_by_slot = 0).
 * One call serves every row of every sequence: the number of launches of a chunk does not depend on the batch.  The
 * selection uses the histogram method; workspaces are sized for B rows (ha_select_workspace_bytes(B, ...),
 * ha_sparse_decode_workspace_bytes(B, ...)).
 */
int ha_select_rows(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes,
                   int B, int rows_per_sequence, int H, int Hc, int W, int max_seq_len, const int32_t *seq_lens,
                   int init_budget, int recent_budget, double heavy_budget, int mode, int depth,
                   int32_t *out_idx, int64_t idx_cap, int32_t *out_counts,
                   void *workspace, size_t workspace_bytes, void *stream);
int ha_sparse_decode_rows(const void *q, int64_t q_stride_b, int64_t q_stride_h,
                          const void *k, const void *v, int kv_dtype,
                          int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                          int B, int rows_per_sequence, int H, int Hkv,
                          const int32_t *idx, int64_t idx_cap, const int32_t *counts, float sm_scale,
                          const float *mask, int64_t mask_stride_b, int mask_len,
                          void *out, void *workspace, size_t workspace_bytes, void *stream);

/*
 * ha_select without a workspace argument, for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The selection's scratch
 * (chunk histograms, row thresholds, chunk prefixes: what ha_select keeps in its workspace) lives in a device array of
 * ha_select_static_max_bytes() = 8 MiB built into the library, one copy per GPU, held until the process ends.  The call
 * allocates and frees nothing.  Always the histogram method; same lists and counts as ha_select, bit for bit.
 * Shapes whose scratch would not fit (B * H * ceil(max_seq_len / 4096) * (32 W + 3) * 4 bytes, roughly) are refused
 * with HA_ERR_WORKSPACE.  All calls on one GPU share the array: calls that overlap in time on one GPU (two streams or
 * threads) race; calls on one stream are ordered.  The first call on a GPU resolves the array's address
 * (hipGetSymbolAddress): make one call before capturing a graph that contains another.
 */
size_t ha_select_static_max_bytes(void);
int ha_select_static(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes,
                     int B, int H, int Hc, int W, int max_seq_len, const int32_t *seq_lens,
                     int init_budget, int recent_budget, double heavy_budget, int mode, int depth,
                     int32_t *out_idx, int64_t idx_cap, int32_t *out_counts, void *stream);

/*
 * Gather-only decode attention: out[b, h] = softmax(q[b, h] . K[b, h/G, idx] * sm_scale) V[b, h/G, idx]
 * over the first counts[b, h] entries of idx[b, h]; fp32 online softmax, split over the index list
 * and merged by log-sum-exp.  Replaces flash_fwd_sparse / fwd_sparse
 * (efficiency/kernels/flash_fwd_sparse.py:396-554, 775-815; sparse.py:12-187) and the masked dense
 * softmax of hashattention_llama.py:585-615.
 *   q   [B, H, 128] kv_dtype, strides q_stride_{b,h}
 *   k,v [B, Hkv, ., 128] kv_dtype, strides kv_stride_{b,h,s}; rows 16-byte aligned.  Any layout the three strides
 *       describe is read in place: [B, Hkv, S, 128] (the Hugging Face cache) as well as the prototype's token-major
 *       [B * S, H, 128] (torchatt.py:148-151, sparse.py:224-226: kv_stride_b = S * H * 128, kv_stride_h = 128,
 *       kv_stride_s = H * 128)
 *   idx The ORDER of a list is free: ascending (what ha_select writes, best for DRAM locality), torch.topk's score order
 *       (torchatt.py:66-67) or a random permutation (sparse.py:231-233) give the same output up to the order of the fp32
 *       additions.  An index that occurs twice counts twice, as in the reference's kernels.  Entries must lie inside the
 *       cache: they are not range-checked.
 *   out [B, H, 128] kv_dtype contiguous
 *   workspace  ha_sparse_decode_workspace_bytes(...) bytes, 256-byte aligned; calls that share a
 *              workspace must not overlap
 */
size_t ha_sparse_decode_workspace_bytes(int B, int H, int64_t idx_cap);
int ha_sparse_decode(const void *q, int64_t q_stride_b, int64_t q_stride_h,
                     const void *k, const void *v, int kv_dtype,
                     int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                     int B, int H, int Hkv, const int32_t *idx, int64_t idx_cap, const int32_t *counts,
                     float sm_scale, void *out, void *workspace, size_t workspace_bytes, void *stream);

/*
 * ha_sparse_decode with an additive mask: out[b, h] = softmax(q . K[idx] * sm_scale + mask term) V[idx].
 * mask is fp32 [B, mask_len] (row stride mask_stride_b, in elements; 0 shares one row), in natural-log
 * units, one row per sequence shared by its heads; entries of -inf (or the dtype's most negative value,
 * as the reference fills them) remove a list entry from the softmax.
 *   mask_by_slot = 0: the term of a list entry is mask[b, token position] - the `attention_mask` the
 *                     patched layer adds before its softmax (hashattention_llama.py:593-598: padding of a
 *                     batch, on top of the selection); mask_len >= the largest position in the lists
 *                     (positions beyond it read the row's last value);
 *   mask_by_slot = 1: the term is mask[b, place in the list], the `Mask` argument of fwd_sparse
 *                     (efficiency/kernels/sparse.py:14, 46-58, 190-212); mask_len >= idx_cap.
 * A row whose entries are all removed gives a zero output.
 */
int ha_sparse_decode_masked(const void *q, int64_t q_stride_b, int64_t q_stride_h,
                            const void *k, const void *v, int kv_dtype,
                            int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                            int B, int H, int Hkv, const int32_t *idx, int64_t idx_cap, const int32_t *counts,
                            float sm_scale, const float *mask, int64_t mask_stride_b, int mask_len, int mask_by_slot,
                            void *out, void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same attention in two launches that may overlap in time.  The sink [0, init) and recent [S - recent, S)
 * windows are known before any selection is made and are shared by the query heads of a KV group:
 * ha_window_partial attends to them alone (each row read once per KV head) and leaves an unnormalised partial
 * (acc[128], m, l: ha_window_partial_bytes) per (sequence, query head).  It depends only on q, K and V, so a
 * caller can issue it on a second stream while ha_encode_step and ha_select run.  ha_sparse_decode_heavy then
 * takes the index lists of ha_select (same budgets, same seq_lens), skips their window entries and merges the
 * partial: the output equals ha_sparse_decode's up to fp32 summation order.  No counterpart in the reference,
 * whose prototype has no windows at all (efficiency/kernels/torchatt.py:52-71).
 */
size_t ha_window_partial_bytes(int B, int H);
int ha_window_partial(const void *q, int64_t q_stride_b, int64_t q_stride_h,
                      const void *k, const void *v, int kv_dtype,
                      int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                      int B, int H, int Hkv, int max_seq_len, const int32_t *seq_lens,
                      int init_budget, int recent_budget, float sm_scale, float *window_partial, void *stream);
int ha_sparse_decode_heavy(const void *q, int64_t q_stride_b, int64_t q_stride_h,
                           const void *k, const void *v, int kv_dtype,
                           int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                           int B, int H, int Hkv, const int32_t *idx, int64_t idx_cap, const int32_t *counts,
                           float sm_scale, void *out, void *workspace, size_t workspace_bytes,
                           const float *window_partial, int init_budget, int recent_budget,
                           int max_seq_len, const int32_t *seq_lens, void *stream);

/*
 * Selection fused into the attention launch.  ha_select_prepare runs the first two launches of the histogram
 * method only: it leaves in the workspace, per (sequence, query head), the threshold distance T, the number of ties
 * taken and the heavy count, and per 1024..4096-token chunk how many selected tokens precede it, and writes
 * out_counts.  ha_sparse_decode_fused then rebuilds each row's ordered index list in LDS straight from the codes
 * (the same tokens as ha_select's list in another fixed order, so the output equals that of ha_select + ha_sparse_decode
 * up to the order of the fp32 additions) and attends to it: the list never travels through memory and the compaction
 * launch disappears.
 * Budgets, seq_lens and code arguments must be those given to ha_select_prepare; `select_workspace` is the
 * workspace it filled.  With thresholds_ready = 0 the workspace needs only the chunk histograms (ha_select_histogram,
 * the first launch alone): every workgroup of the attention launch derives its row's threshold and prefixes
 * itself and out_counts (may be NULL) is written by that launch - one launch less per step; rows of at most 64
 * chunks (max_seq_len <= 262144, ha_sparse_decode_fused_local_thresholds returns 1).  Only HA_SELECT_SIMPLE, and only while
 * init + recent + heavy <= 8192 entries: a row's list is kept in LDS (ha_sparse_decode_fused_applies returns 1);
 * otherwise use ha_select + ha_sparse_decode.  Replaces the same
 * reference lines as those two (hashattention_llama.py:401-446, 585-615; efficiency/kernels/torchatt.py:52-71).
 */
int ha_select_histogram(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes,
                        int B, int H, int Hc, int W, int max_seq_len, const int32_t *seq_lens,
                        int init_budget, int recent_budget, void *workspace, size_t workspace_bytes, void *stream);
int ha_select_prepare(const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes,
                      int B, int H, int Hc, int W, int max_seq_len, const int32_t *seq_lens,
                      int init_budget, int recent_budget, double heavy_budget, int mode, int depth,
                      int32_t *out_counts, void *workspace, size_t workspace_bytes, void *stream);
int ha_sparse_decode_fused_applies(int B, int H, int Hc, int W, int max_seq_len,
                                   int init_budget, int recent_budget, double heavy_budget, int mode);
int ha_sparse_decode_fused_local_thresholds(int B, int Hc, int max_seq_len);
size_t ha_sparse_decode_fused_workspace_bytes(int B, int H, int Hc, int max_seq_len);
int ha_sparse_decode_fused(const void *q, int64_t q_stride_b, int64_t q_stride_h,
                           const void *k, const void *v, int kv_dtype,
                           int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                           const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes,
                           int B, int H, int Hkv, int Hc, int W, int max_seq_len, const int32_t *seq_lens,
                           int init_budget, int recent_budget, double heavy_budget,
                           const void *select_workspace, size_t select_workspace_bytes,
                           int thresholds_ready, int32_t *out_counts,
                           float sm_scale, void *out, void *workspace, size_t workspace_bytes, void *stream);

/*
 * ha_sparse_decode_fused for a LEFT-PADDED batch: the additive attention mask the reference adds to the scores
 * (hashattention_llama.py:593-598) blocks, for one new token per sequence, exactly the padding in front of each prompt, so
 * it is handed over as one number per sequence: tokens [0, masked_prefix[b]) of sequence b score -inf.  As in the
 * reference the selection does not see the mask: such tokens are counted and listed like any other (out_counts as
 * ha_sparse_decode_fused), they only add nothing to the softmax.  Output equals ha_select + ha_sparse_decode_masked with the
 * mask {-inf below masked_prefix[b], 0 from there on} up to the order of the fp32 additions.  masked_prefix int32 [B] in
 * device memory; every other argument as ha_sparse_decode_fused.  A row whose every listed token is masked gives zeros.
 */
int ha_sparse_decode_fused_prefix_masked(const void *q, int64_t q_stride_b, int64_t q_stride_h,
                                         const void *k, const void *v, int kv_dtype,
                                         int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                                         const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes,
                                         int B, int H, int Hkv, int Hc, int W, int max_seq_len, const int32_t *seq_lens,
                                         int init_budget, int recent_budget, double heavy_budget,
                                         const void *select_workspace, size_t select_workspace_bytes,
                                         int thresholds_ready, int32_t *out_counts, const int32_t *masked_prefix,
                                         float sm_scale, void *out, void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same two attention launches over a cache addressed through a token -> slot table: the row of token j of sequence b
 * is row slot_of_token[b * slot_stride_b + j] of k and v, i.e. it lies at k + b * kv_stride_b + (h / G) * kv_stride_h +
 * slot * kv_stride_s.  This is the `Req_to_tokens [B, S]` table of the reference's sparse flash-decode
 * (efficiency/kernels/flash_fwd_sparse.py:396-470; built at efficiency/kernels/torchatt.py:165), whose K and V are one pool
 * [n_slots, Hkv, 128] shared by all sequences: pass kv_stride_b = 0, kv_stride_h = 128, kv_stride_s = Hkv * 128 for that
 * layout.  Index lists, counts, masks by token position, seq_lens, codes and budgets keep speaking of token POSITIONS; only
 * the K/V row addresses go through the table.  slot_of_token is int32 (the reference: int64), n_slots the number of rows
 * k and v hold per (sequence, KV head) view - slots must lie in [0, n_slots); the fused launch clamps list entries to it.
 *
 * ha_sparse_decode_paged covers ha_sparse_decode, _masked and _rows: mask may be NULL, rows_per_sequence is 1 for one query
 * per sequence (with more, kv_stride_b and slot_stride_b are strides between SEQUENCES, as for ha_sparse_decode_rows).
 * ha_sparse_decode_fused_paged is ha_sparse_decode_fused with the table: the fused launch translates a token when it is
 * placed in the row's LDS list (memory -> LDS requests that overwrite the entry, no register involved) and gathers one
 * scan round behind the selection.  Outputs equal those of the unpaged entry points on the cache the table describes.
 */
int ha_sparse_decode_paged(const void *q, int64_t q_stride_b, int64_t q_stride_h,
                           const void *k, const void *v, int kv_dtype,
                           int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                           int B, int rows_per_sequence, int H, int Hkv,
                           const int32_t *idx, int64_t idx_cap, const int32_t *counts, float sm_scale,
                           const float *mask, int64_t mask_stride_b, int mask_len, int mask_by_slot,
                           const int32_t *slot_of_token, int64_t slot_stride_b, int64_t n_slots,
                           void *out, void *workspace, size_t workspace_bytes, void *stream);
int ha_sparse_decode_fused_paged(const void *q, int64_t q_stride_b, int64_t q_stride_h,
                                 const void *k, const void *v, int kv_dtype,
                                 int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                                 const uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, const uint32_t *qcodes,
                                 int B, int H, int Hkv, int Hc, int W, int max_seq_len, const int32_t *seq_lens,
                                 int init_budget, int recent_budget, double heavy_budget,
                                 const void *select_workspace, size_t select_workspace_bytes,
                                 int thresholds_ready, int32_t *out_counts,
                                 const int32_t *slot_of_token, int64_t slot_stride_b, int64_t n_slots,
                                 float sm_scale, void *out, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Dense flash-decode over all seq_len[b] keys (the baseline the sparse path is compared with).
 * Replaces flash_decode_attention_fwd (efficiency/kernels/flash_fwd_sparse.py:21-321) and
 * torch_attention_naive (efficiency/kernels/torchatt.py:17-30).  Each K/V row is read once per KV
 * head and shared by the query heads of its group.  Workspace rules as for ha_sparse_decode.
 */
size_t ha_dense_decode_workspace_bytes(int B, int H, int max_seq_len);
int ha_dense_decode(const void *q, int64_t q_stride_b, int64_t q_stride_h,
                    const void *k, const void *v, int kv_dtype,
                    int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                    int B, int H, int Hkv, int max_seq_len, const int32_t *seq_lens,
                    float sm_scale, void *out, void *workspace, size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------------------------------------
 * The two elementwise steps of a decoder layer next to the attention step, for a decode loop that wants them as
 * one launch each (the reference's end-to-end harness leaves them to torch.compile: efficiency/model.py:236-250
 * QKV split, rotary embedding and cache update, :88-96 KVCache.update, :304-305 FeedForward).
 *
 * ha_rope_append: qkv [B, >= (H + 2 Hkv) * 128] holds one new token per sequence, heads in the order q | k | v.
 * q and k are rotated in the rotate-half convention (pairs (i, i + 64), transformers' apply_rotary_pos_emb; not
 * the interleaved pairs of efficiency/model.py:333-345) by the angle pos * inv_freq[i], the cos/sin table rounded
 * to `dtype` as transformers does; q goes to q_out [B, H, 128], k and v into the caches at token position `pos`
 * (or pos_dev[b] when pos_dev is not NULL; a sequence whose pos_dev[b] lies outside [0, cache_len) gets its rotated query
 * but no key or value is written for it).  Cache strides in elements.
 * ha_swiglu: out[b, i] = silu(gate_up[b, i]) * gate_up[b, F + i], silu rounded to `dtype` before the product.
 */
int ha_rope_append(const void *qkv, int64_t qkv_stride_b, int dtype, int B, int H, int Hkv, int pos, const int32_t *pos_dev,
                   const float *inv_freq, void *q_out, void *k_cache, void *v_cache,
                   int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int64_t cache_len, void *stream);
int ha_swiglu(const void *gate_up, int64_t gate_up_stride_b, int dtype, int B, int F, void *out, void *stream);
/*
 * RMSNorm of M rows of K elements as one launch: out = round(round(x * rsqrt(mean_k x^2 + eps)) * weight), both roundings
 * to `dtype` - the module of the reference's harness (efficiency/model.py:308-319: `self._norm(x.float()).type_as(x)` times
 * the weight) and transformers' LlamaRMSNorm.  For batches too large for the norm-in-front form of ha_linear_skinny_fused.
 * Strides in elements; `out` must not overlap `x`.
 */
int ha_rmsnorm(const void *x, int64_t x_stride_m, const void *weight, int dtype, int M, int K, float eps,
               void *out, int64_t out_stride_m, void *stream);
/*
 * ha_rope_append followed by ha_encode_step, in one launch: the workgroup that hashes a head also rotates it.  qkv as for
 * ha_rope_append; the rotated query goes to q_out, the rotated key and the value into the caches at position pos (or
 * pos_dev[b]); the key written is hashed by the Hc key-side MLPs into kcodes at the same position, the query written
 * by the H query-side MLPs into qcodes [B, H, W] (hashattention_llama.py:567-579 rotary + cache update, :204-226 and
 * :411-414 the embeddings of the new key and the query).  Bit for bit what the two launches produce.  128-wide heads.
 * A sequence whose pos_dev[b] lies outside [0, cache_len) (or beyond its code row) writes no key, value or key code.
 */
int ha_rope_encode_step(const void *qkv, int64_t qkv_stride_b, int x_dtype, int B, int H, int Hkv, int Hc, int pos,
                        const int32_t *pos_dev, const float *inv_freq, void *q_out, void *k_cache, void *v_cache,
                        int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s, int64_t cache_len,
                        const float *weights_k, const float *weights_q, int n_layers, int head_dim, int int_dim, int final_dim,
                        int arith, uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h, uint32_t *qcodes, void *stream);
/*
 * ha_rope_encode_step with the rotation handed over as tables: cos, sin [B, 128] of x_dtype (row stride cos_sin_stride_b in
 * elements; 0: one row for every sequence), the `position_embeddings` a transformers decoder layer passes to its attention
 * module (what the patched layer receives: hashattention_llama.py:560-571).  The rotation follows transformers'
 * apply_rotary_pos_emb to the rounding: q * cos and rotate_half(q) * sin each rounded to x_dtype, then their sum.  `pos`
 * (or pos_dev[b]) is only the cache position the new key, value and key code are written to.
 */
int ha_rope_encode_step_cos_sin(const void *qkv, int64_t qkv_stride_b, int x_dtype, int B, int H, int Hkv, int Hc, int pos,
                                const int32_t *pos_dev, const void *cos, const void *sin, int64_t cos_sin_stride_b, void *q_out,
                                void *k_cache, void *v_cache, int64_t kv_stride_b, int64_t kv_stride_h, int64_t kv_stride_s,
                                int64_t cache_len, const float *weights_k, const float *weights_q, int n_layers, int head_dim,
                                int int_dim, int final_dim, int arith, uint32_t *kcodes, int64_t kc_stride_b, int64_t kc_stride_h,
                                uint32_t *qcodes, void *stream);
/*
 * out[m, n] = sum_k x[m, k] * w[n, k] (+ residual[m, n]): a Linear layer (weight [N, K] as nn.Linear keeps it) applied to
 * M <= 16 rows, bf16 in and out, fp32 accumulation; with a residual the product is rounded to bf16 before the addition
 * and the sum rounded again, as `x + linear(h)` rounds (efficiency/model.py:190-191).  The decode step's projections (efficiency/model.py:236, 261,
 * 304-305: wqkv, wo, w1/w3, w2, and the lm_head of :158) are this shape: they stream every weight once per token, so
 * the kernel is bound by HBM.  K must be a multiple of 32, rows 16-byte aligned; strides in elements.
 */
int ha_linear_skinny(const void *x, int64_t x_stride_m, const void *w, int64_t w_stride_n,
                     const void *residual, int64_t residual_stride_m, void *out, int64_t out_stride_m,
                     int M, int N, int K, void *stream);
/*
 * The same product with the neighbouring elementwise steps of the decoder layer folded in (efficiency/model.py:308-319
 * RMSNorm, :261 feed-forward `w2(silu(w1 x) * w3 x)`):
 *   norm_weight != NULL  x is RMS-normalised first: x <- bf16(bf16(x * rsqrt(mean_k x^2 + eps)) * norm_weight[k]), the two
 *                        roundings of the module it replaces (efficiency/model.py:314-319; transformers' LlamaRMSNorm);
 *   act == HA_ACT_SWIGLU w holds F gate rows followed by F up rows (N = 2 F); out [M, F] = silu(gate) * up with the
 *                        roundings of ha_swiglu on a bf16 gate/up buffer; no residual.
 * Both need M <= 8 and K <= 16384 (the row-streaming kernel).  With norm_weight == NULL and act == HA_ACT_NONE this is
 * ha_linear_skinny.
 */
enum { HA_ACT_NONE = 0, HA_ACT_SWIGLU = 1 };
int ha_linear_skinny_fused(const void *x, int64_t x_stride_m, const void *w, int64_t w_stride_n, const void *residual,
                           int64_t residual_stride_m, const void *norm_weight, float eps, int act, void *out,
                           int64_t out_stride_m, int M, int N, int K, void *stream);

/*
 * The same products for 9 to 32 rows of x (and fewer) from a TILED copy of the weights: tiles of 16 rows x 32 inputs laid out
 * as the operand of the bf16 matrix instruction, so that a wave load is one contiguous KiB (row-major weights give such a
 * batch 64-byte pieces of 16 rows per load, 2.5 - 4 TB/s).  For callers that own a copy of the weights anyway (a decoding
 * harness as efficiency/model.py:236-262, 304-305; the stacked QKV and gate/up matrices of a patched layer).
 *   ha_weight_tiles_elems  bf16 elements of the tiled copy of a [N, K] matrix (rows padded to whole tiles), 0 for a bad shape
 *   ha_pack_weight_tiles   w [N, K] bf16 row-major (row stride w_stride_n) -> tiles.  glu = 1: w is [F gate rows; F up rows]
 *                          and every tile holds 8 gate rows followed by the 8 up rows of the same columns
 *   ha_linear_tiled        out [M, N] = x [M, K] . W^T (+ residual), K a multiple of 32; M <= 16, or M <= 32 with K <= 4096
 *                          (every weight operand is then multiplied with two blocks of 16 rows); with K > 8192 (the down
 *                          projection) x is requested next to the tiles instead of kept in registers: M <= 16, no activation;
 *                          act = HA_ACT_SWIGLU (tiles packed with glu = 1, N = 2 F): out [M, F] = silu(gate) * up.
 *                          Roundings as ha_linear_skinny_fused: those of the modules replaced.  (An RMSNorm in front is
 *                          ha_rmsnorm, a launch of its own, for batches of this size.)
 */
int64_t ha_weight_tiles_elems(int N, int K, int glu);
int ha_pack_weight_tiles(const void *w, int64_t w_stride_n, int N, int K, int glu, void *tiles, void *stream);
int ha_linear_tiled(const void *x, int64_t x_stride_m, const void *tiles, const void *residual, int64_t residual_stride_m,
                    int act, void *out, int64_t out_stride_m, int M, int N, int K, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HASHATTN_H */

/*
 * hipattn -- MI355X (gfx950) kernels for HiP / InfiniteHiP attention, C ABI.
 *
 * The reference operator is Python + Triton and has no C interface of its own; each entry
 * point below names the reference function or kernel launch it stands in for (paths relative
 * to the reference repository root).  Conventions:
 *   - extern "C", plain pointers and sizes only; every pointer is a DEVICE pointer unless the
 *     comment says host; strides are in ELEMENTS; the innermost (head-dim) stride is 1.
 *   - the caller owns every buffer; nothing here allocates device memory.
 *   - work is enqueued on `stream` (a hipStream_t passed as void*); nothing synchronises.
 *   - return value: 0 = ok, negative = argument error (HIPATTN_E_*), positive = hipError_t.
 *     hipattn_last_error() returns a host string describing the last failure of this thread.
 */
#ifndef HIPATTN_H
#define HIPATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HIPATTN_F32 0
#define HIPATTN_BF16 1
#define HIPATTN_FP8_E5M2 2 /* storage only (offload pools and caches): K / V bytes that kernels widen to bf16 on load */

#define HIPATTN_E_ARG (-1)       /* null pointer / negative size / inconsistent shapes */
#define HIPATTN_E_UNSUPPORTED (-2) /* valid request the kernels do not cover (head dim, limits) */
#define HIPATTN_E_ALIGN (-3)     /* pointer or stride not aligned for 16-byte row loads */

/* Rotary embedding applied while rows are loaded -- HiPAttentionArgs.using_extend with need_apply_rope,
 * rope_cos / rope_sin, scan_extend_backend / sa_extend_backend (src/hip_attn/v1_2/attention_metadata.py:191-198):
 * q and K are stored WITHOUT rotation and every loaded row x becomes x*cos[p] + rot(x)*sin[p], rot(x)[i] =
 * -x[i + HID/2] below HID/2 and x[i - HID/2] above, each product and the sum rounded to the element type
 * (load_keys_with_rope, src/hip_attn/v1_2/attention_extend.py:289-407; queries :626-690;
 * src/hip_attn/v1_2/attention_extend_bsa.py:248-380, :796-852).  The position p depends on `backend`:
 *   mask stage   RELATIVE  left sample 0, right sample 1, query 1 + sw_eff
 *                STREAMING key: number of its chunk in the stage's list, query: min(pos, n + sw_eff)
 *                INFLLM    key 0, query sw_eff
 *   attention    query: its own position; window keys: their own position; sink and selected keys:
 *                STREAMING max(0, slot + pmin - sliding_window - sink - (ks_end - ks_start)*block_size_k + 1),
 *                          slot = token for sink tokens, (j + sink / block_size_k) * block_size_k + e for
 *                          element e of index entry j; pmin = smallest position in the query block
 *                INFLLM    max(0, pmin - sliding_window)
 *   DYNAMIC, mask stage (attention_extend.py:249-274, :635-636): the query at its own position; with
 *                pmax = pmin + the number of valid strided query rows, W = model_context_length / 4, the sampled
 *                key at token t keeps position t when t >= pmax - W or pmax <= model_context_length, else it moves
 *                to int32((float(t) - float(pmin - W)) * (float(model_context_length - W) / float(pmin - W)))
 *                + (pmin - W), all in float32; the result is raised to at least pmax - model_context_length
 *   DYNAMIC, attention (attention_extend_bsa.py:271-292, :323-357): sink and selected keys are rotated with a blend of
 *                two table rows, 0.75 of the row of their STREAMING position and 0.25 of the row of the position
 *                the mask-stage formula above gives for their token (pmin = smallest position of the query block,
 *                pmax = pmin + its valid rows; decode: pmax = pmin + 1); both products and the sum are rounded to
 *                the element type.  (bf16, head dim 64 / 128: the matrix-core kernels; other shapes: the portable ones.)
 *   SELF, mask stage only (attention_extend.py:275-289, :637-638): the query at its own position; the sampled key at
 *                token t keeps position t when t >= pmax - 8192 or pmax <= model_context_length, else it moves to
 *                (t - pmin) / 16 + pmin with the quotient truncated toward zero (the kernel's int32 division;
 *                moved keys lie below pmin, so flooring would give another position), then max(0, .).  The
 *                reference's attention kernels raise on this rule (attention_extend_bsa.py:62-63), and so does the
 *                attention entry here.
 * Positions are clamped into [0, len).  The mode that re-rotates keys stored WITH rotation (need_apply_rope = False)
 * is not built. */
#define HIPATTN_EXTEND_RELATIVE 1
#define HIPATTN_EXTEND_STREAMING 2
#define HIPATTN_EXTEND_INFLLM 3
#define HIPATTN_EXTEND_DYNAMIC 4
#define HIPATTN_EXTEND_SELF 5

typedef struct hipattn_rope {
    const void *cos; /* [len, >= HID/2], q's dtype, 16-byte aligned rows; column i = frequency i */
    const void *sin;
    int64_t stride_t; /* elements between rows */
    int64_t len;
    int32_t backend;  /* HIPATTN_EXTEND_* for this call */
    /* hipattn_mask_stage with k_prescaled != 0 and the RELATIVE rule: kv->k holds the keys rotated to position 0
     * and scaled (hipattn_prescale_k_rope), and the copy rotated to position 1, which the right-hand samples
     * read, starts this many elements behind it.  INFLLM needs the position-0 copy only; STREAMING on a first stage
     * takes the copy hipattn_prescale_k_rope_chunks makes.  Unused otherwise. */
    int64_t k_side_delta;
    /* HiPAttentionArgs.model_context_length (attention_extend.py:250); read by the DYNAMIC rule, which needs at
     * least 512, and by the SELF rule */
    int64_t model_context_length;
} hipattn_rope_t;

/* Query tensor q[B, TDST, HEAD, HID] and its token positions (0-based, int64)
 * -- the (q, position_ids) pair of dual_stage_quadratic_hip_attention,
 * src/hip_attn/v1_2/attention_extend.py:1918-1987. */
typedef struct hipattn_q {
    const void *ptr;
    int64_t stride_b, stride_t, stride_h;
    const int64_t *pos; /* [B, TDST] */
    int64_t pos_stride_b, pos_stride_t;
    int32_t B, TDST, HEAD, HID;
    int32_t dtype; /* HIPATTN_F32 / HIPATTN_BF16; K and V share it */
    const hipattn_rope_t *rope; /* host pointer; NULL: rows are used as stored */
    /* HiPAttentionArgs.logit_softcap: 0 = off, else attention logits become tanh(qk / cap) * cap before the
     * softmax (src/hip_attn/v1_2/attention_extend_bsa.py:507-508).  Read by the bsa entry points only; the mask
     * stage scores are never capped (the reference's scan kernel has no such option). */
    float logit_softcap;
    /* HiPAttentionArgs.is_causal == False (src/hip_attn/v1_2/attention_extend_bsa.py:511-523, :743-752; read by the
     * bsa entry points only): != 0 drops the position tests of the attention mask, so every valid sink, selected
     * and window key the kernels walk is attended (a key that is both selected and in the window counts twice, as in
     * the reference).  The reference's query-block kernel then also takes MAX_TSRC for every row's position; the
     * caller passes such positions in `pos` (max_tsrc - 1), the decode kernel keeps the true ones (:118). */
    int32_t non_causal;
} hipattn_q_t;

/* Key/value storage: dense k,v[B, TSRC, HKV, HID] or a paged cache [pages, page_size, HKV, HID]
 * addressed through block_table[B, cols] -- HiPAttentionArgs.args_paged_kv_cache,
 * src/hip_attn/v1_2/attention_metadata.py:282-330, and load_tokens,
 * src/hip_attn/v1_2/uvm_gpu_cache.py:843-890,1034-1042.
 * Row address: dense  ptr + b*stride_b + t*stride_t + h*stride_h
 *              paged  ptr + page*stride_b + (t % page_size)*stride_t + h*stride_h,
 *                     page = (0 <= t < cache_seq_lens[b]) ? block_table[b][t / page_size] : 0
 * Dense reads at t >= tsrc return zeros. */
typedef struct hipattn_kv {
    const void *k;
    const void *v;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t v_stride_b, v_stride_t, v_stride_h;
    int64_t tsrc;     /* dense only */
    int64_t max_tsrc; /* TSRC, or extend_context_length when paged */
    const void *block_table;    /* int32 or int64 [B, cols] */
    const void *cache_seq_lens; /* int32 or int64 [B] */
    int64_t bt_stride_b;
    int32_t bt_is64, sl_is64;
    int32_t paged, page_size;
    int32_t HKV;
    /* Offload: NULL, or a block cache in device memory in front of K/V that live in pinned host
     * memory (see hipattn_cache_create).  Requires paged != 0. */
    const struct hipattn_cache *cache;
    /* Access statistics (HiPAttentionCacheAccessStatistics, src/hip_attn/v1_2/attention_metadata.py:76-81,
     * stores at src/hip_attn/v1_2/uvm_gpu_cache.py:845-862,1365-1372): NULL, or uint8 [B, HKV, pages]
     * (pages = tsrc when dense) where every page whose key row was loaded is set to 1, and the same
     * for loads the offload cache could not serve.  Only hipattn_mask_stage and the bsa entry points
     * write them.  The reference keeps int32 counters that only ever hold 0 or 1; a byte per page is what a decode
     * step at 1M keys can afford to clear (two tensors of 8 MB instead of 32 MB) and leaves more of the memory-side
     * cache to the key rows.  The host widens them to the reference's int32 layout when a caller reads them. */
    uint8_t *access_flags;
    uint8_t *miss_flags;
    int64_t flags_stride_b, flags_stride_h;
    /* fp8 != 0: k and v hold one byte per element, the uint8 view of a float8_e5m2 paged cache
     * (src/hip_attn/v1_2/paged_hip.py:409-418, src/hip_attn/v1_2/uvm_gpu_cache.py:1043-1046); every loaded value is
     * widened to bf16 (exact).  Needs paged != 0, a bf16 q, no offload cache; strides stay in elements (= bytes) and
     * must be multiples of 8. */
    int32_t fp8;
} hipattn_kv_t;

const char *hipattn_version(void);
const char *hipattn_last_error(void);

/* One scan stage of mask estimation: per (batch, scan row, head, chunk) binary-search refinement
 * and score.  Replaces the launch of chunk_controllable_sampling_mask_cuda,
 * src/hip_attn/v1_2/attention_extend.py:412-1249 (launch :2516-2563).
 *   chunk_left  int32 [B, BS, HG, n]   start of every candidate chunk, ascending; HG = 1 when
 *                                      scores are max-reduced over heads, else HEAD
 *   right = min(left + chunk_size, right_clamp)
 *   scores      f32   [B, BS, HEAD, n] written for every chunk (-32000 where not scored); with
 *                     reduce_heads != 0 (needs hg == 1): [B, BS, 1, n], set to -inf by the entry point
 *                     (reduce_heads = 1) or already by the caller, e.g. through hipattn_select_stage's next_scores
 *                     (reduce_heads = 2), and then raised to the maximum over heads (the torch.max at :2566-2570
 *                     folded into the scan)
 *   left_out    int32 [B, BS, HEAD, n] refined left edge per head, or NULL
 *   block_chunk = chunks per reference program (16/32/64): fixes the program-level gate and
 *   iteration count (:595-601,736-737).
 *   k_prescaled: bit 0: kv->k already holds bf16(K * c_k) (see hipattn_prescale_k); bit 1: the workspace already
 *   holds the query rows of this stage, left there by an earlier call with the same q, bs, bq, stride_q, scan_stride
 *   and no rotation (stages that differ only in their chunks share them).  Only calls that average several query rows
 *   per scan row (stride_q > 1) on more than one query token fill the workspace: the others scale their rows inside
 *   the scan kernel and leave it unwritten, so bit 1 may only follow such a call.  Bit 2, paged pools only: the caller
 *   states that every key row of the pool lies less than 32 GiB from kv->k, which admits the launches that pass the
 *   places of rows between lanes as 31-bit numbers of 16-byte pieces.  Without it a paged pool is scanned by the
 *   variants that form 64-bit addresses (the description of a pool carries no page count); for a dense tensor the
 *   library works the extent out itself from B, tsrc, HKV and the strides (hipattn_kv_rows_beyond_32gib).
 *   workspace: device scratch of hipattn_mask_stage_workspace_bytes(...) bytes. */
int hipattn_mask_stage(const hipattn_q_t *q, const hipattn_kv_t *kv, const int32_t *chunk_left,
                       int32_t hg, int32_t n, int32_t chunk_size, int64_t right_clamp,
                       int32_t bs, int32_t bq, int32_t stride_q, int32_t block_chunk,
                       int32_t scan_stride, int32_t sw_eff, int32_t terminate_size,
                       int32_t k_prescaled, int32_t reduce_heads, void *workspace, float *scores,
                       int32_t *left_out, void *stream);

/* 1 when a key row of `kv` can lie 32 GiB or more beyond kv->k (a dense tensor: from B, tsrc, HKV and the strides; a
 * paged pool: always, its size is not part of the description), 0 when not, negative on bad arguments.  The rule
 * hipattn_mask_stage applies before it picks a launch; host arithmetic only.  No counterpart in the reference, whose
 * Triton kernels form 64-bit offsets throughout (src/hip_attn/v1_2/uvm_gpu_cache.py:1034-1046). */
int hipattn_kv_rows_beyond_32gib(const hipattn_kv_t *kv, int32_t B, int32_t HID, int32_t dtype);

/* Bytes of caller-allocated scratch hipattn_mask_stage needs (bf16: the averaged, scaled query rows
 * of every scan program, [B, BS, HEAD, bq/stride_q, HID]; f32: 0, workspace may be NULL). */
int64_t hipattn_mask_stage_workspace_bytes(int32_t dtype, int32_t B, int32_t bs, int32_t HEAD, int32_t HID,
                                           int32_t bq, int32_t stride_q);

/* K^ = bf16(K * c_k) for a whole bf16 key tensor viewed as [n0, n1, n2, HID] with element strides
 * (stride0, stride1, stride2, 1); `out` is contiguous [n0, n1, n2, HID].  Passing `out` as kv->k
 * with k_prescaled = 1 lets hipattn_mask_stage skip the per-sample scaling the reference performs on
 * every loaded key (src/hip_attn/v1_2/attention_extend.py:932-937); results are identical. */
int hipattn_prescale_k(const void *k, int64_t stride0, int64_t stride1, int64_t stride2, int64_t n0,
                       int32_t n1, int32_t n2, int32_t HID, void *out, void *stream);

/* The same with a rotation first: out = bf16(rot(K, p) * c_k) for ONE position p whose table rows (HID/2 bf16
 * entries each, 16-byte aligned) are cos_row / sin_row.  The RELATIVE and INFLLM scan rules rotate every sampled
 * key to position 0 or 1 whatever the token, so two such copies replace the per-sample rotation
 * (see hipattn_rope_t.k_side_delta). */
int hipattn_prescale_k_rope(const void *k, int64_t stride0, int64_t stride1, int64_t stride2, int64_t n0,
                            int32_t n1, int32_t n2, int32_t HID, const void *cos_row, const void *sin_row,
                            void *out, void *stream);

/* The same for the STREAMING rule on the FIRST stage of a scan (attention_extend.py:289-298: a sampled key is rotated
 * to the place of its chunk in the stage's list): a first stage's list is every chunk in order, chunk c starting at
 * token `first + c * chunk`, so the position of token t is (t - first) / chunk whatever the query, and
 * out[b, t, h] = bf16(rot(K[b, t, h], min((t - first) / chunk, table_len - 1)) * c_k) (tokens below `first` are never
 * sampled there and are rotated to position 0).  K is a dense [B, T, HKV, HID] tensor with the element strides given,
 * `out` contiguous; cos / sin are the whole tables ([table_len, >= HID/2], table_stride elements between rows).
 * hipattn_mask_stage takes `out` as kv->k with k_prescaled = 1 and the STREAMING rule. */
int hipattn_prescale_k_rope_chunks(const void *k, int64_t stride_b, int64_t stride_t, int64_t stride_h, int64_t B,
                                   int32_t T, int32_t HKV, int32_t HID, const void *cos, const void *sin,
                                   int64_t table_stride, int64_t table_len, int32_t first, int32_t chunk, void *out,
                                   void *stream);

/* Between two stages: max over heads, top-k under (score desc, position asc), realign, split.
 * Replaces the ATen glue at src/hip_attn/v1_2/attention_extend.py:2566-2570 (head reduce),
 * :2710-2728 (topk + gather) and :2072-2165 (truncate, realign, sort, re-tile, split).
 *   scores      f32   [B, BS_in, HEAD, n]  (HEAD = 1 for scores already reduced over heads)
 *   chunk_left  int32 [B, BS_in, HG, n]
 *   next_left   int32 [B, BS_out, HG, k*splits]; chunk j of a kept parent starts at
 *               left + j*(chunk_size/splits)
 *   output row o reads input row (o + row_rep*BS_in - BS_out) / row_rep
 *   (repeat_interleave(row_rep, 1)[:, -BS_out:], :2092-2123).
 *   next_left64 / next_right64: NULL, or int64 buffers of next_left's shape that receive the same list as
 *   (left, left + chunk_size/splits), the layout of HiPAttentionStageInputCache.indices_left / indices_right
 *   (src/hip_attn/v1_2/attention_metadata.py:111-115).
 *   next_scores: NULL, or (hg == 1 only) the next stage's head-reduced scores, f32 [B, BS_out, 1, k*splits]: every
 *   entry is set to -inf, so that the next hipattn_mask_stage can be called with reduce_heads = 2 and needs no
 *   launch of its own to initialise them. */
int hipattn_select_stage(const float *scores, const int32_t *chunk_left, int32_t B, int32_t bs_in,
                         int32_t bs_out, int32_t row_rep, int32_t HEAD, int32_t hg, int32_t n,
                         int32_t k, int32_t chunk_size, int32_t splits, int32_t *next_left,
                         int64_t *next_left64, int64_t *next_right64, float *next_scores, void *stream);

/* After the last stage: top-K chunks, block alignment, de-duplication, active count, in the
 * reference's metadata layout.  Replaces src/hip_attn/v1_2/attention_extend.py:2757-2776 and
 * :2906-2924.
 *   scores      f32   [B, BS, score_heads, n], score_heads = HEAD or 1 (already reduced, needs hg == 1)
 *   left_out    int32 [B, BS, HEAD, n]  refined left edges from the last hipattn_mask_stage
 *   indices     int64 [B*HEAD, BDST, BK] ascending unique block starts then INT64_MAX
 *   ks          int64 [B*HEAD, BDST]     entries below pos[b, qb*bq] + bq
 *   ks_start_end int32 [B*HEAD, BDST, 2] = (0, ks)
 *   BK = min(K, n); output row qb reads scan row (qb + scan_stride*BS - BDST) / scan_stride. */
int hipattn_finalize_indices(const float *scores, const int32_t *left_out, const int64_t *pos,
                             int64_t pos_stride_b, int64_t pos_stride_t, int32_t B, int32_t bs,
                             int32_t bdst, int32_t scan_stride, int32_t HEAD, int32_t score_heads, int32_t hg,
                             int32_t n, int32_t K, int32_t chunk_size, int32_t bq, int64_t *indices,
                             int64_t *ks, int32_t *ks_start_end, void *stream);

/* Block-sparse flash attention over selected blocks + sink + sliding window.  Replaces
 * block_sparse_attention, src/hip_attn/v1_2/attention_extend_bsa.py:1641-1777 (kernel :607-1638).
 *   indices int64 [B*HEAD, idx_rows, BK], ks_start_end int32 [B*HEAD, idx_rows, 2]
 *   out has q's dtype; out strides in elements.
 *   share_first_head != 0: every head of a GQA group reads the index row of the group's first
 *   head (decode kernel behaviour, src/hip_attn/v1_2/attention_decode_bsa.py:150).
 *   impl: 0 = pick automatically, 1 = portable row-at-a-time kernel, 2 = MFMA tile kernel.
 *   k_prescaled: NULL, or bf16(K * c_k) with exactly the layout and strides of kv->k (the buffer
 *   hipattn_prescale_k fills when K itself is contiguous); only the tile kernel reads it. */
int hipattn_bsa_prefill(const hipattn_q_t *q, const hipattn_kv_t *kv, const int64_t *indices,
                        const int32_t *ks_start_end, int32_t idx_rows, int32_t BK,
                        int32_t block_size_q, int32_t block_size_k, int32_t sliding_window,
                        int32_t sink, int32_t share_first_head, int32_t impl,
                        const void *k_prescaled, void *out,
                        int64_t out_stride_b, int64_t out_stride_t, int64_t out_stride_h,
                        void *stream);

/* Decode (TDST == 1) split-KV attention.  Replaces decode_block_sparse_attention,
 * src/hip_attn/v1_2/attention_decode_bsa.py:1331-1435: _fwd_kernel_stage1 (:22-1045) writes
 * per-split partials, _fwd_kernel_stage2 (:1148-1226) merges them by log-sum-exp.  The merge folds every
 * (1024 / HID)-th split into a running (maximum, numerator, denominator) and then folds those parts, so its f32
 * summation order depends on HID and is not the split order: outputs are held to the attention tolerance, not to
 * bits, across builds and head dims (HID must divide 1024: 32, 64, 128, 256).
 *   workspace: f32, hipattn_bsa_decode_workspace_bytes(...) bytes, caller-allocated.
 *   nsplits: how many workgroups share one (sequence, kv head); hipattn_bsa_decode_default_splits picks one.
 *   second_stage_k: args.second_stage_k of the call being replaced, or 0.  The reference's launcher divides the
 *   index row among min(12, ceil(second_stage_k / ceil((second_stage_k + sink + window) / 8))) programs (:1070-1076)
 *   that walk their share in tiles of 16 / block_size_k entries (:1391-1393) and mask a tile against the end of the
 *   row only (:239-247): when the share is not a whole number of tiles, the entries at the start of the next share
 *   are attended twice.  With second_stage_k > 0 those entries get the same weight here, so the output equals the
 *   reference's; with 0 every selected block counts once.  The sink is likewise divided among
 *   min(12, ceil(sink / ceil((second_stage_k + sink + window) / 8))) programs (:1077, :514-518), each numbering its
 *   tokens from its first token rounded down to a multiple of block_size_k (:740); under the "streaming" rotation
 *   rule a sink token is therefore rotated (share start % block_size_k) positions lower than its own number, which
 *   second_stage_k > 0 reproduces as well. */
int64_t hipattn_bsa_decode_workspace_bytes(int32_t B, int32_t HEAD, int32_t HID, int32_t nsplits);
int32_t hipattn_bsa_decode_default_splits(int32_t B, int32_t HKV, int32_t tokens);
int hipattn_bsa_decode_partial(const hipattn_q_t *q, const hipattn_kv_t *kv, const int64_t *indices,
                               const int32_t *ks_start_end, int32_t idx_rows, int32_t BK,
                               int32_t block_size_k, int32_t sliding_window, int32_t sink,
                               int32_t second_stage_k, int32_t nsplits, void *workspace, void *stream);
int hipattn_bsa_decode_merge(const void *workspace, int32_t B, int32_t HEAD, int32_t HID,
                             int32_t nsplits, int32_t dtype, void *out, int64_t out_stride_b,
                             int64_t out_stride_h, void *stream);
/* The two calls above as one (two launches; the same decode_block_sparse_attention,
 * attention_decode_bsa.py:1331-1435): for hosts on which a call into the library costs as much as a launch. */
int hipattn_bsa_decode(const hipattn_q_t *q, const hipattn_kv_t *kv, const int64_t *indices,
                       const int32_t *ks_start_end, int32_t idx_rows, int32_t BK, int32_t block_size_k,
                       int32_t sliding_window, int32_t sink, int32_t second_stage_k, int32_t nsplits,
                       void *workspace, void *out, int64_t out_stride_b, int64_t out_stride_h, void *stream);

/* Decode attention that allocates nothing and needs no workspace: hipattn_bsa_decode_partial followed by
 * hipattn_bsa_decode_merge with the split partials kept in a device array inside the library.  It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory around the call: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Arguments as for the two calls it
 * combines; nsplits <= 0 picks hipattn_bsa_decode_default_splits.
 *   Limit: B * HEAD * nsplits * (HID + 4) * 4 bytes of partials must fit HIPATTN_DECODE_SCRATCH_BYTES, otherwise
 *   HIPATTN_E_UNSUPPORTED (the batched 16-sequence decode with 32 heads, head dim 128 and 9 splits needs 2.4 MB, one
 *   sequence with 64 splits 1.1 MB).  Each GPU the library runs on holds the array until the process ends.
 *   The first call on a device looks the array's address up (make it outside a graph capture).  All calls on one
 *   GPU share the array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream, or
 *   ordered by events, do not.  No hipMalloc, hipFree or allocating library call is made. */
#define HIPATTN_DECODE_SCRATCH_BYTES (4 * 1024 * 1024)
int hipattn_bsa_decode_static(const hipattn_q_t *q, const hipattn_kv_t *kv, const int64_t *indices,
                              const int32_t *ks_start_end, int32_t idx_rows, int32_t BK, int32_t block_size_k,
                              int32_t sliding_window, int32_t sink, int32_t second_stage_k, int32_t nsplits,
                              void *out, int64_t out_stride_b, int64_t out_stride_h, void *stream);

/* ---------------------------------------------------------------------------------------------
 * Offload cache: K (and V) of a layer live in pinned host memory as a pool [pool_rows, HKV, HID]
 * addressed through the paged view (row = page * page_size + offset); a block cache in device
 * memory holds `slots` blocks of `block_tokens` consecutive pool rows of ONE kv head.  Stands in for
 * GPUCache / HiPOffloadCache, src/hip_attn/v1_2/uvm_gpu_cache.py:204-566,569-700: token -> slot
 * table, least-recently-used replacement by last-access step, reads that miss go to host memory and
 * are recorded, recorded misses are brought in after the step.
 *
 * Kernels given kv->cache look every row up in `table`; a resident block is read from `bank` and
 * stamped with the current step, a missing one is read from the host pool over the host link and
 * flagged in `miss`.  Results are therefore the same bytes with or without the cache.
 * After the step:  hipattn_cache_lookup_and_schedule gathers the flagged blocks (ascending
 * head-major block id, at most max_fetch) and picks as many victims: the slots with the smallest
 * (last-use step, slot id), never one used in the current step;  hipattn_cache_commit copies the
 * blocks host -> bank, relinks the table, and advances the step counter.  Both only enqueue work;
 * the caller orders them after the kernels of the step and before those of the next one (they may
 * run on another stream, overlapped with unrelated work).
 * All buffers are the caller's; sizes from hipattn_cache_sizes. */
typedef struct hipattn_cache hipattn_cache_t;

typedef struct hipattn_cache_desc {
    int32_t dtype;        /* HIPATTN_F32 / HIPATTN_BF16 / HIPATTN_FP8_E5M2 (with hipattn_kv_t.fp8 and bf16 queries) */
    int32_t HKV, HID;
    int32_t block_tokens; /* power of two, 1..64 */
    int32_t with_v;       /* 0: K only (mask estimation cache), 1: K and V per slot (attention cache) */
    int64_t pool_rows;    /* rows of the host pool */
    int64_t slots;
    const void *host_k;   /* device-visible address of the pinned pool; strides in elements */
    const void *host_v;   /* NULL when with_v == 0 */
    int64_t host_stride_row, host_stride_h;
    void *bank;           /* slots * (1 + with_v) * block_tokens * HID elements */
    int32_t *table;       /* [HKV, n_blocks], n_blocks = ceil(pool_rows / block_tokens) */
    int32_t *last_use;    /* [slots] */
    int32_t *backref;     /* [slots] */
    uint8_t *miss;        /* [HKV, n_blocks] */
    void *workspace;      /* hipattn_cache_sizes(...).workspace bytes */
} hipattn_cache_desc_t;

typedef struct hipattn_cache_sizes {
    int64_t n_blocks;
    int64_t bank_bytes, table_bytes, last_use_bytes, backref_bytes, miss_bytes, workspace_bytes;
} hipattn_cache_sizes_t;

int hipattn_cache_sizes(const hipattn_cache_desc_t *desc, int64_t max_fetch, hipattn_cache_sizes_t *out);
/* Builds the handle (host memory only) and enqueues the kernels that empty the cache. max_fetch bounds
 * the blocks one commit can bring in. */
int hipattn_cache_create(const hipattn_cache_desc_t *desc, int64_t max_fetch, hipattn_cache_t **out, void *stream);
void hipattn_cache_destroy(hipattn_cache_t *cache);
/* Empties the cache (GPUCache.flush, src/hip_attn/v1_2/uvm_gpu_cache.py:294-300). */
int hipattn_cache_flush(hipattn_cache_t *cache, void *stream);
int hipattn_cache_lookup_and_schedule(hipattn_cache_t *cache, void *stream);
int hipattn_cache_commit(hipattn_cache_t *cache, void *stream);
/* Write-through after the host pool changed (HiPOffloadCache.set_kv_buffer / on_set_kv_buffer,
 * src/hip_attn/v1_2/uvm_gpu_cache.py:629-688,548-563): rows int64 [n] pool rows, k_rows / v_rows
 * device [n, HKV, HID] contiguous; resident blocks receive the new rows, others are left alone. */
int hipattn_cache_write_rows(hipattn_cache_t *cache, const int64_t *rows, int64_t n, const void *k_rows,
                             const void *v_rows, void *stream);
/* Scatter device rows src[n, HKV, HID] (contiguous) into a pinned host pool at int64 rows[n] -- the GPU-side
 * store of HiPOffloadCache.set_kv_buffer (src/hip_attn/v1_2/uvm_gpu_cache.py:665-668).  dtype is the pool's storage
 * format (HIPATTN_F32 / HIPATTN_BF16 / HIPATTN_FP8_E5M2); rows are copied as stored, strides are in elements. */
int hipattn_pool_write_rows(void *pool, int64_t stride_row, int64_t stride_h, int32_t HKV, int32_t HID,
                            int32_t dtype, const int64_t *rows, int64_t n, const void *src, void *stream);
/* The gather in the other direction: dst[i, h, :] = pool[rows[i], h, :] for int64 rows[n] (negative: zero row); dst is
 * device memory [n, HKV, HID] with dst_stride_row elements between rows.  The device reads the pinned pool in place, on
 * `stream` -- the copy half of HiPOffloadCache.prefetch_prefix_kv_buffer (src/hip_attn/v1_2/uvm_gpu_cache.py:690-700),
 * which the reference does with a host gather and a blocking upload. */
int hipattn_pool_read_rows(const void *pool, int64_t stride_row, int64_t stride_h, int32_t HKV, int32_t HID,
                           int32_t dtype, const int64_t *rows, int64_t n, void *dst, int64_t dst_stride_row,
                           void *stream);
/* Pinned host memory for a pool.  coherent != 0 asks for memory the GPU never caches, so that rows the CPU
 * writes are seen by the next kernel without any cache maintenance; pools written by the CPU need it. */
int hipattn_host_alloc(int64_t bytes, int32_t coherent, void **host_out);
int hipattn_host_free(void *host);
/* Device-visible address of memory obtained from hipHostMalloc (HOST pointer in, device pointer out). */
int hipattn_host_device_pointer(void *host, void **device_out);
/* Copies the counters to host memory and waits for `stream`:
 * out[0] steps committed, [1] resident blocks touched (summed over steps), [2] blocks missed,
 * [3] blocks fetched, [4] blocks evicted, [5] touched in the last step, [6] missed in the last step,
 * [7] fetched in the last step. */
int hipattn_cache_stats(hipattn_cache_t *cache, int64_t out[8], void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HIPATTN_H */

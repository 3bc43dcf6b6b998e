// Parameter block shared by the mask-estimation scan kernels.
#pragma once

#include <type_traits>

#include "common.hpp"

namespace hipattn {

struct MaskParamsBase {
    const void *q;
    int64_t q_sb, q_st, q_sh;
    const int64_t *pos;
    int64_t pos_sb, pos_st;
    KVView kv;
    const int32_t *chunk_left;
    int hg, n, chunk;
    int64_t right_clamp;
    int B, TDST, HEAD, G, BS, BDST, BQ, stride_q, nrows, block_chunk, scan_stride, sw_eff;
    float terminate;
    int ngroups;
    int group_reps;  // bf16 path: consecutive chunk groups walked by one wave (set by its launcher)
    int share_first; // bf16 path, coalesced fetch: the four heads of a workgroup fetch the rows of a search's first round once
    long long total;
    float c_q, c_k;
    float *scores;
    int reduce_heads;  // scores is [B, BS, 1, n], pre-filled with -inf, and receives the max over heads
    int32_t *left_out;
    const uint16_t *qhat;  // bf16 path: workspace [B, BS, HEAD][nrows * HID] filled by the entry point (fragment order)
};

// the extended kernels (statistics, offload cache) take the same block with the extras appended
struct MaskParams : MaskParamsBase {
    KVExt kx;
    RopeView rope;
};
template <bool EXT>
using MaskParamsFor = std::conditional_t<EXT, MaskParams, MaskParamsBase>;

// Score of one (head, chunk): a plain store, or the running maximum over heads.  The maximum uses the usual
// split on the sign (ordered as int for non-negative floats, reverse-ordered as unsigned for negative ones);
// -0 is folded into +0 first, and the target starts at -inf.
__device__ __forceinline__ void store_score(const MaskParamsBase &p, int64_t row_out, int64_t red_out, int c, float v) {
    if (!p.reduce_heads) {
        p.scores[row_out + c] = v;
        return;
    }
    if (v == 0.0f) v = 0.0f;
    float *a = p.scores + red_out + c;
    if (v >= 0.0f) atomicMax(reinterpret_cast<int *>(a), __float_as_int(v));
    else atomicMin(reinterpret_cast<unsigned int *>(a), __float_as_uint(v));
}

// bf16, prescaled keys, chunks of 2 .. 16 tokens on wide launches: every token of every chunk is scored once per
// GQA group and the searches are replayed on the scores (mask_stage_dense.hip).
// mask_stage_dense_applies: is this launch one the kernel covers (and, by the default rule, worth it)?
// mask_stage_dense_launch: expects the scores initialised (reduce_heads) and either p.qhat filled or, with
// q_inline (stride_q == 1 only: a query row is its own mean), nothing: the kernel then scales the query rows itself.
bool mask_stage_dense_applies(const MaskParams &p, int HID, int rows_eff);
int mask_stage_dense_launch(const MaskParams &p, int HID, int rows_eff, bool q_inline, hipStream_t st);
// -inf into the head-reduced scores of a stage (what the query preparation launch otherwise does on its way)
void mask_stage_fill_scores(const MaskParams &p, hipStream_t st);

// bf16 path on the matrix cores (mask_stage_mfma.hip)
int mask_stage_mfma_launch(const MaskParams &p, int HID, int rows_eff, int prescaled, hipStream_t st);

}  // namespace hipattn

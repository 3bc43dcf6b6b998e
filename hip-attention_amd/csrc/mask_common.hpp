// Parameter block shared by the mask-estimation scan kernels.
#pragma once

#include "common.hpp"

namespace hipattn {

struct MaskParams {
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
    long long total;
    float c_q, c_k;
    float *scores;
    int32_t *left_out;
    const uint16_t *qhat;  // bf16 path: workspace [B, BS, HEAD, nrows, HID] filled by the entry point
};

// bf16 path on the matrix cores (mask_stage_mfma.hip)
int mask_stage_mfma_launch(const MaskParams &p, int HID, int rows_eff, int prescaled, hipStream_t st);

}  // namespace hipattn

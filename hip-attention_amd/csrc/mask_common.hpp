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
    long long total;
    float c_q, c_k;
    float *scores;
    int32_t *left_out;
    const uint16_t *qhat;  // bf16 path: workspace [B, BS, HEAD, nrows, HID] filled by the entry point
};

// the extended kernels (statistics, offload cache) take the same block with the extras appended
struct MaskParams : MaskParamsBase {
    KVExt kx;
};
template <bool EXT>
using MaskParamsFor = std::conditional_t<EXT, MaskParams, MaskParamsBase>;

// bf16 path on the matrix cores (mask_stage_mfma.hip)
int mask_stage_mfma_launch(const MaskParams &p, int HID, int rows_eff, int prescaled, hipStream_t st);

}  // namespace hipattn

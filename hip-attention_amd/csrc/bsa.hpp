// Parameter block shared by the block-sparse attention kernels.
#pragma once

#include <type_traits>

#include "common.hpp"

namespace hipattn {

struct BsaParamsBase {
    const void *q;
    int64_t q_sb, q_st, q_sh;
    const int64_t *pos;
    int64_t pos_sb, pos_st;
    KVView kv;
    const int64_t *indices;
    const int32_t *kse;
    int idx_rows, BK, bq, bk, sw, sink, share_first_head;
    int k_prescaled;  // kv.k already holds bf16(K * c_k) (tile kernel only)
    // Decode only: the reference's decode kernel gives each of its programs `seam_blocks` entries of the index row but
    // masks a program's last tile against the end of the row only, so the first `seam_extra` entries of the next
    // program's share are attended once more (attention_decode_bsa.py:239-247); 0 / 0 = every entry once.
    int seam_blocks, seam_extra;
    // Decode with the "streaming" rotation rule only: the reference's decode programs take `sink_share` sink tokens
    // each and number them from their first token rounded down to a multiple of the block size
    // (attention_decode_bsa.py:514-518, 740), so a token is rotated (share start % bk) positions lower; 0 = off.
    int sink_share;
    int non_causal;  // no position tests in the mask (is_causal = False, attention_extend_bsa.py:511-523)
    int B, TDST, HEAD, G, NBQ;
    float c_q, c_k;
    void *out;
    int64_t o_sb, o_st, o_sh;
};

// the extended kernels (statistics, offload cache) take the same block with the extras appended
struct BsaParams : BsaParamsBase {
    KVExt kx;
    RopeView rope;
    float softcap;  // 0 = off; logits become tanh(qk / softcap) * softcap (attention_extend_bsa.py:507-508)
};

// tanh(x / cap) * cap through one exp2 and one reciprocal: tanh(y) = 1 - 2 / (exp(2y) + 1)
__device__ __forceinline__ float softcap_logit(float x, float cap, float two_log2e_over_cap) {
    const float e = __builtin_amdgcn_exp2f(x * two_log2e_over_cap);
    return cap * (1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f));
}
// How often the reference's decode programs visit entry j of an index row: once by the program that owns it, and
// once by each earlier program whose tile-rounded walk reaches it.
__host__ __device__ __forceinline__ int bsa_seam_multiplicity(int j, int seam_blocks, int seam_extra) {
    const int s = j / seam_blocks, r = j - s * seam_blocks;
    const int earlier = (seam_blocks + seam_extra - r - 1) / seam_blocks;
    return 1 + (earlier < s ? earlier : s);
}
// The number under which the reference's decode kernel rotates sink token t.
__host__ __device__ __forceinline__ long long bsa_decode_sink_slot(long long t, int sink_share, int bk) {
    return sink_share > 0 ? t - ((t / sink_share) * sink_share) % bk : t;
}
// Rotated position of a sink or selected key (attention_extend_bsa.py:256-299): "streaming" packs them, in the
// order of the index row, into the positions that end just below the window of the block's first query;
// "infllm" puts all of them at that edge.  `slot` = token for sink tokens, (j + sink / bk) * bk + e for element e
// of index entry j; `shift` = pmin - sw - sink - (ks_end - ks_start) * bk + 1.
__device__ __forceinline__ int64_t bsa_rope_far_pos(const RopeView &r, long long slot, long long shift, long long pmin,
                                                    int sw) {
    const long long v = r.backend == HIPATTN_EXTEND_INFLLM ? pmin - sw : slot + shift;
    return v < 0 ? 0 : v;
}

// The "dynamic_extend" rule inside attention (attention_extend_bsa.py:271-292, :323-357): a sink or selected key is
// rotated with a blend of two table rows, 0.75 of the row of its "streaming" position and 0.25 of the row of its own
// position squeezed into the model's context (dynamic_extend_pos); both products and the sum are rounded to T.
template <typename T>
__device__ __forceinline__ float rope_blend(float stream, float dyn) {
    return Elem<T>::round(__fadd_rn(Elem<T>::round(__fmul_rn(stream, 0.75f)), Elem<T>::round(__fmul_rn(dyn, 0.25f))));
}

// ---------------------------------------------------------------- pieces shared by the matrix-core attention kernels
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int KPAD = 8;       // bf16 elements of row padding for a K^ tile in LDS
constexpr int VPAD = 32;      // bf16 elements of row padding for a V tile: four consecutive rows tile all banks
constexpr float LOG2E = 1.44269504f;
constexpr float RESCALE_STEP = 8.0f;  // raise the running max only when it grows by more than this (log2 units)

__device__ __forceinline__ uint32_t cvt_pk_bf16(float a, float b) {  // one v_cvt_pk_bf16_f32
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// Transposing LDS read (ds_read_b64_tr_b16): lane l of a 16-lane group receives column l % 4 of the four 8-byte rows
// addressed by lanes l / 4, l / 4 + 4, l / 4 + 8, l / 4 + 12 of its group.
typedef __attribute__((ext_vector_type(4))) short s16x4;
__device__ __forceinline__ uint2 lds_read_tr16(const uint16_t *p) {
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p);
    return __builtin_bit_cast(uint2, v);
}

union Frag {
    bf16x8 v;
    uint32_t u[4];
    uint2 d[2];
    uint4 q;
};

template <bool EXT>
using BsaParamsFor = std::conditional_t<EXT, BsaParams, BsaParamsBase>;

// validates arguments and fills the parameter block (host)
int bsa_fill_params(const hipattn_q_t *q, const hipattn_kv_t *kv, const int64_t *indices, const int32_t *kse,
                    int idx_rows, int BK, int bq, int bk, int sw, int sink, int share_first_head, void *out,
                    int64_t o_sb, int64_t o_st, int64_t o_sh, BsaParams *p);
int bsa_simple_launch(const BsaParams &p, int dtype, int HID, hipStream_t st);
// returns HIPATTN_E_UNSUPPORTED (without setting an error) when the tile kernel does not cover the case
int bsa_mfma_launch(const BsaParams &p, int dtype, int HID, hipStream_t st);
// decode partials on the matrix cores; HIPATTN_E_UNSUPPORTED (no error text) when the case is not covered
int bsa_decode_mfma_launch(const BsaParams &p, int dtype, int HID, int nsplits, float *ws, hipStream_t st);

}  // namespace hipattn

// Decode (one query token per sequence) block-sparse attention: split-KV partials + merge.
//
// A workgroup owns one (sequence, kv head, split) and all G query heads of the GQA group, so every
// gathered K/V row is read once for the whole group.  Sixteen lanes share a token row (HID/16
// contiguous elements each: one coalesced 16-lane load per row, four rows per load instruction per
// wave); each 16-lane group keeps its own online-softmax state and output slice, and the sixteen
// states of a workgroup are merged through LDS before the partial is written.
#include <stdlib.h>

#include <atomic>

#include "bsa.hpp"

namespace hipattn {

template <bool EXT>
struct DecodeParamsT {
    BsaParamsFor<EXT> a;
    int nsplits;
    int parts;  // workgroups that share one GQA group, G heads each (group size = parts * G)
    float *ws;  // [B, HEAD, nsplits, HID + 4]: acc / l, then m + log2(l)
};
using DecodeParams = DecodeParamsT<true>;

// ROPE = true (extended parameter block only): query and keys are rotated on load; lanes dl and dl ^ 8 of a
// 16-lane group hold the two halves of a row.
// CAP = true (extended parameter block only): logits are soft-capped.
// KV8 = true (extended parameter block only): K / V rows are fp8 (e5m2) bytes, widened on load.
template <typename T, int HID, int G, bool EXT, bool ROPE = false, bool CAP = false, bool KV8 = false>
__global__ __launch_bounds__(256) void bsa_decode_partial_kernel(DecodeParamsT<EXT> dp) {
    static_assert((!ROPE && !CAP && !KV8) || EXT, "rope / softcap / fp8 variants take the extended parameter block");
    constexpr int SEG = HID / 16;
    const BsaParamsFor<EXT> &p = dp.a;
    const KVExt *kx = nullptr;
    if constexpr (EXT) kx = &p.kx;
    __shared__ float s_m[16][G];
    __shared__ float s_l[16][G];
    __shared__ float s_acc[16][G][HID];

    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int sub = lane >> 4, dl = lane & 15;
    const int grp = wid * 4 + sub;  // 16-lane group id inside the workgroup
    const int split = blockIdx.x, kvh = blockIdx.y / dp.parts, b = blockIdx.z;
    const int h0 = kvh * p.G + (blockIdx.y % dp.parts) * G;
    const int64_t irow = ((int64_t)b * p.HEAD + kvh * p.G) * p.idx_rows;  // query block 0, first head of the group

    const long long ppos = p.pos[(int64_t)b * p.pos_sb];
    const long long curr = ppos + 1;
    int rs = p.kse[irow * 2 + 0], re = p.kse[irow * 2 + 1];
    const long long rope_shift = ppos - p.sw - p.sink - (long long)(re - rs) * p.bk + 1;
    if (p.BK <= 0) { rs = 0; re = 0; }
    const int jend = rs + p.BK < re ? rs + p.BK : re;
    const int nsel = jend > rs ? jend - rs : 0;
    const long long n_sel_tok = (long long)nsel * p.bk;
    const long long sink_end = curr < p.sink ? curr : p.sink;
    long long ws0 = curr - p.sw - 1;  // block_size_q = 1 for decode
    if (ws0 < 0) ws0 = 0;
    const long long n_win = p.sw > 0 ? curr - ws0 : 0;
    const long long total = n_sel_tok + sink_end + n_win;
    long long per = (total + dp.nsplits - 1) / dp.nsplits;
    per = (per + 15) / 16 * 16;
    const long long o_begin = (long long)split * per;
    const long long o_end = o_begin + per < total ? o_begin + per : total;

    const int64_t seqlen = p.kv.paged ? p.kv.seq_len(b) : 0;
    const void *kbase = p.kv.k;
    const void *vbase = p.kv.v;

    float qh[G][SEG];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const T *qrow = reinterpret_cast<const T *>(p.q) + (int64_t)b * p.q_sb + (int64_t)(h0 + g) * p.q_sh;
        load_elems<T, SEG>(qrow + dl * SEG, qh[g]);
        if constexpr (ROPE) {  // the query keeps its own position (attention_decode_bsa.py:135-262)
            float other[SEG], rc[SEG], rsn[SEG];
            load_elems<T, SEG>(qrow + (dl ^ 8) * SEG, other);
            const int64_t tr = p.rope.row(ppos) + (dl & 7) * SEG;
            load_elems<T, SEG>(reinterpret_cast<const T *>(p.rope.cos) + tr, rc);
            load_elems<T, SEG>(reinterpret_cast<const T *>(p.rope.sin) + tr, rsn);
#pragma unroll
            for (int e = 0; e < SEG; e++) qh[g][e] = rope_elem<T>(qh[g][e], dl < 8 ? -other[e] : other[e], rc[e], rsn[e]);
        }
#pragma unroll
        for (int e = 0; e < SEG; e++) qh[g][e] = Elem<T>::round(qh[g][e] * p.c_q);
    }
    float m[G], l[G], acc[G][SEG];
#pragma unroll
    for (int g = 0; g < G; g++) {
        m[g] = -INFINITY;
        l[g] = 0.0f;
#pragma unroll
        for (int e = 0; e < SEG; e++) acc[g][e] = 0.0f;
    }

    for (long long base = o_begin; base < o_end; base += 16) {
        const long long o = base + grp;
        long long t = -1;
        int kind = 0;
        bool valid = false;
        long long rpos = 0;  // rotated position of the key (ROPE only)
        float visits = 1.0f;  // how often the reference's programs attend this token
        if (o < o_end) {
            if (o < n_sel_tok) {
                const long long st = p.indices[irow * p.BK + rs + o / p.bk];
                if (p.seam_extra > 0) visits = (float)bsa_seam_multiplicity(rs + (int)(o / p.bk), p.seam_blocks, p.seam_extra);
                t = st + o % p.bk;
                valid = (t >= 0) && (t < p.kv.max_tsrc) && (t < curr) && (t >= p.sink);
                if constexpr (ROPE)
                    rpos = bsa_rope_far_pos(p.rope, (rs + o / p.bk + p.sink / p.bk) * (long long)p.bk + o % p.bk, rope_shift,
                                            ppos, p.sw);
            } else if (o < n_sel_tok + sink_end) {
                t = o - n_sel_tok;
                valid = true;
                if constexpr (ROPE)
                    rpos = bsa_rope_far_pos(p.rope, bsa_decode_sink_slot(t, p.sink_share, p.bk), rope_shift, ppos, p.sw);
            } else {
                t = ws0 + (o - n_sel_tok - sink_end);
                kind = 1;
                valid = true;
                rpos = t;
            }
        }
        const bool att = valid && (p.non_causal || (kind == 0 ? (t + p.sw <= ppos) : (t <= ppos && ppos < t + p.sw)));
        int64_t koff, voff;
        if (!att) {  // uniform inside the 16-lane group; shuffles below stay inside the group
            // staged but masked out: still an access as far as the statistics and the cache are concerned
            if (EXT && valid && dl == 0) kv_rows<false, EXT>(p.kv, kx, b, t, kvh, seqlen, koff, voff, true);
            continue;
        }
        kv_rows<true, EXT>(p.kv, kx, b, t, kvh, seqlen, koff, voff, dl == 0);
        float kh[SEG], vv[SEG];
        if (koff != NO_ROW) {
            load_kv_elems<T, SEG, KV8>(kbase, koff + dl * SEG, kh);
        } else {
#pragma unroll
            for (int e = 0; e < SEG; e++) kh[e] = 0.0f;
        }
        if (voff != NO_ROW) {
            load_kv_elems<T, SEG, KV8>(vbase, voff + dl * SEG, vv);
        } else {
#pragma unroll
            for (int e = 0; e < SEG; e++) vv[e] = 0.0f;
        }
        if constexpr (ROPE) {
            float rc[SEG], rsn[SEG];
            const int64_t tr = p.rope.row(rpos) + (dl & 7) * SEG;
            load_elems<T, SEG>(reinterpret_cast<const T *>(p.rope.cos) + tr, rc);
            load_elems<T, SEG>(reinterpret_cast<const T *>(p.rope.sin) + tr, rsn);
            if (kind == 0 && p.rope.backend == HIPATTN_EXTEND_DYNAMIC) {  // one query row: pmax = its position + 1
                float dc[SEG], ds[SEG];
                const int64_t td = p.rope.row(dynamic_extend_pos(t, ppos, ppos + 1, p.rope.model_ctx)) + (dl & 7) * SEG;
                load_elems<T, SEG>(reinterpret_cast<const T *>(p.rope.cos) + td, dc);
                load_elems<T, SEG>(reinterpret_cast<const T *>(p.rope.sin) + td, ds);
#pragma unroll
                for (int e = 0; e < SEG; e++) {
                    rc[e] = rope_blend<T>(rc[e], dc[e]);
                    rsn[e] = rope_blend<T>(rsn[e], ds[e]);
                }
            }
#pragma unroll
            for (int e = 0; e < SEG; e++) {
                const float other = __shfl_xor(kh[e], 8);
                kh[e] = rope_elem<T>(kh[e], dl < 8 ? -other : other, rc[e], rsn[e]);
            }
        }
#pragma unroll
        for (int e = 0; e < SEG; e++) kh[e] = Elem<T>::round(kh[e] * p.c_k);
#pragma unroll
        for (int g = 0; g < G; g++) {
            float d = 0.0f;
#pragma unroll
            for (int e = 0; e < SEG; e++) d = __fmaf_rn(qh[g][e], kh[e], d);
            d += __shfl_xor(d, 1);
            d += __shfl_xor(d, 2);
            d += __shfl_xor(d, 4);
            d += __shfl_xor(d, 8);
            if constexpr (CAP) d = tanhf(d / p.softcap) * p.softcap;
            const float x = d * 1.44269504f;
            const float m_new = fmaxf(m[g], x);
            const float alpha = exp2f(m[g] - m_new);
            const float pr = exp2f(x - m_new);
            l[g] = l[g] * alpha + pr * visits;
            const float prT = Elem<T>::round(pr) * visits;
#pragma unroll
            for (int e = 0; e < SEG; e++) acc[g][e] = __fmaf_rn(prT, vv[e], acc[g][e] * alpha);
            m[g] = m_new;
        }
    }

    // merge the 16 group states
#pragma unroll
    for (int g = 0; g < G; g++) {
        if (dl == 0) {
            s_m[grp][g] = m[g];
            s_l[grp][g] = l[g];
        }
#pragma unroll
        for (int e = 0; e < SEG; e++) s_acc[grp][g][dl * SEG + e] = acc[g][e];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * HID; idx += 256) {
        const int g = idx / HID, d = idx % HID;
        float mm = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) mm = fmaxf(mm, s_m[i][g]);
        float ll = 0.0f, aa = 0.0f;
        if (mm > -INFINITY) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float w = exp2f(s_m[i][g] - mm);
                ll += s_l[i][g] * w;
                aa += s_acc[i][g][d] * w;
            }
        }
        float *wrow = dp.ws + (((int64_t)b * p.HEAD + h0 + g) * dp.nsplits + split) * (HID + 4);
        wrow[d] = ll > 0.0f ? aa / ll : 0.0f;
        if (d == 0) wrow[HID] = ll > 0.0f ? mm + log2f(ll) : -INFINITY;
    }
}

// Merge of the per-split partials of one (batch, head): out = sum_s w_s x_s / sum_s w_s with w_s = 2^(lse_s - max lse).
// The partials were written by workgroups all over the chip, so every read is a long-latency one, and the launch is
// small (one workgroup per head): what counts is the number of dependent trips to memory.  A workgroup's 1024 threads
// are 1024 / HID parts x HID columns: a part takes every (1024 / HID)-th split and folds its partials into a running
// (maximum, numerator, denominator), eight splits' loads in flight at a time and no pass over the log-sum-exps
// beforehand; the parts are then folded through LDS (53 splits of 128 columns: one trip; it was three, 6.2 us).
constexpr int MERGE_THREADS = 1024;
constexpr int MERGE_BATCH = 8;

template <typename T, int HID>
__global__ __launch_bounds__(MERGE_THREADS) void bsa_decode_merge_kernel(const float *ws, int HEAD, int nsplits, T *out,
                                                                        int64_t o_sb, int64_t o_sh) {
    constexpr int ROW = HID + 4;
    static_assert(MERGE_THREADS % HID == 0, "a part is a whole row of HID threads");
    constexpr int PARTS = MERGE_THREADS / HID;
    __shared__ float s_m[PARTS][HID], s_num[PARTS][HID], s_den[PARTS][HID];
    const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int part = tid / HID, d = tid % HID;
    const float *base = ws + ((int64_t)b * HEAD + h) * nsplits * ROW;
    float m = -INFINITY, num = 0.0f, den = 0.0f;
    for (int s0 = part; s0 < nsplits; s0 += PARTS * MERGE_BATCH) {
        float lse[MERGE_BATCH], val[MERGE_BATCH];
#pragma unroll
        for (int j = 0; j < MERGE_BATCH; j++) {
            const int s = s0 + j * PARTS;
            const bool ok = s < nsplits;
            const float *row = base + (int64_t)(ok ? s : part) * ROW;
            const float l = row[HID], v = row[d];
            lse[j] = ok ? l : -INFINITY;
            val[j] = v;
        }
#pragma unroll
        for (int j = 0; j < MERGE_BATCH; j++) {
            if (lse[j] > -INFINITY) {
                const float mn = fmaxf(m, lse[j]);
                const float keep = exp2f(m - mn), w = exp2f(lse[j] - mn);  // m = -inf: keep = 0
                num = num * keep + w * val[j];
                den = den * keep + w;
                m = mn;
            }
        }
    }
    s_m[part][d] = m;
    s_num[part][d] = num;
    s_den[part][d] = den;
    __syncthreads();
    if (tid < HID) {
        float mm = -INFINITY;
#pragma unroll
        for (int q = 0; q < PARTS; q++) mm = fmaxf(mm, s_m[q][tid]);
        float n = 0.0f, dd = 0.0f;
        if (mm > -INFINITY) {
#pragma unroll
            for (int q = 0; q < PARTS; q++) {
                const float w = exp2f(s_m[q][tid] - mm);  // parts without a split: exp2(-inf) = 0
                n += w * s_num[q][tid];
                dd += w * s_den[q][tid];
            }
        }
        out[(int64_t)b * o_sb + (int64_t)h * o_sh + tid] = Elem<T>::narrow(dd > 0.0f ? n / dd : 0.0f);
    }
}

template <typename T, int HID>
static int launch_partial(const DecodeParams &dp_in, hipStream_t st) {
    // a workgroup keeps GG heads of a group in registers (GG * HID <= 512); larger groups are shared by several
    // workgroups, each of which reads the rows again
    dim3 grid, block(256);
    bool launched = false;
    DecodeParams dp = dp_in;
#define DEC_CASE(GG)                                                                                   \
    if constexpr (GG * HID <= 512) {                                                                   \
        if (!launched && dp.a.G % GG == 0) {                                                           \
            dp.parts = dp.a.G / GG;                                                                    \
            grid = dim3((unsigned)dp.nsplits, (unsigned)(dp.a.kv.HKV * dp.parts), (unsigned)dp.a.B);   \
            if (sizeof(T) == 2 && dp.a.kx.kv8) {                                                       \
                if constexpr (sizeof(T) == 2) {                                                        \
                    const bool r_ = dp.a.rope.cos != nullptr, c_ = dp.a.softcap != 0.0f;               \
                    if (r_ && c_) hipLaunchKernelGGL((bsa_decode_partial_kernel<T, HID, GG, true, true, true, true>), grid, block, 0, st, dp); \
                    else if (r_) hipLaunchKernelGGL((bsa_decode_partial_kernel<T, HID, GG, true, true, false, true>), grid, block, 0, st, dp); \
                    else if (c_) hipLaunchKernelGGL((bsa_decode_partial_kernel<T, HID, GG, true, false, true, true>), grid, block, 0, st, dp); \
                    else hipLaunchKernelGGL((bsa_decode_partial_kernel<T, HID, GG, true, false, false, true>), grid, block, 0, st, dp); \
                }                                                                                      \
            } else if (dp.a.softcap != 0.0f) {                                                         \
                if (dp.a.rope.cos)                                                                     \
                    hipLaunchKernelGGL((bsa_decode_partial_kernel<T, HID, GG, true, true, true>), grid, block, 0, st, dp); \
                else                                                                                   \
                    hipLaunchKernelGGL((bsa_decode_partial_kernel<T, HID, GG, true, false, true>), grid, block, 0, st, dp); \
            } else if (dp.a.rope.cos) {                                                                \
                hipLaunchKernelGGL((bsa_decode_partial_kernel<T, HID, GG, true, true>), grid, block, 0, st, dp); \
            } else if (dp.a.kx.extended()) {                                                           \
                hipLaunchKernelGGL((bsa_decode_partial_kernel<T, HID, GG, true>), grid, block, 0, st, dp);  \
            } else {                                                                                   \
                DecodeParamsT<false> dq;                                                               \
                dq.a = static_cast<const BsaParamsBase &>(dp.a);                                       \
                dq.nsplits = dp.nsplits;                                                               \
                dq.parts = dp.parts;                                                                   \
                dq.ws = dp.ws;                                                                         \
                hipLaunchKernelGGL((bsa_decode_partial_kernel<T, HID, GG, false>), grid, block, 0, st, dq); \
            }                                                                                          \
            launched = true;                                                                           \
        }                                                                                              \
    }
    DEC_CASE(8) DEC_CASE(4) DEC_CASE(2) DEC_CASE(1)
#undef DEC_CASE
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

}  // namespace hipattn

using namespace hipattn;

extern "C" int64_t hipattn_bsa_decode_workspace_bytes(int32_t B, int32_t HEAD, int32_t HID, int32_t nsplits) {
    if (B <= 0 || HEAD <= 0 || HID <= 0 || nsplits <= 0) return 0;
    return (int64_t)B * HEAD * nsplits * (HID + 4) * (int64_t)sizeof(float);
}

extern "C" int32_t hipattn_bsa_decode_default_splits(int32_t B, int32_t HKV, int32_t tokens) {
    if (B <= 0 || HKV <= 0) return 1;
    int64_t groups = (int64_t)B * HKV;
    int64_t s = (512 + groups - 1) / groups;  // two workgroups per compute unit: all of them resident at once
    int64_t by_tokens = (tokens + 63) / 64;
    if (s > by_tokens) s = by_tokens;
    if (s > 64) s = 64;
    if (s < 1) s = 1;
    return (int32_t)s;
}

extern "C" int hipattn_bsa_decode_partial(const hipattn_q_t *q, const hipattn_kv_t *kv, const int64_t *indices,
                                          const int32_t *ks_start_end, int32_t idx_rows, int32_t BK,
                                          int32_t block_size_k, int32_t sliding_window, int32_t sink,
                                          int32_t second_stage_k, int32_t nsplits, void *workspace, void *stream) {
    DecodeParams dp;
    HIPATTN_CHECK_ARG(workspace, HIPATTN_E_ARG, "decode: null workspace");
    HIPATTN_CHECK_ARG(nsplits >= 1 && nsplits <= 1024, HIPATTN_E_ARG, "decode: nsplits %d out of range", nsplits);
    int rc = bsa_fill_params(q, kv, indices, ks_start_end, idx_rows, BK, 1, block_size_k, sliding_window, sink, 1,
                             workspace, 0, 0, 0, &dp.a);
    if (rc) return rc;
    HIPATTN_CHECK_ARG(q->TDST == 1, HIPATTN_E_ARG, "decode: TDST must be 1, got %d", q->TDST);
    HIPATTN_CHECK_ARG(second_stage_k >= 0, HIPATTN_E_ARG, "decode: negative second_stage_k");
    if (second_stage_k > 0) {
        // the reference launcher's own division of the work among its programs (attention_decode_bsa.py:1070-1077)
        const int64_t total = (int64_t)second_stage_k + sink + sliding_window;
        const int64_t chunk = (total + 7) / 8;
        if (BK > 0) {  // programs over the index row, walking tiles of 16 / block_size_k entries (:1391-1393, :239-247)
            int64_t programs = (second_stage_k + chunk - 1) / chunk;
            if (programs > 12) programs = 12;
            int tile = 16 / block_size_k;
            tile = tile < 1 ? 1 : tile;
            const int share = (int)((BK + programs - 1) / programs);
            dp.a.seam_blocks = share;
            dp.a.seam_extra = (share + tile - 1) / tile * tile - share;
        }
        if (sink > 0) {  // programs over the sink (:514-518)
            int64_t sink_programs = (sink + chunk - 1) / chunk;
            if (sink_programs > 12) sink_programs = 12;
            dp.a.sink_share = (int)((sink + sink_programs - 1) / sink_programs);
        }
    }
    dp.nsplits = nsplits;
    dp.ws = reinterpret_cast<float *>(workspace);
    hipStream_t st = (hipStream_t)stream;
    {
        // matrix-core kernel where it applies (bf16, head dim 64 / 128, groups of up to 8 heads);
        // HIPATTN_DECODE_IMPL=1 keeps the vector-unit kernel (tuning and cross-checking aid)
        static int impl = -1;
        if (impl < 0) {
            const char *e = getenv("HIPATTN_DECODE_IMPL");
            impl = e ? atoi(e) : 0;
        }
        if (impl != 1) {
            rc = bsa_decode_mfma_launch(dp.a, q->dtype, q->HID, nsplits, dp.ws, st);
            if (rc != HIPATTN_E_UNSUPPORTED) return rc;
        }
    }
    if (q->dtype == HIPATTN_BF16) {
        switch (q->HID) {
            case 32: return launch_partial<bf16_t, 32>(dp, st);
            case 64: return launch_partial<bf16_t, 64>(dp, st);
            case 128: return launch_partial<bf16_t, 128>(dp, st);
            case 256: return launch_partial<bf16_t, 256>(dp, st);
        }
    } else {
        switch (q->HID) {
            case 32: return launch_partial<float, 32>(dp, st);
            case 64: return launch_partial<float, 64>(dp, st);
            case 128: return launch_partial<float, 128>(dp, st);
        }
    }
    set_error("decode: head dim %d with dtype %d is not built", q->HID, q->dtype);
    return HIPATTN_E_UNSUPPORTED;
}

extern "C" int hipattn_bsa_decode_merge(const void *workspace, int32_t B, int32_t HEAD, int32_t HID, int32_t nsplits,
                                        int32_t dtype, void *out, int64_t out_stride_b, int64_t out_stride_h,
                                        void *stream);

extern "C" int hipattn_bsa_decode(const hipattn_q_t *q, const hipattn_kv_t *kv, const int64_t *indices,
                                  const int32_t *ks_start_end, int32_t idx_rows, int32_t BK, int32_t block_size_k,
                                  int32_t sliding_window, int32_t sink, int32_t second_stage_k, int32_t nsplits,
                                  void *workspace, void *out, int64_t out_stride_b, int64_t out_stride_h, void *stream) {
    HIPATTN_CHECK_ARG(q && out, HIPATTN_E_ARG, "decode: null pointer");
    const int rc = hipattn_bsa_decode_partial(q, kv, indices, ks_start_end, idx_rows, BK, block_size_k, sliding_window,
                                              sink, second_stage_k, nsplits, workspace, stream);
    if (rc) return rc;
    return hipattn_bsa_decode_merge(workspace, q->B, q->HEAD, q->HID, nsplits, q->dtype, out, out_stride_b, out_stride_h, stream);
}

extern "C" int hipattn_bsa_decode_merge(const void *workspace, int32_t B, int32_t HEAD, int32_t HID, int32_t nsplits,
                                        int32_t dtype, void *out, int64_t out_stride_b, int64_t out_stride_h,
                                        void *stream) {
    HIPATTN_CHECK_ARG(workspace && out, HIPATTN_E_ARG, "decode merge: null pointer");
    HIPATTN_CHECK_ARG(B > 0 && HEAD > 0 && nsplits > 0, HIPATTN_E_ARG, "decode merge: non-positive size");
    HIPATTN_CHECK_ARG(aligned16(workspace), HIPATTN_E_ALIGN, "decode merge: workspace must be 16-byte aligned");
    dim3 grid((unsigned)HEAD, (unsigned)B), block(MERGE_THREADS);
    const float *ws = reinterpret_cast<const float *>(workspace);
    hipStream_t st = (hipStream_t)stream;
#define MERGE_CASE(TT, HH)                                                                                         \
    hipLaunchKernelGGL((bsa_decode_merge_kernel<TT, HH>), grid, block, 0, st, ws, HEAD, nsplits, (TT *)out, \
                       out_stride_b, out_stride_h)
    if (dtype == HIPATTN_BF16) {
        switch (HID) {
            case 32: MERGE_CASE(bf16_t, 32); break;
            case 64: MERGE_CASE(bf16_t, 64); break;
            case 128: MERGE_CASE(bf16_t, 128); break;
            case 256: MERGE_CASE(bf16_t, 256); break;
            default: set_error("decode merge: head dim %d", HID); return HIPATTN_E_UNSUPPORTED;
        }
    } else if (dtype == HIPATTN_F32) {
        switch (HID) {
            case 32: MERGE_CASE(float, 32); break;
            case 64: MERGE_CASE(float, 64); break;
            case 128: MERGE_CASE(float, 128); break;
            default: set_error("decode merge: head dim %d", HID); return HIPATTN_E_UNSUPPORTED;
        }
    } else {
        set_error("decode merge: dtype %d", dtype);
        return HIPATTN_E_UNSUPPORTED;
    }
#undef MERGE_CASE
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

// ------------------------------------------------------------------------------------------------
// Decode attention for callers that cannot allocate: the split partials live in a device array that is
// part of the library's code object instead of a caller-allocated workspace.  Every GPU the library runs
// on holds its own copy of the array at its own address for the life of the process.
namespace hipattn {

constexpr size_t DECODE_SCRATCH_BYTES = HIPATTN_DECODE_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[DECODE_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
static std::atomic<void *> g_scratch_ptr[MAX_DEVICES];

// Device address of `scratch` on the current device, looked up once per device.  The array's name is only a
// host-side handle: kernels and stream operations must be given this address, never the name.
static int decode_scratch(void **out) {
    int dev = -1;
    HIPATTN_CHECK_HIP(hipGetDevice(&dev));
    HIPATTN_CHECK_ARG(dev >= 0 && dev < MAX_DEVICES, HIPATTN_E_UNSUPPORTED, "decode (static scratch): device %d", dev);
    void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        HIPATTN_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        HIPATTN_CHECK_ARG(ptr != nullptr, HIPATTN_E_UNSUPPORTED, "decode (static scratch): no device address");
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // every thread that looks it up gets the same address
    }
    *out = ptr;
    return 0;
}

}  // namespace hipattn

extern "C" int hipattn_bsa_decode_static(const hipattn_q_t *q, const hipattn_kv_t *kv, const int64_t *indices,
                                         const int32_t *ks_start_end, int32_t idx_rows, int32_t BK,
                                         int32_t block_size_k, int32_t sliding_window, int32_t sink,
                                         int32_t second_stage_k, int32_t nsplits, void *out, int64_t out_stride_b,
                                         int64_t out_stride_h, void *stream) {
    HIPATTN_CHECK_ARG(q && kv && out, HIPATTN_E_ARG, "decode (static scratch): null pointer");
    HIPATTN_CHECK_ARG(q->B > 0 && q->HEAD > 0 && q->HID > 0, HIPATTN_E_ARG, "decode (static scratch): non-positive size");
    if (nsplits <= 0) nsplits = hipattn_bsa_decode_default_splits(q->B, kv->HKV, BK * block_size_k + sink + sliding_window + 1);
    const int64_t need = hipattn_bsa_decode_workspace_bytes(q->B, q->HEAD, q->HID, nsplits);
    HIPATTN_CHECK_ARG(need > 0 && (uint64_t)need <= DECODE_SCRATCH_BYTES, HIPATTN_E_UNSUPPORTED,
                      "decode (static scratch): B %d x HEAD %d x nsplits %d x (HID %d + 4) floats = %lld bytes of partials "
                      "exceed the %lld-byte scratch array; use hipattn_bsa_decode_partial with a workspace",
                      q->B, q->HEAD, nsplits, q->HID, (long long)need, (long long)DECODE_SCRATCH_BYTES);
    void *ws = nullptr;
    int rc = decode_scratch(&ws);
    if (rc) return rc;
    // every (sequence, head, split) row of the partials is written by the first launch before the second reads it,
    // so nothing left over from the call before can be seen and nothing needs clearing
    rc = hipattn_bsa_decode_partial(q, kv, indices, ks_start_end, idx_rows, BK, block_size_k, sliding_window, sink,
                                    second_stage_k, nsplits, ws, stream);
    if (rc) return rc;
    return hipattn_bsa_decode_merge(ws, q->B, q->HEAD, q->HID, nsplits, q->dtype, out, out_stride_b, out_stride_h, stream);
}

// Portable block-sparse attention kernel: one wavefront walks one query row at a time.
//
// Covers every dtype / head dim / block size the operator accepts (f32 inputs, odd shapes) and
// serves as the in-library cross-check for the MFMA tile kernel.  It is not the fast path.
// Attended set and softmax follow the same definition as the tile kernel: selected blocks and
// sink tokens at distance >= sliding_window from the query, window tokens at distance <
// sliding_window, base-2 online softmax over f32 logits, probabilities rounded to the input
// type before the value product.
#include "bsa.hpp"

namespace hipattn {

template <typename T, int HID, bool ROPE, bool KV8 = false>
__global__ __launch_bounds__(256) void bsa_simple_kernel(BsaParams p) {
    constexpr int DPL = (HID + 63) / 64;  // output elements per lane
    constexpr int HALF = HID / 2;
    __shared__ float s_q[4][HID];
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int qb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int kvh = h / p.G;
    const int hrow = p.share_first_head ? kvh * p.G : h;
    const int64_t irow = ((int64_t)b * p.HEAD + hrow) * p.idx_rows + qb;

    // CURR = largest position + 1 over the block's rows
    long long curr = 0, pmin = 0x7fffffffffffffffLL;
    int nvalid = 0;  // valid rows of the block
    for (int j = lane; j < p.bq; j += 64) {
        long long it = (long long)qb * p.bq + j;
        if (it < p.TDST) {
            nvalid++;
            long long sl = p.pos[(int64_t)b * p.pos_sb + it * p.pos_st] + 1;
            curr = sl > curr ? sl : curr;
            pmin = sl - 1 < pmin ? sl - 1 : pmin;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        long long w = __shfl_xor(curr, o);
        curr = w > curr ? w : curr;
        long long w2 = __shfl_xor(pmin, o);
        pmin = w2 < pmin ? w2 : pmin;
        nvalid += __shfl_xor(nvalid, o);
    }
    int rs = p.kse[irow * 2 + 0], re = p.kse[irow * 2 + 1];
    const long long rope_shift = pmin - p.sw - p.sink - (long long)(re - rs) * p.bk + 1;
    if (p.BK <= 0) { rs = 0; re = 0; }
    int jend = rs + p.BK < re ? rs + p.BK : re;
    const int nsel = jend > rs ? jend - rs : 0;
    const long long n_sel_tok = (long long)nsel * p.bk;
    const long long sink_end = curr < p.sink ? curr : p.sink;
    long long ws = curr - p.sw - p.bq;
    if (ws < 0) ws = 0;
    const long long n_win = p.sw > 0 ? curr - ws : 0;
    const long long total = n_sel_tok + sink_end + n_win;
    const int64_t seqlen = p.kv.paged ? p.kv.seq_len(b) : 0;
    const void *kbase = p.kv.k;
    const void *vbase = p.kv.v;

    for (int j = wid; j < p.bq; j += 4) {
        const long long it = (long long)qb * p.bq + j;
        if (it >= p.TDST) break;  // uniform per wave
        const long long ppos = p.pos[(int64_t)b * p.pos_sb + it * p.pos_st];
        const T *qrow = reinterpret_cast<const T *>(p.q) + (int64_t)b * p.q_sb + it * p.q_st + (int64_t)h * p.q_sh;
        for (int d = lane; d < HID; d += 64) {
            float x = Elem<T>::widen(qrow[d]);
            if constexpr (ROPE) {  // the query keeps its own position (attention_extend_bsa.py:796-852)
                const int64_t tr = p.rope.row(ppos) + d % HALF;
                const float other = Elem<T>::widen(qrow[(d + HALF) % HID]);
                x = rope_elem<T>(x, d < HALF ? -other : other, Elem<T>::widen(reinterpret_cast<const T *>(p.rope.cos)[tr]),
                                 Elem<T>::widen(reinterpret_cast<const T *>(p.rope.sin)[tr]));
            }
            s_q[wid][d] = Elem<T>::round(x * p.c_q);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        float m = -INFINITY, l = 1.0f;
        float acc[DPL];
#pragma unroll
        for (int e = 0; e < DPL; e++) acc[e] = 0.0f;

        for (long long base = 0; base < total; base += 64) {
            long long o = base + lane;
            long long t = -1;
            int kind = 0;
            bool valid = false;
            long long rpos = 0;  // rotated position of the key (ROPE only)
            if (o < n_sel_tok) {
                const long long st = p.indices[irow * p.BK + rs + o / p.bk];
                t = st + o % p.bk;
                valid = (t >= 0) && (t < p.kv.max_tsrc) && (t < curr) && (t >= p.sink);
                if constexpr (ROPE)
                    rpos = bsa_rope_far_pos(p.rope, (rs + o / p.bk + p.sink / p.bk) * (long long)p.bk + o % p.bk, rope_shift,
                                            pmin, p.sw);
            } else if (o < n_sel_tok + sink_end) {
                t = o - n_sel_tok;
                valid = true;
                if constexpr (ROPE) rpos = bsa_rope_far_pos(p.rope, t, rope_shift, pmin, p.sw);
            } else if (o < total) {
                t = ws + (o - n_sel_tok - sink_end);
                kind = 1;
                valid = true;
                rpos = t;
            }
            const bool att = valid && (p.non_causal || (kind == 0 ? (t + p.sw <= ppos) : (t <= ppos && ppos < t + p.sw)));
            float logit = -INFINITY;
            int64_t voff = NO_ROW;
            if (valid && !att && j == wid && (p.kx.access_flags || p.kx.cached)) {
                // staged for this query block but masked out for this row: the tile kernel loads such rows, so
                // they count as accessed (first row pass of each wave records them)
                int64_t ko, vo;
                kv_rows<false, true>(p.kv, &p.kx, b, t, kvh, seqlen, ko, vo);
            }
            if (att) {
                int64_t koff;
                kv_rows<true, true>(p.kv, &p.kx, b, t, kvh, seqlen, koff, voff);
                float dot = 0.0f;
                if (koff != NO_ROW) {
                    constexpr int CH = 16 / (int)sizeof(T) < HID ? 16 / (int)sizeof(T) : HID;
                    for (int d0 = 0; d0 < HID; d0 += CH) {
                        float kk[CH];
                        load_kv_elems<T, CH, KV8>(kbase, koff + d0, kk);
                        if constexpr (ROPE) {
                            float other[CH], rc[CH], rsn[CH];
                            load_kv_elems<T, CH, KV8>(kbase, koff + (d0 + HALF) % HID, other);
                            const int64_t tr = p.rope.row(rpos) + d0 % HALF;
                            load_elems<T, CH>(reinterpret_cast<const T *>(p.rope.cos) + tr, rc);
                            load_elems<T, CH>(reinterpret_cast<const T *>(p.rope.sin) + tr, rsn);
                            if (kind == 0 && p.rope.backend == HIPATTN_EXTEND_DYNAMIC) {
                                float dc[CH], ds[CH];
                                const int64_t td = p.rope.row(dynamic_extend_pos(t, pmin, pmin + nvalid, p.rope.model_ctx)) + d0 % HALF;
                                load_elems<T, CH>(reinterpret_cast<const T *>(p.rope.cos) + td, dc);
                                load_elems<T, CH>(reinterpret_cast<const T *>(p.rope.sin) + td, ds);
#pragma unroll
                                for (int e = 0; e < CH; e++) {
                                    rc[e] = rope_blend<T>(rc[e], dc[e]);
                                    rsn[e] = rope_blend<T>(rsn[e], ds[e]);
                                }
                            }
#pragma unroll
                            for (int e = 0; e < CH; e++)
                                kk[e] = rope_elem<T>(kk[e], d0 < HALF ? -other[e] : other[e], rc[e], rsn[e]);
                        }
#pragma unroll
                        for (int e = 0; e < CH; e++)
                            dot = __fmaf_rn(s_q[wid][d0 + e], Elem<T>::round(kk[e] * p.c_k), dot);
                    }
                }
                if (p.softcap != 0.0f) dot = tanhf(dot / p.softcap) * p.softcap;
                logit = dot * 1.44269504f;
            }
            const float tile_max = wave_max(logit);
            const float m_new = fmaxf(m, tile_max);
            if (m_new > -INFINITY) {  // uniform
                const float pr = att ? exp2f(logit - m_new) : 0.0f;
                const float alpha = exp2f(m - m_new);
                l = l * alpha + wave_sum(pr);
#pragma unroll
                for (int e = 0; e < DPL; e++) acc[e] *= alpha;
                const float prT = Elem<T>::round(pr);
                unsigned long long live = __ballot(att);
                while (live) {
                    const int src = __ffsll((long long)live) - 1;
                    live &= live - 1;
                    const float pj = __shfl(prT, src);
                    const long long vo = __shfl((long long)voff, src);
                    if (vo != (long long)NO_ROW) {
#pragma unroll
                        for (int e = 0; e < DPL; e++) {
                            const int d = lane + e * 64;
                            if (d < HID) acc[e] = __fmaf_rn(pj, load_kv_elem<T, KV8>(vbase, vo + d), acc[e]);
                        }
                    }
                }
                m = m_new;
            }
        }
        const float denom = (l == 0.0f) ? 1e-20f : l;
        T *orow = reinterpret_cast<T *>(p.out) + (int64_t)b * p.o_sb + it * p.o_st + (int64_t)h * p.o_sh;
#pragma unroll
        for (int e = 0; e < DPL; e++) {
            const int d = lane + e * 64;
            if (d < HID) orow[d] = Elem<T>::narrow(acc[e] / denom);
        }
        __builtin_amdgcn_wave_barrier();
    }
}

template <typename T, int HID>
static int launch_simple(const BsaParams &p, hipStream_t stream) {
    dim3 grid((unsigned)p.NBQ, (unsigned)p.HEAD, (unsigned)p.B), block(256);
    if constexpr (sizeof(T) == 2) {
        if (p.kx.kv8) {
            if (p.rope.cos) hipLaunchKernelGGL((bsa_simple_kernel<T, HID, true, true>), grid, block, 0, stream, p);
            else hipLaunchKernelGGL((bsa_simple_kernel<T, HID, false, true>), grid, block, 0, stream, p);
            HIPATTN_CHECK_HIP(hipGetLastError());
            return 0;
        }
    }
    if (p.rope.cos) hipLaunchKernelGGL((bsa_simple_kernel<T, HID, true>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((bsa_simple_kernel<T, HID, false>), grid, block, 0, stream, p);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

int bsa_fill_params(const hipattn_q_t *q, const hipattn_kv_t *kv, const int64_t *indices, const int32_t *kse,
                    int idx_rows, int BK, int bq, int bk, int sw, int sink, int share_first_head, void *out,
                    int64_t o_sb, int64_t o_st, int64_t o_sh, BsaParams *p) {
    int rc = check_q(q);
    if (rc) return rc;
    HIPATTN_CHECK_ARG(kv && out && kse, HIPATTN_E_ARG, "bsa: null pointer");
    HIPATTN_CHECK_ARG(BK <= 0 || indices, HIPATTN_E_ARG, "bsa: indices is null with BK > 0");
    HIPATTN_CHECK_ARG(bq > 0 && bk > 0 && sw >= 0 && sink >= 0 && idx_rows > 0, HIPATTN_E_ARG, "bsa: bad sizes");
    rc = make_kv_view(kv, q->B, q->HID, q->dtype, &p->kv, &p->kx);
    if (rc) return rc;
    rc = make_rope_view(q, (1u << HIPATTN_EXTEND_STREAMING) | (1u << HIPATTN_EXTEND_INFLLM) | (1u << HIPATTN_EXTEND_DYNAMIC), "bsa",
                        &p->rope);
    if (rc) return rc;
    HIPATTN_CHECK_ARG(q->logit_softcap >= 0.0f, HIPATTN_E_ARG, "bsa: negative logit_softcap");
    p->softcap = q->logit_softcap;
    HIPATTN_CHECK_ARG(q->HEAD % p->kv.HKV == 0, HIPATTN_E_ARG, "bsa: HEAD %% HKV != 0");
    p->q = q->ptr; p->q_sb = q->stride_b; p->q_st = q->stride_t; p->q_sh = q->stride_h;
    p->pos = q->pos; p->pos_sb = q->pos_stride_b; p->pos_st = q->pos_stride_t;
    p->indices = indices; p->kse = kse; p->idx_rows = idx_rows; p->BK = BK; p->bq = bq; p->bk = bk;
    p->sw = sw; p->sink = sink; p->share_first_head = share_first_head;
    p->k_prescaled = 0;
    p->seam_blocks = 0; p->seam_extra = 0; p->sink_share = 0;
    p->non_causal = q->non_causal != 0;
    p->B = q->B; p->TDST = q->TDST; p->HEAD = q->HEAD; p->G = q->HEAD / p->kv.HKV;
    p->NBQ = (q->TDST + bq - 1) / bq;
    HIPATTN_CHECK_ARG(p->NBQ <= idx_rows, HIPATTN_E_ARG, "bsa: %d query blocks but only %d index rows", p->NBQ, idx_rows);
    scale_constants(q->HID, q->dtype, &p->c_q, &p->c_k);
    p->out = out; p->o_sb = o_sb; p->o_st = o_st; p->o_sh = o_sh;
    return 0;
}

int bsa_simple_launch(const BsaParams &p, int dtype, int HID, hipStream_t st) {
    if (dtype == HIPATTN_BF16) {
        switch (HID) {
            case 32: return launch_simple<bf16_t, 32>(p, st);
            case 64: return launch_simple<bf16_t, 64>(p, st);
            case 128: return launch_simple<bf16_t, 128>(p, st);
            case 256: return launch_simple<bf16_t, 256>(p, st);
        }
    } else if (dtype == HIPATTN_F32) {
        switch (HID) {
            case 32: return launch_simple<float, 32>(p, st);
            case 64: return launch_simple<float, 64>(p, st);
            case 128: return launch_simple<float, 128>(p, st);
            case 256: return launch_simple<float, 256>(p, st);
        }
    }
    set_error("bsa: head dim %d with dtype %d is not built", HID, dtype);
    return HIPATTN_E_UNSUPPORTED;
}

}  // namespace hipattn

// Mask-estimation scan stage: per (batch, scan row, head, chunk) binary-search refinement + score.
//
// One wavefront plays one program of the reference kernel (a group of `block_chunk` <= 64 chunks
// of one (batch, head, scan row)), because the reference's gate and iteration count are
// program-level quantities.  Inside the wave, 16 lanes share one sampled key row (each lane owns
// HID/16 contiguous head-dim elements, so a row is one fully coalesced 16-lane load), four key
// rows are in flight per load instruction, and the dot product is reduced across the 16 lanes in
// the fixed order  [FMA chain over the lane's elements] -> [adjacent-pair tree over lanes],
// which makes scores reproducible bit for bit on any implementation that follows the same order.
#include "mask_common.hpp"

namespace hipattn {

template <int N>
__device__ __forceinline__ void rs_step(const float (&in)[N], float (&out)[N / 2], bool hi, int xmask) {
#pragma unroll
    for (int i = 0; i < N / 2; i++) {
        float a = in[2 * i], b = in[2 * i + 1];
        float keep = hi ? b : a;
        float send = hi ? a : b;
        out[i] = keep + __shfl_xor(send, xmask);
    }
}

// Sum part[r] over the 16 lanes of a row group in adjacent-pair tree order.  Returns, in lane dl,
// the total for row (dl & (ROWS-1)).
template <int ROWS>
__device__ __forceinline__ float reduce16(const float (&part)[ROWS], int dl) {
    if constexpr (ROWS == 16) {
        float a[8], b[4], c[2], d[1];
        rs_step<16>(part, a, dl & 1, 1);
        rs_step<8>(a, b, dl & 2, 2);
        rs_step<4>(b, c, dl & 4, 4);
        rs_step<2>(c, d, dl & 8, 8);
        return d[0];
    } else if constexpr (ROWS == 4) {
        float a[2], b[1];
        rs_step<4>(part, a, dl & 1, 1);
        rs_step<2>(a, b, dl & 2, 2);
        float v = b[0];
        v += __shfl_xor(v, 4);
        v += __shfl_xor(v, 8);
        return v;
    } else {
        static_assert(ROWS == 1, "ROWS is 1, 4 or 16");
        float v = part[0];
        v += __shfl_xor(v, 1);
        v += __shfl_xor(v, 2);
        v += __shfl_xor(v, 4);
        v += __shfl_xor(v, 8);
        return v;
    }
}

// Position a query row is rotated to in the mask stage (attention_extend.py:632-647)
__device__ __forceinline__ int64_t mask_rope_qpos(const RopeView &r, long long pos, int n, int sw_eff) {
    if (r.backend == HIPATTN_EXTEND_RELATIVE) return 1 + (int64_t)sw_eff;
    if (r.backend == HIPATTN_EXTEND_INFLLM) return sw_eff;
    if (rope_follows_token(r.backend)) return pos;
    const long long cap = (long long)n + sw_eff;
    return pos < cap ? pos : cap;
}
// Position the sampled key of chunk `c`, token `t`, is rotated to (attention_extend.py:254-298)
__device__ __forceinline__ int64_t mask_rope_kpos(const RopeView &r, int c, int side, int t, int64_t pmin, int64_t pmax) {
    if (r.backend == HIPATTN_EXTEND_RELATIVE) return side;
    if (r.backend == HIPATTN_EXTEND_STREAMING) return c;
    if (rope_follows_token(r.backend)) return token_extend_pos(r, t, pmin, pmax);
    return 0;
}

template <typename T, int HID, int ROWS, int MAXROWS, int STEPS, bool ROPE>
__global__ __launch_bounds__(64) void mask_stage_kernel(MaskParams p) {
    constexpr int SEG = HID / 16;
    constexpr int HALF = HID / 2;
    __shared__ int64_t s_koff[128];
    __shared__ float s_sc[128];
    __shared__ int s_kt[ROPE ? 128 : 1];  // token of each sample (the DYNAMIC rule rotates by it)
    __shared__ __align__(16) T s_q[MAXROWS * HID];

    const int lane = threadIdx.x;
    const int sub = lane >> 4;
    const int dl = lane & 15;

    long long L = xcd_remap((long long)blockIdx.x, p.total);
    const int hin = (int)(L % p.G);
    L /= p.G;
    const int s = (int)(L % p.BS);
    L /= p.BS;
    const int g = (int)(L % p.ngroups);
    L /= p.ngroups;
    const int kvh = (int)(L % p.kv.HKV);
    const int b = (int)(L / p.kv.HKV);
    const int h = kvh * p.G + hin;

    const int BC = p.block_chunk;
    const int ci = g * BC + lane;
    const bool real = (lane < BC) && (ci < p.n);
    const int hgi = p.hg == 1 ? 0 : h;
    const int64_t row_in = (((int64_t)b * p.BS + s) * p.hg + hgi) * p.n;
    const int64_t row_out = (((int64_t)b * p.BS + s) * p.HEAD + h) * p.n;
    const int64_t red_out = ((int64_t)b * p.BS + s) * p.n;

    int l = (int)p.kv.max_tsrc, r = (int)p.kv.max_tsrc;
    if (real) {
        l = p.chunk_left[row_in + ci];
        int64_t rr = (int64_t)l + p.chunk;
        r = (int)(rr < p.right_clamp ? rr : p.right_clamp);
    }
    float score = -32000.0f;

    // rows of this program
    const long long qb = (long long)(p.BDST - 1) - (long long)(p.BS - 1) * p.scan_stride + (long long)s * p.scan_stride;
    long long myrow = qb * p.BQ + (long long)lane * p.stride_q;
    bool rv = (lane < p.nrows) && (myrow >= 0) && (myrow < p.TDST);
    const unsigned long long rowmask = __ballot(rv);
    long long mypos = rv ? p.pos[(int64_t)b * p.pos_sb + myrow * p.pos_st] : 0x7fffffffffffffffLL;
    const long long pmin = wave_min_ll(mypos);

    bool run = (rowmask != 0ull) && (pmin >= 0);
    int lim = 0;
    float width = 0.0f;
    if (run) {
        long long lm = pmin - p.sw_eff;
        lim = (int)(lm < 0 ? 0 : lm);
        const int minl = wave_min_i(l);
        run = (pmin + (long long)p.BQ * p.scan_stride >= (long long)minl);
        width = (float)wave_max_i(r - l);
    }
    if (!run || !(width >= p.terminate)) {
        if (real) {
            store_score(p, row_out, red_out, ci, score);
            if (p.left_out) p.left_out[row_out + ci] = l;
        }
        return;
    }

    // q^ rows: strided mean -> T -> *c_q -> T, staged in LDS
    const T *qbase = reinterpret_cast<const T *>(p.q) + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
    const int rows_here = p.nrows < MAXROWS ? p.nrows : MAXROWS;
    for (int idx = lane; idx < rows_here * HID; idx += 64) {
        const int j = idx / HID, d = idx % HID;
        float qh = 0.0f;
        if ((rowmask >> j) & 1ull) {
            const long long it = qb * p.BQ + (long long)j * p.stride_q;
            float sum = 0.0f;
            int cnt = 0;
            float rc = 0.0f, rsn = 0.0f;
            if constexpr (ROPE) {
                // every strided row is rotated to the position derived from the base row
                const int64_t tr = p.rope.row(mask_rope_qpos(p.rope, p.pos[(int64_t)b * p.pos_sb + it * p.pos_st], p.n, p.sw_eff));
                rc = Elem<T>::widen(reinterpret_cast<const T *>(p.rope.cos)[tr + d % HALF]);
                rsn = Elem<T>::widen(reinterpret_cast<const T *>(p.rope.sin)[tr + d % HALF]);
            }
            for (int o = 0; o < p.stride_q; o++) {
                if (it + o < p.TDST) {
                    float x = Elem<T>::widen(qbase[(it + o) * p.q_st + d]);
                    if constexpr (ROPE) {
                        const float other = Elem<T>::widen(qbase[(it + o) * p.q_st + (d + HALF) % HID]);
                        x = rope_elem<T>(x, d < HALF ? -other : other, rc, rsn);
                    }
                    sum += x;
                    cnt++;
                }
            }
            float mean = Elem<T>::round(__fdiv_rn(sum, (float)cnt + 1e-12f));
            qh = Elem<T>::round(mean * p.c_q);
        }
        s_q[idx] = Elem<T>::narrow(qh);
    }
    __syncthreads();

    const int npass = (rows_here + ROWS - 1) / ROWS;
    float qh[ROWS][SEG];
    auto load_q_pass = [&](int pass) {
#pragma unroll
        for (int rr = 0; rr < ROWS; rr++) {
            const int j = pass * ROWS + rr;
            if (j < rows_here) {
                load_elems<T, SEG>(&s_q[j * HID + dl * SEG], qh[rr]);
            } else {
#pragma unroll
                for (int e = 0; e < SEG; e++) qh[rr][e] = 0.0f;
            }
        }
    };
    if (npass == 1) load_q_pass(0);

    const int64_t seqlen = p.kv.paged ? p.kv.seq_len(b) : 0;
    const T *kbase = reinterpret_cast<const T *>(p.kv.k);
    const int nsteps = BC / 2;

    while (width >= p.terminate) {
        width *= 0.5f;
        const bool active = real && (l < r) && (l <= lim) && (l >= 0);
        const int c = (l + r) >> 1;
        if (lane < BC) {
            int64_t o0 = NO_ROW, o1 = NO_ROW;
            if (active) {
                o0 = kv_k_row<true>(p.kv, &p.kx, b, (l + c) >> 1, kvh, seqlen);
                o1 = kv_k_row<true>(p.kv, &p.kx, b, (c + r) >> 1, kvh, seqlen);
            }
            s_koff[2 * lane] = o0;
            s_koff[2 * lane + 1] = o1;
            if constexpr (ROPE) {
                s_kt[2 * lane] = (l + c) >> 1;
                s_kt[2 * lane + 1] = (c + r) >> 1;
            }
            s_sc[2 * lane] = -INFINITY;
            s_sc[2 * lane + 1] = -INFINITY;
        }
        __syncthreads();

        for (int cs = 0; cs < nsteps; cs += STEPS) {
            RawSlice<T, SEG> raw[STEPS];
#pragma unroll
            for (int st = 0; st < STEPS; st++) {
                const int krow = (cs + st) * 4 + sub;
                const int64_t off = (cs + st) < nsteps ? s_koff[krow] : -1;
                if (off != NO_ROW) raw[st].load(kbase + off + dl * SEG);
                else raw[st].zero();
            }
            for (int pass = 0; pass < npass; pass++) {
                if (npass > 1) load_q_pass(pass);
                const int j = pass * ROWS + (dl & (ROWS - 1));
                const bool jvalid = (j < p.nrows) && ((rowmask >> j) & 1ull);
#pragma unroll
                for (int st = 0; st < STEPS; st++) {
                    if ((cs + st) < nsteps) {
                        float kh[SEG];
                        raw[st].widen(kh);
                        if constexpr (ROPE) {
                            // lanes dl and dl ^ 8 of a row group hold the two halves of the row
                            const int krow = (cs + st) * 4 + sub;
                            const int64_t tr = p.rope.row(mask_rope_kpos(p.rope, g * BC + (krow >> 1), krow & 1, s_kt[krow], pmin,
                                                                      pmin + __popcll(rowmask))) + (dl & 7) * SEG;
                            float rc[SEG], rsn[SEG];
                            load_elems<T, SEG>(reinterpret_cast<const T *>(p.rope.cos) + tr, rc);
                            load_elems<T, SEG>(reinterpret_cast<const T *>(p.rope.sin) + tr, rsn);
#pragma unroll
                            for (int e = 0; e < SEG; e++) {
                                const float other = __shfl_xor(kh[e], 8);
                                kh[e] = rope_elem<T>(kh[e], dl < 8 ? -other : other, rc[e], rsn[e]);
                            }
                        }
#pragma unroll
                        for (int e = 0; e < SEG; e++) kh[e] = Elem<T>::round(kh[e] * p.c_k);
                        float part[ROWS];
#pragma unroll
                        for (int rr = 0; rr < ROWS; rr++) {
                            float acc = 0.0f;
#pragma unroll
                            for (int e = 0; e < SEG; e++) acc = __fmaf_rn(qh[rr][e], kh[e], acc);
                            part[rr] = acc;
                        }
                        float v = Elem<T>::round(reduce16<ROWS>(part, dl));
                        v = jvalid ? v : -INFINITY;
                        if constexpr (ROWS > 1) {
                            v = fmaxf(v, __shfl_xor(v, 1));
                            if constexpr (ROWS > 2) v = fmaxf(v, __shfl_xor(v, 2));
                            if constexpr (ROWS > 4) {
                                v = fmaxf(v, __shfl_xor(v, 4));
                                v = fmaxf(v, __shfl_xor(v, 8));
                            }
                        }
                        if (dl == 0) {
                            const int krow = (cs + st) * 4 + sub;
                            s_sc[krow] = fmaxf(s_sc[krow], v);
                        }
                    }
                }
            }
        }
        __syncthreads();
        if (active) {
            const float sL = s_sc[2 * lane], sR = s_sc[2 * lane + 1];
            const bool win = sL > sR;
            if (win) r = c; else l = c;
            score = fmaxf(score, win ? sL : sR);
        }
        __syncthreads();
    }
    if (real) {
        store_score(p, row_out, red_out, ci, score);
        if (p.left_out) p.left_out[row_out + ci] = l;
    }
}

__global__ void fill_scores_kernel(float *scores, long long n, float v) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
        scores[i] = v;
}

template <typename T, int HID, bool ROPE>
static int launch_mask(const MaskParams &p, int rows_eff, hipStream_t stream) {
    dim3 grid((unsigned)p.total), block(64);
    if (rows_eff <= 1) {
        if (p.block_chunk == 64)
            hipLaunchKernelGGL((mask_stage_kernel<T, HID, 1, 1, 32, ROPE>), grid, block, 0, stream, p);
        else
            hipLaunchKernelGGL((mask_stage_kernel<T, HID, 1, 1, 8, ROPE>), grid, block, 0, stream, p);
    } else if (rows_eff <= 4) {
        hipLaunchKernelGGL((mask_stage_kernel<T, HID, 4, 4, 8, ROPE>), grid, block, 0, stream, p);
    } else if (rows_eff <= 16) {
        hipLaunchKernelGGL((mask_stage_kernel<T, HID, 16, 16, 8, ROPE>), grid, block, 0, stream, p);
    } else if (rows_eff <= 64) {
        hipLaunchKernelGGL((mask_stage_kernel<T, HID, 16, 64, 8, ROPE>), grid, block, 0, stream, p);
    } else {
        set_error("mask stage: %d query rows per program exceed the supported 64", rows_eff);
        return HIPATTN_E_UNSUPPORTED;
    }
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

}  // namespace hipattn

using namespace hipattn;

extern "C" int hipattn_mask_stage(const hipattn_q_t *q, const hipattn_kv_t *kv, const int32_t *chunk_left,
                                  int32_t hg, int32_t n, int32_t chunk_size, int64_t right_clamp,
                                  int32_t bs, int32_t bq, int32_t stride_q, int32_t block_chunk,
                                  int32_t scan_stride, int32_t sw_eff, int32_t terminate_size,
                                  int32_t k_prescaled, int32_t reduce_heads, void *workspace, float *scores,
                                  int32_t *left_out, void *stream) {
    int rc = check_q(q);
    if (rc) return rc;
    HIPATTN_CHECK_ARG(kv && chunk_left && scores, HIPATTN_E_ARG, "mask stage: null pointer");
    HIPATTN_CHECK_ARG(n >= 0 && chunk_size > 0 && bs > 0 && bq > 0 && stride_q > 0 && scan_stride > 0,
                      HIPATTN_E_ARG, "mask stage: non-positive size");
    HIPATTN_CHECK_ARG(hg == 1 || hg == q->HEAD, HIPATTN_E_ARG, "mask stage: hg must be 1 or HEAD");
    HIPATTN_CHECK_ARG(block_chunk == 16 || block_chunk == 32 || block_chunk == 64, HIPATTN_E_UNSUPPORTED,
                      "mask stage: block_chunk %d not in {16,32,64}", block_chunk);
    HIPATTN_CHECK_ARG(bq % stride_q == 0 || bq / stride_q > 0, HIPATTN_E_ARG, "mask stage: bad stride_q");
    HIPATTN_CHECK_ARG(terminate_size >= 1, HIPATTN_E_ARG, "mask stage: terminate_size < 1");
    if (n == 0) return 0;
    MaskParams p;
    p.group_reps = 1;
    p.share_first = 0;
    rc = make_kv_view(kv, q->B, q->HID, q->dtype, &p.kv, &p.kx);
    if (rc) return rc;
    rc = make_rope_view(q, (1u << HIPATTN_EXTEND_RELATIVE) | (1u << HIPATTN_EXTEND_STREAMING) | (1u << HIPATTN_EXTEND_INFLLM) |
                               (1u << HIPATTN_EXTEND_DYNAMIC) | (1u << HIPATTN_EXTEND_SELF),
                        "mask stage", &p.rope);
    if (rc) return rc;
    HIPATTN_CHECK_ARG(k_prescaled >= 0 && k_prescaled <= 7, HIPATTN_E_ARG, "mask stage: k_prescaled %d not in 0..7", k_prescaled);
    // (STREAMING: the caller vouches that every key row was rotated to the place of its chunk in THIS stage's list,
    // hipattn_prescale_k_rope_chunks; that holds for a first stage, whose list is every chunk in order)
    HIPATTN_CHECK_ARG(!(p.rope.cos && (k_prescaled & 1)) || p.rope.backend == HIPATTN_EXTEND_RELATIVE ||
                          p.rope.backend == HIPATTN_EXTEND_INFLLM || p.rope.backend == HIPATTN_EXTEND_STREAMING,
                      HIPATTN_E_ARG, "mask stage: prescaled keys need a rule with key positions known ahead (relative, infllm, "
                                     "streaming on a first stage)");
    if (p.rope.backend != HIPATTN_EXTEND_RELATIVE || !(k_prescaled & 1)) p.rope.k_side_delta = 0;
    HIPATTN_CHECK_ARG(p.rope.k_side_delta % 8 == 0, HIPATTN_E_ALIGN, "mask stage: k_side_delta must keep 16-byte alignment");
    HIPATTN_CHECK_ARG(q->HEAD % p.kv.HKV == 0, HIPATTN_E_ARG, "mask stage: HEAD %% HKV != 0");
    p.q = q->ptr; p.q_sb = q->stride_b; p.q_st = q->stride_t; p.q_sh = q->stride_h;
    p.pos = q->pos; p.pos_sb = q->pos_stride_b; p.pos_st = q->pos_stride_t;
    p.chunk_left = chunk_left; p.hg = hg; p.n = n; p.chunk = chunk_size; p.right_clamp = right_clamp;
    p.B = q->B; p.TDST = q->TDST; p.HEAD = q->HEAD; p.G = q->HEAD / p.kv.HKV;
    p.BQ = bq; p.BDST = (q->TDST + bq - 1) / bq; p.BS = bs; p.stride_q = stride_q;
    p.nrows = bq / stride_q;
    HIPATTN_CHECK_ARG(p.nrows >= 1, HIPATTN_E_ARG, "mask stage: stride_q larger than block");
    HIPATTN_CHECK_ARG(bs == (p.BDST + scan_stride - 1) / scan_stride, HIPATTN_E_ARG,
                      "mask stage: bs %d does not match cdiv(BDST %d, scan_stride %d)", bs, p.BDST, scan_stride);
    p.block_chunk = block_chunk; p.scan_stride = scan_stride; p.sw_eff = sw_eff;
    p.terminate = (float)terminate_size;
    p.ngroups = (n + block_chunk - 1) / block_chunk;
    p.total = (long long)q->B * q->HEAD * bs * p.ngroups;
    HIPATTN_CHECK_ARG(p.total < 0x7fffffffLL, HIPATTN_E_UNSUPPORTED, "mask stage: grid too large");
    scale_constants(q->HID, q->dtype, &p.c_q, &p.c_k);
    p.scores = scores; p.left_out = left_out;
    HIPATTN_CHECK_ARG(reduce_heads >= 0 && reduce_heads <= 2, HIPATTN_E_ARG, "mask stage: reduce_heads %d not in {0, 1, 2}", reduce_heads);
    p.reduce_heads = reduce_heads;  // 2: the scores were set to -inf by the caller
    HIPATTN_CHECK_ARG(!reduce_heads || hg == 1, HIPATTN_E_ARG, "mask stage: reduce_heads needs one shared chunk list (hg == 1)");
    int rows_max = (q->TDST + stride_q - 1) / stride_q;
    int rows_eff = p.nrows < rows_max ? p.nrows : rows_max;
    if (p.nrows > 64) {
        set_error("mask stage: %d query rows per program exceed the supported 64", p.nrows);
        return HIPATTN_E_UNSUPPORTED;
    }
    // the kernel indexes rows up to nrows; MAXROWS must cover every row that can be valid
    hipStream_t st = (hipStream_t)stream;
    if (q->dtype == HIPATTN_BF16) {
        HIPATTN_CHECK_ARG(workspace && aligned16(workspace), HIPATTN_E_ARG,
                          "mask stage: bf16 inputs need a 16-byte aligned workspace (hipattn_mask_stage_workspace_bytes)");
        p.qhat = reinterpret_cast<const uint16_t *>(workspace);
        return mask_stage_mfma_launch(p, q->HID, rows_eff, k_prescaled, st);  // bit 0: keys, bit 1: query rows ready, bit 2: paged pool under 32 GiB
    } else if (q->dtype == HIPATTN_F32) {
        HIPATTN_CHECK_ARG(!(k_prescaled & 1), HIPATTN_E_ARG, "mask stage: prescaled keys are a bf16-only option");
        if (p.reduce_heads == 1) {
            const long long nscores = (long long)p.B * p.BS * p.n;
            hipLaunchKernelGGL(fill_scores_kernel, dim3((unsigned)((nscores + 255) / 256 < 4096 ? (nscores + 255) / 256 : 4096)),
                               dim3(256), 0, st, scores, nscores, -INFINITY);
        }
        const bool rope = p.rope.cos != nullptr;
        switch (q->HID) {
            case 32: return rope ? launch_mask<float, 32, true>(p, rows_eff, st) : launch_mask<float, 32, false>(p, rows_eff, st);
            case 64: return rope ? launch_mask<float, 64, true>(p, rows_eff, st) : launch_mask<float, 64, false>(p, rows_eff, st);
            case 128: return rope ? launch_mask<float, 128, true>(p, rows_eff, st) : launch_mask<float, 128, false>(p, rows_eff, st);
        }
    }
    set_error("mask stage: head dim %d with dtype %d is not built", q->HID, q->dtype);
    return HIPATTN_E_UNSUPPORTED;
}

extern "C" int hipattn_kv_rows_beyond_32gib(const hipattn_kv_t *kv, int32_t B, int32_t HID, int32_t dtype) {
    if (!kv || B < 0 || HID <= 0) return HIPATTN_E_ARG;
    KVView v{};
    v.paged = kv->paged;
    v.k_stride_b = kv->k_stride_b;
    v.k_stride_t = kv->k_stride_t;
    v.k_stride_h = kv->k_stride_h;
    v.tsrc = kv->tsrc;
    v.HKV = kv->HKV;
    const int esz = kv->fp8 ? 1 : dtype == HIPATTN_F32 ? 4 : 2;
    return kv_rows_beyond_32gib(v, B, HID, esz, 0, false) ? 1 : 0;
}

extern "C" int64_t hipattn_mask_stage_workspace_bytes(int32_t dtype, int32_t B, int32_t bs, int32_t HEAD, int32_t HID,
                                                      int32_t bq, int32_t stride_q) {
    if (dtype != HIPATTN_BF16 || B <= 0 || bs <= 0 || HEAD <= 0 || HID <= 0 || bq <= 0 || stride_q <= 0) return 0;
    return (int64_t)B * bs * HEAD * (bq / stride_q) * HID * 2;
}

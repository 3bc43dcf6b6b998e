// MFMA tile kernel for block-sparse attention (bf16, head dim 64 / 128, query block <= 64 rows).
//
// One workgroup = one (batch, kv head, query block) and up to four query heads of the GQA group,
// one head per wavefront, so every gathered K/V tile in LDS is consumed by the whole group.
// Per 64-token tile:   S^T[token, query] = K^ . Q^^T      (v_mfma_f32_32x32x16_bf16, K^ from LDS,
//                                                           Q^ resident in registers)
//                      online softmax down the token axis  (a lane owns one query column)
//                      O^T[d, query]    += V^T . P^T        (V staged transposed in LDS; P^T is
//                                                           taken straight from the S^T registers)
// Working on the transposed problem keeps the softmax statistics lane-local and lets P feed the
// second MFMA without a trip through LDS.  Global loads of tile i+1 are issued before the math of
// tile i; LDS is double-buffered so one barrier per tile suffices.
#include "bsa.hpp"

namespace hipattn {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int TN = 64;        // tokens per tile
constexpr int KPAD = 8;       // bf16 elements of row padding for the K^ tile
constexpr int VPAD = 4;       // bf16 elements of row padding for the V^T tile
constexpr float LOG2E = 1.44269504f;

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    return (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(b) << 16);
}

union Frag {
    bf16x8 v;
    uint32_t u[4];
    uint2 d[2];
    uint4 q;
};

template <int HID>
struct MfmaSmem {
    uint16_t k[2][TN][HID + KPAD];
    uint16_t vt[2][HID][TN + VPAD];
    int tok[2][TN];
};

template <int HID>
__global__ __launch_bounds__(256) void bsa_mfma_kernel(BsaParams p, int hgroups, int hpw, long long total_wg) {
    constexpr int KS = HID / 16;   // k-steps of the first product
    constexpr int DB = HID / 32;   // 32-row blocks of O^T
    constexpr int CPT = TN * (HID / 8) / 256;  // 16-byte chunks per thread per tile
    extern __shared__ __align__(16) unsigned char smem_raw[];
    MfmaSmem<HID> &sm = *reinterpret_cast<MfmaSmem<HID> *>(smem_raw);

    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int col = lane & 31, hh = lane >> 5;

    long long L = xcd_remap((long long)blockIdx.x, total_wg);
    const int qb = (int)(L % p.NBQ);
    L /= p.NBQ;
    const int hgrp = (int)(L % hgroups);
    L /= hgroups;
    const int kvh = (int)(L % p.kv.HKV);
    const int b = (int)(L / p.kv.HKV);
    const int hin = hgrp * hpw + wid;
    const bool head_ok = (wid < hpw) && (hin < p.G);
    const int h = kvh * p.G + (head_ok ? hin : 0);
    // index row: the group's first head when rows are shared, else the single head this workgroup serves
    const int hrow = p.share_first_head ? kvh * p.G : kvh * p.G + hgrp * hpw;
    const int64_t irow = ((int64_t)b * p.HEAD + hrow) * p.idx_rows + qb;

    // ---- query block geometry
    int pm[2];
    int pmin_blk = 0x7fffffff, pmax_blk = -1;
    {
        long long cur = -1, mn = 0x7fffffff;
        for (int j = lane; j < p.bq; j += 64) {
            long long it = (long long)qb * p.bq + j;
            if (it < p.TDST) {
                long long ps = p.pos[(int64_t)b * p.pos_sb + it * p.pos_st];
                cur = ps > cur ? ps : cur;
                mn = ps < mn ? ps : mn;
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            long long w = __shfl_xor(cur, o);
            cur = w > cur ? w : cur;
            long long w2 = __shfl_xor(mn, o);
            mn = w2 < mn ? w2 : mn;
        }
        pmax_blk = (int)cur;
        pmin_blk = (int)mn;
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
            const int j = mb * 32 + col;
            const long long it = (long long)qb * p.bq + j;
            pm[mb] = (j < p.bq && it < p.TDST) ? (int)p.pos[(int64_t)b * p.pos_sb + it * p.pos_st] : -0x40000000;
        }
    }
    const int curr = pmax_blk + 1;
    int rs = p.kse[irow * 2 + 0], re = p.kse[irow * 2 + 1];
    if (p.BK <= 0) { rs = 0; re = 0; }
    const int jend = rs + p.BK < re ? rs + p.BK : re;
    const int nsel = jend > rs ? jend - rs : 0;
    const int n_sel_tok = nsel * p.bk;
    const int sink_end = curr < p.sink ? curr : p.sink;
    int ws = curr - p.sw - p.bq;
    if (ws < 0) ws = 0;
    const int n_win = p.sw > 0 ? curr - ws : 0;
    const int tiles_sel = (n_sel_tok + TN - 1) / TN;
    const int tiles_sink = (sink_end + TN - 1) / TN;
    const int tiles_win = (n_win + TN - 1) / TN;
    const int ntiles = tiles_sel + tiles_sink + tiles_win;

    // ---- Q^ fragments (B operand of the first product), resident for the whole kernel
    Frag qf[2][KS];
    {
        const uint16_t *qbase = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
            const int j = mb * 32 + col;
            const long long it = (long long)qb * p.bq + j;
            const bool ok = head_ok && (j < p.bq) && (it < p.TDST);
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                uint4 raw = make_uint4(0, 0, 0, 0);
                if (ok) raw = *reinterpret_cast<const uint4 *>(qbase + it * p.q_st + ks * 16 + hh * 8);
                const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float lo = __uint_as_float(w[e] << 16) * p.c_q;
                    const float hi = __uint_as_float(w[e] & 0xffff0000u) * p.c_q;
                    qf[mb][ks].u[e] = pack_bf16(lo, hi);
                }
            }
        }
    }

    const int64_t seqlen = p.kv.paged ? p.kv.seq_len(b) : 0;
    const uint16_t *kbase = reinterpret_cast<const uint16_t *>(p.kv.k);
    const uint16_t *vbase = reinterpret_cast<const uint16_t *>(p.kv.v);

    // ---- staging: thread handles chunks c = tid + 256*j: token slot c / (HID/8), 16-byte piece c % (HID/8)
    uint4 kreg[CPT], vreg[CPT];
    int treg[CPT];
    auto prefetch = [&](int tile) {
        int kind, base;  // kind 0 selected, 1 sink, 2 window
        if (tile < tiles_sel) { kind = 0; base = tile * TN; }
        else if (tile < tiles_sel + tiles_sink) { kind = 1; base = (tile - tiles_sel) * TN; }
        else { kind = 2; base = (tile - tiles_sel - tiles_sink) * TN; }
#pragma unroll
        for (int j = 0; j < CPT; j++) {
            const int c = tid + 256 * j;
            const int slot = c / (HID / 8), piece = c % (HID / 8);
            const int o = base + slot;
            long long t = -1;
            if (kind == 0) {
                if (o < n_sel_tok) {
                    const long long st = p.indices[irow * p.BK + rs + o / p.bk];
                    t = st + o % p.bk;
                    if (!(t >= 0 && t < p.kv.max_tsrc && t < curr && t >= p.sink)) t = -1;
                }
            } else if (kind == 1) {
                if (o < sink_end) t = o;
            } else {
                if (o < n_win) t = ws + o;
            }
            treg[j] = (int)t;
            kreg[j] = make_uint4(0, 0, 0, 0);
            vreg[j] = make_uint4(0, 0, 0, 0);
            if (t >= 0) {
                const int64_t ko = p.kv.k_row(b, t, kvh, seqlen);
                const int64_t vo = p.kv.v_row(b, t, kvh, seqlen);
                if (ko >= 0) kreg[j] = *reinterpret_cast<const uint4 *>(kbase + ko + piece * 8);
                if (vo >= 0) vreg[j] = *reinterpret_cast<const uint4 *>(vbase + vo + piece * 8);
            }
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int j = 0; j < CPT; j++) {
            const int c = tid + 256 * j;
            const int slot = c / (HID / 8), piece = c % (HID / 8);
            const uint32_t kw[4] = {kreg[j].x, kreg[j].y, kreg[j].z, kreg[j].w};
            uint32_t ko[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float lo = __uint_as_float(kw[e] << 16) * p.c_k;
                const float hi = __uint_as_float(kw[e] & 0xffff0000u) * p.c_k;
                ko[e] = pack_bf16(lo, hi);
            }
            *reinterpret_cast<uint4 *>(&sm.k[buf][slot][piece * 8]) = make_uint4(ko[0], ko[1], ko[2], ko[3]);
            const uint32_t vw[4] = {vreg[j].x, vreg[j].y, vreg[j].z, vreg[j].w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                sm.vt[buf][piece * 8 + 2 * e][slot] = (uint16_t)(vw[e] & 0xffffu);
                sm.vt[buf][piece * 8 + 2 * e + 1][slot] = (uint16_t)(vw[e] >> 16);
            }
            if (piece == 0) sm.tok[buf][slot] = treg[j];
        }
    };

    // ---- running state (per lane: two query columns)
    f32x16 oacc[DB][2];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
            for (int i = 0; i < 16; i++) oacc[db][mb][i] = 0.0f;
    float m_run[2] = {-INFINITY, -INFINITY};
    float l_run[2] = {0.0f, 0.0f};

    if (ntiles > 0) prefetch(0);
    for (int tile = 0; tile < ntiles; tile++) {
        const int buf = tile & 1;
        commit(buf);
        __syncthreads();
        if (tile + 1 < ntiles) prefetch(tile + 1);
        const bool window = tile >= tiles_sel + tiles_sink;

        // tile summary (token range, all valid?) computed redundantly per wave
        const int tk = sm.tok[buf][lane];
        int tmin = tk < 0 ? 0x7fffffff : tk, tmax = tk;
        tmin = wave_min_i(tmin);
        tmax = wave_max_i(tmax);
        const bool all_valid = __all(tk >= 0);
        bool full;  // every (valid row, token) pair of the tile is attended
        if (!window) full = all_valid && ((long long)tmax + p.sw <= pmin_blk);
        else full = all_valid && (tmax <= pmin_blk) && ((long long)pmax_blk < (long long)tmin + p.sw);
        if (tmax < 0) continue;  // nothing valid in this tile (uniform)

        // ---- S^T = K^ Q^^T
        f32x16 sacc[2][2];
#pragma unroll
        for (int nb = 0; nb < 2; nb++)
#pragma unroll
            for (int mb = 0; mb < 2; mb++)
#pragma unroll
                for (int i = 0; i < 16; i++) sacc[nb][mb][i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            Frag a0, a1;
            a0.q = *reinterpret_cast<const uint4 *>(&sm.k[buf][col][ks * 16 + hh * 8]);
            a1.q = *reinterpret_cast<const uint4 *>(&sm.k[buf][32 + col][ks * 16 + hh * 8]);
            sacc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0.v, qf[0][ks].v, sacc[0][0], 0, 0, 0);
            sacc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0.v, qf[1][ks].v, sacc[0][1], 0, 0, 0);
            sacc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1.v, qf[0][ks].v, sacc[1][0], 0, 0, 0);
            sacc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1.v, qf[1][ks].v, sacc[1][1], 0, 0, 0);
            if (ks % 2 == 1) __builtin_amdgcn_sched_barrier(0);
        }

        // ---- mask + online softmax; element (nb, i) of a lane is token slot nb*32 + (i/4)*8 + hh*4 + i%4
        Frag pf[2][4];
        float alpha[2];
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
            float mx = -INFINITY;
            if (full) {
#pragma unroll
                for (int nb = 0; nb < 2; nb++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        sacc[nb][mb][i] *= LOG2E;
                        mx = fmaxf(mx, sacc[nb][mb][i]);
                    }
            } else {
                const int pq = pm[mb];
#pragma unroll
                for (int nb = 0; nb < 2; nb++)
#pragma unroll
                    for (int i4 = 0; i4 < 4; i4++) {
                        const int4 tt = *reinterpret_cast<const int4 *>(&sm.tok[buf][nb * 32 + i4 * 8 + hh * 4]);
                        const int ts[4] = {tt.x, tt.y, tt.z, tt.w};
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const int t = ts[e];
                            bool att;
                            if (!window) att = (t >= 0) && ((long long)t + p.sw <= pq);
                            else att = (t >= 0) && (t <= pq) && ((long long)pq < (long long)t + p.sw);
                            const float s = att ? sacc[nb][mb][i4 * 4 + e] * LOG2E : -INFINITY;
                            sacc[nb][mb][i4 * 4 + e] = s;
                            mx = fmaxf(mx, s);
                        }
                    }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run[mb], mx);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            alpha[mb] = __builtin_amdgcn_exp2f(m_run[mb] - m_use);  // m_run = -inf -> 0
            float lsum = 0.0f;
#pragma unroll
            for (int nb = 0; nb < 2; nb++)
#pragma unroll
                for (int u = 0; u < 2; u++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float p0 = __builtin_amdgcn_exp2f(sacc[nb][mb][u * 8 + 2 * e] - m_use);
                        const float p1 = __builtin_amdgcn_exp2f(sacc[nb][mb][u * 8 + 2 * e + 1] - m_use);
                        lsum += p0 + p1;
                        pf[mb][nb * 2 + u].u[e] = pack_bf16(p0, p1);
                    }
            l_run[mb] = l_run[mb] * alpha[mb] + lsum;
            m_run[mb] = m_new;
        }

        // ---- O^T += V^T P^T
        const bool rescale = __any((alpha[0] != 1.0f) || (alpha[1] != 1.0f));
        if (rescale) {
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int mb = 0; mb < 2; mb++)
#pragma unroll
                    for (int i = 0; i < 16; i++) oacc[db][mb][i] *= alpha[mb];
        }
#pragma unroll
        for (int db = 0; db < DB; db++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                Frag a;
                a.d[0] = *reinterpret_cast<const uint2 *>(&sm.vt[buf][db * 32 + col][j * 16 + hh * 4]);
                a.d[1] = *reinterpret_cast<const uint2 *>(&sm.vt[buf][db * 32 + col][j * 16 + 8 + hh * 4]);
                oacc[db][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, pf[0][j].v, oacc[db][0], 0, 0, 0);
                oacc[db][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, pf[1][j].v, oacc[db][1], 0, 0, 0);
                if (j % 2 == 1) __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // ---- epilogue: O^T[d, m] / l -> out[b, m, h, d]
    if (!head_ok) return;
    uint16_t *obase = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh;
#pragma unroll
    for (int mb = 0; mb < 2; mb++) {
        const int j = mb * 32 + col;
        const long long it = (long long)qb * p.bq + j;
        float l = l_run[mb] + __shfl_xor(l_run[mb], 32);
        if (!(j < p.bq && it < p.TDST)) continue;
        const float inv = 1.0f / (l == 0.0f ? 1.0f : l);
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++) {
                const int d = db * 32 + i4 * 8 + hh * 4;
                uint2 o;
                o.x = pack_bf16(oacc[db][mb][i4 * 4 + 0] * inv, oacc[db][mb][i4 * 4 + 1] * inv);
                o.y = pack_bf16(oacc[db][mb][i4 * 4 + 2] * inv, oacc[db][mb][i4 * 4 + 3] * inv);
                *reinterpret_cast<uint2 *>(obase + it * p.o_st + d) = o;
            }
    }
}

template <int HID>
static int launch_mfma(const BsaParams &p, hipStream_t st) {
    const int hpw = p.share_first_head ? 4 : 1;  // per-head index rows: one head per workgroup
    const int hgroups = (p.G + hpw - 1) / hpw;
    const long long total = (long long)p.B * p.kv.HKV * hgroups * p.NBQ;
    if (total >= 0x7fffffffLL) return HIPATTN_E_UNSUPPORTED;
    const size_t smem = sizeof(MfmaSmem<HID>);
    static bool attr_set = false;
    if (!attr_set) {
        HIPATTN_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&bsa_mfma_kernel<HID>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    hipLaunchKernelGGL((bsa_mfma_kernel<HID>), dim3((unsigned)total), dim3(256), smem, st, p, hgroups, hpw, total);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

int bsa_mfma_launch(const BsaParams &p, int dtype, int HID, hipStream_t st) {
    if (dtype != HIPATTN_BF16) return HIPATTN_E_UNSUPPORTED;
    if (p.bq > 64) return HIPATTN_E_UNSUPPORTED;
    if ((p.o_st % 4) != 0 || (p.o_sh % 4) != 0 || (p.o_sb % 4) != 0) return HIPATTN_E_UNSUPPORTED;
    switch (HID) {
        case 64: return launch_mfma<64>(p, st);
        case 128: return launch_mfma<128>(p, st);
    }
    return HIPATTN_E_UNSUPPORTED;
}

}  // namespace hipattn

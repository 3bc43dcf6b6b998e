// MFMA tile kernel for block-sparse attention (bf16, head dim 64 / 128 / 256, query block <= 64 rows).
//
// One workgroup = one (batch, kv head, query block) and up to four query heads of the GQA group;
// a wavefront owns one head and one 32-row half of the query block, so every gathered K/V tile in
// LDS is consumed by the whole group (eight waves, two per SIMD: while one wave of a SIMD runs its
// softmax on the vector unit the other keeps the matrix unit busy).
// Per 64-token tile:   S^T[token, query] = K^ . Q^^T      (v_mfma_f32_32x32x16_bf16, K^ from LDS,
//                                                           Q^ resident in registers)
//                      online softmax down the token axis  (a lane owns one query column)
//                      O^T[d, query]    += V^T . P^T        (V staged row-major in LDS and read through
//                                                           the transposing LDS load; P^T is taken
//                                                           straight from the S^T registers)
// Working on the transposed problem keeps the softmax statistics lane-local and lets P feed the
// second MFMA without a trip through LDS.  Global loads of tile i+1 are issued before the math of
// tile i; LDS is double-buffered so one barrier per tile suffices.  The running maximum is only
// raised when it grows by more than 2^8, so the accumulator is rescaled a handful of times per row.
#include "bsa.hpp"

namespace hipattn {

// a row of zeros in device memory: empty token slots of a tile are loaded from here, so that the loads of a tile
// need no branches
__device__ __align__(16) uint16_t g_zero_row[256];

constexpr int TN = 64;        // tokens per tile
constexpr int NTHREADS = 512;
constexpr int MAX_LDS_IDX = 1024;  // selected-block starts kept in LDS

// what wave 0 posts about the 64 token slots of a tile
template <int HID>
struct MfmaMeta {
    long long ko[TN], vo[TN];  // addresses of the K / V rows (an empty slot: the row of zeros)
    int tok[TN];               // token, -1 for an empty slot
    int rp[TN];                // row of the RoPE tables the key is rotated with
    int rp2[HID <= 128 ? TN : 1];  // dynamic rule: the second row a far key's tables are blended from, -1 = no blend
    int tmin, tmax, all_valid; // smallest / largest token of the tile (tmax < 0: empty tile), no empty slot
    int full;                  // every (valid row, token) pair of the tile is attended: the mask can be skipped
};

// Tiles are resolved in batches of META_BATCH, one batch ahead of their use: the ring holds two batches.
template <int HID>
constexpr int META_BATCH = HID <= 128 ? 16 : 4;

// Columns of V, and of the output, that one wave works on.  Head dim 256 is served in two passes of 128 columns by
// two waves, each forming all of the logits of its 32 rows: with 256 columns a wave would need 128 accumulator
// registers beside 64 of query fragments and 32 of logits, and spilled about 110; half again as many products
// cost less than that.  The passes of a head sit in one workgroup (which then serves two heads instead of four) and
// share its K and V tiles.
template <int HID>
constexpr int V_COLS = HID <= 128 ? HID : 128;

template <int HID>
struct MfmaSmem {
    uint16_t k[2][TN][HID + KPAD];
    uint16_t v[2][TN][HID + VPAD];
    MfmaMeta<HID> meta[2 * META_BATCH<HID>];
    int idx[MAX_LDS_IDX];
};
static_assert(sizeof(MfmaSmem<256>) <= 160 * 1024, "LDS of a compute unit");


// ---------------------------------------------------------------- the pipelined tile loop (head dim <= 128)
// The matrix unit and the vector unit of a SIMD run side by side: while a 32x32x16 product occupies the matrix unit
// for 32 cycles, the same wave can issue about six ordinary vector instructions for free.  A tile loop made of phases
// (products, then softmax, then products) never offers the two units work at the same time, so the loop below is
// software-pipelined by half tiles of 32 tokens: one step issues the products S^T(h+1) = K^ Q^^T and
// O^T += V^T P^T(h-1) together with the softmax of S^T(h), none of which depends on another, and the compiler is
// told to interleave them (sched_group_barrier).  K of tile i and V of tile i-1 are staged in the same iteration, so
// that every iteration reads one K buffer and one V buffer and one barrier per tile still suffices.

// One pipeline step: the products S^T(next half) = K^ Q^^T and O^T += V^T P^T(previous half) beside the online
// softmax of the half in between.  kh: this lane's K^ fragment address in the half tile whose logits are produced
// (k-step ks at + 16 * ks elements); vh: this lane's address for the transposing reads of the half tile whose P^T is
// consumed (k-step u at + 16 * u rows, 32-row block db of O^T at + 32 * db elements, second four tokens 8 rows
// further).  QK = false: the step after the last tile (no logits to produce).
//
// The softmax of a block of logits is cut in two.  Its head (mask, maximum, new reference point, the factor alpha
// that the accumulator is due) runs in the tail of the step that produced the block, once the products have
// delivered it; its body (exponentials, row sums, packing P) runs in the next step.  So a step opens with its first
// product and every vector instruction of the loop sits in the shadow of a product.  State handed from step to step
// with a block: its logits, minus its reference point (m_neg) and alpha.
//
// Element i of a lane's S^T block is token slot (i / 4) * 8 + hh * 4 + i % 4 of its half.  mask_next (wave-uniform):
// a token t of the produced block is attended iff (unsigned)(t - att_lo) < att_span (empty slots hold -1); only the
// masking itself sits in a branch, so that the accumulators have one home whichever way a step goes.
// The order of the instructions is laid down here and fenced (sched_barrier): operands of a product are read from
// LDS DEPTH products ahead and every product is followed by its share of the vector work.  chore(c), c = 0..15, is
// called behind product c * NM / 16: the staging work of the loop (reading posted row addresses, storing the staged
// rows of the next tile into LDS, issuing the loads of the tile after it) rides in the same shadow.
#define PIN3(a, b, c) asm volatile("" : "+v"(a), "+v"(b), "+v"(c))  // keeps what computes a, b, c in front of it
struct SoftmaxCarry {
    float m_neg;   // minus the reference point of the block (0 while nothing has been seen)
    float alpha;   // what raising the reference point to it costs the accumulator and the row sum
};
template <int HID, bool CAP, bool QK, typename Chore>
__device__ __forceinline__ void pipe_step(const uint16_t *kh, const uint16_t *vh, const Frag (&qf)[HID / 16],
                                          f32x16 (&oacc)[HID / 32], const Frag (&p_in)[2], f32x16 &s_out, f32x16 &s,
                                          Frag (&pf)[2], const SoftmaxCarry cur, SoftmaxCarry &next, float &m_run,
                                          float &l_run, bool mask_next, const int *tok_next, int hh, int att_lo,
                                          unsigned att_span, float cap, float cap_k2, Chore &&chore) {
    constexpr int KS = QK ? HID / 16 : 0, DB = HID / 32, VROW = HID + VPAD;
    constexpr int NM = KS + 2 * DB;   // products of this step
    constexpr int DEPTH = 4 < NM ? 4 : NM;  // operands in flight
    constexpr int EPS = 16 / NM;      // exponentials per product
    constexpr int MSPLIT = QK ? 10 * NM / 16 : NM;  // the produced block is complete before this product
    static_assert(NM * EPS == 16, "the step spreads 16 logits over its products");
    static_assert(!QK || MSPLIT >= KS + 1, "the head of the next softmax starts behind the last product that feeds it");
    auto fetch = [&](int m) {
        Frag a;
        if (m < KS) {
            a.q = *reinterpret_cast<const uint4 *>(kh + m * 16);
        } else {
            const int u = (m - KS) / DB, db = (m - KS) % DB;
            a.d[0] = lds_read_tr16(vh + u * 16 * VROW + db * 32);
            a.d[1] = lds_read_tr16(vh + (u * 16 + 8) * VROW + db * 32);
        }
        return a;
    };
    Frag ring[DEPTH];
#pragma unroll
    for (int m = 0; m < DEPTH; m++) ring[m] = fetch(m);
    const float m_neg = cur.m_neg;
    float lsum0 = 0.0f, lsum1 = 0.0f;
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.0f;
    float mx = -INFINITY, m_use = m_run, alpha_n = 1.0f;
    auto product = [&](int m) {
        if (m < KS) {
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[m % DEPTH].v, qf[m < KS ? m : 0].v, acc, 0, 0, 0);
        } else {
            const int u = (m - KS) / DB, db = (m - KS) % DB;
            oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[m % DEPTH].v, p_in[u].v, oacc[db], 0, 0, 0);
        }
        if (m + DEPTH < NM) ring[m % DEPTH] = fetch(m + DEPTH);
    };
    auto body = [&](int m) {  // exponentials of the block in hand
#pragma unroll
        for (int j = 0; j < EPS; j += 2) {
            if constexpr (EPS >= 2) {
                const int i = m * EPS + j;
                const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], LOG2E, m_neg));
                const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i + 1], LOG2E, m_neg));
                lsum0 += p0;
                lsum1 += p1;
                pf[i / 8].u[(i % 8) / 2] = cvt_pk_bf16(p0, p1);
                PIN3(lsum0, lsum1, pf[i / 8].u[(i % 8) / 2]);
            }
        }
        if constexpr (EPS == 1) {
            // one logit per product: the pair is packed behind every other one
            const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s[m], LOG2E, m_neg));
            s[m] = pv;
            if (m & 1) {
                lsum0 += s[m - 1];
                lsum1 += pv;
                pf[m / 8].u[(m % 8) / 2] = cvt_pk_bf16(s[m - 1], pv);
                PIN3(lsum0, lsum1, pf[m / 8].u[(m % 8) / 2]);
            }
        }
    };
    auto head = [&](int c) {  // head of the softmax of the produced block, in five pieces (c = 10 .. 14)
        if (c == 10) {
            mx = fmaxf(acc[0], acc[1]);
#pragma unroll
            for (int i = 2; i < 8; i += 2) mx = fmaxf(fmaxf(mx, acc[i]), acc[i + 1]);   // v_max3_f32
        }
        if (c == 11) {
#pragma unroll
            for (int i = 8; i < 16; i += 2) mx = fmaxf(fmaxf(mx, acc[i]), acc[i + 1]);
        }
        if (c == 12) mx = fmaxf(mx, swap_halves(mx)) * LOG2E;
        if (c == 13) {
            // raise the reference point only when the maximum grew noticeably
            const bool raise = mx > m_run + RESCALE_STEP || m_run == -INFINITY;
            m_use = raise ? fmaxf(m_run, mx) : m_run;
            alpha_n = __builtin_amdgcn_exp2f(m_run - m_use);  // an unchanged point gives 1, a first one 0
            PIN3(mx, m_use, alpha_n);
        }
        if (c == 14) {
            next.alpha = (m_use == -INFINITY) ? 1.0f : alpha_n;   // nothing seen yet: -inf - -inf
            next.m_neg = (m_use == -INFINITY) ? 0.0f : -m_use;
            m_run = m_use;
            PIN3(next.alpha, next.m_neg, m_run);
        }
    };
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < MSPLIT; m++) {
        product(m);
        body(m);
#pragma unroll
        for (int c = m * 16 / NM; c < (m + 1) * 16 / NM; c++) chore(c);
        __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (QK) {
        if constexpr (CAP) {
#pragma unroll
            for (int i = 0; i < 16; i++) acc[i] = softcap_logit(acc[i], cap, cap_k2);
        }
        if (mask_next) {
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++) {
                const int4 tt = *reinterpret_cast<const int4 *>(tok_next + i4 * 8 + hh * 4);
                const int ts[4] = {tt.x, tt.y, tt.z, tt.w};
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[i4 * 4 + e] = ((unsigned)(ts[e] - att_lo) < att_span) ? acc[i4 * 4 + e] : -INFINITY;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = MSPLIT; m < NM; m++) {
            product(m);
            body(m);
#pragma unroll
            for (int c = m * 16 / NM; c < (m + 1) * 16 / NM; c++) {
                head(c);
                chore(c);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    l_run = l_run * cur.alpha + (lsum0 + lsum1);
    s_out = acc;
}

// ROPE = true (extended parameter block, unscaled keys): query rows and staged key rows are rotated on load.
// A query lane holds both halves of its row (k-steps ks and ks + KS/2); the two halves of a staged key row are
// fetched by lanes tid and tid ^ (HID/16) of one wave.
// CAP = true (extended parameter block): logits are soft-capped before the softmax.
// KV8 = true (extended parameter block): K / V rows are fp8 (e5m2) bytes, widened on load.
// DYN = true (rope variant, head dim <= 128): the "dynamic_extend" rule, far keys rotated with a blend of two table rows.
template <int HID, bool KSCALED, bool EXT, bool ROPE = false, bool CAP = false, bool KV8 = false, bool DYN = false>
__global__ __launch_bounds__(NTHREADS) void bsa_mfma_kernel(BsaParamsFor<EXT> p, int hgroups, int hpw, long long total_wg) {
    static_assert(!ROPE || (EXT && !KSCALED), "rope variant: extended parameter block, keys scaled in the kernel");
    static_assert(!CAP || EXT, "softcap variant: extended parameter block");
    static_assert(!KV8 || (EXT && !KSCALED), "fp8 storage: extended parameter block, keys scaled in the kernel");
    static_assert(!DYN || (ROPE && HID <= 128), "dynamic rule: a rope variant of the pipelined loop");
    const KVExt *kx = nullptr;
    if constexpr (EXT) kx = &p.kx;
    constexpr int KS = HID / 16;   // k-steps of the first product
    constexpr int DV = V_COLS<HID>, NPASS = HID / DV;
    constexpr int DB = DV / 32;    // 32-row blocks of O^T
    constexpr int CPT = TN * (HID / 8) / NTHREADS;  // 16-byte chunks per thread per tile
    extern __shared__ __align__(16) unsigned char smem_raw[];
    MfmaSmem<HID> &sm = *reinterpret_cast<MfmaSmem<HID> *>(smem_raw);

    // wave-uniform quantities are marked as such (readfirstlane), so that the tile loop and its branches run on the
    // scalar unit instead of under execution masks
    const int tid = threadIdx.x, lane = tid & 63, wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, hh = lane >> 5;
    const int half = wid & 1;
    const int whead = (wid >> 1) / NPASS;            // head slot of the workgroup
    const int dv0 = ((wid >> 1) % NPASS) * DV;       // first output column of this wave

    long long L = xcd_remap((long long)blockIdx.x, total_wg);
    const int qb = (int)(L % p.NBQ);
    L /= p.NBQ;
    const int hgrp = (int)(L % hgroups);
    L /= hgroups;
    const int kvh = (int)(L % p.kv.HKV);
    const int b = (int)(L / p.kv.HKV);
    const int hin = hgrp * hpw + whead;
    const bool head_ok = (whead < hpw) && (hin < p.G) && (half * 32 < p.bq);
    const int h = kvh * p.G + ((whead < hpw && hin < p.G) ? hin : 0);
    // index row: the group's first head when rows are shared, else the single head this workgroup serves
    const int hrow = p.share_first_head ? kvh * p.G : kvh * p.G + hgrp * hpw;
    const int64_t irow = ((int64_t)b * p.HEAD + hrow) * p.idx_rows + qb;

    // ---- query block geometry
    int pmin_blk, pmax_blk;
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
        pmax_blk = __builtin_amdgcn_readfirstlane((int)cur);
        pmin_blk = __builtin_amdgcn_readfirstlane((int)mn);
    }
    const int myj = half * 32 + col;                       // this lane's query row inside the block
    const long long myit = (long long)qb * p.bq + myj;
    const bool row_ok = (myj < p.bq) && (myit < p.TDST);
    const int pq = row_ok ? (int)p.pos[(int64_t)b * p.pos_sb + myit * p.pos_st] : -0x40000000;

    const int curr = pmax_blk + 1;
    int rs = p.kse[irow * 2 + 0], re = p.kse[irow * 2 + 1];
    const long long rope_shift = (long long)pmin_blk - p.sw - p.sink - (long long)(re - rs) * p.bk + 1;
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

    // selected block starts -> LDS (removes a dependent global load from every tile's prefetch)
    const bool idx_in_lds = nsel <= MAX_LDS_IDX;
    if (idx_in_lds) {
        for (int i = tid; i < nsel; i += NTHREADS) {
            const long long st = p.indices[irow * p.BK + rs + i];
            sm.idx[i] = (st >= 0 && st < 0x7fffffffLL) ? (int)st : -0x40000000;
        }
    }

    // ---- Q^ fragments (B operand of the first product), resident for the whole kernel
    Frag qf[KS];
    {
        const uint16_t *qbase = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
        const bool ok = head_ok && row_ok;
        uint4 qraw[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            qraw[ks] = make_uint4(0, 0, 0, 0);
            if (ok) qraw[ks] = *reinterpret_cast<const uint4 *>(qbase + myit * p.q_st + ks * 16 + hh * 8);
        }
        if constexpr (ROPE) {
            if (ok) {  // the query keeps its own position (attention_extend_bsa.py:796-852)
                const uint16_t *ct = reinterpret_cast<const uint16_t *>(p.rope.cos) + p.rope.row(pq);
                const uint16_t *st = reinterpret_cast<const uint16_t *>(p.rope.sin) + p.rope.row(pq);
#pragma unroll
                for (int ks = 0; ks < KS / 2; ks++) {
                    const uint4 c = *reinterpret_cast<const uint4 *>(ct + ks * 16 + hh * 8);
                    const uint4 sn = *reinterpret_cast<const uint4 *>(st + ks * 16 + hh * 8);
                    const uint4 lo = qraw[ks], hi = qraw[ks + KS / 2];
                    qraw[ks] = rope_piece(lo, hi, c, sn, true);
                    qraw[ks + KS / 2] = rope_piece(hi, lo, c, sn, false);
                }
            }
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const uint4 raw = qraw[ks];
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int e = 0; e < 4; e++)
                qf[ks].u[e] = cvt_pk_bf16(__uint_as_float(w[e] << 16) * p.c_q, __uint_as_float(w[e] & 0xffff0000u) * p.c_q);
        }
    }
    __syncthreads();  // sm.idx visible

    const int64_t seqlen = p.kv.paged ? p.kv.seq_len(b) : 0;

    // ---- staging.  The token list is resolved a batch of tiles at a time, one tile per wave (lane = token slot of
    // the tile): the token, its K / V row offsets (page lookup, statistics, offload cache) and, with RoPE, its rotated
    // position are posted in LDS a batch ahead of the loads, so that no wave carries this work on every tile.
    // All threads then fetch rows by posted offset: chunk c = tid + NTHREADS*j is 16-byte piece c % (HID/8) of token
    // slot c / (HID/8).
    constexpr int HB = META_BATCH<HID>;
    const int bk_shift = (p.bk & (p.bk - 1)) == 0 ? __builtin_ctz(p.bk) : -1;  // block sizes are usually powers of two
    const int tlimit = (int)(p.kv.max_tsrc < (long long)curr ? p.kv.max_tsrc : (long long)curr);
    auto resolve = [&](int tile) {  // one wave per tile
        int kind, base;  // kind 0 selected, 1 sink, 2 window
        if (tile < tiles_sel) { kind = 0; base = tile * TN; }
        else if (tile < tiles_sel + tiles_sink) { kind = 1; base = (tile - tiles_sel) * TN; }
        else { kind = 2; base = (tile - tiles_sel - tiles_sink) * TN; }
        const int o = base + lane;
        int t = -1;
        long long rpos = 0;  // rotated position of the key (ROPE only)
        if (kind == 0) {
            if (o < n_sel_tok) {
                const int bi = bk_shift >= 0 ? (o >> bk_shift) : o / p.bk;
                const int e = o - bi * p.bk;
                int st;
                if (idx_in_lds) {
                    st = sm.idx[bi];
                } else {
                    const long long s64 = p.indices[irow * p.BK + rs + bi];
                    st = (s64 >= 0 && s64 < 0x7fffffffLL) ? (int)s64 : -0x40000000;
                }
                t = st + e;  // st is below 2^31 - 1 or the large negative marker: no overflow
                if (!(t >= p.sink && t < tlimit)) t = -1;
                if constexpr (ROPE)
                    rpos = bsa_rope_far_pos(p.rope, (long long)(rs + bi + p.sink / p.bk) * p.bk + e, rope_shift, pmin_blk,
                                            p.sw);
            }
        } else if (kind == 1) {
            if (o < sink_end) t = o;
            if constexpr (ROPE) rpos = bsa_rope_far_pos(p.rope, o, rope_shift, pmin_blk, p.sw);
        } else {
            if (o < n_win) t = ws + o;
            rpos = t;
        }
        int64_t ko = NO_ROW, vo = NO_ROW;
        if (t >= 0) kv_rows<true, EXT>(p.kv, kx, b, t, kvh, seqlen, ko, vo, true);
        MfmaMeta<HID> &mt = sm.meta[tile & (2 * HB - 1)];
        constexpr int ESZ = KV8 ? 1 : 2;
        mt.ko[lane] = ko != NO_ROW ? (long long)(reinterpret_cast<const char *>(p.kv.k) + ko * ESZ) : (long long)g_zero_row;
        mt.vo[lane] = vo != NO_ROW ? (long long)(reinterpret_cast<const char *>(p.kv.v) + vo * ESZ) : (long long)g_zero_row;
        mt.tok[lane] = t;
        if constexpr (ROPE) mt.rp[lane] = (int)p.rope.clamp(rpos);
        if constexpr (DYN) {
            // sink and selected keys: second row = the key's own position squeezed into the model's context, with
            // pmax = pmin + the block's valid rows (attention_extend_bsa.py:271-292)
            const long long nvalid = (long long)p.TDST - (long long)qb * p.bq < p.bq ? (long long)p.TDST - (long long)qb * p.bq : p.bq;
            mt.rp2[lane] = (kind != 2 && t >= 0)
                               ? (int)p.rope.clamp(dynamic_extend_pos(t, pmin_blk, pmin_blk + nvalid, p.rope.model_ctx))
                               : -1;
        }
        // tile summary for the mask shortcut, once for the whole workgroup
        const int tmin = wave_min_i(t < 0 ? 0x7fffffff : t);
        const int tmax = wave_max_i(t);
        const int allv = __all(t >= 0) ? 1 : 0;
        if (lane == 0) {
            mt.tmin = tmin;
            mt.tmax = tmax;
            mt.all_valid = allv;
            // far keys need t + sw <= p for every row, window keys t <= p < t + sw
            mt.full = allv && (p.non_causal || (kind != 2 ? ((long long)tmax + p.sw <= pmin_blk)
                                                          : (tmax <= pmin_blk && (long long)pmax_blk < (long long)tmin + p.sw)));
        }
    };
    // tiles first .. first + HB - 1, spread over the waves; the two tiles past the end resolve to rows of zeros, so
    // that the pipelined loop can stage ahead without asking where the list ends
    auto resolve_batch = [&](int first) {
        for (int t = first + wid; t < first + HB && t <= ntiles + 1; t += NTHREADS / 64) resolve(t);
    };
    uint4 kreg[CPT], vreg[CPT];
    uint4 creg[ROPE ? CPT : 1], sreg[ROPE ? CPT : 1];  // cos / sin pieces of the staged key rows
    // head dim 256: the table pieces are requested late in a tile (prefetch_rope), when the key fragments of its
    // logits are dead, instead of together with the rows; 32 registers less while the logits are formed
    constexpr bool LATE_ROPE = ROPE && HID > 128;
    int rp_late[LATE_ROPE ? CPT : 1];
    // dynamic rule: the pieces of the second table row and, per staged piece, whether it takes the blend
    uint4 creg2[DYN ? CPT : 1], sreg2[DYN ? CPT : 1];
    unsigned blend_bits = 0;
    auto prefetch_k = [&](int tile) {
        const MfmaMeta<HID> &mt = sm.meta[tile & (2 * HB - 1)];
        long long ka[CPT];
        int rp[CPT], rp2[DYN ? CPT : 1];
#pragma unroll
        for (int j = 0; j < CPT; j++) {
            const int slot = (tid + NTHREADS * j) / (HID / 8);
            ka[j] = mt.ko[slot];
            if constexpr (ROPE) rp[j] = mt.rp[slot];
            if constexpr (DYN) rp2[j] = mt.rp2[slot];
        }
        if constexpr (DYN) blend_bits = 0;
#pragma unroll
        for (int j = 0; j < CPT; j++) {
            const int piece = (tid + NTHREADS * j) % (HID / 8);
            if constexpr (ROPE && !LATE_ROPE) {
                const int64_t tr = (int64_t)rp[j] * p.rope.stride_t + (piece % (HID / 16)) * 8;
                creg[j] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.cos) + tr);
                sreg[j] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.sin) + tr);
            }
            if constexpr (LATE_ROPE) rp_late[j] = rp[j];
            if constexpr (DYN) {
                const int64_t tr2 = (int64_t)(rp2[j] < 0 ? 0 : rp2[j]) * p.rope.stride_t + (piece % (HID / 16)) * 8;
                creg2[j] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.cos) + tr2);
                sreg2[j] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.sin) + tr2);
                blend_bits |= (rp2[j] >= 0 ? 1u : 0u) << j;
            }
            kreg[j] = load_kv_piece_global<KV8>(ka[j], piece * 8);
        }
    };
    auto prefetch_rope = [&]() {
        if constexpr (LATE_ROPE) {
#pragma unroll
            for (int j = 0; j < CPT; j++) {
                const int piece = (tid + NTHREADS * j) % (HID / 8);
                const int64_t tr = (int64_t)rp_late[j] * p.rope.stride_t + (piece % (HID / 16)) * 8;
                creg[j] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.cos) + tr);
                sreg[j] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.sin) + tr);
            }
        }
    };
    auto prefetch_v = [&](int tile) {
        const MfmaMeta<HID> &mt = sm.meta[tile & (2 * HB - 1)];
        long long va[CPT];
#pragma unroll
        for (int j = 0; j < CPT; j++) va[j] = mt.vo[(tid + NTHREADS * j) / (HID / 8)];
#pragma unroll
        for (int j = 0; j < CPT; j++) vreg[j] = load_kv_piece_global<KV8>(va[j], ((tid + NTHREADS * j) % (HID / 8)) * 8);
    };
    auto commit_k = [&](int buf) {
#pragma unroll
        for (int j = 0; j < CPT; j++) {
            const int c = tid + NTHREADS * j;
            const int slot = c / (HID / 8), piece = c % (HID / 8);
            uint4 kq = kreg[j];
            if constexpr (ROPE) {
                const uint4 oth = make_uint4(lane_xor<HID / 16>(kq.x), lane_xor<HID / 16>(kq.y), lane_xor<HID / 16>(kq.z),
                                             lane_xor<HID / 16>(kq.w));
                uint4 cc = creg[j], sn = sreg[j];
                if constexpr (DYN) {
                    const bool bl = (blend_bits >> j) & 1u;
                    const float wa = bl ? 0.75f : 1.0f, wb = bl ? 0.25f : 0.0f;
                    cc = rope_blend_piece(cc, creg2[j], wa, wb);
                    sn = rope_blend_piece(sn, sreg2[j], wa, wb);
                }
                kq = rope_piece(kq, oth, cc, sn, piece < HID / 16);
            }
            if (!KSCALED) {
                kq.x = cvt_pk_bf16(__uint_as_float(kq.x << 16) * p.c_k, __uint_as_float(kq.x & 0xffff0000u) * p.c_k);
                kq.y = cvt_pk_bf16(__uint_as_float(kq.y << 16) * p.c_k, __uint_as_float(kq.y & 0xffff0000u) * p.c_k);
                kq.z = cvt_pk_bf16(__uint_as_float(kq.z << 16) * p.c_k, __uint_as_float(kq.z & 0xffff0000u) * p.c_k);
                kq.w = cvt_pk_bf16(__uint_as_float(kq.w << 16) * p.c_k, __uint_as_float(kq.w & 0xffff0000u) * p.c_k);
            }
            *reinterpret_cast<uint4 *>(&sm.k[buf][slot][piece * 8]) = kq;
        }
    };
    auto commit_v = [&](int buf) {
#pragma unroll
        for (int j = 0; j < CPT; j++) {
            const int c = tid + NTHREADS * j;
            *reinterpret_cast<uint4 *>(&sm.v[buf][c / (HID / 8)][(c % (HID / 8)) * 8]) = vreg[j];
        }
    };

    // ---- running state (a lane owns one query column)
    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] = 0.0f;
    float m_run = -INFINITY;   // in log2 units, already multiplied by log2(e)
    float l_run = 0.0f;

    // what the mask shortcut needs of a tile: is every (valid row, token) pair attended, and is it a window tile
    auto tile_full = [&](int tile, bool &window) {
        const MfmaMeta<HID> &mt = sm.meta[tile & (2 * HB - 1)];
        const int tmin = __builtin_amdgcn_readfirstlane(mt.tmin), tmax = __builtin_amdgcn_readfirstlane(mt.tmax);
        const bool all_valid = __builtin_amdgcn_readfirstlane(mt.all_valid) != 0;
        window = tile >= tiles_sel + tiles_sink;
        if (p.non_causal) return all_valid;
        if (!window) return all_valid && ((long long)tmax + p.sw <= pmin_blk);
        return all_valid && (tmax <= pmin_blk) && ((long long)pmax_blk < (long long)tmin + p.sw);
    };

    if constexpr (HID <= 128) {
        // ---- pipelined loop (see pipe_step)
        constexpr int KROW = HID + KPAD, VROW = HID + VPAD;
        // the V buffer the first iteration multiplies by P = 0 must hold finite values
        for (int c = tid; c < TN * VROW / 8; c += NTHREADS) reinterpret_cast<uint4 *>(&sm.v[1][0][0])[c] = make_uint4(0, 0, 0, 0);
        const int k_off = col * KROW + hh * 8;
        const int v_off = (hh * 4 + ((lane & 15) >> 2)) * VROW + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
        // attended token ranges of this lane's query row: far keys 0 <= t <= pq - sw, window keys
        // max(0, pq - sw + 1) <= t <= pq; a row that does not exist attends nothing
        const long long far_hi = (long long)pq - p.sw;
        unsigned far_span = far_hi >= 0 ? (unsigned)far_hi + 1u : 0u;
        int win_lo = far_hi + 1 > 0 ? (int)(far_hi + 1) : 0;
        unsigned win_span = pq >= win_lo ? (unsigned)(pq - win_lo) + 1u : 0u;
        if (p.non_causal) {  // every valid token of an existing row
            win_lo = 0;
            far_span = win_span = row_ok ? 0x80000000u : 0u;
        }
        float cap = 0.0f, cap_k2 = 0.0f;
        if constexpr (CAP) {
            cap = p.softcap;
            cap_k2 = 2.0f * LOG2E / p.softcap;
        }
        f32x16 s_a, s_b;   // logits of the first / second half of a tile
        Frag p_a[2], p_b[2];
#pragma unroll
        for (int i = 0; i < 16; i++) { s_a[i] = -INFINITY; s_b[i] = -INFINITY; }
#pragma unroll
        for (int u = 0; u < 2; u++) { p_a[u].q = make_uint4(0, 0, 0, 0); p_b[u].q = make_uint4(0, 0, 0, 0); }
        SoftmaxCarry c_a = {0.0f, 1.0f}, c_b = {0.0f, 1.0f};
        auto rescale = [&](float alpha) {
            if (__any(alpha != 1.0f)) {
#pragma unroll
                for (int db = 0; db < DB; db++)
#pragma unroll
                    for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;
            }
        };
        // posted row addresses of the rows this thread stages, read a step ahead of their loads, and the summary of
        // the next tile
        long long ka[CPT], va[CPT];
        int rpk[ROPE ? CPT : 1], rp2k[DYN ? CPT : 1];
        int nx_full = 0;
        auto read_posted = [&](int i) {  // iteration i loads K of tile i + 2 and V of tile i + 1
            const MfmaMeta<HID> &mk = sm.meta[(i + 2) & (2 * HB - 1)], &mv = sm.meta[(i + 1) & (2 * HB - 1)];
#pragma unroll
            for (int j = 0; j < CPT; j++) {
                const int slot = (tid + NTHREADS * j) / (HID / 8);
                ka[j] = mk.ko[slot];
                va[j] = mv.vo[slot];
                if constexpr (ROPE) rpk[j] = mk.rp[slot];
                if constexpr (DYN) rp2k[j] = mk.rp2[slot];
            }
            nx_full = mv.full;
        };
        auto issue_loads = [&]() {
            if constexpr (DYN) blend_bits = 0;
#pragma unroll
            for (int j = 0; j < CPT; j++) {
                const int piece = (tid + NTHREADS * j) % (HID / 8);
                if constexpr (ROPE) {
                    const int64_t tr = (int64_t)rpk[j] * p.rope.stride_t + (piece % (HID / 16)) * 8;
                    creg[j] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.cos) + tr);
                    sreg[j] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.sin) + tr);
                }
                if constexpr (DYN) {
                    const int64_t tr2 = (int64_t)(rp2k[j] < 0 ? 0 : rp2k[j]) * p.rope.stride_t + (piece % (HID / 16)) * 8;
                    creg2[j] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.cos) + tr2);
                    sreg2[j] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.sin) + tr2);
                    blend_bits |= (rp2k[j] >= 0 ? 1u : 0u) << j;
                }
                kreg[j] = load_kv_piece_global<KV8>(ka[j], piece * 8);
                vreg[j] = load_kv_piece_global<KV8>(va[j], piece * 8);
            }
        };
        if (ntiles > 0) {
            // K of tile 0 into LDS, K of tile 1 and V of tile 0 on their way
            resolve_batch(0);
            __syncthreads();
            prefetch_k(0);
            commit_k(0);
            prefetch_k(1);
            prefetch_v(0);
            bool window_cur;
            bool full_cur = tile_full(0, window_cur);
            if (!head_ok) {
                // a wave without rows of its own stages its share of every tile and keeps the barriers company (a
                // loop of its own: merged with the other as a branch, the staging registers of the two paths meet
                // in copies at the end of every iteration, behind a wait for the loads in flight)
                for (int i = 0; i < ntiles; i++) {
                    __syncthreads();
                    if (((i + 3) & (HB - 1)) == 0 && i + 3 <= ntiles + 1) resolve_batch(i + 3);
                    read_posted(i);
                    commit_k((i + 1) & 1);
                    commit_v(i & 1);
                    issue_loads();
                }
                __syncthreads();
                return;
            }
            for (int i = 0; i < ntiles; i++) {
                __syncthreads();  // K of tile i and V of tile i - 1 are in LDS (stored during the last iteration)
                // the batch of tiles whose addresses are read three iterations from now
                if (((i + 3) & (HB - 1)) == 0 && i + 3 <= ntiles + 1) resolve_batch(i + 3);
                const uint16_t *kt = &sm.k[i & 1][0][0] + k_off;
                const uint16_t *vt = &sm.v[(i - 1) & 1][0][0] + v_off;
                const int *tok_cur = sm.meta[i & (2 * HB - 1)].tok;
                // step A: logits of the first half of tile i, O += V P of the first half of tile i - 1, exponentials
                // of the second half of tile i - 1
                pipe_step<HID, CAP, true>(kt, vt, qf, oacc, p_a, s_a, s_b, p_b, c_b, c_a, m_run, l_run, !full_cur, tok_cur, hh,
                                          window_cur ? win_lo : 0, window_cur ? win_span : far_span, cap, cap_k2,
                                          [&](int c) { if (c == 1) read_posted(i); });
                rescale(c_b.alpha);
                // step B: logits of the second half of tile i, O += V P of the second half of tile i - 1,
                // exponentials of the first half of tile i.  Beside it K of tile i + 1 and V of tile i go to LDS (their
                // buffers were last read before this iteration's barrier) and the loads of the tile after are issued.
                pipe_step<HID, CAP, true>(kt + 32 * KROW, vt + 32 * VROW, qf, oacc, p_b, s_b, s_a, p_a, c_a, c_b, m_run, l_run, !full_cur,
                                          tok_cur + 32, hh, window_cur ? win_lo : 0, window_cur ? win_span : far_span, cap, cap_k2,
                                          [&](int c) {
                                              if (c == 1) commit_k((i + 1) & 1);
                                              if (c == 3) commit_v(i & 1);
                                              if (c == 6) issue_loads();
                                          });
                rescale(c_a.alpha);
                full_cur = __builtin_amdgcn_readfirstlane(nx_full) != 0;
                window_cur = i + 1 >= tiles_sel + tiles_sink;
            }
            // drain: the softmax of the last tile's second half and its two products with V
            __syncthreads();
            {
                const uint16_t *vt = &sm.v[(ntiles - 1) & 1][0][0] + v_off;
                f32x16 s_none;
                pipe_step<HID, CAP, false>(nullptr, vt, qf, oacc, p_a, s_none, s_b, p_b, c_b, c_a, m_run, l_run, false, nullptr, hh, 0, 0u,
                                           cap, cap_k2, [](int) {});
                rescale(c_b.alpha);
#pragma unroll
                for (int u = 0; u < 2; u++)
#pragma unroll
                    for (int db = 0; db < DB; db++) {
                        Frag a;
                        a.d[0] = lds_read_tr16(vt + (32 + u * 16) * VROW + db * 32);
                        a.d[1] = lds_read_tr16(vt + (32 + u * 16 + 8) * VROW + db * 32);
                        oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, p_b[u].v, oacc[db], 0, 0, 0);
                    }
            }
        }
    } else {
    if (ntiles > 0) {
        resolve_batch(0);
        __syncthreads();
        prefetch_k(0);
        prefetch_rope();
        prefetch_v(0);
    }
    for (int tile = 0; tile < ntiles; tile++) {
        const int buf = tile & 1;
        commit_k(buf);
        commit_v(buf);
        __syncthreads();
        if (tile + 1 < ntiles) {
            prefetch_k(tile + 1);
            prefetch_v(tile + 1);
        }
        // the next batch of tiles: its half of the ring was last read a batch ago, and the barrier of the next
        // round stands between these writes and their first use
        if (((tile + 2) & (HB - 1)) == 0 && tile + 2 < ntiles) resolve_batch(tile + 2);
        const MfmaMeta<HID> &mt = sm.meta[tile & (2 * HB - 1)];
        bool window;
        const bool full = tile_full(tile, window);
        const int tmax = __builtin_amdgcn_readfirstlane(mt.tmax);
        if (tmax < 0 || !head_ok) {  // nothing valid in this tile, or an idle wave (both wave-uniform)
            prefetch_rope();
            continue;
        }
        // a half tile of 32 tokens at a time (logits, softmax, products with V): one block of logits and one of P
        // live beside the accumulators and the query fragments
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
            // ---- S^T = K^ Q^^T
            f32x16 sacc;
#pragma unroll
            for (int i = 0; i < 16; i++) sacc[i] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                Frag a0;
                a0.q = *reinterpret_cast<const uint4 *>(&sm.k[buf][nb * 32 + col][ks * 16 + hh * 8]);
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0.v, qf[ks].v, sacc, 0, 0, 0);
                // keeps the fragment reads of at most four k-steps in flight (left alone the scheduler hoists all
                // sixteen and spills the accumulators)
                if ((ks & 3) == 3) __builtin_amdgcn_sched_barrier(0);
            }
            if (nb == 1) prefetch_rope();
            if constexpr (CAP) {
                const float k2 = 2.0f * LOG2E / p.softcap;
#pragma unroll
                for (int i = 0; i < 16; i++) sacc[i] = softcap_logit(sacc[i], p.softcap, k2);
            }

            // ---- mask + online softmax; element i of a lane is token slot nb*32 + (i/4)*8 + hh*4 + i%4
            float mx = -INFINITY;
            if (full) {
#pragma unroll
                for (int i = 0; i < 16; i++) mx = fmaxf(mx, sacc[i]);
            } else {
#pragma unroll
                for (int i4 = 0; i4 < 4; i4++) {
                    const int4 tt = *reinterpret_cast<const int4 *>(&mt.tok[nb * 32 + i4 * 8 + hh * 4]);
                    const int ts[4] = {tt.x, tt.y, tt.z, tt.w};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int t = ts[e];
                        // branch-free: far keys need t + sw <= pq, window keys t <= pq < t + sw
                        const long long tsw = (long long)t + p.sw;
                        const bool att = (t >= 0) & (p.non_causal ? row_ok : window ? ((t <= pq) & ((long long)pq < tsw)) : (tsw <= (long long)pq));
                        const float s = att ? sacc[i4 * 4 + e] : -INFINITY;
                        sacc[i4 * 4 + e] = s;
                        mx = fmaxf(mx, s);
                    }
                }
            }
            mx = fmaxf(mx, swap_halves(mx)) * LOG2E;
            // raise the reference point only when the maximum grew noticeably
            float m_use = m_run;
            float alpha = 1.0f;
            if (mx > m_run + RESCALE_STEP || m_run == -INFINITY) {
                m_use = fmaxf(m_run, mx);
                alpha = (m_use == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_use);  // m_run = -inf -> 0
            }
            const float m_sub = (m_use == -INFINITY) ? 0.0f : m_use;
            Frag pf[2];
            float lsum = 0.0f;
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[u * 8 + 2 * e], LOG2E, -m_sub));
                    const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[u * 8 + 2 * e + 1], LOG2E, -m_sub));
                    lsum += p0 + p1;
                    pf[u].u[e] = cvt_pk_bf16(p0, p1);
                }
            l_run = l_run * alpha + lsum;
            m_run = m_use;
            // ---- O^T += V^T P^T
            if (__any(alpha != 1.0f)) {
#pragma unroll
                for (int db = 0; db < DB; db++)
#pragma unroll
                    for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;
            }
#pragma unroll
            for (int db = 0; db < DB; db++) {
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    // V^T fragments straight from the row-major tile: a transposing LDS read hands lane l of a
                    // 16-lane group column l % 4 of the four rows addressed by lanes l / 4, l / 4 + 4, + 8, + 12 of the
                    // group, so with source lane s pointing at (token T0 + s / 4, d = D0 + 4 * (s % 4)) lane l
                    // receives tokens T0 .. T0 + 3 at d = D0 + l.
                    Frag a;
                    const int trow = nb * 32 + u * 16 + hh * 4 + ((lane & 15) >> 2);
                    const int tcol = dv0 + db * 32 + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
                    a.d[0] = lds_read_tr16(&sm.v[buf][trow][tcol]);
                    a.d[1] = lds_read_tr16(&sm.v[buf][trow + 8][tcol]);
                    oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, pf[u].v, oacc[db], 0, 0, 0);
                }
                if (db & 1) __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    }

    // ---- epilogue: O^T[d, m] / l -> out[b, m, h, d]
    if (!head_ok) return;
    const float l = l_run + swap_halves(l_run);
    if (!row_ok) return;
    const float inv = 1.0f / (l == 0.0f ? 1.0f : l);
    uint16_t *obase = reinterpret_cast<uint16_t *>(p.out) + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + myit * p.o_st;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
            const int d = dv0 + db * 32 + i4 * 8 + hh * 4;
            uint2 o;
            o.x = cvt_pk_bf16(oacc[db][i4 * 4 + 0] * inv, oacc[db][i4 * 4 + 1] * inv);
            o.y = cvt_pk_bf16(oacc[db][i4 * 4 + 2] * inv, oacc[db][i4 * 4 + 3] * inv);
            *reinterpret_cast<uint2 *>(obase + d) = o;
        }
}

// Access statistics without touching the attention kernel: walks exactly the tokens the tile kernel stages
// for a (batch, kv head, head group, query block) and records them, loading no keys.
__global__ __launch_bounds__(256) void bsa_mark_kernel(BsaParams p, int hgroups, int hpw) {
    long long L = blockIdx.x;
    const int qb = (int)(L % p.NBQ);
    L /= p.NBQ;
    const int hgrp = (int)(L % hgroups);
    L /= hgroups;
    const int kvh = (int)(L % p.kv.HKV);
    const int b = (int)(L / p.kv.HKV);
    const int hrow = p.share_first_head ? kvh * p.G : kvh * p.G + hgrp * hpw;
    const int64_t irow = ((int64_t)b * p.HEAD + hrow) * p.idx_rows + qb;
    __shared__ long long s_cur;
    if (threadIdx.x == 0) s_cur = -1;
    __syncthreads();
    for (int j = threadIdx.x; j < p.bq; j += blockDim.x) {
        const long long it = (long long)qb * p.bq + j;
        if (it < p.TDST) atomicMax(&s_cur, (long long)p.pos[(int64_t)b * p.pos_sb + it * p.pos_st]);
    }
    __syncthreads();
    const int curr = (int)s_cur + 1;
    int rs = p.kse[irow * 2 + 0], re = p.kse[irow * 2 + 1];
    if (p.BK <= 0) { rs = 0; re = 0; }
    const int jend = rs + p.BK < re ? rs + p.BK : re;
    const int n_sel_tok = (jend > rs ? jend - rs : 0) * p.bk;
    const int sink_end = curr < p.sink ? curr : p.sink;
    int ws = curr - p.sw - p.bq;
    if (ws < 0) ws = 0;
    const int n_win = p.sw > 0 ? curr - ws : 0;
    const int64_t seqlen = p.kv.paged ? p.kv.seq_len(b) : 0;
    const int total = n_sel_tok + sink_end + n_win;
    for (int o = threadIdx.x; o < total; o += blockDim.x) {
        long long t = -1;
        if (o < n_sel_tok) {
            const long long st = p.indices[irow * p.BK + rs + o / p.bk];
            t = st + o % p.bk;
            if (!(t >= 0 && t < p.kv.max_tsrc && t < curr && t >= p.sink)) t = -1;
        } else if (o < n_sel_tok + sink_end) {
            t = o - n_sel_tok;
        } else {
            t = ws + (o - n_sel_tok - sink_end);
        }
        if (t >= 0) {
            int64_t ko, vo;
            kv_rows<false, true, false>(p.kv, &p.kx, b, t, kvh, seqlen, ko, vo, true);
        }
    }
}

template <int HID, bool KSCALED, bool EXT, bool ROPE = false, bool CAP = false, bool KV8 = false, bool DYN = false>
static int launch_mfma(const BsaParams &p, hipStream_t st) {
    const int hpw = p.share_first_head ? 4 / (HID / V_COLS<HID>) : 1;  // per-head index rows: one head per workgroup
    const int hgroups = (p.G + hpw - 1) / hpw;
    const long long total = (long long)p.B * p.kv.HKV * hgroups * p.NBQ;
    if (total >= 0x7fffffffLL) return HIPATTN_E_UNSUPPORTED;
    const size_t smem = sizeof(MfmaSmem<HID>);
    static bool attr_set = false;
    if (!attr_set) {
        HIPATTN_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&bsa_mfma_kernel<HID, KSCALED, EXT, ROPE, CAP, KV8, DYN>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    const BsaParamsFor<EXT> &pk = p;  // the plain kernel takes the block without the extras
    hipLaunchKernelGGL((bsa_mfma_kernel<HID, KSCALED, EXT, ROPE, CAP, KV8, DYN>), dim3((unsigned)total), dim3(NTHREADS), smem, st, pk, hgroups,
                       hpw, total);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

int bsa_mfma_launch(const BsaParams &p, int dtype, int HID, hipStream_t st) {
    if (dtype != HIPATTN_BF16) return HIPATTN_E_UNSUPPORTED;
    if (p.bq > 64) return HIPATTN_E_UNSUPPORTED;
    // the dynamic rule blends two table rows per key: variants of the pipelined loop (head dim 256: the portable kernel)
    const bool dyn = p.rope.cos && p.rope.backend == HIPATTN_EXTEND_DYNAMIC;
    if (dyn && HID > 128) return HIPATTN_E_UNSUPPORTED;
    if ((p.o_st % 4) != 0 || (p.o_sh % 4) != 0 || (p.o_sb % 4) != 0) return HIPATTN_E_UNSUPPORTED;
    bool ext = p.kx.extended();
    BsaParams plain;
    if ((p.kx.access_flags || p.kx.miss_flags) && !p.kx.cached && (HID == 64 || HID == 128 || HID == 256)) {
        // statistics only: a cheap marking pass, then the plain kernel
        const int hpw = p.share_first_head ? 4 : 1;
        const int hgroups = (p.G + hpw - 1) / hpw;
        const long long total = (long long)p.B * p.kv.HKV * hgroups * p.NBQ;
        if (total >= 0x7fffffffLL) return HIPATTN_E_UNSUPPORTED;
        hipLaunchKernelGGL(bsa_mark_kernel, dim3((unsigned)total), dim3(256), 0, st, p, hgroups, hpw);
        HIPATTN_CHECK_HIP(hipGetLastError());
        plain = p;
        plain.kx.access_flags = nullptr;
        plain.kx.miss_flags = nullptr;
        return bsa_mfma_launch(plain, dtype, HID, st);
    }
    if (p.rope.cos && p.k_prescaled) {
        set_error("bsa: prescaled keys cannot be combined with rope applied on load");
        return HIPATTN_E_ARG;
    }
#define BSA_PICK(H)                                                                  \
    case H:                                                                          \
        if (p.kx.kv8) {                                                              \
            if (p.k_prescaled) return HIPATTN_E_UNSUPPORTED;                         \
            if (p.softcap != 0.0f)                                                   \
                return p.rope.cos ? launch_mfma<H, false, true, true, true, true>(p, st)   \
                                  : launch_mfma<H, false, true, false, true, true>(p, st); \
            return p.rope.cos ? launch_mfma<H, false, true, true, false, true>(p, st)      \
                              : launch_mfma<H, false, true, false, false, true>(p, st);    \
        }                                                                            \
        if (p.softcap != 0.0f) {                                                     \
            if (p.k_prescaled) return HIPATTN_E_UNSUPPORTED;                         \
            return p.rope.cos ? launch_mfma<H, false, true, true, true>(p, st)       \
                              : launch_mfma<H, false, true, false, true>(p, st);     \
        }                                                                            \
        if (p.rope.cos) return launch_mfma<H, false, true, true>(p, st);             \
        if (p.k_prescaled) return ext ? launch_mfma<H, true, true>(p, st) : launch_mfma<H, true, false>(p, st); \
        return ext ? launch_mfma<H, false, true>(p, st) : launch_mfma<H, false, false>(p, st);
#define BSA_PICK_DYN(H)                                                                         \
    case H:                                                                                     \
        if (p.k_prescaled) return HIPATTN_E_UNSUPPORTED;                                        \
        if (p.kx.kv8)                                                                           \
            return p.softcap != 0.0f ? launch_mfma<H, false, true, true, true, true, true>(p, st)   \
                                     : launch_mfma<H, false, true, true, false, true, true>(p, st); \
        return p.softcap != 0.0f ? launch_mfma<H, false, true, true, true, false, true>(p, st)      \
                                 : launch_mfma<H, false, true, true, false, false, true>(p, st);
    if (dyn) {
        switch (HID) {
            BSA_PICK_DYN(64)
            BSA_PICK_DYN(128)
        }
        return HIPATTN_E_UNSUPPORTED;
    }
#undef BSA_PICK_DYN
    switch (HID) {
        BSA_PICK(64)
        BSA_PICK(128)
        BSA_PICK(256)
    }
#undef BSA_PICK
    return HIPATTN_E_UNSUPPORTED;
}

}  // namespace hipattn

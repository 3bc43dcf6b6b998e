// Decode (one query token per sequence) split-KV attention on the matrix cores (bf16, head dim 64 / 128).
//
// A workgroup owns one (sequence, kv head, split); its four waves walk the split's token list independently, 32
// tokens at a time (16 or 8 when the split is too short to give every wave a tile), each in a private LDS region, so
// nothing inside the loop synchronises across waves.  The G query
// heads of the GQA group play the role of query rows: S^T[token, head] = K^ . Q^^T and O^T[d, head] += V^T . P^T
// use v_mfma_f32_32x32x16_bf16 with G of the 32 columns occupied.  The matrix unit is mostly idle by design; what the
// layout buys is that a gathered K / V row is fetched once, coalesced (16 lanes per row), and that the per-token
// work on the vector unit no longer grows with G.  Partials go to the same workspace the merge kernel reads:
// [B, HEAD, nsplits, HID + 4] = acc / l, then m + log2(l).
#include "bsa.hpp"

namespace hipattn {

constexpr int DT = 32;        // tokens per wave tile
constexpr int DWAVES = 4;

template <int HID>
struct DecWaveSmem {
    uint16_t k[DT][HID + KPAD];
    uint16_t v[DT][HID + VPAD];
    // what lanes 0..31 post about the token slots of a tile, double-buffered
    long long ko[2][DT], vo[2][DT];  // row offsets (NO_ROW: zero row)
    float bias[2][DT];               // added to the slot's logit: 0, log of the visit count, -inf: empty or masked
    int rp[2][DT];                   // row of the RoPE tables
    int rp2[2][DT];                  // dynamic rule: the second row a far key's tables are blended from, -1 = no blend
};

struct DecodeMfmaParams {
    BsaParams a;
    int nsplits;
    float *ws;
};

template <int HID, bool EXT, bool ROPE, bool CAP, bool KV8>
__global__ __launch_bounds__(DWAVES * 64, 2) void bsa_decode_mfma_kernel(DecodeMfmaParams dp) {
    constexpr int KS = HID / 16;
    constexpr int DB = HID / 32;
    constexpr int PPR = HID / 8;            // 16-byte pieces per row
    constexpr int CPT = DT * PPR / 64;      // pieces per lane per tile
    constexpr int SPJ = 64 / PPR;           // token slots covered by one piece per lane
    const BsaParams &p = dp.a;
    const KVExt *kx = &p.kx;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    DecWaveSmem<HID> *all = reinterpret_cast<DecWaveSmem<HID> *>(smem_raw);

    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int col = lane & 31, hh = lane >> 5;
    DecWaveSmem<HID> &sm = all[wid];
    const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    const int G = p.G;
    const int h0 = kvh * G;
    const int64_t irow = ((int64_t)b * p.HEAD + h0) * p.idx_rows;  // query block 0, first head of the group

    const long long ppos = p.pos[(int64_t)b * p.pos_sb];
    const long long curr = ppos + 1;
    int rs = p.kse[irow * 2 + 0], re = p.kse[irow * 2 + 1];
    const long long rope_shift = ppos - p.sw - p.sink - (long long)(re - rs) * p.bk + 1;
    if (p.BK <= 0) { rs = 0; re = 0; }
    const int jend = rs + p.BK < re ? rs + p.BK : re;
    const int nsel = jend > rs ? jend - rs : 0;
    const int n_sel_tok = nsel * p.bk;
    const int sink_end = (int)(curr < p.sink ? curr : p.sink);
    long long ws0 = curr - p.sw - 1;  // block_size_q = 1
    if (ws0 < 0) ws0 = 0;
    const int n_win = p.sw > 0 ? (int)(curr - ws0) : 0;
    const int total = n_sel_tok + sink_end + n_win;
    int per = (total + dp.nsplits - 1) / dp.nsplits;
    per = (per + DT - 1) / DT * DT;
    const int o_begin = split * per;
    const int o_end = o_begin + per < total ? o_begin + per : total;
    // A split shorter than the four waves' tiles together is cut into tiles of 16 or 8 tokens, so that every wave has
    // one: a wave walks a chain of trips to memory with the staging arithmetic of its tile in between, and four
    // quarter-filled tiles side by side are a shorter chain than one or two full ones.  Slots from dte on stay empty.
    int dte = DT;
    while (dte > 8 && (o_end - o_begin + dte - 1) / dte * 2 <= DWAVES) dte >>= 1;
    const int ntiles = o_end > o_begin ? (o_end - o_begin + dte - 1) / dte : 0;
    const int bk_shift = (p.bk & (p.bk - 1)) == 0 ? __builtin_ctz(p.bk) : -1;
    const int tlimit = (int)(p.kv.max_tsrc < curr ? p.kv.max_tsrc : curr);
    const int64_t seqlen = p.kv.paged ? p.kv.seq_len(b) : 0;

    // ---- Q^ fragments: column = head of the group (B operand of the first product)
    Frag qf[KS];
    if constexpr (!ROPE) {
        const bool ok = col < G;
        const uint16_t *qrow = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_sb + (int64_t)(h0 + (ok ? col : 0)) * p.q_sh;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            uint4 qraw = make_uint4(0, 0, 0, 0);
            if (ok) qraw = *reinterpret_cast<const uint4 *>(qrow + ks * 16 + hh * 8);
            const uint32_t w[4] = {qraw.x, qraw.y, qraw.z, qraw.w};
#pragma unroll
            for (int e = 0; e < 4; e++)
                qf[ks].u[e] = cvt_pk_bf16(__uint_as_float(w[e] << 16) * p.c_q, __uint_as_float(w[e] & 0xffff0000u) * p.c_q);
        }
    } else {
        // The query keeps its own position (attention_decode_bsa.py:135-262).  A wave is one tile deep in a chain of
        // trips to memory here, so every instruction of this prologue is paid in full: instead of the G lanes that
        // own a column rotating their whole row (8 pieces of 100 instructions), every lane rotates and scales one
        // 16-byte piece (column c of its half-wave: head c % GP, k-step c / GP; the partner piece of the rotation is
        // KS / 2 k-steps away, i.e. 16 lanes) and the owners collect their KS pieces from their half-wave.
        constexpr int GP = 32 / KS;  // heads per pass
        const uint16_t *ct = reinterpret_cast<const uint16_t *>(p.rope.cos) + p.rope.row(ppos);
        const uint16_t *st = reinterpret_cast<const uint16_t *>(p.rope.sin) + p.rope.row(ppos);
        const int pks = col / GP, pg = col % GP;
        const uint4 tc = *reinterpret_cast<const uint4 *>(ct + (pks % (KS / 2)) * 16 + hh * 8);
        const uint4 ts = *reinterpret_cast<const uint4 *>(st + (pks % (KS / 2)) * 16 + hh * 8);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) qf[ks].q = make_uint4(0, 0, 0, 0);
        for (int g0 = 0; g0 < G; g0 += GP) {  // one pass unless the group has more heads than a pass holds
            const bool have = g0 + pg < G;
            const uint16_t *qrow = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_sb + (int64_t)(h0 + (have ? g0 + pg : 0)) * p.q_sh;
            const uint4 own = *reinterpret_cast<const uint4 *>(qrow + pks * 16 + hh * 8);
            const uint4 oth = make_uint4(lane_xor<16>(own.x), lane_xor<16>(own.y), lane_xor<16>(own.z), lane_xor<16>(own.w));
            const uint4 rot = rope_piece(own, oth, tc, ts, pks < KS / 2);
            const uint32_t w[4] = {rot.x, rot.y, rot.z, rot.w};
            uint32_t sc[4];
#pragma unroll
            for (int e = 0; e < 4; e++)
                sc[e] = cvt_pk_bf16(__uint_as_float(w[e] << 16) * p.c_q, __uint_as_float(w[e] & 0xffff0000u) * p.c_q);
            const bool mine = col >= g0 && col < g0 + GP && col < G;  // this lane owns column col, served by this pass
            const int src0 = mine ? ((lane & 32) | (col - g0)) : (lane & 32);
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t got = (uint32_t)__shfl((int)sc[e], src0 + GP * ks);
                    if (mine) qf[ks].u[e] = got;
                }
            }
        }
    }

    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] = 0.0f;
    float m_run = -INFINITY;  // log2 units
    float l_run = 0.0f;

    // ---- pipeline over this wave's tiles (wid, wid + 4, ...): token slots are resolved two tiles ahead (index and
    // page-table loads in flight), posted one tile ahead, and the K / V rows of the next tile are in flight while the
    // current tile is multiplied
    long long m_ko = NO_ROW, m_vo = NO_ROW;
    int m_rp = 0, m_rp2 = -1;
    float m_bias = -INFINITY;
    bool dyn = false;  // the "dynamic_extend" rule: sink and selected keys rotated with a blend of two table rows
    if constexpr (ROPE) dyn = p.rope.backend == HIPATTN_EXTEND_DYNAMIC;
    // The index entry of a slot is requested one resolve ahead of the resolve that uses it, and the plain build looks
    // a token's page up once for K and V: a resolve then waits for one trip to memory (the page-table entry; none on
    // a dense tensor) instead of three in a row (index entry, page for K, page for V).
    long long pre_s64 = 0;
    auto index_of = [&](int tile) -> long long {  // the index entry of this lane's slot of `tile`, 0 where it has none
        const int o = o_begin + tile * dte + lane;
        if (lane < dte && o < o_end && o < n_sel_tok) {
            const int bi = bk_shift >= 0 ? (o >> bk_shift) : o / p.bk;
            return p.indices[irow * p.BK + rs + bi];
        }
        return 0;
    };
    auto resolve = [&](int tile) {  // lanes 0..31
        const long long s64 = pre_s64;
        pre_s64 = (tile + DWAVES < ntiles) ? index_of(tile + DWAVES) : 0;
        if (lane >= DT) return;
        const int o = o_begin + tile * dte + lane;
        int t = -1, win = 0;
        long long rpos = 0;
        float bias = 0.0f;
        if (lane < dte && o < o_end) {
            if (o < n_sel_tok) {
                const int bi = bk_shift >= 0 ? (o >> bk_shift) : o / p.bk;
                const int e = o - bi * p.bk;
                if (p.seam_extra > 0) {  // weight of a token attended v times: v * exp(logit) = exp(logit + log v)
                    const int visits = bsa_seam_multiplicity(rs + bi, p.seam_blocks, p.seam_extra);
                    if (visits > 1) bias = __logf((float)visits);
                }
                const int st = (s64 >= 0 && s64 < 0x7fffffffLL) ? (int)s64 : -0x40000000;
                t = st + e;
                if (!(t >= p.sink && t < tlimit)) t = -1;
                if constexpr (ROPE)
                    rpos = bsa_rope_far_pos(p.rope, (long long)(rs + bi + p.sink / p.bk) * p.bk + e, rope_shift, ppos, p.sw);
            } else if (o < n_sel_tok + sink_end) {
                t = o - n_sel_tok;
                if constexpr (ROPE)
                    rpos = bsa_rope_far_pos(p.rope, bsa_decode_sink_slot(t, p.sink_share, p.bk), rope_shift, ppos, p.sw);
            } else {
                t = (int)ws0 + (o - n_sel_tok - sink_end);
                win = 1;
                rpos = t;
            }
        }
        int64_t ko = NO_ROW, vo = NO_ROW;
        // access flags of a paged cache are per page, and the slots of a tile are mostly runs of consecutive tokens:
        // the first slot of a run inside a page stores the flag for the run (an offload cache keeps its own marks
        // per block, which need not be pages: there every slot marks)
        bool flag_leader = true;
        if constexpr (EXT) {
            const int t_before = __shfl_up(t, 1);
            if (p.kv.paged && !kx->cached)
                flag_leader = lane == 0 || t < 0 || t_before != t - 1 || (t & (p.kv.page_size - 1)) == 0 || (int64_t)t >= seqlen;
        }
        if (t >= 0) {
            const bool att = p.non_causal || (win ? ((long long)t <= ppos && ppos < (long long)t + p.sw) : ((long long)t + p.sw <= ppos));
            // a staged but masked token still counts as an access; its rows are not needed
            if (att) {
                if constexpr (EXT) {
                    // (flags are stored without looking first: a look is a trip to memory in a chain of them)
                    kv_rows<true, EXT, false>(p.kv, kx, b, t, kvh, seqlen, ko, vo, flag_leader);
                } else if (!p.kv.paged) {
                    if (t < p.kv.tsrc) {
                        ko = (int64_t)b * p.kv.k_stride_b + (int64_t)t * p.kv.k_stride_t + (int64_t)kvh * p.kv.k_stride_h;
                        vo = (int64_t)b * p.kv.v_stride_b + (int64_t)t * p.kv.v_stride_t + (int64_t)kvh * p.kv.v_stride_h;
                    }
                } else {
                    const int64_t page = p.kv.page_of(b, t, seqlen), inpage = t & (p.kv.page_size - 1);
                    ko = page * p.kv.k_stride_b + inpage * p.kv.k_stride_t + (int64_t)kvh * p.kv.k_stride_h;
                    vo = page * p.kv.v_stride_b + inpage * p.kv.v_stride_t + (int64_t)kvh * p.kv.v_stride_h;
                }
            } else {
                if constexpr (EXT) kv_rows<false, EXT>(p.kv, kx, b, t, kvh, seqlen, ko, vo, true);
                ko = NO_ROW;
                vo = NO_ROW;
                t = -1;
            }
        }
        m_ko = ko;
        m_vo = vo;
        m_bias = t >= 0 ? bias : -INFINITY;
        if constexpr (ROPE) {
            m_rp = (int)p.rope.clamp(rpos);
            // one query row: pmax = its position + 1 (attention_decode_bsa.py, as in the query-block kernel)
            m_rp2 = (dyn && !win && t >= 0) ? (int)p.rope.clamp(dynamic_extend_pos(t, ppos, ppos + 1, p.rope.model_ctx)) : -1;
        }
    };
    auto post = [&](int slot2) {  // lanes 0..31 -> meta buffer slot2 (0 / 1)
        if (lane >= DT) return;
        sm.ko[slot2][lane] = m_ko;
        sm.vo[slot2][lane] = m_vo;
        sm.bias[slot2][lane] = m_bias;
        if constexpr (ROPE) {
            sm.rp[slot2][lane] = m_rp;
            sm.rp2[slot2][lane] = m_rp2;
        }
    };
    auto wave_sync = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    uint4 kreg[CPT], vreg[CPT];
    auto fetch = [&](int slot2) {  // piece c = lane + 64 j is 16-byte piece c % PPR of slot c / PPR
#pragma unroll
        for (int j = 0; j < CPT; j++) {
            if (j * SPJ >= dte) break;  // (wave-uniform) slots from dte on are empty
            const int c = lane + 64 * j;
            const int slot = c / PPR, piece = c % PPR;
            const long long ko = sm.ko[slot2][slot], vo = sm.vo[slot2][slot];
            kreg[j] = make_uint4(0, 0, 0, 0);
            vreg[j] = make_uint4(0, 0, 0, 0);
            if (ko != NO_ROW) kreg[j] = load_kv_piece<KV8>(p.kv.k, ko + piece * 8);
            if (vo != NO_ROW) vreg[j] = load_kv_piece<KV8>(p.kv.v, vo + piece * 8);
        }
    };
    auto scale_store_k = [&](uint4 kq, int slot, int piece) {
        kq.x = cvt_pk_bf16(__uint_as_float(kq.x << 16) * p.c_k, __uint_as_float(kq.x & 0xffff0000u) * p.c_k);
        kq.y = cvt_pk_bf16(__uint_as_float(kq.y << 16) * p.c_k, __uint_as_float(kq.y & 0xffff0000u) * p.c_k);
        kq.z = cvt_pk_bf16(__uint_as_float(kq.z << 16) * p.c_k, __uint_as_float(kq.z & 0xffff0000u) * p.c_k);
        kq.w = cvt_pk_bf16(__uint_as_float(kq.w << 16) * p.c_k, __uint_as_float(kq.w & 0xffff0000u) * p.c_k);
        *reinterpret_cast<uint4 *>(&sm.k[slot][piece * 8]) = kq;
    };
    auto commit = [&](int slot2) {
        if constexpr (!ROPE) {
#pragma unroll
            for (int j = 0; j < CPT; j++) {
                if (j * SPJ >= dte) break;
                const int c = lane + 64 * j;
                const int slot = c / PPR, piece = c % PPR;
                scale_store_k(kreg[j], slot, piece);
                *reinterpret_cast<uint4 *>(&sm.v[slot][piece * 8]) = vreg[j];
            }
        } else {
            // V first: its registers then hold the table pieces.  The table pieces of half the tile's K pieces are
            // requested back to back and used after one wait: left to the register allocator, which has nothing to
            // spare here, each piece's two loads were requested and waited for on their own, eight trips per tile.
#pragma unroll
            for (int j = 0; j < CPT; j++) {
                if (j * SPJ >= dte) break;
                const int c = lane + 64 * j;
                *reinterpret_cast<uint4 *>(&sm.v[c / PPR][(c % PPR) * 8]) = vreg[j];
            }
            constexpr int HB = CPT / 2 > 0 ? CPT / 2 : 1;
#pragma unroll
            for (int j0 = 0; j0 < CPT; j0 += HB) {
                if (j0 * SPJ >= dte) break;
                uint4 cc[HB], sn[HB];
#pragma unroll
                for (int jj = 0; jj < HB; jj++) {
                    if ((j0 + jj) * SPJ >= dte) break;
                    const int c = lane + 64 * (j0 + jj);
                    const int slot = c / PPR, piece = c % PPR;
                    const int64_t tr = (int64_t)sm.rp[slot2][slot] * p.rope.stride_t + (piece % (PPR / 2)) * 8;
                    cc[jj] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.cos) + tr);
                    sn[jj] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.sin) + tr);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int jj = 0; jj < HB; jj++) {
                    if ((j0 + jj) * SPJ >= dte) break;
                    const int c = lane + 64 * (j0 + jj);
                    const int slot = c / PPR, piece = c % PPR;
                    uint4 kq = kreg[j0 + jj];
                    if (dyn) {  // wave-uniform
                        const int r2 = sm.rp2[slot2][slot];
                        const int64_t tr2 = (int64_t)(r2 < 0 ? 0 : r2) * p.rope.stride_t + (piece % (PPR / 2)) * 8;
                        const uint4 c2 = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.cos) + tr2);
                        const uint4 s2 = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.sin) + tr2);
                        const float wa = r2 >= 0 ? 0.75f : 1.0f, wb = r2 >= 0 ? 0.25f : 0.0f;
                        cc[jj] = rope_blend_piece(cc[jj], c2, wa, wb);
                        sn[jj] = rope_blend_piece(sn[jj], s2, wa, wb);
                    }
                    const uint4 oth = make_uint4(lane_xor<PPR / 2>(kq.x), lane_xor<PPR / 2>(kq.y), lane_xor<PPR / 2>(kq.z),
                                                 lane_xor<PPR / 2>(kq.w));
                    scale_store_k(rope_piece(kq, oth, cc[jj], sn[jj], piece < PPR / 2), slot, piece);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    const int my_tiles = ntiles > wid ? (ntiles - wid + DWAVES - 1) / DWAVES : 0;
    if (my_tiles > 0 && dte < DT) {  // rows of the slots that never get a token: read by the products, so zero
#pragma unroll
        for (int j = 0; j < CPT; j++) {
            if (j * SPJ < dte) continue;
            const int c = lane + 64 * j;
            *reinterpret_cast<uint4 *>(&sm.k[c / PPR][(c % PPR) * 8]) = make_uint4(0, 0, 0, 0);
            *reinterpret_cast<uint4 *>(&sm.v[c / PPR][(c % PPR) * 8]) = make_uint4(0, 0, 0, 0);
        }
    }
    if (my_tiles > 0) {
        pre_s64 = index_of(wid);
        resolve(wid);
        post(0);
        wave_sync();
        // Slots are resolved before the rows of the tile ahead are requested, never after: a resolve waits for its
        // index and page-table entries, vector-memory operations complete in order, and behind the row loads that
        // wait would expose their whole latency ahead of the math that is meant to hide it.
        if (my_tiles > 1) resolve(wid + DWAVES);
        fetch(0);
    }
    for (int it = 0; it < my_tiles; it++) {
        const int cur = it & 1;
        commit(cur);                                   // rows of tile `it` -> LDS
        if (it + 1 < my_tiles) post(cur ^ 1);          // slots of tile it + 1
        wave_sync();
        if (it + 2 < my_tiles) resolve(wid + (it + 2) * DWAVES);
        if (it + 1 < my_tiles) fetch(cur ^ 1);         // rows of tile it + 1 fly during the math below

        // ---- S^T = K^ Q^^T  (32 tokens x 32 columns, G of them live)
        f32x16 sacc;
#pragma unroll
        for (int i = 0; i < 16; i++) sacc[i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            Frag a;
            a.q = *reinterpret_cast<const uint4 *>(&sm.k[col][ks * 16 + hh * 8]);
            sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, qf[ks].v, sacc, 0, 0, 0);
        }
        if constexpr (CAP) {
            const float k2 = 2.0f * LOG2E / p.softcap;
#pragma unroll
            for (int i = 0; i < 16; i++) sacc[i] = softcap_logit(sacc[i], p.softcap, k2);
        }
        // ---- mask + online softmax; element i of a lane is token slot (i/4)*8 + hh*4 + i%4 (masked tokens were
        // posted as empty slots)
        float mx = -INFINITY;
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
            const float4 tt = *reinterpret_cast<const float4 *>(&sm.bias[cur][i4 * 8 + hh * 4]);
            const float ts[4] = {tt.x, tt.y, tt.z, tt.w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float s = sacc[i4 * 4 + e] + ts[e];
                sacc[i4 * 4 + e] = s;
                mx = fmaxf(mx, s);
            }
        }
        mx = fmaxf(mx, swap_halves(mx)) * LOG2E;
        float m_use = m_run;
        float alpha = 1.0f;
        if (mx > m_run + RESCALE_STEP || m_run == -INFINITY) {
            m_use = fmaxf(m_run, mx);
            alpha = (m_use == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_use);
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
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;
        }
        // ---- O^T += V^T P^T through transposing LDS reads of the row-major V tile
#pragma unroll
        for (int db = 0; db < DB; db++) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                Frag a;
                const int trow = j * 16 + hh * 4 + ((lane & 15) >> 2);
                const int tcol = db * 32 + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
                a.d[0] = lds_read_tr16(&sm.v[trow][tcol]);
                a.d[1] = lds_read_tr16(&sm.v[trow + 8][tcol]);
                oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, pf[j].v, oacc[db], 0, 0, 0);
            }
        }
        __builtin_amdgcn_wave_barrier();
    }

    // ---- merge the four waves' states through LDS, write the partial of this split
    const float l_all = l_run + swap_halves(l_run);
    __syncthreads();  // every wave is done with its tile region
    float *s_m = reinterpret_cast<float *>(smem_raw);             // [DWAVES][32]
    float *s_l = s_m + DWAVES * 32;                               // [DWAVES][32]
    float *s_acc = s_l + DWAVES * 32;                             // [DWAVES][G][HID]
    if (col < G) {
        if (hh == 0) {
            s_m[wid * 32 + col] = m_run;
            s_l[wid * 32 + col] = l_all;
        }
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int i = 0; i < 16; i++)
                s_acc[((int64_t)wid * G + col) * HID + db * 32 + (i >> 2) * 8 + hh * 4 + (i & 3)] = oacc[db][i];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * HID; idx += DWAVES * 64) {
        const int g = idx / HID, d = idx % HID;
        float mm = -INFINITY;
#pragma unroll
        for (int w = 0; w < DWAVES; w++) mm = fmaxf(mm, s_m[w * 32 + g]);
        float ll = 0.0f, aa = 0.0f;
        if (mm > -INFINITY) {
#pragma unroll
            for (int w = 0; w < DWAVES; w++) {
                const float wgt = exp2f(s_m[w * 32 + g] - mm);
                ll += s_l[w * 32 + g] * wgt;
                aa += s_acc[((int64_t)w * G + g) * HID + d] * wgt;
            }
        }
        float *wrow = dp.ws + (((int64_t)b * p.HEAD + h0 + g) * dp.nsplits + split) * (HID + 4);
        wrow[d] = ll > 0.0f ? aa / ll : 0.0f;
        if (d == 0) wrow[HID] = ll > 0.0f ? mm + log2f(ll) : -INFINITY;
    }
}

template <int HID, bool EXT, bool ROPE, bool CAP, bool KV8>
static int launch_dec(const DecodeMfmaParams &dp, hipStream_t st) {
    const size_t tile_bytes = sizeof(DecWaveSmem<HID>) * DWAVES;
    const size_t merge_bytes = (size_t)(2 * DWAVES * 32 + DWAVES * dp.a.G * HID) * sizeof(float);
    const size_t smem = tile_bytes > merge_bytes ? tile_bytes : merge_bytes;
    if (smem > 160 * 1024) return HIPATTN_E_UNSUPPORTED;
    static bool attr_set = false;
    static size_t attr_bytes = 0;
    if (!attr_set || smem > attr_bytes) {
        HIPATTN_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&bsa_decode_mfma_kernel<HID, EXT, ROPE, CAP, KV8>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)(160 * 1024)));
        attr_set = true;
        attr_bytes = 160 * 1024;
    }
    dim3 grid((unsigned)dp.nsplits, (unsigned)dp.a.kv.HKV, (unsigned)dp.a.B), block(DWAVES * 64);
    hipLaunchKernelGGL((bsa_decode_mfma_kernel<HID, EXT, ROPE, CAP, KV8>), grid, block, smem, st, dp);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

template <int HID>
static int pick_dec(const DecodeMfmaParams &dp, hipStream_t st) {
    const BsaParams &p = dp.a;
    const bool rope = p.rope.cos != nullptr, cap = p.softcap != 0.0f, kv8 = p.kx.kv8 != 0;
    const bool ext = p.kx.cached || p.kx.access_flags || p.kx.miss_flags;
    // the plain build covers the common step; every option runs in the extended build
    if (!rope && !cap && !kv8) return ext ? launch_dec<HID, true, false, false, false>(dp, st)
                                          : launch_dec<HID, false, false, false, false>(dp, st);
    if (kv8) {
        if (rope) return cap ? launch_dec<HID, true, true, true, true>(dp, st) : launch_dec<HID, true, true, false, true>(dp, st);
        return cap ? launch_dec<HID, true, false, true, true>(dp, st) : launch_dec<HID, true, false, false, true>(dp, st);
    }
    // rotation without any other option is every cached step of a serving loop that rotates: it gets the plain build
    if (rope && !cap && !ext) return launch_dec<HID, false, true, false, false>(dp, st);
    if (rope) return cap ? launch_dec<HID, true, true, true, false>(dp, st) : launch_dec<HID, true, true, false, false>(dp, st);
    return launch_dec<HID, true, false, true, false>(dp, st);
}

int bsa_decode_mfma_launch(const BsaParams &p, int dtype, int HID, int nsplits, float *ws, hipStream_t st) {
    if (dtype != HIPATTN_BF16 || p.G > 8) return HIPATTN_E_UNSUPPORTED;
    DecodeMfmaParams dp;
    dp.a = p;
    dp.nsplits = nsplits;
    dp.ws = ws;
    switch (HID) {
        case 64: return pick_dec<64>(dp, st);
        case 128: return pick_dec<128>(dp, st);
    }
    return HIPATTN_E_UNSUPPORTED;
}

}  // namespace hipattn

// Mask-estimation scan stage for bf16 inputs on the matrix cores.
//
// Scores of a binary-search iteration are S[query row, sampled token] = q^ . k^.  One
// v_mfma_f32_32x32x16_bf16 covers 32 query rows x 32 sampled tokens x 16 head-dim elements with
//   A = Q^ rows     (resident in registers for the whole kernel),
//   B = K^ rows     (lane n%32 <-> token; rows are fetched with fully coalesced 16-lane-per-row loads,
//                    parked in a per-wave LDS tile with an XOR swizzle of the 16-byte pieces, and read
//                    back in operand layout without bank conflicts),
//   D[row, token]   (a lane ends up with 16 query rows of ITS token: the max over rows is in-lane).
// A wave owns NB blocks of 32 tokens = 16*NB chunks (left and right sample of a chunk sit in
// adjacent lanes); the program-level gate and iteration count of the reference (a "program" is a
// group of block_chunk chunks) are recomputed by every wave from the group's chunk list, so a
// program can be split over several waves without changing results.
//
// Accumulation order of the dot product is the hardware's: two groups of 8 per instruction,
// instructions chained through the f32 accumulator; head-dim element of (instruction ks, lane half
// hh, i) is  hh*HID/2 + ks*8 + i.  The order is part of the operator's numeric definition.
#include <stdlib.h>

#include "mask_common.hpp"

namespace hipattn {
static __device__ __align__(16) uint16_t g_scan_zero_row[256];

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

union BFrag {
    bf16x8 v;
    uint32_t u[4];
    uint4 q;
};

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;

// two f32 -> packed bf16 pair with round-to-nearest-even (one v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t cvt_pk_bf16(float a, float b) {
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

__device__ __forceinline__ uint32_t scale_pack(uint32_t w, float c) {
    return cvt_pk_bf16(__uint_as_float(w << 16) * c, __uint_as_float(w & 0xffff0000u) * c);
}

// rotated position of a query row / of the sampled key of chunk c (attention_extend.py:632-647, :289-298)
__device__ __forceinline__ int64_t rope_qpos(const RopeView &r, long long pos, int n, int sw_eff) {
    if (r.backend == HIPATTN_EXTEND_RELATIVE) return 1 + (int64_t)sw_eff;
    if (r.backend == HIPATTN_EXTEND_INFLLM) return sw_eff;
    if (rope_follows_token(r.backend)) return pos;
    const long long cap = (long long)n + sw_eff;
    return pos < cap ? pos : cap;
}
__device__ __forceinline__ int64_t rope_kpos(const RopeView &r, int c, int side) {
    if (r.backend == HIPATTN_EXTEND_RELATIVE) return side;
    if (r.backend == HIPATTN_EXTEND_STREAMING) return c;
    return 0;
}

// Waves per SIMD the register allocator is held to: the scans are chains of dependent round trips (token logic, row
// loads, products, compares) that only other waves can fill, so a variant that drifts a few registers over the
// boundary of its class loses a quarter of its throughput (the coalesced variant had grown to 144 registers).
template <int HID>
constexpr bool PPR_OK = HID / 8 <= 16;
constexpr int mask_stage_waves(int HID, int MB, int NB, int RMODE) {
    const int w = RMODE == 1 ? (MB == 2 ? 1 : 2) : (RMODE == 10 || RMODE == 11) ? 3
                : (MB == 1 && NB == 1) ? 4 : (MB == 1 || (NB == 1 && RMODE == 3)) ? 3 : 2;
    return HID > 128 ? (w + 1) / 2 : w;  // 256-element rows: twice the fragments
}
// RMODE = 1 (direct path, one token block per wave, extended parameter block): every sampled key row is rotated
// before it is scaled.  The two halves of a row sit in the two half-waves (lane and lane ^ 32) at the same k-step,
// and under the RELATIVE, STREAMING and INFLLM rules the rotated position of a lane's key never changes over the
// iterations, so its cos/sin entries are loaded once and stay in registers.  The DYNAMIC rule rotates by the
// sampled token itself (attention_extend.py:254-274) and reloads them with every sample.
// RMODE = 2 (prescaled keys, extended parameter block): the keys were rotated and scaled ahead of the scan, one
// copy per sample side; right-hand samples read the copy k_side_delta elements further on.
// RMODE = 4 (prescaled keys, one token block per wave, wide launches): the 32 sampled rows of an iteration are fetched
// with eight direct-to-LDS load instructions in which sixteen consecutive lanes cover one 256-byte row (a lane reading
// its own half row makes every load instruction touch 64 cache lines, and the address unit then passes one line per
// clock: 9.5 TB/s over the chip on L2-resident rows where the coalesced shape reaches 30), into an 8 KB tile of the
// wave with the 16-byte pieces of row r permuted by r, and read back in operand layout.
// RMODE = 7 / 8 (as 5 / 4, programs of up to 16 query rows): the products run on v_mfma_f32_16x16x32_bf16, whose four
// groups of eight elements per instruction are given the order in which two steps of the 32x32x16 instruction take
// theirs (k-step 2j lower half, 2j upper half, 2j + 1 lower, 2j + 1 upper): the accumulation chain of a score, and
// with it every bit of the result, is the same (compared on 2M products of adversarial inputs, while any other order
// of the groups differs in a quarter of them), at half the matrix cycles, 24 registers fewer and no rows of zeros.
// RMODE = 9: as 6, with the 32-bit row offsets of RMODE = 5 (a dense key tensor under 4 GB per batch item).
// RMODE = 6: a single query token (as RMODE = 3) with the rows fetched as under RMODE = 4; keys prescaled or scaled
// after the tile is read back.
// RMODE = 10 / 11 (as 7 / 8 on keys as stored, rotation on load under the RELATIVE rule): left-hand samples sit at
// position 0 and right-hand samples at position 1, so the wave's tile holds the sixteen left-hand rows first and the
// sixteen right-hand rows behind them, and the products of the 16-token halves are formed one after the other:
// only the second half's fragments are rotated (with the one table row of position 1, kept in registers; the partner
// piece of a fragment is read from the same tile row), and a rotation to position 0 changes nothing as long as the
// table's first row is (1, 0), which every wave checks for itself (a table that is scaled there takes the slow way:
// the first half is rotated too).  Half the rotation work of RMODE = 1 and its load shape exchanged for the
// coalesced one.
// RMODE = 3 (no rotation, one token block per wave, a single query token): the one valid program row is that token's
// row, which the kernel scales itself; no preparation launch is needed.
// KV8 = true (extended parameter block, unscaled keys): key rows are fp8 (e5m2) bytes, widened on load.
template <int HID, int MB, int NB, bool PRESCALED, bool VIA_LDS, bool EXT, int RMODE = 0, bool KV8 = false>
__global__ __launch_bounds__(VIA_LDS ? 64 : 256) __attribute__((amdgpu_waves_per_eu(mask_stage_waves(HID, MB, NB, RMODE))))
void mask_stage_mfma_kernel(MaskParamsFor<EXT> p, int nsub, int hpw) {
    constexpr bool ROPE = RMODE == 1;
    constexpr bool QINL = RMODE == 3 || RMODE == 6 || RMODE == 9;  // query rows scaled here instead of read from the prepared workspace
    static_assert(!QINL || NB == 1, "inline query rows: the one-token-block variants only");
    constexpr bool DMA = RMODE >= 4 && RMODE <= 11;  // rows fetched coalesced, straight into a per-wave LDS tile
    constexpr bool OFF32 = RMODE == 5 || RMODE == 7 || RMODE == 9 || RMODE == 10;  // their addresses: 32-bit byte offsets from the batch item's first key row
    constexpr bool M16 = RMODE == 7 || RMODE == 8 || RMODE == 10 || RMODE == 11;    // programs of up to 16 query rows on the 16x16x32 instruction
    constexpr bool SPLIT = RMODE == 10 || RMODE == 11;  // RELATIVE rule on keys as stored: tile rows ordered by sample side
    static_assert(!DMA || (!VIA_LDS && NB == 1 && !KV8), "coalesced direct-to-LDS rows: one token block per wave, bf16 keys");
    static_assert(!DMA || RMODE == 6 || RMODE == 9 || SPLIT || PRESCALED, "coalesced rows on wide launches: prescaled keys");
    static_assert(!SPLIT || (EXT && !PRESCALED && PPR_OK<HID>), "side-split variant: extended build, keys as stored, sixteen pieces per row at most");
    static_assert(!M16 || (MB == 1 && HID % 32 == 0), "16-row variant: one row block, head dim a multiple of 32");
    static_assert(!KV8 || (EXT && !PRESCALED), "fp8 keys: extended build, scaled in the kernel");
    static_assert(!ROPE || (EXT && !VIA_LDS && !PRESCALED), "rope variant: direct path of the extended build");
    static_assert(RMODE != 2 || (EXT && PRESCALED), "two-sided prescaled keys: extended build of the prescaled path");
    const KVExt *kx = nullptr;
    if constexpr (EXT) kx = &p.kx;
    constexpr int KS = HID / 16;
    constexpr int HALF = HID / 2;
    constexpr int PPR = HID / 8;                  // 16-byte pieces per key row
    constexpr int RPI = 64 / PPR;                 // rows fetched per load instruction
    constexpr int NROWS = NB * 32;                // sampled rows per iteration of this wave
    constexpr int SWZ = (PPR < 16 ? PPR : 16) - 1;
    constexpr int SWZ_DIV = PPR < 16 ? 16 / PPR : 1;
    constexpr bool SHAREABLE = DMA && PRESCALED && RMODE != 6 && RMODE != 9;  // prefill variants: the first round's rows can be fetched once per workgroup
    __shared__ __align__(16) uint4 s_rows[VIA_LDS ? NROWS * PPR : DMA ? (SHAREABLE ? 5 : 4) * 32 * PPR : 1];  // DMA: one tile per wave (up to four), one shared
    __shared__ int64_t s_off[VIA_LDS ? NROWS : 1];
    // a workgroup holds `hpw` waves = `hpw` query heads of one GQA group working on the same chunks:
    // their early-iteration samples coincide, so they share cache lines in the CU's L1
    const int lane = threadIdx.x & 63;
    const int n = lane & 31, hh = lane >> 5;
    const int side = n & 1;

    long long L = xcd_remap((long long)blockIdx.x, p.total);
    const int hblocks = (p.G + hpw - 1) / hpw;
    const int hin = (int)(L % hblocks) * hpw + (int)(threadIdx.x >> 6);
    L /= hblocks;
    if (hin >= p.G) return;
    const int sub = (int)(L % nsub);
    L /= nsub;
    const int s = (int)(L % p.BS);
    L /= p.BS;
    const int group_reps = (MB == 2 || DMA) ? p.group_reps : 1;
    const int groups_outer = (p.ngroups + group_reps - 1) / group_reps;
    const int g0 = (int)(L % groups_outer) * group_reps;
    L /= groups_outer;
    const int kvh = (int)(L % p.kv.HKV);
    const int b = (int)(L / p.kv.HKV);
    const int h = kvh * p.G + hin;

    const int BC = p.block_chunk;
    const int hgi = p.hg == 1 ? 0 : h;
    const int64_t row_in = (((int64_t)b * p.BS + s) * p.hg + hgi) * p.n;
    const int64_t row_out = (((int64_t)b * p.BS + s) * p.HEAD + h) * p.n;
    const int64_t red_out = ((int64_t)b * p.BS + s) * p.n;

    // ---- rows of this program
    const long long qb = (long long)(p.BDST - 1) - (long long)(p.BS - 1) * p.scan_stride + (long long)s * p.scan_stride;
    const long long myrow = qb * p.BQ + (long long)lane * p.stride_q;
    const bool rv = (lane < p.nrows) && (myrow >= 0) && (myrow < p.TDST);
    const unsigned long long rowmask = __ballot(rv);
    const long long mypos = rv ? p.pos[(int64_t)b * p.pos_sb + myrow * p.pos_st] : 0x7fffffffffffffffLL;
    const long long pmin = wave_min_ll(mypos);

    // ---- Q^ fragments: lane (row = mb*32 + n, half hh) holds elements hh*HALF + ks*8 .. +8.
    // Rows were averaged, rounded and scaled once per stage by qhat_kernel: [B, BS, HEAD] blocks of nrows * HID
    // elements, laid out by (k-step, row half, row) so that the lanes of a load instruction read consecutive pieces.
    // They are fetched when the first chunk group of this wave has work and then serve all of its groups.
    BFrag qf[M16 ? 1 : MB][M16 ? 1 : KS];
    BFrag qf16[M16 ? KS / 2 : 1];  // 16-row variant: lane (row l % 16, group l / 16) holds k-step 2j + (l / 32), half (l / 16) % 2
    bool q_loaded = false;
    if constexpr (QINL) {
        // A single query token: row 0 of the program is that token's row of this head, scaled here; no preparation
        // launch ran.  Every wave of the launch wants one of a handful of rows, so they are read through the
        // scalar cache (uniform address, constant address space): as vector loads, thousands of waves queue up on
        // the same few cache lines (1M-key decode: the 256-token stage 122 us against 116).
        typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
        typedef const u32x4_t __attribute__((address_space(4))) *cptr_t;
        const uint64_t qaddr = (uint64_t)(reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh);
        const uint64_t qaddr_u = ((uint64_t)__builtin_amdgcn_readfirstlane((int)(qaddr >> 32)) << 32) |
                                 (uint32_t)__builtin_amdgcn_readfirstlane((int)(qaddr & 0xffffffffu));
        cptr_t qs = (cptr_t)qaddr_u;
        const bool mine = (n == 0) && (rowmask & 1ull);
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                const u32x4_t lo = qs[ks], hi = qs[KS + ks];  // the k-step's pieces of the two halves of the row
                uint32_t w[4];
#pragma unroll
                for (int e = 0; e < 4; e++) w[e] = (mb == 0 && mine) ? scale_pack(hh ? hi[e] : lo[e], p.c_q) : 0u;
                qf[mb][ks].q = make_uint4(w[0], w[1], w[2], w[3]);
            }
        q_loaded = true;
    }
    // which of this lane's accumulator elements belong to valid query rows:
    // element (mb, i) <-> row mb*32 + (i/4)*8 + hh*4 + i%4
    unsigned vm[MB];
    bool all_rows = true;
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        vm[mb] = 0;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int j = mb * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
            if ((j < p.nrows) && ((rowmask >> j) & 1ull)) vm[mb] |= 1u << i;
        }
    }
    // fast paths: exactly the first 16 / 32 / 64 rows valid
    const int fast_rows = (p.nrows == 16 && rowmask == 0xffffull) ? 16
                        : (p.nrows == 32 && rowmask == 0xffffffffull) ? 32
                        : (MB == 2 && p.nrows == 64 && rowmask == ~0ull) ? 64 : 0;
    (void)all_rows;

    const int64_t seqlen = p.kv.paged ? p.kv.seq_len(b) : 0;
    // Coalesced variants (no block cache, the key buffer under 32 GiB): a row's place is a 32-bit number of 16-byte
    // pieces, formed here with 32-bit products (one 24-bit multiply on OFF32's dense tensors); the general routine's
    // 64-bit products, its cached branches and the scalar registers they pin (spilled and re-read in every iteration)
    // stay out of the loop.  OFF32 counts pieces from the batch item's first row, the others from kv.k.
    const uint32_t piece_st = DMA ? (uint32_t)(p.kv.k_stride_t >> 3) : 0u;
    const uint32_t piece_sb = DMA ? (uint32_t)(p.kv.k_stride_b >> 3) : 0u;  // paged: pieces per page
    const uint32_t piece_h = !DMA ? 0u
                             : (uint32_t)(((int64_t)kvh * p.kv.k_stride_h + ((OFF32 || p.kv.paged) ? 0 : (int64_t)b * p.kv.k_stride_b)) >> 3);
    const int tsrc32 = DMA ? (int)p.kv.tsrc : 0;
    // keys rotated ahead, one copy per sample side (the relative rule): this lane's samples come from its side's copy
    uint32_t side_pieces = 0u;
    if constexpr (DMA && EXT) side_pieces = side ? (uint32_t)(p.rope.k_side_delta >> 3) : 0u;
    uint8_t *flag_row = nullptr;
    if constexpr (DMA) {
        if (kx->access_flags) flag_row = kx->access_flags + (int64_t)b * kx->flags_stride_b + (int64_t)kvh * kx->flags_stride_h;
    }
    // ---- a wave walks p.group_reps consecutive chunk groups of its (scan row, head) with the same Q^ fragments
    // (only the 64-row variant: with 16 or 32 rows the fragments are a tenth of the traffic, and the loop costs the
    // registers of a third wave per SIMD)
    const int reps = (MB == 2 || DMA) ? p.group_reps : 1;
    for (int rep = 0; rep < reps; rep++) {
    const int g = g0 + rep;
    if (g >= p.ngroups) break;
    // ---- program-level quantities over the whole group of BC chunks
    int gl = (int)p.kv.max_tsrc, gr = (int)p.kv.max_tsrc;
    {
        const int ci = g * BC + lane;
        if (lane < BC && ci < p.n) {
            gl = p.chunk_left[row_in + ci];
            const int64_t rr = (int64_t)gl + p.chunk;
            gr = (int)(rr < p.right_clamp ? rr : p.right_clamp);
        }
    }
    // ---- this wave's chunks
    int cl[NB], cr[NB], cidx[NB];
    bool real[NB];
    float score[NB];
#pragma unroll
    for (int tb = 0; tb < NB; tb++) {
        const int local = (sub * NB + tb) * 16 + (n >> 1);
        cidx[tb] = g * BC + local;
        real[tb] = (local < BC) && (cidx[tb] < p.n);
        cl[tb] = (int)p.kv.max_tsrc;
        cr[tb] = (int)p.kv.max_tsrc;
        if (real[tb]) {
            cl[tb] = p.chunk_left[row_in + cidx[tb]];
            const int64_t rr = (int64_t)cl[tb] + p.chunk;
            cr[tb] = (int)(rr < p.right_clamp ? rr : p.right_clamp);
        }
        score[tb] = -32000.0f;
    }

    bool run = (rowmask != 0ull) && (pmin >= 0);
    int lim = 0;
    float width = 0.0f;
    if (run) {
        const long long lm = pmin - p.sw_eff;
        lim = (int)(lm < 0 ? 0 : lm);
        run = (pmin + (long long)p.BQ * p.scan_stride >= (long long)wave_min_i(gl));
        width = (float)wave_max_i(gr - gl);
    }
    auto store_out = [&]() {
        if (hh == 0 && side == 0) {
#pragma unroll
            for (int tb = 0; tb < NB; tb++)
                if (real[tb]) {
                    store_score(p, row_out, red_out, cidx[tb], score[tb]);
                    if (p.left_out) p.left_out[row_out + cidx[tb]] = cl[tb];
                }
        }
    };
    if (!run || !(width >= p.terminate)) {
        store_out();
        continue;
    }

    if (!q_loaded) {
        q_loaded = true;
        if constexpr (M16) {
            const uint16_t *qh = p.qhat + ((((int64_t)b * p.BS + s) * p.HEAD + h) * p.nrows) * HID;
            const int j16 = lane & 15, kb = lane >> 4;
            const bool jv = (j16 < p.nrows) && ((rowmask >> j16) & 1ull);
#pragma unroll
            for (int j = 0; j < KS / 2; j++) {
                const int ks = 2 * j + (kb >> 1), qhh = kb & 1;
                qf16[j].q = make_uint4(0, 0, 0, 0);
                if (jv) qf16[j].q = *reinterpret_cast<const uint4 *>(qh + ((int64_t)(ks * 2 + qhh) * p.nrows + j16) * 8);
            }
        } else if constexpr (!QINL) {
            const uint16_t *qh = p.qhat + ((((int64_t)b * p.BS + s) * p.HEAD + h) * p.nrows) * HID;
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
                const int j = mb * 32 + n;
                const bool jv = (j < p.nrows) && ((rowmask >> j) & 1ull);
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    qf[mb][ks].q = make_uint4(0, 0, 0, 0);
                    if (jv) qf[mb][ks].q = *reinterpret_cast<const uint4 *>(qh + ((int64_t)(ks * 2 + hh) * p.nrows + j) * 8);
                }
            }
        }
    }

    uint4 rcos[ROPE ? NB : 1][ROPE ? KS : 1], rsin[ROPE ? NB : 1][ROPE ? KS : 1];
    if constexpr (ROPE) {
#pragma unroll
        for (int tb = 0; tb < NB; tb++) {
            const int64_t tr = p.rope.row(rope_kpos(p.rope, cidx[tb], side));
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                rcos[tb][ks] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.cos) + tr + ks * 8);
                rsin[tb][ks] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.sin) + tr + ks * 8);
            }
        }
    }

    const int lrow = lane / PPR, lpos = lane % PPR;  // loader role: row within an instruction, piece slot
    // The last iterations of a search sample tokens again: in a range of two tokens one of the samples is the winner
    // of the iteration before, in a range of one both are.  A lane keeps its previous sample (token, score) and
    // takes a repeated token's score from there, or from its partner of the other side, instead of loading the row
    // and multiplying again; the score of a token depends on nothing else.  Under the relative rule (and with keys
    // rotated ahead per side) the rotation follows the side, so only the lane's own side counts there.
    bool cross_side = RMODE != 2;
    if constexpr (ROPE) cross_side = p.rope.backend != HIPATTN_EXTEND_RELATIVE;
    if constexpr (DMA && EXT) cross_side = p.rope.k_side_delta == 0;
    if constexpr (SPLIT) cross_side = false;  // a score belongs to (token, side)
    // SPLIT: the table row of position 1 for this lane's fragments (k-step 2j + kb / 2 of the half kb % 2), and whether
    // the row of position 0 leaves a key as it is
    uint4 cos1[SPLIT ? KS / 2 : 1], sin1[SPLIT ? KS / 2 : 1];
    bool left_plain = true;
    if constexpr (SPLIT) {
        const int kb = lane >> 4;
        const uint16_t *ct = reinterpret_cast<const uint16_t *>(p.rope.cos), *st = reinterpret_cast<const uint16_t *>(p.rope.sin);
        const int64_t r0 = p.rope.row(0), r1 = p.rope.row(1);
        bool ok = true;
#pragma unroll
        for (int j = 0; j < KS / 2; j++) {
            const int col = (2 * j + (kb >> 1)) * 8;
            cos1[j] = *reinterpret_cast<const uint4 *>(ct + r1 + col);
            sin1[j] = *reinterpret_cast<const uint4 *>(st + r1 + col);
            const uint4 c0 = *reinterpret_cast<const uint4 *>(ct + r0 + col), s0 = *reinterpret_cast<const uint4 *>(st + r0 + col);
            ok = ok && c0.x == 0x3f803f80u && c0.y == 0x3f803f80u && c0.z == 0x3f803f80u && c0.w == 0x3f803f80u &&
                 (s0.x & 0x7fff7fffu) == 0u && (s0.y & 0x7fff7fffu) == 0u && (s0.z & 0x7fff7fffu) == 0u && (s0.w & 0x7fff7fffu) == 0u;
        }
        left_plain = __all(ok) != 0;
    }
    int ptok[NB];
    float pscore[NB];
    // Paged keys, coalesced fetch: a round first needs its token's page-table entry, a trip to memory ahead of the
    // trip for the row.  Which token a lane samples next depends only on which half wins this round, so both
    // candidates' entries are requested now, ahead of this round's rows, and have arrived when the round ends.
    int last_mark[NB];       // the access flag this lane stored last in this search (-1: none yet)
    int pf_tok[NB][2];       // the candidates (-1: none, or outside the sequence: page 0)
    uint32_t pf_page[NB][2]; // their entries, not looked at before the next round
    bool pf_in[NB][2];
#pragma unroll
    for (int tb = 0; tb < NB; tb++) {
        ptok[tb] = -1;
        pscore[tb] = 0.0f;
        last_mark[tb] = -1;
        pf_tok[tb][0] = pf_tok[tb][1] = -1;
        pf_page[tb][0] = pf_page[tb][1] = 0u;
        pf_in[tb][0] = pf_in[tb][1] = false;
    }
    // The first round of a search samples tokens that do not depend on the query: the four heads of a workgroup
    // (same chunks, same keys) want the same 32 rows, so each wave fetches a quarter of them into a tile they all read
    // (the vector-memory path of the CU is what holds these launches, and rows that hit L1 pass through it too).
    // Every condition on the way here is the same for the waves of a workgroup, so they meet at the barriers.
    bool first = true;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    while (width >= p.terminate) {
        width *= 0.5f;
        bool share_now = false;
        if constexpr (SHAREABLE) share_now = p.share_first != 0 && first;
        bool active[NB], reuse[NB], fresh[NB];
        int ctr[NB], tok[NB];
        float rscore[NB];
        uint4 raw[(VIA_LDS || DMA) ? 1 : NB][(VIA_LDS || DMA) ? 1 : KS];
        int64_t offs[NB];
        int pieces[NB];  // OFF32: the sampled row as a piece number, -1 = none
        int mark[NB];    // coalesced fetch: the access flag (token or page) this lane sets for its sample, -1 = none
        int64_t late_mark[NB];  // direct loads: the same, set once the rows of the round have been requested
#pragma unroll
        for (int tb = 0; tb < NB; tb++) late_mark[tb] = -1;
#pragma unroll
        for (int tb = 0; tb < NB; tb++) {
            active[tb] = real[tb] && (cl[tb] < cr[tb]) && (cl[tb] <= lim) && (cl[tb] >= 0);
            ctr[tb] = (cl[tb] + cr[tb]) >> 1;
            tok[tb] = side ? ((ctr[tb] + cr[tb]) >> 1) : ((cl[tb] + ctr[tb]) >> 1);
            {
                const int otok = __shfl_xor(ptok[tb], 1);
                const float oscore = __shfl_xor(pscore[tb], 1);
                const bool mine = tok[tb] == ptok[tb];
                reuse[tb] = active[tb] && (mine || (cross_side && tok[tb] == otok));
                rscore[tb] = mine ? pscore[tb] : oscore;
            }
            fresh[tb] = __any(active[tb] && !reuse[tb]) != 0;
            int64_t off = NO_ROW;
            if constexpr (DMA) {
                pieces[tb] = -1;
                mark[tb] = -1;
                if (active[tb] && !reuse[tb]) {
                    const int t = tok[tb];
                    if (OFF32 || !p.kv.paged) {
                        if (t >= 0 && t < tsrc32) {
                            pieces[tb] = OFF32 ? (int)(__umul24((uint32_t)t, piece_st) + piece_h + side_pieces)
                                               : (int)((uint32_t)t * piece_st + piece_h + side_pieces);
                            if (flag_row && hh == 0 && !(share_now && wv != 0)) mark[tb] = t;
                        }
                    } else if (t >= 0) {
                        // the block table's entry, or page 0 beyond the sequence (as the general routine reads it)
                        uint32_t page;
                        if (t == pf_tok[tb][0]) page = pf_in[tb][0] ? pf_page[tb][0] : 0u;
                        else if (t == pf_tok[tb][1]) page = pf_in[tb][1] ? pf_page[tb][1] : 0u;
                        else page = (uint32_t)p.kv.page_of(b, t, seqlen);
                        pieces[tb] = (int)(page * piece_sb + (uint32_t)(t & (p.kv.page_size - 1)) * piece_st + piece_h + side_pieces);
                        if (flag_row && hh == 0 && !(share_now && wv != 0)) mark[tb] = (int)page;
                    }
                }
                if constexpr (!OFF32 && RMODE != 4) {  // (the 32-row variant has no registers to spare for it)
                    if (p.kv.paged) {
                        // next round's token of this lane if the left half wins, and if the right half does
                        const int ctr_l = (cl[tb] + ctr[tb]) >> 1, ctr_r = (ctr[tb] + cr[tb]) >> 1;
                        const int cand[2] = {side ? ((ctr_l + ctr[tb]) >> 1) : ((cl[tb] + ctr_l) >> 1),
                                             side ? ((ctr_r + cr[tb]) >> 1) : ((ctr[tb] + ctr_r) >> 1)};
#pragma unroll
                        for (int w = 0; w < 2; w++) {
                            // no load in a branch: a token outside the sequence reads the entry of the sequence's
                            // first token and is given page 0, as the general routine gives it
                            const bool in_seq = cand[w] >= 0 && (int64_t)cand[w] < seqlen;
                            const int64_t e = (int64_t)b * p.kv.bt_stride_b + (in_seq ? (cand[w] >> p.kv.page_shift) : 0);
                            // the low word of an entry is the page number, in a table of either width
                            const uint32_t entry = reinterpret_cast<const uint32_t *>(p.kv.block_table)[p.kv.bt_is64 ? 2 * e : e];
                            pf_tok[tb][w] = cand[w];
                            pf_page[tb][w] = entry;
                            pf_in[tb][w] = in_seq;
                        }
                    }
                }
            } else if (active[tb] && !reuse[tb]) {
                const int t = tok[tb];
                // access flags: wide launches (prefill) revisit rows constantly, so they look before they store;
                // narrow ones (decode) touch mostly fresh rows and store blindly
                if constexpr (EXT && !VIA_LDS && !DMA) {
                    off = kv_k_row<EXT, NB == 2, true>(p.kv, kx, b, t, kvh, seqlen, hh == 0, &late_mark[tb]);
                } else {
                    off = kv_k_row<EXT, NB == 2>(p.kv, kx, b, t, kvh, seqlen, hh == 0);
                }
                if constexpr (RMODE == 2) {
                    if (side && off != NO_ROW) off += p.rope.k_side_delta;
                }
                if constexpr (ROPE) {
                    if (rope_follows_token(p.rope.backend)) {
                        const int64_t tr = p.rope.row(token_extend_pos(p.rope, t, pmin, pmin + __popcll(rowmask)));
#pragma unroll
                        for (int ks = 0; ks < KS; ks++) {
                            rcos[tb][ks] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.cos) + tr + ks * 8);
                            rsin[tb][ks] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.sin) + tr + ks * 8);
                        }
                    }
                }
            }
            offs[tb] = off;
            if constexpr (VIA_LDS) {
                if (hh == 0) s_off[tb * 32 + n] = off;
            } else if constexpr (!DMA) {
                // no load in a branch of its own: lanes without a row read a row of zeros, so that the pieces of a
                // row are requested back to back and arrive after one trip to memory, not one after the other
                if (fresh[tb]) {
                    const void *rbase = off != NO_ROW ? p.kv.k : static_cast<const void *>(g_scan_zero_row);
                    const int64_t roff = off != NO_ROW ? off + hh * HALF : 0;
#pragma unroll
                    for (int ks = 0; ks < KS; ks++) raw[tb][ks] = load_kv_piece<KV8>(rbase, roff + ks * 8);
                }
            }
        }
        if constexpr (EXT && !VIA_LDS && !DMA) {
            // access flags of the round's samples, stored behind the requests for their rows and without looking
            // first: a look asked for ahead of the rows was a trip to memory of its own per token block, and behind
            // them it still costs more than the stores it saves (64-row stage under rotation, 32k x 128k: 5.1 ms
            // with the look ahead of the rows, 5.0 behind them, 4.6 with blind stores, 4.2 without statistics)
            if (kx->access_flags) {
                uint8_t *frow = kx->access_flags + (int64_t)b * kx->flags_stride_b + (int64_t)kvh * kx->flags_stride_h;
#pragma unroll
                for (int tb = 0; tb < NB; tb++)
                    if (late_mark[tb] >= 0) mark_flag<false>(frow + late_mark[tb]);
            }
        }
        uint4 *my_tile = &s_rows[DMA ? (threadIdx.x >> 6) * 32 * PPR : 0];
        const uint32_t tile_addr = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)my_tile);  // LDS address: low 32 bits
        const uint4 *rd_tile = my_tile;   // where this round's fragments are read from
        uint32_t dst_addr = tile_addr;
        if constexpr (SHAREABLE) {
            if (share_now) {
                rd_tile = &s_rows[4 * 32 * PPR];
                dst_addr = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)rd_tile);
            }
        }
        if constexpr (DMA) {
            if (fresh[0]) {
                // instruction i fetches rows 4i .. 4i+3: lane l takes slot l % 16 of row 4i + l / 16, which holds the
                // row's piece (l % 16) ^ (row % 16); the row's offset is held by the lane of that row.  Rows that are
                // not sampled afresh are left as they are: a lane only ever looks at the column of its own row.
                // (offsets are multiples of eight elements: they travel between lanes as 32-bit piece numbers)
                // (OFF32: a lane without a fresh sample sends the first row of its kv head: any row will do, its
                // products are not looked at, and no load needs a select or sits in a branch)
                const int my_piece0 = OFF32 ? (pieces[0] < 0 ? (int)piece_h : pieces[0]) : pieces[0];
                // all cross-lane reads first, then the loads back to back: the load statements keep their order, so a
                // cross-lane read between two of them would be waited for there
                constexpr int NI = 32 * PPR / 64;
                int o[NI];
#pragma unroll
                for (int i = 0; i < NI; i++) {
                    const int r = i * (64 / PPR) + lane / PPR;  // tile row; SPLIT: row side * 16 + c is the sample of lane 2 c + side
                    o[i] = __shfl(my_piece0, SPLIT ? (((r & 15) << 1) | (r >> 4)) : r);
                }
                if constexpr (OFF32) {
                    const uint16_t *kb = reinterpret_cast<const uint16_t *>(p.kv.k) + (int64_t)b * p.kv.k_stride_b;
                    uint32_t so[NI];
#pragma unroll
                    for (int i = 0; i < NI; i++) {
                        const int r = i * (64 / PPR) + lane / PPR;
                        const int q = (lane % PPR) ^ (r & (PPR - 1));
                        so[i] = (uint32_t)(o[i] + q) << 4;
                    }
                    if (share_now) __syncthreads();  // everyone is done with the shared tile of the search before
#pragma unroll
                    for (int i = 0; i < NI; i++)
                        if (!share_now || (i & 3) == wv) load_to_lds16_at_s(kb, so[i], dst_addr + i * 1024);
                } else {
                    // Rows that are not sampled afresh come from a row of zeros, so that no load sits in a branch.
                    const uint4 *src[NI];
#pragma unroll
                    for (int i = 0; i < NI; i++) {
                        const int r = i * (64 / PPR) + lane / PPR;
                        const int q = (lane % PPR) ^ (r & (PPR - 1));
                        src[i] = o[i] >= 0 ? reinterpret_cast<const uint4 *>(p.kv.k) + ((int64_t)o[i] + q)
                                           : reinterpret_cast<const uint4 *>(g_scan_zero_row) + (lane % PPR);
                    }
                    if (share_now) __syncthreads();
#pragma unroll
                    for (int i = 0; i < NI; i++)
                        if (!share_now || (i & 3) == wv) load_to_lds16_at(src[i], dst_addr + i * 1024);
                }
                wait_vmcnt<0>();
                if (share_now) __syncthreads();  // every wave's quarter has landed
            }
            // the access flags of the round's samples are set once its rows have landed: vector-memory operations
            // complete in order, so a store requested ahead of the rows would have to be acknowledged before the
            // wait for them ends; from here the stores have the products of the round to complete behind
            // (a search that has narrowed to a few tokens keeps sampling the same page: its flag is stored once)
            if (flag_row) {
#pragma unroll
                for (int tb = 0; tb < NB; tb++)
                    if (mark[tb] >= 0 && mark[tb] != last_mark[tb]) {
                        flag_row[mark[tb]] = 1;
                        last_mark[tb] = mark[tb];
                    }
            }
        }
        bool any_fresh = false;  // uniform over the wave, and the LDS path's workgroups are one wave
#pragma unroll
        for (int tb = 0; tb < NB; tb++) any_fresh = any_fresh || fresh[tb];
        if (VIA_LDS && any_fresh) {
            __syncthreads();
            // coalesced fetch: PPR lanes cover one row; piece q of row r is parked at slot q ^ swz(r).  Eight loads
            // are requested before the first is used, and none sits in a branch (rows that are not sampled come
            // from a row of zeros): one trip to memory per eight instead of one per load.
            constexpr int NLOAD = NROWS / RPI;
            constexpr int LB = NLOAD < 8 ? NLOAD : 8;
#pragma unroll
            for (int i0 = 0; i0 < NLOAD; i0 += LB) {
                uint4 v[LB];
#pragma unroll
                for (int j = 0; j < LB; j++) {
                    const int r = (i0 + j) * RPI + lrow;
                    const int64_t off = s_off[r];
                    const int q = lpos ^ ((r / SWZ_DIV) & SWZ);
                    const void *rbase = off != NO_ROW ? p.kv.k : static_cast<const void *>(g_scan_zero_row);
                    v[j] = load_kv_piece<KV8>(rbase, (off != NO_ROW ? off : 0) + q * 8);
                }
#pragma unroll
                for (int j = 0; j < LB; j++) {
                    const int r = (i0 + j) * RPI + lrow;
                    if (!PRESCALED) {
                        v[j].x = scale_pack(v[j].x, p.c_k);
                        v[j].y = scale_pack(v[j].y, p.c_k);
                        v[j].z = scale_pack(v[j].z, p.c_k);
                        v[j].w = scale_pack(v[j].w, p.c_k);
                    }
                    s_rows[r * PPR + lpos] = v[j];
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int tb = 0; tb < NB; tb++) {
            float v = -INFINITY;
            if constexpr (M16) {
                if (fresh[tb]) {
                    // D[row, token]: lane (token c = l % 16 of a half, row group g = l / 16) holds rows 4g .. 4g + 3
                    typedef __attribute__((ext_vector_type(4))) float f32x4;
                    const int c = lane & 15, kb = lane >> 4;
                    float vh[2];
#pragma unroll
                    for (int half = 0; half < 2; half++) {
                        f32x4 acc4 = {0.0f, 0.0f, 0.0f, 0.0f};
                        const int t = half * 16 + c;
                        BFrag kf16[KS / 2];
#pragma unroll
                        for (int j = 0; j < KS / 2; j++) {
                            const int piece = (kb & 1) * (PPR / 2) + 2 * j + (kb >> 1);
                            kf16[j].q = rd_tile[t * PPR + (piece ^ (t & (PPR - 1)))];
                            if constexpr (SPLIT) {
                                // rows as stored: the right-hand half is rotated to position 1 (the partner piece is
                                // the same columns of the row's other half), then every row is scaled
                                if (half == 1 || !left_plain) {
                                    const uint4 oth = rd_tile[t * PPR + ((piece ^ (PPR / 2)) ^ (t & (PPR - 1)))];
                                    uint4 cc = cos1[j], sn = sin1[j];
                                    if (half == 0) {  // a table whose first row is not (1, 0): rotate to position 0 as well
                                        const int64_t r0 = p.rope.row(0);
                                        const int colx = (2 * j + (kb >> 1)) * 8;
                                        cc = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.cos) + r0 + colx);
                                        sn = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.sin) + r0 + colx);
                                    }
                                    kf16[j].q = rope_piece(kf16[j].q, oth, cc, sn, (kb & 1) == 0);
                                }
#pragma unroll
                                for (int e = 0; e < 4; e++) kf16[j].u[e] = scale_pack(kf16[j].u[e], p.c_k);
                            }
                        }
#pragma unroll
                        for (int j = 0; j < KS / 2; j++)
                            acc4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf16[j].v, kf16[j].v, acc4, 0, 0, 0);
                        float m = -INFINITY;
                        if (fast_rows == 16) {
                            m = fmaxf(fmaxf(acc4[0], acc4[1]), fmaxf(acc4[2], acc4[3]));
                        } else {
#pragma unroll
                            for (int r = 0; r < 4; r++) {
                                const int row = kb * 4 + r;
                                const bool ok = (row < p.nrows) && ((rowmask >> row) & 1ull);
                                m = fmaxf(m, ok ? acc4[r] : -INFINITY);
                            }
                        }
                        vh[half] = m;
                    }
                    // fold the four row groups: after the exchange over lane ^ 16 a lane holds its own token
                    // (l % 32) over two groups, after lane ^ 32 over all four
                    const bool upper = (lane & 16) != 0;
                    const float keep = upper ? vh[1] : vh[0], send = upper ? vh[0] : vh[1];
                    v = fmaxf(keep, __shfl_xor(send, 16));
                    v = fmaxf(v, __shfl_xor(v, 32));
                    v = round_bf16(v);
                    if constexpr (SPLIT) v = __shfl(v, ((n & 1) << 4) | (n >> 1));  // from the lane of this lane's tile row
                    if constexpr (OFF32) {
                        if (pieces[tb] < 0) v = 0.0f;
                    }
                }
            } else if (fresh[tb]) {
            f32x16 acc[MB];
#pragma unroll
            for (int mb = 0; mb < MB; mb++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[mb][i] = 0.0f;
            const int r = tb * 32 + n;
            const int sw = (r / SWZ_DIV) & SWZ;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                BFrag kf;
                if constexpr (VIA_LDS) {
                    kf.q = s_rows[r * PPR + ((hh * (PPR / 2) + ks) ^ sw)];
                } else if constexpr (DMA) {
                    kf.q = rd_tile[n * PPR + ((hh * (PPR / 2) + ks) ^ (n & (PPR - 1)))];
                    if constexpr (!PRESCALED) {  // the tile holds the rows as stored
#pragma unroll
                        for (int e = 0; e < 4; e++) kf.u[e] = scale_pack(kf.u[e], p.c_k);
                    }
                } else if constexpr (PRESCALED) {
                    kf.q = raw[tb][ks];
                } else if constexpr (ROPE) {
                    const uint4 own = raw[tb][ks];
                    const uint4 oth = make_uint4(__shfl_xor(own.x, 32), __shfl_xor(own.y, 32), __shfl_xor(own.z, 32),
                                                 __shfl_xor(own.w, 32));
                    const uint4 rot = rope_piece(own, oth, rcos[tb][ks], rsin[tb][ks], hh == 0);
                    kf.u[0] = scale_pack(rot.x, p.c_k);
                    kf.u[1] = scale_pack(rot.y, p.c_k);
                    kf.u[2] = scale_pack(rot.z, p.c_k);
                    kf.u[3] = scale_pack(rot.w, p.c_k);
                } else {
                    kf.u[0] = scale_pack(raw[tb][ks].x, p.c_k);
                    kf.u[1] = scale_pack(raw[tb][ks].y, p.c_k);
                    kf.u[2] = scale_pack(raw[tb][ks].z, p.c_k);
                    kf.u[3] = scale_pack(raw[tb][ks].w, p.c_k);
                }
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
                    acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qf[mb][ks].v, kf.v, acc[mb], 0, 0, 0);
            }
            if constexpr (QINL) {
                v = hh == 0 ? acc[0][0] : -INFINITY;  // the one valid row is row 0: element 0 of the lower half-wave
            } else if (fast_rows == 16) {
#pragma unroll
                for (int i = 0; i < 8; i++) v = fmaxf(v, acc[0][i]);
            } else if (fast_rows == 32) {
#pragma unroll
                for (int i = 0; i < 16; i++) v = fmaxf(v, acc[0][i]);
            } else if (fast_rows == 64) {
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
#pragma unroll
                    for (int i = 0; i < 16; i++) v = fmaxf(v, acc[mb][i]);
            } else {
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
#pragma unroll
                    for (int i = 0; i < 16; i++) v = fmaxf(v, ((vm[mb] >> i) & 1u) ? acc[mb][i] : -INFINITY);
            }
            v = fmaxf(v, __shfl_xor(v, 32));
            v = round_bf16(v);
            if constexpr (OFF32) {
                if (pieces[tb] < 0) v = 0.0f;  // a token without a row scores as a row of zeros
            }
            }
            if (reuse[tb]) v = rscore[tb];
            if (active[tb]) {
                ptok[tb] = tok[tb];
                pscore[tb] = v;
            }
            const float other = __shfl_xor(v, 1);
            const float sL = side ? other : v;
            const float sR = side ? v : other;
            if (active[tb]) {
                const bool win = sL > sR;
                if (win) cr[tb] = ctr[tb]; else cl[tb] = ctr[tb];
                score[tb] = fmaxf(score[tb], win ? sL : sR);
            }
        }
        first = false;
    }
    store_out();
    }

}

// Q^ rows of every scan program: strided mean of stride_q query rows in f32, rounded to bf16, scaled
// by c_q, rounded again (attention_extend.py:607-734,924-931).  One thread makes 8 elements.
__global__ void qhat_kernel(MaskParams p, int hid, uint16_t *out) {
    const int per_row = hid / 8;
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long total = (long long)p.B * p.BS * p.HEAD * p.nrows * per_row;
    if (p.reduce_heads == 1) {
        // the scan folds the maximum over heads into scores [B, BS, 1, n]: start it at -inf here, in the launch that
        // precedes the scan on the stream anyway
        const long long nscores = (long long)p.B * p.BS * p.n;
        for (long long i = gid; i < nscores; i += (long long)gridDim.x * blockDim.x) p.scores[i] = -INFINITY;
    }
    if (gid >= total) return;
    const int piece = (int)(gid % per_row);
    long long r = gid / per_row;
    const int j = (int)(r % p.nrows);
    r /= p.nrows;
    const int h = (int)(r % p.HEAD);
    r /= p.HEAD;
    const int s = (int)(r % p.BS);
    const int b = (int)(r / p.BS);
    const long long qb = (long long)(p.BDST - 1) - (long long)(p.BS - 1) * p.scan_stride + (long long)s * p.scan_stride;
    const long long it = qb * p.BQ + (long long)j * p.stride_q;
    uint4 o = make_uint4(0, 0, 0, 0);
    if (it >= 0 && it < p.TDST) {
        const uint16_t *qbase = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
        float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        int cnt = 0;
        const bool rope = p.rope.cos != nullptr;
        const int ppiece = (piece + per_row / 2) % per_row;  // the piece holding the partner elements
        uint4 rc = make_uint4(0, 0, 0, 0), rs = rc;
        if (rope) {
            // every strided row is rotated to the position derived from the base row (attention_extend.py:626-690)
            const int64_t tr = p.rope.row(rope_qpos(p.rope, p.pos[(int64_t)b * p.pos_sb + it * p.pos_st], p.n, p.sw_eff)) +
                               (piece % (per_row / 2)) * 8;
            rc = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.cos) + tr);
            rs = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p.rope.sin) + tr);
        }
        for (int oo = 0; oo < p.stride_q; oo++) {
            if (it + oo < p.TDST) {
                uint4 raw = *reinterpret_cast<const uint4 *>(qbase + (it + oo) * p.q_st + piece * 8);
                if (rope) {
                    const uint4 oth = *reinterpret_cast<const uint4 *>(qbase + (it + oo) * p.q_st + ppiece * 8);
                    raw = rope_piece(raw, oth, rc, rs, piece < per_row / 2);
                }
                const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    sum[2 * e] += __uint_as_float(w[e] << 16);
                    sum[2 * e + 1] += __uint_as_float(w[e] & 0xffff0000u);
                }
                cnt++;
            }
        }
        const float den = (float)cnt + 1e-12f;
        uint32_t ow[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float m0 = round_bf16(__fdiv_rn(sum[2 * e], den));
            const float m1 = round_bf16(__fdiv_rn(sum[2 * e + 1], den));
            ow[e] = cvt_pk_bf16(m0 * p.c_q, m1 * p.c_q);
        }
        o = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
    // stored in the order the scan kernel's lanes fetch them: per (b, s, h) the 16-byte piece of k-step ks, row half hh
    // and row j sits at ((ks * 2 + hh) * nrows + j), so one load instruction of a wave reads consecutive pieces
    {
        const int half_pieces = per_row / 2;
        const int hh = piece / half_pieces, ks = piece % half_pieces;
        const long long base = (gid / per_row / p.nrows) * (long long)p.nrows * hid;
        *reinterpret_cast<uint4 *>(out + base + ((long long)(ks * 2 + hh) * p.nrows + j) * 8) = o;
    }
}

static int g_mask_via_lds = -1;  // -1: decide per shape; 0 / 1: forced through HIPATTN_MASK_VIA_LDS (tuning aid)

template <int HID>
static int launch_mfma_hid(const MaskParams &p0, int rows_eff, int flags, hipStream_t st) {
    const int prescaled = flags & 1;          // keys scaled (and rotated) ahead of the scan
    const bool q_ready = (flags & 2) != 0;    // the workspace holds this stage's query rows already
    // key rows may lie 32 GiB or more beyond kv.k: the coalesced variants, whose lanes exchange the rows' places as
    // 31-bit numbers of 16-byte pieces, are not used.  Worked out here for a dense tensor; for a paged pool the
    // caller vouches for its size with bit 2.
    const bool far_rows = kv_rows_beyond_32gib(p0.kv, p0.B, HID, p0.kx.kv8 ? 1 : 2, p0.rope.k_side_delta, (flags & 4) != 0);
    MaskParams p = p0;
    const int BC = p.block_chunk;
    const bool two = rows_eff > 32;
    // two token blocks (32 chunks) per wave when programs are plentiful, else one block per wave
    const long long programs = (long long)p.B * p.HEAD * p.BS * p.ngroups;
    const bool wide = (BC >= 32) && (programs >= 16384);
    static int env_nb = -1;
    if (env_nb < 0) {
        const char *e = getenv("HIPATTN_MASK_NB");
        env_nb = e ? atoi(e) : 0;
    }
    // HIPATTN_MASK_DMA: wide launches on prescaled keys fetch their rows coalesced, straight into LDS (default);
    // 0 = each lane loads its own half row, as the other launches do (read on every call: tests switch it)
    // (2 = on every launch the variant can serve, however small: testing)
    const char *e_dma = getenv("HIPATTN_MASK_DMA");
    const int dma_mode = e_dma ? atoi(e_dma) : 1;
    // (keys rotated ahead under the relative / infllm rules are prescaled keys like any other: the kernel takes a
    // right-hand sample from the second copy)
    const bool dma = dma_mode != 0 && !far_rows && (wide || dma_mode == 2) && prescaled && p.rope.k_side_delta >= 0 && !p.kx.kv8 &&
                     !p.kx.cached && HID <= 128 && env_nb != 2 && !two;  // (64-row programs: 204 registers, 6.7 against 3.9 ms)
    // small chunks on wide launches: every token scored once per GQA group, searches replayed on the scores
    const bool dense = prescaled && !far_rows && p.rope.cos == nullptr && mask_stage_dense_applies(p, HID, rows_eff);
    // Launches with a single query token fetch their rows that way too, from keys as stored (HIPATTN_MASK_DMA_INLINE=0:
    // never; 2: only from 16384 waves on, e.g. a batch of sequences).  1M-key decode: 63 / 11 / 11 us against 66 / 12 /
    // 12 us for the three stages, 16 sequences: 582 against 622 us per refresh.
    const char *e_di = getenv("HIPATTN_MASK_DMA_INLINE");
    const int di = e_di ? atoi(e_di) : 1;
    const long long waves_one_block = (long long)p.B * p.HEAD * p.BS * p.ngroups * (BC / 16);
    const bool dma_inline = dma_mode != 0 && !far_rows && di != 0 && !dense && p.TDST == 1 && !two &&
                            p.rope.cos == nullptr && !p.kx.kv8 && !p.kx.cached && HID <= 128 && env_nb != 2 &&
                            (di == 1 || waves_one_block >= 16384);
    const int nb0 = (dma || dma_inline) ? 1 : (env_nb == 2 && BC >= 32) ? 2 : (env_nb == 1 ? 1 : (wide ? 2 : 1));
    // LDS path: one wave per workgroup (it uses workgroup barriers); direct path: up to 4 heads per workgroup
    // (measured: sharing pays with one query-row block per program, not with two)
    if (g_mask_via_lds < 0) {
        const char *e = getenv("HIPATTN_MASK_VIA_LDS");
        g_mask_via_lds = e ? (e[0] == '1' ? 1 : 0) : 2;
    }
    // The extended build (statistics, offload cache) exists for the direct path and for the one-block LDS path.
    // It is also used for wide single-row-block launches without extras: measured 10-15% faster there than the
    // plain build of the same source (the compiler schedules its row loads earlier), and its extra branches are
    // never taken.
    const bool rope = p.rope.cos != nullptr && !prescaled;  // rotate every sample in the kernel
    const bool two_sided = p.rope.cos != nullptr && prescaled;
    const int nb = rope ? 1 : nb0;
    const int nsub = (BC / 16) / nb;
    // narrow launches: chunks of up to 32 tokens keep a search inside a few KB that the heads of a group share
    // through L1, and direct loads win (decode at 1M keys: 31 / 22 us against 38 / 28 us for the 32- and 8-token
    // stages); wide chunks scatter the samples of a search, and rows fetched coalesced through LDS win (124 against
    // 182 us for the 256-token stage)
    bool via_lds = (dma || dma_inline) ? false : g_mask_via_lds == 2 ? (!wide && p.chunk > 32) : (g_mask_via_lds == 1);
    if (((p.kx.extended() || two_sided) && nb == 2) || rope) via_lds = false;
    const bool ext = rope || two_sided || p.kx.extended() || (wide && !two && !via_lds);
    static int env_hpw2 = -1;
    if (env_hpw2 < 0) {
        const char *e = getenv("HIPATTN_MASK_HPW_TWO");
        env_hpw2 = e ? atoi(e) : 1;
    }
    const int hpw_two = env_hpw2 < p.G ? env_hpw2 : p.G;
    const int hpw = via_lds ? 1 : two ? hpw_two : (p.G < 4 ? p.G : 4);
    const int hblocks = (p.G + hpw - 1) / hpw;
    // wide launches with 64 query rows: a wave keeps its Q^ fragments for several chunk groups (they are 16 KB
    // against the 40 KB of key rows that 32 searches over 8 tokens read; cfg-2-like prefill: 4.9 ms for one group
    // per wave, 4.3 / 4.0 / 3.9 ms for 2 / 4 / 8)
    static int env_reps = -1;
    if (env_reps < 0) {
        const char *e = getenv("HIPATTN_MASK_GROUP_REPS");
        env_reps = e ? atoi(e) : 0;
    }
    p.group_reps = (!two && !dma) ? 1 : env_reps > 0 ? env_reps : dma ? 16 : (wide ? 8 : 1);
    if (p.group_reps > p.ngroups) p.group_reps = p.ngroups;
    // HIPATTN_MASK_SHARE_FIRST=0: every head fetches the rows of a search's first round itself
    const char *e_sf = getenv("HIPATTN_MASK_SHARE_FIRST");
    p.share_first = (dma && hpw == 4 && p.G % 4 == 0 && p.hg == 1 && (e_sf ? atoi(e_sf) : 1) != 0) ? 1 : 0;
    const int groups_outer = (p.ngroups + p.group_reps - 1) / p.group_reps;
    p.total = (long long)p.B * p.kv.HKV * hblocks * p.BS * groups_outer * nsub;
    if (p.total >= 0x7fffffffLL) {
        set_error("mask stage: grid too large");
        return HIPATTN_E_UNSUPPORTED;
    }
    // Where every program row is the mean of exactly one query row and is not rotated (the dense kernel with
    // stride_q == 1; the narrow sampling kernels with a single query token), the kernels scale the rows themselves: the preparation launch
    // (a pass over all of q) shrinks to the fill of the head-reduced scores, and to nothing when the caller has
    // initialised those (reduce_heads == 2).
    const bool q_inline = !rope && !two_sided && ((dense && p.stride_q == 1) || (!dense && p.TDST == 1 && nb == 1 && !p.kx.kv8));
    if (q_inline || q_ready) {
        mask_stage_fill_scores(p, st);
    } else {
        const long long work = (long long)p.B * p.BS * p.HEAD * p.nrows * (HID / 8);
        const long long blocks = (work + 255) / 256;
        hipLaunchKernelGGL(qhat_kernel, dim3((unsigned)blocks), dim3(256), 0, st, p, HID, const_cast<uint16_t *>(p.qhat));
    }
    if (dense) {
        const int rc = mask_stage_dense_launch(p, HID, rows_eff, q_inline, st);
        if (rc != HIPATTN_E_UNSUPPORTED || q_inline) return rc;
    }
    dim3 grid((unsigned)p.total), block(64 * hpw);
    const MaskParamsBase &pb = p;  // the plain kernels take the block without the extras
#define MS_LAUNCH(MBv, NBv, PSv, VLv)                                                                                 \
    do {                                                                                                              \
        constexpr bool EXT_BUILT = !(VLv) || (NBv) == 1;                                                              \
        if constexpr (!(PSv) && EXT_BUILT) {                                                                          \
            if (p.kx.kv8) {                                                                                           \
                hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, MBv, NBv, false, VLv, true, 0, true>), grid, block, 0, st, \
                                   p, nsub, hpw);                                                                     \
                break;                                                                                                \
            }                                                                                                         \
        }                                                                                                             \
        if constexpr ((PSv) && EXT_BUILT) {                                                                           \
            if (two_sided) {                                                                                          \
                hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, MBv, NBv, true, VLv, true, 2>), grid, block, 0, st, p, \
                                   nsub, hpw);                                                                        \
                break;                                                                                                \
            }                                                                                                         \
        }                                                                                                             \
        if (ext && EXT_BUILT)                                                                                         \
            hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, MBv, NBv, PSv, VLv, EXT_BUILT>), grid, block, 0, st, p, nsub, \
                               hpw);                                                                                  \
        else                                                                                                          \
            hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, MBv, NBv, PSv, VLv, false>), grid, block, 0, st, pb, nsub, hpw); \
    } while (0)
#define MS_PICK(MBv, NBv)                                                \
    do {                                                                  \
        if (prescaled) { if (via_lds) MS_LAUNCH(MBv, NBv, true, true); else MS_LAUNCH(MBv, NBv, true, false); } \
        else { if (via_lds) MS_LAUNCH(MBv, NBv, false, true); else MS_LAUNCH(MBv, NBv, false, false); }        \
    } while (0)
    if (p.kx.kv8 && prescaled) {
        set_error("mask stage: prescaled keys cannot be combined with fp8 key storage");
        return HIPATTN_E_ARG;
    }
    // a dense key tensor whose batch items span less than 4 GB: row addresses as 32-bit offsets
    const long long item_bytes = 2LL * ((p.kv.tsrc - 1) * p.kv.k_stride_t + (long long)(p.kv.HKV - 1) * p.kv.k_stride_h + HID +
                                        (p.rope.k_side_delta > 0 ? p.rope.k_side_delta : 0));
    const bool off32 = !p.kv.paged && p.kv.k_stride_t >= 0 && p.kv.k_stride_h >= 0 && p.kv.k_stride_t % 8 == 0 &&
                       p.kv.k_stride_h % 8 == 0 && p.kv.k_stride_b % 8 == 0 && item_bytes < (1LL << 32) &&
                       p.kv.tsrc < (1LL << 24) && (p.kv.k_stride_t >> 3) < (1LL << 24);
    if (dma && !q_inline) {
        if constexpr (HID <= 128) {
            // Programs of up to 16 query rows take the 16x16x32 form of the products (HIPATTN_MASK_M16=0: the 32x32x16
            // form).  Same bits, half the matrix cycles, 92 registers instead of 128, and the same time to within 2%
            // (cfg-2-like prefill: 2.07 / 2.65 against 2.07 / 2.66 ms): these launches are held by the vector-memory
            // path of a CU, not by products, registers or waves.
            const char *e_m16 = getenv("HIPATTN_MASK_M16");
            const bool m16 = rows_eff <= 16 && p.nrows <= 16 && (e_m16 ? atoi(e_m16) : 1) != 0;
            if constexpr (HID % 32 == 0) {
                if (m16) {
                    if (off32) hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, true, false, true, 7>), grid, block, 0, st, p, nsub, hpw);
                    else hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, true, false, true, 8>), grid, block, 0, st, p, nsub, hpw);
                    HIPATTN_CHECK_HIP(hipGetLastError());
                    return 0;
                }
            }
            if (off32) hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, true, false, true, 5>), grid, block, 0, st, p, nsub, hpw);
            else hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, true, false, true, 4>), grid, block, 0, st, p, nsub, hpw);
            HIPATTN_CHECK_HIP(hipGetLastError());
            return 0;
        }
    }
    if (dma_inline) {
        if constexpr (HID <= 128) {
            if (off32) {
                if (prescaled) hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, true, false, true, 9>), grid, block, 0, st, p, nsub, hpw);
                else hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, false, false, true, 9>), grid, block, 0, st, p, nsub, hpw);
            } else if (prescaled) {
                hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, true, false, true, 6>), grid, block, 0, st, p, nsub, hpw);
            } else {
                hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, false, false, true, 6>), grid, block, 0, st, p, nsub, hpw);
            }
            HIPATTN_CHECK_HIP(hipGetLastError());
            return 0;
        }
    }
    if (q_inline) {  // narrow launch, one token block per wave, query rows scaled in the kernel
#define MS_INLINE(MBv, PSv, VLv)                                                                                       \
    do {                                                                                                              \
        if (ext) hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, MBv, 1, PSv, VLv, true, 3>), grid, block, 0, st, p, nsub, hpw); \
        else hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, MBv, 1, PSv, VLv, false, 3>), grid, block, 0, st, pb, nsub, hpw);   \
    } while (0)
#define MS_INLINE_PICK(MBv)                                                                          \
    do {                                                                                             \
        if (prescaled) { if (via_lds) MS_INLINE(MBv, true, true); else MS_INLINE(MBv, true, false); } \
        else { if (via_lds) MS_INLINE(MBv, false, true); else MS_INLINE(MBv, false, false); }         \
    } while (0)
        if (two) MS_INLINE_PICK(2); else MS_INLINE_PICK(1);
#undef MS_INLINE_PICK
#undef MS_INLINE
        HIPATTN_CHECK_HIP(hipGetLastError());
        return 0;
    }
    // rotation on load under the relative rule, programs of up to 16 rows (decode above all): coalesced rows with the
    // tile ordered by sample side, so that only the right-hand half is rotated (HIPATTN_MASK_DMA=0: the variant below)
    if constexpr (HID <= 128 && HID % 32 == 0) {
        // (rows_eff: the valid rows of a program are its first ones; a stage of 64-row programs under a single query
        // token has one)
        if (rope && p.rope.backend == HIPATTN_EXTEND_RELATIVE && dma_mode != 0 && !far_rows && !two && rows_eff <= 16 &&
            !p.kx.kv8 && !p.kx.cached && nb == 1) {
            if (off32) hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, false, false, true, 10>), grid, block, 0, st, p, nsub, hpw);
            else hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, false, false, true, 11>), grid, block, 0, st, p, nsub, hpw);
            HIPATTN_CHECK_HIP(hipGetLastError());
            return 0;
        }
    }
    if (rope && p.kx.kv8) {
        if (two) hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 2, 1, false, false, true, 1, true>), grid, block, 0, st, p, nsub, hpw);
        else hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, false, false, true, 1, true>), grid, block, 0, st, p, nsub, hpw);
    } else if (rope) {
        if (two) hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 2, 1, false, false, true, 1>), grid, block, 0, st, p, nsub, hpw);
        else hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, 1, 1, false, false, true, 1>), grid, block, 0, st, p, nsub, hpw);
    } else if (two) { if (nb == 2) MS_PICK(2, 2); else MS_PICK(2, 1); }
    else { if (nb == 2) MS_PICK(1, 2); else MS_PICK(1, 1); }
#undef MS_PICK
#undef MS_LAUNCH
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

int mask_stage_mfma_launch(const MaskParams &p, int HID, int rows_eff, int prescaled, hipStream_t st) {
    switch (HID) {
        case 32: return launch_mfma_hid<32>(p, rows_eff, prescaled, st);
        case 64: return launch_mfma_hid<64>(p, rows_eff, prescaled, st);
        case 128: return launch_mfma_hid<128>(p, rows_eff, prescaled, st);
        case 256: return launch_mfma_hid<256>(p, rows_eff, prescaled, st);
    }
    set_error("mask stage: head dim %d is not built for bf16", HID);
    return HIPATTN_E_UNSUPPORTED;
}

// K^ = bf16(K * c_k) for a whole key tensor, 8 elements per thread
__global__ void prescale_k_kernel(const uint16_t *in, uint16_t *out, long long rows, int hid, int64_t s0, int64_t s1,
                                  int64_t s2, int d1, int d2, float c_k) {
    // rows are indexed (i0, i1, i2) with extents (., d1, d2) and input strides (s0, s1, s2); output is contiguous
    const int per_row = hid / 8;
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= rows * per_row) return;
    const long long r = gid / per_row;
    const int piece = (int)(gid % per_row);
    const long long i2 = r % d2, i1 = (r / d2) % d1, i0 = r / ((long long)d1 * d2);
    const uint4 raw = *reinterpret_cast<const uint4 *>(in + i0 * s0 + i1 * s1 + i2 * s2 + piece * 8);
    uint4 o;
    o.x = scale_pack(raw.x, c_k);
    o.y = scale_pack(raw.y, c_k);
    o.z = scale_pack(raw.z, c_k);
    o.w = scale_pack(raw.w, c_k);
    *reinterpret_cast<uint4 *>(out + r * hid + piece * 8) = o;
}

// the same after rotating every row to one fixed position (table rows cos_row / sin_row), or, with chunk > 0, row
// (., t, .) to position (t - first) / chunk, clamped into the tables: the place of token t's chunk in the list of a
// scan's first stage (chunk c starts at first + c * chunk)
__global__ void prescale_k_rope_kernel(const uint16_t *in, uint16_t *out, long long rows, int hid, int64_t s0, int64_t s1,
                                       int64_t s2, int d1, int d2, float c_k, const uint16_t *cos_row,
                                       const uint16_t *sin_row, int64_t table_stride, int64_t table_len, int first, int chunk) {
    const int per_row = hid / 8;
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= rows * per_row) return;
    const long long r = gid / per_row;
    const int piece = (int)(gid % per_row);
    const int ppiece = (piece + per_row / 2) % per_row;
    const long long i2 = r % d2, i1 = (r / d2) % d1, i0 = r / ((long long)d1 * d2);
    const uint16_t *row = in + i0 * s0 + i1 * s1 + i2 * s2;
    const uint4 raw = *reinterpret_cast<const uint4 *>(row + piece * 8);
    const uint4 oth = *reinterpret_cast<const uint4 *>(row + ppiece * 8);
    if (chunk > 0) {
        long long pos = i1 >= first ? (i1 - first) / chunk : 0;
        pos = pos < table_len ? pos : table_len - 1;
        cos_row += pos * table_stride;
        sin_row += pos * table_stride;
    }
    const uint4 c = *reinterpret_cast<const uint4 *>(cos_row + (piece % (per_row / 2)) * 8);
    const uint4 sn = *reinterpret_cast<const uint4 *>(sin_row + (piece % (per_row / 2)) * 8);
    const uint4 rot = rope_piece(raw, oth, c, sn, piece < per_row / 2);
    uint4 o;
    o.x = scale_pack(rot.x, c_k);
    o.y = scale_pack(rot.y, c_k);
    o.z = scale_pack(rot.z, c_k);
    o.w = scale_pack(rot.w, c_k);
    *reinterpret_cast<uint4 *>(out + r * hid + piece * 8) = o;
}

}  // namespace hipattn

using namespace hipattn;

extern "C" int hipattn_prescale_k_rope(const void *k, int64_t stride0, int64_t stride1, int64_t stride2, int64_t n0,
                                       int32_t n1, int32_t n2, int32_t HID, const void *cos_row, const void *sin_row,
                                       void *out, void *stream) {
    HIPATTN_CHECK_ARG(k && out && cos_row && sin_row, HIPATTN_E_ARG, "prescale: null pointer");
    HIPATTN_CHECK_ARG(n0 > 0 && n1 > 0 && n2 > 0 && HID > 0 && HID % 32 == 0, HIPATTN_E_ARG, "prescale: bad sizes");
    HIPATTN_CHECK_ARG(aligned16(k) && aligned16(out) && aligned16(cos_row) && aligned16(sin_row) && stride0 % 8 == 0 &&
                          stride1 % 8 == 0 && stride2 % 8 == 0,
                      HIPATTN_E_ALIGN, "prescale: pointers and strides must be 16-byte aligned");
    float c_q, c_k;
    scale_constants(HID, HIPATTN_BF16, &c_q, &c_k);
    const long long rows = (long long)n0 * n1 * n2;
    const long long work = rows * (HID / 8);
    const int threads = 256;
    const long long blocks = (work + threads - 1) / threads;
    HIPATTN_CHECK_ARG(blocks < 0x7fffffffLL, HIPATTN_E_UNSUPPORTED, "prescale: tensor too large");
    hipLaunchKernelGGL(prescale_k_rope_kernel, dim3((unsigned)blocks), dim3(threads), 0, (hipStream_t)stream,
                       reinterpret_cast<const uint16_t *>(k), reinterpret_cast<uint16_t *>(out), rows, HID, stride0,
                       stride1, stride2, n1, n2, c_k, reinterpret_cast<const uint16_t *>(cos_row),
                       reinterpret_cast<const uint16_t *>(sin_row), (int64_t)0, (int64_t)1, 0, 0);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

extern "C" int hipattn_prescale_k_rope_chunks(const void *k, int64_t stride_b, int64_t stride_t, int64_t stride_h, int64_t B,
                                              int32_t T, int32_t HKV, int32_t HID, const void *cos, const void *sin,
                                              int64_t table_stride, int64_t table_len, int32_t first, int32_t chunk,
                                              void *out, void *stream) {
    HIPATTN_CHECK_ARG(k && out && cos && sin, HIPATTN_E_ARG, "prescale: null pointer");
    HIPATTN_CHECK_ARG(B > 0 && T > 0 && HKV > 0 && HID > 0 && HID % 32 == 0, HIPATTN_E_ARG, "prescale: bad sizes");
    HIPATTN_CHECK_ARG(chunk > 0 && first >= 0 && table_len > 0 && table_stride >= HID / 2, HIPATTN_E_ARG,
                      "prescale: bad chunk list or table description");
    HIPATTN_CHECK_ARG(aligned16(k) && aligned16(out) && aligned16(cos) && aligned16(sin) && stride_b % 8 == 0 &&
                          stride_t % 8 == 0 && stride_h % 8 == 0 && table_stride % 8 == 0,
                      HIPATTN_E_ALIGN, "prescale: pointers, strides and table rows must be 16-byte aligned");
    float c_q, c_k;
    scale_constants(HID, HIPATTN_BF16, &c_q, &c_k);
    const long long rows = (long long)B * T * HKV;
    const long long work = rows * (HID / 8);
    const int threads = 256;
    const long long blocks = (work + threads - 1) / threads;
    HIPATTN_CHECK_ARG(blocks < 0x7fffffffLL, HIPATTN_E_UNSUPPORTED, "prescale: tensor too large");
    hipLaunchKernelGGL(prescale_k_rope_kernel, dim3((unsigned)blocks), dim3(threads), 0, (hipStream_t)stream,
                       reinterpret_cast<const uint16_t *>(k), reinterpret_cast<uint16_t *>(out), rows, HID, stride_b,
                       stride_t, stride_h, T, HKV, c_k, reinterpret_cast<const uint16_t *>(cos),
                       reinterpret_cast<const uint16_t *>(sin), table_stride, table_len, first, chunk);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

extern "C" int hipattn_prescale_k(const void *k, int64_t stride0, int64_t stride1, int64_t stride2, int64_t n0,
                                  int32_t n1, int32_t n2, int32_t HID, void *out, void *stream) {
    HIPATTN_CHECK_ARG(k && out, HIPATTN_E_ARG, "prescale: null pointer");
    HIPATTN_CHECK_ARG(n0 > 0 && n1 > 0 && n2 > 0 && HID > 0 && HID % 8 == 0, HIPATTN_E_ARG, "prescale: bad sizes");
    HIPATTN_CHECK_ARG(aligned16(k) && aligned16(out) && stride0 % 8 == 0 && stride1 % 8 == 0 && stride2 % 8 == 0,
                      HIPATTN_E_ALIGN, "prescale: pointers and strides must be 16-byte aligned");
    float c_q, c_k;
    scale_constants(HID, HIPATTN_BF16, &c_q, &c_k);
    const long long rows = (long long)n0 * n1 * n2;
    const long long work = rows * (HID / 8);
    const int threads = 256;
    const long long blocks = (work + threads - 1) / threads;
    HIPATTN_CHECK_ARG(blocks < 0x7fffffffLL, HIPATTN_E_UNSUPPORTED, "prescale: tensor too large");
    hipLaunchKernelGGL(prescale_k_kernel, dim3((unsigned)blocks), dim3(threads), 0, (hipStream_t)stream,
                       reinterpret_cast<const uint16_t *>(k), reinterpret_cast<uint16_t *>(out), rows, HID, stride0,
                       stride1, stride2, n1, n2, c_k);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

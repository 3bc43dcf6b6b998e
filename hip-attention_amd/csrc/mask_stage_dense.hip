// Mask-estimation scan stage for small chunks on wide launches: score every token once, replay the searches.
//
// A binary search over a chunk of 2^k tokens samples 2 (k + 1) - 3 distinct tokens; the four heads of a GQA group
// search the same chunks of the same keys and part ways after the first rounds, so together they load about
// 4 * (2 (k + 1) - 3) key rows per chunk through the gather path, two cache lines per row and one row per lane.
// For chunks of 8 tokens that is 20 rows where the chunk holds 8.  The score of a token,
//     s[t] = bf16(max over the block's query rows of q^ . k^[t]),
// depends on nothing but the token, so this kernel loads every token of every chunk once per (query block, kv head)
// into LDS, fully coalesced and straight from global memory, lets each head of the group score all of them on the
// matrix cores, and then walks the reference's search (attention_extend.py:736-745, 1183-1215) on the scores held
// in registers: the samples, comparisons, winners, chunk score and refined left edge are those of the sampling
// kernel, bit for bit, because every score is produced by the same chain of matrix instructions in the same order
// (mask_stage_mfma.hip).  Access flags are set for the tokens the search samples, not for the tokens loaded.
// Keys come from a dense tensor or from a paged cache.
//
// Workgroup = (batch, kv head, scan row) x up to four heads of the group, one wave per head; the wave keeps its Q^
// fragments (A operand) in registers and consumes tiles of 64 tokens (B operand) from LDS.
#include <stdlib.h>

#include "mask_common.hpp"

namespace hipattn {

typedef __attribute__((ext_vector_type(8))) __bf16 md_bf16x8;
typedef __attribute__((ext_vector_type(16))) float md_f32x16;

union MdFrag {
    md_bf16x8 v;
    uint4 q;
};

constexpr int MD_TN = 64;              // tokens per tile
constexpr int MD_DIST = 3;             // tiles whose loads are issued ahead of the tile being consumed
constexpr int MD_NBUF = MD_DIST + 1;   // the buffer refilled at tile t is the one tile t - 1 was read from
constexpr int MD_MAX_CHUNKS = 1024;    // chunk list kept in LDS
constexpr int MD_PASS = 8;             // tiles between two replays of the searches

static __device__ __align__(16) uint16_t md_zero_row[256];

typedef __attribute__((ext_vector_type(2))) __bf16 md_bf16x2;
typedef __attribute__((ext_vector_type(2))) float md_f32x2;
// a packed pair of bf16, each times c, rounded to nearest even
__device__ __forceinline__ uint32_t md_scale_pack(uint32_t w, float c) {
    md_f32x2 v = {__uint_as_float(w << 16) * c, __uint_as_float(w & 0xffff0000u) * c};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, md_bf16x2));
}

// HPW = waves (heads) per workgroup; MB = 32-row blocks of query rows per program (1: up to 32 rows, 2: up to 64);
// PAGED: keys live in a paged cache, the page of every token slot is looked up a pass ahead (below)
// QINLINE: the programs' query rows are the tensor's own rows (stride_q == 1): scaled here instead of read from the
// workspace that the query preparation launch would have filled
template <int HID, int MB, int HPW, bool EXT, bool PAGED, bool QINLINE>
__global__ __launch_bounds__(64 * HPW) void mask_stage_dense_kernel(MaskParamsFor<EXT> p, long long total_wg) {
    constexpr int NT = 64 * HPW;
    constexpr int KS = HID / 16;
    constexpr int PPR = HID / 8;               // 16-byte pieces per key row
    constexpr int CPT = MD_TN * PPR / NT;      // pieces a thread moves per tile = its load instructions per tile
    static_assert((MD_DIST - 1) * CPT < 64, "in-flight loads must fit the counter");
    const KVExt *kx = nullptr;
    if constexpr (EXT) kx = &p.kx;
    // rows of exactly HID elements, the 16-byte pieces of row r permuted by r (piece q sits at q ^ (r % PPR)): the
    // lanes of a fragment read (consecutive rows, same piece) then hit different bank groups
    __shared__ __align__(16) uint16_t s_rows[MD_NBUF][MD_TN][HID];
    // The chunk list of this (batch, scan row), read from global memory once: a vector-memory load inside the tile
    // loop would make the compiler wait for everything in flight, the tile loads included, before it uses the value.
    __shared__ int s_left[MD_MAX_CHUNKS];
    __shared__ float s_gwidth[MD_MAX_CHUNKS / 16];       // per group of block_chunk chunks: widest chunk, 0 = not searched
    __shared__ uint16_t s_score[HPW][MD_PASS * MD_TN];   // per head: scores (bf16 bits) of the tokens of the last MD_PASS tiles
    // Paged keys: the pool page of every token slot of a pass of MD_PASS tiles (-1: slot not loaded), two passes.
    // The block table is read with ordinary loads, which drain the tile loads in flight (see s_left), so it is read
    // once per pass, for the whole next pass, instead of inside the prefetch of every tile.
    __shared__ int s_page[PAGED ? 2 : 1][PAGED ? MD_PASS * MD_TN : 1];

    const int tid = threadIdx.x, lane = tid & 63, wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, hh = lane >> 5;

    long long L = xcd_remap((long long)blockIdx.x, total_wg);
    const int hblocks = (p.G + HPW - 1) / HPW;
    const int hin = (int)(L % hblocks) * HPW + wid;
    L /= hblocks;
    const int s = (int)(L % p.BS);
    L /= p.BS;
    const int kvh = (int)(L % p.kv.HKV);
    const int b = (int)(L / p.kv.HKV);
    const bool head_ok = hin < p.G;
    const int h = kvh * p.G + (head_ok ? hin : 0);

    const int BC = p.block_chunk;
    const int CH = p.chunk;                       // power of two, 2 .. 32
    const int ch_shift = __builtin_ctz(CH);
    const int64_t row_in = ((int64_t)b * p.BS + s) * p.n;  // one chunk list for all heads (hg == 1)
    const int64_t row_out = (((int64_t)b * p.BS + s) * p.HEAD + h) * p.n;
    const int64_t red_out = ((int64_t)b * p.BS + s) * p.n;

    // ---- rows of this program (as in the sampling kernel)
    const long long qb = (long long)(p.BDST - 1) - (long long)(p.BS - 1) * p.scan_stride + (long long)s * p.scan_stride;
    const long long myrow = qb * p.BQ + (long long)lane * p.stride_q;
    const bool rv = (lane < p.nrows) && (myrow >= 0) && (myrow < p.TDST);
    const unsigned long long rowmask = __ballot(rv);
    const long long mypos = rv ? p.pos[(int64_t)b * p.pos_sb + myrow * p.pos_st] : 0x7fffffffffffffffLL;
    const long long pmin = wave_min_ll(mypos);
    unsigned vm[MB];  // which accumulator elements belong to valid rows: element (mb, i) <-> row mb*32 + (i/4)*8 + hh*4 + i%4
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        vm[mb] = 0;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int j = mb * 32 + (i >> 2) * 8 + hh * 4 + (i & 3);
            if ((j < p.nrows) && ((rowmask >> j) & 1ull)) vm[mb] |= 1u << i;
        }
    }
    const int fast_rows = (p.nrows == 16 && rowmask == 0xffffull) ? 16
                        : (p.nrows == 32 && rowmask == 0xffffffffull) ? 32
                        : (MB == 2 && p.nrows == 64 && rowmask == ~0ull) ? 64 : 0;
    const bool any_rows = (rowmask != 0ull) && (pmin >= 0);
    int lim = 0;
    if (any_rows) {
        const long long lm = pmin - p.sw_eff;
        lim = (int)(lm < 0 ? 0 : lm);
    }
    const int64_t seqlen = p.kv.paged ? p.kv.seq_len(b) : 0;
    for (int i = tid; i < MD_MAX_CHUNKS; i += NT) s_left[i] = i < p.n ? p.chunk_left[row_in + i] : -1;

    // ---- Q^ fragments, in the order qhat_kernel stores them (k-step, row half, row)
    MdFrag qf[MB][KS];
    if constexpr (QINLINE) {
        // a row is its own mean: bf16(q * c_q), the k-step's eight elements at hh * HID/2 + ks * 8
        const uint16_t *qbase = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            const int j = mb * 32 + n;
            const bool jv = head_ok && (j < p.nrows) && ((rowmask >> j) & 1ull);
            const long long it = qb * p.BQ + j;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                uint4 w = make_uint4(0, 0, 0, 0);
                if (jv) {
                    w = *reinterpret_cast<const uint4 *>(qbase + it * p.q_st + hh * (HID / 2) + ks * 8);
                    w.x = md_scale_pack(w.x, p.c_q);
                    w.y = md_scale_pack(w.y, p.c_q);
                    w.z = md_scale_pack(w.z, p.c_q);
                    w.w = md_scale_pack(w.w, p.c_q);
                }
                qf[mb][ks].q = w;
            }
        }
    } else {
        const uint16_t *qh = p.qhat + ((((int64_t)b * p.BS + s) * p.HEAD + h) * p.nrows) * HID;
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            const int j = mb * 32 + n;
            const bool jv = head_ok && (j < p.nrows) && ((rowmask >> j) & 1ull);
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                qf[mb][ks].q = make_uint4(0, 0, 0, 0);
                if (jv) qf[mb][ks].q = *reinterpret_cast<const uint4 *>(qh + ((int64_t)(ks * 2 + hh) * p.nrows + j) * 8);
            }
        }
    }

    // ---- tiles: tile x holds the tokens of chunks x * (64 / CH) ... in list order, CH consecutive slots per chunk
    const int cpt_shift = 6 - ch_shift;  // log2(chunks per tile)
    const int ntiles = (p.n + (1 << cpt_shift) - 1) >> cpt_shift;
    // piece slot c = tid + NT * j of a tile is position c % PPR of token slot c / PPR; one load instruction of a wave
    // fills 64 consecutive piece slots
    const uint16_t *pf_base[CPT];
    int pf_e[CPT];
#pragma unroll
    for (int j = 0; j < CPT; j++) {
        const int c = tid + NT * j;
        const int slot = c / PPR, pos = c % PPR;
        pf_e[j] = slot & (CH - 1);
        pf_base[j] = reinterpret_cast<const uint16_t *>(p.kv.k) + (int64_t)b * p.kv.k_stride_b +
                     (int64_t)pf_e[j] * p.kv.k_stride_t + (int64_t)kvh * p.kv.k_stride_h + ((pos ^ slot) & (PPR - 1)) * 8;
    }
    const unsigned lim_u = any_rows ? (unsigned)lim : 0u;
    const bool none_u = !any_rows;  // then even cl == 0 must fail
    const int t_end = none_u ? -0x7fffffff : (int)(p.right_clamp < (int64_t)p.kv.tsrc ? p.right_clamp : (int64_t)p.kv.tsrc);
    // the address of the row of zeros, formed once (the compiler would fetch it from the offset table at every use)
    const uint16_t *zero_row = md_zero_row;
    asm volatile("" : "+s"(zero_row));
    auto prefetch = [&](int tile) {
        const int buf = tile % MD_NBUF;
        // all addresses first, then the loads back to back: the load statements keep their order, so an LDS read
        // between two of them would be waited for there
        const uint16_t *src[CPT];
        if constexpr (PAGED) {
#pragma unroll
            for (int j = 0; j < CPT; j++) {
                const int slot = (tid + NT * j) / PPR, pos = (tid + NT * j) % PPR;
                const int ci = (tile << cpt_shift) + (slot >> ch_shift);
                src[j] = zero_row;
                const int pg = s_page[(tile / MD_PASS) & 1][(tile % MD_PASS) * MD_TN + slot];
                if (pg >= 0) {
                    const int t = s_left[ci] + (slot & (CH - 1));  // pg >= 0 implies ci < p.n
                    src[j] = reinterpret_cast<const uint16_t *>(p.kv.k) + (int64_t)pg * p.kv.k_stride_b +
                             (int64_t)(t & (p.kv.page_size - 1)) * p.kv.k_stride_t + (int64_t)kvh * p.kv.k_stride_h +
                             ((pos ^ slot) & (PPR - 1)) * 8;
                }
            }
        } else {
            // Dense keys: the row address is plain arithmetic, and all of it but the chunk's left edge is the same
            // for every tile (pf_base).  A chunk that starts beyond the block's reach is never searched (its left
            // edge only moves right): 0 <= cl <= lim as one unsigned compare; entries of the list beyond its end
            // hold -1.  Rows at or beyond the end of the chunk (right_clamp) or of the tensor read as zeros.
            // The list entries of all loads are read from LDS together, and nothing below branches: the offset of a
            // row from its chunk's left edge is one 24-bit multiply (the product fits 31 bits and its factors 24:
            // checked before the launch).
            int cl[CPT];
#pragma unroll
            for (int j = 0; j < CPT; j++) cl[j] = s_left[(tile << cpt_shift) + (((tid + NT * j) / PPR) >> ch_shift)];
#pragma unroll
            for (int j = 0; j < CPT; j++) {
                const int t = cl[j] + pf_e[j];
                const bool ok = ((unsigned)cl[j] <= lim_u) & (t < t_end);
                const uint16_t *row = pf_base[j] + (int64_t)(int)__umul24((uint32_t)cl[j], (uint32_t)p.kv.k_stride_t);
                src[j] = ok ? row : zero_row;
            }
        }
#pragma unroll
        for (int j = 0; j < CPT; j++) load_to_lds16(src[j], &s_rows[buf][0][0] + (wid * 64 + NT * j) * 8);
    };
    // pages of the token slots of pass `pass` (tiles pass * MD_PASS ...), by all threads
    auto lookup_pages = [&](int pass) {
        if constexpr (PAGED) {
            for (int i = tid; i < MD_PASS * MD_TN; i += NT) {
                const int ci = ((pass * MD_PASS) << cpt_shift) + (i >> ch_shift);
                int pg = -1;
                if (ci < p.n) {
                    const int cl = s_left[ci];
                    const int64_t rr = (int64_t)cl + CH;
                    const int cr = (int)(rr < p.right_clamp ? rr : p.right_clamp);
                    const int t = cl + (i & (CH - 1));
                    if (t < cr && cl <= lim && cl >= 0 && any_rows) pg = (int)p.kv.page_of(b, t, seqlen);
                }
                s_page[pass & 1][i] = pg;
            }
        }
    };
    __syncthreads();  // s_left visible (the loads above are complete: their values were stored)
    if constexpr (PAGED) {
        lookup_pages(0);
        __syncthreads();
    }
    for (int x = 0; x < MD_DIST && x < ntiles; x++) prefetch(x);

    // ---- program-level gate and iteration count of the reference, per group of block_chunk chunks, once
    for (int g = tid; g < p.ngroups; g += NT) {
        int glmin = 0x7fffffff, wmax = -0x7fffffff;
        for (int i = 0; i < BC; i++) {
            const int ci = g * BC + i;
            int gl = (int)p.kv.max_tsrc, gr = (int)p.kv.max_tsrc;  // padding entries of a short last group
            if (ci < p.n) {
                gl = s_left[ci];
                const int64_t rr = (int64_t)gl + CH;
                gr = (int)(rr < p.right_clamp ? rr : p.right_clamp);
            }
            glmin = gl < glmin ? gl : glmin;
            wmax = (gr - gl) > wmax ? (gr - gl) : wmax;
        }
        const bool run = any_rows && (pmin + (long long)p.BQ * p.scan_stride >= (long long)glmin);
        s_gwidth[g] = (run && (float)wmax >= p.terminate) ? (float)wmax : 0.0f;  // 0: the group is not searched
    }
    __syncthreads();

    // The searches are replayed once per PASS tiles, one lane per chunk, on the scores the tiles left in LDS: replaying
    // them tile by tile would keep 64 lanes busy with the four or eight chunks of a block.
    uint16_t *my_scores = &s_score[wid][0];
    auto replay = [&](int first_tile, int last_tile) {  // chunks of tiles [first_tile, last_tile]
        const int c_begin = first_tile << cpt_shift;
        int c_end = (last_tile + 1) << cpt_shift;
        c_end = c_end < p.n ? c_end : p.n;
        for (int cidx = c_begin + lane; cidx < c_end; cidx += 64) {
            int cl = s_left[cidx];
            const int64_t rr = (int64_t)cl + CH;
            int cr = (int)(rr < p.right_clamp ? rr : p.right_clamp);
            const int cl0 = cl;
            float score = -32000.0f;
            float width = s_gwidth[cidx / BC];
            const uint16_t *sc = my_scores + ((cidx - c_begin) << ch_shift);  // s[cl0 + e] at sc[e]
            unsigned touched = 0;  // bit e: the search sampled token cl0 + e
            while (width >= p.terminate) {
                width *= 0.5f;
                const bool active = (cl < cr) && (cl <= lim) && (cl >= 0);
                if (active) {
                    const int ctr = (cl + cr) >> 1;
                    const int eL = ((cl + ctr) >> 1) - cl0, eR = ((ctr + cr) >> 1) - cl0;
                    const float sL = __uint_as_float((uint32_t)sc[eL] << 16), sR = __uint_as_float((uint32_t)sc[eR] << 16);
                    touched |= (1u << eL) | (1u << eR);
                    const bool win = sL > sR;
                    if (win) cr = ctr; else cl = ctr;
                    score = fmaxf(score, win ? sL : sR);
                }
            }
            if constexpr (EXT) {
                // access flags for the rows the sampling kernel would have loaded, stored without looking first
                for (int e = 0; e < CH; e++)
                    if ((touched >> e) & 1u) {
                        if constexpr (PAGED) {
                            // paged flags are per pool page; the page was looked up with the slot
                            const int pg = s_page[(first_tile / MD_PASS) & 1][((cidx - c_begin) << ch_shift) + e];
                            if (kx->access_flags && pg >= 0)
                                mark_flag<false>(kx->access_flags + (int64_t)b * kx->flags_stride_b +
                                                 (int64_t)kvh * kx->flags_stride_h + pg);
                        } else {
                            // (written out: the general routine's paged and cached branches hold loads, and a load
                            // the compiler tracks anywhere in the tile loop makes it drain the tile loads in flight)
                            const int t = cl0 + e;
                            if (kx->access_flags && t >= 0 && t < p.kv.tsrc)
                                mark_flag<false>(kx->access_flags + (int64_t)b * kx->flags_stride_b +
                                                 (int64_t)kvh * kx->flags_stride_h + t);
                        }
                    }
            }
            store_score(p, row_out, red_out, cidx, score);
            if (p.left_out) p.left_out[row_out + cidx] = cl;
        }
    };

    for (int tile = 0; tile < ntiles; tile++) {
        const int buf = tile % MD_NBUF;
        // this wave's loads of the tile have landed (those of later tiles may still be in flight); after the barrier
        // everyone's have, and everyone is done with the buffer of the tile before, which the next loads overwrite
        const int newer = ntiles - 1 - tile;
        if (newer >= MD_DIST - 1) wait_vmcnt<(MD_DIST - 1) * CPT>();
        else if (newer == 1 && MD_DIST > 2) wait_vmcnt<CPT>();
        else wait_vmcnt<0>();
        __syncthreads();
        if (tile + MD_DIST < ntiles) prefetch(tile + MD_DIST);
        if constexpr (PAGED) {
            // the next pass's pages: written here, made visible by the barrier of the next round, first read by the
            // prefetch of the round after
            static_assert(MD_PASS - MD_DIST - 2 >= 0, "room for the lookup before the first prefetch of a pass");
            if ((tile % MD_PASS) == MD_PASS - MD_DIST - 2 && (tile / MD_PASS + 1) * MD_PASS < ntiles)
                lookup_pages(tile / MD_PASS + 1);
        }
        if (!head_ok) continue;
        // a block of 32 tokens lies inside one group (block_chunk * CH is a multiple of 32)
        bool searched[2];
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
            const int c0 = ((tile * 2 + nb) * 32) >> ch_shift;  // first chunk of this block of 32 tokens
            searched[nb] = c0 < p.n && __builtin_amdgcn_readfirstlane(__float_as_int(s_gwidth[c0 / BC])) != 0;
        }
        if (!searched[0] && !searched[1]) continue;
        // ---- s[token] for the 64 tokens of the tile: all K^ fragments of the tile are fetched from LDS first, then
        // the four accumulation chains (two token blocks x two row blocks) keep the matrix unit fed back to back
        MdFrag kf[2][KS];
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
            const int r = nb * 32 + n;
#pragma unroll
            for (int ks = 0; ks < KS; ks++)
                kf[nb][ks].q = *reinterpret_cast<const uint4 *>(&s_rows[buf][r][(((hh * (PPR / 2) + ks) ^ r) & (PPR - 1)) * 8]);
        }
        // the compiler's scheduler would otherwise sink every fragment read to just before its first use and wait
        // for it there, one LDS round trip per k-step
        __builtin_amdgcn_sched_barrier(0);
        md_f32x16 acc[2][MB];
#pragma unroll
        for (int nb = 0; nb < 2; nb++)
#pragma unroll
            for (int mb = 0; mb < MB; mb++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[nb][mb][i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
#pragma unroll
            for (int nb = 0; nb < 2; nb++)
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
                    acc[nb][mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qf[mb][ks].v, kf[nb][ks].v, acc[nb][mb], 0, 0, 0);
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
            float v = -INFINITY;
            if (fast_rows == 16) {
#pragma unroll
                for (int i = 0; i < 8; i++) v = fmaxf(v, acc[nb][0][i]);
            } else if (fast_rows == 32) {
#pragma unroll
                for (int i = 0; i < 16; i++) v = fmaxf(v, acc[nb][0][i]);
            } else if (fast_rows == 64) {
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
#pragma unroll
                    for (int i = 0; i < 16; i++) v = fmaxf(v, acc[nb][mb][i]);
            } else {
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
#pragma unroll
                    for (int i = 0; i < 16; i++) v = fmaxf(v, ((vm[mb] >> i) & 1u) ? acc[nb][mb][i] : -INFINITY);
            }
            v = fmaxf(v, swap_halves(v));
            if (hh == 0 && searched[nb]) my_scores[(tile % MD_PASS) * MD_TN + nb * 32 + n] = (uint16_t)(__float_as_uint(round_bf16(v)) >> 16);
        }
        if ((tile % MD_PASS) == MD_PASS - 1 || tile == ntiles - 1) replay(tile - (tile % MD_PASS), tile);  // the wave's own LDS writes
    }
}

__global__ void md_fill_scores_kernel(float *scores, long long n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
        scores[i] = -INFINITY;
}

void mask_stage_fill_scores(const MaskParams &p, hipStream_t st) {
    if (p.reduce_heads != 1) return;  // 0: plain stores; 2: the caller has initialised them
    const long long nscores = (long long)p.B * p.BS * p.n;
    const long long blocks = (nscores + 255) / 256;
    hipLaunchKernelGGL(md_fill_scores_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, st, p.scores, nscores);
}

template <int HID, int MB, int HPW, bool QINLINE>
static int launch_dense(const MaskParams &p, hipStream_t st) {
    const int hblocks = (p.G + HPW - 1) / HPW;
    const long long total = (long long)p.B * p.kv.HKV * p.BS * hblocks;
    if (total >= 0x7fffffffLL) return HIPATTN_E_UNSUPPORTED;
    dim3 grid((unsigned)total), block(64 * HPW);
    const MaskParamsBase &pb = p;
    if (p.kx.extended()) {
        if (p.kv.paged) hipLaunchKernelGGL((mask_stage_dense_kernel<HID, MB, HPW, true, true, QINLINE>), grid, block, 0, st, p, total);
        else hipLaunchKernelGGL((mask_stage_dense_kernel<HID, MB, HPW, true, false, QINLINE>), grid, block, 0, st, p, total);
    } else {
        if (p.kv.paged) hipLaunchKernelGGL((mask_stage_dense_kernel<HID, MB, HPW, false, true, QINLINE>), grid, block, 0, st, pb, total);
        else hipLaunchKernelGGL((mask_stage_dense_kernel<HID, MB, HPW, false, false, QINLINE>), grid, block, 0, st, pb, total);
    }
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

template <int HID, bool QINLINE>
static int launch_dense_hid(const MaskParams &p, int rows_eff, hipStream_t st) {
    const bool two = rows_eff > 32;
    if (p.G >= 4) return two ? launch_dense<HID, 2, 4, QINLINE>(p, st) : launch_dense<HID, 1, 4, QINLINE>(p, st);
    if (p.G >= 2) return two ? launch_dense<HID, 2, 2, QINLINE>(p, st) : launch_dense<HID, 1, 2, QINLINE>(p, st);
    return HIPATTN_E_UNSUPPORTED;
}

bool mask_stage_dense_applies(const MaskParams &p, int HID, int rows_eff) {
    // HIPATTN_MASK_DENSE: 0 = never, 1 = where it pays (default), 2 = wherever the kernel applies (testing)
    const char *e = getenv("HIPATTN_MASK_DENSE");  // read on every call: tests switch it inside one process
    const int mode = e ? atoi(e) : 1;
    if (mode == 0) return false;
    const int CH = p.chunk;
    // (mode 2 also takes chunks of 32 tokens, for measurements: there the kernel streams four times the bytes of the
    // 8-token stage and loses to the sampling kernel, 7.0 against 2.5 ms on 32k queries x 128k keys)
    if (CH < 2 || CH > (mode == 2 ? 32 : 16) || (CH & (CH - 1)) != 0) return false;
    if (p.hg != 1 || p.rope.cos || p.kx.cached || p.kx.kv8) return false;
    if (p.nrows > 64 || p.n > MD_MAX_CHUNKS) return false;
    if (HID != 64 && HID != 128) return false;
    if (p.G < 2) return false;  // one head per group: nothing to share, the sampling kernel reads fewer rows
    if (mode == 1) {
        // pays when the group's searches together load more rows than the chunks hold, on launches wide enough to
        // keep the chip busy with one workgroup per (batch, kv head, scan row)
        const int iters = 32 - __builtin_clz((unsigned)CH);  // floor(log2(CH)) + 1
        const int per_search = 2 * iters - 3;
        const long long wgs = (long long)p.B * p.kv.HKV * p.BS;
        if (!(per_search * p.G >= 2 * CH) || wgs < 1024 || p.n < 64) return false;
    }
    // dense keys: a row's offset from its chunk's left edge is formed with one 24-bit multiply
    if (!p.kv.paged && !(p.kv.k_stride_t > 0 && p.kv.k_stride_t < (1 << 24) && p.kv.tsrc < (1 << 24) &&
                         p.kv.tsrc * p.kv.k_stride_t < (1LL << 31)))
        return false;
    const int hpw = p.G >= 4 ? 4 : 2;
    const long long total = (long long)p.B * p.kv.HKV * p.BS * ((p.G + hpw - 1) / hpw);
    (void)rows_eff;
    return total < 0x7fffffffLL;
}

int mask_stage_dense_launch(const MaskParams &p, int HID, int rows_eff, bool q_inline, hipStream_t st) {
    if (q_inline && p.stride_q != 1) return HIPATTN_E_UNSUPPORTED;
    switch (HID) {
        case 64: return q_inline ? launch_dense_hid<64, true>(p, rows_eff, st) : launch_dense_hid<64, false>(p, rows_eff, st);
        case 128: return q_inline ? launch_dense_hid<128, true>(p, rows_eff, st) : launch_dense_hid<128, false>(p, rows_eff, st);
    }
    return HIPATTN_E_UNSUPPORTED;
}

}  // namespace hipattn

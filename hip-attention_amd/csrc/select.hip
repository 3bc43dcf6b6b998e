// Selection between scan stages and the final metadata layout.
//
// One workgroup owns one (batch, output scan row, head group).  Chunk lists are kept ascending by
// start position at every stage, so "gather the top-k, then sort by position" is a stream
// compaction in position order: no sort is needed.  The top-k set is found by an exact radix
// select on order-preserving integer keys; ties at the threshold are broken by position, which
// is the fixed tie-break rule (score descending, position ascending).
#include <stdlib.h>

#include "common.hpp"

namespace hipattn {

constexpr int SEL_THREADS = 256;
constexpr int SEL_MAX_N = 16384;

__device__ __forceinline__ uint32_t score_key(float f) {
    if (f == 0.0f) f = 0.0f;  // -0 and +0 tie
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// block-wide exclusive scan of one int per thread; returns the exclusive prefix, total in *total
__device__ __forceinline__ int block_excl_scan(int v, int *s_tmp, int *total) {
    const int tid = threadIdx.x;
    const int lane = tid & 63, wid = tid >> 6;
    int incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        int t = __shfl_up(incl, o);
        if (lane >= o) incl += t;
    }
    if (lane == 63) s_tmp[wid] = incl;
    __syncthreads();
    int base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < SEL_THREADS / 64; w++) {
        int x = s_tmp[w];
        if (w < wid) base += x;
        tot += x;
    }
    __syncthreads();
    *total = tot;
    return base + incl - v;
}

// Shared front end: keys[c] = max over the heads of the group, then the k-th largest key.
// On return s_keys holds the keys, *thr the threshold key and *need how many entries equal to the
// threshold are taken (in position order).
__device__ void topk_threshold(const float *scores_row /* [nheads, n] with stride n */, int nheads, int n, int k,
                               uint32_t *s_keys, int *s_hist, int *s_misc, uint32_t *thr, int *need_out) {
    const int tid = threadIdx.x;
    for (int c = tid; c < n; c += SEL_THREADS) {
        float m = scores_row[c];
        for (int hh = 1; hh < nheads; hh++) m = fmaxf(m, scores_row[(int64_t)hh * n + c]);
        s_keys[c] = score_key(m);
    }
    __syncthreads();
    uint32_t prefix = 0, mask = 0;
    int need = k;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = tid; i < 256; i += SEL_THREADS) s_hist[i] = 0;
        __syncthreads();
        {
            // scores cluster: most keys of a pass fall into a handful of bins, so a thread adds up the run of
            // equal bins it meets before it touches the shared counter
            int cur = -1, cnt = 0;
            for (int c = tid; c < n; c += SEL_THREADS) {
                const uint32_t key = s_keys[c];
                if ((key & mask) == prefix) {
                    const int bin = (int)((key >> shift) & 255u);
                    if (bin == cur) {
                        cnt++;
                    } else {
                        if (cnt) atomicAdd(&s_hist[cur], cnt);
                        cur = bin;
                        cnt = 1;
                    }
                }
            }
            if (cnt) atomicAdd(&s_hist[cur], cnt);
        }
        __syncthreads();
        if (tid < 64) {
            // first wave: lane l owns bins 255-4l .. 252-4l; a prefix sum from the top finds the bin in which
            // the need-th largest key falls
            int hv[4];
            int mine = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                hv[j] = s_hist[255 - 4 * tid - j];
                mine += hv[j];
            }
            int incl = mine;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int up = __shfl_up(incl, o);
                if (tid >= o) incl += up;
            }
            int cum = incl - mine;
            if (cum < need && need <= incl) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if (cum < need && need <= cum + hv[j]) {
                        s_misc[0] = 255 - 4 * tid - j;
                        s_misc[1] = need - cum;
                    }
                    cum += hv[j];
                }
            }
        }
        __syncthreads();
        prefix |= ((uint32_t)s_misc[0]) << shift;
        mask |= 255u << shift;
        need = s_misc[1];
        __syncthreads();
    }
    *thr = prefix;
    *need_out = need;
}

// Marks the selected entries and returns, per thread, the output rank of the first selected entry
// of its contiguous segment.  seg = entries per thread.
struct SegScan {
    int seg, begin, end, out_base, eq_base;
};

__device__ __forceinline__ SegScan selection_scan(const uint32_t *s_keys, int n, uint32_t thr, int need, int *s_tmp) {
    SegScan r;
    r.seg = (n + SEL_THREADS - 1) / SEL_THREADS;
    r.begin = threadIdx.x * r.seg;
    r.end = r.begin + r.seg < n ? r.begin + r.seg : n;
    int eq = 0, gt = 0;
    for (int c = r.begin; c < r.end; c++) {
        uint32_t key = s_keys[c];
        eq += (key == thr);
        gt += (key > thr);
    }
    int tot;
    r.eq_base = block_excl_scan(eq, s_tmp, &tot);
    // selected in this segment = gt + clamp(need - eq_base, 0, eq)
    int take = need - r.eq_base;
    take = take < 0 ? 0 : (take > eq ? eq : take);
    r.out_base = block_excl_scan(gt + take, s_tmp, &tot);
    return r;
}

__global__ __launch_bounds__(SEL_THREADS) void select_stage_kernel(const float *scores, const int32_t *chunk_left,
                                                                  int bs_in, int bs_out, int row_rep, int HEAD, int hg,
                                                                  int n, int k, int sub_chunk, int splits,
                                                                  int32_t *next_left, int64_t *left64,
                                                                  int64_t *right64, float *next_scores) {
    __shared__ uint32_t s_keys[SEL_MAX_N];
    __shared__ int s_hist[256];
    __shared__ int s_misc[2];
    __shared__ int s_tmp[SEL_THREADS / 64];
    int *s_sel = reinterpret_cast<int *>(s_keys);  // reused after selection: positions of selected chunks

    const int hgi = blockIdx.x % hg;
    const int o = (blockIdx.x / hg) % bs_out;
    const int b = blockIdx.x / (hg * bs_out);
    const int i = (o + row_rep * bs_in - bs_out) / row_rep;
    const int nheads = HEAD / hg;
    const float *srow = scores + (((int64_t)b * bs_in + i) * HEAD + (int64_t)hgi * nheads) * n;
    const int32_t *lrow = chunk_left + (((int64_t)b * bs_in + i) * hg + hgi) * n;
    const int64_t obase = (((int64_t)b * bs_out + o) * hg + hgi) * ((int64_t)k * splits);

    uint32_t thr;
    int need;
    if (k >= n) {
        thr = 0;
        need = 0;
        for (int c = threadIdx.x; c < n; c += SEL_THREADS) s_keys[c] = 1u;  // everything > thr
        __syncthreads();
    } else {
        topk_threshold(srow, nheads, n, k, s_keys, s_hist, s_misc, &thr, &need);
    }
    SegScan sc = selection_scan(s_keys, n, thr, need, s_tmp);
    // each thread notes which entries of its segment are selected (keys are still being read by others), then the
    // positions are listed in output order
    int out = sc.out_base, eqr = sc.eq_base;
    unsigned long long selbits = 0ull;  // seg <= 64 since n <= 16384
    for (int c = sc.begin; c < sc.end; c++) {
        uint32_t key = s_keys[c];
        bool sel = key > thr;
        if (key == thr) {
            sel = eqr < need;
            eqr++;
        }
        if (sel) selbits |= 1ull << (c - sc.begin);
    }
    __syncthreads();
    for (int c = sc.begin; c < sc.end; c++) {
        if ((selbits >> (c - sc.begin)) & 1ull) s_sel[out++] = c;
    }
    __syncthreads();
    // exactly k entries are selected (k <= n); every thread emits sub-chunks of its own, all loads independent
    const int total = k * splits;
    for (int idx = threadIdx.x; idx < total; idx += SEL_THREADS) {
        const int e = idx / splits, j = idx - e * splits;
        const int left = lrow[s_sel[e]] + j * sub_chunk;
        next_left[obase + idx] = left;
        if (next_scores) next_scores[obase + idx] = -INFINITY;  // the next stage's head-reduced scores start here
        if (left64) {  // the same list as the next stage's cached inputs: int64 edges (left, left + chunk)
            left64[obase + idx] = left;
            right64[obase + idx] = (int64_t)left + sub_chunk;
        }
    }
}

// The same selection for launches of a few workgroups (decode: one per sequence), where the time is the length of the
// dependent chain and not the work: 1024 threads hold ITEMS consecutive keys (and chunk edges) each in registers, so
// the radix passes re-read nothing, the output ranks come from one block scan of packed counts, and the trips to
// memory are two: every load is requested before the first is used (no load sits in a branch: an entry past the end
// reads the last one and is ignored), and the output is written by all threads at once from a list in LDS.  Keys whose
// low 16 bits follow from their sign (scores that were rounded to bf16) need two radix passes instead of four.
constexpr int FAST_THREADS = 1024;
constexpr int FAST_MAX_K = 8192;  // selected entries a workgroup can list in LDS

template <int ITEMS>
constexpr int FAST_LIST = ITEMS * FAST_THREADS < FAST_MAX_K ? ITEMS * FAST_THREADS : FAST_MAX_K;

// keys of entries c0 .. c0+ITEMS-1: the maximum over the heads of the group, as order-preserving integers
template <int ITEMS>
__device__ __forceinline__ void fast_load_keys(const float *srow, int nheads, int n, int c0, uint32_t (&key)[ITEMS],
                                               bool *plain_low_out) {
    float m[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; i++) m[i] = srow[c0 + i < n ? c0 + i : n - 1];
    for (int hh = 1; hh < nheads; hh++) {
        float x[ITEMS];
#pragma unroll
        for (int i = 0; i < ITEMS; i++) x[i] = srow[(int64_t)hh * n + (c0 + i < n ? c0 + i : n - 1)];
#pragma unroll
        for (int i = 0; i < ITEMS; i++) m[i] = fmaxf(m[i], x[i]);
    }
    bool plain_low = true;  // low 16 bits are all zero (positive) / all one (negative) in every key
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
        key[i] = c0 + i < n ? score_key(m[i]) : 0u;
        if (c0 + i < n) plain_low = plain_low && ((key[i] & 0xffffu) == ((key[i] >> 31) ? 0u : 0xffffu));
    }
    *plain_low_out = plain_low;
}

// The k-th largest key of the workgroup's n keys (k < n): on return an entry is above the threshold when
// (key & mask) > prefix, and of those with (key & mask) == prefix the first `need` in position order are taken.
template <int ITEMS>
__device__ __forceinline__ void fast_threshold(const uint32_t (&key)[ITEMS], int c0, int n, int k, bool plain_low,
                                               int *s_hist, int *s_misc, uint32_t *prefix_out, uint32_t *mask_out,
                                               int *need_out) {
    const int tid = threadIdx.x;
    uint32_t prefix = 0, mask = 0;
    int need = k;
    const int last_shift = __syncthreads_and(plain_low ? 1 : 0) ? 16 : 0;
    for (int shift = 24; shift >= last_shift; shift -= 8) {
        if (tid < 256) s_hist[tid] = 0;
        __syncthreads();
        {
            int cur = -1, cnt = 0;
#pragma unroll
            for (int i = 0; i < ITEMS; i++) {
                if (c0 + i < n && (key[i] & mask) == prefix) {
                    const int bin = (int)((key[i] >> shift) & 255u);
                    if (bin == cur) {
                        cnt++;
                    } else {
                        if (cnt) atomicAdd(&s_hist[cur], cnt);
                        cur = bin;
                        cnt = 1;
                    }
                }
            }
            if (cnt) atomicAdd(&s_hist[cur], cnt);
        }
        __syncthreads();
        if (tid < 64) {  // lane l owns bins 255-4l .. 252-4l; a prefix sum from the top finds the need-th largest
            int hv[4];
            int mine = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                hv[j] = s_hist[255 - 4 * tid - j];
                mine += hv[j];
            }
            int incl = mine;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int up = __shfl_up(incl, off);
                if (tid >= off) incl += up;
            }
            int cum = incl - mine;
            if (cum < need && need <= incl) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if (cum < need && need <= cum + hv[j]) {
                        s_misc[0] = 255 - 4 * tid - j;
                        s_misc[1] = need - cum;
                    }
                    cum += hv[j];
                }
            }
        }
        __syncthreads();
        prefix |= ((uint32_t)s_misc[0]) << shift;
        mask |= 255u << shift;
        need = s_misc[1];
    }
    *prefix_out = prefix;
    *mask_out = mask;
    *need_out = need;
}

// block-wide exclusive sum of one packed pair of 16-bit counts per thread (1024 threads); *total: the sum over all
__device__ __forceinline__ uint32_t fast_excl_scan(uint32_t packed, uint32_t *s_wave, uint32_t *total) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    uint32_t incl = packed;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
    }
    if (lane == 63) s_wave[wid] = incl;
    __syncthreads();
    // the sixteen wave totals: lane w of every wave takes one, a scan over sixteen lanes gives base and total
    uint32_t wt = lane < FAST_THREADS / 64 ? s_wave[lane] : 0u;
    uint32_t winc = wt;
#pragma unroll
    for (int off = 1; off < FAST_THREADS / 64; off <<= 1) {
        const uint32_t up = __shfl_up(winc, off);
        if (lane >= off) winc += up;
    }
    const uint32_t base = __shfl(winc - wt, wid);
    *total = __shfl(winc, FAST_THREADS / 64 - 1);
    return base + incl - packed;
}

// Output rank of every selected entry of this thread (-1: not selected).  all: every entry is selected.
template <int ITEMS>
__device__ __forceinline__ void fast_ranks(const uint32_t (&key)[ITEMS], int c0, int n, bool all, uint32_t prefix,
                                           uint32_t mask, int need, uint32_t *s_wave, int (&rank)[ITEMS]) {
    uint32_t packed = 0;  // low half: entries above the threshold, high half: entries equal to it
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
        if (c0 + i < n) {
            const uint32_t mk = key[i] & mask;
            packed += all ? 1u : ((mk > prefix ? 1u : 0u) + (mk == prefix ? 0x10000u : 0u));
        }
    }
    uint32_t total;
    const uint32_t before = fast_excl_scan(packed, s_wave, &total);
    int gt_before = (int)(before & 0xffffu), eq_before = (int)(before >> 16);
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
        rank[i] = -1;
        if (c0 + i >= n) continue;
        const uint32_t mk = key[i] & mask;
        const bool gt = all || mk > prefix;
        const bool eq = !all && mk == prefix;
        if (gt || (eq && eq_before < need)) rank[i] = gt_before + (eq_before < need ? eq_before : need);
        gt_before += gt ? 1 : 0;
        eq_before += eq ? 1 : 0;
    }
}

template <int ITEMS>
__global__ __launch_bounds__(FAST_THREADS) void select_stage_fast_kernel(const float *scores, const int32_t *chunk_left,
                                                                        int bs_in, int bs_out, int row_rep, int HEAD,
                                                                        int hg, int n, int k, int sub_chunk, int splits,
                                                                        int32_t *next_left, int64_t *left64,
                                                                        int64_t *right64, float *next_scores) {
    __shared__ int s_hist[256];
    __shared__ int s_misc[2];
    __shared__ uint32_t s_wave[FAST_THREADS / 64];
    __shared__ int s_left[FAST_LIST<ITEMS>];  // left edges of the selected chunks in output order

    const int tid = threadIdx.x;
    const int hgi = blockIdx.x % hg;
    const int o = (blockIdx.x / hg) % bs_out;
    const int b = blockIdx.x / (hg * bs_out);
    const int i_in = (o + row_rep * bs_in - bs_out) / row_rep;
    const int nheads = HEAD / hg;
    const float *srow = scores + (((int64_t)b * bs_in + i_in) * HEAD + (int64_t)hgi * nheads) * n;
    const int32_t *lrow = chunk_left + (((int64_t)b * bs_in + i_in) * hg + hgi) * n;
    const int64_t obase = (((int64_t)b * bs_out + o) * hg + hgi) * ((int64_t)k * splits);

    const int c0 = tid * ITEMS;
    int left[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; i++) left[i] = lrow[c0 + i < n ? c0 + i : n - 1];
    uint32_t key[ITEMS];
    bool plain_low;
    fast_load_keys<ITEMS>(srow, nheads, n, c0, key, &plain_low);

    uint32_t prefix = 0, mask = 0;
    int need = 0;  // k >= n: everything is selected, no key equals the (empty) threshold
    if (k < n) fast_threshold<ITEMS>(key, c0, n, k, plain_low, s_hist, s_misc, &prefix, &mask, &need);
    int rank[ITEMS];
    fast_ranks<ITEMS>(key, c0, n, k >= n, prefix, mask, need, s_wave, rank);
#pragma unroll
    for (int i = 0; i < ITEMS; i++)
        if (rank[i] >= 0) s_left[rank[i]] = left[i];
    __syncthreads();
    // exactly k entries are selected (k <= n): every thread emits sub-chunks of its own
    const int total = k * splits;
    for (int idx = tid; idx < total; idx += FAST_THREADS) {
        const int e = idx / splits, j = idx - e * splits;
        const int v = s_left[e] + j * sub_chunk;
        next_left[obase + idx] = v;
        if (next_scores) next_scores[obase + idx] = -INFINITY;  // the next stage's head-reduced scores start here
        if (left64) {  // the same list as the next stage's cached inputs: int64 edges (left, left + chunk)
            left64[obase + idx] = v;
            right64[obase + idx] = (int64_t)v + sub_chunk;
        }
    }
}

__global__ __launch_bounds__(SEL_THREADS) void finalize_kernel(const float *scores, const int32_t *left_out,
                                                               const int64_t *pos, int64_t pos_sb, int64_t pos_st,
                                                               int bs, int bdst, int scan_stride, int HEAD,
                                                               int score_heads, int hg, int hsplit, int n, int K,
                                                               int chunk, int bq, int64_t *indices, int64_t *ks,
                                                               int32_t *ks_start_end) {
    __shared__ uint32_t s_keys[SEL_MAX_N];
    __shared__ int s_hist[256];
    __shared__ int s_misc[2];
    __shared__ int s_tmp[SEL_THREADS / 64];
    int *s_sel = reinterpret_cast<int *>(s_keys);  // reused after selection: positions of selected chunks

    // workgroup = (batch, query block, head group, slice of the group's heads): every slice repeats the
    // selection, then lays out the rows of its own heads
    const int hs = blockIdx.x % hsplit;
    const int wg = blockIdx.x / hsplit;
    const int hgi = wg % hg;
    const int qb = (wg / hg) % bdst;
    const int b = wg / (hg * bdst);
    const int i = (qb + scan_stride * bs - bdst) / scan_stride;
    const int nheads = HEAD / hg;
    const int nsh = score_heads / hg;
    const int BK = K < n ? K : n;
    const float *srow = scores + (((int64_t)b * bs + i) * score_heads + (int64_t)hgi * nsh) * n;

    uint32_t thr;
    int need;
    if (BK >= n) {
        thr = 0;
        need = 0;
        for (int c = threadIdx.x; c < n; c += SEL_THREADS) s_keys[c] = 1u;
        __syncthreads();
    } else {
        topk_threshold(srow, nsh, n, BK, s_keys, s_hist, s_misc, &thr, &need);
    }
    SegScan sc = selection_scan(s_keys, n, thr, need, s_tmp);
    // each thread lists its selected positions in registers first (keys are still being read by others)
    int out = sc.out_base, eqr = sc.eq_base;
    unsigned long long selbits = 0ull;  // seg <= 64 since n <= 16384
    for (int c = sc.begin; c < sc.end; c++) {
        uint32_t key = s_keys[c];
        bool sel = key > thr;
        if (key == thr) {
            sel = eqr < need;
            eqr++;
        }
        if (sel) selbits |= 1ull << (c - sc.begin);
    }
    __syncthreads();
    for (int c = sc.begin; c < sc.end; c++) {
        if ((selbits >> (c - sc.begin)) & 1ull) s_sel[out++] = c;
    }
    __syncthreads();

    const int64_t first_pos = pos[(int64_t)b * pos_sb + (int64_t)qb * bq * pos_st];
    const int64_t limit = first_pos + bq;
    const int per = (BK + SEL_THREADS - 1) / SEL_THREADS;
    const int o0 = threadIdx.x * per;
    const int o1 = o0 + per < BK ? o0 + per : BK;
    const int hper = (nheads + hsplit - 1) / hsplit;
    const int hh_end = (hs + 1) * hper < nheads ? (hs + 1) * hper : nheads;
    for (int hh = hs * hper; hh < hh_end; hh++) {
        const int h = hgi * nheads + hh;
        const int32_t *lrow = left_out + (((int64_t)b * bs + i) * HEAD + h) * n;
        int64_t *irow = indices + (((int64_t)b * HEAD + h) * bdst + qb) * BK;
        // value of entry o: refined left edge aligned down to the block grid
        auto val = [&](int o) -> int64_t {
            int64_t v = lrow[s_sel[o]];
            return v / chunk * chunk;
        };
        int uniq = 0, act = 0;
        for (int o = o0; o < o1; o++) {
            const int64_t v = val(o);
            const int64_t prev = val(o == 0 ? BK - 1 : o - 1);  // roll(1): entry 0 is compared with the last
            if (v != prev) {
                uniq++;
                act += (v < limit);
            }
        }
        int tot_u, tot_a;
        int ubase = block_excl_scan(uniq, s_tmp, &tot_u);
        (void)block_excl_scan(act, s_tmp, &tot_a);
        for (int o = o0; o < o1; o++) {
            const int64_t v = val(o);
            const int64_t prev = val(o == 0 ? BK - 1 : o - 1);
            if (v != prev) irow[ubase++] = v;
        }
        for (int o = tot_u + threadIdx.x; o < BK; o += SEL_THREADS) irow[o] = 0x7fffffffffffffffLL;
        if (threadIdx.x == 0) {
            const int64_t r = ((int64_t)b * HEAD + h) * bdst + qb;
            ks[r] = tot_a;
            ks_start_end[r * 2 + 0] = 0;
            ks_start_end[r * 2 + 1] = tot_a;
        }
    }
}

// The same layout for launches of a few query blocks (decode), one workgroup of 1024 threads per (batch, query
// block, head): like select_stage_fast_kernel the selection runs on keys held in registers, the refined left edge of
// every entry is requested together with its scores, and the row is deduplicated from a list in LDS, so that the
// kernel makes two trips to memory.
template <int ITEMS>
__global__ __launch_bounds__(FAST_THREADS) void finalize_fast_kernel(const float *scores, const int32_t *left_out,
                                                                    const int64_t *pos, int64_t pos_sb, int64_t pos_st,
                                                                    int bs, int bdst, int scan_stride, int HEAD,
                                                                    int score_heads, int hg, int n, int K, int chunk,
                                                                    int bq, int64_t *indices, int64_t *ks,
                                                                    int32_t *ks_start_end) {
    __shared__ int s_hist[256];
    __shared__ int s_misc[2];
    __shared__ uint32_t s_wave[FAST_THREADS / 64];
    __shared__ int s_val[ITEMS * FAST_THREADS];  // block-aligned left edges of the selected entries in output order

    const int tid = threadIdx.x;
    const int nheads = HEAD / hg;
    const int hh = blockIdx.x % nheads;
    const int wg = blockIdx.x / nheads;
    const int hgi = wg % hg;
    const int qb = (wg / hg) % bdst;
    const int b = wg / (hg * bdst);
    const int i_in = (qb + scan_stride * bs - bdst) / scan_stride;
    const int nsh = score_heads / hg;
    const int BK = K < n ? K : n;
    const int h = hgi * nheads + hh;
    const float *srow = scores + (((int64_t)b * bs + i_in) * score_heads + (int64_t)hgi * nsh) * n;
    const int32_t *lrow = left_out + (((int64_t)b * bs + i_in) * HEAD + h) * n;
    int64_t *irow = indices + (((int64_t)b * HEAD + h) * bdst + qb) * BK;

    const int c0 = tid * ITEMS;
    const int64_t first_pos = pos[(int64_t)b * pos_sb + (int64_t)qb * bq * pos_st];
    int val[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; i++) val[i] = lrow[c0 + i < n ? c0 + i : n - 1];
    uint32_t key[ITEMS];
    bool plain_low;
    fast_load_keys<ITEMS>(srow, nsh, n, c0, key, &plain_low);
    const int64_t limit = first_pos + bq;

    uint32_t prefix = 0, mask = 0;
    int need = 0;
    if (BK < n) fast_threshold<ITEMS>(key, c0, n, BK, plain_low, s_hist, s_misc, &prefix, &mask, &need);
    int rank[ITEMS];
    fast_ranks<ITEMS>(key, c0, n, BK >= n, prefix, mask, need, s_wave, rank);
#pragma unroll
    for (int i = 0; i < ITEMS; i++)
        if (rank[i] >= 0) s_val[rank[i]] = val[i] / chunk * chunk;  // aligned down to the block grid
    __syncthreads();

    // entries o0 .. o0+ITEMS-1 of the selected list: an entry is kept when it differs from the one before it
    // (roll(1): entry 0 is compared with the last), and counts as active when it lies before the block's end
    const int o0 = tid * ITEMS;
    int v[ITEMS];
    uint32_t packed = 0;  // low half: kept entries, high half: active ones
    uint32_t keep = 0;
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
        const int o = o0 + i;
        v[i] = 0;
        if (o < BK) {
            v[i] = s_val[o];
            const int prev = s_val[o == 0 ? BK - 1 : o - 1];
            if (v[i] != prev) {
                keep |= 1u << i;
                packed += 1u + (((int64_t)v[i] < limit) ? 0x10000u : 0u);
            }
        }
    }
    uint32_t total;
    const uint32_t before = fast_excl_scan(packed, s_wave, &total);
    int at = (int)(before & 0xffffu);
    const int tot_u = (int)(total & 0xffffu), tot_a = (int)(total >> 16);
#pragma unroll
    for (int i = 0; i < ITEMS; i++)
        if ((keep >> i) & 1u) irow[at++] = v[i];
    for (int o = tot_u + tid; o < BK; o += FAST_THREADS) irow[o] = 0x7fffffffffffffffLL;
    if (tid == 0) {
        const int64_t r = ((int64_t)b * HEAD + h) * bdst + qb;
        ks[r] = tot_a;
        ks_start_end[r * 2 + 0] = 0;
        ks_start_end[r * 2 + 1] = tot_a;
    }
}

}  // namespace hipattn

using namespace hipattn;

extern "C" int hipattn_select_stage(const float *scores, const int32_t *chunk_left, int32_t B, int32_t bs_in,
                                    int32_t bs_out, int32_t row_rep, int32_t HEAD, int32_t hg, int32_t n,
                                    int32_t k, int32_t chunk_size, int32_t splits, int32_t *next_left,
                                    int64_t *next_left64, int64_t *next_right64, float *next_scores, void *stream) {
    HIPATTN_CHECK_ARG(scores && chunk_left && next_left, HIPATTN_E_ARG, "select stage: null pointer");
    HIPATTN_CHECK_ARG((next_left64 == nullptr) == (next_right64 == nullptr), HIPATTN_E_ARG,
                      "select stage: give both 64-bit outputs or neither");
    HIPATTN_CHECK_ARG(B > 0 && bs_in > 0 && bs_out > 0 && row_rep > 0 && HEAD > 0 && n > 0 && k > 0 && splits > 0,
                      HIPATTN_E_ARG, "select stage: non-positive size");
    HIPATTN_CHECK_ARG(hg == 1 || hg == HEAD, HIPATTN_E_ARG, "select stage: hg must be 1 or HEAD");
    HIPATTN_CHECK_ARG(!next_scores || hg == 1, HIPATTN_E_ARG, "select stage: next_scores needs one shared chunk list (hg == 1)");
    HIPATTN_CHECK_ARG(k <= n, HIPATTN_E_ARG, "select stage: k %d > n %d", k, n);
    HIPATTN_CHECK_ARG(chunk_size % splits == 0, HIPATTN_E_ARG, "select stage: chunk %d %% splits %d", chunk_size, splits);
    HIPATTN_CHECK_ARG(bs_out <= row_rep * bs_in, HIPATTN_E_ARG, "select stage: bs_out > row_rep*bs_in");
    HIPATTN_CHECK_ARG(n <= SEL_MAX_N, HIPATTN_E_UNSUPPORTED, "select stage: %d chunks exceed the limit %d", n, SEL_MAX_N);
    dim3 grid((unsigned)(B * bs_out * hg)), block(SEL_THREADS);
    // HIPATTN_SELECT_FAST=0 keeps the throughput kernel everywhere (read on every call: tests switch it in one process)
    const char *fast_env = getenv("HIPATTN_SELECT_FAST");
    const bool fast = !(fast_env && fast_env[0] == '0');
    if (fast && grid.x <= 64 && k <= FAST_MAX_K) {  // a few workgroups: the latency kernel
        dim3 fblock(FAST_THREADS);
#define SEL_FAST(IT)                                                                                                  \
    hipLaunchKernelGGL(select_stage_fast_kernel<IT>, grid, fblock, 0, (hipStream_t)stream, scores, chunk_left, bs_in, \
                       bs_out, row_rep, HEAD, hg, n, k, chunk_size / splits, splits, next_left, next_left64,          \
                       next_right64, next_scores)
        if (n <= FAST_THREADS) SEL_FAST(1);
        else if (n <= 4 * FAST_THREADS) SEL_FAST(4);
        else SEL_FAST(16);
#undef SEL_FAST
        HIPATTN_CHECK_HIP(hipGetLastError());
        return 0;
    }
    hipLaunchKernelGGL(select_stage_kernel, grid, block, 0, (hipStream_t)stream, scores, chunk_left, bs_in, bs_out,
                       row_rep, HEAD, hg, n, k, chunk_size / splits, splits, next_left, next_left64, next_right64,
                       next_scores);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

extern "C" int hipattn_finalize_indices(const float *scores, const int32_t *left_out, const int64_t *pos,
                                        int64_t pos_stride_b, int64_t pos_stride_t, int32_t B, int32_t bs,
                                        int32_t bdst, int32_t scan_stride, int32_t HEAD, int32_t score_heads,
                                        int32_t hg, int32_t n, int32_t K, int32_t chunk_size, int32_t bq,
                                        int64_t *indices, int64_t *ks, int32_t *ks_start_end, void *stream) {
    HIPATTN_CHECK_ARG(scores && left_out && pos && indices && ks && ks_start_end, HIPATTN_E_ARG,
                      "finalize: null pointer");
    HIPATTN_CHECK_ARG(B > 0 && bs > 0 && bdst > 0 && scan_stride > 0 && HEAD > 0 && n > 0 && K > 0 && chunk_size > 0 &&
                          bq > 0,
                      HIPATTN_E_ARG, "finalize: non-positive size");
    HIPATTN_CHECK_ARG(hg == 1 || hg == HEAD, HIPATTN_E_ARG, "finalize: hg must be 1 or HEAD");
    HIPATTN_CHECK_ARG(score_heads == HEAD || (score_heads == 1 && hg == 1), HIPATTN_E_ARG,
                      "finalize: score_heads must be HEAD, or 1 with hg == 1");
    HIPATTN_CHECK_ARG(bdst <= scan_stride * bs, HIPATTN_E_ARG, "finalize: bdst > scan_stride*bs");
    HIPATTN_CHECK_ARG(n <= SEL_MAX_N, HIPATTN_E_UNSUPPORTED, "finalize: %d chunks exceed the limit %d", n, SEL_MAX_N);
    const long long groups = (long long)B * bdst * hg;
    const int nheads = HEAD / hg;
    // HIPATTN_SELECT_FAST=0 keeps the throughput kernel everywhere (read on every call: tests switch it in one process)
    const char *fast_env = getenv("HIPATTN_SELECT_FAST");
    const bool fast = !(fast_env && fast_env[0] == '0');
    if (fast && groups * nheads <= 1024 && n <= 4 * FAST_THREADS) {  // few query blocks (decode): the latency kernel
        dim3 fgrid((unsigned)(groups * nheads)), fblock(FAST_THREADS);
#define FIN_FAST(IT)                                                                                                  \
    hipLaunchKernelGGL(finalize_fast_kernel<IT>, fgrid, fblock, 0, (hipStream_t)stream, scores, left_out, pos,        \
                       pos_stride_b, pos_stride_t, bs, bdst, scan_stride, HEAD, score_heads, hg, n, K, chunk_size, bq, \
                       indices, ks, ks_start_end)
        if (n <= FAST_THREADS) FIN_FAST(1);
        else FIN_FAST(4);
#undef FIN_FAST
        HIPATTN_CHECK_HIP(hipGetLastError());
        return 0;
    }
    // otherwise slice each group's heads over several workgroups while the launch is small
    int hsplit = 1;
    while (hsplit < nheads && groups * hsplit < 512) hsplit *= 2;
    if (hsplit > nheads) hsplit = nheads;
    dim3 grid((unsigned)(groups * hsplit)), block(SEL_THREADS);
    hipLaunchKernelGGL(finalize_kernel, grid, block, 0, (hipStream_t)stream, scores, left_out, pos, pos_stride_b,
                       pos_stride_t, bs, bdst, scan_stride, HEAD, score_heads, hg, hsplit, n, K, chunk_size, bq, indices,
                       ks, ks_start_end);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

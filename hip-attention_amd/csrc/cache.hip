// Block cache in device memory in front of K/V pools that live in pinned host memory.
//
// Stands in for GPUCache / HiPOffloadCache of the reference (src/hip_attn/v1_2/uvm_gpu_cache.py:204-566,
// 569-700): a (kv head, block) -> slot table consulted by every key/value row load, least-recently-used
// replacement by last-access step, misses recorded by the readers and brought in afterwards.  Everything
// here runs on the device and is stream-ordered: no host round trip decides what is fetched or evicted.
//
// Replacement is exact and deterministic: the blocks flagged as missed are taken in ascending
// (head, block) order, the victims are the slots with the smallest (last-use step, slot id); the i-th
// flagged block goes to the i-th victim in ascending slot order.  A 4-pass byte-wise radix select over the
// last-use steps finds the eviction threshold; prefix sums over 2048-entry tiles place both lists.
#include <string.h>

#include <new>

#include <stdlib.h>

#include "common.hpp"

struct hipattn_cache {
    hipattn_cache_desc_t d;
    int64_t n_blocks;
    int64_t max_fetch;
    int shift, esz;
    int64_t flag_entries;  // HKV * n_blocks
    int tiles_flags, tiles_slots;
    // carved out of d.workspace
    int32_t *step;
    int64_t *stats;
    int32_t *ctl;
    int32_t *hist;
    int32_t *tile_miss, *tile_lt, *tile_eq;
    int32_t *miss_list, *victim_list;
};

namespace hipattn {

constexpr int CT_THREADS = 256;
constexpr int CT_PER = 8;
constexpr int CT_TILE = CT_THREADS * CT_PER;

// ctl words
enum { C_NMISS = 0, C_HITS = 1, C_M = 2, C_T = 3, C_NEQ = 4, C_EVICTED = 5, C_WORDS = 16 };

struct CacheDev {
    int32_t *table;
    int32_t *last_use;
    int32_t *backref;
    uint8_t *miss;
    int32_t *step;
    int64_t *stats;
    int32_t *ctl;
    int32_t *hist;  // [4][256], most significant byte first
    int32_t *tile_miss, *tile_lt, *tile_eq;
    int32_t *miss_list, *victim_list;
    int64_t slots, n_blocks, flag_entries, max_fetch, pool_rows;
    int tiles_flags, tiles_slots;
    // copy geometry
    const char *host_k, *host_v;
    char *bank;
    int64_t host_stride_row_b, host_stride_h_b;  // bytes
    int64_t slot_bytes, row_bytes;
    int block_tokens, shift, with_v;
};

static CacheDev dev_of(const hipattn_cache *c) {
    CacheDev v;
    v.table = c->d.table; v.last_use = c->d.last_use; v.backref = c->d.backref; v.miss = c->d.miss;
    v.step = c->step; v.stats = c->stats; v.ctl = c->ctl; v.hist = c->hist;
    v.tile_miss = c->tile_miss; v.tile_lt = c->tile_lt; v.tile_eq = c->tile_eq;
    v.miss_list = c->miss_list; v.victim_list = c->victim_list;
    v.slots = c->d.slots; v.n_blocks = c->n_blocks; v.flag_entries = c->flag_entries; v.max_fetch = c->max_fetch;
    v.pool_rows = c->d.pool_rows;
    v.tiles_flags = c->tiles_flags; v.tiles_slots = c->tiles_slots;
    v.host_k = (const char *)c->d.host_k; v.host_v = (const char *)c->d.host_v; v.bank = (char *)c->d.bank;
    v.host_stride_row_b = c->d.host_stride_row * c->esz; v.host_stride_h_b = c->d.host_stride_h * c->esz;
    v.row_bytes = (int64_t)c->d.HID * c->esz;
    v.slot_bytes = v.row_bytes * c->d.block_tokens * (1 + c->d.with_v);
    v.block_tokens = c->d.block_tokens; v.shift = c->shift; v.with_v = c->d.with_v;
    return v;
}

// last-use step -> radix key: never-used slots (step -1) sort first
__device__ __forceinline__ uint32_t key_of(int32_t last_use) { return (uint32_t)(last_use + 1); }

// exclusive prefix sum over the 256 threads of a workgroup; *total = sum.  `lds` holds 8 ints.
__device__ __forceinline__ int block_excl_scan(int v, int *total, int *lds) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    int incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(incl, o);
        if (lane >= o) incl += up;
    }
    __syncthreads();  // protect lds from the previous use
    if (lane == 63) lds[wid] = incl;
    __syncthreads();
    int base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < CT_THREADS / 64; w++) {
        const int s = lds[w];
        if (w < wid) base += s;
        tot += s;
    }
    *total = tot;
    return base + incl - v;
}

// how many blocks this commit moves: flagged, bounded by max_fetch and by the slots not used in this step
__device__ __forceinline__ int fetch_count(const CacheDev &c) {
    long long m = c.ctl[C_NMISS];
    if (m > c.max_fetch) m = c.max_fetch;
    const long long free_slots = c.slots - c.ctl[C_HITS];
    if (m > free_slots) m = free_slots;
    return (int)(m < 0 ? 0 : m);
}

// Radix select, run by the first wave of a workgroup: walks the finished histogram passes and returns the
// key prefix chosen so far and how many keys are still to be taken inside that prefix.
__device__ __forceinline__ void pick_chain(const CacheDev &c, int passes, int m, uint32_t *prefix_out, int *rem_out) {
    const int lane = threadIdx.x & 63;
    uint32_t prefix = 0;
    int rem = m;
    for (int p = 0; p < passes; p++) {
        const int4 h = *reinterpret_cast<const int4 *>(c.hist + p * 256 + lane * 4);
        const int mine = h.x + h.y + h.z + h.w;
        int incl = mine;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int up = __shfl_up(incl, o);
            if (lane >= o) incl += up;
        }
        const int excl = incl - mine;
        // the lane whose bins contain the rem-th smallest key
        const bool here = excl < rem && rem <= incl;
        int digit = 0, below = 0;
        if (here) {
            const int hv[4] = {h.x, h.y, h.z, h.w};
            int acc = excl, found = -1, b4 = excl;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (found < 0 && acc + hv[j] >= rem) {
                    found = j;
                    b4 = acc;
                }
                acc += hv[j];
            }
            digit = lane * 4 + found;
            below = b4;
        }
        const unsigned long long who = __ballot(here);
        const int src = who ? (int)__builtin_ctzll(who) : 0;
        digit = __shfl(digit, src);
        below = __shfl(below, src);
        prefix = (prefix << 8) | (uint32_t)digit;
        rem -= below;
    }
    *prefix_out = prefix;
    *rem_out = rem;
}

__global__ void cache_fill_kernel(int32_t *p, long long n, int32_t value) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = value;
}
__global__ void cache_fill8_kernel(uint8_t *p, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

__global__ void cache_begin_kernel(CacheDev c) {
    for (int i = threadIdx.x; i < C_WORDS + 4 * 256; i += blockDim.x) {
        if (i < C_WORDS) c.ctl[i] = 0;
        else c.hist[i - C_WORDS] = 0;
    }
}

// pass 0: per-tile count of flagged blocks, hits of this step, histogram of the top key byte
__global__ __launch_bounds__(CT_THREADS) void cache_scan_kernel(CacheDev c) {
    __shared__ int lds[8];
    __shared__ int hist[256];
    const int tile = blockIdx.x;
    hist[threadIdx.x] = 0;
    __syncthreads();
    if (tile < c.tiles_flags) {
        const long long base = (long long)tile * CT_TILE + threadIdx.x * CT_PER;
        int cnt = 0;
#pragma unroll
        for (int j = 0; j < CT_PER; j++)
            if (base + j < c.flag_entries && c.miss[base + j]) cnt++;
        int total;
        block_excl_scan(cnt, &total, lds);
        if (threadIdx.x == 0) {
            c.tile_miss[tile] = total;
            if (total) atomicAdd(c.ctl + C_NMISS, total);
        }
    }
    if (tile < c.tiles_slots) {
        const int now = *c.step;
        const long long base = (long long)tile * CT_TILE + threadIdx.x * CT_PER;
        int hits = 0;
#pragma unroll
        for (int j = 0; j < CT_PER; j++) {
            if (base + j < c.slots) {
                const int32_t lu = c.last_use[base + j];
                if (lu == now) hits++;
                atomicAdd(&hist[key_of(lu) >> 24], 1);
            }
        }
        int total;
        block_excl_scan(hits, &total, lds);
        if (threadIdx.x == 0 && total) atomicAdd(c.ctl + C_HITS, total);
        __syncthreads();
        const int h = hist[threadIdx.x];
        if (h) atomicAdd(c.hist + threadIdx.x, h);
    }
}

// passes 1..3: histogram of the next key byte among the slots that match the prefix chosen so far
__global__ __launch_bounds__(CT_THREADS) void cache_hist_kernel(CacheDev c, int pass) {
    __shared__ int hist[256];
    __shared__ uint32_t s_prefix;
    __shared__ int s_m;
    hist[threadIdx.x] = 0;
    if (threadIdx.x < 64) {
        const int m = fetch_count(c);
        uint32_t prefix = 0;
        int rem = 0;
        if (m > 0) pick_chain(c, pass, m, &prefix, &rem);
        if (threadIdx.x == 0) {
            s_prefix = prefix;
            s_m = m;
        }
    }
    __syncthreads();
    if (s_m == 0) return;
    const uint32_t prefix = s_prefix;
    const int hi_shift = 8 * (4 - pass), lo_shift = 8 * (3 - pass);
    const long long base = (long long)blockIdx.x * CT_TILE + threadIdx.x * CT_PER;
#pragma unroll
    for (int j = 0; j < CT_PER; j++) {
        if (base + j < c.slots) {
            const uint32_t key = key_of(c.last_use[base + j]);
            if ((key >> hi_shift) == prefix) atomicAdd(&hist[(key >> lo_shift) & 255u], 1);
        }
    }
    __syncthreads();
    const int h = hist[threadIdx.x];
    if (h) atomicAdd(c.hist + pass * 256 + threadIdx.x, h);
}

// per-tile counts of slots below / at the eviction threshold
__global__ __launch_bounds__(CT_THREADS) void cache_tiles_kernel(CacheDev c) {
    __shared__ int lds[8];
    __shared__ uint32_t s_T;
    __shared__ int s_m, s_neq;
    if (threadIdx.x < 64) {
        const int m = fetch_count(c);
        uint32_t T = 0;
        int neq = 0;
        if (m > 0) pick_chain(c, 4, m, &T, &neq);
        if (threadIdx.x == 0) {
            s_T = T;
            s_m = m;
            s_neq = neq;
        }
    }
    __syncthreads();
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        c.ctl[C_M] = s_m;
        c.ctl[C_T] = (int32_t)s_T;
        c.ctl[C_NEQ] = s_neq;
    }
    const uint32_t T = s_T;
    const bool any = s_m > 0;
    const long long base = (long long)blockIdx.x * CT_TILE + threadIdx.x * CT_PER;
    int lt = 0, eq = 0;
    if (any) {
#pragma unroll
        for (int j = 0; j < CT_PER; j++) {
            if (base + j < c.slots) {
                const uint32_t key = key_of(c.last_use[base + j]);
                lt += key < T;
                eq += key == T;
            }
        }
    }
    int tot_lt, tot_eq;
    block_excl_scan(lt, &tot_lt, lds);
    block_excl_scan(eq, &tot_eq, lds);
    if (threadIdx.x == 0) {
        c.tile_lt[blockIdx.x] = tot_lt;
        c.tile_eq[blockIdx.x] = tot_eq;
    }
}

// one workgroup: exclusive prefix sums over the tile counts, in place
__global__ __launch_bounds__(CT_THREADS) void cache_scan_tiles_kernel(CacheDev c) {
    __shared__ int lds[8];
    int32_t *arrs[3] = {c.tile_miss, c.tile_lt, c.tile_eq};
    const int lens[3] = {c.tiles_flags, c.tiles_slots, c.tiles_slots};
    for (int a = 0; a < 3; a++) {
        int carry = 0;
        for (int base = 0; base < lens[a]; base += CT_THREADS) {
            const int i = base + threadIdx.x;
            const int v = i < lens[a] ? arrs[a][i] : 0;
            int total;
            const int ex = block_excl_scan(v, &total, lds);
            if (i < lens[a]) arrs[a][i] = carry + ex;
            carry += total;
        }
    }
}

// writes the two lists and clears the miss flags
__global__ __launch_bounds__(CT_THREADS) void cache_emit_kernel(CacheDev c) {
    __shared__ int lds[8];
    const int tile = blockIdx.x;
    const int m = c.ctl[C_M];
    const long long base = (long long)tile * CT_TILE + threadIdx.x * CT_PER;
    if (tile < c.tiles_flags) {
        int cnt = 0;
        bool f[CT_PER];
#pragma unroll
        for (int j = 0; j < CT_PER; j++) {
            f[j] = base + j < c.flag_entries && c.miss[base + j];
            cnt += f[j];
        }
        int total;
        int pos = c.tile_miss[tile] + block_excl_scan(cnt, &total, lds);
#pragma unroll
        for (int j = 0; j < CT_PER; j++) {
            if (f[j]) {
                if (pos < m) c.miss_list[pos] = (int32_t)(base + j);
                pos++;
                c.miss[base + j] = 0;
            }
        }
    }
    if (tile < c.tiles_slots && m > 0) {
        const uint32_t T = (uint32_t)c.ctl[C_T];
        const int neq = c.ctl[C_NEQ];
        int lt = 0, eq = 0;
        uint32_t keys[CT_PER];
#pragma unroll
        for (int j = 0; j < CT_PER; j++) {
            keys[j] = base + j < c.slots ? key_of(c.last_use[base + j]) : 0xffffffffu;
            const bool in = base + j < c.slots;
            lt += in && keys[j] < T;
            eq += in && keys[j] == T;
        }
        int total;
        int lt_lower = c.tile_lt[tile] + block_excl_scan(lt, &total, lds);
        int eq_lower = c.tile_eq[tile] + block_excl_scan(eq, &total, lds);
#pragma unroll
        for (int j = 0; j < CT_PER; j++) {
            if (base + j >= c.slots) continue;
            if (keys[j] < T) {
                c.victim_list[lt_lower + min(eq_lower, neq)] = (int32_t)(base + j);
                lt_lower++;
            } else if (keys[j] == T) {
                if (eq_lower < neq) c.victim_list[lt_lower + eq_lower] = (int32_t)(base + j);
                eq_lower++;
            }
        }
    }
}

// a workgroup per fetched block (grid-stride over the list): unlink the victim, copy host -> bank, link
__global__ __launch_bounds__(CT_THREADS) void cache_fetch_kernel(CacheDev c) {
    const int m = c.ctl[C_M];
    const int pieces_per_row = (int)(c.row_bytes / 16);
    const int total = c.block_tokens * pieces_per_row * (1 + c.with_v);
    for (int i = blockIdx.x; i < m; i += gridDim.x) {
        const int32_t e = c.miss_list[i];
        const int32_t slot = c.victim_list[i];
        const int64_t h = e / c.n_blocks, blk = e % c.n_blocks;
        char *dst = c.bank + (int64_t)slot * c.slot_bytes;
        // four 16-byte pieces per thread in flight before the first is stored: the few workgroups of this kernel have
        // to cover the latency of the host link with their own loads
        for (int w0 = threadIdx.x; w0 < total; w0 += 4 * CT_THREADS) {
            uint4 val[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int w = w0 + u * CT_THREADS;
                val[u] = make_uint4(0, 0, 0, 0);
                if (w < total) {
                    const int part = w / (c.block_tokens * pieces_per_row);
                    const int r = (w / pieces_per_row) % c.block_tokens;
                    const int piece = w % pieces_per_row;
                    const int64_t row = (blk << c.shift) + r;
                    if (row < c.pool_rows) {
                        const char *src = (part ? c.host_v : c.host_k) + row * c.host_stride_row_b + h * c.host_stride_h_b;
                        val[u] = *reinterpret_cast<const uint4 *>(src + piece * 16);
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int w = w0 + u * CT_THREADS;
                if (w < total) {
                    const int part = w / (c.block_tokens * pieces_per_row);
                    const int r = (w / pieces_per_row) % c.block_tokens;
                    const int piece = w % pieces_per_row;
                    *reinterpret_cast<uint4 *>(dst + ((int64_t)part * c.block_tokens + r) * c.row_bytes + piece * 16) = val[u];
                }
            }
        }
        if (threadIdx.x == 0) {
            const int32_t old = c.backref[slot];
            if (old >= 0) {
                c.table[old] = -1;
                atomicAdd(c.ctl + C_EVICTED, 1);
            }
            c.backref[slot] = e;
            c.table[e] = slot;
            c.last_use[slot] = *c.step;
        }
    }
}

__global__ void cache_step_kernel(CacheDev c) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const int hits = c.ctl[C_HITS], nmiss = c.ctl[C_NMISS], m = c.ctl[C_M], ev = c.ctl[C_EVICTED];
    c.stats[0] += 1;
    c.stats[1] += hits;
    c.stats[2] += nmiss;
    c.stats[3] += m;
    c.stats[4] += ev;
    c.stats[5] = hits;
    c.stats[6] = nmiss;
    c.stats[7] = m;
    *c.step = *c.step + 1;
    // a second commit without a new schedule moves nothing
    c.ctl[C_M] = 0;
    c.ctl[C_HITS] = 0;
    c.ctl[C_NMISS] = 0;
    c.ctl[C_EVICTED] = 0;
}

// resident blocks receive the freshly written rows
__global__ __launch_bounds__(CT_THREADS) void cache_write_rows_kernel(CacheDev c, const int64_t *rows, int64_t n, int HKV,
                                                                      const char *k_rows, const char *v_rows) {
    const int pieces_per_row = (int)(c.row_bytes / 16);
    const int64_t total = n * HKV * pieces_per_row;
    const int64_t w = (int64_t)blockIdx.x * CT_THREADS + threadIdx.x;
    if (w >= total) return;
    const int piece = (int)(w % pieces_per_row);
    const int h = (int)((w / pieces_per_row) % HKV);
    const int64_t i = w / ((int64_t)pieces_per_row * HKV);
    const int64_t row = rows[i];
    if (row < 0 || row >= c.pool_rows) return;
    const int32_t slot = c.table[(int64_t)h * c.n_blocks + (row >> c.shift)];
    if (slot < 0) return;
    const int r = (int)(row & (c.block_tokens - 1));
    char *dst = c.bank + (int64_t)slot * c.slot_bytes + (int64_t)r * c.row_bytes + piece * 16;
    const int64_t src = (i * HKV + h) * c.row_bytes + piece * 16;
    *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(k_rows + src);
    if (c.with_v)
        *reinterpret_cast<uint4 *>(dst + (int64_t)c.block_tokens * c.row_bytes) =
            *reinterpret_cast<const uint4 *>(v_rows + src);
}

__global__ void pool_write_rows_kernel(char *pool, int64_t stride_row_b, int64_t stride_h_b, int HKV, int row_bytes,
                                       const int64_t *rows, int64_t n, const char *src) {
    const int pieces = row_bytes / 16;
    const int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (w >= n * HKV * pieces) return;
    const int piece = (int)(w % pieces);
    const int h = (int)((w / pieces) % HKV);
    const int64_t i = w / ((int64_t)pieces * HKV);
    const int64_t row = rows[i];
    if (row < 0) return;
    *reinterpret_cast<uint4 *>(pool + row * stride_row_b + h * stride_h_b + piece * 16) =
        *reinterpret_cast<const uint4 *>(src + (i * HKV + h) * (int64_t)row_bytes + piece * 16);
}

// gather: dst[i, h, :] = pool[rows[i], h, :]; rows below zero give zero rows
__global__ void pool_read_rows_kernel(const char *pool, int64_t stride_row_b, int64_t stride_h_b, int HKV, int row_bytes,
                                      const int64_t *rows, int64_t n, char *dst, int64_t dst_row_b) {
    const int pieces = row_bytes / 16;
    const int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (w >= n * HKV * pieces) return;
    const int piece = (int)(w % pieces);
    const int h = (int)((w / pieces) % HKV);
    const int64_t i = w / ((int64_t)pieces * HKV);
    const int64_t row = rows[i];
    uint4 v = make_uint4(0, 0, 0, 0);
    if (row >= 0) v = *reinterpret_cast<const uint4 *>(pool + row * stride_row_b + h * stride_h_b + piece * 16);
    *reinterpret_cast<uint4 *>(dst + i * dst_row_b + (int64_t)h * row_bytes + piece * 16) = v;
}

// bytes per stored element; 0 for a dtype code that is not a storage format
static int storage_esz(int dtype) {
    return dtype == HIPATTN_F32 ? 4 : dtype == HIPATTN_BF16 ? 2 : dtype == HIPATTN_FP8_E5M2 ? 1 : 0;
}

static int tiles_of(int64_t n) { return (int)((n + CT_TILE - 1) / CT_TILE); }

static int check_desc(const hipattn_cache_desc_t *d, int64_t max_fetch, int *shift_out) {
    HIPATTN_CHECK_ARG(d, HIPATTN_E_ARG, "cache: null descriptor");
    HIPATTN_CHECK_ARG(storage_esz(d->dtype) > 0, HIPATTN_E_UNSUPPORTED, "cache: dtype %d", d->dtype);
    HIPATTN_CHECK_ARG(d->HKV > 0 && d->HID > 0 && d->pool_rows > 0 && d->slots > 0 && max_fetch > 0, HIPATTN_E_ARG,
                      "cache: non-positive size");
    int shift = -1;
    for (int s = 0; s <= 6; s++)
        if (d->block_tokens == (1 << s)) shift = s;
    HIPATTN_CHECK_ARG(shift >= 0, HIPATTN_E_ARG, "cache: block_tokens %d is not a power of two in 1..64", d->block_tokens);
    const int esz = storage_esz(d->dtype);
    HIPATTN_CHECK_ARG(((int64_t)d->HID * esz) % 16 == 0, HIPATTN_E_ALIGN, "cache: rows must be whole 16-byte packs");
    const int64_t n_blocks = (d->pool_rows + d->block_tokens - 1) / d->block_tokens;
    HIPATTN_CHECK_ARG(n_blocks * d->HKV < 0x7fffffffLL && d->slots < 0x7fffffffLL && max_fetch < 0x7fffffffLL,
                      HIPATTN_E_UNSUPPORTED, "cache: more than 2^31 blocks or slots");
    *shift_out = shift;
    return 0;
}

static int64_t align_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

struct WsLayout {
    int64_t step, stats, ctl, hist, tile_miss, tile_lt, tile_eq, miss_list, victim_list, total;
};

static WsLayout ws_layout(int tiles_flags, int tiles_slots, int64_t max_fetch) {
    WsLayout w;
    int64_t o = 0;
    w.step = o; o += 256;
    w.stats = o; o += 256;
    w.ctl = o; o += 256;
    w.hist = o; o += 4 * 256 * 4;
    w.tile_miss = o; o += align_up((int64_t)tiles_flags * 4, 256);
    w.tile_lt = o; o += align_up((int64_t)tiles_slots * 4, 256);
    w.tile_eq = o; o += align_up((int64_t)tiles_slots * 4, 256);
    w.miss_list = o; o += align_up(max_fetch * 4, 256);
    w.victim_list = o; o += align_up(max_fetch * 4, 256);
    w.total = o;
    return w;
}

static int launch_fill(int32_t *p, int64_t n, int32_t value, hipStream_t st) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(cache_fill_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, p, (long long)n, value);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

int cache_view_for(const hipattn_cache *c, const hipattn_kv_t *kv, const KVView *o, int HID, int dtype, KVExt *x) {
    HIPATTN_CHECK_ARG(kv->paged, HIPATTN_E_ARG, "kv: an offload cache needs the paged view");
    const int stored = kv->fp8 ? HIPATTN_FP8_E5M2 : dtype;
    HIPATTN_CHECK_ARG(c->d.dtype == stored && c->d.HID == HID && c->d.HKV == kv->HKV, HIPATTN_E_ARG,
                      "kv: cache was built for dtype %d, head dim %d, %d kv heads", c->d.dtype, c->d.HID, c->d.HKV);
    HIPATTN_CHECK_ARG(kv->k == c->d.host_k && (!c->d.with_v || !kv->v || kv->v == c->d.host_v), HIPATTN_E_ARG,
                      "kv: K/V pointers differ from the pools the cache was built over");
    const int ps = kv->page_size ? kv->page_size : 1;
    HIPATTN_CHECK_ARG(kv->k_stride_t == c->d.host_stride_row && kv->k_stride_b == c->d.host_stride_row * ps &&
                          kv->k_stride_h == c->d.host_stride_h,
                      HIPATTN_E_ARG, "kv: paged strides do not describe the pool the cache was built over");
    x->cached = 1;
    CacheView &v = x->cache;
    v.table = c->d.table;
    v.last_use = c->d.last_use;
    v.miss = c->d.miss;
    v.step = c->step;
    const int64_t part = (int64_t)c->d.block_tokens * c->d.HID;
    v.k_delta = ((const char *)c->d.bank - (const char *)kv->k) / c->esz;
    v.v_delta = c->d.with_v ? ((const char *)c->d.bank - (const char *)o->v) / c->esz + part : 0;
    v.slot_stride = part * (1 + c->d.with_v);
    v.n_blocks = c->n_blocks;
    v.shift = c->shift;
    v.row_elems = c->d.HID;
    v.with_v = c->d.with_v;
    return 0;
}

}  // namespace hipattn

using namespace hipattn;

extern "C" int hipattn_cache_sizes(const hipattn_cache_desc_t *d, int64_t max_fetch, hipattn_cache_sizes_t *out) {
    int shift;
    int rc = check_desc(d, max_fetch, &shift);
    if (rc) return rc;
    HIPATTN_CHECK_ARG(out, HIPATTN_E_ARG, "cache: null output");
    const int esz = storage_esz(d->dtype);
    const int64_t n_blocks = (d->pool_rows + d->block_tokens - 1) / d->block_tokens;
    out->n_blocks = n_blocks;
    out->bank_bytes = d->slots * (1 + (d->with_v ? 1 : 0)) * d->block_tokens * (int64_t)d->HID * esz;
    out->table_bytes = n_blocks * d->HKV * 4;
    out->last_use_bytes = d->slots * 4;
    out->backref_bytes = d->slots * 4;
    out->miss_bytes = n_blocks * d->HKV;
    out->workspace_bytes = ws_layout(tiles_of(n_blocks * d->HKV), tiles_of(d->slots), max_fetch).total;
    return 0;
}

extern "C" int hipattn_cache_create(const hipattn_cache_desc_t *d, int64_t max_fetch, hipattn_cache_t **out,
                                    void *stream) {
    int shift;
    int rc = check_desc(d, max_fetch, &shift);
    if (rc) return rc;
    HIPATTN_CHECK_ARG(out, HIPATTN_E_ARG, "cache: null output");
    HIPATTN_CHECK_ARG(d->host_k && d->bank && d->table && d->last_use && d->backref && d->miss && d->workspace &&
                          (!d->with_v || d->host_v),
                      HIPATTN_E_ARG, "cache: null buffer");
    const int esz = storage_esz(d->dtype);
    const int64_t al = 16 / esz;
    HIPATTN_CHECK_ARG(aligned16(d->host_k) && aligned16(d->host_v) && aligned16(d->bank) && aligned16(d->workspace) &&
                          d->host_stride_row % al == 0 && d->host_stride_h % al == 0,
                      HIPATTN_E_ALIGN, "cache: pools, bank and workspace must be 16-byte aligned");
    hipattn_cache *c = new (std::nothrow) hipattn_cache;
    HIPATTN_CHECK_ARG(c, HIPATTN_E_ARG, "cache: out of host memory");
    c->d = *d;
    c->d.with_v = d->with_v ? 1 : 0;
    c->shift = shift;
    c->esz = esz;
    c->n_blocks = (d->pool_rows + d->block_tokens - 1) / d->block_tokens;
    c->max_fetch = max_fetch;
    c->flag_entries = c->n_blocks * d->HKV;
    c->tiles_flags = tiles_of(c->flag_entries);
    c->tiles_slots = tiles_of(d->slots);
    const WsLayout w = ws_layout(c->tiles_flags, c->tiles_slots, max_fetch);
    char *ws = (char *)d->workspace;
    c->step = (int32_t *)(ws + w.step);
    c->stats = (int64_t *)(ws + w.stats);
    c->ctl = (int32_t *)(ws + w.ctl);
    c->hist = (int32_t *)(ws + w.hist);
    c->tile_miss = (int32_t *)(ws + w.tile_miss);
    c->tile_lt = (int32_t *)(ws + w.tile_lt);
    c->tile_eq = (int32_t *)(ws + w.tile_eq);
    c->miss_list = (int32_t *)(ws + w.miss_list);
    c->victim_list = (int32_t *)(ws + w.victim_list);
    rc = launch_fill((int32_t *)ws, (256 * 3) / 4, 0, (hipStream_t)stream);  // step, stats, ctl
    if (!rc) rc = hipattn_cache_flush(c, stream);
    if (rc) {
        delete c;
        return rc;
    }
    *out = c;
    return 0;
}

extern "C" void hipattn_cache_destroy(hipattn_cache_t *cache) { delete cache; }

extern "C" int hipattn_cache_flush(hipattn_cache_t *c, void *stream) {
    HIPATTN_CHECK_ARG(c, HIPATTN_E_ARG, "cache: null handle");
    hipStream_t st = (hipStream_t)stream;
    int rc = launch_fill(c->d.table, c->flag_entries, -1, st);
    if (!rc) rc = launch_fill(c->d.last_use, c->d.slots, -1, st);
    if (!rc) rc = launch_fill(c->d.backref, c->d.slots, -1, st);
    if (rc) return rc;
    hipLaunchKernelGGL(cache_fill8_kernel, dim3((unsigned)((c->flag_entries + 255) / 256)), dim3(256), 0, st, c->d.miss,
                       (long long)c->flag_entries);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

extern "C" int hipattn_cache_lookup_and_schedule(hipattn_cache_t *c, void *stream) {
    HIPATTN_CHECK_ARG(c, HIPATTN_E_ARG, "cache: null handle");
    hipStream_t st = (hipStream_t)stream;
    const CacheDev v = dev_of(c);
    const int tiles = c->tiles_flags > c->tiles_slots ? c->tiles_flags : c->tiles_slots;
    hipLaunchKernelGGL(cache_begin_kernel, dim3(1), dim3(256), 0, st, v);
    hipLaunchKernelGGL(cache_scan_kernel, dim3(tiles), dim3(CT_THREADS), 0, st, v);
    for (int pass = 1; pass < 4; pass++)
        hipLaunchKernelGGL(cache_hist_kernel, dim3(c->tiles_slots), dim3(CT_THREADS), 0, st, v, pass);
    hipLaunchKernelGGL(cache_tiles_kernel, dim3(c->tiles_slots), dim3(CT_THREADS), 0, st, v);
    hipLaunchKernelGGL(cache_scan_tiles_kernel, dim3(1), dim3(CT_THREADS), 0, st, v);
    hipLaunchKernelGGL(cache_emit_kernel, dim3(tiles), dim3(CT_THREADS), 0, st, v);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

extern "C" int hipattn_cache_commit(hipattn_cache_t *c, void *stream) {
    HIPATTN_CHECK_ARG(c, HIPATTN_E_ARG, "cache: null handle");
    hipStream_t st = (hipStream_t)stream;
    const CacheDev v = dev_of(c);
    // A bounded grid walks the fetch list: how many blocks there are is only known on the device.  Two workgroups
    // per compute unit keep far more bytes in flight than the host link needs (4 MB against a few hundred KB) and
    // leave the wave slots of the chip to whatever runs beside the fetch on another stream; a grid that fills every
    // slot with waves waiting on the host link starves those kernels (measured: no overlap at all with 4096).
    static int env_grid = -1;
    if (env_grid < 0) {
        const char *e = getenv("HIPATTN_CACHE_FETCH_GRID");  // tuning aid
        env_grid = e ? atoi(e) : 0;
    }
    const long long want = env_grid > 0 ? env_grid : 64;
    const unsigned fetch_grid = (unsigned)(c->max_fetch < want ? c->max_fetch : want);
    hipLaunchKernelGGL(cache_fetch_kernel, dim3(fetch_grid), dim3(CT_THREADS), 0, st, v);
    hipLaunchKernelGGL(cache_step_kernel, dim3(1), dim3(64), 0, st, v);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

extern "C" int hipattn_cache_write_rows(hipattn_cache_t *c, const int64_t *rows, int64_t n, const void *k_rows,
                                        const void *v_rows, void *stream) {
    HIPATTN_CHECK_ARG(c, HIPATTN_E_ARG, "cache: null handle");
    if (n == 0) return 0;
    HIPATTN_CHECK_ARG(rows && k_rows && n > 0 && (!c->d.with_v || v_rows), HIPATTN_E_ARG, "cache write: null pointer");
    HIPATTN_CHECK_ARG(aligned16(k_rows) && aligned16(v_rows), HIPATTN_E_ALIGN, "cache write: rows must be 16-byte aligned");
    const CacheDev v = dev_of(c);
    const int64_t total = n * c->d.HKV * (v.row_bytes / 16);
    const int64_t blocks = (total + CT_THREADS - 1) / CT_THREADS;
    HIPATTN_CHECK_ARG(blocks < 0x7fffffffLL, HIPATTN_E_UNSUPPORTED, "cache write: too many rows");
    hipLaunchKernelGGL(cache_write_rows_kernel, dim3((unsigned)blocks), dim3(CT_THREADS), 0, (hipStream_t)stream, v, rows,
                       n, c->d.HKV, (const char *)k_rows, (const char *)v_rows);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

extern "C" int hipattn_cache_stats(hipattn_cache_t *c, int64_t out[8], void *stream) {
    HIPATTN_CHECK_ARG(c && out, HIPATTN_E_ARG, "cache: null pointer");
    HIPATTN_CHECK_HIP(hipMemcpyAsync(out, c->stats, 8 * sizeof(int64_t), hipMemcpyDeviceToHost, (hipStream_t)stream));
    HIPATTN_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

extern "C" int hipattn_pool_write_rows(void *pool, int64_t stride_row, int64_t stride_h, int32_t HKV, int32_t HID,
                                       int32_t dtype, const int64_t *rows, int64_t n, const void *src, void *stream) {
    if (n == 0) return 0;
    HIPATTN_CHECK_ARG(pool && rows && src && n > 0 && HKV > 0 && HID > 0, HIPATTN_E_ARG, "pool write: bad argument");
    HIPATTN_CHECK_ARG(storage_esz(dtype) > 0, HIPATTN_E_UNSUPPORTED, "pool write: dtype %d", dtype);
    const int esz = storage_esz(dtype);
    HIPATTN_CHECK_ARG(aligned16(pool) && aligned16(src) && (stride_row * esz) % 16 == 0 && (stride_h * esz) % 16 == 0 &&
                          ((int64_t)HID * esz) % 16 == 0,
                      HIPATTN_E_ALIGN, "pool write: rows must be whole, aligned 16-byte packs");
    const int64_t total = n * HKV * ((int64_t)HID * esz / 16);
    const int64_t blocks = (total + 255) / 256;
    HIPATTN_CHECK_ARG(blocks < 0x7fffffffLL, HIPATTN_E_UNSUPPORTED, "pool write: too many rows");
    hipLaunchKernelGGL(pool_write_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (char *)pool,
                       stride_row * esz, stride_h * esz, HKV, HID * esz, rows, n, (const char *)src);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

extern "C" int hipattn_pool_read_rows(const void *pool, int64_t stride_row, int64_t stride_h, int32_t HKV, int32_t HID,
                                      int32_t dtype, const int64_t *rows, int64_t n, void *dst, int64_t dst_stride_row,
                                      void *stream) {
    if (n == 0) return 0;
    HIPATTN_CHECK_ARG(pool && rows && dst && n > 0 && HKV > 0 && HID > 0, HIPATTN_E_ARG, "pool read: bad argument");
    HIPATTN_CHECK_ARG(storage_esz(dtype) > 0, HIPATTN_E_UNSUPPORTED, "pool read: dtype %d", dtype);
    const int esz = storage_esz(dtype);
    HIPATTN_CHECK_ARG(aligned16(pool) && aligned16(dst) && (stride_row * esz) % 16 == 0 && (stride_h * esz) % 16 == 0 &&
                          (dst_stride_row * esz) % 16 == 0 && ((int64_t)HID * esz) % 16 == 0 &&
                          dst_stride_row >= (int64_t)HKV * HID,
                      HIPATTN_E_ALIGN, "pool read: rows must be whole, aligned 16-byte packs");
    const int64_t total = n * HKV * ((int64_t)HID * esz / 16);
    const int64_t blocks = (total + 255) / 256;
    HIPATTN_CHECK_ARG(blocks < 0x7fffffffLL, HIPATTN_E_UNSUPPORTED, "pool read: too many rows");
    hipLaunchKernelGGL(pool_read_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const char *)pool, stride_row * esz, stride_h * esz, HKV, HID * esz, rows, n, (char *)dst,
                       dst_stride_row * esz);
    HIPATTN_CHECK_HIP(hipGetLastError());
    return 0;
}

extern "C" int hipattn_host_device_pointer(void *host, void **device_out) {
    HIPATTN_CHECK_ARG(host && device_out, HIPATTN_E_ARG, "host pointer: null");
    HIPATTN_CHECK_HIP(hipHostGetDevicePointer(device_out, host, 0));
    return 0;
}

extern "C" int hipattn_host_alloc(int64_t bytes, int32_t coherent, void **host_out) {
    HIPATTN_CHECK_ARG(bytes > 0 && host_out, HIPATTN_E_ARG, "host alloc: bad argument");
    const unsigned flags = hipHostMallocMapped | hipHostMallocPortable |
                           (coherent ? hipHostMallocCoherent : hipHostMallocNonCoherent);
    HIPATTN_CHECK_HIP(hipHostMalloc(host_out, (size_t)bytes, flags));
    return 0;
}

extern "C" int hipattn_host_free(void *host) {
    if (!host) return 0;
    HIPATTN_CHECK_HIP(hipHostFree(host));
    return 0;
}

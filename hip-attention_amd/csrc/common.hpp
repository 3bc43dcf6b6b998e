// Shared device/host helpers for the hipattn kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hipattn.h"

namespace hipattn {

constexpr int WAVE = 64;

// ---------------------------------------------------------------- host-side error plumbing
void set_error(const char *fmt, ...);

#define HIPATTN_CHECK_ARG(cond, code, ...)  \
    do {                                    \
        if (!(cond)) {                      \
            ::hipattn::set_error(__VA_ARGS__); \
            return (code);                  \
        }                                   \
    } while (0)

#define HIPATTN_CHECK_HIP(expr)                                                       \
    do {                                                                              \
        hipError_t _e = (expr);                                                       \
        if (_e != hipSuccess) {                                                       \
            ::hipattn::set_error("%s failed: %s", #expr, hipGetErrorString(_e));      \
            return (int)_e;                                                           \
        }                                                                             \
    } while (0)

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---------------------------------------------------------------- element types
// bf16 is carried as raw 16-bit patterns; all arithmetic happens in f32.
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// round-to-nearest-even f32 -> bf16, result widened back to f32 (NaN inputs are not expected)
__device__ __forceinline__ float round_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return __uint_as_float(u & 0xffff0000u);
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <typename T>
struct Elem;

template <>
struct Elem<float> {
    static constexpr int dtype = HIPATTN_F32;
    __device__ static __forceinline__ float widen(float x) { return x; }
    __device__ static __forceinline__ float round(float x) { return x; }
    __device__ static __forceinline__ float narrow(float x) { return x; }
};

template <>
struct Elem<bf16_t> {
    static constexpr int dtype = HIPATTN_BF16;
    __device__ static __forceinline__ float widen(bf16_t x) { return bf16_to_f32(x.bits); }
    __device__ static __forceinline__ float round(float x) { return round_bf16(x); }
    __device__ static __forceinline__ bf16_t narrow(float x) { return bf16_t{f32_to_bf16_bits(x)}; }
};

// scale constants: c_q = T(sqrt(HID)/sqrt(sqrt(HID))), c_k = T(1/sqrt(sqrt(HID))), f32 IEEE ops.
// Computed on the host (correctly rounded sqrtf and division) and passed to kernels.
void scale_constants(int hid, int dtype, float *c_q, float *c_k);

// ---------------------------------------------------------------- vector row loads
// A row slice of N elements of T kept as raw dwords (N*sizeof(T) is a multiple of 4 bytes and the
// address is aligned to min(16, N*sizeof(T)) bytes).
template <typename T, int N>
struct RawSlice {
    static constexpr int BYTES = N * (int)sizeof(T);
    static_assert(BYTES % 4 == 0, "row slices are whole dwords");
    static_assert(BYTES < 16 || BYTES % 16 == 0, "wide slices are whole 16-byte packs");
    uint32_t w[BYTES / 4];

    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < BYTES / 4; i++) w[i] = 0u;
    }
    __device__ __forceinline__ void load(const T *p) {
        if constexpr (BYTES >= 16) {
            const uint4 *pp = reinterpret_cast<const uint4 *>(p);
#pragma unroll
            for (int i = 0; i < BYTES / 16; i++) {
                uint4 v = pp[i];
                w[i * 4 + 0] = v.x; w[i * 4 + 1] = v.y; w[i * 4 + 2] = v.z; w[i * 4 + 3] = v.w;
            }
        } else if constexpr (BYTES == 8) {
            uint2 v = *reinterpret_cast<const uint2 *>(p);
            w[0] = v.x; w[1] = v.y;
        } else {
            w[0] = *reinterpret_cast<const uint32_t *>(p);
        }
    }
    __device__ __forceinline__ void widen(float (&out)[N]) const {
#pragma unroll
        for (int i = 0; i < BYTES / 4; i++) {
            if constexpr (sizeof(T) == 4) {
                out[i] = __uint_as_float(w[i]);
            } else {
                out[i * 2] = __uint_as_float(w[i] << 16);
                out[i * 2 + 1] = __uint_as_float(w[i] & 0xffff0000u);
            }
        }
    }
};

template <typename T, int N>
__device__ __forceinline__ void load_elems(const T *p, float (&out)[N]) {
    RawSlice<T, N> r;
    r.load(p);
    r.widen(out);
}

// ---------------------------------------------------------------- KV addressing (device copy of hipattn_kv_t)
// Block cache in front of a host-resident pool: what the kernels need of a hipattn_cache_t.
// "no such row" marker for row offsets.  Offsets are relative to the K / V base pointer and may be negative
// when they lead into an offload cache's bank, so the marker is not simply "below zero".
constexpr int64_t NO_ROW = INT64_MIN;

struct CacheView {
    const int32_t *table;   // [HKV, n_blocks] slot or -1
    int32_t *last_use;      // [slots] step of the last read
    uint8_t *miss;          // [HKV, n_blocks] set when a read went to the host pool
    const int32_t *step;    // current step counter
    int64_t k_delta;        // element offset from KVView::k to the K part of slot 0
    int64_t v_delta;        // element offset from KVView::v to the V part of slot 0
    int64_t slot_stride;    // elements per slot
    int64_t n_blocks;
    int32_t shift;          // log2(block_tokens)
    int32_t row_elems;      // HID
    int32_t with_v;         // slots hold V rows too
};

// CHECK = true reads first and stores only a flag that is still clear (right for readers that revisit the
// same rows many times); CHECK = false stores blindly (right for one pass over mostly distinct rows).
// Racing lanes store the same value; a stale read only repeats the store.
template <bool CHECK = true>
__device__ __forceinline__ void mark_flag(uint8_t *f) {
    if (!CHECK || *f == 0) *f = 1;
}

struct KVView {
    const void *k;
    const void *v;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t v_stride_b, v_stride_t, v_stride_h;
    int64_t tsrc;
    int64_t max_tsrc;
    const void *block_table;
    const void *cache_seq_lens;
    int64_t bt_stride_b;
    int bt_is64, sl_is64, paged, page_size, HKV;
    int page_shift;  // log2(page_size): page sizes are powers of two

    __device__ __forceinline__ int64_t seq_len(int b) const {
        return sl_is64 ? reinterpret_cast<const int64_t *>(cache_seq_lens)[b]
                       : (int64_t) reinterpret_cast<const int32_t *>(cache_seq_lens)[b];
    }
    __device__ __forceinline__ int64_t page_of(int b, int64_t t, int64_t seqlen) const {
        int64_t page = 0;
        if (t >= 0 && t < seqlen) {
            int64_t i = (int64_t)b * bt_stride_b + (t >> page_shift);
            page = bt_is64 ? reinterpret_cast<const int64_t *>(block_table)[i]
                           : (int64_t) reinterpret_cast<const int32_t *>(block_table)[i];
        }
        return page;
    }
    __device__ __forceinline__ int64_t k_plain(int b, int64_t t, int h, int64_t seqlen) const {
        if (!paged) {
            if (t < 0 || t >= tsrc) return NO_ROW;
            return (int64_t)b * k_stride_b + t * k_stride_t + (int64_t)h * k_stride_h;
        }
        const int64_t page = page_of(b, t, seqlen);
        if (t < 0) return NO_ROW;
        return page * k_stride_b + (t & (page_size - 1)) * k_stride_t + (int64_t)h * k_stride_h;
    }
    __device__ __forceinline__ int64_t v_plain(int b, int64_t t, int h, int64_t seqlen) const {
        if (!paged) {
            if (t < 0 || t >= tsrc) return NO_ROW;
            return (int64_t)b * v_stride_b + t * v_stride_t + (int64_t)h * v_stride_h;
        }
        const int64_t page = page_of(b, t, seqlen);
        if (t < 0) return NO_ROW;
        return page * v_stride_b + (t & (page_size - 1)) * v_stride_t + (int64_t)h * v_stride_h;
    }
};

// ---------------------------------------------------------------- fp8 (e5m2) key/value storage
// KV8 = true: K / V rows hold one byte per element (the uint8 view of a float8_e5m2 paged cache,
// uvm_gpu_cache.py:1043-1046); every value is widened to bf16 on load, which is exact.  Offsets stay in elements.
typedef __attribute__((ext_vector_type(2))) float kv_f32x2;

// eight fp8 (e5m2) bytes widened to four packed bf16 pairs (exact, so plain truncation packs the pairs)
__device__ __forceinline__ uint4 widen_bf8x8(uint2 r) {
    const kv_f32x2 a = __builtin_amdgcn_cvt_pk_f32_bf8((int)r.x, false), b = __builtin_amdgcn_cvt_pk_f32_bf8((int)r.x, true);
    const kv_f32x2 c = __builtin_amdgcn_cvt_pk_f32_bf8((int)r.y, false), d = __builtin_amdgcn_cvt_pk_f32_bf8((int)r.y, true);
    return make_uint4((__float_as_uint(a[0]) >> 16) | (__float_as_uint(a[1]) & 0xffff0000u),
                      (__float_as_uint(b[0]) >> 16) | (__float_as_uint(b[1]) & 0xffff0000u),
                      (__float_as_uint(c[0]) >> 16) | (__float_as_uint(c[1]) & 0xffff0000u),
                      (__float_as_uint(d[0]) >> 16) | (__float_as_uint(d[1]) & 0xffff0000u));
}

// 8 consecutive elements as four packed bf16 pairs
template <bool KV8>
__device__ __forceinline__ uint4 load_kv_piece(const void *base, int64_t off) {
    if constexpr (!KV8) return *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(base) + off);
    else return widen_bf8x8(*reinterpret_cast<const uint2 *>(reinterpret_cast<const uint8_t *>(base) + off));
}
// The same from an address that went through memory as an integer (a posted row address): said to be global memory,
// because a load through a generic pointer also counts as an LDS operation, and while one is in flight every wait for
// an LDS read has to wait for all of them.
typedef uint32_t kv_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t kv_u32x2 __attribute__((ext_vector_type(2)));
template <bool KV8>
__device__ __forceinline__ uint4 load_kv_piece_global(long long row_addr, int elem_off) {
    if constexpr (!KV8) {
        const kv_u32x4 r = *(const kv_u32x4 __attribute__((address_space(1))) *)(uintptr_t)(row_addr + 2 * elem_off);
        return make_uint4(r.x, r.y, r.z, r.w);
    } else {
        const kv_u32x2 r = *(const kv_u32x2 __attribute__((address_space(1))) *)(uintptr_t)(row_addr + elem_off);
        return widen_bf8x8(make_uint2(r.x, r.y));
    }
}

// N consecutive elements widened to f32 (N in {2, 4, 8, 16} for fp8 storage)
template <typename T, int N, bool KV8>
__device__ __forceinline__ void load_kv_elems(const void *base, int64_t off, float (&out)[N]) {
    if constexpr (!KV8) {
        load_elems<T, N>(reinterpret_cast<const T *>(base) + off, out);
    } else {
        const uint8_t *p = reinterpret_cast<const uint8_t *>(base) + off;
        if constexpr (N == 2) {
            const kv_f32x2 a = __builtin_amdgcn_cvt_pk_f32_bf8((int)*reinterpret_cast<const uint16_t *>(p), false);
            out[0] = a[0]; out[1] = a[1];
        } else {
            static_assert(N % 4 == 0, "fp8 row slices are whole dwords");
            uint32_t w[N / 4];
            if constexpr (N == 4) {
                w[0] = *reinterpret_cast<const uint32_t *>(p);
            } else if constexpr (N == 8) {
                const uint2 r = *reinterpret_cast<const uint2 *>(p);
                w[0] = r.x; w[1] = r.y;
            } else {
                static_assert(N == 16, "fp8 row slices hold 2, 4, 8 or 16 elements");
                const uint4 r = *reinterpret_cast<const uint4 *>(p);
                w[0] = r.x; w[1] = r.y; w[2] = r.z; w[3] = r.w;
            }
#pragma unroll
            for (int i = 0; i < N / 4; i++) {
                const kv_f32x2 a = __builtin_amdgcn_cvt_pk_f32_bf8((int)w[i], false), b = __builtin_amdgcn_cvt_pk_f32_bf8((int)w[i], true);
                out[4 * i] = a[0]; out[4 * i + 1] = a[1]; out[4 * i + 2] = b[0]; out[4 * i + 3] = b[1];
            }
        }
    }
}

// one element
template <typename T, bool KV8>
__device__ __forceinline__ float load_kv_elem(const void *base, int64_t off) {
    if constexpr (!KV8) return Elem<T>::widen(reinterpret_cast<const T *>(base)[off]);
    else return __builtin_amdgcn_cvt_f32_bf8((int)reinterpret_cast<const uint8_t *>(base)[off], 0);
}

// What only the extended builds of the kernels read: the offload cache and the statistics flags.  Kept out
// of KVView (and at the end of the parameter blocks) so that the plain kernels' arguments stay small.
struct KVExt {
    int cached;
    CacheView cache;
    uint8_t *access_flags, *miss_flags;  // one byte per page (a quarter of the words to clear and to keep in cache)
    int64_t flags_stride_b, flags_stride_h;
    int kv8;  // host: K / V are stored as fp8 (e5m2) bytes, kernels are launched in their KV8 builds
    // host: does a launch need the EXT build of its kernel
    bool extended() const { return cached || access_flags || miss_flags || kv8; }
};

// Element offsets (from kv.k and kv.v) of the rows of token t, kv head h; NO_ROW = "zero row".
// WANT_V = false skips the V side.  EXT = true also records the access and consults the block cache through
// `kx` (ignored otherwise).  Several lanes usually fetch pieces of one row: `leader` is true for the one that
// records the access.  DEFER = true: the access flag is not touched here; `*mark_out` receives its index in the
// (batch item, kv head) row of flags (token or page; untouched when there is nothing to record), and the caller
// marks it once its row loads are on their way: a look at the flag is a trip to memory, and ahead of the row loads
// it is a trip of its own.
template <bool WANT_V, bool EXT, bool CHECK = true, bool DEFER = false>
__device__ __forceinline__ void kv_rows(const KVView &kv, const KVExt *kx, int b, int64_t t, int h, int64_t seqlen,
                                        int64_t &ko, int64_t &vo, bool leader = true, int64_t *mark_out = nullptr) {
    if constexpr (!EXT) {
        // Plain path: K and V offsets as two independent selects.  Sharing the range test and the page lookup
        // between them reads better but made the attention tile kernel 18% slower (the compiler then keeps both
        // row loads inside one divergent region and serialises them behind its waits).
        ko = kv.k_plain(b, t, h, seqlen);
        vo = WANT_V ? kv.v_plain(b, t, h, seqlen) : NO_ROW;
        return;
    }
    ko = NO_ROW;
    vo = NO_ROW;
    if (!kv.paged) {
        if (t < 0 || t >= kv.tsrc) return;
        if constexpr (EXT) {
            if (kx->access_flags && leader) {
                if constexpr (DEFER) *mark_out = t;
                else mark_flag<CHECK>(kx->access_flags + (int64_t)b * kx->flags_stride_b + (int64_t)h * kx->flags_stride_h + t);
            }
        }
        ko = (int64_t)b * kv.k_stride_b + t * kv.k_stride_t + (int64_t)h * kv.k_stride_h;
        if (WANT_V) vo = (int64_t)b * kv.v_stride_b + t * kv.v_stride_t + (int64_t)h * kv.v_stride_h;
        return;
    }
    if (t < 0) return;
    const int64_t page = kv.page_of(b, t, seqlen);
    const int64_t inpage = t & (kv.page_size - 1);
    if constexpr (EXT) {
        if (kx->access_flags && leader) {
            if constexpr (DEFER) *mark_out = page;
            else mark_flag<CHECK>(kx->access_flags + (int64_t)b * kx->flags_stride_b + (int64_t)h * kx->flags_stride_h + page);
        }
        if (kx->cached) {
            const CacheView &c = kx->cache;
            const int64_t row = (page << kv.page_shift) + inpage;
            const int64_t e = (int64_t)h * c.n_blocks + (row >> c.shift);
            const int32_t slot = c.table[e];
            if (slot >= 0) {
                if (leader) {
                    const int32_t now = *c.step;
                    if (c.last_use[slot] != now) c.last_use[slot] = now;
                }
                const int64_t o = (int64_t)slot * c.slot_stride + (row & ((1LL << c.shift) - 1)) * c.row_elems;
                ko = c.k_delta + o;
                if (WANT_V)
                    vo = c.with_v ? c.v_delta + o
                                  : page * kv.v_stride_b + inpage * kv.v_stride_t + (int64_t)h * kv.v_stride_h;
                return;
            }
            if (leader) {
                if (c.miss[e] == 0) c.miss[e] = 1;
                if (kx->miss_flags)
                    mark_flag(kx->miss_flags + (int64_t)b * kx->flags_stride_b + (int64_t)h * kx->flags_stride_h + page);
            }
        }
    }
    ko = page * kv.k_stride_b + inpage * kv.k_stride_t + (int64_t)h * kv.k_stride_h;
    if (WANT_V) vo = page * kv.v_stride_b + inpage * kv.v_stride_t + (int64_t)h * kv.v_stride_h;
}

template <bool EXT, bool CHECK = true, bool DEFER = false>
__device__ __forceinline__ int64_t kv_k_row(const KVView &kv, const KVExt *kx, int b, int64_t t, int h,
                                            int64_t seqlen, bool leader = true, int64_t *mark_out = nullptr) {
    int64_t ko, vo;
    kv_rows<false, EXT, CHECK, DEFER>(kv, kx, b, t, h, seqlen, ko, vo, leader, mark_out);
    return ko;
}

// ---------------------------------------------------------------- rotary embedding applied on load
// Device copy of hipattn_rope_t.  cos == nullptr: rows are used as stored.
struct RopeView {
    const void *cos, *sin;
    int64_t stride_t, len;
    int backend;  // HIPATTN_EXTEND_*
    int64_t k_side_delta;  // prescaled RELATIVE scan: offset of the position-1 copy of the keys
    int64_t model_ctx;     // DYNAMIC rule: the model's context length
    __device__ __forceinline__ int64_t clamp(int64_t pos) const { return pos < 0 ? 0 : (pos >= len ? len - 1 : pos); }
    __device__ __forceinline__ int64_t row(int64_t pos) const {  // element offset of the table row of a position
        return clamp(pos) * stride_t;
    }
};

// Position the sampled key at token t is rotated to under the DYNAMIC rule (attention_extend.py:254-274): a query
// block that reaches beyond the model's context squeezes the keys older than a quarter of that context into the
// rest of it, linearly and in float32.  pmin: position of the block's first strided row; pmax = pmin + its number
// of valid strided rows.  The host refuses model_ctx < 512, which keeps pmin - window positive wherever the
// quotient is used (pmax > model_ctx and at most 64 rows).
__device__ __forceinline__ int64_t dynamic_extend_pos(int64_t t, int64_t pmin, int64_t pmax, int64_t model_ctx) {
    const int64_t window = model_ctx / 4;
    int64_t pos = t;
    if (!(t >= pmax - window || pmax <= model_ctx)) {
        const float off = __fsub_rn((float)t, (float)(pmin - window));
        const float ratio = __fdiv_rn((float)(model_ctx - window), (float)(pmin - window));
        pos = (int64_t)(int)__fmul_rn(off, ratio) + (pmin - window);
    }
    const int64_t lowest = pmax - model_ctx;
    return pos > lowest ? pos : lowest;
}

// The SELF rule (attention_extend.py:275-289): keys older than 8192 positions are grouped by sixteen once the query
// block reaches beyond the model's context; the quotient truncates toward zero, as the compiled kernel's does.
__device__ __forceinline__ int64_t self_extend_pos(int64_t t, int64_t pmin, int64_t pmax, int64_t model_ctx) {
    int64_t pos = t;
    if (!(t >= pmax - 8192 || pmax <= model_ctx)) pos = (t - pmin) / 16 + pmin;
    return pos > 0 ? pos : 0;
}
// rules under which a sampled key's rotated position follows its token (the table row is reloaded with every sample)
__device__ __forceinline__ bool rope_follows_token(int backend) {
    return backend == HIPATTN_EXTEND_DYNAMIC || backend == HIPATTN_EXTEND_SELF;
}
__device__ __forceinline__ int64_t token_extend_pos(const RopeView &r, int64_t t, int64_t pmin, int64_t pmax) {
    return r.backend == HIPATTN_EXTEND_SELF ? self_extend_pos(t, pmin, pmax, r.model_ctx)
                                            : dynamic_extend_pos(t, pmin, pmax, r.model_ctx);
}

// One element of a rotated row: x*c + o*s with `o` the partner element, already signed (-x[i + HID/2] in the
// lower half, +x[i - HID/2] in the upper); both products and the sum are rounded to T, never fused.
template <typename T>
__device__ __forceinline__ float rope_elem(float x, float o, float c, float s) {
    return Elem<T>::round(__fadd_rn(Elem<T>::round(__fmul_rn(x, c)), Elem<T>::round(__fmul_rn(o, s))));
}

typedef __attribute__((ext_vector_type(2))) __bf16 rope_bf16x2;
typedef __attribute__((ext_vector_type(2))) float rope_f32x2;
__device__ __forceinline__ uint32_t rope_pk(float a, float b) {  // two f32 -> packed bf16, round to nearest even
    rope_f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, rope_bf16x2));
}
// The same on a packed pair of bf16: w own pair, o partner pair, c and s table pairs; `s` must already carry the
// sign of the half (xor 0x80008000 for the lower half).
__device__ __forceinline__ uint32_t rope_pair(uint32_t w, uint32_t o, uint32_t c, uint32_t s) {
    const uint32_t a = rope_pk(__fmul_rn(__uint_as_float(w << 16), __uint_as_float(c << 16)),
                               __fmul_rn(__uint_as_float(w & 0xffff0000u), __uint_as_float(c & 0xffff0000u)));
    const uint32_t b = rope_pk(__fmul_rn(__uint_as_float(o << 16), __uint_as_float(s << 16)),
                               __fmul_rn(__uint_as_float(o & 0xffff0000u), __uint_as_float(s & 0xffff0000u)));
    return rope_pk(__fadd_rn(__uint_as_float(a << 16), __uint_as_float(b << 16)),
                   __fadd_rn(__uint_as_float(a & 0xffff0000u), __uint_as_float(b & 0xffff0000u)));
}
// Blend of two packed table pairs, T(T(a * wa) + T(b * wb)) per element: the "dynamic_extend" rule of attention
// rotates a far key with 0.75 of the table row of its packed position and 0.25 of the row of its own squeezed
// position (attention_extend_bsa.py:323-357); weights (1, 0) hand back `a` unchanged.
__device__ __forceinline__ uint32_t rope_blend_pair(uint32_t a, uint32_t b, float wa, float wb) {
    const uint32_t x = rope_pk(__fmul_rn(__uint_as_float(a << 16), wa), __fmul_rn(__uint_as_float(a & 0xffff0000u), wa));
    const uint32_t y = rope_pk(__fmul_rn(__uint_as_float(b << 16), wb), __fmul_rn(__uint_as_float(b & 0xffff0000u), wb));
    return rope_pk(__fadd_rn(__uint_as_float(x << 16), __uint_as_float(y << 16)),
                   __fadd_rn(__uint_as_float(x & 0xffff0000u), __uint_as_float(y & 0xffff0000u)));
}
__device__ __forceinline__ uint4 rope_blend_piece(uint4 a, uint4 b, float wa, float wb) {
    return make_uint4(rope_blend_pair(a.x, b.x, wa, wb), rope_blend_pair(a.y, b.y, wa, wb),
                      rope_blend_pair(a.z, b.z, wa, wb), rope_blend_pair(a.w, b.w, wa, wb));
}
__device__ __forceinline__ uint4 rope_piece(uint4 w, uint4 o, uint4 c, uint4 s, bool lower) {
    const uint32_t sg = lower ? 0x80008000u : 0u;
    return make_uint4(rope_pair(w.x, o.x, c.x, s.x ^ sg), rope_pair(w.y, o.y, c.y, s.y ^ sg),
                      rope_pair(w.z, o.z, c.z, s.z ^ sg), rope_pair(w.w, o.w, c.w, s.w ^ sg));
}

// Can a key row lie 32 GiB or more beyond view.k?  The scan variants that pass the places of rows between lanes as
// 31-bit numbers of 16-byte pieces hold only below that.  A dense tensor's extent follows from its shape and strides
// (`extra_elems`: a second copy of the keys that far behind the first, see RopeView::k_side_delta); a paged pool has
// no page count in its description, so it counts as far unless the caller says otherwise.
inline bool kv_rows_beyond_32gib(const KVView &kv, int B, int HID, int elem_bytes, int64_t extra_elems, bool pool_is_near) {
    if (kv.paged) return !pool_is_near;
    auto mag = [](int64_t x) { return x < 0 ? -x : x; };
    const long double elems = (long double)(B > 0 ? B - 1 : 0) * mag(kv.k_stride_b) +
                              (long double)(kv.tsrc > 0 ? kv.tsrc - 1 : 0) * mag(kv.k_stride_t) +
                              (long double)(kv.HKV > 0 ? kv.HKV - 1 : 0) * mag(kv.k_stride_h) + HID + mag(extra_elems);
    return elems * elem_bytes >= (long double)(1LL << 35);
}

// validates q->rope (may be NULL) and fills the view; `allowed` is a bit mask of HIPATTN_EXTEND_* values
int make_rope_view(const hipattn_q_t *q, unsigned allowed, const char *who, RopeView *out);
int make_kv_view(const hipattn_kv_t *kv, int B, int HID, int dtype, KVView *out, KVExt *ext);
int cache_view_for(const hipattn_cache *c, const hipattn_kv_t *kv, const KVView *view, int HID, int dtype, KVExt *ext);
int check_q(const hipattn_q_t *q);

// ---------------------------------------------------------------- wave helpers
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ int wave_min_i(int v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ int wave_max_i(int v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ long long wave_min_ll(long long v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        long long w = __shfl_xor(v, o);
        v = w < v ? w : v;
    }
    return v;
}

// Value held by the lane 32 positions away (lane ^ 32): one v_permlane32_swap instead of a trip through LDS.
// The instruction swaps the upper half of its first operand with the lower half of its second; fed the same
// value twice it leaves (lower half everywhere, upper half everywhere), and each lane picks the half that is
// not its own.
__device__ __forceinline__ uint32_t swap_halves(uint32_t x) {
    const auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return (threadIdx.x & 32) ? r[0] : r[1];
}
__device__ __forceinline__ float swap_halves(float x) { return __uint_as_float(swap_halves(__float_as_uint(x))); }
// The value held by lane ^ N.  N = 8 is a rotation of every row of 16 lanes by eight places, which the data-parallel
// path does in one vector instruction; the general exchange goes through the LDS crossbar and has to be waited for.
template <int N>
__device__ __forceinline__ uint32_t lane_xor(uint32_t x) {
    if constexpr (N == 8) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x128 /* row_ror:8 */, 0xf, 0xf, false);
    else if constexpr (N == 32) return swap_halves(x);
    else return (uint32_t)__shfl_xor((int)x, N);
}

// ---------------------------------------------------------------- direct global -> LDS loads
// 16 bytes per lane from global memory straight into LDS (global_load_lds_dwordx4): lane i's piece lands at
// lds_base + 16 * i, lds_base being wave-uniform; each lane supplies its own global address.  No registers and no
// LDS stores are spent on staging.  Written as an asm statement: the compiler would order every later LDS read,
// also of other buffers, behind a full wait on the vector-memory counter.  A kernel that uses it waits itself
// (wait_vmcnt, then the workgroup barrier) before anything reads the buffer the loads fill.  A load cannot be
// predicated into writing zeros: rows that do not exist are fetched from a row of zeros in device memory.
__device__ __forceinline__ void load_to_lds16(const void *gsrc, void *lds_base) {
    const uint32_t base = (uint32_t)(uintptr_t)lds_base;  // LDS addresses are the low 32 bits of the flat pointer
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gsrc), "s"(__builtin_amdgcn_readfirstlane(base))
                 : "memory", "m0");
}
// the same with the LDS address given as a wave-uniform 32-bit value (kept in a scalar register by the caller)
__device__ __forceinline__ void load_to_lds16_at(const void *gsrc, uint32_t lds_addr_uniform) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gsrc), "s"(lds_addr_uniform)
                 : "memory", "m0");
}
// the same with the global address given as a wave-uniform base (scalar register pair) plus a 32-bit byte offset per
// lane: half the address registers, and no 64-bit additions per lane
__device__ __forceinline__ void load_to_lds16_at_s(const void *gbase_uniform, uint32_t byte_off, uint32_t lds_addr_uniform) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(byte_off), "s"(gbase_uniform), "s"(lds_addr_uniform)
                 : "memory", "m0");
}
// wait until at most N vector-memory operations of this wave are outstanding (they complete in order)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));  // expcnt and lgkmcnt left at their maxima
}

// XCD-aware remap: consecutive workgroup ids are dealt round-robin to the 8 XCDs (each with its
// own L2), so give every XCD one contiguous range of logical work ids.
__device__ __forceinline__ long long xcd_remap(long long bid, long long total) {
    constexpr long long NX = 8;
    long long per = total / NX;
    long long main = per * NX;
    if (bid >= main) return bid;  // tail that does not divide evenly keeps its id
    return (bid % NX) * per + bid / NX;
}

}  // namespace hipattn

// Host-side plumbing of the C ABI: error strings, argument checks, scale constants, dispatch.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "bsa.hpp"

namespace hipattn {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

static float host_round_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    memcpy(&f, &u, 4);
    return f;
}

void scale_constants(int hid, int dtype, float *c_q, float *c_k) {
    volatile float s = sqrtf((float)hid);
    volatile float ss = sqrtf(s);
    volatile float cq = s / ss;
    volatile float ck = 1.0f / ss;
    *c_q = dtype == HIPATTN_BF16 ? host_round_bf16(cq) : (float)cq;
    *c_k = dtype == HIPATTN_BF16 ? host_round_bf16(ck) : (float)ck;
}

int check_q(const hipattn_q_t *q) {
    HIPATTN_CHECK_ARG(q && q->ptr && q->pos, HIPATTN_E_ARG, "q: null pointer");
    HIPATTN_CHECK_ARG(q->B > 0 && q->TDST > 0 && q->HEAD > 0 && q->HID > 0, HIPATTN_E_ARG, "q: non-positive shape");
    HIPATTN_CHECK_ARG(q->dtype == HIPATTN_F32 || q->dtype == HIPATTN_BF16, HIPATTN_E_UNSUPPORTED, "q: dtype %d",
                      q->dtype);
    HIPATTN_CHECK_ARG(q->HID % 16 == 0, HIPATTN_E_UNSUPPORTED, "q: head dim %d is not a multiple of 16", q->HID);
    const int esz = q->dtype == HIPATTN_BF16 ? 2 : 4;
    const int64_t al = 16 / esz;
    HIPATTN_CHECK_ARG(aligned16(q->ptr) && q->stride_b % al == 0 && q->stride_t % al == 0 && q->stride_h % al == 0,
                      HIPATTN_E_ALIGN, "q: base pointer and strides must be 16-byte aligned");
    return 0;
}

int make_rope_view(const hipattn_q_t *q, unsigned allowed, const char *who, RopeView *o) {
    memset(o, 0, sizeof(*o));
    const hipattn_rope_t *r = q->rope;
    if (!r) return 0;
    HIPATTN_CHECK_ARG(r->cos && r->sin && r->len > 0, HIPATTN_E_ARG, "%s: rope tables are null or empty", who);
    HIPATTN_CHECK_ARG(r->backend >= 1 && r->backend < 32 && ((allowed >> r->backend) & 1u), HIPATTN_E_UNSUPPORTED,
                      "%s: extend backend %d is not built for this entry point", who, r->backend);
    const int esz = q->dtype == HIPATTN_BF16 ? 2 : 4;
    HIPATTN_CHECK_ARG(aligned16(r->cos) && aligned16(r->sin) && (r->stride_t * esz) % 16 == 0 &&
                          r->stride_t >= q->HID / 2,
                      HIPATTN_E_ALIGN, "%s: rope table rows must be 16-byte aligned and hold HID/2 columns", who);
    HIPATTN_CHECK_ARG(q->HID % 32 == 0, HIPATTN_E_UNSUPPORTED, "%s: rope needs a head dim that is a multiple of 32", who);
    o->cos = r->cos; o->sin = r->sin; o->stride_t = r->stride_t; o->len = r->len; o->backend = r->backend;
    o->k_side_delta = r->k_side_delta;
    o->model_ctx = r->model_context_length;
    HIPATTN_CHECK_ARG(r->backend != HIPATTN_EXTEND_DYNAMIC || r->model_context_length >= 512, HIPATTN_E_ARG,
                      "%s: the dynamic rule needs model_context_length >= 512 (got %lld)", who,
                      (long long)r->model_context_length);
    return 0;
}

int make_kv_view(const hipattn_kv_t *kv, int B, int HID, int dtype, KVView *o, KVExt *x) {
    (void)B;
    HIPATTN_CHECK_ARG(kv && kv->k, HIPATTN_E_ARG, "kv: null K pointer");
    HIPATTN_CHECK_ARG(kv->HKV > 0, HIPATTN_E_ARG, "kv: HKV <= 0");
    if (kv->fp8) {
        HIPATTN_CHECK_ARG(dtype == HIPATTN_BF16 && kv->paged, HIPATTN_E_UNSUPPORTED,
                          "kv: fp8 storage needs a bf16 query and the paged view");
        HIPATTN_CHECK_ARG(HID % 32 == 0, HIPATTN_E_UNSUPPORTED, "kv: fp8 storage needs a head dim that is a multiple of 32");
    }
    const int esz = kv->fp8 ? 1 : (dtype == HIPATTN_BF16 ? 2 : 4);
    const int64_t al = kv->fp8 ? 8 : 16 / esz;  // fp8 rows are fetched in 8-byte pieces
    const void *v = kv->v ? kv->v : kv->k;
    HIPATTN_CHECK_ARG(aligned16(kv->k) && aligned16(v) && kv->k_stride_b % al == 0 && kv->k_stride_t % al == 0 &&
                          kv->k_stride_h % al == 0 && kv->v_stride_b % al == 0 && kv->v_stride_t % al == 0 &&
                          kv->v_stride_h % al == 0 && ((int64_t)HID * esz) % 16 == 0,
                      HIPATTN_E_ALIGN, "kv: base pointers and strides must be 16-byte aligned");
    if (kv->paged) {
        HIPATTN_CHECK_ARG(kv->block_table && kv->cache_seq_lens, HIPATTN_E_ARG, "kv: paged without block table / lengths");
        const int ps = kv->page_size;
        HIPATTN_CHECK_ARG(ps == 1 || ps == 2 || ps == 4 || ps == 8 || ps == 16 || ps == 32, HIPATTN_E_ARG,
                          "kv: page size %d not in {1,2,4,8,16,32}", ps);
    } else {
        HIPATTN_CHECK_ARG(kv->tsrc > 0, HIPATTN_E_ARG, "kv: dense with tsrc <= 0");
    }
    HIPATTN_CHECK_ARG(kv->max_tsrc > 0 && kv->max_tsrc < 0x7fffffffLL, HIPATTN_E_ARG, "kv: max_tsrc out of range");
    o->k = kv->k; o->v = v;
    o->k_stride_b = kv->k_stride_b; o->k_stride_t = kv->k_stride_t; o->k_stride_h = kv->k_stride_h;
    o->v_stride_b = kv->v ? kv->v_stride_b : kv->k_stride_b;
    o->v_stride_t = kv->v ? kv->v_stride_t : kv->k_stride_t;
    o->v_stride_h = kv->v ? kv->v_stride_h : kv->k_stride_h;
    o->tsrc = kv->tsrc; o->max_tsrc = kv->max_tsrc;
    o->block_table = kv->block_table; o->cache_seq_lens = kv->cache_seq_lens; o->bt_stride_b = kv->bt_stride_b;
    o->bt_is64 = kv->bt_is64; o->sl_is64 = kv->sl_is64; o->paged = kv->paged; o->page_size = kv->page_size ? kv->page_size : 1;
    o->page_shift = 0;
    while ((1 << o->page_shift) < o->page_size) o->page_shift++;
    o->HKV = kv->HKV;
    memset(x, 0, sizeof(*x));
    x->access_flags = kv->access_flags;
    x->miss_flags = kv->miss_flags;
    x->flags_stride_b = kv->flags_stride_b;
    x->flags_stride_h = kv->flags_stride_h;
    x->kv8 = kv->fp8 ? 1 : 0;
    if (kv->cache) return cache_view_for(kv->cache, kv, o, HID, dtype, x);
    return 0;
}

}  // namespace hipattn

using namespace hipattn;

extern "C" const char *hipattn_version(void) { return "hipattn 0.1 (gfx950)"; }
extern "C" const char *hipattn_last_error(void) { return g_err; }

extern "C" int hipattn_bsa_prefill(const hipattn_q_t *q, const hipattn_kv_t *kv, const int64_t *indices,
                                   const int32_t *ks_start_end, int32_t idx_rows, int32_t BK, int32_t block_size_q,
                                   int32_t block_size_k, int32_t sliding_window, int32_t sink,
                                   int32_t share_first_head, int32_t impl, const void *k_prescaled, void *out,
                                   int64_t out_stride_b,
                                   int64_t out_stride_t, int64_t out_stride_h, void *stream) {
    BsaParams p;
    int rc = bsa_fill_params(q, kv, indices, ks_start_end, idx_rows, BK, block_size_q, block_size_k, sliding_window,
                             sink, share_first_head, out, out_stride_b, out_stride_t, out_stride_h, &p);
    if (rc) return rc;
    HIPATTN_CHECK_ARG(impl >= 0 && impl <= 2, HIPATTN_E_ARG, "bsa: impl %d not in {0,1,2}", impl);
    hipStream_t st = (hipStream_t)stream;
    if (impl != 1) {
        BsaParams pm = p;
        if (k_prescaled) {  // same layout and strides as kv->k
            HIPATTN_CHECK_ARG(!kv->cache, HIPATTN_E_ARG, "bsa: k_prescaled cannot be combined with an offload cache");
            HIPATTN_CHECK_ARG(aligned16(k_prescaled), HIPATTN_E_ALIGN, "bsa: k_prescaled must be 16-byte aligned");
            pm.kv.k = k_prescaled;
            pm.k_prescaled = 1;
        }
        rc = bsa_mfma_launch(pm, q->dtype, q->HID, st);
        if (rc != HIPATTN_E_UNSUPPORTED) return rc;
        if (impl == 2) {
            set_error("bsa: the MFMA tile kernel does not cover dtype %d, head dim %d, block_size_q %d, block_size_k %d",
                      q->dtype, q->HID, block_size_q, block_size_k);
            return rc;
        }
    }
    return bsa_simple_launch(p, q->dtype, q->HID, st);
}

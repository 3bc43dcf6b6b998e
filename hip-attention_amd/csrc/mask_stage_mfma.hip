// Mask-estimation scan stage for bf16 inputs on the matrix cores.
//
// Scores of a binary-search iteration are S[query row, sampled token] = q^ . k^.  One
// v_mfma_f32_32x32x16_bf16 covers 32 query rows x 32 sampled tokens x 16 head-dim elements with
//   A = Q^ rows     (resident in registers for the whole kernel),
//   B = K^ rows     (lane n%32 <-> token, loaded straight from global memory: a lane reads one half
//                    of its token's row, HID bytes contiguous, no LDS staging and no barriers),
//   D[row, token]   (a lane ends up with 16 query rows of ITS token: the max over rows is in-lane).
// A wave owns NB blocks of 32 tokens = 16*NB chunks (left and right sample of a chunk sit in
// adjacent lanes); the program-level gate and iteration count of the reference (a "program" is a
// group of block_chunk chunks) are recomputed by every wave from the group's chunk list, so a
// program can be split over several waves without changing results.
//
// Accumulation order of the dot product is the hardware's: two groups of 8 per instruction,
// instructions chained through the f32 accumulator; head-dim element of (instruction ks, lane half
// hh, i) is  hh*HID/2 + ks*8 + i.  The order is part of the operator's numeric definition.
#include "mask_common.hpp"

namespace hipattn {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

union BFrag {
    bf16x8 v;
    uint32_t u[4];
    uint4 q;
};

__device__ __forceinline__ uint32_t scale_pack(uint32_t w, float c) {
    const float lo = __uint_as_float(w << 16) * c;
    const float hi = __uint_as_float(w & 0xffff0000u) * c;
    return (uint32_t)f32_to_bf16_bits(lo) | ((uint32_t)f32_to_bf16_bits(hi) << 16);
}

template <int HID, int MB, int NB, bool PRESCALED>
__global__ __launch_bounds__(64) void mask_stage_mfma_kernel(MaskParams p, int nsub) {
    constexpr int KS = HID / 16;
    constexpr int HALF = HID / 2;
    const int lane = threadIdx.x;
    const int n = lane & 31, hh = lane >> 5;
    const int side = n & 1;

    long long L = xcd_remap((long long)blockIdx.x, p.total);
    const int hin = (int)(L % p.G);
    L /= p.G;
    const int sub = (int)(L % nsub);
    L /= nsub;
    const int s = (int)(L % p.BS);
    L /= p.BS;
    const int g = (int)(L % p.ngroups);
    L /= p.ngroups;
    const int kvh = (int)(L % p.kv.HKV);
    const int b = (int)(L / p.kv.HKV);
    const int h = kvh * p.G + hin;

    const int BC = p.block_chunk;
    const int hgi = p.hg == 1 ? 0 : h;
    const int64_t row_in = (((int64_t)b * p.BS + s) * p.hg + hgi) * p.n;
    const int64_t row_out = (((int64_t)b * p.BS + s) * p.HEAD + h) * p.n;

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

    // ---- rows of this program
    const long long qb = (long long)(p.BDST - 1) - (long long)(p.BS - 1) * p.scan_stride + (long long)s * p.scan_stride;
    const long long myrow = qb * p.BQ + (long long)lane * p.stride_q;
    const bool rv = (lane < p.nrows) && (myrow >= 0) && (myrow < p.TDST);
    const unsigned long long rowmask = __ballot(rv);
    const long long mypos = rv ? p.pos[(int64_t)b * p.pos_sb + myrow * p.pos_st] : 0x7fffffffffffffffLL;
    const long long pmin = wave_min_ll(mypos);

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
                    p.scores[row_out + cidx[tb]] = score[tb];
                    if (p.left_out) p.left_out[row_out + cidx[tb]] = cl[tb];
                }
        }
    };
    if (!run || !(width >= p.terminate)) {
        store_out();
        return;
    }

    // ---- Q^ fragments: lane (row = mb*32 + n, half hh) holds elements hh*HALF + ks*8 .. +8
    BFrag qf[MB][KS];
    {
        const uint16_t *qbase = reinterpret_cast<const uint16_t *>(p.q) + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            const int j = mb * 32 + n;
            const bool jv = (j < p.nrows) && ((rowmask >> j) & 1ull);
            const long long it = qb * p.BQ + (long long)j * p.stride_q;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                int cnt = 0;
                if (jv) {
                    for (int o = 0; o < p.stride_q; o++) {
                        if (it + o < p.TDST) {
                            const uint4 raw = *reinterpret_cast<const uint4 *>(qbase + (it + o) * p.q_st + hh * HALF + ks * 8);
                            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                            for (int e = 0; e < 4; e++) {
                                sum[2 * e] += __uint_as_float(w[e] << 16);
                                sum[2 * e + 1] += __uint_as_float(w[e] & 0xffff0000u);
                            }
                            cnt++;
                        }
                    }
                }
                const float den = (float)cnt + 1e-12f;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float m0 = round_bf16(__fdiv_rn(sum[2 * e], den));
                    const float m1 = round_bf16(__fdiv_rn(sum[2 * e + 1], den));
                    qf[mb][ks].u[e] = jv ? ((uint32_t)f32_to_bf16_bits(m0 * p.c_q) |
                                            ((uint32_t)f32_to_bf16_bits(m1 * p.c_q) << 16))
                                         : 0u;
                }
            }
        }
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
    const uint16_t *kbase = reinterpret_cast<const uint16_t *>(p.kv.k);

    while (width >= p.terminate) {
        width *= 0.5f;
        bool active[NB];
        int ctr[NB];
        uint4 raw[NB][KS];
#pragma unroll
        for (int tb = 0; tb < NB; tb++) {
            active[tb] = real[tb] && (cl[tb] < cr[tb]) && (cl[tb] <= lim) && (cl[tb] >= 0);
            ctr[tb] = (cl[tb] + cr[tb]) >> 1;
            int64_t off = -1;
            if (active[tb]) {
                const int t = side ? ((ctr[tb] + cr[tb]) >> 1) : ((cl[tb] + ctr[tb]) >> 1);
                off = p.kv.k_row(b, t, kvh, seqlen);
            }
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                raw[tb][ks] = make_uint4(0, 0, 0, 0);
                if (off >= 0) raw[tb][ks] = *reinterpret_cast<const uint4 *>(kbase + off + hh * HALF + ks * 8);
            }
        }
#pragma unroll
        for (int tb = 0; tb < NB; tb++) {
            f32x16 acc[MB];
#pragma unroll
            for (int mb = 0; mb < MB; mb++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[mb][i] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                BFrag kf;
                if (PRESCALED) {
                    kf.q = raw[tb][ks];
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
            float v = -INFINITY;
            if (fast_rows == 16) {
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
            const float other = __shfl_xor(v, 1);
            const float sL = side ? other : v;
            const float sR = side ? v : other;
            if (active[tb]) {
                const bool win = sL > sR;
                if (win) cr[tb] = ctr[tb]; else cl[tb] = ctr[tb];
                score[tb] = fmaxf(score[tb], win ? sL : sR);
            }
        }
    }
    store_out();
}

template <int HID>
static int launch_mfma_hid(const MaskParams &p0, int rows_eff, int prescaled, hipStream_t st) {
    MaskParams p = p0;
    const int BC = p.block_chunk;
    const bool two = rows_eff > 32;
    // one wave per program (4 token blocks) when programs are plentiful, else one block per wave
    const long long programs = (long long)p.B * p.HEAD * p.BS * p.ngroups;
    const bool wide = (BC == 64) && (programs >= 16384);
    const int nb = wide ? 4 : 1;
    const int nsub = (BC / 16) / nb;
    p.total = programs * nsub;
    if (p.total >= 0x7fffffffLL) {
        set_error("mask stage: grid too large");
        return HIPATTN_E_UNSUPPORTED;
    }
    dim3 grid((unsigned)p.total), block(64);
#define MS_LAUNCH(MBv, NBv, PSv) \
    hipLaunchKernelGGL((mask_stage_mfma_kernel<HID, MBv, NBv, PSv>), grid, block, 0, st, p, nsub)
    if (two) {
        if (wide) { if (prescaled) MS_LAUNCH(2, 4, true); else MS_LAUNCH(2, 4, false); }
        else { if (prescaled) MS_LAUNCH(2, 1, true); else MS_LAUNCH(2, 1, false); }
    } else {
        if (wide) { if (prescaled) MS_LAUNCH(1, 4, true); else MS_LAUNCH(1, 4, false); }
        else { if (prescaled) MS_LAUNCH(1, 1, true); else MS_LAUNCH(1, 1, false); }
    }
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

}  // namespace hipattn

using namespace hipattn;

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

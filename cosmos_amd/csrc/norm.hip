// adaLN-modulated RMSNorm (bf16 out, or e4m3 + per-token scale out) and per-row e4m3 quantisation.
// HBM-bound: every element of x is read once and every element of y written once; the per-channel
// modulation vectors are folded into two register-resident fp32 vectors per thread and reused for
// all rows a workgroup walks over.
#include "cdm_common.h"

namespace {

constexpr int kThreads = 256;
constexpr float kE4M3Max = 448.0f;

__device__ __forceinline__ void unpack8(const uint4& u, float* f) {
    f[0] = bf16lo(u.x); f[1] = bf16hi(u.x); f[2] = bf16lo(u.y); f[3] = bf16hi(u.y);
    f[4] = bf16lo(u.z); f[5] = bf16hi(u.z); f[6] = bf16lo(u.w); f[7] = bf16hi(u.w);
}

// 8 floats (|v| <= 448 after clamping) -> 8 e4m3 bytes
__device__ __forceinline__ uint2 pack_e4m3x8(const float* f) {
    float c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) c[i] = fminf(fmaxf(f[i], -kE4M3Max), kE4M3Max);
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(c[4], c[5], hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(c[6], c[7], hi, true);
    return make_uint2((uint32_t)lo, (uint32_t)hi);
}

// block-wide reduction over 4 waves with a double-buffered LDS slot: one barrier per call
template <bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float (*slot)[4], int& parity) {
    v = IS_MAX ? wave_max(v) : wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) slot[parity][wave] = v;
    __syncthreads();
    float a = slot[parity][0], b = slot[parity][1], c = slot[parity][2], d = slot[parity][3];
    parity ^= 1;
    return IS_MAX ? fmaxf(fmaxf(a, b), fmaxf(c, d)) : (a + b) + (c + d);
}

// MAXC = chunks of 8 channels per thread (d <= 2048 * MAXC); XF32: the input rows are fp32 instead of bf16
template <int MAXC, bool QUANT, bool XF32>
__global__ __launch_bounds__(kThreads) void adaln_rmsnorm_kernel(
    const void* __restrict__ x, const uint4* __restrict__ w, const float* __restrict__ shift,
    const float* __restrict__ scale, void* __restrict__ y, float* __restrict__ s_tok, int64_t n_tokens,
    int d, float eps) {
    __shared__ float slot_sum[2][4];
    __shared__ float slot_max[2][4];
    int par_sum = 0, par_max = 0;
    const int tid = threadIdx.x;
    const int nchunk = d >> 3;

    float a[MAXC][8], b[MAXC][8];
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int idx = c * kThreads + tid;
        if (idx < nchunk) {
            // 16-byte loads: a workgroup walks over a few rows only (see the grid), so this set-up must stay cheap
            float wv[8];
            unpack8(w[idx], wv);
            float4 s0 = make_float4(0.f, 0.f, 0.f, 0.f), s1 = s0, h0 = s0, h1 = s0;
            if (scale) { s0 = reinterpret_cast<const float4*>(scale)[2 * idx]; s1 = reinterpret_cast<const float4*>(scale)[2 * idx + 1]; }
            if (shift) { h0 = reinterpret_cast<const float4*>(shift)[2 * idx]; h1 = reinterpret_cast<const float4*>(shift)[2 * idx + 1]; }
            const float sc[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
            const float sh[8] = {h0.x, h0.y, h0.z, h0.w, h1.x, h1.y, h1.z, h1.w};
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                a[c][i] = wv[i] * (1.0f + sc[i]);
                b[c][i] = sh[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) { a[c][i] = 0.0f; b[c][i] = 0.0f; }
        }
    }

    const float inv_d = 1.0f / (float)d;
    // the next row's loads are issued before the current row is reduced, so a workgroup always has a row in flight
    // XF32 (residual stream kept in fp32): a chunk of 8 channels is 32 bytes of the row instead of 16
    uint4 raw[MAXC][XF32 ? 2 : 1];
    auto fetch = [&](int64_t row) {
        const uint4* xr = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(x) + row * (int64_t)d * (XF32 ? 4 : 2));
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            const int idx = c * kThreads + tid;
#pragma unroll
            for (int h = 0; h < (XF32 ? 2 : 1); ++h)
                raw[c][h] = idx < nchunk ? xr[(XF32 ? 2 : 1) * idx + h] : make_uint4(0, 0, 0, 0);
        }
    };
    if ((int64_t)blockIdx.x < n_tokens) fetch(blockIdx.x);
    for (int64_t row = blockIdx.x; row < n_tokens; row += gridDim.x) {
        float xv[MAXC][8];
        float ss = 0.0f;
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            if constexpr (XF32) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    xv[c][4 * h + 0] = __uint_as_float(raw[c][h].x); xv[c][4 * h + 1] = __uint_as_float(raw[c][h].y);
                    xv[c][4 * h + 2] = __uint_as_float(raw[c][h].z); xv[c][4 * h + 3] = __uint_as_float(raw[c][h].w);
                }
            } else {
                unpack8(raw[c][0], xv[c]);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += xv[c][i] * xv[c][i];
        }
        if (row + gridDim.x < n_tokens) fetch(row + gridDim.x);
        ss = block_reduce<false>(ss, slot_sum, par_sum);
        const float r = rsqrtf(ss * inv_d + eps);
        float amax = 0.0f;
#pragma unroll
        for (int c = 0; c < MAXC; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                xv[c][i] = (xv[c][i] * r) * a[c][i] + b[c][i];
                if (QUANT) amax = fmaxf(amax, fabsf(xv[c][i]));
            }
        if (!QUANT) {
            uint4* yr = reinterpret_cast<uint4*>(y) + row * nchunk;
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                const int idx = c * kThreads + tid;
                if (idx < nchunk) {
                    uint4 o;
                    o.x = pack_bf16x2(xv[c][0], xv[c][1]); o.y = pack_bf16x2(xv[c][2], xv[c][3]);
                    o.z = pack_bf16x2(xv[c][4], xv[c][5]); o.w = pack_bf16x2(xv[c][6], xv[c][7]);
                    yr[idx] = o;
                }
            }
        } else {
            // the bf16 block rounds y to bf16 before the next linear; quantise that rounded value
#pragma unroll
            for (int c = 0; c < MAXC; ++c)
#pragma unroll
                for (int i = 0; i < 8; i += 2) {
                    const uint32_t p = pack_bf16x2(xv[c][i], xv[c][i + 1]);
                    xv[c][i] = bf16lo(p); xv[c][i + 1] = bf16hi(p);
                }
            amax = 0.0f;
#pragma unroll
            for (int c = 0; c < MAXC; ++c)
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(xv[c][i]));
            amax = block_reduce<true>(amax, slot_max, par_max);
            float s = amax / kE4M3Max;
            if (s == 0.0f) s = 1.0f;
            if (tid == 0) s_tok[row] = s;
            uint2* yr = reinterpret_cast<uint2*>(y) + row * nchunk;
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                const int idx = c * kThreads + tid;
                if (idx < nchunk) {
                    float q[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) q[i] = xv[c][i] / s;
                    yr[idx] = pack_e4m3x8(q);
                }
            }
        }
    }
}

// one workgroup per row, row read twice (second pass hits L2 for rows up to 64 KB)
__global__ __launch_bounds__(kThreads) void quant_rows_kernel(const bf16_t* __restrict__ a, int64_t lda,
                                                              uint8_t* __restrict__ q, float* __restrict__ s,
                                                              int64_t rows, int cols) {
    __shared__ float slot_max[2][4];
    int par = 0;
    const int nchunk = cols >> 3;
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const uint4* ar = reinterpret_cast<const uint4*>(a + row * lda);
        float amax = 0.0f;
        for (int idx = threadIdx.x; idx < nchunk; idx += kThreads) {
            float f[8];
            unpack8(ar[idx], f);
#pragma unroll
            for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(f[i]));
        }
        amax = block_reduce<true>(amax, slot_max, par);
        float sc = amax / kE4M3Max;
        if (sc == 0.0f) sc = 1.0f;
        if (threadIdx.x == 0) s[row] = sc;
        uint2* qr = reinterpret_cast<uint2*>(q + row * (int64_t)cols);
        for (int idx = threadIdx.x; idx < nchunk; idx += kThreads) {
            float f[8];
            unpack8(ar[idx], f);
#pragma unroll
            for (int i = 0; i < 8; ++i) f[i] = f[i] / sc;
            qr[idx] = pack_e4m3x8(f);
        }
    }
}

// the same quantisation where the producer of `a` left partial row maxima behind ([rows, n_parts], entry = largest |a|
// of the row within one column range): the row is read once
__global__ __launch_bounds__(kThreads) void quant_rows_parts_kernel(const bf16_t* __restrict__ a, int64_t lda,
                                                                    const float* __restrict__ parts, int64_t ldp, int n_parts,
                                                                    uint8_t* __restrict__ q, float* __restrict__ s,
                                                                    int64_t rows, int cols) {
    __shared__ float slot_max[2][4];
    int par = 0;
    const int nchunk = cols >> 3;
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const uint4* ar = reinterpret_cast<const uint4*>(a + row * lda);
        // the row's first chunks are requested before the maxima are reduced (eight per thread in flight: 32 KB of a row)
        constexpr int PRE = 8;
        uint4 raw[PRE];
#pragma unroll
        for (int c = 0; c < PRE; ++c) {
            const int idx = c * kThreads + threadIdx.x;
            raw[c] = idx < nchunk ? ar[idx] : make_uint4(0, 0, 0, 0);
        }
        float amax = 0.0f;
        for (int i = threadIdx.x; i < n_parts; i += kThreads) amax = fmaxf(amax, parts[row * ldp + i]);
        amax = block_reduce<true>(amax, slot_max, par);
        float sc = amax / kE4M3Max;
        if (sc == 0.0f) sc = 1.0f;
        if (threadIdx.x == 0) s[row] = sc;
        uint2* qr = reinterpret_cast<uint2*>(q + row * (int64_t)cols);
#pragma unroll
        for (int c = 0; c < PRE; ++c) {
            const int idx = c * kThreads + threadIdx.x;
            if (idx < nchunk) {
                float f[8];
                unpack8(raw[c], f);
#pragma unroll
                for (int i = 0; i < 8; ++i) f[i] = f[i] / sc;
                qr[idx] = pack_e4m3x8(f);
            }
        }
        for (int idx = PRE * kThreads + threadIdx.x; idx < nchunk; idx += kThreads) {
            float f[8];
            unpack8(ar[idx], f);
#pragma unroll
            for (int i = 0; i < 8; ++i) f[i] = f[i] / sc;
            qr[idx] = pack_e4m3x8(f);
        }
    }
}

template <bool QUANT, bool XF32>
int32_t launch_norm(const void* x, const void* w, const float* shift, const float* scale, void* y, float* s_tok,
                    int64_t n_tokens, int64_t d, float eps, hipStream_t st) {
    // 64 workgroups per CU's worth of rows in flight: at 56 k rows a workgroup walks over three or four rows.  Measured in
    // the 56,832 x 4096 stack (fp32 rows in, bf16 out): 2048 workgroups 5.37 TB/s, 4096 5.53, 8192 5.63, 16384 5.75, 32768
    // 5.52, one row each 5.04 (the per-channel vectors are then loaded as often as the rows)
    const int64_t max_blocks = 256 * 64;
    const int grid = (int)(n_tokens < max_blocks ? n_tokens : max_blocks);
    const int chunks = (int)((d / 8 + kThreads - 1) / kThreads);
#define CDM_NORM_LAUNCH(C)                                                                                  \
    adaln_rmsnorm_kernel<C, QUANT, XF32><<<grid, kThreads, 0, st>>>(x, (const uint4*)w, shift, scale, y, s_tok, \
                                                                    n_tokens, (int)d, eps)
    if (chunks <= 1) CDM_NORM_LAUNCH(1);
    else if (chunks == 2) CDM_NORM_LAUNCH(2);
    else CDM_NORM_LAUNCH(4);
#undef CDM_NORM_LAUNCH
    return cdm_check_launch("adaln_rmsnorm");
}

int32_t check_norm_args(const void* x, const void* w, const void* y, int64_t n_tokens, int64_t d, const float* shift,
                        const float* scale) {
    CDM_REQUIRE(x && w && y, CDM_ERR_BAD_ARG, "adaln_rmsnorm: null pointer");
    CDM_REQUIRE(n_tokens >= 0 && d > 0, CDM_ERR_BAD_ARG, "adaln_rmsnorm: negative size");
    CDM_REQUIRE(d % 8 == 0 && d <= 8192, CDM_ERR_BAD_SHAPE, "adaln_rmsnorm: d=%lld must be a multiple of 8 and <= 8192",
                (long long)d);
    CDM_REQUIRE(cdm_aligned16(x) && cdm_aligned16(w) && cdm_aligned16(y) && cdm_aligned16(shift) && cdm_aligned16(scale),
                CDM_ERR_BAD_ALIGN, "adaln_rmsnorm: pointers must be 16-byte aligned");
    return CDM_OK;
}

}  // namespace

extern "C" int32_t cdm_adaln_rmsnorm_bf16(const void* x, const void* w, const float* shift, const float* scale,
                                          void* y, int64_t n_tokens, int64_t d, float eps, void* stream) {
    int32_t rc = check_norm_args(x, w, y, n_tokens, d, shift, scale);
    if (rc) return rc;
    if ((rc = cdm_require_device())) return rc;
    if (n_tokens == 0) return CDM_OK;
    return launch_norm<false, false>(x, w, shift, scale, y, nullptr, n_tokens, d, eps, (hipStream_t)stream);
}

extern "C" int32_t cdm_adaln_rmsnorm_f32(const float* x, const void* w, const float* shift, const float* scale,
                                         void* y, int64_t n_tokens, int64_t d, float eps, void* stream) {
    int32_t rc = check_norm_args(x, w, y, n_tokens, d, shift, scale);
    if (rc) return rc;
    if ((rc = cdm_require_device())) return rc;
    if (n_tokens == 0) return CDM_OK;
    return launch_norm<false, true>(x, w, shift, scale, y, nullptr, n_tokens, d, eps, (hipStream_t)stream);
}

extern "C" int32_t cdm_adaln_rmsnorm_quant_e4m3(const void* x, const void* w, const float* shift,
                                                const float* scale, void* yq, float* s_tok, int64_t n_tokens,
                                                int64_t d, float eps, void* stream) {
    int32_t rc = check_norm_args(x, w, yq, n_tokens, d, shift, scale);
    if (rc) return rc;
    CDM_REQUIRE(s_tok, CDM_ERR_BAD_ARG, "adaln_rmsnorm_quant: null s_tok");
    if ((rc = cdm_require_device())) return rc;
    if (n_tokens == 0) return CDM_OK;
    return launch_norm<true, false>(x, w, shift, scale, yq, s_tok, n_tokens, d, eps, (hipStream_t)stream);
}

extern "C" int32_t cdm_adaln_rmsnorm_f32_quant_e4m3(const float* x, const void* w, const float* shift,
                                                    const float* scale, void* yq, float* s_tok, int64_t n_tokens,
                                                    int64_t d, float eps, void* stream) {
    int32_t rc = check_norm_args(x, w, yq, n_tokens, d, shift, scale);
    if (rc) return rc;
    CDM_REQUIRE(s_tok, CDM_ERR_BAD_ARG, "adaln_rmsnorm_quant: null s_tok");
    if ((rc = cdm_require_device())) return rc;
    if (n_tokens == 0) return CDM_OK;
    return launch_norm<true, true>(x, w, shift, scale, yq, s_tok, n_tokens, d, eps, (hipStream_t)stream);
}

extern "C" int32_t cdm_quant_rows_e4m3(const void* a, int64_t lda, void* q, float* s, int64_t rows, int64_t cols,
                                       void* stream) {
    CDM_REQUIRE(a && q && s, CDM_ERR_BAD_ARG, "quant_rows: null pointer");
    CDM_REQUIRE(rows >= 0 && cols > 0 && lda >= cols, CDM_ERR_BAD_ARG, "quant_rows: bad sizes");
    CDM_REQUIRE(cols % 8 == 0 && cols <= 32768, CDM_ERR_BAD_SHAPE, "quant_rows: cols=%lld must be a multiple of 8 and <= 32768",
                (long long)cols);
    CDM_REQUIRE(cdm_aligned16(a) && cdm_aligned16(q) && (lda % 8 == 0), CDM_ERR_BAD_ALIGN,
                "quant_rows: pointers/strides must be 16-byte aligned");
    int32_t rc = cdm_require_device();
    if (rc) return rc;
    if (rows == 0) return CDM_OK;
    // one row per workgroup: nothing is set up per workgroup, and rows then stream in address order (56,832 x 4096 and
    // x 16384 bf16 rows: 6.0 TB/s against 5.2 with 2048 workgroups walking over the rows, 5.8 with 8192)
    const int64_t max_blocks = (1ll << 31) - 1;
    const int grid = (int)(rows < max_blocks ? rows : max_blocks);
    quant_rows_kernel<<<grid, kThreads, 0, (hipStream_t)stream>>>((const bf16_t*)a, lda, (uint8_t*)q, s, rows,
                                                                  (int)cols);
    return cdm_check_launch("quant_rows");
}

extern "C" int32_t cdm_quant_rows_from_parts_e4m3(const void* a, int64_t lda, const float* parts, int64_t ldp,
                                                  int64_t n_parts, void* q, float* s, int64_t rows, int64_t cols,
                                                  void* stream) {
    CDM_REQUIRE(a && q && s && parts, CDM_ERR_BAD_ARG, "quant_rows_from_parts: null pointer");
    CDM_REQUIRE(rows >= 0 && cols > 0 && lda >= cols, CDM_ERR_BAD_ARG, "quant_rows_from_parts: bad sizes");
    CDM_REQUIRE(n_parts >= 1 && n_parts <= 4096 && ldp >= n_parts, CDM_ERR_BAD_ARG,
                "quant_rows_from_parts: n_parts=%lld must be 1..4096 with ldp >= n_parts", (long long)n_parts);
    CDM_REQUIRE(cols % 8 == 0 && cols <= 32768, CDM_ERR_BAD_SHAPE,
                "quant_rows_from_parts: cols=%lld must be a multiple of 8 and <= 32768", (long long)cols);
    CDM_REQUIRE(cdm_aligned16(a) && cdm_aligned16(q) && (lda % 8 == 0) && (reinterpret_cast<uintptr_t>(parts) & 3u) == 0,
                CDM_ERR_BAD_ALIGN, "quant_rows_from_parts: pointers/strides must be 16-byte aligned (parts: 4-byte)");
    int32_t rc = cdm_require_device();
    if (rc) return rc;
    if (rows == 0) return CDM_OK;
    // one row per workgroup: nothing is set up per workgroup, and rows then stream in address order (56,832 x 4096 and
    // x 16384 bf16 rows: 6.0 TB/s against 5.2 with 2048 workgroups walking over the rows, 5.8 with 8192)
    const int64_t max_blocks = (1ll << 31) - 1;
    const int grid = (int)(rows < max_blocks ? rows : max_blocks);
    quant_rows_parts_kernel<<<grid, kThreads, 0, (hipStream_t)stream>>>((const bf16_t*)a, lda, parts, ldp, (int)n_parts,
                                                                        (uint8_t*)q, s, rows, (int)cols);
    return cdm_check_launch("quant_rows_from_parts");
}

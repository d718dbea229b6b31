// The elementwise step either side of the transformer forward inside a denoising iteration: classifier-free
// guidance combine of the conditional / unconditional predictions, fused with the scheduler's linear update of
// the latents (HBM-bound; one pass instead of one pass per term).
#include "cdm_common.h"

namespace {

constexpr int kMaxHist = 4;
constexpr int kMaxOut = 3;

struct StepParams {
    const float* x;
    const bf16_t* vc;
    const bf16_t* vu;          // null = no guidance (v = vc)
    const float* hist[kMaxHist];
    float c[kMaxOut][2 + kMaxHist];      // row j: coefficients of output j for (x, v, hist[0..])
    float* out[kMaxOut];
    int n_hist, n_out;
    float guidance;
    int64_t n;
};

__device__ __forceinline__ float combine(float c, float u, float g, bool guided) { return guided ? u + g * (c - u) : c; }

// 4 elements per thread per iteration: 8-byte loads of the bf16 predictions, 16-byte loads/stores of the fp32 tensors.
// Every input element is read before any output element of the same index is written and elements are independent,
// so an output may be the very tensor of an input (the latents in place, a history slot being recycled).
__global__ __launch_bounds__(256) void cfg_step_kernel(const StepParams p) {
    const bool guided = p.vu != nullptr;
    const int64_t n4 = p.n >> 2;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        const uint2 c2 = reinterpret_cast<const uint2*>(p.vc)[i];
        uint2 u2 = c2;
        if (guided) u2 = reinterpret_cast<const uint2*>(p.vu)[i];
        const float4 x4 = reinterpret_cast<const float4*>(p.x)[i];
        const float x[4] = {x4.x, x4.y, x4.z, x4.w};
        const float v[4] = {combine(bf16lo(c2.x), bf16lo(u2.x), p.guidance, guided), combine(bf16hi(c2.x), bf16hi(u2.x), p.guidance, guided),
                            combine(bf16lo(c2.y), bf16lo(u2.y), p.guidance, guided), combine(bf16hi(c2.y), bf16hi(u2.y), p.guidance, guided)};
        float h[kMaxHist][4];
#pragma unroll
        for (int k = 0; k < kMaxHist; ++k)
            if (k < p.n_hist) {
                const float4 h4 = reinterpret_cast<const float4*>(p.hist[k])[i];
                h[k][0] = h4.x; h[k][1] = h4.y; h[k][2] = h4.z; h[k][3] = h4.w;
            }
#pragma unroll
        for (int j = 0; j < kMaxOut; ++j)
            if (j < p.n_out) {
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = p.c[j][0] * x[e] + p.c[j][1] * v[e];
#pragma unroll
                for (int k = 0; k < kMaxHist; ++k)
                    if (k < p.n_hist) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) o[e] += p.c[j][2 + k] * h[k][e];
                    }
                reinterpret_cast<float4*>(p.out[j])[i] = make_float4(o[0], o[1], o[2], o[3]);
            }
    }
    // tail (n % 4 elements), one thread each
    const int64_t t = (n4 << 2) + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < p.n) {
        const float c = bf16_bits_to_f32(p.vc[t]);
        const float u = guided ? bf16_bits_to_f32(p.vu[t]) : c;
        const float v = combine(c, u, p.guidance, guided);
        const float x = p.x[t];
        float h[kMaxHist];
        for (int k = 0; k < p.n_hist; ++k) h[k] = p.hist[k][t];
        for (int j = 0; j < p.n_out; ++j) {
            float o = p.c[j][0] * x + p.c[j][1] * v;
            for (int k = 0; k < p.n_hist; ++k) o += p.c[j][2 + k] * h[k];
            p.out[j][t] = o;
        }
    }
}

}  // namespace

extern "C" int32_t cdm_cfg_step_f32(const float* x, const void* v_cond, const void* v_uncond, float guidance,
                                    const float* const* hist, int32_t n_hist, const float* coef, float* const* outs,
                                    int32_t n_out, int64_t n, void* stream) {
    CDM_REQUIRE(x && v_cond && outs && coef, CDM_ERR_BAD_ARG, "cfg_step: null pointer");
    CDM_REQUIRE(n >= 0, CDM_ERR_BAD_ARG, "cfg_step: negative size");
    CDM_REQUIRE(n_hist >= 0 && n_hist <= kMaxHist, CDM_ERR_BAD_ARG, "cfg_step: n_hist=%d must be 0..%d", n_hist, kMaxHist);
    CDM_REQUIRE(n_out >= 1 && n_out <= kMaxOut, CDM_ERR_BAD_ARG, "cfg_step: n_out=%d must be 1..%d", n_out, kMaxOut);
    CDM_REQUIRE(n_hist == 0 || hist, CDM_ERR_BAD_ARG, "cfg_step: history pointers missing");
    CDM_REQUIRE(cdm_aligned16(x) && cdm_aligned16(v_cond) && cdm_aligned16(v_uncond), CDM_ERR_BAD_ALIGN,
                "cfg_step: pointers must be 16-byte aligned");
    StepParams p{};
    p.x = x; p.vc = (const bf16_t*)v_cond; p.vu = (const bf16_t*)v_uncond;
    for (int h = 0; h < n_hist; ++h) {
        CDM_REQUIRE(hist[h] && cdm_aligned16(hist[h]), CDM_ERR_BAD_ARG, "cfg_step: history tensor %d null or misaligned", h);
        p.hist[h] = hist[h];
    }
    for (int j = 0; j < n_out; ++j) {
        CDM_REQUIRE(outs[j] && cdm_aligned16(outs[j]), CDM_ERR_BAD_ARG, "cfg_step: output tensor %d null or misaligned", j);
        for (int k = 0; k < j; ++k) CDM_REQUIRE(outs[j] != outs[k], CDM_ERR_BAD_ARG, "cfg_step: outputs %d and %d coincide", k, j);
        p.out[j] = outs[j];
        for (int k = 0; k < 2 + n_hist; ++k) p.c[j][k] = coef[j * (2 + n_hist) + k];
    }
    p.n_hist = n_hist; p.n_out = n_out; p.guidance = guidance; p.n = n;
    if (n == 0) return CDM_OK;
    int32_t rc = cdm_require_device();
    if (rc) return rc;
    const int64_t work = (n + 3) / 4;
    int64_t blocks = (work + 255) / 256;
    if (blocks > 256 * 256) blocks = 256 * 256;      // measured on the update of 2^26 values: 4096 workgroups 5.0 - 5.1 TB/s, 16384 5.2 - 5.3, 65536 5.5 - 5.7
    if (blocks < 1) blocks = 1;
    cfg_step_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(p);
    return cdm_check_launch("cfg_step");
}

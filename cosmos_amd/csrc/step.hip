// The elementwise step either side of the transformer forward inside a denoising iteration: classifier-free
// guidance combine of the conditional / unconditional predictions, fused with the scheduler's linear update of
// the latents (HBM-bound; one pass instead of one pass per term).
#include "cdm_common.h"

namespace {

constexpr int kMaxHist = 4;

struct StepParams {
    const float* x;
    const bf16_t* vc;
    const bf16_t* vu;          // null = no guidance (v = vc)
    const float* hist[kMaxHist];
    float c_x, c_v, c_h[kMaxHist];
    int n_hist;
    float guidance;
    float* v_out;              // null or the combined prediction (fp32), the next call's history
    float* out;
    int64_t n;
};

__device__ __forceinline__ float combine(float c, float u, float g, bool guided) { return guided ? u + g * (c - u) : c; }

// 4 elements per thread per iteration: 8-byte loads of the bf16 predictions, 16-byte loads/stores of the fp32 tensors
__global__ __launch_bounds__(256) void cfg_step_kernel(const StepParams p) {
    const bool guided = p.vu != nullptr;
    const int64_t n4 = p.n >> 2;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        const uint2 c2 = reinterpret_cast<const uint2*>(p.vc)[i];
        uint2 u2 = c2;
        if (guided) u2 = reinterpret_cast<const uint2*>(p.vu)[i];
        const float4 x4 = reinterpret_cast<const float4*>(p.x)[i];
        float v[4] = {combine(bf16lo(c2.x), bf16lo(u2.x), p.guidance, guided), combine(bf16hi(c2.x), bf16hi(u2.x), p.guidance, guided),
                      combine(bf16lo(c2.y), bf16lo(u2.y), p.guidance, guided), combine(bf16hi(c2.y), bf16hi(u2.y), p.guidance, guided)};
        float o[4] = {p.c_x * x4.x + p.c_v * v[0], p.c_x * x4.y + p.c_v * v[1], p.c_x * x4.z + p.c_v * v[2],
                      p.c_x * x4.w + p.c_v * v[3]};
#pragma unroll
        for (int h = 0; h < kMaxHist; ++h)
            if (h < p.n_hist) {
                const float4 h4 = reinterpret_cast<const float4*>(p.hist[h])[i];
                o[0] += p.c_h[h] * h4.x; o[1] += p.c_h[h] * h4.y; o[2] += p.c_h[h] * h4.z; o[3] += p.c_h[h] * h4.w;
            }
        if (p.v_out) reinterpret_cast<float4*>(p.v_out)[i] = make_float4(v[0], v[1], v[2], v[3]);
        reinterpret_cast<float4*>(p.out)[i] = make_float4(o[0], o[1], o[2], o[3]);
    }
    // tail (n % 4 elements), one thread each
    const int64_t t = (n4 << 2) + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < p.n) {
        const float c = bf16_bits_to_f32(p.vc[t]);
        const float u = guided ? bf16_bits_to_f32(p.vu[t]) : c;
        const float v = combine(c, u, p.guidance, guided);
        float o = p.c_x * p.x[t] + p.c_v * v;
        for (int h = 0; h < p.n_hist; ++h) o += p.c_h[h] * p.hist[h][t];
        if (p.v_out) p.v_out[t] = v;
        p.out[t] = o;
    }
}

}  // namespace

extern "C" int32_t cdm_cfg_step_f32(const float* x, const void* v_cond, const void* v_uncond, float guidance,
                                    const float* const* hist, const float* coef, int32_t n_hist, float* v_out,
                                    float* out, int64_t n, void* stream) {
    CDM_REQUIRE(x && v_cond && out && coef, CDM_ERR_BAD_ARG, "cfg_step: null pointer");
    CDM_REQUIRE(n >= 0, CDM_ERR_BAD_ARG, "cfg_step: negative size");
    CDM_REQUIRE(n_hist >= 0 && n_hist <= kMaxHist, CDM_ERR_BAD_ARG, "cfg_step: n_hist=%d must be 0..%d", n_hist, kMaxHist);
    CDM_REQUIRE(n_hist == 0 || hist, CDM_ERR_BAD_ARG, "cfg_step: history pointers missing");
    CDM_REQUIRE(cdm_aligned16(x) && cdm_aligned16(v_cond) && cdm_aligned16(v_uncond) && cdm_aligned16(out) &&
                    cdm_aligned16(v_out),
                CDM_ERR_BAD_ALIGN, "cfg_step: pointers must be 16-byte aligned");
    StepParams p{};
    p.x = x; p.vc = (const bf16_t*)v_cond; p.vu = (const bf16_t*)v_uncond;
    p.c_x = coef[0]; p.c_v = coef[1];
    for (int h = 0; h < n_hist; ++h) {
        CDM_REQUIRE(hist[h] && cdm_aligned16(hist[h]), CDM_ERR_BAD_ARG, "cfg_step: history tensor %d null or misaligned", h);
        p.hist[h] = hist[h];
        p.c_h[h] = coef[2 + h];
    }
    p.n_hist = n_hist; p.guidance = guidance; p.v_out = v_out; p.out = out; p.n = n;
    if (n == 0) return CDM_OK;
    int32_t rc = cdm_require_device();
    if (rc) return rc;
    const int64_t work = (n + 3) / 4;
    int64_t blocks = (work + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    if (blocks < 1) blocks = 1;
    cfg_step_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(p);
    return cdm_check_launch("cfg_step");
}

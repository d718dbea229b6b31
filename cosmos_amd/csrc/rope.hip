// Standalone rotate-half mRoPE on Q and K (in place): an HBM-bound streaming kernel.
#include "cdm_common.h"

namespace {

// One thread rotates 8 pairs (i..i+7, i+half..i+half+7) of one head of one token.
// items per token = n_heads * head_dim / 16; Q and K are both handled by the same thread.
__global__ __launch_bounds__(256) void mrope_qk_kernel(bf16_t* __restrict__ q, int64_t ldq, bf16_t* __restrict__ k,
                                                       int64_t ldk, const float* __restrict__ cos,
                                                       const float* __restrict__ sin, int64_t n_tokens, int n_heads,
                                                       int head_dim) {
    const int half = head_dim >> 1;
    const int per_head = half >> 3;                 // 8-pair groups per head
    const int per_tok = n_heads * per_head;
    const int64_t total = n_tokens * per_tok;
    for (int64_t it = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; it < total;
         it += (int64_t)gridDim.x * blockDim.x) {
        const int64_t tok = it / per_tok;
        const int r = (int)(it - tok * per_tok);
        const int head = r / per_head;
        const int g = r - head * per_head;
        const float4* cp = reinterpret_cast<const float4*>(cos + tok * half + g * 8);
        const float4* sp = reinterpret_cast<const float4*>(sin + tok * half + g * 8);
        const float4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
        const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
        const float s[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
        for (int which = 0; which < 2; ++which) {
            bf16_t* base = which == 0 ? q : k;
            if (base == nullptr) continue;
            const int64_t ld = which == 0 ? ldq : ldk;
            uint4* p1 = reinterpret_cast<uint4*>(base + tok * ld + head * head_dim + g * 8);
            uint4* p2 = reinterpret_cast<uint4*>(base + tok * ld + head * head_dim + half + g * 8);
            const uint4 u1 = *p1, u2 = *p2;
            const uint32_t w1[4] = {u1.x, u1.y, u1.z, u1.w}, w2[4] = {u2.x, u2.y, u2.z, u2.w};
            uint32_t o1[4], o2[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float a0 = bf16lo(w1[j]), a1 = bf16hi(w1[j]);
                const float b0 = bf16lo(w2[j]), b1 = bf16hi(w2[j]);
                o1[j] = pack_bf16x2(a0 * c[2 * j] - b0 * s[2 * j], a1 * c[2 * j + 1] - b1 * s[2 * j + 1]);
                o2[j] = pack_bf16x2(b0 * c[2 * j] + a0 * s[2 * j], b1 * c[2 * j + 1] + a1 * s[2 * j + 1]);
            }
            *p1 = make_uint4(o1[0], o1[1], o1[2], o1[3]);
            *p2 = make_uint4(o2[0], o2[1], o2[2], o2[3]);
        }
    }
}

}  // namespace

extern "C" int32_t cdm_mrope_qk_bf16(void* q, int64_t ldq, void* k, int64_t ldk, const float* cos, const float* sin,
                                     int64_t n_tokens, int32_t n_heads, int32_t head_dim, void* stream) {
    CDM_REQUIRE(q && cos && sin, CDM_ERR_BAD_ARG, "mrope_qk: null pointer");
    CDM_REQUIRE(n_tokens >= 0 && n_heads > 0, CDM_ERR_BAD_ARG, "mrope_qk: bad sizes");
    CDM_REQUIRE(head_dim == 64 || head_dim == 128, CDM_ERR_BAD_SHAPE, "mrope_qk: head_dim=%d must be 64 or 128", head_dim);
    CDM_REQUIRE(ldq >= (int64_t)n_heads * head_dim && (!k || ldk >= (int64_t)n_heads * head_dim), CDM_ERR_BAD_ARG,
                "mrope_qk: row stride smaller than n_heads*head_dim");
    CDM_REQUIRE(cdm_aligned16(q) && cdm_aligned16(k) && cdm_aligned16(cos) && cdm_aligned16(sin) && ldq % 8 == 0 &&
                    ldk % 8 == 0,
                CDM_ERR_BAD_ALIGN, "mrope_qk: pointers/strides must be 16-byte aligned");
    int32_t rc = cdm_require_device();
    if (rc) return rc;
    if (n_tokens == 0) return CDM_OK;
    const int64_t total = n_tokens * n_heads * (head_dim / 16);
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 256) blocks = 256 * 256;      // measured on the in-place rotation of 56,320 x 4096 Q and K: 4096 workgroups 5.0 - 5.1 TB/s, 16384 5.2 - 5.3, 65536 5.5 - 5.7
    mrope_qk_kernel<<<(int)blocks, 256, 0, (hipStream_t)stream>>>((bf16_t*)q, ldq, (bf16_t*)k, ldk, cos, sin,
                                                                  n_tokens, n_heads, head_dim);
    return cdm_check_launch("mrope_qk");
}

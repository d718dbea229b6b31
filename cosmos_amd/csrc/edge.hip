// Linear layers at the edges of the stack: patchify / un-patchify projections and the action / audio projections
// (proj_in, proj_out, action_proj_in/out, audio_proj_in/out: nn.Linear WITH bias, one side of the product only a few
// dozen elements wide).  Such a layer moves the token rows once - it is bound by HBM, not by the matrix cores - and has
// K or N far below what the tiled GEMM needs, so it gets a small kernel of its own: 64 token rows per workgroup, all
// output columns walked in passes, operands staged through LDS in 256-byte row pieces.
#include "cdm_common.h"

namespace {

constexpr int EM = 64;        // token rows per workgroup (4 waves x 16)

struct EdgeParams {
    const bf16_t* A; int64_t lda;
    const bf16_t* W; int64_t ldw;
    const bf16_t* bias;          // [N] or null
    bf16_t* C; int64_t ldc;
    int M, N, K;
    int passes_per_wg;           // column passes per workgroup (blockIdx.y selects the range)
};

// 8 bf16 of a row from column k on; columns >= K read as zero.  Rows are never masked: callers clamp the row pointer
// into the matrix, and what a row outside it contributes only reaches output rows / columns that are not stored.
// VEC: one 16-byte load (K % 8 == 0, so a chunk is in or out as a whole, and rows start on 16-byte boundaries);
// otherwise element by element (widths like 6 or 10: the action and audio streams of small configurations).
template <bool VEC>
__device__ __forceinline__ uint4 load_chunk(const bf16_t* rowp, int k, int K) {
    if constexpr (VEC) {
        const uint4 v = *reinterpret_cast<const uint4*>(rowp + (k < K ? k : 0));
        const bool in = k < K;
        return make_uint4(in ? v.x : 0u, in ? v.y : 0u, in ? v.z : 0u, in ? v.w : 0u);
    } else {
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k0 = k + 2 * e, k1 = k + 2 * e + 1;
            const uint32_t lo = rowp[k0 < K ? k0 : 0], hi = rowp[k1 < K ? k1 : 0];
            w[e] = (k0 < K ? lo : 0u) | ((k1 < K ? hi : 0u) << 16);
        }
        return make_uint4(w[0], w[1], w[2], w[3]);
    }
}

// NB = 16-column blocks per pass (4: N <= 64, 8 otherwise); KC = k elements per staged chunk (64 where K <= 64, else
// 128).  A workgroup owns 64 token rows and walks over the output columns 16 NB at a time (a pass) and, inside a pass,
// over K in chunks of KC.  Both operands of a chunk travel global -> registers -> LDS with whole 2 KC-byte row pieces per
// 8 or 16 lanes (a fragment read straight from global memory would touch 16 rows per 16 lanes: four times the tag
// look-ups) and are read back as MFMA fragments; the loads of the next chunk are in flight while the matrix cores work
// on the present one, and where K is a single chunk the A rows stay in LDS for all passes.  A pass leaves through
// wave-private staging rows, 32 NB bytes of each of the wave's 16 rows at a time.
template <int NB, int KC, bool VEC>
__global__ __launch_bounds__(256) void edge_linear_kernel(const EdgeParams p) {
    constexpr int WR = NB * 16;                              // W rows (output columns) per pass
    constexpr int PPR = KC / 8, RPL = 256 / PPR;             // 16-byte pieces per staged row; rows per load of all threads
    constexpr int LPITCH = KC * 2 + 16;                      // bytes per staged operand row: 16 rows of one fragment read fall on distinct banks
    constexpr int A_LD = EM / RPL, W_LD = WR / RPL;          // 16-byte loads per thread and chunk
    constexpr int CPITCH = NB * 32 + 16;                     // bytes per staged output row
    // a narrow output (one pass) stages its rows over the W chunk, behind one more barrier: 35 KB of LDS, four workgroups per CU
    constexpr bool C_OVER_W = NB == 4;
    static_assert(!C_OVER_W || EM * CPITCH <= WR * LPITCH, "staged output rows exceed the W chunk");
    __shared__ __attribute__((aligned(16))) char smem[EM * LPITCH + WR * LPITCH + (C_OVER_W ? 0 : EM * CPITCH)];
    char* const s_a = smem;
    char* const s_w = smem + EM * LPITCH;
    char* const s_c = C_OVER_W ? s_w : s_w + WR * LPITCH;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;
    const int m0 = blockIdx.x * EM;
    const int chunks = (p.K + KC - 1) / KC;
    // this workgroup's range of column passes (few token rows: the passes are dealt over blockIdx.y)
    const int n_lo = blockIdx.y * p.passes_per_wg * WR;
    const int n_hi = min(p.N, n_lo + p.passes_per_wg * WR);
    const int passes = (n_hi - n_lo + WR - 1) / WR;
    // Rows of C are a power of two apart in the shapes this kernel is for (8 KB at d = 4096): workgroups that walk the
    // columns in the same order would all write through the same memory channel at the same time, so each starts its
    // walk somewhere else and wraps around.
    int n0 = n_lo + (int)(blockIdx.x % (unsigned)passes) * WR;

    // loader role of this thread: row lr (+ 16 per further load) and 16-byte piece lc of the chunk
    const int lr = tid / PPR, lc = tid % PPR;
    uint4 ra[A_LD], rw[W_LD];
    const bool a_stays = chunks == 1;                         // the A rows of the only chunk are staged once
    auto fetch = [&](int n_at, int kc, bool with_a) {
        const int k = kc * KC + lc * 8;
        if (with_a) {
#pragma unroll
            for (int i = 0; i < A_LD; ++i) {
                const int m = m0 + lr + RPL * i;
                ra[i] = load_chunk<VEC>(p.A + (int64_t)(m < p.M ? m : p.M - 1) * p.lda, k, p.K);
            }
        }
#pragma unroll
        for (int i = 0; i < W_LD; ++i) {
            const int n = n_at + lr + RPL * i;
            rw[i] = load_chunk<VEC>(p.W + (int64_t)(n < p.N ? n : p.N - 1) * p.ldw, k, p.K);
        }
    };
    auto stash = [&](bool with_a) {
        if (with_a) {
#pragma unroll
            for (int i = 0; i < A_LD; ++i) *reinterpret_cast<uint4*>(s_a + (lr + RPL * i) * LPITCH + lc * 16) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < W_LD; ++i) *reinterpret_cast<uint4*>(s_w + (lr + RPL * i) * LPITCH + lc * 16) = rw[i];
    };

    fetch(n0, 0, true);
    for (int pass = 0; pass < passes; ++pass) {
        const int n_next = n0 + WR < n_hi ? n0 + WR : n_lo;
        f32x4 acc[NB];
        // the pass's bias values go out ahead of the next chunk's loads: waiting for them in the epilogue then does not
        // wait for those (loads return in order)
        uint2 braw[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};
            braw[nb] = make_uint2(0u, 0u);
            const int n = n0 + 16 * nb + 4 * g4;
            if (p.bias != nullptr) {
                if constexpr (VEC) {      // N % 8 == 0: four columns are in or out together; bias is 8-byte aligned
                    braw[nb] = *reinterpret_cast<const uint2*>(p.bias + (n < p.N ? n : 0));
                } else {
                    uint32_t v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = p.bias[n + e < p.N ? n + e : 0];
                    braw[nb] = make_uint2(v[0] | (v[1] << 16), v[2] | (v[3] << 16));
                }
            }
        }
        for (int kc = 0; kc < chunks; ++kc) {
            __syncthreads();                                  // every wave is done with the chunk in LDS (and with s_c)
            stash(!a_stays || pass == 0);
            __syncthreads();
            if (kc + 1 < chunks) fetch(n0, kc + 1, true);
            else if (pass + 1 < passes) fetch(n_next, 0, !a_stays);
            // D[i][j] = sum_k W[n0 + 16 nb + i][k] A[row_j][k]: the lane then owns ONE token row (j = lane % 16) and
            // four consecutive output columns per block (i = 4 (lane / 16) + e)
            const int ksteps = (min(p.K - kc * KC, KC) + 31) >> 5;
            for (int ks = 0; ks < ksteps; ++ks) {
                const bf16x8 a = *reinterpret_cast<const bf16x8*>(s_a + (wave * 16 + r16) * LPITCH + (4 * ks + g4) * 16);
                bf16x8 w[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    w[nb] = *reinterpret_cast<const bf16x8*>(s_w + (16 * nb + r16) * LPITCH + (4 * ks + g4) * 16);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[nb], a, acc[nb], 0, 0, 0);
            }
        }
        // bias, one rounding to bf16, staged as rows (wave-private rows of s_c: no workgroup barrier needed here; the
        // barrier at the top of the next chunk orders the next pass's staging after this pass's reads)
        if constexpr (C_OVER_W) __syncthreads();             // every wave is done with the W chunk the rows are staged over
        char* stage = s_c + wave * (16 * CPITCH);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const float b[4] = {bf16lo(braw[nb].x), bf16hi(braw[nb].x), bf16lo(braw[nb].y), bf16hi(braw[nb].y)};
            uint2 o;
            o.x = pack_bf16x2(acc[nb][0] + b[0], acc[nb][1] + b[1]);
            o.y = pack_bf16x2(acc[nb][2] + b[2], acc[nb][3] + b[3]);
            *reinterpret_cast<uint2*>(stage + r16 * CPITCH + (16 * nb + 4 * g4) * 2) = o;
        }
        __builtin_amdgcn_wave_barrier();
        constexpr int CPR = NB * 2;                          // 16-byte pieces per staged row
#pragma unroll
        for (int idx = lane; idx < 16 * CPR; idx += 64) {
            const int r = idx / CPR, c = idx % CPR;
            const int m = m0 + wave * 16 + r, n = n0 + c * 8;
            if (m >= p.M || n >= p.N) continue;
            if constexpr (VEC) {      // N % 8 == 0 and rows of C start on 16-byte boundaries
                *reinterpret_cast<uint4*>(p.C + (int64_t)m * p.ldc + n) = *reinterpret_cast<const uint4*>(stage + r * CPITCH + c * 16);
            } else {
                const bf16_t* src = reinterpret_cast<const bf16_t*>(stage + r * CPITCH + c * 16);
                for (int e = 0; e < 8 && n + e < p.N; ++e) p.C[(int64_t)m * p.ldc + n + e] = src[e];
            }
        }
        n0 = n_next;
    }
}

}  // namespace

extern "C" int32_t cdm_linear_bias_bf16(const void* A, int64_t lda, const void* W, int64_t ldw, const void* bias, void* C,
                                        int64_t ldc, int64_t M, int64_t N, int64_t K, void* stream) {
    CDM_REQUIRE(A && W && C, CDM_ERR_BAD_ARG, "linear_bias: null pointer");
    CDM_REQUIRE(M >= 0 && N > 0 && K > 0, CDM_ERR_BAD_ARG, "linear_bias: bad sizes M=%lld N=%lld K=%lld", (long long)M,
                (long long)N, (long long)K);
    CDM_REQUIRE(M < (1ll << 31) - EM && N < (1ll << 22) && K < (1ll << 24), CDM_ERR_BAD_SHAPE, "linear_bias: sizes out of range");
    CDM_REQUIRE(lda >= K && ldw >= K && ldc >= N, CDM_ERR_BAD_ARG, "linear_bias: row stride smaller than row length");
    CDM_REQUIRE(((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(W) | reinterpret_cast<uintptr_t>(C) |
                  reinterpret_cast<uintptr_t>(bias)) & 1u) == 0,
                CDM_ERR_BAD_ALIGN, "linear_bias: pointers must be 2-byte aligned");
    // 16-byte accesses where every row of A, W and C starts on a 16-byte boundary and K, N are multiples of 8
    const bool vec = cdm_aligned16(A) && cdm_aligned16(W) && cdm_aligned16(C) && lda % 8 == 0 && ldw % 8 == 0 && ldc % 8 == 0 &&
                     N % 8 == 0 && K % 8 == 0 && (reinterpret_cast<uintptr_t>(bias) & 7u) == 0;
    if (M == 0) return CDM_OK;
    int32_t rc = cdm_require_device();
    if (rc) return rc;
    EdgeParams p{(const bf16_t*)A, lda, (const bf16_t*)W, ldw, (const bf16_t*)bias, (bf16_t*)C, ldc, (int)M, (int)N, (int)K, 1};
    hipStream_t st = (hipStream_t)stream;
    const int64_t gx = (M + EM - 1) / EM;
    const int wr = N <= 64 ? 64 : 128;
    const int64_t passes = (N + wr - 1) / wr;
    // a workgroup walks all column passes of its rows (whole rows of C per workgroup) unless the rows are too few to fill
    // the chip: then the passes are dealt over a second grid dimension, up to about four workgroups per CU
    int64_t gy = gx >= 1024 ? 1 : (1024 + gx - 1) / gx;
    if (gy > passes) gy = passes;
    p.passes_per_wg = (int)((passes + gy - 1) / gy);
    gy = (passes + p.passes_per_wg - 1) / p.passes_per_wg;
    const dim3 grid((unsigned)gx, (unsigned)gy);
#define CDM_EDGE_LAUNCH(NB_, KC_)                                                             \
    if (vec) edge_linear_kernel<NB_, KC_, true><<<grid, 256, 0, st>>>(p);                     \
    else edge_linear_kernel<NB_, KC_, false><<<grid, 256, 0, st>>>(p)
    if (N <= 64 && K <= 64) { CDM_EDGE_LAUNCH(4, 64); }
    else if (N <= 64) { CDM_EDGE_LAUNCH(4, 128); }
    else if (K <= 64) { CDM_EDGE_LAUNCH(8, 64); }
    else { CDM_EDGE_LAUNCH(8, 128); }
#undef CDM_EDGE_LAUNCH
    return cdm_check_launch("linear_bias");
}

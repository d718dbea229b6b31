// Non-causal full self-attention (flash-style, online softmax) on the gfx950 matrix cores.
//
// Work split: one workgroup owns 256 query rows of one head and streams all keys in tiles of 64.
// Each wave owns 32*QSUB query rows.  Scores are computed TRANSPOSED, S^T = K . Q^T, with
// v_mfma_f32_32x32x16_bf16: the A operand is a K tile row (plain 16-byte LDS read), the B operand
// is Q held in registers for the whole kernel.  In the accumulator layout every lane then owns ONE
// query column and 16 keys per 32-key block, so the row max / row sum of the online softmax are
// in-lane reductions plus one exchange between the two half-waves.  The probabilities never move
// between lanes: packed to bf16 they are already the B operand of O^T += V^T . P^T, whose A operand
// is a row of V^T (V is transposed once per call into the caller's workspace, [head][dh][token]).
// The K rows of a 32-key block are fetched in a permuted order so that the 8 keys a lane holds in
// accumulator registers 8j..8j+7 are the 8 consecutive keys the second product expects.
// K and V^T tiles go global -> LDS directly (global_load_lds_dwordx4), double buffered, with an
// XOR swizzle applied on the source side so fragment reads are bank-conflict free.
#include "cdm_common.h"

namespace {

constexpr int BN = 64;       // keys per tile
constexpr int BMQ = 256;     // query rows per workgroup
typedef __attribute__((address_space(3))) void lds_void;

template <int CHUNKS>
__device__ __forceinline__ int swz(int row) {
    return CHUNKS == 16 ? (row & 15) : ((row ^ (row >> 3)) & 7);
}

// row permutation inside a 32-key block: MFMA output row i holds key pi(i)
__device__ __forceinline__ int key_perm(int i) {
    const int g = i >> 3, b = (i >> 2) & 1, r = i & 3;
    return 16 * (g >> 1) + 8 * b + 4 * (g & 1) + r;
}

struct AttnParams {
    const bf16_t* q; int64_t ldq;
    const bf16_t* k; int64_t ldk;
    const bf16_t* vt;            // [n_heads][HD][n_pad]
    bf16_t* o; int64_t ldo;
    int n_tokens, n_pad, n_heads;
    float scale_log2e;           // log2(e) / sqrt(HD)
};

template <int HD, int QSUB, int NW>
struct Cfg {
    static constexpr int KCH = HD / 8;                   // 16-byte chunks per K tile row
    static constexpr int K_TILE_BYTES = BN * HD * 2;
    static constexpr int V_TILE_BYTES = HD * BN * 2;
    static constexpr int K_INSTR = K_TILE_BYTES / 1024;  // wave-level direct-to-LDS instructions per tile
    static constexpr int V_INSTR = V_TILE_BYTES / 1024;
    static constexpr int K_PER_WAVE = K_INSTR / NW;
    static constexpr int V_PER_WAVE = V_INSTR / NW;
    static constexpr int K_ROWS_PER_INSTR = 64 / KCH;    // 4 (HD=128) or 8 (HD=64)
    static_assert(K_INSTR % NW == 0 && V_INSTR % NW == 0, "tile loads must divide over the waves");
};

template <int HD, int QSUB, int NW>
__device__ __forceinline__ void issue_tile(const char* kbase, const char* vbase,
                                           const uint32_t (&ko)[Cfg<HD, QSUB, NW>::K_PER_WAVE],
                                           const uint32_t (&vo)[Cfg<HD, QSUB, NW>::V_PER_WAVE], char* sk, char* sv,
                                           int wave) {
    using C = Cfg<HD, QSUB, NW>;
#pragma unroll
    for (int i = 0; i < C::K_PER_WAVE; ++i)
        __builtin_amdgcn_global_load_lds(kbase + ko[i], (lds_void*)(sk + (i * NW + wave) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < C::V_PER_WAVE; ++i)
        __builtin_amdgcn_global_load_lds(vbase + vo[i], (lds_void*)(sv + (i * NW + wave) * 1024), 16, 0, 0);
}

template <int HD, int QSUB, int NW>
__device__ __forceinline__ void k_offsets(int wave, int lane, int64_t ldk, int rows_valid,
                                          uint32_t (&ko)[Cfg<HD, QSUB, NW>::K_PER_WAVE]) {
    using C = Cfg<HD, QSUB, NW>;
#pragma unroll
    for (int i = 0; i < C::K_PER_WAVE; ++i) {
        const int row = (i * NW + wave) * C::K_ROWS_PER_INSTR + lane / C::KCH;
        const int chunk = (lane % C::KCH) ^ swz<C::KCH>(row);
        const int rr = row < rows_valid ? row : rows_valid - 1;
        ko[i] = (uint32_t)(rr * (int)ldk + chunk * 8) * 2u;
    }
}

// One key tile: S^T = K Q^T, online softmax, O^T += V^T P^T.
template <int HD, int QSUB, int NW>
__device__ __forceinline__ void process_tile(const char* sk, const char* sv, const bf16x8 (&qf)[QSUB][HD / 16],
                                             f32x16 (&oacc)[QSUB][HD / 32], float (&m_run)[QSUB],
                                             float (&l_run)[QSUB], float c, int lane, int keys_valid) {
    using C = Cfg<HD, QSUB, NW>;
    const int r32 = lane & 31, kh = lane >> 5;
    const int prow = key_perm(r32);

    f32x16 s[QSUB][2];
#pragma unroll
    for (int qs = 0; qs < QSUB; ++qs)
#pragma unroll
        for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
            for (int v = 0; v < 16; ++v) s[qs][kvb][v] = 0.0f;

#pragma unroll
    for (int kvb = 0; kvb < 2; ++kvb) {
        const int row = kvb * 32 + prow;
        const char* rowp = sk + row * (HD * 2);
        const int sw = swz<C::KCH>(row);
#pragma unroll
        for (int ks = 0; ks < HD / 16; ++ks) {
            const bf16x8 kf = *reinterpret_cast<const bf16x8*>(rowp + (((2 * ks + kh) ^ sw) << 4));
#pragma unroll
            for (int qs = 0; qs < QSUB; ++qs)
                s[qs][kvb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qs][ks], s[qs][kvb], 0, 0, 0);
        }
    }

    bf16x8 pf[QSUB][4];
#pragma unroll
    for (int qs = 0; qs < QSUB; ++qs) {
        if (keys_valid < BN) {   // wave-uniform: only the last, ragged tile
#pragma unroll
            for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int key = 32 * kvb + 16 * (v >> 3) + 8 * kh + (v & 7);
                    if (key >= keys_valid) s[qs][kvb][v] = -INFINITY;
                }
        }
        float mx = s[qs][0][0];
#pragma unroll
        for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
            for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[qs][kvb][v]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run[qs], mx * c);
        const float alpha = __builtin_amdgcn_exp2f(m_run[qs] - m_new);
        const bool grew = m_new > m_run[qs];
        m_run[qs] = m_new;
        float psum = 0.0f;
#pragma unroll
        for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float pv = __builtin_amdgcn_exp2f(s[qs][kvb][v] * c - m_new);
                s[qs][kvb][v] = pv;
                psum += pv;
            }
        l_run[qs] = l_run[qs] * alpha + psum;
        if (__builtin_amdgcn_ballot_w64(grew) != 0) {    // rescale only when some row's max moved
#pragma unroll
            for (int t = 0; t < HD / 32; ++t)
#pragma unroll
                for (int v = 0; v < 16; ++v) oacc[qs][t][v] *= alpha;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            bf16x8 p8;
#pragma unroll
            for (int e = 0; e < 8; ++e) p8[e] = (__bf16)s[qs][j >> 1][8 * (j & 1) + e];
            pf[qs][j] = p8;
        }
    }

#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int t = 0; t < HD / 32; ++t) {
            const int row = 32 * t + r32;
            const bf16x8 vf =
                *reinterpret_cast<const bf16x8*>(sv + row * (BN * 2) + (((2 * j + kh) ^ swz<8>(row)) << 4));
#pragma unroll
            for (int qs = 0; qs < QSUB; ++qs)
                oacc[qs][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[qs][j], oacc[qs][t], 0, 0, 0);
        }
}

template <int HD, int QSUB, int NW>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(NW / 4, NW / 4))) void attn_fwd_kernel(
    const AttnParams p) {
    using C = Cfg<HD, QSUB, NW>;
    static_assert(QSUB * NW * 32 == BMQ, "workgroup must cover BMQ query rows");
    __shared__ __attribute__((aligned(1024))) char sk0[C::K_TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) char sv0[C::V_TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) char sk1[C::K_TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) char sv1[C::V_TILE_BYTES];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r32 = lane & 31, kh = lane >> 5;
    const int qtile = blockIdx.x, head = blockIdx.y;
    const int q0 = qtile * BMQ + wave * (32 * QSUB);

    // ---- Q fragments (B operand of S^T = K Q^T): lane holds query r32, channels 16ks + 8kh .. +7
    bf16x8 qf[QSUB][HD / 16];
#pragma unroll
    for (int qs = 0; qs < QSUB; ++qs) {
        int qrow = q0 + qs * 32 + r32;
        qrow = qrow < p.n_tokens ? qrow : p.n_tokens - 1;
        const bf16_t* qp = p.q + (int64_t)qrow * p.ldq + head * HD + 8 * kh;
#pragma unroll
        for (int ks = 0; ks < HD / 16; ++ks) qf[qs][ks] = *reinterpret_cast<const bf16x8*>(qp + 16 * ks);
    }

    f32x16 oacc[QSUB][HD / 32];
    float m_run[QSUB], l_run[QSUB];
#pragma unroll
    for (int qs = 0; qs < QSUB; ++qs) {
        m_run[qs] = -INFINITY;
        l_run[qs] = 0.0f;
#pragma unroll
        for (int t = 0; t < HD / 32; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) oacc[qs][t][v] = 0.0f;
    }

    // ---- per-lane byte offsets of this wave's share of the tile loads
    uint32_t ko[C::K_PER_WAVE], ko_last[C::K_PER_WAVE], vo[C::V_PER_WAVE];
    const int NT = (p.n_tokens + BN - 1) / BN;
    const int last_valid = p.n_tokens - (NT - 1) * BN;      // keys in the last tile (1..64)
    k_offsets<HD, QSUB, NW>(wave, lane, p.ldk, BN, ko);
    k_offsets<HD, QSUB, NW>(wave, lane, p.ldk, last_valid, ko_last);
#pragma unroll
    for (int i = 0; i < C::V_PER_WAVE; ++i) {
        const int row = (i * NW + wave) * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ swz<8>(row);
        vo[i] = (uint32_t)(row * p.n_pad + chunk * 8) * 2u;
    }
    const char* kbase = reinterpret_cast<const char*>(p.k + head * HD);
    const char* vbase = reinterpret_cast<const char*>(p.vt + (int64_t)head * HD * p.n_pad);
    const int64_t kstep = (int64_t)BN * p.ldk * 2;    // bytes per key tile
    const int64_t vstep = (int64_t)BN * 2;
    const float c = p.scale_log2e;

    // tile j lives in buffer j & 1
    if (NT == 1) issue_tile<HD, QSUB, NW>(kbase, vbase, ko_last, vo, sk0, sv0, wave);
    else issue_tile<HD, QSUB, NW>(kbase, vbase, ko, vo, sk0, sv0, wave);
    int j = 0;
    for (; j + 1 < NT; j += 2) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (j + 2 == NT) issue_tile<HD, QSUB, NW>(kbase + (j + 1) * kstep, vbase + (j + 1) * vstep, ko_last, vo, sk1, sv1, wave);
        else issue_tile<HD, QSUB, NW>(kbase + (j + 1) * kstep, vbase + (j + 1) * vstep, ko, vo, sk1, sv1, wave);
        __builtin_amdgcn_sched_barrier(0);
        process_tile<HD, QSUB, NW>(sk0, sv0, qf, oacc, m_run, l_run, c, lane, BN);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (j + 2 < NT) {
            if (j + 3 == NT) issue_tile<HD, QSUB, NW>(kbase + (j + 2) * kstep, vbase + (j + 2) * vstep, ko_last, vo, sk0, sv0, wave);
            else issue_tile<HD, QSUB, NW>(kbase + (j + 2) * kstep, vbase + (j + 2) * vstep, ko, vo, sk0, sv0, wave);
        }
        __builtin_amdgcn_sched_barrier(0);
        process_tile<HD, QSUB, NW>(sk1, sv1, qf, oacc, m_run, l_run, c, lane, (j + 2 == NT) ? last_valid : BN);
    }
    if (j < NT) {   // odd tile count: the last tile sits in buffer 0
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        process_tile<HD, QSUB, NW>(sk0, sv0, qf, oacc, m_run, l_run, c, lane, last_valid);
    }

    // ---- normalise and store: lane owns query r32; accumulator v of block t is channel 32t + 8(v/4) + 4kh + v%4
#pragma unroll
    for (int qs = 0; qs < QSUB; ++qs) {
        const float l_tot = l_run[qs] + __shfl_xor(l_run[qs], 32, 64);
        const float inv = 1.0f / l_tot;
        const int qrow = q0 + qs * 32 + r32;
        if (qrow < p.n_tokens) {
            bf16_t* op = p.o + (int64_t)qrow * p.ldo + head * HD + 4 * kh;
#pragma unroll
            for (int t = 0; t < HD / 32; ++t)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    uint2 w;
                    w.x = pack_bf16x2(oacc[qs][t][4 * g + 0] * inv, oacc[qs][t][4 * g + 1] * inv);
                    w.y = pack_bf16x2(oacc[qs][t][4 * g + 2] * inv, oacc[qs][t][4 * g + 3] * inv);
                    *reinterpret_cast<uint2*>(op + 32 * t + 8 * g) = w;
                }
        }
    }
}

// V[n_tokens, n_heads, HD] (row stride ldv) -> Vt[n_heads][HD][n_pad], zero beyond n_tokens
template <int HD>
__global__ __launch_bounds__(256) void transpose_v_kernel(const bf16_t* __restrict__ v, int64_t ldv,
                                                          bf16_t* __restrict__ vt, int n_tokens, int n_pad) {
    __shared__ bf16_t tile[64][HD + 2];
    const int t0 = blockIdx.x * 64, head = blockIdx.y;
    constexpr int CPR = HD / 8;      // 16-byte chunks per token row
    for (int idx = threadIdx.x; idx < 64 * CPR; idx += 256) {
        const int r = idx / CPR, ch = idx % CPR;
        uint4 u = make_uint4(0, 0, 0, 0);
        if (t0 + r < n_tokens) u = *reinterpret_cast<const uint4*>(v + (int64_t)(t0 + r) * ldv + head * HD + ch * 8);
        uint32_t* dst = reinterpret_cast<uint32_t*>(&tile[r][ch * 8]);
        dst[0] = u.x; dst[1] = u.y; dst[2] = u.z; dst[3] = u.w;
    }
    __syncthreads();
    // each thread writes 8 consecutive tokens of one channel
    for (int idx = threadIdx.x; idx < HD * 8; idx += 256) {
        const int ch = idx >> 3, tg = idx & 7;
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            w[e] = (uint32_t)tile[tg * 8 + 2 * e][ch] | ((uint32_t)tile[tg * 8 + 2 * e + 1][ch] << 16);
        *reinterpret_cast<uint4*>(vt + ((int64_t)head * HD + ch) * n_pad + t0 + tg * 8) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

inline int64_t pad_tokens(int64_t n) { return (n + BN - 1) / BN * BN; }

template <int HD, int QSUB, int NW>
void launch_attn(const AttnParams& p, hipStream_t st) {
    dim3 grid((p.n_tokens + BMQ - 1) / BMQ, p.n_heads);
    attn_fwd_kernel<HD, QSUB, NW><<<grid, NW * 64, 0, st>>>(p);
}

}  // namespace

extern "C" int64_t cdm_attn_workspace_bytes(int64_t n_tokens, int32_t n_heads, int32_t head_dim) {
    if (n_tokens < 0 || n_heads <= 0 || head_dim <= 0) return 0;
    return pad_tokens(n_tokens) * n_heads * head_dim * 2;
}

namespace {

int32_t check_attn_common(const char* who, int64_t n_tokens, int32_t n_heads, int32_t head_dim) {
    CDM_REQUIRE(n_tokens >= 0 && n_heads > 0, CDM_ERR_BAD_ARG, "%s: bad sizes", who);
    CDM_REQUIRE(head_dim == 64 || head_dim == 128, CDM_ERR_BAD_SHAPE, "%s: head_dim=%d must be 64 or 128", who, head_dim);
    CDM_REQUIRE(n_tokens < (1ll << 23) && n_heads <= 65535, CDM_ERR_BAD_SHAPE, "%s: sizes out of range", who);
    return CDM_OK;
}

}  // namespace

extern "C" int32_t cdm_transpose_v_bf16(const void* v, int64_t ldv, void* vt, int64_t vt_bytes, int64_t n_tokens,
                                        int32_t n_heads, int32_t head_dim, void* stream) {
    CDM_REQUIRE(v && vt, CDM_ERR_BAD_ARG, "transpose_v: null pointer");
    int32_t rc = check_attn_common("transpose_v", n_tokens, n_heads, head_dim);
    if (rc) return rc;
    CDM_REQUIRE(ldv >= (int64_t)n_heads * head_dim, CDM_ERR_BAD_ARG, "transpose_v: row stride smaller than n_heads*head_dim");
    CDM_REQUIRE(cdm_aligned16(v) && cdm_aligned16(vt) && ldv % 8 == 0, CDM_ERR_BAD_ALIGN,
                "transpose_v: pointers/strides must be 16-byte aligned");
    const int64_t need = cdm_attn_workspace_bytes(n_tokens, n_heads, head_dim);
    CDM_REQUIRE(vt_bytes >= need, CDM_ERR_BAD_ARG, "transpose_v: output of at least %lld bytes required", (long long)need);
    if (n_tokens == 0) return CDM_OK;
    if ((rc = cdm_require_device())) return rc;
    const int n_pad = (int)pad_tokens(n_tokens);
    dim3 tgrid(n_pad / 64, n_heads);
    hipStream_t st = (hipStream_t)stream;
    if (head_dim == 128)
        transpose_v_kernel<128><<<tgrid, 256, 0, st>>>((const bf16_t*)v, ldv, (bf16_t*)vt, (int)n_tokens, n_pad);
    else
        transpose_v_kernel<64><<<tgrid, 256, 0, st>>>((const bf16_t*)v, ldv, (bf16_t*)vt, (int)n_tokens, n_pad);
    return cdm_check_launch("transpose_v");
}

extern "C" int32_t cdm_attn_fwd_vt_bf16(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* vt,
                                        void* o, int64_t ldo, int64_t n_tokens, int32_t n_heads, int32_t head_dim,
                                        void* stream) {
    CDM_REQUIRE(q && k && vt && o, CDM_ERR_BAD_ARG, "attn_fwd: null pointer");
    int32_t rc = check_attn_common("attn_fwd", n_tokens, n_heads, head_dim);
    if (rc) return rc;
    const int64_t d = (int64_t)n_heads * head_dim;
    CDM_REQUIRE(ldq >= d && ldk >= d && ldo >= d, CDM_ERR_BAD_ARG, "attn_fwd: row stride smaller than n_heads*head_dim");
    CDM_REQUIRE(ldk * 64 * 2 < (1ll << 31), CDM_ERR_BAD_SHAPE, "attn_fwd: ldk out of range");
    CDM_REQUIRE(cdm_aligned16(q) && cdm_aligned16(k) && cdm_aligned16(vt) && cdm_aligned16(o) && ldq % 8 == 0 &&
                    ldk % 8 == 0 && ldo % 4 == 0,
                CDM_ERR_BAD_ALIGN, "attn_fwd: pointers/strides must be 16-byte aligned");
    if (n_tokens == 0) return CDM_OK;
    if ((rc = cdm_require_device())) return rc;
    AttnParams p;
    p.q = (const bf16_t*)q; p.ldq = ldq;
    p.k = (const bf16_t*)k; p.ldk = ldk;
    p.vt = (const bf16_t*)vt;
    p.o = (bf16_t*)o; p.ldo = ldo;
    p.n_tokens = (int)n_tokens; p.n_pad = (int)pad_tokens(n_tokens); p.n_heads = n_heads;
    p.scale_log2e = 1.4426950408889634f / sqrtf((float)head_dim);
    hipStream_t st = (hipStream_t)stream;
    const int variant = cdm_get_variant(0);
    // variant 0: 8 waves x 32 query rows (two waves per SIMD overlap softmax with MFMA);
    // variant 1: 4 waves x 64 query rows (half the LDS traffic per flop, one wave per SIMD)
    if (head_dim == 128) {
        if (variant == 1) launch_attn<128, 2, 4>(p, st);
        else launch_attn<128, 1, 8>(p, st);
    } else {
        if (variant == 1) launch_attn<64, 2, 4>(p, st);
        else launch_attn<64, 1, 8>(p, st);
    }
    return cdm_check_launch("attn_fwd");
}

extern "C" int32_t cdm_attn_fwd_bf16(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v,
                                     int64_t ldv, void* o, int64_t ldo, int64_t n_tokens, int32_t n_heads,
                                     int32_t head_dim, void* workspace, int64_t workspace_bytes, void* stream) {
    CDM_REQUIRE(q && k && v && o, CDM_ERR_BAD_ARG, "attn_fwd: null pointer");
    int32_t rc = check_attn_common("attn_fwd", n_tokens, n_heads, head_dim);
    if (rc) return rc;
    if (n_tokens == 0) return CDM_OK;
    const int64_t need = cdm_attn_workspace_bytes(n_tokens, n_heads, head_dim);
    CDM_REQUIRE(workspace && cdm_aligned16(workspace) && workspace_bytes >= need, CDM_ERR_BAD_ARG,
                "attn_fwd: workspace of at least %lld bytes required", (long long)need);
    // validate the second stage's arguments before the first stage is enqueued
    const int64_t d = (int64_t)n_heads * head_dim;
    CDM_REQUIRE(ldq >= d && ldk >= d && ldv >= d && ldo >= d, CDM_ERR_BAD_ARG, "attn_fwd: row stride smaller than n_heads*head_dim");
    CDM_REQUIRE(ldk * 64 * 2 < (1ll << 31), CDM_ERR_BAD_SHAPE, "attn_fwd: ldk out of range");
    CDM_REQUIRE(cdm_aligned16(q) && cdm_aligned16(k) && cdm_aligned16(v) && cdm_aligned16(o) && ldq % 8 == 0 &&
                    ldk % 8 == 0 && ldv % 8 == 0 && ldo % 4 == 0,
                CDM_ERR_BAD_ALIGN, "attn_fwd: pointers/strides must be 16-byte aligned");
    if ((rc = cdm_transpose_v_bf16(v, ldv, workspace, workspace_bytes, n_tokens, n_heads, head_dim, stream))) return rc;
    return cdm_attn_fwd_vt_bf16(q, ldq, k, ldk, workspace, o, ldo, n_tokens, n_heads, head_dim, stream);
}

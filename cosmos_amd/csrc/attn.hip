// Full self-attention over the joint sequence (flash-style, online softmax) on the gfx950 matrix cores; optional
// hybrid mask (a causal prefix that is blind to the rest), grouped K / V heads, prefix key images packed by an
// earlier call, per-head RMSNorm of Q and K.
//
// Work split: one workgroup owns 256 query rows of one head and streams all keys in tiles of 64.
// Scores are computed TRANSPOSED, S^T = K . Q^T, with v_mfma_f32_16x16x32_bf16 (the small shape moves a fifth fewer
// register bytes per flop than 32x32x16, and on random operands the chip is bound by its power limit): the A operand
// is a K tile row (plain 16-byte LDS read), the B operand is Q held in registers for the whole kernel.  In the
// accumulator layout every lane then owns ONE query column and 4 keys per 16-key block, so the row max / row sum of
// the online softmax are in-lane reductions plus two exchanges between the four quarter-waves.  The probabilities
// never move between lanes: packed to bf16, the lane's values of key blocks 2s and 2s + 1 are its 8 k-values of the B
// operand of O^T += V^T . P^T for the 32-key step s, whose A operand is a row of V^T; the V^T image lists the keys of
// a step in that order (lane quarter g, element e: keys 32 s + 4 g + e and 32 s + 16 + 4 g + e, e = 0..3).
// Rotate-half mRoPE (and the QK-RMSNorm ahead of it) is applied in registers: to K while it is re-tiled for the
// kernel, to Q when the kernel loads its Q fragments (both members of a rotary pair sit in the same lane).
#include <mutex>

#include "cdm_common.h"

namespace {

constexpr int BN = 64;       // keys per tile
constexpr int BMQ = 256;     // query rows per workgroup
constexpr int KB = BN / 16;  // 16-key blocks per tile
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// ---------------------------------------------------------------------------------------------
// Software-pipelined kernel over PRE-TILED K and V.
//  * K and V are first re-laid out in the workspace as the exact LDS image of each 64-key tile,
//    chunk-major:  Kp[head][tile][c = dh/8][key r = 0..63][8 ch]   and
//                  Vp[head][tile][c = 0..7][channel row = 0..HD-1][8 keys]  (V transposed; chunk c = 4 s + g holds
//                  keys 32 s + 4 g + {0..3} and 32 s + 16 + 4 g + {0..3}).
//    A tile is then one contiguous 16 KB (HD=128) stream for the direct-to-LDS loads, every fragment
//    read is  lane_base + compile-time offset  (no swizzle arithmetic, two address registers in
//    total) and 16 consecutive lanes always read 16 distinct 16-byte slots (no bank conflicts).
//    Keys beyond n_tokens are zero in the workspace and masked to -inf in the last tile.
//  * the scores of tile j+1 (S^T = K Q^T, 32 MFMAs) are issued BEFORE the softmax of tile j, so one
//    wave always has matrix work in flight under its own exp/convert VALU work;
//  * Q is pre-multiplied by log2(e)/sqrt(dh) and the score accumulators start at -m_ref instead of 0,
//    so a score leaves the MFMA already shifted and p = exp2(S) needs no per-score FMA;
//  * m_ref is a running reference that only moves when a row's tile maximum exceeds it by more than
//    2^kGrowLog2 (then O and l are rescaled: exact, merely a different reference);
//  * the row sum adds the fp32 exponentials (v_add_f32); the probabilities are rounded to bf16 once, for the second product.
// ---------------------------------------------------------------------------------------------
constexpr float kGrowLog2 = 4.0f;

// K fragment of k-step ks (32 channels), key block kb: lane reads key row 16 kb + lane % 16, chunk 4 ks + lane / 16
template <int HD>
__device__ __forceinline__ bf16x8 k_frag(const char* sk, int ks, int kb, int lane) {
    return *reinterpret_cast<const bf16x8*>(sk + (lane >> 4) * 1024 + (lane & 15) * 16 + ks * 4096 + kb * 256);
}
// V^T fragment of key step s (32 keys), channel block hb: lane reads channel row 16 hb + lane % 16, chunk 4 s + lane / 16
template <int HD>
__device__ __forceinline__ bf16x8 v_frag(const char* sv, int s, int hb, int lane) {
    return *reinterpret_cast<const bf16x8*>(sv + (lane >> 4) * (HD * 16) + (lane & 15) * 16 + s * (HD * 64) + hb * 256);
}

// Whole score tile with plain just-in-time fragment reads (prologue only).
template <int HD, int QB>
__device__ __forceinline__ void scores_tile(const char* sk, const bf16x8 (&qf)[QB][HD / 32], f32x4 (&s)[KB][QB], int lane) {
#pragma unroll
    for (int ks = 0; ks < HD / 32; ++ks)
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            const bf16x8 kf = k_frag<HD>(sk, ks, kb, lane);
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) s[kb][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[qb][ks], s[kb][qb], 0, 0, 0);
        }
}

constexpr int KWIN = 2;     // k-steps of K fragments kept in flight (x4 key blocks)
constexpr int VWIN = 8;     // V^T fragments kept in flight

template <int HD>
__device__ __forceinline__ void preload_k(const char* sk, bf16x8 (&kw)[KWIN][KB], int lane) {
#pragma unroll
    for (int ks = 0; ks < KWIN; ++ks)
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) kw[ks][kb] = k_frag<HD>(sk, ks, kb, lane);
}

// Scores of keys >= keys_valid[qb] (ragged last tile, causal rows) become -inf.  Register e of key block kb holds key
// 16 kb + 4 (lane / 16) + e: the compile-time part is compared against ONE per-lane threshold so that no per-register
// key index is ever materialised.
template <int QB>
__device__ __forceinline__ void mask_scores(f32x4 (&s)[KB][QB], const int (&keys_valid)[QB], int lane) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const int thr = keys_valid[qb] - 4 * (lane >> 4);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int e = 0; e < 4; ++e) s[kb][qb][e] = (16 * kb + e >= thr) ? -INFINITY : s[kb][qb][e];
    }
}

template <int QB>
__device__ __forceinline__ float tile_row_max(const f32x4 (&s)[KB][QB], int qb) {
    float mx = __builtin_fmaxf(s[0][qb][0], s[0][qb][1]);
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int e = (kb == 0 ? 2 : 0); e < 4; e += 2) mx = __builtin_fmaxf(__builtin_fmaxf(mx, s[kb][qb][e]), s[kb][qb][e + 1]);   // v_max3_f32
    mx = __builtin_fmaxf(mx, __shfl_xor(mx, 16, 64));
    return __builtin_fmaxf(mx, __shfl_xor(mx, 32, 64));
}

// Index of the first tile after `after` whose bit is set in the wave's table (bit t of lane l = tile 32 l + t), or a
// value no tile index reaches.  Wave-uniform.
__device__ __forceinline__ int next_hot_tile(uint32_t hot, int after, int lane) {
    const int wl = after >> 5, bit = after & 31;
    uint32_t w = lane < wl ? 0u : hot;
    if (lane == wl) w = bit == 31 ? 0u : (w & (~0u << (bit + 1)));
    const uint64_t lanes = __builtin_amdgcn_ballot_w64(w != 0u);
    if (lanes == 0) return 0x7fffffff;
    const int l = __builtin_ctzll(lanes);
    return 32 * l + __builtin_ctz((uint32_t)__builtin_amdgcn_readlane((int)w, l));
}

// One pipeline step.  Everything the first MFMAs need is already in registers when the workgroup barrier at
// the top of the step releases the wave, and all softmax arithmetic is placed under MFMAs:
//   block A  : S(j+1) = K(j+1) Q^T - m_ref, 32 MFMAs seeded with -m_ref (rolling K fragment window, first
//              KWIN k-steps preloaded in the previous step)
//              ||  p = exp2(s_cur), bf16 pack, row sum of tile j ; first V^T fragments of tile j (a wave that
//              takes the step's barrier behind block A reads them before that barrier: V(j) is complete one
//              barrier early)
//   block B  : O^T += V^T P^T, 32 MFMAs (rolling V^T window)
//              ||  row maximum of S(j+1) ; first K fragments of tile j+2 (that tile landed before this barrier)
//   tail     : if some row maximum exceeds the reference by more than 2^kGrowLog2 (rare), move the reference
//              and rescale O and l.  Scores stay raw (log2 units), so nothing else depends on the reference.
// The kernel bounds the scores of its rows against every key tile (|q| max|k| over the tile).  Where no score of the
//   wave's rows against tile j+1 can exceed the reference by more than 2^kSafeLog2 (wave-uniform, decided per tile
//   at set-up), the row maximum of that tile and the reference update are skipped; where the bound fails - a
//   tile with an outlier key, un-normalised huge logits - they run in the tail, after block B (one loop body for both
//   cases: two copies of the loop do not fit the register budget).
template <int HD, int QB, bool LATE, class Mid>
__device__ __forceinline__ void pipe_step(Mid&& mid, float late_r, const char* sk_next, const char* sv_cur, const char* sk_next2,
                                          const bf16x8 (&qf)[QB][HD / 32], bf16x8 (&kw)[KWIN][KB],
                                          f32x4 (&s_cur)[KB][QB], f32x4 (&s_next)[KB][QB],
                                          f32x4 (&oacc)[HD / 16][QB], f32x4 (&negm)[QB], float (&l_run)[QB], int lane,
                                          bool next_masked, const int (&next_keys_valid)[QB], int next_tile,
                                          int& next_hot, bool need_always, uint32_t hot) {
    constexpr int KS = HD / 32, HB = HD / 16, NV = 2 * HB;
    // Both blocks are written as a sequence of slots, one MFMA each, fenced so that the compiler keeps them: an odd
    // slot carries one fragment read, an even slot (head_dim 64: every slot) one piece of the softmax arithmetic.
    // ---- block A.  (In the very last step there is no next tile: the MFMAs then chew on a stale K slot, a second
    // copy of the last tile, and their result is never used - cheaper than a second copy of the step.  When the last
    // tile is ragged that step masks all of its scores like the one before it masked the padding: the zero keys of the
    // padding would otherwise show up as scores of -m_ref, and with every real logit far below zero the tail would
    // move the reference up to them and scale O and l towards zero.)
    constexpr int NA = KS * KB * QB;              // MFMAs of block A
    constexpr int NREFILL = (KS - KWIN) * KB;     // K fragments read inside block A
    constexpr int NSM = QB * 8;                   // softmax pieces: 2 exp, 2 add, 1 pack each
    constexpr int SMI = NA / NSM;                 // one softmax piece every SMI slots (2 at head_dim 128, 1 at 64)
    static_assert(SMI >= 1 && NREFILL + (VWIN < NV ? VWIN : NV) <= NA / 2 + NREFILL, "block A has too few slots");
    u32x4 pw[QB][2];       // the probabilities, packed: B operands of block B
    bf16x8 vw[VWIN];
    float psum0[QB], psum1[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) psum0[qb] = psum1[qb] = 0.0f;
    // Block A is the longer of the two (its exponentials alone take as many issue cycles as its MFMAs), so the wave
    // runs it with raised priority: it takes every issue slot it can use and the other wave of the SIMD, in its
    // block B, fills the rest with MFMAs (-2.9 % kernel time against the priority raised in block B, -2.6 % against
    // equal priorities).
    __builtin_amdgcn_s_setprio(1);
    int n_v = 0;       // V^T fragments read so far (compile-time after unrolling)
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        const int ks = i / (KB * QB), kb = (i / QB) % KB, qb = i % QB;
        s_next[kb][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kw[ks % KWIN][kb], qf[qb][ks],
                                                                 ks == 0 ? negm[qb] : s_next[kb][qb], 0, 0, 0);
        // the row sum adds the fp32 exponentials with plain v_add_f32 (two chains): next to MFMAs a v_dot2c_f32_bf16 on
        // the packed pairs costs the matrix pipe several times what two adds cost it
        if (i % SMI == 0 && i / SMI < NSM) {
            const int m = i / SMI, q = m / 8, st = (m / 4) % 2, h = (m / 2) % 2, e = 2 * (m % 2);
            // the empty asm statements tie the piece to its slot: left alone the compiler gathers all exponentials and
            // conversions of the tile in one place (behind the MFMAs of this block), where nothing overlaps them
            if (e == 0) asm volatile("" : "+v"(s_cur[2 * st + h][q]));
            // LATE: Q went in scaled by a power of two only (exact), the rest of log2(e)/sqrt(HD) multiplies the fp32 score
            const float e0 = __builtin_amdgcn_exp2f(LATE ? s_cur[2 * st + h][q][e] * late_r : s_cur[2 * st + h][q][e]);
            const float e1 = __builtin_amdgcn_exp2f(LATE ? s_cur[2 * st + h][q][e + 1] * late_r : s_cur[2 * st + h][q][e + 1]);
            psum0[q] += e0;
            psum1[q] += e1;
            uint32_t w = pack_bf16x2(e0, e1);
            asm volatile("" : "+v"(w), "+v"(psum0[q]), "+v"(psum1[q]));
            pw[q][st][2 * h + e / 2] = w;
        }
        // a K fragment is replaced right behind its last MFMA; the first V^T fragments follow
        if (qb == QB - 1 && ks + KWIN < KS) {
            kw[ks % KWIN][kb] = k_frag<HD>(sk_next, ks + KWIN, kb, lane);
        } else if (i % 2 == 1 && n_v < VWIN && n_v < NV) {
            vw[n_v] = v_frag<HD>(sv_cur, n_v / HB, n_v % HB, lane);
            ++n_v;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (; n_v < VWIN && n_v < NV; ++n_v) vw[n_v] = v_frag<HD>(sv_cur, n_v / HB, n_v % HB, lane);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) l_run[qb] += psum0[qb] + psum1[qb];
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(0);
    mid();                 // the step's synchronisation point for the waves that take it between the two blocks
    __builtin_amdgcn_sched_barrier(0);
    if (next_masked)       // wave-uniform: before a ragged last tile, and in every step of a causal query block
        mask_scores<QB>(s_next, next_keys_valid, lane);

    // ---- block B: pure matrix work, while the other wave of the SIMD is in its VALU-heavy block A at this time.
    constexpr int NB = NV * QB;                   // MFMAs of block B
    static_assert((NV > VWIN ? NV - VWIN : 0) + KWIN * KB <= NB, "block B has too few slots");
    int n_kpre = 0;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int f = i / QB, st = f / HB, hb = f % HB, qb = i % QB;
        oacc[hb][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vw[f % VWIN], __builtin_bit_cast(bf16x8, pw[qb][st]), oacc[hb][qb], 0, 0, 0);
        if (qb == QB - 1 && f + VWIN < NV) {
            vw[f % VWIN] = v_frag<HD>(sv_cur, (f + VWIN) / HB, (f + VWIN) % HB, lane);
        } else if (i % 2 == 1 && n_kpre < KWIN * KB && (f + VWIN >= NV || qb != QB - 1)) {
            kw[n_kpre / KB][n_kpre % KB] = k_frag<HD>(sk_next2, n_kpre / KB, n_kpre % KB, lane);
            ++n_kpre;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (; n_kpre < KWIN * KB; ++n_kpre) kw[n_kpre / KB][n_kpre % KB] = k_frag<HD>(sk_next2, n_kpre / KB, n_kpre % KB, lane);
    __builtin_amdgcn_sched_barrier(0);
    // tile j + 1 needs row maxima only if it is the wave's next marked tile (one scalar compare on the common path);
    // the tile after it is looked up behind the maxima (need_always: every tile is the next one)
    if (next_tile != next_hot) return;
    next_hot = need_always ? next_tile + 1 : next_hot_tile(hot, next_tile, lane);
    float mx[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) mx[qb] = tile_row_max<QB>(s_next, qb);

    // ---- tail.  mx is relative to the reference (the scores are); moving the reference by d means: O and l
    // shrink by 2^-d, the scores already computed for tile j+1 drop by d, and so does the accumulator seed.
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        if (__builtin_amdgcn_ballot_w64(mx[qb] > kGrowLog2) != 0) {
            const float d = mx[qb] > kGrowLog2 ? mx[qb] : 0.0f;
            const float fac = __builtin_amdgcn_exp2f(LATE ? -d * late_r : -d);      // the probabilities are exp2(late_r s)
            l_run[qb] *= fac;
#pragma unroll
            for (int hb = 0; hb < HB; ++hb)
#pragma unroll
                for (int e = 0; e < 4; ++e) oacc[hb][qb][e] *= fac;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) s_next[kb][qb][e] -= d;
                negm[qb][e] -= d;
            }
        }
    }
}

// Per-head RMSNorm of Q / K ahead of the rotation: y = x * rsqrt(mean(x^2) + eps) * w[segment], in fp32.
// Segments are contiguous token ranges [seg_end[i-1], seg_end[i]) with their own weight row (MoT branches).
struct QkNormDev {
    const float* w;        // [n_seg, HD] or null = no normalisation
    int seg_end[8];
    int n_seg;
    float eps;
    __device__ __forceinline__ const float* row(int token, int hd) const {
        int sidx = 0;
#pragma unroll
        for (int i = 0; i < 7; ++i) sidx += (i < n_seg - 1 && token >= seg_end[i]) ? 1 : 0;
        return w + sidx * hd;
    }
};

struct PackedParams {
    const bf16_t* q; int64_t ldq;
    const char* kp;              // [n_kv_heads][n_tiles][tile bytes]
    const char* vp;
    const float* kmax;           // [n_kv_heads][n_tiles]: largest key norm of each tile (after QK-norm / rotation)
    const char* kp_prefix;       // optional tile images of keys that precede those of kp / vp (whole tiles)
    const char* vp_prefix;
    const float* kmax_prefix;
    int n_prefix_tiles;
    int prefix_last_valid;       // keys of the last prefix tile that exist (1..64; the rest of that tile is zero padding)
    int causal_prefix;           // query rows < causal_prefix see keys <= their own index only; the others see all keys
    bf16_t* o; int64_t ldo;
    float* row_amax;             // optional [n_tokens, n_heads]: largest |o| of each output row within each head (as stored)
    const float* cos; const float* sin;   // optional rotary tables [n_tokens, HD/2] applied to Q at load
    QkNormDev qn;                          // optional per-head RMSNorm of Q, applied before the rotation
    int n_tokens, n_heads, n_qblocks;
    int kv_group;                // query heads per K / V head (1 = multi-head attention)
    int always_max;              // cross-check: take the row maxima of every tile whatever the norm bound says
    float scale_log2e;           // factor on Q ahead of its rounding to bf16: log2(e)/sqrt(HD), or only its power of two
    float late_r;                // ... with the rest of it (in [1, 2)) applied to the fp32 scores (LATE kernels)
    // Split of the last, partial round of workgroups (see SplitPlan): the last `split_tail` workgroups of every XCD
    // are replaced by `split` units each, which cover consecutive ranges of the key tiles and leave a normalised partial
    // output and the row's log-sum in scratch memory for merge_split_kernel.  split = 1: no split.
    int split, split_tail;
    bf16_t* part_o;              // [8 * split_tail * split][256][HD]
    float* part_lse;             // [8 * split_tail * split][256]   log2 of the unit's sum of exponentials, reference added
};

// QS = query sub-tiles (of 32 rows = two 16-row blocks) per wave: QS = 1 -> 8 waves, two per SIMD, 256 registers each;
// QS = 2 -> 4 waves, one per SIMD with the 512-register budget; every K / V^T fragment read from LDS then feeds
// four MFMAs instead of two.
constexpr float kSafeLog2 = 60.0f;      // largest excess over the reference that needs no reference update

// LATE: Q arrives as exact bf16 values that nothing in here touches (no rotation, no norm).  Folding log2(e)/sqrt(HD) into
// Q would then round every element once more than the reference does (it scales the fp32 scores): percent-level in the
// probabilities where logits of 50 - 150 compete.  Such calls scale Q by the power-of-two part of the factor (exact)
// and the fp32 scores by the rest, one multiplication per score; calls that rotate or normalise Q round it once anyway
// and fold the whole factor into that rounding.
constexpr int kMaxKm = 2048;            // key tiles that get a decision of their own (131,072 keys); longer sequences: one per head
constexpr int kMaxSplit = 8;            // most key ranges a query block of the last round is split into

template <int HD, int QS, bool LATE>
__global__ __launch_bounds__(512 / QS) __attribute__((amdgpu_waves_per_eu(2 / QS, 2 / QS))) void attn_fwd_pipe_kernel(
    const PackedParams p) {
    constexpr int NW = 8 / QS;
    constexpr int QB = 2 * QS;                         // 16-row query blocks per wave
    constexpr int KS = HD / 32, HB = HD / 16;
    constexpr int TILE_BYTES = BN * HD * 2;            // same for K and V tiles
    constexpr int PER_WAVE = TILE_BYTES / 1024 / NW;   // direct-to-LDS instructions per wave per tile
    // K(t) lives in slot t % 3 and V(t) in slot t % 4.  V is loaded one step further ahead than its first use by
    // the in-phase waves needs: the out-of-phase waves read the first fragments of V(j) BEFORE barrier j, so V(j)
    // has to be complete at barrier j - 1
    constexpr int RING = 3, RING_V = 4;
    __shared__ __attribute__((aligned(1024))) char sk[RING * TILE_BYTES];
    __shared__ __attribute__((aligned(1024))) char sv[RING_V * TILE_BYTES];
    __shared__ float s_km[kMaxKm];       // largest key norm of every tile of this K / V head, prefix tiles first (set-up only)

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r16 = lane & 15, g4 = lane >> 4;
    // XCD-aware placement: workgroup ids are dealt round-robin over the 8 XCDs.  All query blocks of a head go to
    // ONE XCD, so a head's K / V tile images are fetched into one L2 instead of eight, and an XCD owns a contiguous
    // range of heads, so the query heads that share a K / V head (grouped-query attention) share an L2 as well.
    int head, qblk;
    int unit = -1, part = 0;      // split unit: index into the scratch arrays, and which range of the key tiles
    {
        const int nqb = p.n_qblocks, nh = p.n_heads;
        const int xcd = blockIdx.x & 7;
        int k = blockIdx.x >> 3;                                  // k-th workgroup of its XCD
        const int hpx = (nh + 7) >> 3;                            // heads per XCD (the last XCDs may own fewer)
        if (p.split > 1) {
            // the last split_tail query blocks of the XCD come `split` times, ordered by key range first: units that run
            // side by side then stream the same tiles of the same head
            const int whole = hpx * nqb - p.split_tail;
            if (k >= whole) {
                const int u = k - whole;
                part = u / p.split_tail;
                k = whole + (u - part * p.split_tail);
                unit = xcd * p.split_tail * p.split + u;
            }
        }
        const int hi = k / nqb;
        head = xcd * hpx + hi;
        qblk = k - hi * nqb;
        if (hi >= hpx || head >= nh) return;
    }
    const int kv_head = head / p.kv_group;
    const int q0 = qblk * BMQ + wave * (32 * QS);

    // ---- Q fragments: rotate-half mRoPE (if tables are given) and the factor log2(e)/sqrt(HD), both in fp32 and
    // with ONE rounding to bf16.  The lane holds channels 32ks + 8g .. +7 (g = lane / 16) of its query row for every
    // ks, so the partner of a channel in k-step ks (< KS/2) is the same register element of k-step ks + KS/2.
    // An upper bound of every score of a row against a key tile: |q| max_{k in tile} |k| (Cauchy-Schwarz on the very
    // bf16 values the matrix cores multiply).  The per-tile key norms of this K / V head pass through LDS once: each
    // wave turns them into one bit per tile ("this tile needs row maxima for my rows"), 32 tiles per lane of one
    // register, and keeps the index of the next such tile in a scalar register: a step compares its tile index with it
    // (one scalar instruction) and looks the following one up only after a hit.
    // A sequence of more than kMaxKm tiles falls back to one bound per head (kmax_all).
    // A split unit works in a frame of its own: tile 0 is the first tile of its range [t0, t0 + NT), the prefix tiles
    // are the first NP of that frame (NP <= 0: none left), per-row key limits count from the frame's first key.
    const int NM = (p.n_tokens + BN - 1) / BN;
    const int NT_all = p.n_prefix_tiles + NM;
    const int t0 = unit < 0 ? 0 : (int)((int64_t)NT_all * part / p.split);
    const int t1 = unit < 0 ? NT_all : (int)((int64_t)NT_all * (part + 1) / p.split);
    const int NP = p.n_prefix_tiles - t0;
    const int NT = t1 - t0;
    const bool per_tile = NT <= kMaxKm;
    float kmax_all = 0.0f;
    {
        const float* km = p.kmax + (int64_t)kv_head * NM - p.n_prefix_tiles + t0;      // indexed by the frame's tile number
        const float* kmp = p.kmax_prefix + (int64_t)kv_head * p.n_prefix_tiles + t0;
        if (per_tile) {
            for (int i = threadIdx.x; i < kMaxKm; i += 512 / QS) s_km[i] = i >= NT ? 0.0f : (i < NP ? kmp[i] : km[i]);
        } else {
            for (int i = lane; i < NT; i += 64) kmax_all = fmaxf(kmax_all, i < NP ? kmp[i] : km[i]);
            kmax_all = wave_max(kmax_all);
        }
    }
    float qnorm[QB];
    bf16x8 qf[QB][KS];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        int qrow = q0 + qb * 16 + r16;
        qrow = qrow < p.n_tokens ? qrow : p.n_tokens - 1;
        const bf16_t* qp = p.q + (int64_t)qrow * p.ldq + head * HD + 8 * g4;
        uint4 raw[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) raw[ks] = *reinterpret_cast<const uint4*>(qp + 32 * ks);
        // per-head RMSNorm: the lane holds 8 channels per k-step, the other three quarter-waves the rest of the row
        float rnorm = 1.0f;
        const float* nw = nullptr;
        if (p.qn.w != nullptr) {
            float ss = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const uint32_t w[4] = {raw[ks].x, raw[ks].y, raw[ks].z, raw[ks].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) { const float a = bf16lo(w[j]), b = bf16hi(w[j]); ss += a * a + b * b; }
            }
            ss += __shfl_xor(ss, 16, 64);
            ss += __shfl_xor(ss, 32, 64);
            rnorm = rsqrtf(ss * (1.0f / HD) + p.qn.eps);
            nw = p.qn.row(qrow, HD) + 8 * g4;
        }
#pragma unroll
        for (int ks = 0; ks < KS / 2; ++ks) {
            const uint32_t w1[4] = {raw[ks].x, raw[ks].y, raw[ks].z, raw[ks].w};
            const uint32_t w2[4] = {raw[ks + KS / 2].x, raw[ks + KS / 2].y, raw[ks + KS / 2].z, raw[ks + KS / 2].w};
            float n1[8], n2[8];      // norm factors of the channels of k-step ks and of its rotary partners
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                n1[e] = nw ? rnorm * nw[32 * ks + e] : 1.0f;
                n2[e] = nw ? rnorm * nw[32 * (ks + KS / 2) + e] : 1.0f;
            }
            float c[8], sn[8];
            if (p.cos != nullptr) {
                const float4* cp = reinterpret_cast<const float4*>(p.cos + (int64_t)qrow * (HD / 2) + 32 * ks + 8 * g4);
                const float4* sp = reinterpret_cast<const float4*>(p.sin + (int64_t)qrow * (HD / 2) + 32 * ks + 8 * g4);
                const float4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
                c[0] = c0.x; c[1] = c0.y; c[2] = c0.z; c[3] = c0.w; c[4] = c1.x; c[5] = c1.y; c[6] = c1.z; c[7] = c1.w;
                sn[0] = s0.x; sn[1] = s0.y; sn[2] = s0.z; sn[3] = s0.w; sn[4] = s1.x; sn[5] = s1.y; sn[6] = s1.z; sn[7] = s1.w;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) { c[e] = 1.0f; sn[e] = 0.0f; }
            }
            uint32_t o1[4], o2[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float a0 = bf16lo(w1[j]) * n1[2 * j], a1 = bf16hi(w1[j]) * n1[2 * j + 1];
                const float b0 = bf16lo(w2[j]) * n2[2 * j], b1 = bf16hi(w2[j]) * n2[2 * j + 1];
                o1[j] = pack_bf16x2((a0 * c[2 * j] - b0 * sn[2 * j]) * p.scale_log2e,
                                    (a1 * c[2 * j + 1] - b1 * sn[2 * j + 1]) * p.scale_log2e);
                o2[j] = pack_bf16x2((b0 * c[2 * j] + a0 * sn[2 * j]) * p.scale_log2e,
                                    (b1 * c[2 * j + 1] + a1 * sn[2 * j + 1]) * p.scale_log2e);
            }
            qf[qb][ks] = __builtin_bit_cast(bf16x8, make_uint4(o1[0], o1[1], o1[2], o1[3]));
            qf[qb][ks + KS / 2] = __builtin_bit_cast(bf16x8, make_uint4(o2[0], o2[1], o2[2], o2[3]));
        }
        {      // norm of the scaled, rotated, rounded query row (a quarter of it in each quarter-wave)
            float ss = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const uint4 u = __builtin_bit_cast(uint4, qf[qb][ks]);
                const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) { const float a = bf16lo(w[j]), b = bf16hi(w[j]); ss += a * a + b * b; }
            }
            ss += __shfl_xor(ss, 16, 64);
            ss += __shfl_xor(ss, 32, 64);
            qnorm[qb] = sqrtf(ss);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // Q is in registers: from here on vmcnt counts tile loads only

    f32x4 oacc[HB][QB];
    // negm = minus the softmax reference of the lane's query row (log2 units), replicated over a 4-register
    // block so that it can seed the score accumulators: the MFMAs then deliver s - m_ref and no subtraction is
    // left in the exp path
    f32x4 negm[QB];
    float l_run[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        l_run[qb] = 0.0f;
#pragma unroll
        for (int hb = 0; hb < HB; ++hb) oacc[hb][qb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }

    // key tiles: NP whole tiles of the prefix images, then the NM tiles of the main images
    // keys of the frame: a range that ends ahead of the sequence's last tile ends on a full tile - unless that tile is the
    // prefix's partly filled last one, which then is this frame's ragged last tile (prefix_last_valid = BN otherwise)
    const int n_keys = t1 < NT_all ? NT * BN - (t1 == p.n_prefix_tiles ? BN - p.prefix_last_valid : 0)
                                   : p.n_prefix_tiles * BN + p.n_tokens - t0 * BN;
    const int last_valid = n_keys - (NT - 1) * BN;
    // per-row key limit and the tiles this workgroup needs: a query block inside the causal prefix stops at its
    // own last row, and every tile it visits is masked per row
    const int b0 = qblk * BMQ;
    const bool causal_wg = b0 < p.causal_prefix;
    int klim[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const int qrow = q0 + qb * 16 + r16;
        klim[qb] = qrow < p.causal_prefix ? qrow + 1 : n_keys;
    }
    const int kmax = (causal_wg && b0 + BMQ <= p.causal_prefix) ? (b0 + BMQ < n_keys ? b0 + BMQ : n_keys) : n_keys;
    const int NTW = (kmax + BN - 1) / BN;
    const uint32_t lane_off = (uint32_t)(wave * 1024 + lane * 16);
    // tile t of the key sequence [prefix tiles | main tiles] lives at pre + t * TILE_BYTES (t < NP) or at
    // base + t * TILE_BYTES with base shifted back by the prefix length: one 32-bit offset serves both
    const char* kbase = p.kp + ((int64_t)kv_head * NM - NP) * TILE_BYTES;
    const char* vbase = p.vp + ((int64_t)kv_head * NM - NP) * TILE_BYTES;
    const char* kpre = p.kp_prefix + ((int64_t)kv_head * p.n_prefix_tiles + t0) * TILE_BYTES;
    const char* vpre = p.vp_prefix + ((int64_t)kv_head * p.n_prefix_tiles + t0) * TILE_BYTES;
    const uint32_t sk_addr = lds_addr_of(sk) + wave * 1024, sv_addr = lds_addr_of(sv) + wave * 1024;

    // tile `t` (clamped to the last tile, so that every step issues the same number of loads and the
    // vmcnt arithmetic below stays valid at the end of the sequence) -> ring slot `slot`
    auto issue = [&](const char* base, const char* pre, uint32_t dst_addr, int t, int slot) {
        const int tc = t < NT ? t : NT - 1;
        const char* src = (tc < NP ? pre : base) + (uint32_t)tc * (uint32_t)TILE_BYTES;      // images stay below 4 GB per head
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i)
            lds_dma16(src + i * (NW * 1024), lane_off, dst_addr + slot * TILE_BYTES + i * (NW * 1024));
    };

    // ---- prologue: K(0) | K(1), V(0) | K(2), V(1) | V(2); scores of tile 0 with an exact first reference
    issue(kbase, kpre, sk_addr, 0, 0);
    issue(kbase, kpre, sk_addr, 1, 1);
    issue(vbase, vpre, sv_addr, 0, 0);
    issue(kbase, kpre, sk_addr, 2, 2);
    issue(vbase, vpre, sv_addr, 1, 1);
    issue(vbase, vpre, sv_addr, 2, 2);
    // K(0), K(1), V(0) have landed, and every wave's share of the key-norm table is in LDS
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(3 * PER_WAVE) : "memory");
    f32x4 s_a[KB][QB], s_b[KB][QB];      // score tiles ping-pong between the two halves of the unrolled loop
    const bool ragged = last_valid < BN;
    bool need_always = p.always_max != 0;
    float t_lane = INFINITY;      // largest tile key norm this lane's rows tolerate without row maxima
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) s_a[kb][qb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    scores_tile<HD, QB>(sk, qf, s_a, lane);
    // the padding of a prefix that does not fill its last tile sits in the MIDDLE of the key sequence: that one tile is
    // masked like a ragged last tile (pre_rag_tile = its index, or -1)
    const int pre_rag_tile = (NP > 0 && p.prefix_last_valid < BN) ? NP - 1 : -1;
    int pre_valid[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) pre_valid[qb] = p.prefix_last_valid;
    if (causal_wg || (NT == 1 && ragged)) mask_scores<QB>(s_a, klim, lane);
    if (pre_rag_tile == 0) mask_scores<QB>(s_a, pre_valid, lane);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const float m0 = tile_row_max<QB>(s_a, qb);      // exact first reference: every row has at least one finite score
        // a tile whose largest key norm is at most thr cannot raise any score of this row more than 2^kSafeLog2 above its
        // reference (1 % slack for the fp32 accumulation of the dot products and of the norms); a reference that is not
        // a number asks for the maxima everywhere
        const float thr = (kSafeLog2 + m0) / (qnorm[qb] * 1.01f);
        need_always = need_always || __builtin_amdgcn_ballot_w64(thr != thr) != 0;
        t_lane = fminf(t_lane, thr);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) s_a[kb][qb][e] -= m0;
            negm[qb][e] = -m0;
        }
    }
    float t_wave = t_lane;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) t_wave = fminf(t_wave, __shfl_xor(t_wave, off, 64));
    if (!per_tile) need_always = need_always || !(kmax_all <= t_wave);
    uint32_t hot = 0u;      // bit t in lane l: tile 32 l + t needs row maxima for this wave's rows
    if (per_tile && !need_always) {
#pragma unroll
        for (int c4 = 0; c4 < 8; ++c4) {
            const float4 v = *reinterpret_cast<const float4*>(&s_km[32 * lane + 4 * c4]);
            hot |= (uint32_t)(!(v.x <= t_wave)) << (4 * c4) | (uint32_t)(!(v.y <= t_wave)) << (4 * c4 + 1) |
                   (uint32_t)(!(v.z <= t_wave)) << (4 * c4 + 2) | (uint32_t)(!(v.w <= t_wave)) << (4 * c4 + 3);
        }
    }
    // tile 0 had its exact maxima above; need_always = every tile is "the next one"
    int next_hot = need_always ? 1 : next_hot_tile(hot, 0, lane);
    bf16x8 kw[KWIN][KB];
    preload_k<HD>(sk + TILE_BYTES, kw, lane);      // K(1) for step 0

    // step j: S(j+1) from K slot (j+1)%3, P(j) V(j) from V slot j%4, K(j+2) fragments preloaded from slot (j+2)%3.
    // At the barrier everything but the most recently issued group, V(j+2), must have landed
    // (s_waitcnt vmcnt(1 tile)): K(j+2) is read at the end of this very step and the first fragments of V(j+1)
    // possibly before the next barrier.  After the barrier every wave is done with K(j) and V(j-1), whose slots
    // are refilled with K(j+3) and V(j+3).
    int ks_next = 1, ks_cur = 0;      // K ring slots (j+1)%3 and j%3
    // Two waves share a SIMD (wave w and w + 4).  Block A of a step is VALU-heavy (exp, pack) and block B is pure
    // MFMA; if both waves of a SIMD took the step's barrier at the same point they would need the VALU together and
    // the matrix pipe together.  So the upper four waves take the SAME barrier between block A and block B
    // instead of in front of block A: they run half a step out of phase, and while one wave of a SIMD is in its
    // VALU-heavy block the other is in its MFMA block.  Such a wave reads K(j+1) and the first fragments of V(j)
    // before barrier j: both tiles are complete at barrier j - 1 (neither is the most recently issued group there),
    // and their slots are not refilled before barrier j + 1.
    const bool late_sync = QS == 1 && wave >= 4;
#define CDM_ATTN_STEP(SCUR, SNEXT)                                                                              \
    {                                                                                                           \
        const int k_fill = ks_cur;                              /* slot of K(j)   == j % 3     */               \
        const int k_next2 = ks_next == 2 ? 0 : ks_next + 1;     /* slot of K(j+2) == (j+2) % 3 */               \
        const int v_cur = j & 3, v_fill = (j + 3) & 3;          /* slots of V(j) and of V(j-1) */               \
        /* the K loads go out at the synchronisation point, the V loads half a step later: two bursts of two   */ \
        /* loads per wave instead of one of four (a wave sits in the vector-memory issue queue while its loads   */ \
        /* are accepted); both tiles were released by the same barrier                                           */ \
        auto sync = [&]() { asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(PER_WAVE) : "memory"); };      \
        auto load_k = [&]() { issue(kbase, kpre, sk_addr, j + 3, k_fill); };                                    \
        auto load_v = [&]() { issue(vbase, vpre, sv_addr, j + 3, v_fill); };                                    \
        if (!late_sync) { sync(); load_k(); }                                                                   \
        __builtin_amdgcn_sched_barrier(0);                                                                      \
        int nvalid[QB];                                                                                         \
        const bool pre_rag = j + 1 == pre_rag_tile;                                                             \
        _Pragma("unroll") for (int qb = 0; qb < QB; ++qb)                                                       \
            nvalid[qb] = pre_rag ? p.prefix_last_valid : klim[qb] - (j + 1) * BN;                               \
        /* does tile j + 1 (the scores block A computes) need row maxima?  its bit of the wave's table */      \
        pipe_step<HD, QB, LATE>([&]() { if (late_sync) { sync(); load_k(); } else load_v(); }, p.late_r,       \
                          sk + ks_next * TILE_BYTES, sv + v_cur * TILE_BYTES, sk + k_next2 * TILE_BYTES, qf, kw, \
                          SCUR, SNEXT, oacc, negm, l_run, lane, causal_wg || pre_rag || (ragged && j + 2 >= NT), nvalid, \
                          j + 1, next_hot, need_always, hot);     /* tile j + 1: the scores block A computes */ \
        __builtin_amdgcn_sched_barrier(0);                                                                      \
        if (late_sync) load_v();                                                                                \
        ks_cur = ks_next;                                                                                       \
        ks_next = ks_next == 2 ? 0 : ks_next + 1;                                                               \
    }
    for (int j = 0; j < NTW; ++j) {
        CDM_ATTN_STEP(s_a, s_b)
        if (++j >= NTW) break;
        CDM_ATTN_STEP(s_b, s_a)
    }
#undef CDM_ATTN_STEP
    // no direct-to-LDS write may outlive the workgroup; after the barrier no wave reads the K / V rings any more and
    // each wave stages its output rows there, so that they leave as whole 2 * HD-byte rows (16 bytes per lane, 4 or 8 rows
    // per store) instead of 8-byte pieces of 16 different rows
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    constexpr int PITCH = HD * 2 + 16;
    static_assert((NW / 2) * 32 * QS * PITCH <= RING * TILE_BYTES, "staging area exceeds a ring");
    char* stage = (wave < NW / 2 ? sk : sv) + (wave % (NW / 2)) * (32 * QS * PITCH);     // half the waves per ring
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        float l_tot = l_run[qb] + __shfl_xor(l_run[qb], 16, 64);
        l_tot += __shfl_xor(l_tot, 32, 64);
        const float inv = 1.0f / l_tot;
        float amax = 0.0f;
#pragma unroll
        for (int hb = 0; hb < HB; ++hb) {
            uint2 w;
            w.x = pack_bf16x2(oacc[hb][qb][0] * inv, oacc[hb][qb][1] * inv);
            w.y = pack_bf16x2(oacc[hb][qb][2] * inv, oacc[hb][qb][3] * inv);
            *reinterpret_cast<uint2*>(stage + (qb * 16 + r16) * PITCH + (16 * hb + 4 * g4) * 2) = w;
            amax = fmaxf(fmaxf(amax, fmaxf(fabsf(bf16lo(w.x)), fabsf(bf16hi(w.x)))), fmaxf(fabsf(bf16lo(w.y)), fabsf(bf16hi(w.y))));
        }
        if (unit >= 0) {      // a split unit leaves log2 of its sum of exponentials (reference added back) beside its rows
            // (a LATE kernel keeps the reference in the units of its accumulators: late_r times that is the exponent's)
            if (g4 == 0)
                p.part_lse[(int64_t)unit * BMQ + wave * (32 * QS) + qb * 16 + r16] =
                    __log2f(l_tot) - negm[qb][0] * (LATE ? p.late_r : 1.0f);
        } else if (p.row_amax != nullptr) {      // the row's channels of this head are spread over the four quarter-waves
            amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
            amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
            const int qrow = q0 + qb * 16 + r16;
            if (g4 == 0 && qrow < p.n_tokens) p.row_amax[(int64_t)qrow * p.n_heads + head] = amax;
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");      // the wave's own staging writes have landed
    constexpr int LPR = HD / 8, RPI = 64 / LPR;             // lanes per row, rows per store instruction
    const int rl = lane / LPR, ch = lane % LPR;
    bf16_t* orow = unit < 0 ? p.o + (int64_t)q0 * p.ldo + head * HD
                            : p.part_o + ((int64_t)unit * BMQ + wave * (32 * QS)) * HD;      // row of the wave's first query
    const int64_t ldo = unit < 0 ? p.ldo : HD;
#pragma unroll
    for (int it = 0; it < 32 * QS / RPI; ++it) {
        const int rloc = it * RPI + rl;
        const uint4 v = *reinterpret_cast<const uint4*>(stage + rloc * PITCH + ch * 16);
        if (q0 + rloc < p.n_tokens) *reinterpret_cast<uint4*>(orow + rloc * ldo + ch * 8) = v;
    }
}

// Merge of the split units' partial results: one workgroup per query block of the split tail.  Part i of a row holds
// o_i = (sum_k p_k v_k) / l_i over its key range and lse_i = log2(l_i) + m_i; the row of the whole range is
// sum_i w_i o_i / sum_i w_i with w_i = 2^(lse_i - max_i lse_i).
template <int HD>
__global__ __launch_bounds__(256) void merge_split_kernel(const PackedParams p) {
    constexpr int LPR = HD / 8;                       // lanes per row: 16 bytes each
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;      // j-th query block of the XCD's tail
    const int nqb = p.n_qblocks, hpx = (p.n_heads + 7) >> 3;
    const int k = hpx * nqb - p.split_tail + j;
    const int hi = k / nqb, head = xcd * hpx + hi, qblk = k - hi * nqb;
    for (int idx = threadIdx.x; idx < BMQ * LPR; idx += 256) {
        const int r = idx / LPR, ch = idx % LPR;
        const int qrow = qblk * BMQ + r;
        float lse[kMaxSplit], mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < kMaxSplit; ++i) {
            lse[i] = i < p.split ? p.part_lse[((int64_t)xcd * p.split_tail * p.split + i * p.split_tail + j) * BMQ + r] : -INFINITY;
            mx = fmaxf(mx, lse[i]);
        }
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, den = 0.0f;
#pragma unroll
        for (int i = 0; i < kMaxSplit; ++i) {
            if (i >= p.split) break;
            const float w = exp2f(lse[i] - mx);
            den += w;
            const uint4 u = *reinterpret_cast<const uint4*>(
                p.part_o + (((int64_t)xcd * p.split_tail * p.split + i * p.split_tail + j) * BMQ + r) * HD + ch * 8);
            const uint32_t q[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) { acc[2 * e] += w * bf16lo(q[e]); acc[2 * e + 1] += w * bf16hi(q[e]); }
        }
        const float inv = 1.0f / den;
        uint4 o;
        o.x = pack_bf16x2(acc[0] * inv, acc[1] * inv); o.y = pack_bf16x2(acc[2] * inv, acc[3] * inv);
        o.z = pack_bf16x2(acc[4] * inv, acc[5] * inv); o.w = pack_bf16x2(acc[6] * inv, acc[7] * inv);
        if (qrow < p.n_tokens) *reinterpret_cast<uint4*>(p.o + (int64_t)qrow * p.ldo + head * HD + ch * 8) = o;
        if (p.row_amax != nullptr) {      // LPR consecutive lanes hold the row
            const uint32_t q[4] = {o.x, o.y, o.z, o.w};
            float amax = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) amax = fmaxf(amax, fmaxf(fabsf(bf16lo(q[e])), fabsf(bf16hi(q[e]))));
#pragma unroll
            for (int off = 1; off < LPR; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
            if (ch == 0 && qrow < p.n_tokens) p.row_amax[(int64_t)qrow * p.n_heads + head] = amax;
        }
    }
}

// K, V [n_tokens, n_heads, HD] -> tile images Kp, Vp (see above); one workgroup per (64-key tile, head).
// With cos/sin tables ([n_tokens, HD/2] fp32) K is rotated on the way (rotate-half pairs (i, i + HD/2)).
template <int HD>
__global__ __launch_bounds__(256) void pack_kv_kernel(const bf16_t* __restrict__ k, int64_t ldk,
                                                      const bf16_t* __restrict__ v, int64_t ldv,
                                                      const float* __restrict__ cos, const float* __restrict__ sin,
                                                      const QkNormDev kn, char* __restrict__ kp, char* __restrict__ vp,
                                                      float* __restrict__ kmax, int n_tokens, int n_tiles) {
    __shared__ bf16_t tile[64][HD + 2];
    __shared__ float wave_kmax[4];
    float ksq_max = 0.0f;      // largest squared norm among the keys this thread has helped with
    constexpr int CPR = HD / 8;                 // 16-byte chunks per token row
    constexpr int HALF = HD / 2;
    constexpr int TILE_BYTES = BN * HD * 2;
    // heads vary fastest over the grid: the K / V rows of neighbouring heads are adjacent in memory, so the
    // workgroups that run together share DRAM pages and cache lines
    const int tile_idx = blockIdx.y, head = blockIdx.x;
    const int t0 = tile_idx * 64;
    char* kt = kp + ((int64_t)head * n_tiles + tile_idx) * TILE_BYTES;
    char* vt = vp + ((int64_t)head * n_tiles + tile_idx) * TILE_BYTES;
    // one thread handles the chunk pair (ch, ch + CPR/2) of one token: the two halves of 8 rotary pairs
    for (int idx = threadIdx.x; idx < 64 * (CPR / 2); idx += 256) {
        const int r = idx / (CPR / 2), ch = idx % (CPR / 2);
        uint4 k1 = make_uint4(0, 0, 0, 0), k2 = k1, v1 = k1, v2 = k1;
        if (t0 + r < n_tokens) {
            const bf16_t* kr = k + (int64_t)(t0 + r) * ldk + head * HD + ch * 8;
            const bf16_t* vr = v + (int64_t)(t0 + r) * ldv + head * HD + ch * 8;
            k1 = *reinterpret_cast<const uint4*>(kr);
            k2 = *reinterpret_cast<const uint4*>(kr + HALF);
            v1 = *reinterpret_cast<const uint4*>(vr);
            v2 = *reinterpret_cast<const uint4*>(vr + HALF);
            if (cos != nullptr || kn.w != nullptr) {
                float c[8], sn[8], n1[8], n2[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) { c[e] = 1.0f; sn[e] = 0.0f; n1[e] = 1.0f; n2[e] = 1.0f; }
                const uint32_t w1[4] = {k1.x, k1.y, k1.z, k1.w}, w2[4] = {k2.x, k2.y, k2.z, k2.w};
                if (kn.w != nullptr) {
                    // per-head RMSNorm: the CPR/2 consecutive threads of a token hold its HD channels
                    float ss = 0.0f;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float a0 = bf16lo(w1[j]), a1 = bf16hi(w1[j]), b0 = bf16lo(w2[j]), b1 = bf16hi(w2[j]);
                        ss += a0 * a0 + a1 * a1 + b0 * b0 + b1 * b1;
                    }
#pragma unroll
                    for (int off = 1; off < CPR / 2; off <<= 1) ss += __shfl_xor(ss, off, 64);
                    const float rn = rsqrtf(ss * (1.0f / HD) + kn.eps);
                    const float* nw = kn.row(t0 + r, HD) + ch * 8;
#pragma unroll
                    for (int e = 0; e < 8; ++e) { n1[e] = rn * nw[e]; n2[e] = rn * nw[HALF + e]; }
                }
                if (cos != nullptr) {
                    const float4* cp = reinterpret_cast<const float4*>(cos + (int64_t)(t0 + r) * HALF + ch * 8);
                    const float4* sp = reinterpret_cast<const float4*>(sin + (int64_t)(t0 + r) * HALF + ch * 8);
                    const float4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
                    c[0] = c0.x; c[1] = c0.y; c[2] = c0.z; c[3] = c0.w; c[4] = c1.x; c[5] = c1.y; c[6] = c1.z; c[7] = c1.w;
                    sn[0] = s0.x; sn[1] = s0.y; sn[2] = s0.z; sn[3] = s0.w; sn[4] = s1.x; sn[5] = s1.y; sn[6] = s1.z; sn[7] = s1.w;
                }
                uint32_t o1[4], o2[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float a0 = bf16lo(w1[j]) * n1[2 * j], a1 = bf16hi(w1[j]) * n1[2 * j + 1];
                    const float b0 = bf16lo(w2[j]) * n2[2 * j], b1 = bf16hi(w2[j]) * n2[2 * j + 1];
                    o1[j] = pack_bf16x2(a0 * c[2 * j] - b0 * sn[2 * j], a1 * c[2 * j + 1] - b1 * sn[2 * j + 1]);
                    o2[j] = pack_bf16x2(b0 * c[2 * j] + a0 * sn[2 * j], b1 * c[2 * j + 1] + a1 * sn[2 * j + 1]);
                }
                k1 = make_uint4(o1[0], o1[1], o1[2], o1[3]);
                k2 = make_uint4(o2[0], o2[1], o2[2], o2[3]);
            }
        }
        {   // squared norm of the key as stored (rounded to bf16): the CPR/2 consecutive threads of a token hold it
            const uint32_t w1[4] = {k1.x, k1.y, k1.z, k1.w}, w2[4] = {k2.x, k2.y, k2.z, k2.w};
            float ss = 0.0f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float a0 = bf16lo(w1[j]), a1 = bf16hi(w1[j]), b0 = bf16lo(w2[j]), b1 = bf16hi(w2[j]);
                ss += a0 * a0 + a1 * a1 + b0 * b0 + b1 * b1;
            }
#pragma unroll
            for (int off = 1; off < CPR / 2; off <<= 1) ss += __shfl_xor(ss, off, 64);
            ksq_max = fmaxf(ksq_max, ss);
        }
        *reinterpret_cast<uint4*>(kt + (ch * 64 + r) * 16) = k1;                  // chunk-major K image
        *reinterpret_cast<uint4*>(kt + ((ch + CPR / 2) * 64 + r) * 16) = k2;
        uint32_t* d1 = reinterpret_cast<uint32_t*>(&tile[r][ch * 8]);
        uint32_t* d2 = reinterpret_cast<uint32_t*>(&tile[r][HALF + ch * 8]);
        d1[0] = v1.x; d1[1] = v1.y; d1[2] = v1.z; d1[3] = v1.w;
        d2[0] = v2.x; d2[1] = v2.y; d2[2] = v2.z; d2[3] = v2.w;
    }
    ksq_max = wave_max(ksq_max);
    if ((threadIdx.x & 63) == 0) wave_kmax[threadIdx.x >> 6] = ksq_max;
    __syncthreads();
    if (threadIdx.x == 0)
        kmax[(int64_t)head * n_tiles + tile_idx] =
            sqrtf(fmaxf(fmaxf(wave_kmax[0], wave_kmax[1]), fmaxf(wave_kmax[2], wave_kmax[3])));
    for (int idx = threadIdx.x; idx < HD * 8; idx += 256) {
        const int row = idx % HD, c = idx / HD;                            // channel row, key chunk
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            // chunk c = 4 s + g lists keys 32 s + 4 g + {0..3}, 32 s + 16 + 4 g + {0..3}: the order in which a lane of the
            // attention kernel holds its probabilities of the 32-key step s
            const int key = 32 * (c >> 2) + 4 * (c & 3) + 16 * (e >> 1) + 2 * (e & 1);
            w[e] = (uint32_t)tile[key][row] | ((uint32_t)tile[key + 1][row] << 16);
        }
        *reinterpret_cast<uint4*>(vt + (c * HD + row) * 16) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

inline int64_t pad_tokens(int64_t n) { return (n + BN - 1) / BN * BN; }
inline int64_t image_bytes(int64_t n_tokens, int n_heads, int head_dim) {      // one packed tensor
    return pad_tokens(n_tokens) * n_heads * head_dim * 2;
}
inline int64_t kmax_bytes(int64_t n_tokens, int n_heads) {      // one float per (head, tile), padded to 16 bytes
    return (pad_tokens(n_tokens) / BN * n_heads * 4 + 15) / 16 * 16;
}

// The last, partial round of workgroups.  An XCD owns heads/8 x query blocks workgroups and runs 32 at a time (one per
// CU: the K / V rings fill the LDS), so a launch takes ceil(workgroups / 32) rounds of equal length however few
// workgroups the last round holds.  The plan cuts each query block of that last round into `split` units by key range
// (the smallest of 2, 4, 8 that minimises ceil(tail * split / 32) / split rounds), which the merge kernel puts together.
// Only where it pays: the chip is power-limited, so a round that leaves CUs idle already runs faster than a full one,
// and every unit repeats the set-up; measured at 56 k tokens x 32 heads, a plan that ends in half a round or less gains
// 1 - 3 % and one that ends in three quarters gains nothing.  So: the split round must take at most half a round, and
// there must be at least two whole rounds, heads a multiple of 8, at least 8 key tiles per unit, and no causal rows in
// the tail's query blocks.
struct SplitPlan { int split, tail; int64_t bytes; };
inline SplitPlan split_plan(int64_t n_tokens, int n_heads, int head_dim, int64_t causal_prefix) {
    SplitPlan none{1, 0, 0};
    const int64_t nqb = (n_tokens + BMQ - 1) / BMQ, per_xcd = (n_heads / 8) * nqb;
    if (n_heads % 8 != 0 || per_xcd < 64) return none;
    const int tail = (int)(per_xcd % 32);
    if (tail == 0) return none;
    if (causal_prefix > 0 && (tail >= nqb || (nqb - tail) * BMQ < causal_prefix)) return none;
    const int64_t nm = (n_tokens + BN - 1) / BN;
    int best = 1;
    double best_cost = 1.0;
    for (int s = 2; s <= kMaxSplit && nm / s >= 8; s *= 2) {
        const double cost = (double)((tail * s + 31) / 32) / s;
        if (cost < best_cost - 1e-9) { best_cost = cost; best = s; }
    }
    if (best == 1 || best_cost > 0.5 + 1e-9) return none;
    const int64_t units = 8ll * tail * best;
    return SplitPlan{best, tail, units * BMQ * ((int64_t)head_dim * 2 + 4)};
}

// host view of the optional QK-norm argument -> kernel descriptor (which = 0: q weights, 1: k weights)
int32_t make_qk_norm(const char* who, const cdm_qk_norm* qn, int which, int64_t n_tokens, QkNormDev* out) {
    out->w = nullptr; out->n_seg = 0; out->eps = 0.0f;
    for (int i = 0; i < 8; ++i) out->seg_end[i] = 0;
    if (qn == nullptr) return CDM_OK;
    const float* w = which == 0 ? qn->q_weight : qn->k_weight;
    CDM_REQUIRE(qn->q_weight && qn->k_weight, CDM_ERR_BAD_ARG, "%s: qk_norm needs both weight tables", who);
    CDM_REQUIRE(qn->n_seg >= 1 && qn->n_seg <= 8 && qn->seg_end, CDM_ERR_BAD_ARG, "%s: qk_norm n_seg=%d must be 1..8", who,
                qn->n_seg);
    CDM_REQUIRE(qn->eps > 0.0f, CDM_ERR_BAD_ARG, "%s: qk_norm eps must be positive", who);
    int64_t prev = 0;
    for (int i = 0; i < qn->n_seg; ++i) {
        CDM_REQUIRE(qn->seg_end[i] >= prev, CDM_ERR_BAD_ARG, "%s: qk_norm segment ends must not decrease", who);
        prev = qn->seg_end[i];
        out->seg_end[i] = (int)(prev < (1ll << 30) ? prev : (1ll << 30));
    }
    CDM_REQUIRE(prev >= n_tokens, CDM_ERR_BAD_ARG, "%s: qk_norm segments cover %lld of %lld tokens", who, (long long)prev,
                (long long)n_tokens);
    out->w = w; out->n_seg = qn->n_seg; out->eps = qn->eps;
    return CDM_OK;
}

int32_t check_attn_common(const char* who, int64_t n_tokens, int32_t n_heads, int32_t head_dim, const float* cos,
                          const float* sin) {
    CDM_REQUIRE(n_tokens >= 0 && n_heads > 0, CDM_ERR_BAD_ARG, "%s: bad sizes", who);
    CDM_REQUIRE(head_dim == 64 || head_dim == 128, CDM_ERR_BAD_SHAPE, "%s: head_dim=%d must be 64 or 128", who, head_dim);
    CDM_REQUIRE(n_tokens <= 65535ll * BN && n_heads <= 65535, CDM_ERR_BAD_SHAPE, "%s: sizes out of range", who);
    CDM_REQUIRE((cos == nullptr) == (sin == nullptr), CDM_ERR_BAD_ARG, "%s: cos and sin must be given together", who);
    CDM_REQUIRE(cdm_aligned16(cos) && cdm_aligned16(sin), CDM_ERR_BAD_ALIGN, "%s: rotary tables must be 16-byte aligned", who);
    return CDM_OK;
}

}  // namespace

// workspace = [Kp | Vp | kmax]: the two tile images and the largest key norm of every tile; n_heads counts K / V heads
extern "C" int64_t cdm_attn_workspace_bytes(int64_t n_tokens, int32_t n_heads, int32_t head_dim) {
    if (n_tokens < 0 || n_heads <= 0 || head_dim <= 0) return 0;
    return 2 * image_bytes(n_tokens, n_heads, head_dim) + kmax_bytes(n_tokens, n_heads);
}

// scratch for the split of the last round of workgroups (0: this shape has nothing to split); n_heads counts QUERY heads
extern "C" int64_t cdm_attn_split_scratch_bytes(int64_t n_tokens, int32_t n_heads, int32_t head_dim) {
    if (n_tokens <= 0 || n_heads <= 0 || (head_dim != 64 && head_dim != 128)) return 0;
    return split_plan(n_tokens, n_heads, head_dim, 0).bytes;
}

extern "C" int32_t cdm_attn_pack_kv_bf16(const void* k, int64_t ldk, const void* v, int64_t ldv, const float* cos,
                                         const float* sin, void* workspace, int64_t workspace_bytes,
                                         int64_t n_tokens, int32_t n_heads, int32_t head_dim,
                                         const cdm_qk_norm* qk_norm, void* stream) {
    CDM_REQUIRE(k && v && workspace, CDM_ERR_BAD_ARG, "attn_pack_kv: null pointer");
    int32_t rc = check_attn_common("attn_pack_kv", n_tokens, n_heads, head_dim, cos, sin);
    if (rc) return rc;
    QkNormDev kn;
    if ((rc = make_qk_norm("attn_pack_kv", qk_norm, 1, n_tokens, &kn))) return rc;
    const int64_t d = (int64_t)n_heads * head_dim;
    CDM_REQUIRE(ldk >= d && ldv >= d, CDM_ERR_BAD_ARG, "attn_pack_kv: row stride smaller than n_heads*head_dim");
    CDM_REQUIRE(cdm_aligned16(k) && cdm_aligned16(v) && cdm_aligned16(workspace) && ldk % 8 == 0 && ldv % 8 == 0,
                CDM_ERR_BAD_ALIGN, "attn_pack_kv: pointers/strides must be 16-byte aligned");
    const int64_t need = cdm_attn_workspace_bytes(n_tokens, n_heads, head_dim);
    CDM_REQUIRE(workspace_bytes >= need, CDM_ERR_BAD_ARG, "attn_pack_kv: workspace of at least %lld bytes required",
                (long long)need);
    if (n_tokens == 0) return CDM_OK;
    if ((rc = cdm_require_device())) return rc;
    const int n_tiles = (int)(pad_tokens(n_tokens) / BN);
    const int64_t img = image_bytes(n_tokens, n_heads, head_dim);
    char* ws = (char*)workspace;
    dim3 grid(n_heads, n_tiles);
    hipStream_t st = (hipStream_t)stream;
    if (head_dim == 128)
        pack_kv_kernel<128><<<grid, 256, 0, st>>>((const bf16_t*)k, ldk, (const bf16_t*)v, ldv, cos, sin, kn, ws, ws + img,
                                                  (float*)(ws + 2 * img), (int)n_tokens, n_tiles);
    else
        pack_kv_kernel<64><<<grid, 256, 0, st>>>((const bf16_t*)k, ldk, (const bf16_t*)v, ldv, cos, sin, kn, ws, ws + img,
                                                 (float*)(ws + 2 * img), (int)n_tokens, n_tiles);
    return cdm_check_launch("attn_pack_kv");
}

extern "C" int32_t cdm_attn_fwd_packed_bf16(const void* q, int64_t ldq, const float* cos, const float* sin,
                                            const void* workspace, void* o, int64_t ldo, int64_t n_tokens,
                                            int32_t n_heads, int32_t n_kv_heads, int32_t head_dim,
                                            const cdm_qk_norm* qk_norm, const void* prefix_workspace,
                                            int64_t n_prefix_tokens, int64_t causal_prefix, float* row_amax,
                                            void* split_scratch, int64_t split_scratch_bytes, void* stream) {
    CDM_REQUIRE(q && workspace && o, CDM_ERR_BAD_ARG, "attn_fwd_packed: null pointer");
    CDM_REQUIRE(cdm_aligned16(split_scratch) && (split_scratch == nullptr || split_scratch_bytes >= 0), CDM_ERR_BAD_ARG,
                "attn_fwd_packed: split_scratch must be 16-byte aligned, its size non-negative");
    CDM_REQUIRE((reinterpret_cast<uintptr_t>(row_amax) & 3u) == 0, CDM_ERR_BAD_ALIGN, "attn_fwd_packed: row_amax must be 4-byte aligned");
    CDM_REQUIRE(n_kv_heads > 0 && n_heads > 0 && n_heads % n_kv_heads == 0, CDM_ERR_BAD_SHAPE,
                "attn_fwd_packed: n_kv_heads=%d must divide n_heads=%d", n_kv_heads, n_heads);
    CDM_REQUIRE(n_prefix_tokens >= 0 && n_prefix_tokens < (1ll << 23), CDM_ERR_BAD_SHAPE,
                "attn_fwd_packed: n_prefix_tokens=%lld out of range", (long long)n_prefix_tokens);
    CDM_REQUIRE((n_prefix_tokens > 0) == (prefix_workspace != nullptr) && cdm_aligned16(prefix_workspace), CDM_ERR_BAD_ARG,
                "attn_fwd_packed: prefix_workspace and n_prefix_tokens must be given together (16-byte aligned)");
    CDM_REQUIRE(causal_prefix >= 0 && causal_prefix <= n_tokens, CDM_ERR_BAD_ARG,
                "attn_fwd_packed: causal_prefix=%lld outside [0, n_tokens]", (long long)causal_prefix);
    CDM_REQUIRE(causal_prefix == 0 || n_prefix_tokens == 0, CDM_ERR_UNSUPPORTED,
                "attn_fwd_packed: a causal prefix cannot be combined with prefix key images");
    int32_t rc = check_attn_common("attn_fwd_packed", n_tokens, n_heads, head_dim, cos, sin);
    if (rc) return rc;
    QkNormDev qn;
    if ((rc = make_qk_norm("attn_fwd_packed", qk_norm, 0, n_tokens, &qn))) return rc;
    const int64_t d = (int64_t)n_heads * head_dim;
    CDM_REQUIRE(ldq >= d && ldo >= d, CDM_ERR_BAD_ARG, "attn_fwd_packed: row stride smaller than n_heads*head_dim");
    CDM_REQUIRE(cdm_aligned16(q) && cdm_aligned16(workspace) && cdm_aligned16(o) && ldq % 8 == 0 && ldo % 8 == 0,
                CDM_ERR_BAD_ALIGN, "attn_fwd_packed: pointers/strides must be 16-byte aligned");
    if (n_tokens == 0) return CDM_OK;
    if ((rc = cdm_require_device())) return rc;
    const int64_t img = image_bytes(n_tokens, n_kv_heads, head_dim);
    PackedParams p;
    p.q = (const bf16_t*)q; p.ldq = ldq;
    p.kp = (const char*)workspace; p.vp = (const char*)workspace + img;
    p.kmax = (const float*)((const char*)workspace + 2 * img);
    p.kp_prefix = (const char*)prefix_workspace;
    p.vp_prefix = (const char*)prefix_workspace + image_bytes(n_prefix_tokens, n_kv_heads, head_dim);
    p.kmax_prefix = (const float*)((const char*)prefix_workspace + 2 * image_bytes(n_prefix_tokens, n_kv_heads, head_dim));
    p.n_prefix_tiles = (int)(pad_tokens(n_prefix_tokens) / BN);
    p.prefix_last_valid = (int)(n_prefix_tokens - (pad_tokens(n_prefix_tokens) - BN));      // BN for whole tiles
    p.causal_prefix = (int)causal_prefix;
    p.o = (bf16_t*)o; p.ldo = ldo;
    p.row_amax = row_amax;
    p.cos = cos; p.sin = sin;
    p.qn = qn;
    p.n_tokens = (int)n_tokens; p.n_heads = n_heads; p.kv_group = n_heads / n_kv_heads;
    // Q untouched by rotation and norm: only the power-of-two part of the factor goes into Q (see LATE above)
    const bool late = cos == nullptr && qk_norm == nullptr;
    const float full = 1.4426950408889634f / sqrtf((float)head_dim);
    int ex = 0;
    const float mant = frexpf(full, &ex);                 // full = mant * 2^ex, mant in [0.5, 1)
    p.scale_log2e = late ? ldexpf(1.0f, ex - 1) : full;
    p.late_r = late ? 2.0f * mant : 1.0f;
    p.n_qblocks = (int)((n_tokens + BMQ - 1) / BMQ);
    // 1-D grid of 8 x ceil(heads / 8) x query blocks ids: id % 8 = XCD, see the kernel's placement rule
    // variant 0 = 32 query rows per wave (8 waves, two per SIMD), row maxima dropped where the norm bound allows;
    // cross-check build only: 1 = 64 query rows per wave (4 waves), 2 = variant 0 with the row maxima always taken
    const int variant = cdm_get_variant(0);
    p.always_max = variant == 2;
    // the last round's query blocks by key range, if the caller brought the scratch memory for it
    p.split = 1; p.split_tail = 0; p.part_o = nullptr; p.part_lse = nullptr;
    const SplitPlan plan = split_plan(n_tokens, n_heads, head_dim, causal_prefix);
    if (split_scratch != nullptr && plan.split > 1 && split_scratch_bytes >= plan.bytes && variant != 1) {
        p.split = plan.split; p.split_tail = plan.tail;
        p.part_o = (bf16_t*)split_scratch;
        p.part_lse = (float*)((char*)split_scratch + 8ll * plan.tail * plan.split * BMQ * head_dim * 2);
    }
    const int64_t nwg = 8ll * ((n_heads + 7) / 8) * p.n_qblocks + 8ll * p.split_tail * (p.split - 1);
    CDM_REQUIRE(nwg < (1ll << 31), CDM_ERR_BAD_SHAPE, "attn_fwd_packed: grid too large");
    dim3 grid((unsigned)nwg);
    hipStream_t st = (hipStream_t)stream;
#define CDM_ATTN_LAUNCH(QS_, THREADS)                                                                      \
    if (head_dim == 128 && late) attn_fwd_pipe_kernel<128, QS_, true><<<grid, THREADS, 0, st>>>(p);       \
    else if (head_dim == 128) attn_fwd_pipe_kernel<128, QS_, false><<<grid, THREADS, 0, st>>>(p);         \
    else if (late) attn_fwd_pipe_kernel<64, QS_, true><<<grid, THREADS, 0, st>>>(p);                      \
    else attn_fwd_pipe_kernel<64, QS_, false><<<grid, THREADS, 0, st>>>(p)
#ifdef CDM_CROSSCHECK
    if (variant == 1) { CDM_ATTN_LAUNCH(2, 256); }
    else
#endif
    { CDM_ATTN_LAUNCH(1, 512); }
#undef CDM_ATTN_LAUNCH
    if (p.split > 1) {
        if ((rc = cdm_check_launch("attn_fwd_packed"))) return rc;
        if (head_dim == 128) merge_split_kernel<128><<<dim3(8u * p.split_tail), 256, 0, st>>>(p);
        else merge_split_kernel<64><<<dim3(8u * p.split_tail), 256, 0, st>>>(p);
    }
    return cdm_check_launch("attn_fwd_packed");
}

extern "C" int32_t cdm_attn_fwd_bf16(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v,
                                     int64_t ldv, const float* cos, const float* sin, void* o, int64_t ldo,
                                     int64_t n_tokens, int32_t n_heads, int32_t n_kv_heads, int32_t head_dim,
                                     void* workspace, int64_t workspace_bytes, const cdm_qk_norm* qk_norm,
                                     int64_t causal_prefix, void* stream) {
    CDM_REQUIRE(q && k && v && o, CDM_ERR_BAD_ARG, "attn_fwd: null pointer");
    int32_t rc = check_attn_common("attn_fwd", n_tokens, n_heads, head_dim, cos, sin);
    if (rc) return rc;
    CDM_REQUIRE(n_kv_heads > 0 && n_heads % n_kv_heads == 0, CDM_ERR_BAD_SHAPE,
                "attn_fwd: n_kv_heads=%d must divide n_heads=%d", n_kv_heads, n_heads);
    {
        QkNormDev tmp;
        if ((rc = make_qk_norm("attn_fwd", qk_norm, 0, n_tokens, &tmp))) return rc;
    }
    if (n_tokens == 0) return CDM_OK;
    const int64_t need = cdm_attn_workspace_bytes(n_tokens, n_kv_heads, head_dim);
    CDM_REQUIRE(workspace && cdm_aligned16(workspace) && workspace_bytes >= need, CDM_ERR_BAD_ARG,
                "attn_fwd: workspace of at least %lld bytes required", (long long)need);
    // validate the second stage's arguments before the first stage is enqueued
    const int64_t d = (int64_t)n_heads * head_dim, dkv = (int64_t)n_kv_heads * head_dim;
    CDM_REQUIRE(ldq >= d && ldk >= dkv && ldv >= dkv && ldo >= d, CDM_ERR_BAD_ARG,
                "attn_fwd: row stride smaller than heads*head_dim");
    CDM_REQUIRE(causal_prefix >= 0 && causal_prefix <= n_tokens, CDM_ERR_BAD_ARG,
                "attn_fwd: causal_prefix=%lld outside [0, n_tokens]", (long long)causal_prefix);
    CDM_REQUIRE(cdm_aligned16(q) && cdm_aligned16(k) && cdm_aligned16(v) && cdm_aligned16(o) && ldq % 8 == 0 &&
                    ldk % 8 == 0 && ldv % 8 == 0 && ldo % 8 == 0,
                CDM_ERR_BAD_ALIGN, "attn_fwd: pointers/strides must be 16-byte aligned");
    if ((rc = cdm_attn_pack_kv_bf16(k, ldk, v, ldv, cos, sin, workspace, workspace_bytes, n_tokens, n_kv_heads, head_dim,
                                    qk_norm, stream)))
        return rc;
    // what the caller's workspace holds beyond the images serves the split of the last round
    const int64_t used = (need + 255) / 256 * 256;
    void* extra = workspace_bytes > used ? (char*)workspace + used : nullptr;
    return cdm_attn_fwd_packed_bf16(q, ldq, cos, sin, workspace, o, ldo, n_tokens, n_heads, n_kv_heads, head_dim, qk_norm,
                                    nullptr, 0, causal_prefix, nullptr, extra, extra ? workspace_bytes - used : 0, stream);
}

// ---------------------------------------------------------------------------------------------
// The same operator for callers that can neither allocate nor bring a workspace: the K / V tile images go into a
// file-scope device array.  In host code the array's NAME is only a handle; its device address is looked up once
// per device (hipGetSymbolAddress, with that device current) and every use below goes through that pointer.
// ---------------------------------------------------------------------------------------------
namespace {

constexpr int64_t kStaticScratchBytes = CDM_ATTN_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};      // device address of `scratch` on each device (null = not looked up yet)

// address of the current device's copy of `scratch`
int32_t static_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices)
        CDM_FAIL(CDM_ERR_NO_DEVICE, "attn_fwd_static: no current device (%s)", hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            CDM_FAIL(CDM_ERR_LAUNCH, "attn_fwd_static: hipGetSymbolAddress failed on device %d: %s", dev,
                     hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return CDM_OK;
}

}  // namespace

// Also the set-up call: with a device visible it resolves the array's address on the current device, so that a caller
// which records cdm_attn_fwd_static_bf16 into a graph can have that done outside the capture.
extern "C" int64_t cdm_attn_static_scratch_bytes(void) {
    if (cdm_device_count() > 0) {
        void* ws = nullptr;
        (void)static_scratch(&ws);      // a failure is reported by the entry point itself
    }
    return kStaticScratchBytes;
}

extern "C" int32_t cdm_attn_fwd_static_bf16(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v,
                                            int64_t ldv, const float* cos, const float* sin, void* o, int64_t ldo,
                                            int64_t n_tokens, int32_t n_heads, int32_t n_kv_heads, int32_t head_dim,
                                            const cdm_qk_norm* qk_norm, int64_t causal_prefix, void* stream) {
    CDM_REQUIRE(n_tokens >= 0 && n_kv_heads > 0 && head_dim > 0, CDM_ERR_BAD_ARG, "attn_fwd_static: bad sizes");
    CDM_REQUIRE(n_tokens <= 65535ll * BN, CDM_ERR_BAD_SHAPE, "attn_fwd_static: sizes out of range");
    const int64_t need = cdm_attn_workspace_bytes(n_tokens, n_kv_heads, head_dim);
    CDM_REQUIRE(need <= kStaticScratchBytes, CDM_ERR_BAD_SHAPE,
                "attn_fwd_static: K/V tile images of %lld tokens x %d K/V heads x %d need %lld bytes, the built-in "
                "scratch holds %lld; use cdm_attn_fwd_bf16 with a caller-owned workspace",
                (long long)n_tokens, n_kv_heads, head_dim, (long long)need, (long long)kStaticScratchBytes);
    void* ws = nullptr;
    if (n_tokens > 0) {
        int32_t rc = cdm_require_device();
        if (rc) return rc;
        if ((rc = static_scratch(&ws))) return rc;
    }
    // exactly the images' size: the array holds no scratch for a split of the last round of workgroups
    return cdm_attn_fwd_bf16(q, ldq, k, ldk, v, ldv, cos, sin, o, ldo, n_tokens, n_heads, n_kv_heads, head_dim, ws,
                             need, qk_norm, causal_prefix, stream);
}

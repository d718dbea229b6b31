// "NT" GEMM  C[M,N] = A[M,K] . W[N,K]^T  on the gfx950 matrix cores with fused epilogues, for bf16
// operands (v_mfma_f32_16x16x32_bf16) and for e4m3 operands with per-row / per-column fp32 scales
// (v_mfma_scale_f32_16x16x128_f8f6f4 with unit block scales; the rank-1 scale sa[i]*sw[j] is applied
// to the fp32 accumulator in the epilogue).  A k-tile is 128 BYTES of K for both types, so the LDS
// geometry, loads and swizzle are shared.
//
// Tiling: one workgroup computes a 256x256 tile with BK = 64.  Default: 8 waves (4x2), each owning a 64x128 sub-tile
// = 4x8 accumulators of 16x16 (128 fp32 registers per lane).  Cross-check: 4 waves (2x2) of 128x128 = 4x4
// v_mfma_f32_32x32x16_bf16 accumulators (256 registers) on a plain two-stage pipeline.
// Both operands are K-contiguous, so A and W fragments are plain 16-byte LDS reads.
// Global -> LDS goes through the direct-to-LDS path (global_load_lds_dwordx4): each wave
// instruction deposits 64 x 16 B = 8 tile rows linearly in LDS; bank conflicts are avoided by
// permuting which 16-byte chunk of a row each lane fetches (XOR swizzle on the source side).
// Two pipelines share tile, swizzle idea and epilogues: a two-stage one (2 x 64 KB of LDS: the loads of k-tile
// t+1 are in flight while k-tile t is multiplied) and the default five-slot ring further down.
// Workgroup ids are remapped so that each XCD (ids are dealt round-robin over the 8 XCDs) works
// on a compact block of tiles and its private L2 sees the reuse.
#include <type_traits>

#include "cdm_common.h"

namespace {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kThreads = 256;
constexpr int kTileBytes = BM * BK * 2;   // 32 KB per operand per stage

typedef __attribute__((address_space(3))) void lds_void;

typedef __attribute__((ext_vector_type(8))) int i32x8;

constexpr int kMaxSeg = 8;

// One launch covers up to kMaxSeg contiguous row segments of A / C / R, each with its own weights (the MoT
// branches): the grid is the concatenation of the segments' tile lists, so the few tiles of a short segment (a
// 256-token action run, a 512-token text run) fill the tail of the long segment's grid instead of paying for a
// launch of their own that cannot fill the chip.
struct GemmSeg {
    int m_start, m_end;                  // token rows [m_start, m_end)
    int tiles_m, tile_end;               // row tiles of the segment; tiles of segments 0..this one
    const void* W; const void* W2;
    const float* gate;
    const float* sw; const float* sw2;   // fp8 only
    const float* knw;                    // QKV_PACK only: the segment's K-norm weight row [head_dim] fp32, or null
};

struct GemmParams {
    const void* A; int64_t lda;          // operand strides in BYTES
    int64_t ldw;
    const float* sa;                     // fp8 only: per-row scale of A, indexed by the global row
    bf16_t* C; int64_t ldc;              // fp32 storage behind the same pointers for CDM_EPI_GATE_RESIDUAL_F32
    int N, K;
    const bf16_t* R; int64_t ldr;
    const float* cos; const float* sin;
    int rope_cols, head_dim;
    // CDM_EPI_QKV_PACK: columns [0, d_q) are Q (written to C), [d_q, d_q + d_kv) K and the rest V; K and V leave as the
    // attention kernel's tile images (64 keys x 128 channels per K / V head), with the largest key norm of every tile
    char* kp; char* vp; float* kmax;
    int d_q, d_kv, n_key_tiles;
    float k_eps;                         // epsilon of the per-head RMSNorm of K (segments with a weight row)
    // CDM_EPI_SWIGLU, optional: [M, amax_ld] fp32, entry (row, c) = largest |output| of the row within output columns
    // 64 c .. 64 c + 63 (as stored): what a per-row quantiser of the output needs, without a pass of its own
    float* row_amax; int64_t amax_ld;
    int tiles_n, total_tiles, n_seg;
    GemmSeg seg[kMaxSeg];
};

// what a workgroup works on
struct Tile {
    int m0, m_end, tn;
    const void* W; const void* W2;
    const float* gate; const float* sw; const float* sw2; const float* knw;
};

// XCD-aware tile assignment: workgroup ids are dealt round-robin over the 8 XCDs, so ids are remapped to give each
// XCD a contiguous range of tiles; inside a segment, tiles are ordered in groups of 4 row tiles x all column tiles,
// column-major inside the group, so that the 32 tiles an XCD runs at a time share 4 A slabs and 8 W slabs in its L2
// (measured best among group heights 2, 3, 4, 6, 8, 16 once the output tiles are stored non-temporally).
template <class T>
__device__ __forceinline__ T* uniform_ptr(T* ptr) {      // wave-uniform value -> scalar registers
    const uint64_t v = reinterpret_cast<uint64_t>(ptr);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<T*>(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ bool locate_tile(const GemmParams& p, Tile& t) {
    const int per_xcd = (p.total_tiles + 7) >> 3;
    int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= p.total_tiles) return false;
    int si = 0;
#pragma unroll
    for (int i = 0; i < kMaxSeg - 1; ++i) si += (i < p.n_seg - 1 && logical >= p.seg[i].tile_end) ? 1 : 0;
    const GemmSeg& sg = p.seg[si];
    logical -= si ? p.seg[si - 1].tile_end : 0;
    constexpr int GM = 4;
    const int group = logical / (GM * p.tiles_n);
    const int first_m = group * GM;
    const int gsz = (sg.tiles_m - first_m) < GM ? (sg.tiles_m - first_m) : GM;
    const int in_group = logical - group * GM * p.tiles_n;
    // everything here is a function of blockIdx: pin it to scalar registers (the segment table is indexed
    // dynamically, which the compiler would otherwise treat as a per-lane value)
    t.m0 = __builtin_amdgcn_readfirstlane(sg.m_start + (first_m + in_group % gsz) * BM);
    t.m_end = __builtin_amdgcn_readfirstlane(sg.m_end);
    t.tn = __builtin_amdgcn_readfirstlane(in_group / gsz);
    t.W = uniform_ptr(sg.W); t.W2 = uniform_ptr(sg.W2);
    t.gate = uniform_ptr(sg.gate); t.sw = uniform_ptr(sg.sw); t.sw2 = uniform_ptr(sg.sw2); t.knw = uniform_ptr(sg.knw);
    return true;
}

// chunk swizzle: 16-byte chunk c of tile row r lives at chunk position c ^ swz(r)
__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }

__device__ __forceinline__ bf16x8 lds_frag(const char* tile, int row, int chunk) {
    return *reinterpret_cast<const bf16x8*>(tile + row * (BK * 2) + ((chunk ^ swz(row)) << 4));
}

#ifdef CDM_CROSSCHECK      // the two-stage pipeline on 32 x 32 MFMAs: main loop pieces
template <bool FP8>
__device__ __forceinline__ void compute_stage(const char* sa, const char* sb, f32x16 (&acc)[4][4], int wm, int wn,
                                              int lane) {
    const int r32 = lane & 31, kh = lane >> 5;
    if (!FP8) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {     // 4 x 16 bf16 = 64 elements = 128 bytes
            bf16x8 af[4], bfr[4];
#pragma unroll
            for (int mi = 0; mi < 4; ++mi) af[mi] = lds_frag(sa, wm * 128 + mi * 32 + r32, 2 * ks + kh);
#pragma unroll
            for (int ni = 0; ni < 4; ++ni) bfr[ni] = lds_frag(sb, wn * 128 + ni * 32 + r32, 2 * ks + kh);
#pragma unroll
            for (int mi = 0; mi < 4; ++mi)
#pragma unroll
                for (int ni = 0; ni < 4; ++ni)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[ni], af[mi], acc[mi][ni], 0, 0, 0);
        }
    } else {
        // 2 x 64 e4m3: a lane supplies 32 consecutive bytes of K (two 16-byte chunks).  The same
        // bytes go into the same operand slots for A and W, which is all the contraction needs.
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            i32x8 af[4], bfr[4];
#pragma unroll
            for (int mi = 0; mi < 4; ++mi) {
                const bf16x8 lo = lds_frag(sa, wm * 128 + mi * 32 + r32, 4 * ks + 2 * kh);
                const bf16x8 hi = lds_frag(sa, wm * 128 + mi * 32 + r32, 4 * ks + 2 * kh + 1);
                const int4 l4 = __builtin_bit_cast(int4, lo), h4 = __builtin_bit_cast(int4, hi);
                af[mi] = i32x8{l4.x, l4.y, l4.z, l4.w, h4.x, h4.y, h4.z, h4.w};
            }
#pragma unroll
            for (int ni = 0; ni < 4; ++ni) {
                const bf16x8 lo = lds_frag(sb, wn * 128 + ni * 32 + r32, 4 * ks + 2 * kh);
                const bf16x8 hi = lds_frag(sb, wn * 128 + ni * 32 + r32, 4 * ks + 2 * kh + 1);
                const int4 l4 = __builtin_bit_cast(int4, lo), h4 = __builtin_bit_cast(int4, hi);
                bfr[ni] = i32x8{l4.x, l4.y, l4.z, l4.w, h4.x, h4.y, h4.z, h4.w};
            }
#pragma unroll
            for (int mi = 0; mi < 4; ++mi)
#pragma unroll
                for (int ni = 0; ni < 4; ++ni)
                    acc[mi][ni] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                        bfr[ni], af[mi], acc[mi][ni], 0 /*A: e4m3*/, 0 /*B: e4m3*/, 0, 0x7f7f7f7f /*2^0*/, 0,
                        0x7f7f7f7f);
        }
    }
}

// 8 + 8 direct-to-LDS loads of one k-tile: uniform base pointer (SGPR pair) + per-lane 32-bit byte offset
__device__ __forceinline__ void issue_loads(const char* abase, const char* wbase, const char* w2base,
                                            const uint32_t (&oa)[8], const uint32_t (&ob)[8], uint32_t w2mask,
                                            char* sa, char* sb, int wave) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        __builtin_amdgcn_global_load_lds(abase + oa[i], (lds_void*)(sa + (i * 4 + wave) * 1024), 16, 0, 0);
        const char* wb = ((w2mask >> i) & 1u) ? w2base : wbase;   // wave-uniform choice
        __builtin_amdgcn_global_load_lds(wb + ob[i], (lds_void*)(sb + (i * 4 + wave) * 1024), 16, 0, 0);
    }
}

#endif

// silu(g) = g / (1 + e^-g) with the hardware reciprocal (1 ulp) instead of an IEEE division: the result is rounded to
// bf16 anyway, and a correctly rounded division is ten instructions per output value of a 128 x 64 result per wave
__device__ __forceinline__ float silu_f(float g) {
    return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g));
}

// ---- epilogue shared by both pipelines.
// The MFMAs are issued with the W fragment as the first operand, so an accumulator block holds C TRANSPOSED:
// element v of block (mi, ni) is output row (token) lane % 32 and output column 8 (v / 4) + 4 (lane / 32) + v % 4 of
// its 32x32 block.  A lane therefore owns ONE output row per mi and groups of FOUR consecutive columns, and every
// global access of the epilogue (C, residual, gate, scales, rotary tables) is an 8- or 16-byte vector access.
// N is a multiple of 8 (host-checked), so a group of four columns is either entirely inside or entirely outside.
__device__ __forceinline__ uint2 pack4_bf16(float a, float b, float c, float d) {
    return make_uint2(pack_bf16x2(a, b), pack_bf16x2(c, d));
}

constexpr int kStagePitch = 256 + 16;      // bytes per staged row (16-byte multiple; the pad spreads rows over banks)

// wave-private staging area -> C: COLS (128 or 64) columns of ESIZE bytes (2 = bf16, 4 = fp32) of ROWS rows, whole rows
// per store instruction
template <int COLS, int ESIZE = 2, int ROWS = 128>
__device__ __forceinline__ void copy_out(const GemmParams& p, const Tile& t, const char* stage, int row0, int col0, int lane) {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");      // the wave's own staging writes have landed
    constexpr int LPR = COLS * ESIZE / 16;       // lanes per row (16 bytes each)
    constexpr int RPI = 64 / LPR;                // rows per instruction
    const int rl = lane / LPR, ch = lane % LPR;
    const int col = col0 + ch * (16 / ESIZE);
#pragma unroll
    for (int it = 0; it < ROWS / RPI; ++it) {
        const int rloc = it * RPI + rl;
        const uint4 v = *reinterpret_cast<const uint4*>(stage + rloc * kStagePitch + ch * 16);
        const int row = row0 + rloc;
        // non-temporal: the output is not read again by this kernel, and a tile's 128 KB per CU (4 MB per XCD at a
        // time, the whole L2) would otherwise push the A / W slabs of the next tiles out of the cache
        if (row < t.m_end && col < p.N) {
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            const u32x4 vv = {v.x, v.y, v.z, v.w};
            __builtin_nontemporal_store(vv, reinterpret_cast<u32x4*>(reinterpret_cast<char*>(p.C) +
                                                                     ((int64_t)row * p.ldc + col) * ESIZE));
        }
    }
}

// Views of a wave's accumulators: where in the wave's ROWS x 128 piece of the tile a lane's quads (four consecutive
// columns of one row) sit.  RS row slots x CS column slots per lane; column slot cs + CS / 2 is 64 columns right of cs.
#ifdef CDM_CROSSCHECK
template <int MI>
struct Acc32 {      // MI x 4 blocks of 32 x 32 (v_mfma_*_32x32x*): lane = row % 32 + 32 kh, quads at columns 8 g + 4 kh
    f32x16 (&v)[MI][4];
    static constexpr int RS = MI, CS = 16, ROWS = 32 * MI;
    static __device__ __forceinline__ int row_local(int rs, int lane) { return rs * 32 + (lane & 31); }
    static __device__ __forceinline__ int col_local(int cs, int lane) { return (cs >> 2) * 32 + (cs & 3) * 8 + (lane >> 5) * 4; }
    __device__ __forceinline__ float get(int rs, int cs, int e) const { return v[rs][cs >> 2][4 * (cs & 3) + e]; }
    __device__ __forceinline__ void set(int rs, int cs, int e, float x) { v[rs][cs >> 2][4 * (cs & 3) + e] = x; }
};
#endif
template <int MI>
struct Acc16 {      // MI x 8 blocks of 16 x 16 (v_mfma_*_16x16x*): lane = row % 16 + 16 q, one quad per block at column 4 q
    f32x4 (&v)[MI][8];
    static constexpr int RS = MI, CS = 8, ROWS = 16 * MI;
    static __device__ __forceinline__ int row_local(int rs, int lane) { return rs * 16 + (lane & 15); }
    static __device__ __forceinline__ int col_local(int cs, int lane) { return cs * 16 + (lane >> 4) * 4; }
    __device__ __forceinline__ float get(int rs, int cs, int e) const { return v[rs][cs][e]; }
    __device__ __forceinline__ void set(int rs, int cs, int e, float x) { v[rs][cs][e] = x; }
};

// row0 = first row of the wave's piece of the tile; the piece covers tile columns wn * 128 .. + 127
template <int EPI, bool FP8, class ACC>
__device__ __forceinline__ void epilogue(const GemmParams& p, const Tile& t, ACC acc, int row0, int n0, int wn, int lane,
                                         char* stage) {
    // `stage` (optional): kStagePitch * ROWS bytes of LDS private to this wave.  The finished bf16 values then go
    // there first and leave as whole rows, 16 bytes per lane: a store instruction covers 4 (SWIGLU: 8) output rows of
    // 256 (128) contiguous bytes instead of 32 rows of 16 bytes.  All workgroups reach their epilogue at about the
    // same time, so the epilogue runs at the HBM write rate; partial-line stores (which left the L2 as several
    // writes per line when the row stride is a large power of two) made it up to four times longer.
    constexpr int RS = ACC::RS, CS = ACC::CS, ROWS = ACC::ROWS, HALF = CS / 2, QUARTER = CS / 4;
    if (EPI == CDM_EPI_SWIGLU) {
        const int colw = n0 + wn * 64;       // wave's 128 tile columns = [gate 64 | up 64] of output columns colw .. + 63
#pragma unroll
        for (int rs = 0; rs < RS; ++rs) {
            const int rl = ACC::row_local(rs, lane), row = row0 + rl;
            if (row >= t.m_end) continue;
            const float sr = FP8 ? p.sa[row] : 1.0f;
            bf16_t* crow = p.C + (int64_t)row * p.ldc;
            float amax = 0.0f;
#pragma unroll
            for (int cs = 0; cs < HALF; ++cs) {
                const int cl = ACC::col_local(cs, lane), col = colw + cl;
                if (col >= p.N) continue;
                float sg[4] = {1.f, 1.f, 1.f, 1.f}, su[4] = {1.f, 1.f, 1.f, 1.f};
                if (FP8) {
                    const float4 a = *reinterpret_cast<const float4*>(t.sw + col);
                    const float4 b = *reinterpret_cast<const float4*>(t.sw2 + col);
                    sg[0] = a.x * sr; sg[1] = a.y * sr; sg[2] = a.z * sr; sg[3] = a.w * sr;
                    su[0] = b.x * sr; su[1] = b.y * sr; su[2] = b.z * sr; su[3] = b.w * sr;
                }
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = silu_f(acc.get(rs, cs, e) * sg[e]) * (acc.get(rs, cs + HALF, e) * su[e]);
                const uint2 o2 = pack4_bf16(o[0], o[1], o[2], o[3]);
                if (stage) *reinterpret_cast<uint2*>(stage + rl * kStagePitch + cl * 2) = o2;
                else *reinterpret_cast<uint2*>(crow + col) = o2;
                amax = fmaxf(fmaxf(amax, fmaxf(fabsf(bf16lo(o2.x)), fabsf(bf16hi(o2.x)))), fmaxf(fabsf(bf16lo(o2.y)), fabsf(bf16hi(o2.y))));
            }
            if (p.row_amax != nullptr) {      // lanes r, r + 16, r + 32, r + 48 hold the row's 64 columns of this piece
                amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
                amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
                if ((lane >> 4) == 0 && colw < p.N) p.row_amax[(int64_t)row * p.amax_ld + (colw >> 6)] = amax;
            }
        }
        if (stage) copy_out<64, 2, ROWS>(p, t, stage, row0, colw, lane);
        return;
    }
    const int colw = n0 + wn * 128;
    if (EPI == CDM_EPI_GATE_RESIDUAL_F32) {
        // the residual stream in fp32: R and C are float rows (in place when they coincide).  The wave's result goes
        // through its staging area 64 columns (256 bytes per row) at a time.
        float* C = reinterpret_cast<float*>(p.C);
        const float* R = reinterpret_cast<const float*>(p.R);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int rs = 0; rs < RS; ++rs) {
                const int rl = ACC::row_local(rs, lane), row = row0 + rl;
                if (row >= t.m_end) continue;
                const float sr = FP8 ? p.sa[row] : 1.0f;
#pragma unroll
                for (int c = 0; c < HALF; ++c) {
                    const int cs = h * HALF + c;
                    const int cl = ACC::col_local(cs, lane), col = colw + cl;
                    if (col >= p.N) continue;
                    const float4 r4 = *reinterpret_cast<const float4*>(R + (int64_t)row * p.ldr + col);
                    float4 g4 = make_float4(1.f, 1.f, 1.f, 1.f);
                    if (t.gate) g4 = *reinterpret_cast<const float4*>(t.gate + col);
                    if (FP8) {
                        const float4 w4 = *reinterpret_cast<const float4*>(t.sw + col);
                        g4.x *= sr * w4.x; g4.y *= sr * w4.y; g4.z *= sr * w4.z; g4.w *= sr * w4.w;
                    }
                    const float4 o = make_float4(r4.x + g4.x * acc.get(rs, cs, 0), r4.y + g4.y * acc.get(rs, cs, 1),
                                                 r4.z + g4.z * acc.get(rs, cs, 2), r4.w + g4.w * acc.get(rs, cs, 3));
                    if (stage) *reinterpret_cast<float4*>(stage + rl * kStagePitch + (cl - 64 * h) * 4) = o;
                    else *reinterpret_cast<float4*>(C + (int64_t)row * p.ldc + col) = o;
                }
            }
            if (stage) copy_out<64, 4, ROWS>(p, t, stage, row0, colw + 64 * h, lane);
        }
        return;
    }
    // QKV_PACK: 0 = Q columns (plain output), 1 = K, 2 = V (wave-uniform: the wave's 128 columns are one head of 128
    // channels or two heads of 64, and d_q, d_kv are multiples of 128)
    const int region = EPI != CDM_EPI_QKV_PACK ? 0 : (colw < p.d_q ? 0 : (colw < p.d_q + p.d_kv ? 1 : 2));
    if (EPI == CDM_EPI_QKV_PACK && (colw >= p.N || (region != 0 && row0 >= t.m_end))) return;   // no such head / key tile
    const bool rope = (EPI == CDM_EPI_ROPE_QK && colw < p.rope_cols) ||   // wave-uniform: whole heads of Q or K
                      (EPI == CDM_EPI_QKV_PACK && region == 1 && p.cos != nullptr);
    const int half = p.head_dim >> 1;
    const bool hd64 = EPI == CDM_EPI_QKV_PACK && p.head_dim == 64;      // columns cs < CS/2 are one head, the others the next
    float ksq[2] = {0.0f, 0.0f};      // QKV_PACK, K: largest squared norm among the lane's rows (as stored, rounded to bf16), per head
#pragma unroll
    for (int rs = 0; rs < RS; ++rs) {
        const int rl = ACC::row_local(rs, lane), row = row0 + rl;
        if (row >= t.m_end) {
            if (EPI == CDM_EPI_QKV_PACK && region != 0) {      // padding keys of a ragged last tile are zero in the images
#pragma unroll
                for (int cs = 0; cs < CS; ++cs)
                    *reinterpret_cast<uint2*>(stage + rl * kStagePitch + ACC::col_local(cs, lane) * 2) = make_uint2(0u, 0u);
            }
            continue;
        }
        if (FP8) {      // rank-1 dequantisation scale on the fp32 accumulators
            const float sr = p.sa[row];
#pragma unroll
            for (int cs = 0; cs < CS; ++cs) {
                const int col = colw + ACC::col_local(cs, lane);
                const float4 w4 = col < p.N ? *reinterpret_cast<const float4*>(t.sw + col) : make_float4(0, 0, 0, 0);
                acc.set(rs, cs, 0, acc.get(rs, cs, 0) * (sr * w4.x));
                acc.set(rs, cs, 1, acc.get(rs, cs, 1) * (sr * w4.y));
                acc.set(rs, cs, 2, acc.get(rs, cs, 2) * (sr * w4.z));
                acc.set(rs, cs, 3, acc.get(rs, cs, 3) * (sr * w4.w));
            }
        }
        if (EPI == CDM_EPI_QKV_PACK && region == 1 && t.knw != nullptr) {
            // per-head RMSNorm of K on the fp32 accumulators, ahead of the rotation: the wave's 128 columns are one head,
            // a key's channels are spread over the four quarter-waves (lanes r, r + 16, r + 32, r + 48 share the row)
            float ss[2] = {0.0f, 0.0f};      // the two halves of the wave's columns
#pragma unroll
            for (int cs = 0; cs < CS; ++cs)
#pragma unroll
                for (int e = 0; e < 4; ++e) ss[cs / (CS / 2)] += acc.get(rs, cs, e) * acc.get(rs, cs, e);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                ss[h] += __shfl_xor(ss[h], 16, 64);
                ss[h] += __shfl_xor(ss[h], 32, 64);
            }
            const float rn2[2] = {hd64 ? rsqrtf(ss[0] * (1.0f / 64.0f) + p.k_eps) : rsqrtf((ss[0] + ss[1]) * (1.0f / 128.0f) + p.k_eps),
                                  hd64 ? rsqrtf(ss[1] * (1.0f / 64.0f) + p.k_eps) : rsqrtf((ss[0] + ss[1]) * (1.0f / 128.0f) + p.k_eps)};
#pragma unroll
            for (int cs = 0; cs < CS; ++cs) {
                const float rn = rn2[cs / (CS / 2)];
                const float4 w4 = *reinterpret_cast<const float4*>(t.knw + (ACC::col_local(cs, lane) & (p.head_dim - 1)));
                acc.set(rs, cs, 0, acc.get(rs, cs, 0) * (rn * w4.x));
                acc.set(rs, cs, 1, acc.get(rs, cs, 1) * (rn * w4.y));
                acc.set(rs, cs, 2, acc.get(rs, cs, 2) * (rn * w4.z));
                acc.set(rs, cs, 3, acc.get(rs, cs, 3) * (rn * w4.w));
            }
        }
        if ((EPI == CDM_EPI_ROPE_QK || EPI == CDM_EPI_QKV_PACK) && rope) {
            // rotate-half pairs (i, i + head_dim/2).  head_dim 128: the wave's columns are one head, column slots
            // (c, c + CS/2), pair index = the column of c; head_dim 64: two heads per wave, slots (lo, lo + CS/4)
            // with lo in the first half of either head, pair index = the column inside the head
            const float* cr = p.cos + (int64_t)row * half;
            const float* sr_ = p.sin + (int64_t)row * half;
#pragma unroll
            for (int c = 0; c < HALF; ++c) {
                const bool hd128 = p.head_dim == 128;
                const int lo128 = c, lo64 = (c / QUARTER) * HALF + (c % QUARTER);
                const int i = hd128 ? ACC::col_local(lo128, lane) : (ACC::col_local(lo64, lane) & 31);
                const float4 c4 = *reinterpret_cast<const float4*>(cr + i);
                const float4 s4 = *reinterpret_cast<const float4*>(sr_ + i);
                const float cc[4] = {c4.x, c4.y, c4.z, c4.w}, sn[4] = {s4.x, s4.y, s4.z, s4.w};
                if (hd128) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float x1 = acc.get(rs, lo128, e), x2 = acc.get(rs, lo128 + HALF, e);
                        acc.set(rs, lo128, e, x1 * cc[e] - x2 * sn[e]);
                        acc.set(rs, lo128 + HALF, e, x2 * cc[e] + x1 * sn[e]);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float x1 = acc.get(rs, lo64, e), x2 = acc.get(rs, lo64 + QUARTER, e);
                        acc.set(rs, lo64, e, x1 * cc[e] - x2 * sn[e]);
                        acc.set(rs, lo64 + QUARTER, e, x2 * cc[e] + x1 * sn[e]);
                    }
                }
            }
        }
        bf16_t* crow = p.C + (int64_t)row * p.ldc;
        const bf16_t* rrow = EPI == CDM_EPI_GATE_RESIDUAL ? p.R + (int64_t)row * p.ldr : nullptr;
        float rsq[2] = {0.0f, 0.0f};
#pragma unroll
        for (int cs = 0; cs < CS; ++cs) {
            const int cl = ACC::col_local(cs, lane), col = colw + cl;
            if (col >= p.N) continue;
            float o[4] = {acc.get(rs, cs, 0), acc.get(rs, cs, 1), acc.get(rs, cs, 2), acc.get(rs, cs, 3)};
            if (EPI == CDM_EPI_GATE_RESIDUAL) {
                const uint2 r2 = *reinterpret_cast<const uint2*>(rrow + col);
                float4 g4 = make_float4(1.f, 1.f, 1.f, 1.f);
                if (t.gate) g4 = *reinterpret_cast<const float4*>(t.gate + col);
                o[0] = bf16lo(r2.x) + g4.x * o[0];
                o[1] = bf16hi(r2.x) + g4.y * o[1];
                o[2] = bf16lo(r2.y) + g4.z * o[2];
                o[3] = bf16hi(r2.y) + g4.w * o[3];
            }
            const uint2 o2 = pack4_bf16(o[0], o[1], o[2], o[3]);
            if (stage) *reinterpret_cast<uint2*>(stage + rl * kStagePitch + cl * 2) = o2;
            else *reinterpret_cast<uint2*>(crow + col) = o2;
            if (EPI == CDM_EPI_QKV_PACK && region == 1) {
                const float a = bf16lo(o2.x), b = bf16hi(o2.x), c = bf16lo(o2.y), d = bf16hi(o2.y);
                rsq[cs / (CS / 2)] += a * a + b * b + c * c + d * d;
            }
        }
        if (EPI == CDM_EPI_QKV_PACK && region == 1) {      // the row's channels are spread over the four quarter-waves
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                rsq[h] += __shfl_xor(rsq[h], 16, 64);
                rsq[h] += __shfl_xor(rsq[h], 32, 64);
            }
            if (hd64) { ksq[0] = fmaxf(ksq[0], rsq[0]); ksq[1] = fmaxf(ksq[1], rsq[1]); }
            else ksq[0] = fmaxf(ksq[0], rsq[0] + rsq[1]);
        }
    }
    if (EPI == CDM_EPI_QKV_PACK && region != 0) {
        // the wave's 64 x 128 piece is one (64-key tile, head) image, or two of heads with 64 channels; staged row r = key r
        // of the tile
        static_assert(EPI != CDM_EPI_QKV_PACK || (ROWS == 64 && CS == 8), "QKV_PACK needs the 64 x 128 wave piece");
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");      // the wave's own staging writes have landed
        const int key_tile = row0 >> 6;
        if (hd64) {
            const int head0 = (colw - (region == 1 ? p.d_q : p.d_q + p.d_kv)) >> 6;
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int64_t tile_at = (int64_t)(head0 + hh) * p.n_key_tiles + key_tile;
                if (region == 1) {      // K image, chunk-major [8 chunks of 8 channels][64 keys][16 bytes]
                    char* dst = p.kp + tile_at * (64 * 64 * 2);
#pragma unroll
                    for (int c = 0; c < 8; ++c)
                        *reinterpret_cast<uint4*>(dst + (c * 64 + lane) * 16) =
                            *reinterpret_cast<const uint4*>(stage + lane * kStagePitch + (8 * hh + c) * 16);
                    float kq = ksq[hh];
#pragma unroll
                    for (int off = 1; off < 16; off <<= 1) kq = fmaxf(kq, __shfl_xor(kq, off, 64));
                    if (lane == 0) p.kmax[tile_at] = sqrtf(kq);
                } else {                // V^T image [8 chunks][64 channel rows][8 keys], keys of a chunk as below
                    char* dst = p.vp + tile_at * (64 * 64 * 2);
#pragma unroll
                    for (int c = 0; c < 8; ++c) {
                        uint32_t w[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int key = 32 * (c >> 2) + 4 * (c & 3) + 16 * (e >> 1) + 2 * (e & 1);
                            const uint32_t lo = *reinterpret_cast<const uint16_t*>(stage + key * kStagePitch + (64 * hh + lane) * 2);
                            const uint32_t hi = *reinterpret_cast<const uint16_t*>(stage + (key + 1) * kStagePitch + (64 * hh + lane) * 2);
                            w[e] = lo | (hi << 16);
                        }
                        *reinterpret_cast<uint4*>(dst + (c * 64 + lane) * 16) = make_uint4(w[0], w[1], w[2], w[3]);
                    }
                }
            }
            return;
        }
        const int head = (colw - (region == 1 ? p.d_q : p.d_q + p.d_kv)) >> 7;
        const int64_t img = ((int64_t)head * p.n_key_tiles + key_tile) * (64 * 128 * 2);
        if (region == 1) {
            // K image, chunk-major [16 chunks of 8 channels][64 keys][16 bytes]
            char* dst = p.kp + img;
#pragma unroll
            for (int c = 0; c < 16; ++c)
                *reinterpret_cast<uint4*>(dst + (c * 64 + lane) * 16) =
                    *reinterpret_cast<const uint4*>(stage + lane * kStagePitch + c * 16);
            float kq = ksq[0];
#pragma unroll
            for (int off = 1; off < 16; off <<= 1) kq = fmaxf(kq, __shfl_xor(kq, off, 64));
            if (lane == 0) p.kmax[(int64_t)head * p.n_key_tiles + key_tile] = sqrtf(kq);
        } else {
            // V^T image [8 chunks][128 channel rows][8 keys]; chunk c = 4 s + g lists keys 32 s + 4 g + {0..3} and
            // 32 s + 16 + 4 g + {0..3} (the order in which a lane of the attention kernel holds its probabilities)
            char* dst = p.vp + img;
#pragma unroll
            for (int it = 0; it < 16; ++it) {
                const int c = it >> 1, h = (it & 1) * 64 + lane;
                uint32_t w[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int key = 32 * (c >> 2) + 4 * (c & 3) + 16 * (e >> 1) + 2 * (e & 1);
                    const uint32_t lo = *reinterpret_cast<const uint16_t*>(stage + key * kStagePitch + h * 2);
                    const uint32_t hi = *reinterpret_cast<const uint16_t*>(stage + (key + 1) * kStagePitch + h * 2);
                    w[e] = lo | (hi << 16);
                }
                *reinterpret_cast<uint4*>(dst + (c * 128 + h) * 16) = make_uint4(w[0], w[1], w[2], w[3]);
            }
        }
        return;
    }
    if (stage) copy_out<128, 2, ROWS>(p, t, stage, row0, colw, lane);
}

#ifdef CDM_CROSSCHECK
template <int EPI, bool FP8>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(1024))) char sa0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) char sb0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) char sa1[kTileBytes];
    __shared__ __attribute__((aligned(1024))) char sb1[kTileBytes];

    Tile tile;
    if (!locate_tile(p, tile)) return;
    const int tn = tile.tn;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = tile.m0;
    const int n0 = (EPI == CDM_EPI_SWIGLU) ? tn * (BN / 2) : tn * BN;

    // ---- per-lane byte offsets (relative to the tile's first row) of the 8 + 8 loads of one k-tile
    uint32_t oa[8], ob[8];
    uint32_t w2mask = 0;     // bit i set: load i of this wave reads W2 (up_proj rows of a SWIGLU tile)
    int nb0 = n0;            // first W row of the tile
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int row = (i * 4 + wave) * 8 + (lane >> 3);   // tile row this lane feeds
        const int chunk = (lane & 7) ^ swz(row);            // source chunk that belongs at position lane&7
        int am = row;
        am = (m0 + am) < tile.m_end ? am : tile.m_end - 1 - m0;
        oa[i] = (uint32_t)(am * (int)p.lda + chunk * 16);
        int bn;
        if (EPI == CDM_EPI_SWIGLU) {
            // 64-row groups of the tile alternate gate / up: [g 0-63 | u 0-63 | g 64-127 | u 64-127]
            const int grp = ((i * 4 + wave) * 8) >> 6;       // wave-uniform
            if (grp & 1) w2mask |= 1u << i;
            bn = (grp >> 1) * 64 + (row & 63);
        } else {
            bn = row;
        }
        bn = (nb0 + bn) < p.N ? bn : p.N - 1 - nb0;
        ob[i] = (uint32_t)(bn * (int)p.ldw + chunk * 16);
    }
    const char* abase = reinterpret_cast<const char*>(p.A) + (int64_t)m0 * p.lda;
    const char* wbase = reinterpret_cast<const char*>(tile.W) + (int64_t)nb0 * p.ldw;
    const char* w2base = EPI == CDM_EPI_SWIGLU ? reinterpret_cast<const char*>(tile.W2) + (int64_t)nb0 * p.ldw : wbase;

    f32x16 acc[4][4];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 4; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;

    const int KT = p.K / (FP8 ? 128 : 64);   // k-tiles of 128 bytes; the host guarantees an even count
    issue_loads(abase, wbase, w2base, oa, ob, w2mask, sa0, sb0, wave);
    for (int kt = 0; kt < KT; kt += 2) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        issue_loads(abase + (kt + 1) * 128, wbase + (kt + 1) * 128, w2base + (kt + 1) * 128, oa, ob, w2mask, sa1, sb1,
                    wave);
        __builtin_amdgcn_sched_barrier(0);      // keep the prefetch at the top of the stage
        compute_stage<FP8>(sa0, sb0, acc, wm, wn, lane);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (kt + 2 < KT)
            issue_loads(abase + (kt + 2) * 128, wbase + (kt + 2) * 128, w2base + (kt + 2) * 128, oa, ob, w2mask, sa0,
                        sb0, wave);
        __builtin_amdgcn_sched_barrier(0);
        compute_stage<FP8>(sa1, sb1, acc, wm, wn, lane);
    }

    epilogue<EPI, FP8>(p, tile, Acc32<4>{acc}, m0 + wm * 128, n0, wn, lane, nullptr);
}
#endif

// ---------------------------------------------------------------------------------------------
// Ring pipeline (default): 256 x 256 tile, EIGHT waves (two per SIMD), 16 x 16 MFMAs, 128-byte tile rows (k-tiles of
// 64 bf16 / 128 e4m3 elements) and a five-slot ring of single-operand granules; a wave owns 64 x 128 of the tile as
// 4 x 8 accumulator blocks of 16 x 16 (128 registers).
//  * A direct-to-LDS load instruction that covers 8 rows x 128 bytes (whole cache lines) costs the vector L1 about
//    40 % less time per byte than one that covers 16 rows x 64 bytes, and with 256x256 tiles the L1 path is what
//    the pipeline competes for.  160 KB of LDS hold five 32 KB granules (256 rows x 128 B of A or of W): granule
//    g = 2t + (0: A, 1: W) of k-tile t lives in slot g % 5, so two slots are being read and three are landing.
//  * v_mfma_f32_16x16x32_bf16 moves a fifth fewer register bytes per flop than 32x32x16 (half the accumulator traffic,
//    twice the operand traffic) and the chip runs into its power limit, not its issue rate, on random operands: a loop of
//    nothing but MFMAs sustains 9 % more with the small shape, and this kernel 6 - 11 % more than a 32 x 32 twin.
//  * The second wave of a SIMD feeds the matrix pipe while the first sits in the vector-memory issue queue with a
//    direct-to-LDS load, or in the latencies of its epilogue.
//  * k-step = 32 MFMAs, order: W block ni outer, A block mi inner.  The four A fragments of the NEXT k-step are read under
//    MFMAs 18 - 30 (two register sets), the W fragments stream through a four-entry window three blocks ahead, so a k-step
//    reads 12 fragments for 32 MFMAs.  bf16: two k-steps per k-tile (K 32 each); e4m3: one (K 128).
//  * The window makes the reads of k-tile t reach into its last k-step (until MFMA 16), so the wait + barrier ("every wave
//    has finished reading tile t, and tile t+1 has landed") sits at MFMA 18 of it; it releases the two slots of tile t.
//    The fragments of tile t+1 that the next k-step starts with are read right behind it.  A(t+2) goes out ahead of the
//    barrier, into the slot that W(t-1) left at the previous barrier; W(t+2) behind it, one load every other MFMA, into
//    the slot of A(t).
//  * The instruction order inside a k-step is pinned with scheduling fences, one per MFMA: a wave that issues its loads
//    back to back sits in the vector-memory issue queue for hundreds of cycles; one load per few MFMAs is covered by
//    MFMAs already queued.
//  * The slot numbers live in scalar registers and rotate by renaming.  (A loop unrolled over the five-stage period
//    needs mid-loop exits, and the spill reloads the compiler then places at the loop head wait with vmcnt(0), which
//    drains every direct-to-LDS load in flight.)
// Chunk swizzle of a 128-byte ring row: a fragment read covers 16 rows x 4 chunks (lane = row % 16 + 16 x chunk), and
// the LDS serves 16 lanes of a 16-byte-per-lane read per pass; (row / 2) % 8 puts the 16 rows of one chunk column on the
// 16 distinct 16-byte slots of the 256-byte bank window.  A function of row % 16 only, so that the fragment address of
// row block mi is the lane's address plus a constant.
// ---------------------------------------------------------------------------------------------
constexpr int kGranule = BM * 128;      // 32 KB
__device__ __forceinline__ int swz16(int row) { return (row >> 1) & 7; }

template <int EPI, bool FP8>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_ring_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(1024))) char s_ring[5 * kGranule];

    Tile tile;
    if (!locate_tile(p, tile)) return;
    const int tn = tile.tn;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave >> 1, wn = wave & 1;          // 4 x 2 waves of 64 x 128
    const int m0 = tile.m0;
    const int n0 = (EPI == CDM_EPI_SWIGLU) ? tn * (BN / 2) : tn * BN;

    // per-lane byte offsets of the wave's 4 + 4 loads of one k-tile: load j covers tile rows (8 j + wave) * 8 .. + 7
    uint32_t oa[4], ob[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = (j * 8 + wave) * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ swz16(row);
        int am = row;
        am = (m0 + am) < tile.m_end ? am : tile.m_end - 1 - m0;
        oa[j] = (uint32_t)(am * (int)p.lda + chunk * 16);
        // SWIGLU: tile rows come in 64-row groups [gate | up | gate | up]; the rows of load j lie in group j
        int bn = (EPI == CDM_EPI_SWIGLU) ? (j >> 1) * 64 + (row & 63) : row;
        bn = (n0 + bn) < p.N ? bn : p.N - 1 - n0;
        ob[j] = (uint32_t)(bn * (int)p.ldw + chunk * 16);
    }
    const char* abase = reinterpret_cast<const char*>(p.A) + (int64_t)m0 * p.lda;
    const char* wbase = reinterpret_cast<const char*>(tile.W) + (int64_t)n0 * p.ldw;
    const char* w2base = EPI == CDM_EPI_SWIGLU ? reinterpret_cast<const char*>(tile.W2) + (int64_t)n0 * p.ldw : wbase;
    const uint32_t l0 = lds_addr_of(s_ring) + wave * 1024;

    f32x4 acc[4][8];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 8; ++ni) acc[mi][ni] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int KT = p.K / (FP8 ? 128 : 64);   // k-tiles of 128 bytes (at least 2, host-checked)
    auto gload = [&](int t, int op, int slot, int j) {
        const int ko = (t < KT ? t : KT - 1) * 128;
        if (op == 0) {
            lds_dma16(abase + ko, oa[j], l0 + slot * kGranule + j * 8192);
        } else {
            const char* wb = (EPI == CDM_EPI_SWIGLU && (j & 1)) ? w2base : wbase;
            lds_dma16(wb + ko, ob[j], l0 + slot * kGranule + j * 8192);
        }
    };
    using T = typename std::conditional<FP8, i32x8, bf16x8>::type;
    constexpr int KS = FP8 ? 1 : 2;
    const int r16 = lane & 15, q = lane >> 4;
    uint32_t fa[KS], fb[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        // bf16: 16-byte chunk 4 ks + q of the row; e4m3: chunks 2 q and 2 q + 1 (the second at the address ^ 16)
        const int chunk = FP8 ? 2 * q : 4 * ks + q;
        const uint32_t in_row = (uint32_t)(r16 * 128 + ((chunk ^ swz16(r16)) << 4));
        fa[ks] = in_row + wm * 8192;
        fb[ks] = in_row + wn * 16384;
    }
    auto rd = [&](uint32_t off) {
        if constexpr (FP8) {
            const int4 lo = *reinterpret_cast<const int4*>(s_ring + off);
            const int4 hi = *reinterpret_cast<const int4*>(s_ring + (off ^ 16));
            return i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        } else {
            return *reinterpret_cast<const bf16x8*>(s_ring + off);
        }
    };
    auto afrag = [&](int slot, int ks, int mi) { return rd(fa[ks] + slot * kGranule + mi * 2048); };
    auto bfrag = [&](int slot, int ks, int ni) { return rd(fb[ks] + slot * kGranule + ni * 2048); };

    // prologue: granules 0..3 (tiles 0 and 1)
#pragma unroll
    for (int j = 0; j < 4; ++j) gload(0, 0, 0, j);
#pragma unroll
    for (int j = 0; j < 4; ++j) gload(0, 1, 1, j);
#pragma unroll
    for (int j = 0; j < 4; ++j) gload(1, 0, 2, j);
#pragma unroll
    for (int j = 0; j < 4; ++j) gload(1, 1, 3, j);
    asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");     // tile 0 has landed everywhere
    T X[4], Y[4], B[4];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) X[mi] = afrag(0, 0, mi);
    B[0] = bfrag(1, 0, 0);
    B[1] = bfrag(1, 0, 1);
    B[2] = bfrag(1, 0, 2);

    int sa = 0, sb = 1, na = 2, nb = 3, f2 = 4;
    int t = 0;
    // LAST = the k-step that ends k-tile t (the only one of an e4m3 tile, the second of a bf16 tile)
    auto kstep = [&](auto last_c, T (&cur)[4], T (&nxt)[4]) {
        constexpr bool LAST = decltype(last_c)::value;
        constexpr int ks = LAST ? KS - 1 : 0;           // k-step of the W fragments in flight
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const int ni = i >> 2, mi = i & 3;
            if constexpr (FP8)
                // literal zero scale operands select the unscaled instruction (v_mfma_f32_16x16x128_f8f6f4: block scale 1,
                // no scale-load prefix in front of every MFMA)
                acc[mi][ni] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(B[ni & 3], cur[mi], acc[mi][ni], 0 /*A: e4m3*/,
                                                                               0 /*B: e4m3*/, 0, 0, 0, 0);
            else
                acc[mi][ni] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(B[ni & 3], cur[mi], acc[mi][ni], 0, 0, 0);
            if (!LAST) {
                if (mi == 0) B[(ni + 3) & 3] = ni < 5 ? bfrag(sb, 0, ni + 3) : bfrag(sb, 1, ni - 5);
                if (i >= 18 && (i & 3) == 2) nxt[(i - 18) >> 2] = afrag(sa, 1, (i - 18) >> 2);
                if (i == 9) gload(t + 2, 0, f2, 0);
                if (i == 25) gload(t + 2, 0, f2, 1);
            } else {
                if (mi == 0 && ni < 5) B[(ni + 3) & 3] = bfrag(sb, ks, ni + 3);
                if constexpr (FP8) {
                    if (i == 3) gload(t + 2, 0, f2, 0);
                    if (i == 7) gload(t + 2, 0, f2, 1);
                    if (i == 11) gload(t + 2, 0, f2, 2);
                    if (i == 15) gload(t + 2, 0, f2, 3);
                } else {
                    if (i == 5) gload(t + 2, 0, f2, 2);
                    if (i == 13) gload(t + 2, 0, f2, 3);
                }
                if (i == 18) {
                    asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    __builtin_amdgcn_sched_barrier(0);
                    nxt[0] = afrag(na, 0, 0);
                }
                if (i == 19) nxt[1] = afrag(na, 0, 1);
                if (i == 20) B[0] = bfrag(nb, 0, 0);
                if (i == 21) nxt[2] = afrag(na, 0, 2);
                if (i == 22) nxt[3] = afrag(na, 0, 3);
                if (i == 23) gload(t + 2, 1, sa, 0);
                if (i == 24) B[1] = bfrag(nb, 0, 1);
                if (i == 25) gload(t + 2, 1, sa, 1);
                if (i == 27) gload(t + 2, 1, sa, 2);
                if (i == 28) B[2] = bfrag(nb, 0, 2);
                if (i == 29) gload(t + 2, 1, sa, 3);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto rotate = [&]() {
        const int o_sa = sa, o_sb = sb;
        sa = na; sb = nb; na = f2; nb = o_sa; f2 = o_sb;
        ++t;
    };
    if constexpr (FP8) {
        while (t < KT) {
            kstep(std::true_type{}, X, Y);
            rotate();
            if (t < KT) {
                kstep(std::true_type{}, Y, X);
                rotate();
            }
        }
    } else {
        while (t < KT) {
            kstep(std::false_type{}, X, Y);
            kstep(std::true_type{}, Y, X);
            rotate();
        }
    }
    // surplus loads must not outlive the workgroup's LDS; after the barrier no wave reads the ring any more and
    // each wave owns an eighth of it as the staging area of its epilogue
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    epilogue<EPI, FP8>(p, tile, Acc16<4>{acc}, m0 + wm * 64, n0, wn, lane, s_ring + wave * (64 * kStagePitch));
}

// esize = bytes per operand element (2 = bf16, 1 = e4m3); strides in elements
int32_t validate(const char* who, int esize, const void* A, int64_t lda, const void* W, int64_t ldw, const void* W2,
                 void* C, int64_t ldc, int64_t M, int64_t N, int64_t K, int32_t epi, const void* R, int64_t ldr,
                 const float* cos, const float* sin, int64_t rope_cols, int32_t head_dim) {
    const int64_t kmult = 256 / esize;      // two 128-byte k-tiles
    CDM_REQUIRE(A && W && C, CDM_ERR_BAD_ARG, "%s: null pointer", who);
    CDM_REQUIRE(M >= 0 && N > 0 && K > 0, CDM_ERR_BAD_ARG, "%s: bad sizes M=%lld N=%lld K=%lld", who, (long long)M,
                (long long)N, (long long)K);
    CDM_REQUIRE(epi >= CDM_EPI_NONE && epi <= CDM_EPI_QKV_PACK, CDM_ERR_BAD_ARG, "%s: unknown epilogue %d", who, epi);
    CDM_REQUIRE(K % kmult == 0, CDM_ERR_BAD_SHAPE, "%s: K=%lld must be a multiple of %lld", who, (long long)K,
                (long long)kmult);
    CDM_REQUIRE(N % 8 == 0, CDM_ERR_BAD_SHAPE, "%s: N=%lld must be a multiple of 8", who, (long long)N);
    CDM_REQUIRE(M < (1ll << 31) - 512 && N < (1ll << 31) - 512 && K < (1ll << 24) && lda < (1ll << 22) &&
                    ldw < (1ll << 22),
                CDM_ERR_BAD_SHAPE, "%s: sizes out of range", who);
    // QKV_PACK writes only its first rope_cols (= Q) columns to C
    CDM_REQUIRE(lda >= K && ldw >= K && ldc >= (epi == CDM_EPI_QKV_PACK ? rope_cols : N), CDM_ERR_BAD_ARG,
                "%s: row stride smaller than row length", who);
    CDM_REQUIRE(cdm_aligned16(A) && cdm_aligned16(W) && cdm_aligned16(C) && (lda * esize) % 16 == 0 &&
                    (ldw * esize) % 16 == 0,
                CDM_ERR_BAD_ALIGN, "%s: pointers/strides must be 16-byte aligned", who);
    CDM_REQUIRE(ldc % 8 == 0, CDM_ERR_BAD_ALIGN, "%s: ldc=%lld must be a multiple of 8 elements", who, (long long)ldc);
    if (epi == CDM_EPI_SWIGLU)
        CDM_REQUIRE(W2 && cdm_aligned16(W2), CDM_ERR_BAD_ARG, "%s: SWIGLU needs an aligned W2 (up_proj)", who);
    if (epi == CDM_EPI_GATE_RESIDUAL || epi == CDM_EPI_GATE_RESIDUAL_F32)
    {
        CDM_REQUIRE(R && ldr >= N, CDM_ERR_BAD_ARG, "%s: GATE_RESIDUAL needs R with ldr >= N", who);
        CDM_REQUIRE(cdm_aligned16(R) && ldr % 8 == 0, CDM_ERR_BAD_ALIGN,
                    "%s: residual pointer / row stride must be 16-byte aligned", who);
    }
    if (epi == CDM_EPI_ROPE_QK) {
        CDM_REQUIRE(cos && sin, CDM_ERR_BAD_ARG, "%s: ROPE_QK needs cos/sin tables", who);
        CDM_REQUIRE(cdm_aligned16(cos) && cdm_aligned16(sin), CDM_ERR_BAD_ALIGN, "%s: cos/sin must be 16-byte aligned", who);
        CDM_REQUIRE(head_dim == 64 || head_dim == 128, CDM_ERR_BAD_SHAPE, "%s: head_dim=%d must be 64 or 128", who,
                    head_dim);
        CDM_REQUIRE(rope_cols >= 0 && rope_cols <= N && rope_cols % 256 == 0, CDM_ERR_BAD_SHAPE,
                    "%s: rope_cols=%lld must be a multiple of 256 within N", who, (long long)rope_cols);
    }
    return CDM_OK;
}

// host-side description of one row segment of a (grouped) GEMM
struct HostSeg {
    int64_t start, len;
    const void* W; const void* W2;
    const float* gate; const float* sw; const float* sw2; const float* knw;
};

// Launches the segments kMaxSeg at a time (one grid per batch).  p holds everything that is common to the segments.
template <bool FP8>
int32_t run(GemmParams p, const HostSeg* segs, int n_seg, int64_t N, int32_t epilogue, hipStream_t st, const char* who) {
    const int tile_n = epilogue == CDM_EPI_SWIGLU ? BN / 2 : BN;
    p.tiles_n = (int)((N + tile_n - 1) / tile_n);
    // variant 0 = ring pipeline with eight waves and 16 x 16 MFMAs; 1 (cross-check build only) = two-stage pipeline, four
    // waves, 32 x 32 MFMAs
    const bool ring = cdm_get_variant(1) != 1;
    (void)ring;
    int i = 0;
    while (i < n_seg) {
        int ns = 0, total = 0;
        for (; i < n_seg && ns < kMaxSeg; ++i) {
            if (segs[i].len == 0) continue;
            GemmSeg& g = p.seg[ns++];
            g.m_start = (int)segs[i].start; g.m_end = (int)(segs[i].start + segs[i].len);
            g.tiles_m = (int)((segs[i].len + BM - 1) / BM);
            total += g.tiles_m * p.tiles_n;
            g.tile_end = total;
            g.W = segs[i].W; g.W2 = segs[i].W2; g.gate = segs[i].gate; g.sw = segs[i].sw; g.sw2 = segs[i].sw2;
            g.knw = segs[i].knw;
        }
        if (ns == 0) break;
        p.n_seg = ns; p.total_tiles = total;
        const int grid = ((total + 7) / 8) * 8;
#ifdef CDM_CROSSCHECK
#define CDM_LAUNCH(E)                                                         \
    if (ring) gemm_ring_kernel<E, FP8><<<grid, 512, 0, st>>>(p);            \
    else gemm_kernel<E, FP8><<<grid, kThreads, 0, st>>>(p)
#else
#define CDM_LAUNCH(E) gemm_ring_kernel<E, FP8><<<grid, 512, 0, st>>>(p)
#endif
        switch (epilogue) {
            case CDM_EPI_NONE: CDM_LAUNCH(CDM_EPI_NONE); break;
            case CDM_EPI_SWIGLU: CDM_LAUNCH(CDM_EPI_SWIGLU); break;
            case CDM_EPI_GATE_RESIDUAL: CDM_LAUNCH(CDM_EPI_GATE_RESIDUAL); break;
            case CDM_EPI_GATE_RESIDUAL_F32: CDM_LAUNCH(CDM_EPI_GATE_RESIDUAL_F32); break;
            case CDM_EPI_QKV_PACK: gemm_ring_kernel<CDM_EPI_QKV_PACK, FP8><<<grid, 512, 0, st>>>(p); break;   // ring only
            default: CDM_LAUNCH(CDM_EPI_ROPE_QK); break;
        }
#undef CDM_LAUNCH
        int32_t rc = cdm_check_launch(who);
        if (rc) return rc;
    }
    return CDM_OK;
}

// validates every segment of a grouped call (before anything is enqueued) and fills the host segment list
template <bool FP8>
int32_t grouped(const char* who, const void* A, int64_t lda, const float* sa, const void* const* W, const float* const* sw,
                int64_t ldw, const void* const* W2, const float* const* sw2, void* C, int64_t ldc,
                const int64_t* seg_start, const int64_t* seg_len, int32_t n_seg, int64_t N, int64_t K, int32_t epilogue,
                const void* R, int64_t ldr, const float* const* gate, const float* cos, const float* sin,
                int64_t rope_cols, int32_t head_dim, void* stream, const GemmParams* pack = nullptr,
                const float* k_norm_rows = nullptr, float* row_amax = nullptr, int64_t amax_ld = 0) {
    constexpr int esize = FP8 ? 1 : 2;
    CDM_REQUIRE(A && W && C && seg_start && seg_len, CDM_ERR_BAD_ARG, "%s: null pointer", who);
    CDM_REQUIRE((epilogue == CDM_EPI_QKV_PACK) == (pack != nullptr), CDM_ERR_BAD_ARG,
                "%s: the QKV_PACK epilogue belongs to the qkv_pack entry points", who);
    CDM_REQUIRE(n_seg >= 0 && n_seg <= 64, CDM_ERR_BAD_ARG, "%s: n_seg=%d out of range", who, n_seg);
    if (epilogue == CDM_EPI_SWIGLU) CDM_REQUIRE(W2, CDM_ERR_BAD_ARG, "%s: SWIGLU needs W2", who);
    if (row_amax != nullptr) {
        CDM_REQUIRE(epilogue == CDM_EPI_SWIGLU, CDM_ERR_BAD_ARG, "%s: row_amax belongs to the SWIGLU epilogue", who);
        CDM_REQUIRE((reinterpret_cast<uintptr_t>(row_amax) & 3u) == 0 && amax_ld >= (N + 63) / 64, CDM_ERR_BAD_ARG,
                    "%s: row_amax must be 4-byte aligned with a row stride of at least ceil(N / 64)", who);
    }
    if (FP8) {
        CDM_REQUIRE(sa && sw, CDM_ERR_BAD_ARG, "%s: null scale pointer", who);
        if (epilogue == CDM_EPI_SWIGLU) CDM_REQUIRE(sw2, CDM_ERR_BAD_ARG, "%s: SWIGLU needs sw2", who);
    }
    HostSeg segs[64];
    int64_t max_end = 0;
    for (int g = 0; g < n_seg; ++g) {
        CDM_REQUIRE(seg_start[g] >= 0 && seg_len[g] >= 0, CDM_ERR_BAD_ARG, "%s: negative segment", who);
        CDM_REQUIRE(W[g], CDM_ERR_BAD_ARG, "%s: null weight for segment %d", who, g);
        int32_t rc = validate(who, esize, A, lda, W[g], ldw, W2 ? W2[g] : nullptr, C, ldc, seg_len[g], N, K, epilogue, R, ldr,
                              cos, sin, rope_cols, head_dim);
        if (rc) return rc;
        const float* gt = gate ? gate[g] : nullptr;
        CDM_REQUIRE(cdm_aligned16(gt), CDM_ERR_BAD_ALIGN, "%s: gate of segment %d must be 16-byte aligned", who, g);
        if (FP8) {
            CDM_REQUIRE(sw[g] && cdm_aligned16(sw[g]) && (epilogue != CDM_EPI_SWIGLU || (sw2[g] && cdm_aligned16(sw2[g]))),
                        CDM_ERR_BAD_ARG, "%s: weight scales of segment %d null or misaligned", who, g);
        }
        for (int h = 0; h < g; ++h)
            CDM_REQUIRE(seg_start[g] >= segs[h].start + segs[h].len || seg_start[g] + seg_len[g] <= segs[h].start,
                        CDM_ERR_BAD_ARG, "%s: segments %d and %d overlap", who, h, g);
        segs[g] = HostSeg{seg_start[g], seg_len[g], W[g], W2 ? W2[g] : nullptr, gt, FP8 ? sw[g] : nullptr,
                          (FP8 && sw2) ? sw2[g] : nullptr, k_norm_rows ? k_norm_rows + (int64_t)g * head_dim : nullptr};
        if (seg_start[g] + seg_len[g] > max_end) max_end = seg_start[g] + seg_len[g];
    }
    CDM_REQUIRE(max_end < (1ll << 31) - 512, CDM_ERR_BAD_SHAPE, "%s: sizes out of range", who);
    if (max_end == 0) return CDM_OK;
    int32_t rc = cdm_require_device();
    if (rc) return rc;
    GemmParams p{};
    p.A = A; p.lda = lda * esize; p.ldw = ldw * esize; p.sa = sa;
    p.C = (bf16_t*)C; p.ldc = ldc;
    p.N = (int)N; p.K = (int)K;
    p.R = (const bf16_t*)R; p.ldr = ldr;
    p.cos = cos; p.sin = sin; p.rope_cols = (int)rope_cols; p.head_dim = head_dim;
    p.row_amax = row_amax; p.amax_ld = amax_ld;
    if (pack) {
        p.kp = pack->kp; p.vp = pack->vp; p.kmax = pack->kmax;
        p.d_q = pack->d_q; p.d_kv = pack->d_kv; p.n_key_tiles = pack->n_key_tiles; p.k_eps = pack->k_eps;
    }
    return run<FP8>(p, segs, n_seg, N, epilogue, (hipStream_t)stream, who);
}

// QKV projection whose K and V columns leave as the attention kernel's tile images (see the header for the contract)
template <bool FP8>
int32_t qkv_pack(const char* who, const void* A, int64_t lda, const float* sa, const void* const* W, const float* const* sw,
                 int64_t ldw, void* Q, int64_t ldq, const int64_t* seg_start, const int64_t* seg_len, int32_t n_seg,
                 int64_t K, int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, const float* cos, const float* sin,
                 const cdm_qk_norm* qk_norm, void* workspace, int64_t workspace_bytes, void* stream) {
    CDM_REQUIRE(seg_start && seg_len && workspace, CDM_ERR_BAD_ARG, "%s: null pointer", who);
    CDM_REQUIRE(head_dim == 128 || head_dim == 64, CDM_ERR_UNSUPPORTED, "%s: head_dim=%d (the fused images need 64 or 128)", who,
                head_dim);
    CDM_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0 && n_heads <= 65535, CDM_ERR_BAD_SHAPE,
                "%s: n_kv_heads=%d must divide n_heads=%d", who, n_kv_heads, n_heads);
    // a wave writes the images of 128 consecutive columns: the Q | K | V boundaries must not cut through such a piece
    CDM_REQUIRE(head_dim == 128 || (n_heads % 2 == 0 && n_kv_heads % 2 == 0), CDM_ERR_UNSUPPORTED,
                "%s: head_dim 64 needs even head counts (n_heads=%d, n_kv_heads=%d)", who, n_heads, n_kv_heads);
    CDM_REQUIRE((cos == nullptr) == (sin == nullptr), CDM_ERR_BAD_ARG, "%s: cos and sin must be given together", who);
    CDM_REQUIRE(cdm_aligned16(cos) && cdm_aligned16(sin) && cdm_aligned16(workspace), CDM_ERR_BAD_ALIGN,
                "%s: rotary tables and workspace must be 16-byte aligned", who);
    CDM_REQUIRE(n_seg >= 1 && n_seg <= 64, CDM_ERR_BAD_ARG, "%s: n_seg=%d out of range", who, n_seg);
    // a 64-key tile image is written by one wave: the segments must tile the token range [0, n_tokens) in order,
    // each starting on a tile boundary (only the last may end inside a tile)
    int64_t n_tokens = 0;
    for (int g = 0; g < n_seg; ++g) {
        CDM_REQUIRE(seg_len[g] >= 0 && seg_start[g] == n_tokens && seg_start[g] % 64 == 0, CDM_ERR_UNSUPPORTED,
                    "%s: segment %d must start where the previous one ends, on a multiple of 64 tokens", who, g);
        n_tokens += seg_len[g];
    }
    CDM_REQUIRE(n_tokens <= 65535ll * 64, CDM_ERR_BAD_SHAPE, "%s: sizes out of range", who);
    if (qk_norm != nullptr) {
        // one weight row per GEMM segment: the norm's segments must be the GEMM's
        CDM_REQUIRE(qk_norm->k_weight && cdm_aligned16(qk_norm->k_weight) && qk_norm->seg_end, CDM_ERR_BAD_ARG,
                    "%s: qk_norm needs an aligned k_weight table and seg_end", who);
        CDM_REQUIRE(qk_norm->eps > 0.0f, CDM_ERR_BAD_ARG, "%s: qk_norm eps must be positive", who);
        CDM_REQUIRE(qk_norm->n_seg == n_seg, CDM_ERR_BAD_ARG, "%s: qk_norm has %d segments, the projection %d", who,
                    qk_norm->n_seg, n_seg);
        for (int g = 0; g < n_seg; ++g)
            CDM_REQUIRE(qk_norm->seg_end[g] == seg_start[g] + seg_len[g] || (g == n_seg - 1 && qk_norm->seg_end[g] >= n_tokens),
                        CDM_ERR_BAD_ARG, "%s: qk_norm segment %d does not end where the projection's does", who, g);
    }
    const int64_t need = cdm_attn_workspace_bytes(n_tokens, n_kv_heads, head_dim);
    CDM_REQUIRE(workspace_bytes >= need, CDM_ERR_BAD_ARG, "%s: workspace of at least %lld bytes required", who, (long long)need);
    const int64_t d_q = (int64_t)n_heads * head_dim, d_kv = (int64_t)n_kv_heads * head_dim;
    const int64_t n_key_tiles = (n_tokens + 63) / 64;
    const int64_t img = n_key_tiles * 64 * d_kv * 2;
    // the common checks of a grouped GEMM with N = d_q + 2 d_kv columns, of which only the first d_q exist in Q
    CDM_REQUIRE(Q && ldq >= d_q, CDM_ERR_BAD_ARG, "%s: Q row stride smaller than n_heads*head_dim", who);
    GemmParams pack{};
    pack.kp = (char*)workspace; pack.vp = (char*)workspace + img; pack.kmax = (float*)((char*)workspace + 2 * img);
    pack.d_q = (int)d_q; pack.d_kv = (int)d_kv; pack.n_key_tiles = (int)n_key_tiles;
    pack.k_eps = qk_norm ? qk_norm->eps : 0.0f;
    int32_t rc = grouped<FP8>(who, A, lda, sa, W, sw, ldw, nullptr, nullptr, Q, ldq, seg_start, seg_len, n_seg, d_q + 2 * d_kv, K,
                              CDM_EPI_QKV_PACK, nullptr, 0, nullptr, cos, sin, d_q, head_dim, stream, &pack,
                              qk_norm ? qk_norm->k_weight : nullptr);
    return rc;
}

}  // namespace

extern "C" int32_t cdm_grouped_gemm_qkv_pack_bf16(const void* A, int64_t lda, const void* const* W, int64_t ldw, void* Q,
                                                  int64_t ldq, const int64_t* seg_start, const int64_t* seg_len,
                                                  int32_t n_seg, int64_t K, int32_t n_heads, int32_t n_kv_heads,
                                                  int32_t head_dim, const float* cos, const float* sin,
                                                  const cdm_qk_norm* qk_norm, void* workspace, int64_t workspace_bytes,
                                                  void* stream) {
    return qkv_pack<false>("grouped_gemm_qkv_pack_bf16", A, lda, nullptr, W, nullptr, ldw, Q, ldq, seg_start, seg_len, n_seg,
                           K, n_heads, n_kv_heads, head_dim, cos, sin, qk_norm, workspace, workspace_bytes, stream);
}

extern "C" int32_t cdm_grouped_gemm_qkv_pack_fp8(const void* Aq, int64_t lda, const float* sa, const void* const* Wq,
                                                 const float* const* sw, int64_t ldw, void* Q, int64_t ldq,
                                                 const int64_t* seg_start, const int64_t* seg_len, int32_t n_seg,
                                                 int64_t K, int32_t n_heads, int32_t n_kv_heads, int32_t head_dim,
                                                 const float* cos, const float* sin, const cdm_qk_norm* qk_norm,
                                                 void* workspace, int64_t workspace_bytes, void* stream) {
    return qkv_pack<true>("grouped_gemm_qkv_pack_fp8", Aq, lda, sa, Wq, sw, ldw, Q, ldq, seg_start, seg_len, n_seg, K,
                          n_heads, n_kv_heads, head_dim, cos, sin, qk_norm, workspace, workspace_bytes, stream);
}

extern "C" int32_t cdm_gemm_bf16(const void* A, int64_t lda, const void* W, int64_t ldw, const void* W2, void* C,
                                 int64_t ldc, int64_t M, int64_t N, int64_t K, int32_t epilogue, const void* R,
                                 int64_t ldr, const float* gate, const float* cos, const float* sin,
                                 int64_t rope_cols, int32_t head_dim, void* stream) {
    const int64_t start = 0;
    const void* w2[1] = {W2};
    return grouped<false>("gemm_bf16", A, lda, nullptr, &W, nullptr, ldw, W2 ? w2 : nullptr, nullptr, C, ldc, &start, &M, 1, N,
                          K, epilogue, R, ldr, &gate, cos, sin, rope_cols, head_dim, stream);
}

extern "C" int32_t cdm_gemm_fp8(const void* Aq, int64_t lda, const float* sa, const void* Wq, int64_t ldw,
                                const float* sw, const void* W2q, const float* sw2, void* C, int64_t ldc, int64_t M,
                                int64_t N, int64_t K, int32_t epilogue, const void* R, int64_t ldr, const float* gate,
                                const float* cos, const float* sin, int64_t rope_cols, int32_t head_dim,
                                float* row_amax, int64_t amax_ld, void* stream) {
    const int64_t start = 0;
    const void* w2[1] = {W2q};
    const float* s2[1] = {sw2};
    CDM_REQUIRE(sa && sw, CDM_ERR_BAD_ARG, "gemm_fp8: null scale pointer");
    return grouped<true>("gemm_fp8", Aq, lda, sa, &Wq, &sw, ldw, W2q ? w2 : nullptr, s2, C, ldc, &start, &M, 1, N, K, epilogue,
                         R, ldr, &gate, cos, sin, rope_cols, head_dim, stream, nullptr, nullptr, row_amax, amax_ld);
}

extern "C" int32_t cdm_grouped_gemm_bf16(const void* A, int64_t lda, const void* const* W, int64_t ldw,
                                         const void* const* W2, void* C, int64_t ldc, const int64_t* seg_start,
                                         const int64_t* seg_len, int32_t n_seg, int64_t N, int64_t K,
                                         int32_t epilogue, const void* R, int64_t ldr, const float* const* gate,
                                         const float* cos, const float* sin, int64_t rope_cols, int32_t head_dim,
                                         void* stream) {
    return grouped<false>("grouped_gemm_bf16", A, lda, nullptr, W, nullptr, ldw, W2, nullptr, C, ldc, seg_start, seg_len, n_seg,
                          N, K, epilogue, R, ldr, gate, cos, sin, rope_cols, head_dim, stream);
}

extern "C" int32_t cdm_grouped_gemm_fp8(const void* Aq, int64_t lda, const float* sa, const void* const* Wq,
                                        const float* const* sw, int64_t ldw, const void* const* W2q,
                                        const float* const* sw2, void* C, int64_t ldc, const int64_t* seg_start,
                                        const int64_t* seg_len, int32_t n_seg, int64_t N, int64_t K, int32_t epilogue,
                                        const void* R, int64_t ldr, const float* const* gate, const float* cos,
                                        const float* sin, int64_t rope_cols, int32_t head_dim, float* row_amax,
                                        int64_t amax_ld, void* stream) {
    return grouped<true>("grouped_gemm_fp8", Aq, lda, sa, Wq, sw, ldw, W2q, sw2, C, ldc, seg_start, seg_len, n_seg, N, K,
                         epilogue, R, ldr, gate, cos, sin, rope_cols, head_dim, stream, nullptr, nullptr, row_amax, amax_ld);
}

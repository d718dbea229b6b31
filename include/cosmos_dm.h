/*
 * cosmos_dm.h - C ABI of libcosmos_dm_hip.so: hand-written HIP kernels (gfx950 / MI355X)
 * for the Cosmos 3 Generator-mode diffusion-transformer (DM) block forward.
 *
 * The reference repository (NVIDIA/cosmos) has no FFI of its own for this path: it calls
 * the block through the diffusers pipeline (README.md:238-263,
 * cookbooks/cosmos3/generator/audiovisual/run_with_diffusers.ipynb:523-612), whose
 * transformer -> block -> attention-processor forward runs these operators as torch ops
 * (architecture: README.md:74 and cookbooks/cosmos3/cosmos3-model-architecture.png).
 * Each entry point below names the operator of that forward it replaces.
 *
 * Conventions
 *   - every function returns 0 (CDM_OK) or a negative cdm_status; cdm_last_error() gives
 *     a thread-local message for the last failure on the calling thread;
 *   - all pointers are DEVICE pointers owned by the caller (16-byte aligned unless noted),
 *     tensors are row-major and bf16 (uint16 storage) unless noted; `ld*` are row strides
 *     in ELEMENTS;
 *   - the library never allocates, frees or retains device memory, never synchronises the
 *     device, and enqueues all work on `stream` (a hipStream_t passed as void*);
 *   - arguments are validated on the host before any launch.
 */
#ifndef COSMOS_DM_H
#define COSMOS_DM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum cdm_status {
    CDM_OK = 0,
    CDM_ERR_BAD_ARG = -1,     /* null pointer, negative size, unknown enum value */
    CDM_ERR_BAD_SHAPE = -2,   /* size not supported by the kernels (see each function) */
    CDM_ERR_BAD_ALIGN = -3,   /* pointer or stride not 16-byte aligned */
    CDM_ERR_NO_DEVICE = -4,   /* no HIP device visible to the process */
    CDM_ERR_LAUNCH = -5,      /* hipGetLastError() after a launch was not hipSuccess */
    CDM_ERR_UNSUPPORTED = -6  /* feature combination not built */
} cdm_status;

/* GEMM epilogues (cdm_gemm_bf16 / cdm_gemm_fp8). */
typedef enum cdm_epilogue {
    CDM_EPI_NONE = 0,          /* C = A W^T                                              */
    CDM_EPI_SWIGLU = 1,        /* C = silu(A Wg^T) * (A Wu^T)          (W = Wg, W2 = Wu) */
    CDM_EPI_GATE_RESIDUAL = 2, /* C = R + gate[n] * (A W^T)            (gate may be null = 1) */
    CDM_EPI_ROPE_QK = 3,       /* C = A W^T with rotate-half RoPE applied to the columns
                                  below `rope_cols` (heads of width head_dim)            */
    CDM_EPI_GATE_RESIDUAL_F32 = 4, /* CDM_EPI_GATE_RESIDUAL with C and R stored as fp32: the residual stream kept in
                                  fp32 (28 roundings of the stream to bf16 alone cost percent-level accuracy) */
    CDM_EPI_QKV_PACK = 5       /* internal to cdm_grouped_gemm_qkv_pack_*: rejected by the general GEMM entry points */
} cdm_epilogue;

/* Library version (major*10000 + minor*100 + patch). */
int32_t cdm_version(void);

/* Hash of the sources this library was built from (16 hex digits): a loader compares it with the hash of the
 * sources it sees and refuses, or rebuilds, a stale build. */
const char* cdm_source_hash(void);

/* Message for the last non-zero status returned on this thread ("" if none). */
const char* cdm_last_error(void);

/* Number of HIP devices visible (0 on a host without a GPU); never fails. */
int32_t cdm_device_count(void);

/*
 * adaLN-modulated RMSNorm - replaces the per-branch norm + shift/scale modulation at the
 * head of each half of the block (README.md:74 "per-branch norm"; RMSNorm definition as in
 * transformers Qwen3VLTextRMSNorm.forward, models/qwen3_vl/modeling_qwen3_vl.py:400-405).
 *   y[i,j] = x[i,j] * rsqrt(mean_j x[i,:]^2 + eps) * w[j] * (1 + scale[j]) + shift[j]
 * x, y: [n_tokens, d] bf16 (y may alias x); w: [d] bf16; shift, scale: [d] fp32, either may be
 * null (plain RMSNorm of the AR branch).  d % 8 == 0, d <= 8192; all pointers 16-byte aligned (shift and scale too:
 * slices of a [6 d] modulation row are, since d % 8 == 0).
 */
int32_t cdm_adaln_rmsnorm_bf16(const void* x, const void* w, const float* shift, const float* scale,
                               void* y, int64_t n_tokens, int64_t d, float eps, void* stream);

/* The same operator reading an fp32 residual stream: x [n_tokens, d] fp32, y bf16 (the GEMM operand). */
int32_t cdm_adaln_rmsnorm_f32(const float* x, const void* w, const float* shift, const float* scale,
                              void* y, int64_t n_tokens, int64_t d, float eps, void* stream);

/*
 * Same norm with a per-token e4m3 quantisation epilogue (fp8 variant of the block):
 *   s_tok[i] = max_j |y[i,j]| / 448 (0 -> 1);  yq[i,j] = e4m3(y[i,j] / s_tok[i])
 * yq: [n_tokens, d] bytes (OCP e4m3fn), s_tok: [n_tokens] fp32.
 */
int32_t cdm_adaln_rmsnorm_quant_e4m3(const void* x, const void* w, const float* shift, const float* scale,
                                     void* yq, float* s_tok, int64_t n_tokens, int64_t d, float eps,
                                     void* stream);
int32_t cdm_adaln_rmsnorm_f32_quant_e4m3(const float* x, const void* w, const float* shift, const float* scale,
                                         void* yq, float* s_tok, int64_t n_tokens, int64_t d, float eps,
                                         void* stream);      /* x fp32 */

/*
 * Per-row dynamic e4m3 quantisation of a bf16 matrix (activations before a quantised linear):
 *   s[i] = max_j |a[i,j]| / 448 (0 -> 1);  q[i,j] = e4m3(a[i,j] / s[i]).  cols % 8 == 0, cols <= 32768.
 * Also used offline for weights W[out, in] (per-output-channel scales).
 */
int32_t cdm_quant_rows_e4m3(const void* a, int64_t lda, void* q, float* s, int64_t rows, int64_t cols,
                            void* stream);

/*
 * The same quantisation (bit for bit) where the kernel that produced `a` left partial row maxima behind:
 * parts [rows, n_parts] fp32 (row stride ldp), entry (i, c) = max |a[i, j]| over one range of columns j, the ranges
 * covering the row (cdm_attn_fwd_packed_bf16 writes one entry per head, the SWIGLU epilogue of the e4m3 GEMM one per 64
 * output columns).  s[i] = max_c parts[i, c] / 448; the row is read once instead of twice.  n_parts <= 4096.
 */
int32_t cdm_quant_rows_from_parts_e4m3(const void* a, int64_t lda, const float* parts, int64_t ldp, int64_t n_parts,
                                       void* q, float* s, int64_t rows, int64_t cols, void* stream);

/*
 * bf16 linear layer(s) with a fused epilogue - replaces nn.Linear (no bias) of the DM branch:
 * add_q_proj/add_k_proj/add_v_proj (fused as one [3d, d] weight), to_add_out, and the
 * moe_gen gate/up/down projections (parameter names: transformers
 * models/cosmos3_omni/modeling_cosmos3_omni.py:39-60).
 *   A: [M, K] (lda), W: [N, K] (ldw) row-major "out, in" like nn.Linear.weight, C: [M, N] (ldc).
 *   fp32 accumulation on MFMA, one rounding to bf16 at the end.
 *   CDM_EPI_SWIGLU:        W = gate_proj.weight, W2 = up_proj.weight (same shape/ld), C: [M, N]
 *   CDM_EPI_GATE_RESIDUAL: R: [M, N] (ldr) residual (may alias C), gate: [N] fp32 or null
 *   CDM_EPI_GATE_RESIDUAL_F32: the same with C and R fp32 (ldc, ldr in fp32 elements)
 *   CDM_EPI_ROPE_QK:       cos, sin: [M, head_dim/2] fp32; columns [0, rope_cols) are rotated
 *                          per head (pairs (i, i + head_dim/2)); head_dim in {64, 128};
 *                          rope_cols % 256 == 0
 * K % 128 == 0; M, N >= 1 arbitrary (N % 8 == 0); ldc and ldr multiples of 8 elements (every output and residual
 * row starts on a 16-byte boundary: the epilogue moves groups of four columns per lane).
 */
int32_t cdm_gemm_bf16(const void* A, int64_t lda, const void* W, int64_t ldw, const void* W2,
                      void* C, int64_t ldc, int64_t M, int64_t N, int64_t K, int32_t epilogue,
                      const void* R, int64_t ldr, const float* gate,
                      const float* cos, const float* sin, int64_t rope_cols, int32_t head_dim,
                      void* stream);

/*
 * fp8 (e4m3) linear with per-token and per-output-channel scales - the quantised variant:
 *   C[i,j] = sa[i] * sw[j] * sum_k Aq[i,k] Wq[j,k]   (fp32 accumulate) -> bf16, then the epilogue.
 * Aq: [M, K] bytes, Wq: [N, K] bytes (W2q/sw2 for CDM_EPI_SWIGLU).  K % 256 == 0.
 * row_amax (optional, CDM_EPI_SWIGLU only): [M, amax_ld] fp32, amax_ld >= ceil(N / 64); entry (i, c) receives the largest
 * |C[i, j]| over columns 64 c .. 64 c + 63 (of the bf16 values stored), for cdm_quant_rows_from_parts_e4m3: the hidden
 * activations are quantised per token for the down projection without a pass that searches the row maxima.
 */
int32_t cdm_gemm_fp8(const void* Aq, int64_t lda, const float* sa, const void* Wq, int64_t ldw, const float* sw,
                     const void* W2q, const float* sw2,
                     void* C, int64_t ldc, int64_t M, int64_t N, int64_t K, int32_t epilogue,
                     const void* R, int64_t ldr, const float* gate,
                     const float* cos, const float* sin, int64_t rope_cols, int32_t head_dim,
                     float* row_amax, int64_t amax_ld, void* stream);

/*
 * Standalone 3-D mRoPE on Q and K in place - replaces apply_rotary_pos_emb with mRoPE tables
 * (rotate-half pairs, transformers models/qwen3_vl/modeling_qwen3_vl.py:138-142,412-435;
 * table layouts :352-388 and models/qwen2_vl/modeling_qwen2_vl.py:212-222).
 *   q, k: [n_tokens, n_heads, head_dim] with row strides ldq, ldk (elements); k may be null.
 *   cos, sin: [n_tokens, head_dim/2] fp32 (the axis layout lives entirely in the tables).
 * head_dim in {64, 128}.
 */
int32_t cdm_mrope_qk_bf16(void* q, int64_t ldq, void* k, int64_t ldk, const float* cos, const float* sin,
                          int64_t n_tokens, int32_t n_heads, int32_t head_dim, void* stream);

/*
 * Optional per-head QK-RMSNorm, applied to Q and K in fp32 ahead of the rotation inside the attention entry
 * points - replaces the q_norm / k_norm modules of the attention layer (parameters norm_q / norm_k of the AR
 * branch and norm_added_q / norm_added_k of the DM branch, transformers
 * models/cosmos3_omni/modeling_cosmos3_omni.py:45-46; application order norm -> RoPE:
 * models/qwen3_vl/modeling_qwen3_vl.py:463-466,479-481; RMSNorm :400-405):
 *   y = x * rsqrt(mean_over_head_dim(x^2) + eps) * weight.
 * Tokens form n_seg (1..8) contiguous segments, segment i = [seg_end[i-1], seg_end[i]) with seg_end[-1] = 0 and
 * seg_end[n_seg-1] >= n_tokens; segment i uses row i of the weight tables (one row per MoT branch).
 * The struct itself and seg_end are HOST memory, read during the call; the weight tables are device memory.
 */
typedef struct cdm_qk_norm {
    const float* q_weight;    /* device, [n_seg, head_dim] fp32 */
    const float* k_weight;    /* device, [n_seg, head_dim] fp32 */
    const int64_t* seg_end;   /* host, [n_seg] */
    int32_t n_seg;
    float eps;
} cdm_qk_norm;

/*
 * Shared full (non-causal) self-attention over the joint sequence, with rotate-half mRoPE applied in
 * registers to Q and K on the way in - replaces the attention processor's apply_rotary_pos_emb +
 * scaled_dot_product_attention (README.md:74; eager form transformers
 * models/qwen3_vl/modeling_qwen3_vl.py:171-193 with fp32 softmax; RoPE :138-142, :412-435).
 *   O = softmax(rope(Q) rope(K)^T / sqrt(head_dim)) V per head, no mask.
 *   q: [n_tokens, n_heads, head_dim], k, v: [n_tokens, n_kv_heads, head_dim] with row strides ldq, ldk, ldv;
 *   o: [n_tokens, n_heads*head_dim] (ldo).  n_kv_heads divides n_heads: query head h uses K / V head
 *   h / (n_heads / n_kv_heads) (grouped-query attention: num_key_value_heads,
 *   models/qwen3_vl/configuration_qwen3_vl.py:86; repeat_kv, models/qwen3_vl/modeling_qwen3_vl.py:159-168);
 *   n_kv_heads = n_heads is plain multi-head attention.
 *   cos, sin: [n_tokens, head_dim/2] fp32 rotary tables, or both null when Q and K are already rotated.
 *   qk_norm: null, or the per-head RMSNorm of Q and K described above.
 *   causal_prefix: 0 = full attention.  P > 0 = the hybrid mask of the architecture figure
 *     (cookbooks/cosmos3/cosmos3-model-architecture.png, right panel; README.md:74): the first P tokens (the AR /
 *     text run) attend causally among themselves and to nothing else, every other token attends to all tokens.
 *   workspace: cdm_attn_workspace_bytes(n_tokens, n_kv_heads, head_dim) bytes of caller-owned device memory
 *   (holds K and V re-laid out as 64-key tile images, followed by one fp32 per K/V head and tile: the largest key
 *   norm of the tile, from which the kernel bounds the scores of a row and decides whether it needs running row maxima
 *   at all); its contents are undefined afterwards.
 * head_dim in {64, 128}; n_tokens >= 1 arbitrary.
 */
int64_t cdm_attn_workspace_bytes(int64_t n_tokens, int32_t n_kv_heads, int32_t head_dim);
int32_t cdm_attn_fwd_bf16(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v, int64_t ldv,
                          const float* cos, const float* sin, void* o, int64_t ldo, int64_t n_tokens,
                          int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, void* workspace,
                          int64_t workspace_bytes, const cdm_qk_norm* qk_norm, int64_t causal_prefix, void* stream);

/*
 * The two stages of cdm_attn_fwd_bf16 as separate calls (same operator, same citations): first K (rotated
 * if tables are given) and V are packed into the workspace as tile images (a streaming pass), then the
 * attention kernel proper reads Q (rotating it with the same tables) and the workspace.  A caller that
 * times or profiles the attention kernel alone, or that reuses packed K/V across calls, uses these.
 *   prefix_workspace / n_prefix_tokens (optional): tile images, made by an earlier cdm_attn_pack_kv_bf16 call over
 *   n_prefix_tokens tokens (any count: the padding of a last, partial tile is masked), of keys that PRECEDE the keys of
 *   `workspace`; the n_tokens queries
 *   then attend to n_prefix_tokens + n_tokens keys.  Under the hybrid mask the K/V of the text run do not depend on
 *   the denoising step, so they are packed once per prompt and passed here at every step, and the per-step call
 *   carries only the generator tokens.  Cannot be combined with causal_prefix.
 * cdm_attn_pack_kv_bf16 sees K / V heads only (n_kv_heads of them).
 *   row_amax (optional, 4-byte aligned): [n_tokens, n_heads] fp32; entry (i, h) receives the largest |o| of row i within
 *   head h (of the bf16 values stored) - the partial row maxima cdm_quant_rows_from_parts_e4m3 takes when the attention
 *   output is quantised per token for the e4m3 output projection.
 *   split_scratch / split_scratch_bytes (optional): see cdm_attn_split_scratch_bytes below; null or too small = one pass.
 */
int32_t cdm_attn_pack_kv_bf16(const void* k, int64_t ldk, const void* v, int64_t ldv, const float* cos,
                              const float* sin, void* workspace, int64_t workspace_bytes, int64_t n_tokens,
                              int32_t n_kv_heads, int32_t head_dim, const cdm_qk_norm* qk_norm, void* stream);
int32_t cdm_attn_fwd_packed_bf16(const void* q, int64_t ldq, const float* cos, const float* sin,
                                 const void* workspace, void* o, int64_t ldo, int64_t n_tokens, int32_t n_heads,
                                 int32_t n_kv_heads, int32_t head_dim, const cdm_qk_norm* qk_norm,
                                 const void* prefix_workspace, int64_t n_prefix_tokens, int64_t causal_prefix,
                                 float* row_amax, void* split_scratch, int64_t split_scratch_bytes, void* stream);
/*
 * Scratch memory for splitting the last, partial round of attention workgroups (no counterpart in the reference: a
 * scheduling matter of this kernel).  A launch runs 32 workgroups per XCD at a time, each 256 query rows of one head,
 * and takes ceil(n_heads / 8 * ceil(n_tokens / 256) / 32) rounds however few workgroups the last one holds.  Given
 * `split_scratch` of at least this many bytes, cdm_attn_fwd_packed_bf16 cuts the query blocks of that last round into
 * 2, 4 or 8 units by key range and merges their results with a second, small kernel (same operator; the output
 * differs from the single-pass one by the rounding of the partial results to bf16).  0 = nothing to split for this
 * shape (fewer than two whole rounds, heads not a multiple of 8, a whole number of rounds, or no split that ends in
 * half a round or less - a round with idle CUs runs faster on this power-limited chip, so less does not pay); a launch whose causal
 * prefix reaches into the last round's query blocks is never split.  n_heads counts query heads.
 * cdm_attn_fwd_bf16 uses what its workspace holds beyond cdm_attn_workspace_bytes (rounded up to 256) for this.
 */
int64_t cdm_attn_split_scratch_bytes(int64_t n_tokens, int32_t n_heads, int32_t head_dim);

/*
 * cdm_attn_fwd_bf16 for callers that cannot allocate device memory or carry a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference; the
 * operator and all other arguments are those of cdm_attn_fwd_bf16.  The K / V tile images go into a device array
 * built into the library (CDM_ATTN_STATIC_SCRATCH_BYTES per GPU, held until the process ends); the call allocates
 * nothing.  Shapes whose images (cdm_attn_workspace_bytes) exceed that size are rejected with CDM_ERR_BAD_SHAPE.
 * The result is bit-equal to cdm_attn_fwd_bf16 with a workspace of exactly cdm_attn_workspace_bytes (the array holds
 * no scratch for a split of the last round of workgroups).
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different streams or
 * threads) race; calls on one stream are ordered and need no clearing in between (every call rewrites all
 * tiles it reads, padding included).  The array's address is looked up once per device, by the first call on that
 * device or by cdm_attn_static_scratch_bytes(): before recording the entry point into a graph, call either outside the
 * capture with that device current.
 */
#define CDM_ATTN_STATIC_SCRATCH_BYTES (32ll << 20)
int64_t cdm_attn_static_scratch_bytes(void);
int32_t cdm_attn_fwd_static_bf16(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v, int64_t ldv,
                                 const float* cos, const float* sin, void* o, int64_t ldo, int64_t n_tokens,
                                 int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, const cdm_qk_norm* qk_norm,
                                 int64_t causal_prefix, void* stream);

/*
 * Linear layer WITH bias at the edges of the stack - replaces nn.Linear of proj_in / proj_out (patchify and
 * un-patchify projections), action_proj_in / action_proj_out and audio_proj_in / audio_proj_out (parameter names:
 * transformers models/cosmos3_omni/modeling_cosmos3_omni.py:48-58), where K or N is a few dozen elements and the
 * layer is bound by moving the token rows once.
 *   A: [M, K] (lda), W: [N, K] (ldw) row-major like nn.Linear.weight, bias: [N] bf16 or null, C: [M, N] (ldc), all bf16;
 *   fp32 accumulation on MFMA, bias added in fp32, one rounding to bf16.
 * Any M, N, K >= 1 (a last partial 32-wide k-step is zero-filled).  16-byte accesses are used where A, W, C and their row
 * strides are 16-byte aligned and N, K are multiples of 8; other shapes (an action stream 6 wide) go element by element.
 */
int32_t cdm_linear_bias_bf16(const void* A, int64_t lda, const void* W, int64_t ldw, const void* bias, void* C,
                             int64_t ldc, int64_t M, int64_t N, int64_t K, void* stream);

/*
 * Mixture-of-Transformers routed linear: contiguous token segments, one weight set each
 * (README.md:53,74 - per-modality weights around one shared attention).  Equivalent to
 * cdm_gemm_bf16 on rows [seg_start[g], seg_start[g] + seg_len[g]) with W[g] (and W2[g], gate[g]).
 * seg_* are HOST arrays of n_seg entries; W/W2/gate are HOST arrays of n_seg device pointers
 * (gate[g] may be null = ungated branch).  Segments must not overlap.  All segments run in ONE grid (eight
 * segments per launch): the tiles of a short segment fill the tail of a long segment's grid.
 * A, C, R, cos, sin are the tensors of the whole sequence (rows are addressed by their global index).
 */
int32_t cdm_grouped_gemm_bf16(const void* A, int64_t lda, const void* const* W, int64_t ldw,
                              const void* const* W2, void* C, int64_t ldc,
                              const int64_t* seg_start, const int64_t* seg_len, int32_t n_seg,
                              int64_t N, int64_t K, int32_t epilogue,
                              const void* R, int64_t ldr, const float* const* gate,
                              const float* cos, const float* sin, int64_t rope_cols, int32_t head_dim,
                              void* stream);

/* The same for e4m3 operands (see cdm_gemm_fp8): sa is the per-token scale of the whole sequence, sw[g] / sw2[g] the
 * per-output-channel scales of segment g's weights. */
int32_t cdm_grouped_gemm_fp8(const void* Aq, int64_t lda, const float* sa, const void* const* Wq,
                             const float* const* sw, int64_t ldw, const void* const* W2q,
                             const float* const* sw2, void* C, int64_t ldc,
                             const int64_t* seg_start, const int64_t* seg_len, int32_t n_seg,
                             int64_t N, int64_t K, int32_t epilogue,
                             const void* R, int64_t ldr, const float* const* gate,
                             const float* cos, const float* sin, int64_t rope_cols, int32_t head_dim,
                             float* row_amax, int64_t amax_ld, void* stream);

/* Exported by the cross-check build only (libcosmos_dm_hip_crosscheck.so, compiled with -DCDM_CROSSCHECK), which the
 * parity tests load to compare the default kernels with their predecessors; the product library has no such state.
 * Process-wide (not per thread or stream): selects a kernel variant by name; returns the previous value, or a negative
 * status for an unknown name/value.  Default 0 = the kernels of the product library.
 *   "attn": 1 = 64 query rows per wave (four waves per workgroup), 2 = the default kernel with per-tile row maxima always
 *           taken (the default drops them where the norm bound of the scores allows);
 *   "gemm": 1 = two-stage pipeline with four waves and 32 x 32 MFMAs instead of the five-slot ring with eight waves and
 *           16 x 16 MFMAs. */
#ifdef CDM_CROSSCHECK
int32_t cdm_set_variant(const char* op, int32_t variant);
#endif

/*
 * Fused QKV projection of the shared attention (the three projections add_q_proj / add_k_proj / add_v_proj resp.
 * to_q / to_k / to_v of transformers models/cosmos3_omni/modeling_cosmos3_omni.py:41-46, concatenated row-wise into
 * W[g] = [d_q + 2 d_kv, K] per branch) whose K and V columns never reach memory as rows: each 64-token x 128-channel
 * piece leaves the GEMM as the attention kernel's tile image - K rotated with cos/sin ([n_tokens, 64] fp32, may both
 * be null) on the way, V transposed, the largest key norm of the tile recorded - what cdm_attn_pack_kv_bf16 would
 * have produced from the K / V rows (V bit for bit; K is rotated from the fp32 accumulators here, from the rows
 * rounded to bf16 there: one rounding less).  Q (columns [0, d_q)) is written to
 * Q [n_tokens, ldq] as plain rows, NOT rotated: cdm_attn_fwd_packed_bf16 rotates it at load when given the tables.
 * `workspace` (cdm_attn_workspace_bytes(n_tokens, n_kv_heads, head_dim) bytes, n_tokens = sum of seg_len) is then
 * passed to cdm_attn_fwd_packed_bf16.  qk_norm (optional): the per-head RMSNorm of K (norm_k / norm_added_k) is applied
 * to the fp32 accumulators ahead of the rotation, segment g of the projection using row g of qk_norm->k_weight
 * (qk_norm->n_seg = n_seg, qk_norm->seg_end[g] = seg_start[g] + seg_len[g]); the Q rows leave un-normalised -
 * cdm_attn_fwd_packed_bf16 normalises and rotates them at load when given the same descriptor.
 * Restrictions: head_dim 128, or 64 with even n_heads and n_kv_heads (a wave writes the images of 128 consecutive
 * columns); the segments tile [0, n_tokens) in order and each starts on a multiple of 64 tokens
 * (CDM_ERR_UNSUPPORTED otherwise - callers fall back to the GEMM + cdm_attn_pack_kv_bf16 pair).
 */
int32_t cdm_grouped_gemm_qkv_pack_bf16(const void* A, int64_t lda, const void* const* W, int64_t ldw, void* Q,
                                       int64_t ldq, const int64_t* seg_start, const int64_t* seg_len, int32_t n_seg,
                                       int64_t K, int32_t n_heads, int32_t n_kv_heads, int32_t head_dim,
                                       const float* cos, const float* sin, const cdm_qk_norm* qk_norm, void* workspace,
                                       int64_t workspace_bytes, void* stream);
int32_t cdm_grouped_gemm_qkv_pack_fp8(const void* Aq, int64_t lda, const float* sa, const void* const* Wq,
                                      const float* const* sw, int64_t ldw, void* Q, int64_t ldq,
                                      const int64_t* seg_start, const int64_t* seg_len, int32_t n_seg, int64_t K,
                                      int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, const float* cos,
                                      const float* sin, const cdm_qk_norm* qk_norm, void* workspace,
                                      int64_t workspace_bytes, void* stream);

/*
 * Classifier-free-guidance combine fused with the scheduler's linear latent update - replaces, inside one
 * denoising iteration of the pipeline (Cosmos3OmniPipeline.__call__, README.md:249-263: guidance_scale;
 * README.md:247: UniPCMultistepScheduler with flow_shift), the elementwise tail
 *     v       = v_uncond + guidance * (v_cond - v_uncond)            (v = v_cond when v_uncond is null)
 *     outs[j] = coef[j][0] * x + coef[j][1] * v + sum_k coef[j][2 + k] * hist[k]        j = 0 .. n_out-1
 * which is the form of an Euler flow-matching step (one output, coef = {1, sigma_next - sigma}) and of every linear
 * multistep update: a UniPC step (corrector of the current latents, then predictor) is three outputs - the next
 * latents, the corrected latents the next corrector starts from, and the data prediction x - sigma v kept as
 * history - of the current latents, the prediction, the previous corrected latents and the kept data predictions.
 * The scheduler computes the scalar coefficients on the host; this kernel makes ONE pass over the tensors.
 *   x, hist[k], outs[j]: fp32 [n]; v_cond, v_uncond: bf16 [n] (the transformer's output).
 *   hist, outs: HOST arrays of n_hist (0..4) / n_out (1..3) device pointers; coef: HOST array, row-major
 *   [n_out][2 + n_hist].  An output may be x or a hist tensor itself (in-place latents, a recycled history slot);
 *   two outputs may not coincide.
 */
int32_t cdm_cfg_step_f32(const float* x, const void* v_cond, const void* v_uncond, float guidance,
                         const float* const* hist, int32_t n_hist, const float* coef, float* const* outs,
                         int32_t n_out, int64_t n, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* COSMOS_DM_H */

// Shared device/host helpers for the cosmos_dm HIP kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/cosmos_dm.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef uint16_t bf16_t;   // storage type at the ABI

// ---------------------------------------------------------------- host side
void cdm_set_error(const char* fmt, ...);   // thread-local message, defined in api.hip

#define CDM_FAIL(code, ...)            \
    do {                               \
        cdm_set_error(__VA_ARGS__);    \
        return (code);                 \
    } while (0)

#define CDM_REQUIRE(cond, code, ...)   \
    do {                               \
        if (!(cond)) CDM_FAIL(code, __VA_ARGS__); \
    } while (0)

static inline bool cdm_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static inline int32_t cdm_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) CDM_FAIL(CDM_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
    return CDM_OK;
}

int32_t cdm_require_device(void);           // CDM_OK or CDM_ERR_NO_DEVICE (sets the message)
// Kernel variant selected for an operator (0 = attn, 1 = gemm).  Only the cross-check build (-DCDM_CROSSCHECK) carries
// the superseded kernels and the knob that selects them; the product library always runs the default kernels.
#ifdef CDM_CROSSCHECK
int32_t cdm_get_variant(int which);
#else
static inline int32_t cdm_get_variant(int) { return 0; }
#endif

// -------------------------------------------------------------- device side
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t lo16) { return __uint_as_float(lo16 << 16); }

// unpack two bf16 stored in one 32-bit word
__device__ __forceinline__ float bf16lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// round-to-nearest-even pack of two floats into one 32-bit word (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    bf16x2 p;
    p[0] = (__bf16)a;
    p[1] = (__bf16)b;
    return __builtin_bit_cast(uint32_t, p);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// One 16-byte-per-lane direct-to-LDS load, written as inline assembly so that the compiler's wait-count
// insertion does not see an LDS write it would have to guard conservatively across a loop back-edge (it would
// put s_waitcnt vmcnt(0) in front of fragment reads and drain a multi-stage pipeline).  Every wait on these
// loads is therefore an explicit s_waitcnt vmcnt(n) written by the kernel that issued them.  M0 = LDS byte address of the wave's
// 1 KB destination; one wait state is required between the M0 write and the load.
__device__ __forceinline__ void lds_dma16(const char* uniform_base, uint32_t lane_offset, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(lane_offset), "s"(uniform_base)
                 : "memory", "m0");
}

__device__ __forceinline__ uint32_t lds_addr_of(const char* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)p;
}


// Shared host/device helpers of the gfx950 switched-linear library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>
#include "../../include/kairos_mi.h"

typedef _Float16 half_t;
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));
typedef int i4_t __attribute__((ext_vector_type(4)));
typedef int i16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u4_t __attribute__((ext_vector_type(4)));

#define KMI_WAVE 64

// ---- host side error plumbing -------------------------------------------------------------------
int kmi_set_error(int code, const char* fmt, ...);   // stores the message, returns code
static inline int kmi_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return kmi_set_error(KMI_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return KMI_OK;
}
static inline bool kmi_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#define KMI_REQUIRE_PTR(p)                                                         \
    do {                                                                           \
        if ((p) == nullptr) return kmi_set_error(KMI_E_NULL, "%s: %s is NULL", __func__, #p); \
        if (!kmi_aligned16(p)) return kmi_set_error(KMI_E_ALIGN, "%s: %s is not 16-byte aligned", __func__, #p); \
    } while (0)

#ifdef __HIPCC__
// ---- device helpers -----------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* lds_void_ptr;          // destination of a direct-to-LDS buffer load
typedef const __attribute__((address_space(1))) void* global_void_ptr;
__device__ __forceinline__ h2_t as_h2(uint32_t u) { return __builtin_bit_cast(h2_t, u); }
__device__ __forceinline__ uint32_t as_u32(h2_t h) { return __builtin_bit_cast(uint32_t, h); }

__device__ __forceinline__ h2_t pk_fma(h2_t a, h2_t b, h2_t c) { return __builtin_elementwise_fma(a, b, c); }

// Exact uint4 -> fp16 pairs.  A 32-bit word carries 8 nibbles; nibble `a` of both 16-bit halves
// gives two weights that are adjacent along K.  OR-ing the nibble into the mantissa of 1024.0
// (0x6400) yields 1024+q (low nibble of a byte) or 1024+16q (high nibble); both are turned into the
// exact integer q before the scale is applied, so the result equals fma_f16(q, s, z) bit for bit.
__device__ __forceinline__ h2_t nib_lo_to_q(uint32_t w) {      // nibble at bits [3:0] / [19:16]
    const h2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    return as_h2((w & 0x000F000Fu) | 0x64006400u) - k1024;
}
__device__ __forceinline__ h2_t nib_hi_to_q(uint32_t w) {      // nibble at bits [7:4] / [23:20]
    const h2_t k16th = {(half_t)0.0625f, (half_t)0.0625f};
    const h2_t km64 = {(half_t)-64.0f, (half_t)-64.0f};
    return pk_fma(as_h2((w & 0x00F000F0u) | 0x64006400u), k16th, km64);
}

// One 16-byte chunk (four words) holds 32 weights of one row: word t, nibble a, half c is
// k = 8a + 2t + c.  dequant_nibble<a> returns the eight K-contiguous weights k = 8a .. 8a+7.
template <int A>
__device__ __forceinline__ h8_t dequant_nibble(const u4_t& u, h2_t s2, h2_t z2) {
    h2_t r[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const uint32_t w = (A >= 2) ? (u[t] >> 8) : u[t];
        const h2_t q = (A & 1) ? nib_hi_to_q(w) : nib_lo_to_q(w);
        r[t] = pk_fma(q, s2, z2);
    }
    h8_t o;
    o[0] = r[0][0]; o[1] = r[0][1]; o[2] = r[1][0]; o[3] = r[1][1];
    o[4] = r[2][0]; o[5] = r[2][1]; o[6] = r[3][0]; o[7] = r[3][1];
    return o;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
#endif  // __HIPCC__

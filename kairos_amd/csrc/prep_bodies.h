// Device-side bodies of the two preparation steps of the W8A8 lane -- int4 -> int8/fp16 weight
// conversion (one 16-byte chunk per thread) and the per-token activation quantiser (one workgroup
// per token) -- shared by their stand-alone kernels and by the fused launch that runs both at once.
#ifndef KMI_PREP_BODIES_H
#define KMI_PREP_BODIES_H
#include "kmi_common.h"

enum { OUT_F16 = 0, OUT_I8 = 1, OUT_F16_TILED = 2, OUT_I8_TILED = 3 };

__device__ __forceinline__ uint32_t pack_i8x4(h2_t a, h2_t b) {
    // truncate toward zero after clipping to the int8 range (clip first: the cast is then exact)
    const h2_t lo = {(half_t)-128.0f, (half_t)-128.0f};
    const h2_t hi = {(half_t)127.0f, (half_t)127.0f};
    a = __builtin_elementwise_min(__builtin_elementwise_max(a, lo), hi);
    b = __builtin_elementwise_min(__builtin_elementwise_max(b, lo), hi);
    const uint32_t b0 = (uint32_t)(uint8_t)(int8_t)(short)a[0];
    const uint32_t b1 = (uint32_t)(uint8_t)(int8_t)(short)a[1];
    const uint32_t b2 = (uint32_t)(uint8_t)(int8_t)(short)b[0];
    const uint32_t b3 = (uint32_t)(uint8_t)(int8_t)(short)b[1];
    return b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
}

__device__ __forceinline__ u2_t h8_to_i8x8(h8_t v) {
    h2_t p0 = {v[0], v[1]}, p1 = {v[2], v[3]}, p2 = {v[4], v[5]}, p3 = {v[6], v[7]};
    u2_t o;
    o[0] = pack_i8x4(p0, p1);
    o[1] = pack_i8x4(p2, p3);
    return o;
}

// Workgroup -> chunks, one chunk per thread.  Linear order (chunk = block*256 + thread) would make a workgroup
// convert 32 k-blocks of ONE four-row block: its output is 32 runs of 256 bytes, 8 KiB apart in the tiled layout.
// When the shape allows, a workgroup takes KMI_CVT_KB k-blocks of KMI_CVT_QB consecutive four-row blocks instead
// (QB * KB = 32): reads are runs of KB*128 bytes, writes runs of 4*QB tile rows per k-block.
#ifndef KMI_CVT_QB
#define KMI_CVT_QB 8
#endif
#define KMI_CVT_KB (32 / KMI_CVT_QB)
__device__ __forceinline__ long cvt_chunk_of(long block, int tid, int N, int K) {
    const int per_quad = K >> 3;
    if ((K % (64 * KMI_CVT_KB)) == 0 && (N % (4 * KMI_CVT_QB)) == 0) {
        const long kb_groups = K / (64 * KMI_CVT_KB);
        const long qg = block / kb_groups, kg = block - qg * kb_groups;
        const int qd = tid / (8 * KMI_CVT_KB), rest = tid % (8 * KMI_CVT_KB);   // rest = (k-block, row, half)
        return (qg * KMI_CVT_QB + qd) * per_quad + kg * (8 * KMI_CVT_KB) + rest;
    }
    return block * 256 + tid;
}

// Converts chunk i (32 weights of one row).  `out` layout by OUT; see the kernels' file header.
template <int OUT>
__device__ __forceinline__ void cvt_i4_body(long i, void* __restrict__ out, const u4_t* __restrict__ qw,
                                            const half_t* __restrict__ scales, const half_t* __restrict__ szeros,
                                            int N, int K, long total_chunks) {
    if (i >= total_chunks) return;
    const int per_quad = K >> 3;                 // 16-byte chunks per four-row block
    const int quad = (int)(i / per_quad);
    const int rem = (int)(i - (long)quad * per_quad);
    const int kb64 = rem >> 3;
    const int r = (rem >> 1) & 3;
    const int h = rem & 1;
    const int n = quad * 4 + r;
    const int k0 = kb64 * 64 + h * 32;
    const int g = k0 >> 7;

    const u4_t u = __builtin_nontemporal_load(qw + i);
    const half_t s = scales[(long)g * N + n];
    const half_t z = szeros[(long)g * N + n];
    const h2_t s2 = {s, s};
    const h2_t z2 = {z, z};
    const h8_t w0 = dequant_nibble<0>(u, s2, z2);
    const h8_t w1 = dequant_nibble<1>(u, s2, z2);
    const h8_t w2 = dequant_nibble<2>(u, s2, z2);
    const h8_t w3 = dequant_nibble<3>(u, s2, z2);

    if constexpr (OUT == OUT_F16) {
        h8_t* o = reinterpret_cast<h8_t*>(reinterpret_cast<half_t*>(out) + (long)n * K + k0);
        o[0] = w0; o[1] = w1; o[2] = w2; o[3] = w3;
    } else if constexpr (OUT == OUT_I8) {
        u4_t* o = reinterpret_cast<u4_t*>(reinterpret_cast<int8_t*>(out) + (long)n * K + k0);
        const u2_t a = h8_to_i8x8(w0), b = h8_to_i8x8(w1), c = h8_to_i8x8(w2), d = h8_to_i8x8(w3);
        u4_t lo = {a[0], a[1], b[0], b[1]};
        u4_t hi = {c[0], c[1], d[0], d[1]};
        o[0] = lo; o[1] = hi;
    } else if constexpr (OUT == OUT_F16_TILED) {
        // tile = 128 rows x 32 fp16 (8 KiB): this thread's 32 weights are exactly one tile row;
        // chunk c of row r sits at c ^ ((r>>2)&3)
        const int row = n & (KMI_TILE_N - 1);
        const long tile = (long)(n / KMI_TILE_N) * (K >> 5) + (kb64 * 2 + h);
        char* base = reinterpret_cast<char*>(out) + tile * (KMI_TILE_N * 64) + row * 64;
        const int sw = (row >> 2) & 3;
        *reinterpret_cast<h8_t*>(base + ((0 ^ sw) << 4)) = w0;
        *reinterpret_cast<h8_t*>(base + ((1 ^ sw) << 4)) = w1;
        *reinterpret_cast<h8_t*>(base + ((2 ^ sw) << 4)) = w2;
        *reinterpret_cast<h8_t*>(base + ((3 ^ sw) << 4)) = w3;
    } else {
        // tile = 128 rows x 64 int8 (8 KiB): this thread's 32 weights are half of one tile row
        const int row = n & (KMI_TILE_N - 1);
        const long tile = (long)(n / KMI_TILE_N) * (K >> 6) + kb64;
        char* base = reinterpret_cast<char*>(out) + tile * (KMI_TILE_N * 64) + row * 64;
        const int sw = (row >> 2) & 3;
        const u2_t a = h8_to_i8x8(w0), b = h8_to_i8x8(w1), c = h8_to_i8x8(w2), d = h8_to_i8x8(w3);
        u4_t lo = {a[0], a[1], b[0], b[1]};
        u4_t hi = {c[0], c[1], d[0], d[1]};
        *reinterpret_cast<u4_t*>(base + (((2 * h + 0) ^ sw) << 4)) = lo;
        *reinterpret_cast<u4_t*>(base + (((2 * h + 1) ^ sw) << 4)) = hi;
    }
}

// Eight fp16 values times the token's factor t -> eight int8: q = sat_s8(round_half_even(float(v) * t)), NaN -> 0
// (0 * inf of an all-zero token).  The conversion instruction itself maps NaN to 0 and saturates, so no compare is
// needed; the clamp to the int8 range is an integer median; v_perm gathers the low bytes.
__device__ __forceinline__ int cvt_rne_i32(float p) {
    int q;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(q) : "v"(rintf(p)));
    return q;
}
__device__ __forceinline__ u2_t quantise_h8(const h8_t& v, float t) {
    uint32_t q[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        int i = cvt_rne_i32((float)v[e] * t);
        i = i < -128 ? -128 : (i > 127 ? 127 : i);
        q[e] = (uint32_t)i;
    }
    u2_t o;
    o[0] = __builtin_amdgcn_perm(__builtin_amdgcn_perm(q[3], q[2], 0x0c0c0400u), __builtin_amdgcn_perm(q[1], q[0], 0x0c0c0400u), 0x05040100u);
    o[1] = __builtin_amdgcn_perm(__builtin_amdgcn_perm(q[7], q[6], 0x0c0c0400u), __builtin_amdgcn_perm(q[5], q[4], 0x0c0c0400u), 0x05040100u);
    return o;
}

// Absolute maximum of eight fp16 values, folded into `m` (packed fp16 maxima: NaN operands are ignored, as by fmaxf).
__device__ __forceinline__ h2_t amax_h8(h2_t m, const h8_t& v) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const h2_t a = as_h2(as_u32(h2_t{v[2 * e], v[2 * e + 1]}) & 0x7fff7fffu);
        m = __builtin_elementwise_max(m, a);
    }
    return m;
}

// Quantises one token with the whole 256-thread workgroup (CPT 16-byte chunks per thread).
template <int CPT>
__device__ __forceinline__ void quant_act_body(int token, int8_t* __restrict__ out, half_t* __restrict__ scale,
                                               const half_t* __restrict__ x, int K) {
    const int nchunk = K >> 3;
    const h8_t* row = reinterpret_cast<const h8_t*>(x + (long)token * K);
    h8_t v[CPT];
    h2_t am2 = {(half_t)0.0f, (half_t)0.0f};
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const int c = threadIdx.x + i * 256;
        if (c < nchunk) {
            v[i] = row[c];
            am2 = amax_h8(am2, v[i]);
        }
    }
    float amax = fmaxf((float)am2[0], (float)am2[1]);
    __shared__ float red[4];
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    if (threadIdx.x == 0) scale[token] = (half_t)(amax / 127.0f);
    const float t = 127.0f / amax;              // IEEE division; +inf for an all-zero token
    u2_t* orow = reinterpret_cast<u2_t*>(out + (long)token * K);
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const int c = threadIdx.x + i * 256;
        if (c < nchunk) orow[c] = quantise_h8(v[i], t);
    }
}
#endif  // KMI_PREP_BODIES_H

// On-demand weight conversion: packed uint4 (four-row interleave) -> fp16 / int8, row-major or in
// the tiled layout the MFMA GEMMs copy straight into LDS.  Pure streaming kernels: every thread
// reads one 16-byte chunk (32 weights of one row, K-contiguous after decoding) and writes 64 or 32
// contiguous bytes.  Bound by HBM bandwidth: N*K/2 bytes in, N*K*{2,1} bytes out.
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

template <int OUT>
__global__ __launch_bounds__(256) void cvt_i4_kernel(void* __restrict__ out, const u4_t* __restrict__ qw,
                                                     const half_t* __restrict__ scales,
                                                     const half_t* __restrict__ szeros, int N, int K,
                                                     long total_chunks) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
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

// tiled -> row-major (verification helper): one thread per 16-byte chunk
__global__ __launch_bounds__(256) void untile_kernel(u4_t* __restrict__ out, const u4_t* __restrict__ in, int N,
                                                     int K, int es, long total_chunks) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total_chunks) return;
    const int row_chunks = (K * es) >> 4;        // chunks per matrix row
    const int n = (int)(i / row_chunks);
    const int cg = (int)(i - (long)n * row_chunks);
    const int kt = cg >> 2, c = cg & 3;
    const int row = n & (KMI_TILE_N - 1);
    const long tile = (long)(n / KMI_TILE_N) * (row_chunks >> 2) + kt;
    out[i] = in[tile * (KMI_TILE_N * 4) + row * 4 + (c ^ ((row >> 2) & 3))];
}

static int cvt_common(const char* fn, int kind, void* out, const void* qweight, const void* scales,
                      const void* szeros, int N, int K, int G, void* stream) {
    if (!out || !qweight || !scales || !szeros) return kmi_set_error(KMI_E_NULL, "%s: NULL pointer argument", fn);
    if (!kmi_aligned16(out) || !kmi_aligned16(qweight))
        return kmi_set_error(KMI_E_ALIGN, "%s: out and qweight must be 16-byte aligned", fn);
    if (G != 128) return kmi_set_error(KMI_E_GROUP, "%s: group size %d unsupported (128 only)", fn, G);
    if (N <= 0 || K <= 0 || (N & 3) || (K & 127))
        return kmi_set_error(KMI_E_SHAPE, "%s: need N%%4==0 and K%%128==0, got N=%d K=%d", fn, N, K);
    if ((kind == OUT_F16_TILED || kind == OUT_I8_TILED) && (N % KMI_TILE_N))
        return kmi_set_error(KMI_E_SHAPE, "%s: tiled layout needs N%%%d==0, got N=%d", fn, KMI_TILE_N, N);
    const long chunks = (long)N * K / 32;
    const dim3 grid((unsigned)((chunks + 255) / 256));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const u4_t* q = static_cast<const u4_t*>(qweight);
    const half_t* s = static_cast<const half_t*>(scales);
    const half_t* z = static_cast<const half_t*>(szeros);
    switch (kind) {
        case OUT_F16: hipLaunchKernelGGL(cvt_i4_kernel<OUT_F16>, grid, dim3(256), 0, st, out, q, s, z, N, K, chunks); break;
        case OUT_I8: hipLaunchKernelGGL(cvt_i4_kernel<OUT_I8>, grid, dim3(256), 0, st, out, q, s, z, N, K, chunks); break;
        case OUT_F16_TILED: hipLaunchKernelGGL(cvt_i4_kernel<OUT_F16_TILED>, grid, dim3(256), 0, st, out, q, s, z, N, K, chunks); break;
        default: hipLaunchKernelGGL(cvt_i4_kernel<OUT_I8_TILED>, grid, dim3(256), 0, st, out, q, s, z, N, K, chunks); break;
    }
    return kmi_check_launch(fn);
}

extern "C" int kmi_cvt_i4_to_f16(void* out, const void* qw, const void* s, const void* z, int N, int K, int G, void* st) {
    return cvt_common("kmi_cvt_i4_to_f16", OUT_F16, out, qw, s, z, N, K, G, st);
}
extern "C" int kmi_cvt_i4_to_i8(void* out, const void* qw, const void* s, const void* z, int N, int K, int G, void* st) {
    return cvt_common("kmi_cvt_i4_to_i8", OUT_I8, out, qw, s, z, N, K, G, st);
}
extern "C" int kmi_cvt_i4_to_f16_tiled(void* out, const void* qw, const void* s, const void* z, int N, int K, int G, void* st) {
    return cvt_common("kmi_cvt_i4_to_f16_tiled", OUT_F16_TILED, out, qw, s, z, N, K, G, st);
}
extern "C" int kmi_cvt_i4_to_i8_tiled(void* out, const void* qw, const void* s, const void* z, int N, int K, int G, void* st) {
    return cvt_common("kmi_cvt_i4_to_i8_tiled", OUT_I8_TILED, out, qw, s, z, N, K, G, st);
}

extern "C" int kmi_untile(void* out, const void* tiled, int N, int K, int elem_size, void* stream) {
    if (!out || !tiled) return kmi_set_error(KMI_E_NULL, "kmi_untile: NULL pointer argument");
    if (!kmi_aligned16(out) || !kmi_aligned16(tiled)) return kmi_set_error(KMI_E_ALIGN, "kmi_untile: pointers must be 16-byte aligned");
    if ((elem_size != 1 && elem_size != 2) || N <= 0 || K <= 0 || (N % KMI_TILE_N) || ((K * elem_size) & 63))
        return kmi_set_error(KMI_E_SHAPE, "kmi_untile: need elem_size in {1,2}, N%%%d==0, row bytes %%64==0 (N=%d K=%d es=%d)",
                             KMI_TILE_N, N, K, elem_size);
    const long chunks = (long)N * K * elem_size / 16;
    hipLaunchKernelGGL(untile_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<u4_t*>(out), static_cast<const u4_t*>(tiled), N, K, elem_size, chunks);
    return kmi_check_launch("kmi_untile");
}

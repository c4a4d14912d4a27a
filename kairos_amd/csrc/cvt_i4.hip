// On-demand weight conversion: packed uint4 (four-row interleave) -> fp16 / int8, row-major or in
// the tiled layout the MFMA GEMMs copy straight into LDS.  Pure streaming kernels.  int8 outputs: every thread
// reads one 16-byte chunk (32 weights of one row, K-contiguous after decoding) and writes 32 contiguous bytes.
// fp16 outputs: four threads share a chunk and write 16 bytes each (with 64 bytes per thread the kernel reached
// 3.5 TB/s, with 16 it reaches 5.4).  Bound by HBM bandwidth: N*K/2 bytes in, N*K*{2,1} bytes out.
#include "prep_bodies.h"

template <int OUT>
__global__ __launch_bounds__(256) void cvt_i4_kernel(void* __restrict__ out, const u4_t* __restrict__ qw,
                                                     const half_t* __restrict__ scales,
                                                     const half_t* __restrict__ szeros, int N, int K,
                                                     long total_chunks) {
    cvt_i4_body<OUT>(cvt_chunk_of(blockIdx.x, threadIdx.x, N, K), out, qw, scales, szeros, N, K, total_chunks);
}

// fp16 outputs, one thread per 16 output bytes: the four lanes of a quad share one input chunk (one fetch) and each
// decodes the nibble plane a = lane % 4, i.e. the eight weights k = 8a .. 8a+7, so a store instruction writes runs of
// 64 (tiled) or 128 (row-major) contiguous bytes instead of 16-byte pieces 64 bytes apart.  Same arithmetic as
// dequant_nibble: the nibble, shifted down to bits 3:0, spliced under the exponent of 1024, minus 1024, is the
// exact integer q whichever plane it came from.
template <int OUT>
__global__ __launch_bounds__(256) void cvt_i4_f16_piece_kernel(void* __restrict__ out, const u4_t* __restrict__ qw,
                                                               const half_t* __restrict__ scales,
                                                               const half_t* __restrict__ szeros, int N, int K,
                                                               long total_chunks) {
    // Consecutive chunks per workgroup.  Measured alternatives, both slower: the grouped mapping of the int8 kernels
    // (+7 %), and giving every XCD a contiguous run of workgroups (+3..11 %, although it removes the repeated fetches
    // of the scale-table sectors that eight workgroups on different XCDs share: 8 % of the traffic).
    const long p = (long)blockIdx.x * 256 + threadIdx.x;
    const long i = p >> 2;
    const int a = (int)(p & 3);
    if (i >= total_chunks) return;
    const int per_quad = K >> 3;
    const int quad = (int)(i / per_quad);
    const int rem = (int)(i - (long)quad * per_quad);
    const int kb64 = rem >> 3, r = (rem >> 1) & 3, h = rem & 1;
    const int n = quad * 4 + r;
    const int k0 = kb64 * 64 + h * 32;
    const int g = k0 >> 7;
    const u4_t u = __builtin_nontemporal_load(qw + i);
    const half_t s = scales[(long)g * N + n], z = szeros[(long)g * N + n];
    const h2_t s2 = {s, s}, z2 = {z, z};
    const h2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    h2_t rr[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) rr[t] = pk_fma(as_h2(((u[t] >> (4 * a)) & 0x000F000Fu) | 0x64006400u) - k1024, s2, z2);
    const h8_t w = {rr[0][0], rr[0][1], rr[1][0], rr[1][1], rr[2][0], rr[2][1], rr[3][0], rr[3][1]};
    if constexpr (OUT == OUT_F16) {
        *reinterpret_cast<h8_t*>(reinterpret_cast<half_t*>(out) + (long)n * K + k0 + 8 * a) = w;
    } else {
        const int row = n & (KMI_TILE_N - 1);
        const long tile = (long)(n / KMI_TILE_N) * (K >> 5) + (kb64 * 2 + h);
        char* base = reinterpret_cast<char*>(out) + tile * (KMI_TILE_N * 64) + row * 64;
        *reinterpret_cast<h8_t*>(base + ((a ^ ((row >> 2) & 3)) << 4)) = w;
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
    const dim3 grid((unsigned)((chunks + 255) / 256)), grid4((unsigned)((chunks * 4 + 255) / 256));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const u4_t* q = static_cast<const u4_t*>(qweight);
    const half_t* s = static_cast<const half_t*>(scales);
    const half_t* z = static_cast<const half_t*>(szeros);
    switch (kind) {
        case OUT_F16: hipLaunchKernelGGL(cvt_i4_f16_piece_kernel<OUT_F16>, grid4, dim3(256), 0, st, out, q, s, z, N, K, chunks); break;
        case OUT_I8: hipLaunchKernelGGL(cvt_i4_kernel<OUT_I8>, grid, dim3(256), 0, st, out, q, s, z, N, K, chunks); break;
        case OUT_F16_TILED: hipLaunchKernelGGL(cvt_i4_f16_piece_kernel<OUT_F16_TILED>, grid4, dim3(256), 0, st, out, q, s, z, N, K, chunks); break;
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

// On-demand weight conversion: packed uint4 (four-row interleave) -> fp16 / int8, row-major or in
// the tiled layout the MFMA GEMMs copy straight into LDS.  Pure streaming kernels: every thread
// reads one 16-byte chunk (32 weights of one row, K-contiguous after decoding) and writes 64 or 32
// contiguous bytes.  Bound by HBM bandwidth: N*K/2 bytes in, N*K*{2,1} bytes out.
#include "prep_bodies.h"

template <int OUT>
__global__ __launch_bounds__(256) void cvt_i4_kernel(void* __restrict__ out, const u4_t* __restrict__ qw,
                                                     const half_t* __restrict__ scales,
                                                     const half_t* __restrict__ szeros, int N, int K,
                                                     long total_chunks) {
    cvt_i4_body<OUT>(cvt_chunk_of(blockIdx.x, threadIdx.x, N, K), out, qw, scales, szeros, N, K, total_chunks);
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

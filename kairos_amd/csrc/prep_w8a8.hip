// One launch for both preparation steps of the W8A8 lane: the first M workgroups quantise one token
// each, the others convert the packed int4 weight to int8 (one 16-byte chunk per thread).  The two
// jobs are independent and both stream HBM, so sharing a launch saves a kernel boundary (launch gap,
// ramp-up and drain) on every call that has to convert.  Results are bit-identical to the two
// stand-alone kernels: the same device functions run.
#include "prep_bodies.h"

template <int OUT, int CPT>
__global__ __launch_bounds__(256) void prep_w8a8_kernel(void* __restrict__ w8, const u4_t* __restrict__ qw,
                                                        const half_t* __restrict__ scales,
                                                        const half_t* __restrict__ szeros, int N, int K,
                                                        long total_chunks, int8_t* __restrict__ a8,
                                                        half_t* __restrict__ ascale, const half_t* __restrict__ x,
                                                        int M) {
    if ((int)blockIdx.x < M) {                   // workgroup-uniform: the barrier inside is safe
        quant_act_body<CPT>(blockIdx.x, a8, ascale, x, K);
        return;
    }
    cvt_i4_body<OUT>(cvt_chunk_of((long)blockIdx.x - M, threadIdx.x, N, K), w8, qw, scales, szeros, N, K, total_chunks);
}

template <int OUT>
static void launch_prep(int cpt, dim3 grid, hipStream_t st, void* w8, const u4_t* q, const half_t* s, const half_t* z,
                        int N, int K, long chunks, int8_t* a8, half_t* as, const half_t* x, int M) {
    if (cpt <= 1) hipLaunchKernelGGL((prep_w8a8_kernel<OUT, 1>), grid, dim3(256), 0, st, w8, q, s, z, N, K, chunks, a8, as, x, M);
    else if (cpt <= 2) hipLaunchKernelGGL((prep_w8a8_kernel<OUT, 2>), grid, dim3(256), 0, st, w8, q, s, z, N, K, chunks, a8, as, x, M);
    else if (cpt <= 4) hipLaunchKernelGGL((prep_w8a8_kernel<OUT, 4>), grid, dim3(256), 0, st, w8, q, s, z, N, K, chunks, a8, as, x, M);
    else if (cpt <= 8) hipLaunchKernelGGL((prep_w8a8_kernel<OUT, 8>), grid, dim3(256), 0, st, w8, q, s, z, N, K, chunks, a8, as, x, M);
    else hipLaunchKernelGGL((prep_w8a8_kernel<OUT, 16>), grid, dim3(256), 0, st, w8, q, s, z, N, K, chunks, a8, as, x, M);
}

extern "C" int kmi_prep_w8a8(void* w8_out, int tiled, const void* qweight, const void* scales_to8,
                             const void* scaled_zeros_to8, int N, int K, int G, void* a8_out, void* ascale_f16,
                             const void* x_f16, int M, void* stream) {
    const char* fn = "kmi_prep_w8a8";
    if (!w8_out || !qweight || !scales_to8 || !scaled_zeros_to8 || !a8_out || !ascale_f16 || !x_f16)
        return kmi_set_error(KMI_E_NULL, "%s: NULL pointer argument", fn);
    if (!kmi_aligned16(w8_out) || !kmi_aligned16(qweight) || !kmi_aligned16(a8_out) || !kmi_aligned16(x_f16))
        return kmi_set_error(KMI_E_ALIGN, "%s: w8_out, qweight, a8_out and x must be 16-byte aligned", fn);
    if (G != 128) return kmi_set_error(KMI_E_GROUP, "%s: group size %d unsupported (128 only)", fn, G);
    if (N <= 0 || K <= 0 || (N & 3) || (K & 127) || K > 32768)
        return kmi_set_error(KMI_E_SHAPE, "%s: need N%%4==0, K%%128==0, K<=32768, got N=%d K=%d", fn, N, K);
    if (tiled && (N % KMI_TILE_N))
        return kmi_set_error(KMI_E_SHAPE, "%s: tiled layout needs N%%%d==0, got N=%d", fn, KMI_TILE_N, N);
    if (M < 0) return kmi_set_error(KMI_E_SHAPE, "%s: need M>=0, got %d", fn, M);
    const long chunks = (long)N * K / 32;
    const dim3 grid((unsigned)M + (unsigned)((chunks + 255) / 256));
    const int cpt = ((K >> 3) + 255) / 256;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const u4_t* q = static_cast<const u4_t*>(qweight);
    const half_t* s = static_cast<const half_t*>(scales_to8);
    const half_t* z = static_cast<const half_t*>(scaled_zeros_to8);
    int8_t* a8 = static_cast<int8_t*>(a8_out);
    half_t* as = static_cast<half_t*>(ascale_f16);
    const half_t* x = static_cast<const half_t*>(x_f16);
    if (tiled) launch_prep<OUT_I8_TILED>(cpt, grid, st, w8_out, q, s, z, N, K, chunks, a8, as, x, M);
    else launch_prep<OUT_I8>(cpt, grid, st, w8_out, q, s, z, N, K, chunks, a8, as, x, M);
    return kmi_check_launch(fn);
}

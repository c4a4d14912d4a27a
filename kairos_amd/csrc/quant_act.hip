// Fused per-token activation quantiser: one workgroup per token, the row is read ONCE into
// registers, reduced to its absolute maximum (wave shuffles + LDS), and written as int8 plus an
// fp16 scale.  Algorithmic traffic: 2*M*K bytes in, M*K + 2*M bytes out.
#include "kmi_common.h"

template <int CPT>   // 16-byte chunks (8 fp16) per thread; the block covers 256*CPT*8 columns
__global__ __launch_bounds__(256) void quant_act_kernel(int8_t* __restrict__ out, half_t* __restrict__ scale,
                                                        const half_t* __restrict__ x, int K) {
    const int token = blockIdx.x;
    const int nchunk = K >> 3;
    const h8_t* row = reinterpret_cast<const h8_t*>(x + (long)token * K);
    h8_t v[CPT];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const int c = threadIdx.x + i * 256;
        if (c < nchunk) {
            v[i] = row[c];
#pragma unroll
            for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf((float)v[i][e]));
        }
    }
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
        if (c < nchunk) {
            uint32_t b[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float p = (float)v[i][e] * t;
                p = (p != p) ? 0.0f : p;        // 0 * inf
                p = fminf(fmaxf(rintf(p), -128.0f), 127.0f);
                b[e] = (uint32_t)(uint8_t)(int8_t)(int)p;
            }
            u2_t o;
            o[0] = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
            o[1] = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
            orow[c] = o;
        }
    }
}

extern "C" int kmi_quant_act_i8(void* out_i8, void* scale_f16, const void* x_f16, int M, int K, void* stream) {
    if (!out_i8 || !scale_f16 || !x_f16) return kmi_set_error(KMI_E_NULL, "kmi_quant_act_i8: NULL pointer argument");
    if (!kmi_aligned16(out_i8) || !kmi_aligned16(x_f16))
        return kmi_set_error(KMI_E_ALIGN, "kmi_quant_act_i8: out and x must be 16-byte aligned");
    if (M < 0 || K <= 0 || (K & 7) || K > 32768)
        return kmi_set_error(KMI_E_SHAPE, "kmi_quant_act_i8: need M>=0, K%%8==0, K<=32768 (M=%d K=%d)", M, K);
    if (M == 0) return KMI_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int8_t* o = static_cast<int8_t*>(out_i8);
    half_t* s = static_cast<half_t*>(scale_f16);
    const half_t* x = static_cast<const half_t*>(x_f16);
    const int cpt = ((K >> 3) + 255) / 256;
    const dim3 grid(M), block(256);
    if (cpt <= 1) hipLaunchKernelGGL(quant_act_kernel<1>, grid, block, 0, st, o, s, x, K);
    else if (cpt <= 2) hipLaunchKernelGGL(quant_act_kernel<2>, grid, block, 0, st, o, s, x, K);
    else if (cpt <= 4) hipLaunchKernelGGL(quant_act_kernel<4>, grid, block, 0, st, o, s, x, K);
    else if (cpt <= 8) hipLaunchKernelGGL(quant_act_kernel<8>, grid, block, 0, st, o, s, x, K);
    else hipLaunchKernelGGL(quant_act_kernel<16>, grid, block, 0, st, o, s, x, K);
    return kmi_check_launch("kmi_quant_act_i8");
}

// Fused per-token activation quantiser: one workgroup per token, the row is read ONCE into
// registers, reduced to its absolute maximum (wave shuffles + LDS), and written as int8 plus an
// fp16 scale.  Algorithmic traffic: 2*M*K bytes in, M*K + 2*M bytes out.
#include "prep_bodies.h"

template <int CPT>   // 16-byte chunks (8 fp16) per thread; the block covers 256*CPT*8 columns
__global__ __launch_bounds__(256) void quant_act_kernel(int8_t* __restrict__ out, half_t* __restrict__ scale,
                                                        const half_t* __restrict__ x, int K) {
    quant_act_body<CPT>(blockIdx.x, out, scale, x, K);
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

// The operators in front of a switched linear, fused with the per-token activation quantiser.  Second half of the
// file: SiLU(gate) * up in front of the down projection.  First half:
// RMSNorm (optionally behind a residual add) fused with the per-token activation quantiser: the operator in front
// of a switched linear layer emits the activation format its consumer's lane needs -- fp16, int8 + per-token scale,
// or both -- from ONE read of the hidden state.  One workgroup per token; the row lives in registers between the
// three phases (sum of squares, normalise + absolute maximum, quantise).
//
// Arithmetic, in the order of the eager PyTorch modules this replaces (every intermediate rounded as there):
//   h      = fp16(x + residual)                                  (only with a residual; also written back)
//   var    = (sum_k float(h)^2) / float(K)                        fp32; the squares are exact, the sum runs per thread
//                                                                over its chunks in order, then a butterfly over the
//                                                                wave (xor 32, 16, .., 1), then (w0 + w1) + (w2 + w3)
//   r      = 1.0f / sqrtf(var + eps)                              both correctly rounded
//   y      = fp16(float(gamma) * float(fp16(float(h) * r)))
//   int8   = the per-token quantiser of quant_act_body applied to y
// Algorithmic traffic: 2*M*K bytes in (4*M*K with a residual, plus 2*M*K for the updated one), 2*K for gamma,
// and M*K + 2*M (int8) and / or 2*M*K (fp16) out.
#include "prep_bodies.h"

__device__ __forceinline__ float wave_sum_butterfly(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = v + __shfl_xor(v, off, 64);
    return v;
}

// One workgroup per token; thread t owns the 8-element chunks t, t + 256, ..  (One wave per token, which needs no
// barrier, was measured too: 5 % faster with int8 output only, 6-15 % slower with fp16 output.)
template <int CPT>
__global__ __launch_bounds__(256) void rmsnorm_quant_kernel(int8_t* __restrict__ a8, half_t* __restrict__ ascale,
                                                            half_t* __restrict__ y_out, half_t* __restrict__ h_out,
                                                            const half_t* __restrict__ x,
                                                            const half_t* __restrict__ residual,
                                                            const half_t* __restrict__ gamma, float eps, int K) {
    constexpr int TPT = 256;
    const int tid = threadIdx.x;
    const int token = blockIdx.x;
    const int nchunk = K >> 3;
    const long row0 = (long)token * K;
    const h8_t* xr = reinterpret_cast<const h8_t*>(x + row0);
    const h8_t* rr = residual ? reinterpret_cast<const h8_t*>(residual + row0) : nullptr;
    const h8_t* gr = reinterpret_cast<const h8_t*>(gamma);
    __shared__ float red_ss[4], red_amax[4];

    h8_t v[CPT];
#pragma unroll
    for (int i = 0; i < CPT; ++i) {                            // every load of the row is in flight before the first use
        const int c = tid + i * TPT;
        if (c < nchunk) v[i] = xr[c];
    }
    if (rr) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = tid + i * TPT;
            if (c < nchunk) {
                v[i] = v[i] + rr[c];                           // fp16 adds, one rounding each
                if (h_out) reinterpret_cast<h8_t*>(h_out + row0)[c] = v[i];
            }
        }
    }
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const int c = tid + i * TPT;
        if (c < nchunk) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float f = (float)v[i][e];
                ss = __builtin_fmaf(f, f, ss);                 // f*f is exact in fp32: the same as multiply, then add
            }
        }
    }
    ss = wave_sum_butterfly(ss);
    if ((threadIdx.x & 63) == 0) red_ss[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float total = (red_ss[0] + red_ss[1]) + (red_ss[2] + red_ss[3]);
    const float r = 1.0f / sqrtf(total / (float)K + eps);

    h2_t am2 = {(half_t)0.0f, (half_t)0.0f};
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const int c = tid + i * TPT;
        if (c < nchunk) {
            h8_t t;
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] = (half_t)((float)v[i][e] * r);
            v[i] = gr[c] * t;                                  // fp16 products: the rounding of the exact product
            am2 = amax_h8(am2, v[i]);
            if (y_out) reinterpret_cast<h8_t*>(y_out + row0)[c] = v[i];
        }
    }
    if (!a8) return;                                           // uniform over the grid

    float amax = wave_max(fmaxf((float)am2[0], (float)am2[1]));
    if ((threadIdx.x & 63) == 0) red_amax[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red_amax[0], red_amax[1]), fmaxf(red_amax[2], red_amax[3]));
    if (tid == 0) ascale[token] = (half_t)(amax / 127.0f);
    const float t = 127.0f / amax;                             // IEEE division; +inf for an all-zero token
    u2_t* orow = reinterpret_cast<u2_t*>(a8 + row0);
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const int c = tid + i * TPT;
        if (c < nchunk) orow[c] = quantise_h8(v[i], t);
    }
}

extern "C" int kmi_rmsnorm_quant_act(void* a8_out, void* ascale_f16, void* y_f16_out, void* h_f16_out,
                                     const void* x_f16, const void* residual_f16, const void* gamma_f16, float eps,
                                     int M, int K, void* stream) {
    const char* fn = "kmi_rmsnorm_quant_act";
    if (!x_f16 || !gamma_f16) return kmi_set_error(KMI_E_NULL, "%s: x and gamma must not be NULL", fn);
    if (!a8_out && !y_f16_out) return kmi_set_error(KMI_E_NULL, "%s: at least one of a8_out, y_f16_out is needed", fn);
    if (a8_out && !ascale_f16) return kmi_set_error(KMI_E_NULL, "%s: a8_out needs ascale_f16", fn);
    if (h_f16_out && !residual_f16) return kmi_set_error(KMI_E_NULL, "%s: h_f16_out is only written with a residual", fn);
    if (!kmi_aligned16(a8_out) || !kmi_aligned16(y_f16_out) || !kmi_aligned16(h_f16_out) || !kmi_aligned16(x_f16) ||
        !kmi_aligned16(residual_f16) || !kmi_aligned16(gamma_f16))
        return kmi_set_error(KMI_E_ALIGN, "%s: every tensor must be 16-byte aligned", fn);
    if (M < 0 || K <= 0 || (K & 7) || K > 32768)
        return kmi_set_error(KMI_E_SHAPE, "%s: need M>=0, K%%8==0, K<=32768 (M=%d K=%d)", fn, M, K);
    if (!(eps >= 0.0f)) return kmi_set_error(KMI_E_SHAPE, "%s: eps must be >= 0", fn);
    if (M == 0) return KMI_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int8_t* a8 = static_cast<int8_t*>(a8_out);
    half_t* as = static_cast<half_t*>(ascale_f16);
    half_t* y = static_cast<half_t*>(y_f16_out);
    half_t* h = static_cast<half_t*>(h_f16_out);
    const half_t* x = static_cast<const half_t*>(x_f16);
    const half_t* res = static_cast<const half_t*>(residual_f16);
    const half_t* g = static_cast<const half_t*>(gamma_f16);
    const int cpt = ((K >> 3) + 255) / 256;
    const dim3 grid(M), block(256);
#define KMI_NORM_LAUNCH(C) hipLaunchKernelGGL(rmsnorm_quant_kernel<C>, grid, block, 0, st, a8, as, y, h, x, res, g, eps, K)
    if (cpt <= 1) KMI_NORM_LAUNCH(1);
    else if (cpt <= 2) KMI_NORM_LAUNCH(2);
    else if (cpt <= 4) KMI_NORM_LAUNCH(4);
    else if (cpt <= 8) KMI_NORM_LAUNCH(8);
    else KMI_NORM_LAUNCH(16);
#undef KMI_NORM_LAUNCH
    return kmi_check_launch(fn);
}

// ---- SiLU(gate) * up in front of the down projection --------------------------------------------------------------
// gate_up [M, 2*I] fp16 (gate in columns 0..I-1, up in I..2I-1, the output of the fused gate/up linear):
//   s = fp16(g / (1 + exp(-g)))  evaluated in fp32;   y = fp16(float(s) * float(u));   int8 = quantiser of y.
// The exponential and the reciprocal are the hardware approximations (about 1e-7 relative, four thousand times finer
// than the fp16 rounding that follows), so s can differ from a correctly rounded evaluation by one fp16 step (y by two)
// on roughly one element in a thousand; the int8 output is exactly the quantiser applied to the y this kernel produces.
// One workgroup per token, the row of products stays in registers between the two phases.
// Algorithmic traffic: 4*M*I bytes in, M*I + 2*M (int8) and / or 2*M*I (fp16) out.
template <int CPT>
__global__ __launch_bounds__(256) void silu_mul_quant_kernel(int8_t* __restrict__ a8, half_t* __restrict__ ascale,
                                                             half_t* __restrict__ y_out,
                                                             const half_t* __restrict__ gate_up, int I) {
    const int token = blockIdx.x;
    const int nchunk = I >> 3;
    const h8_t* gr = reinterpret_cast<const h8_t*>(gate_up + (long)token * 2 * I);
    const h8_t* ur = reinterpret_cast<const h8_t*>(gate_up + (long)token * 2 * I + I);
    __shared__ float red_amax[4];

    h8_t v[CPT], u[CPT];
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const int c = threadIdx.x + i * 256;
        if (c < nchunk) { v[i] = gr[c]; u[i] = ur[c]; }
    }
    h2_t am2 = {(half_t)0.0f, (half_t)0.0f};
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const int c = threadIdx.x + i * 256;
        if (c < nchunk) {
            h8_t sg;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float g = (float)v[i][e];
                sg[e] = (half_t)(g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)));
            }
            v[i] = sg * u[i];                                  // fp16 products: the rounding of the exact product
            am2 = amax_h8(am2, v[i]);
            if (y_out) reinterpret_cast<h8_t*>(y_out + (long)token * I)[c] = v[i];
        }
    }
    if (!a8) return;                                           // uniform over the grid

    float amax = wave_max(fmaxf((float)am2[0], (float)am2[1]));
    if ((threadIdx.x & 63) == 0) red_amax[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red_amax[0], red_amax[1]), fmaxf(red_amax[2], red_amax[3]));
    if (threadIdx.x == 0) ascale[token] = (half_t)(amax / 127.0f);
    const float t = 127.0f / amax;                             // IEEE division; +inf for an all-zero token
    u2_t* orow = reinterpret_cast<u2_t*>(a8 + (long)token * I);
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        const int c = threadIdx.x + i * 256;
        if (c < nchunk) orow[c] = quantise_h8(v[i], t);
    }
}

extern "C" int kmi_silu_mul_quant_act(void* a8_out, void* ascale_f16, void* y_f16_out, const void* gate_up_f16, int M,
                                      int I, void* stream) {
    const char* fn = "kmi_silu_mul_quant_act";
    if (!gate_up_f16) return kmi_set_error(KMI_E_NULL, "%s: gate_up must not be NULL", fn);
    if (!a8_out && !y_f16_out) return kmi_set_error(KMI_E_NULL, "%s: at least one of a8_out, y_f16_out is needed", fn);
    if (a8_out && !ascale_f16) return kmi_set_error(KMI_E_NULL, "%s: a8_out needs ascale_f16", fn);
    if (!kmi_aligned16(a8_out) || !kmi_aligned16(y_f16_out) || !kmi_aligned16(gate_up_f16))
        return kmi_set_error(KMI_E_ALIGN, "%s: every tensor must be 16-byte aligned", fn);
    if (M < 0 || I <= 0 || (I & 7) || I > 32768)
        return kmi_set_error(KMI_E_SHAPE, "%s: need M>=0, I%%8==0, I<=32768 (M=%d I=%d)", fn, M, I);
    if (M == 0) return KMI_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int8_t* a8 = static_cast<int8_t*>(a8_out);
    half_t* as = static_cast<half_t*>(ascale_f16);
    half_t* y = static_cast<half_t*>(y_f16_out);
    const half_t* gu = static_cast<const half_t*>(gate_up_f16);
    const int cpt = ((I >> 3) + 255) / 256;
    const dim3 grid(M), block(256);
#define KMI_SILU_LAUNCH(C) hipLaunchKernelGGL(silu_mul_quant_kernel<C>, grid, block, 0, st, a8, as, y, gu, I)
    if (cpt <= 1) KMI_SILU_LAUNCH(1);
    else if (cpt <= 2) KMI_SILU_LAUNCH(2);
    else if (cpt <= 4) KMI_SILU_LAUNCH(4);
    else if (cpt <= 8) KMI_SILU_LAUNCH(8);
    else KMI_SILU_LAUNCH(16);
#undef KMI_SILU_LAUNCH
    return kmi_check_launch(fn);
}

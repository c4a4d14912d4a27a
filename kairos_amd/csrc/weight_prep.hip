// Offline weight preparation on the device: fp16 [N, K] -> per-channel int8 -> per-group asymmetric
// uint4 with an unrounded float zero-point -> the resident packed int4 words and the four [Gp, N]
// scale tables, all in one launch.  Replaces the torch chain of DynamicLinear.from_module
// (kairos/dynamic_linear.py:86-115): quantize_tensor_int8 (kairos/quantization.py:112-141),
// kairos_quantize_tensor_int4 (kairos/dynamic_linear_v2.py:15-41), pack_int_awq and
// trans_qfactor_layout_awq (thirdparty/AWQ/awq_method.py:5-75).
//
// Every arithmetic step is the IEEE fp32 (or fp16) operation of the torch chain, in its order:
//   s1 = max(amax|w|, 1e-7) / 127            w8 = rint(w / s1)
//   s2 = max(hi - lo, 1e-5) / 15             z2 = -(lo / s2)           q = clamp(rint(w8 / s2 + z2), 0, 15)
//   scales_to8 = fp16(s2)                    scaled_zeros_to8 = -fp16(fp32(fp16 s2) * fp32(fp16 z2))
//   scales     = fp16(s2) *_f16 fp16(s1)     scaled_zeros     = -fp16(fp32(scales) * fp32(fp16 z2))
// Divisions are correctly rounded and no step can be contracted into an FMA (every sum follows a division), so the
// results equal the host chain bit for bit.  The 8 + 8 divisions per load share two divisors (s1 per row, s2 per
// group), so they run the fp32 division sequence by hand with its divisor-only half hoisted: r = rcp(d) refined once,
// then q = x*r and two residual corrections q += (x - d*q)*r in FMAs -- the sequence the compiler emits for `/`,
// without the operand pre-scaling that only matters for exponents these values cannot have (|x/d| <= 2^7 here,
// d in [1e-10, 1e3]); a zero numerator may come out with the other sign, which the integer conversion and the sum
// with the zero-point erase.
//
// One workgroup per four-row block (the packing unit), one wave per row.  A row of up to 16384 weights is read once
// and held in registers across the two passes (amax, then quantise); longer rows are read twice.  A 16-byte load is
// 8 weights of one row; 16 lanes
// hold one group of 128, 4 lanes one packed 16-byte chunk (32 weights: word t, nibble a, half c holds
// k = 8a + 2t + c), so lane a of a chunk owns nibble a of all four words and, after an OR across the
// four lanes, stores word a.
#include "kmi_common.h"

// cross-lane moves inside a row of 16 lanes: quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
__device__ __forceinline__ float group16_max(float v) {     // after each step all lanes of the reduced span agree,
    v = fmaxf(v, dpp_f<0xB1>(v));                           // so the mirrors act as the xor-4 and xor-8 exchanges
    v = fmaxf(v, dpp_f<0x4E>(v));
    v = fmaxf(v, dpp_f<0x141>(v));
    return fmaxf(v, dpp_f<0x140>(v));
}
__device__ __forceinline__ float group16_min(float v) {
    v = fminf(v, dpp_f<0xB1>(v));
    v = fminf(v, dpp_f<0x4E>(v));
    v = fminf(v, dpp_f<0x141>(v));
    return fminf(v, dpp_f<0x140>(v));
}

// divisor-only half of the division sequence: rcp refined once
__device__ __forceinline__ float refined_rcp(float d) {
    const float r = __builtin_amdgcn_rcpf(d);
    return __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
}
// x / d, correctly rounded, r = refined_rcp(d)
__device__ __forceinline__ float div_by(float x, float d, float r) {
    float q = x * r;
    q = __builtin_fmaf(__builtin_fmaf(-d, q, x), r, q);
    return __builtin_fmaf(__builtin_fmaf(-d, q, x), r, q);
}

// CPL > 0: the row (up to 64 * CPL 16-byte chunks) is loaded once and stays in registers between the two passes;
// CPL == 0: rows longer than that are read twice, the second time through a one-deep prefetch.
template <int CPL>
__global__ __launch_bounds__(256) void prepare_weight_kernel(const half_t* __restrict__ w, int N, int K, int Gp,
                                                             uint32_t* __restrict__ qweight,
                                                             half_t* __restrict__ scales,
                                                             half_t* __restrict__ szeros,
                                                             half_t* __restrict__ scales8,
                                                             half_t* __restrict__ szeros8,
                                                             half_t* __restrict__ scales1) {
    const int quad = blockIdx.x, r = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n = quad * 4 + r;
    const h8_t* row = reinterpret_cast<const h8_t*>(w + (long)n * K);
    const int nch = K >> 3;                      // 16-byte loads per row; a multiple of 16 (K % 128 == 0)
    const int ng = K >> 7;

    constexpr int HELD = CPL > 0 ? CPL : 1;
    h8_t held[HELD];
    float amax = 0.0f;
    if constexpr (CPL > 0) {
#pragma unroll
        for (int i = 0; i < CPL; ++i)
            if (i * 64 < nch) held[i] = row[min(lane + 64 * i, nch - 1)];             // repeats are harmless
#pragma unroll
        for (int i = 0; i < CPL; ++i)
            if (i * 64 < nch) {
#pragma unroll
                for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf((float)held[i][e]));
            }
    } else {
        for (int base = lane; base < nch; base += 256) {   // four independent loads in flight; repeats are harmless
            h8_t v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = row[min(base + 64 * u, nch - 1)];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf((float)v[u][e]));
        }
    }
    amax = fmaxf(wave_max(amax), 1e-7f);
    const float s1 = amax / 127.0f;
    const half_t s1h = (half_t)s1;
    if (lane == 0) scales1[n] = s1h;

    uint32_t* qrow = qweight + (long)quad * (K >> 3) * 4;      // this four-row block: K/8 chunks of 4 words
    const float r1 = refined_rcp(s1);
    auto quantise_chunk = [&](int base, const h8_t& v) {
        const int c = base + lane;
        const bool valid = c < nch;              // uniform over each group of 16 lanes
        float x[8];
        float hi = -INFINITY, lo = INFINITY;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            x[e] = (float)(int)rintf(div_by((float)v[e], s1, r1));   // through the integer, as the int8 tensor of step 1: -0 -> +0
            hi = fmaxf(hi, x[e]);
            lo = fminf(lo, x[e]);
        }
        hi = group16_max(hi);
        lo = group16_min(lo);
        const float s2 = fmaxf(hi - lo, 1e-5f) / 15.0f;
        const float r2 = refined_rcp(s2);
        const float z2 = -div_by(lo, s2, r2);
        uint32_t word[4];
        const int a = lane & 3;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float q0 = fminf(fmaxf(rintf(div_by(x[2 * t], s2, r2) + z2), 0.0f), 15.0f);
            const float q1 = fminf(fmaxf(rintf(div_by(x[2 * t + 1], s2, r2) + z2), 0.0f), 15.0f);
            word[t] = ((uint32_t)q0 | ((uint32_t)q1 << 16)) << (4 * a);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            word[t] |= dpp_u<0xB1>(word[t]);
            word[t] |= dpp_u<0x4E>(word[t]);
        }
        const uint32_t mine = a == 0 ? word[0] : a == 1 ? word[1] : a == 2 ? word[2] : word[3];
        if (valid) {
            const int chunk = c >> 2;            // 32 weights: k0 = 32 * chunk
            const int kb64 = chunk >> 1, h = chunk & 1;
            qrow[((long)kb64 * 8 + r * 2 + h) * 4 + a] = mine;
            if ((lane & 15) == 0) {
                const int g = c >> 4;
                const half_t s2h = (half_t)s2, z2h = (half_t)z2;
                const half_t sf = (half_t)((float)s2h * (float)s1h);       // exact product, one rounding
                const long at = (long)g * N + n;
                scales8[at] = s2h;
                szeros8[at] = -(half_t)((float)s2h * (float)z2h);
                scales[at] = sf;
                szeros[at] = -(half_t)((float)sf * (float)z2h);
            }
        }
    };
    if constexpr (CPL > 0) {
#pragma unroll
        for (int i = 0; i < CPL; ++i)
            if (i * 64 < nch) quantise_chunk(i * 64, held[i]);       // wave-uniform
    } else {
        h8_t nxt = row[min(lane, nch - 1)];
        for (int base = 0; base < nch; base += 64) {
            const h8_t v = nxt;
            nxt = row[min(base + lane + 64, nch - 1)];
            quantise_chunk(base, v);
        }
    }
    for (int g = ng + lane; g < Gp; g += 64) {   // padded table rows are zero
        const long at = (long)g * N + n;
        scales8[at] = (half_t)0.0f;
        szeros8[at] = (half_t)0.0f;
        scales[at] = (half_t)0.0f;
        szeros[at] = (half_t)0.0f;
    }
}

extern "C" int kmi_padded_groups(int K, int G) {
    if (G != 128 || K <= 0 || (K % G)) return kmi_set_error(KMI_E_SHAPE, "kmi_padded_groups: need G==128 and K%%G==0, got K=%d G=%d", K, G);
    return ((K / G + 7) / 8) * 8;
}

extern "C" int kmi_prepare_weight(const void* w_f16, int N, int K, int G, void* qweight, void* scales,
                                  void* scaled_zeros, void* scales_to8, void* scaled_zeros_to8, void* scales_1,
                                  void* stream) {
    const char* fn = "kmi_prepare_weight";
    if (!w_f16 || !qweight || !scales || !scaled_zeros || !scales_to8 || !scaled_zeros_to8 || !scales_1)
        return kmi_set_error(KMI_E_NULL, "%s: NULL pointer argument", fn);
    if (!kmi_aligned16(w_f16) || !kmi_aligned16(qweight))
        return kmi_set_error(KMI_E_ALIGN, "%s: w_f16 and qweight must be 16-byte aligned", fn);
    if (G != 128) return kmi_set_error(KMI_E_GROUP, "%s: group size %d unsupported (128 only)", fn, G);
    if (N <= 0 || K <= 0 || (N & 3) || (K & 127))
        return kmi_set_error(KMI_E_SHAPE, "%s: need N%%4==0 and K%%128==0, got N=%d K=%d", fn, N, K);
    const int Gp = ((K / G + 7) / 8) * 8;
    const int cpl = (K / 8 + 63) / 64;              // 16-byte chunks per lane of the wave that owns a row
#define KMI_PREP_LAUNCH(C)                                                                                              \
    hipLaunchKernelGGL(prepare_weight_kernel<C>, dim3((unsigned)(N / 4)), dim3(256), 0, static_cast<hipStream_t>(stream), \
                       static_cast<const half_t*>(w_f16), N, K, Gp, static_cast<uint32_t*>(qweight),                     \
                       static_cast<half_t*>(scales), static_cast<half_t*>(scaled_zeros), static_cast<half_t*>(scales_to8), \
                       static_cast<half_t*>(scaled_zeros_to8), static_cast<half_t*>(scales_1))
    if (cpl <= 8) KMI_PREP_LAUNCH(8);
    else if (cpl <= 16) KMI_PREP_LAUNCH(16);
    else if (cpl <= 32) KMI_PREP_LAUNCH(32);
    else KMI_PREP_LAUNCH(0);
#undef KMI_PREP_LAUNCH
    return kmi_check_launch(fn);
}

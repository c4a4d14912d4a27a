// Measurement aid, not on the product path: the rate a register-only loop of the two MFMA instructions of this
// library sustains on the whole GPU, with constant or with random operands.  The matrix pipes draw power by the
// bits that toggle, and under full-chip MFMA load the shader clock settles where the power limit puts it; this
// probe gives the ceiling any GEMM kernel can reach on realistic data, beside the published peak.
#include "kmi_common.h"

template <bool I8>
__global__ __launch_bounds__(256) void probe_mfma_kernel(const i4_t* __restrict__ in, float* __restrict__ out,
                                                         long long* __restrict__ clk, int iters) {
    i4_t a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a[i] = in[threadIdx.x + 256 * i];
        b[i] = in[threadIdx.x + 256 * (4 + i)];
    }
    const long long c0 = clock64(), w0 = wall_clock64();
    float s = 0.0f;
    if constexpr (I8) {
        i16_t acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][e] = 0;
        for (int it = 0; it < iters; ++it)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i * 4 + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i * 4 + j], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) s += (float)acc[i][e];
    } else {
        f16_t acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][e] = 0.0f;
        for (int it = 0; it < iters; ++it)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8_t, a[i]), __builtin_bit_cast(h8_t, b[j]),
                                                                            acc[i * 4 + j], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) s += acc[i][e];
    }
    out[blockIdx.x * 256 + threadIdx.x] = s;                   // keeps the loop alive
    const long long c1 = clock64(), w1 = wall_clock64();
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        clk[0] = c1 - c0;                                      // shader clocks
        clk[1] = w1 - w0;                                      // constant 100 MHz counter
    }
}

extern "C" int kmi_probe_mfma(int int8, const void* operands_32k, void* sink_f32, void* clocks_2xi64, int workgroups,
                              int iters, void* stream) {
    const char* fn = "kmi_probe_mfma";
    if (!operands_32k || !sink_f32 || !clocks_2xi64) return kmi_set_error(KMI_E_NULL, "%s: NULL pointer argument", fn);
    if (!kmi_aligned16(operands_32k)) return kmi_set_error(KMI_E_ALIGN, "%s: operands must be 16-byte aligned", fn);
    if (workgroups <= 0 || iters <= 0) return kmi_set_error(KMI_E_SHAPE, "%s: need workgroups > 0 and iters > 0", fn);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const i4_t* in = static_cast<const i4_t*>(operands_32k);
    float* out = static_cast<float*>(sink_f32);
    long long* clk = static_cast<long long*>(clocks_2xi64);
    if (int8) hipLaunchKernelGGL(probe_mfma_kernel<true>, dim3(workgroups), dim3(256), 0, st, in, out, clk, iters);
    else hipLaunchKernelGGL(probe_mfma_kernel<false>, dim3(workgroups), dim3(256), 0, st, in, out, clk, iters);
    return kmi_check_launch(fn);
}

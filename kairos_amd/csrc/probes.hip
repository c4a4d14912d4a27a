// Measurement probes.  Kernels that only read, for the floors that the streaming kernels of the library are measured
// against (an empty launch, a plain contiguous reader, and a reader that issues exactly the weight loads of the
// small-M W4A16 kernel and nothing else), and register-only loops on the matrix and vector pipes: what the MFMAs sustain
// on the whole chip under its power limit, and how the two pipes of a SIMD share one wave or two.  No product path calls
// them; `python -m kairos_amd.bench_extra floor` and `... pipes` do.
#include "kmi_common.h"

// volatile and with external linkage: a sink that nothing reads would let the compiler drop the stores to it, and with them
// every load of the probes
__device__ volatile uint32_t g_probe_sink;

__global__ void probe_empty_kernel() {
    if (threadIdx.x == 9999) g_probe_sink = 1;
}

// every workgroup reads 256 * 16 * UNR contiguous bytes, all loads issued before the first use
template <int UNR>
__global__ __launch_bounds__(256) void probe_read_kernel(const u4_t* __restrict__ in, long n16) {
    const long i = (long)blockIdx.x * 256 * UNR + threadIdx.x;
    u4_t acc = {0, 0, 0, 0};
    u4_t v[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) v[u] = (i + u * 256 < n16) ? __builtin_nontemporal_load(in + i + u * 256) : acc;
#pragma unroll
    for (int u = 0; u < UNR; ++u) acc ^= v[u];
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345u) g_probe_sink = 1;
}

// The weight loads of the small-M kernel's register form: a workgroup of NW waves on a strip of 16*NT rows, wave w on
// K groups w, w+NW, ..., lane (r16, j) on the 16-byte chunk of row r16 of each tile for k-block j (four 256-byte
// pieces, one per four-row block, per load instruction); U groups per trip as in the kernel.
template <int NT>
__global__ __launch_bounds__(1024) void probe_gemv_read_kernel(const u4_t* __restrict__ qw, int N, int K) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, NW = blockDim.x >> 6;
    const int r16 = lane & 15, j = lane >> 4;
    const int nblk = gridDim.x, xcd = blockIdx.x & 7;
    const int strip = xcd * (nblk >> 3) + min(xcd, nblk & 7) + (blockIdx.x >> 3);
    const int n0 = strip * 16 * NT;
    const int kq = K >> 3, groups = K >> 7;
    constexpr int U = NT <= 2 ? 2 : 1;
    const u4_t* wp[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int n = n0 + nt * 16 + r16;
        n = n < N ? n : N - 1;
        wp[nt] = qw + (long)(n >> 2) * kq + (n & 3) * 2 + (j & 1) + (j >> 1) * 8;
    }
    u4_t acc = {0, 0, 0, 0};
    for (int c0 = wave; c0 < groups; c0 += NW * U) {
        u4_t u[U][NT];
#pragma unroll
        for (int t = 0; t < U; ++t) {
            int c = c0 + t * NW;
            c = c < groups ? c : groups - 1;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) u[t][nt] = __builtin_nontemporal_load(wp[nt] + c * 16);
        }
#pragma unroll
        for (int t = 0; t < U; ++t)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc ^= u[t][nt];
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345u) g_probe_sink = 1;
}

// ---- matrix pipe under load: every wave issues `iters` x 16 independent MFMAs on operands it read once (what the
// operands are -- constants or random bits -- is the caller's choice and decides the power drawn).  clk[0] = shader cycles
// and clk[1] = ticks of the constant 100 MHz counter, both around the loop of workgroup 0.
template <int KIND>   // 0: v_mfma_i32_32x32x32_i8, 1: v_mfma_f32_32x32x16_f16
__global__ __launch_bounds__(256) void probe_mfma_stream_kernel(const u4_t* __restrict__ in, int iters, unsigned long long* clk) {
    u4_t a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a[i] = in[threadIdx.x + 256 * i];
        b[i] = in[threadIdx.x + 256 * (4 + i)];
    }
    const long long c0 = clock64(), w0 = wall_clock64();
    uint32_t fold = 0;
    if constexpr (KIND == 0) {
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
                    acc[i * 4 + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i4_t, a[i]), __builtin_bit_cast(i4_t, b[j]), acc[i * 4 + j], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) fold ^= (uint32_t)acc[i][e];
    } else {
        f16_t acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
        for (int it = 0; it < iters; ++it)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8_t, a[i]), __builtin_bit_cast(h8_t, b[j]), acc[i * 4 + j], 0, 0, 0);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) sum += acc[i][e];
        fold = __builtin_bit_cast(uint32_t, sum);
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    if (fold == 0x12345u) g_probe_sink = fold;                   // keeps the accumulators alive
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        clk[0] = (unsigned long long)(c1 - c0);
        clk[1] = (unsigned long long)(w1 - w0);
    }
}

// ---- the two pipes of a SIMD: ONE workgroup of eight waves (two per SIMD), 2048 int8 MFMAs and / or 16384 v_perm_b32
// per wave between two reads of the shader clock; out[w] = cycles of wave w.  MODE:
//   1  waves 0-3 MFMAs only, the others idle          2  waves 4-7 vector instructions only
//   3  both at once (one wave of each kind per SIMD)  4..8  waves 0-3: each MFMA followed by 0, 4, 8, 12, 16 vector instructions
//   9  all eight waves vector instructions only       10 waves 0-3 MFMA + 16 vector, waves 4-7 MFMAs only
//   11 all eight waves MFMA + 8 vector                12 all eight waves MFMAs only
template <int MODE>
__global__ __launch_bounds__(512) void probe_pipe_kernel(unsigned long long* out) {
    const int wave = threadIdx.x >> 6;
    uint32_t a[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = threadIdx.x * 3 + i;
    const i4_t fa = {(int)a[0], (int)a[1], (int)a[2], (int)a[3]}, fb = {(int)a[4], (int)a[5], (int)a[6], (int)a[7]};
    i16_t acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0;
    const bool do_mfma = ((MODE == 1 || MODE == 3) && wave < 4) || MODE == 12 || (MODE == 10 && wave >= 4);
    const bool do_valu = ((MODE == 2 || MODE == 3) && wave >= 4) || MODE == 9;
    const bool do_mix = (MODE >= 4 && MODE <= 8 && wave < 4) || (MODE == 10 && wave < 4) || MODE == 11;
    constexpr int NV = MODE == 10 ? 4 : MODE == 11 ? 2 : MODE >= 4 && MODE <= 8 ? MODE - 4 : 0;   // groups of four vector instructions per MFMA
#define KMI_PROBE_MFMA(j) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc[j]) : "v"(fa), "v"(fb))
#define KMI_PROBE_VALU4()                                                                                                          \
    asm volatile("v_perm_b32 %0, %0, %1, %2\n\tv_perm_b32 %1, %1, %2, %3\n\tv_perm_b32 %2, %2, %3, %4\n\tv_perm_b32 %3, %3, %4, %5" \
                 : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]) : "v"(a[4]), "v"(a[5]))
    __syncthreads();
    const long long t0 = clock64();
    if (do_mfma) {
        for (int it = 0; it < 512; ++it) {
            KMI_PROBE_MFMA(0); KMI_PROBE_MFMA(1);
            KMI_PROBE_MFMA(2); KMI_PROBE_MFMA(3);
        }
    }
    if (do_valu) {
        for (int it = 0; it < 512; ++it) {
#pragma unroll
            for (int r = 0; r < 8; ++r) KMI_PROBE_VALU4();
        }
    }
    if (do_mix) {
        for (int it = 0; it < 512; ++it) {
            KMI_PROBE_MFMA(0);
#pragma unroll
            for (int r = 0; r < NV; ++r) KMI_PROBE_VALU4();
            KMI_PROBE_MFMA(1);
#pragma unroll
            for (int r = 0; r < NV; ++r) KMI_PROBE_VALU4();
            KMI_PROBE_MFMA(2);
#pragma unroll
            for (int r = 0; r < NV; ++r) KMI_PROBE_VALU4();
            KMI_PROBE_MFMA(3);
#pragma unroll
            for (int r = 0; r < NV; ++r) KMI_PROBE_VALU4();
        }
    }
    asm volatile("s_nop 0" ::: "memory");
    const long long t1 = clock64();
    if ((threadIdx.x & 63) == 0) out[wave] = (unsigned long long)(t1 - t0);
    uint32_t fold = a[0] ^ a[1] ^ a[2] ^ a[3];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) fold ^= (uint32_t)acc[j][e];
    if (fold == 0x12345u) g_probe_sink = fold;
#undef KMI_PROBE_MFMA
#undef KMI_PROBE_VALU4
}

extern "C" int kmi_probe_empty(void* stream) {
    hipLaunchKernelGGL(probe_empty_kernel, dim3(256), dim3(256), 0, static_cast<hipStream_t>(stream));
    return kmi_check_launch("kmi_probe_empty");
}

extern "C" int kmi_probe_stream_read(const void* buf, size_t bytes, void* stream) {
    KMI_REQUIRE_PTR(buf);
    if (bytes < 16) return kmi_set_error(KMI_E_SHAPE, "kmi_probe_stream_read: at least 16 bytes");
    const long n16 = (long)(bytes / 16);
    hipLaunchKernelGGL(probe_read_kernel<4>, dim3((unsigned)((n16 + 1023) / 1024)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const u4_t*>(buf), n16);
    return kmi_check_launch("kmi_probe_stream_read");
}

extern "C" int kmi_probe_gemv_read(const void* qweight, int N, int K, int nt, int nw, void* stream) {
    KMI_REQUIRE_PTR(qweight);
    if (N <= 0 || K <= 0 || (N & 15) || (K & 127) || nt < 1 || nt > 8 || (nw != 4 && nw != 8 && nw != 16))
        return kmi_set_error(KMI_E_SHAPE, "kmi_probe_gemv_read: need N%%16==0, K%%128==0, nt 1..8, nw 4/8/16 (N=%d K=%d nt=%d nw=%d)", N, K, nt, nw);
    const dim3 grid((N / 16 + nt - 1) / nt), block(nw * 64);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const u4_t* q = static_cast<const u4_t*>(qweight);
    switch (nt) {
        case 1: hipLaunchKernelGGL(probe_gemv_read_kernel<1>, grid, block, 0, st, q, N, K); break;
        case 2: hipLaunchKernelGGL(probe_gemv_read_kernel<2>, grid, block, 0, st, q, N, K); break;
        case 3: hipLaunchKernelGGL(probe_gemv_read_kernel<3>, grid, block, 0, st, q, N, K); break;
        case 4: hipLaunchKernelGGL(probe_gemv_read_kernel<4>, grid, block, 0, st, q, N, K); break;
        case 5: hipLaunchKernelGGL(probe_gemv_read_kernel<5>, grid, block, 0, st, q, N, K); break;
        case 6: hipLaunchKernelGGL(probe_gemv_read_kernel<6>, grid, block, 0, st, q, N, K); break;
        case 7: hipLaunchKernelGGL(probe_gemv_read_kernel<7>, grid, block, 0, st, q, N, K); break;
        default: hipLaunchKernelGGL(probe_gemv_read_kernel<8>, grid, block, 0, st, q, N, K); break;
    }
    return kmi_check_launch("kmi_probe_gemv_read");
}

extern "C" int kmi_probe_mfma_stream(int kind, const void* operands, size_t operand_bytes, int workgroups, int iters, void* clocks_u64x2,
                                     void* stream) {
    KMI_REQUIRE_PTR(operands);
    KMI_REQUIRE_PTR(clocks_u64x2);
    if ((kind != 0 && kind != 1) || operand_bytes < 8 * 256 * 16 || workgroups < 1 || workgroups > 65536 || iters < 1 || iters > (1 << 20))
        return kmi_set_error(KMI_E_SHAPE, "kmi_probe_mfma_stream: kind 0/1, at least 32 KiB of operands, 1..65536 workgroups, 1..2^20 iterations");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const u4_t* in = static_cast<const u4_t*>(operands);
    unsigned long long* clk = static_cast<unsigned long long*>(clocks_u64x2);
    if (kind == 0) hipLaunchKernelGGL(probe_mfma_stream_kernel<0>, dim3(workgroups), dim3(256), 0, st, in, iters, clk);
    else hipLaunchKernelGGL(probe_mfma_stream_kernel<1>, dim3(workgroups), dim3(256), 0, st, in, iters, clk);
    return kmi_check_launch("kmi_probe_mfma_stream");
}

extern "C" int kmi_probe_pipe_overlap(int mode, void* cycles_u64x8, void* stream) {
    KMI_REQUIRE_PTR(cycles_u64x8);
    hipStream_t st = static_cast<hipStream_t>(stream);
    unsigned long long* out = static_cast<unsigned long long*>(cycles_u64x8);
    switch (mode) {
#define KMI_PIPE_CASE(m) case m: hipLaunchKernelGGL(probe_pipe_kernel<m>, dim3(1), dim3(512), 0, st, out); break;
        KMI_PIPE_CASE(1) KMI_PIPE_CASE(2) KMI_PIPE_CASE(3) KMI_PIPE_CASE(4) KMI_PIPE_CASE(5) KMI_PIPE_CASE(6)
        KMI_PIPE_CASE(7) KMI_PIPE_CASE(8) KMI_PIPE_CASE(9) KMI_PIPE_CASE(10) KMI_PIPE_CASE(11) KMI_PIPE_CASE(12)
#undef KMI_PIPE_CASE
        default: return kmi_set_error(KMI_E_SHAPE, "kmi_probe_pipe_overlap: mode %d outside 1..12", mode);
    }
    return kmi_check_launch("kmi_probe_pipe_overlap");
}

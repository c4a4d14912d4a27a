// Measurement probes: kernels that only read, for the floors that the streaming kernels of the library are measured
// against (an empty launch, a plain contiguous reader, and a reader that issues exactly the weight loads of the
// small-M W4A16 kernel and nothing else).  No product path calls them; `python -m kairos_amd.bench_extra floor` does.
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

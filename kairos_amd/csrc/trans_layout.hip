// Re-pack of the resident int4 format into the operand layout of the version-2 W4A8 candidate:
// int16 [N/4, K] (four-row interleave) -> int8 [N, K/2] in 32x32 blocks of 512 bytes, block order
// (n/32, k/32); inside a block byte (n%8)*64 + ((k%16)/4)*16 + ((k%32)/16)*8 + ((n%16)/8)*4 + k%4 holds
// rows n (low nibble, n%32 < 16) and n+16 (high nibble).  Replaces trans_layout_c16_to_c8_awq
// (kernels/csrc/kairos_kernel/trans_layout/trans_layout_marlin_c16_to_c8.cu:183-205, one thread per
// output byte there); contract: test/test_trans_layout.py:46-52, trans(pack_awq(A)) == pack_w4a8(A).
//
// Pure nibble shuffle, bound by HBM: N*K/2 bytes in, N*K/2 out.  Four threads per (block, n%8): the 16-byte chunks
// of rows n%8 + {0, 8, 16, 24} (32 weights of one row each: word t, nibble a, half c holds k = 8a + 2t + c) make the
// 64 contiguous bytes these four rows own in the block; each thread reads the half of every chunk that its quarter
// needs and writes 16 bytes, so a store instruction covers a contiguous KiB (with one thread per 64 bytes the kernel
// ran at 0.6 of the rate).
#include "kmi_common.h"

__global__ __launch_bounds__(256) void trans_layout_kernel(u4_t* __restrict__ out, const u2_t* __restrict__ qw,
                                                           int K, long total) {
    const long tid = (long)blockIdx.x * 256 + threadIdx.x;      // one thread per 16 output bytes
    if (tid >= total) return;
    const int k4a = (int)(tid & 3);                              // which quarter of the 64 bytes
    const int r8 = (int)((tid >> 2) & 7);
    const long block = tid >> 5;
    const int kblocks = K >> 5;
    const int n32 = (int)(block / kblocks), k32 = (int)(block - (long)n32 * kblocks);
    const int per_quad = K >> 3;                 // 16-byte chunks per four-row block
    const int in_quad = (k32 >> 1) * 8 + (r8 & 3) * 2 + (k32 & 1);
    const int t0 = 2 * (k4a & 1);                // the two words of each chunk this quarter is made of
    u2_t row[2][2];                              // [n2a: +16][n2b: +8]
#pragma unroll
    for (int hi = 0; hi < 2; ++hi)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const int quad = n32 * 8 + hi * 4 + b * 2 + (r8 >> 2);
            row[hi][b] = __builtin_nontemporal_load(qw + ((long)quad * per_quad + in_quad) * 2 + (t0 >> 1));
        }
    u4_t v;                                      // word index k2*2 + n2b
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const int sh = 4 * (2 * k2 + (k4a >> 1));
            uint32_t y[2];                       // halves of word t0+j: k%4 = 2j (low half) and 2j+1 (high half)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                y[j] = ((row[0][b][j] >> sh) & 0x000F000Fu) | (((row[1][b][j] >> sh) & 0x000F000Fu) << 4);
            v[k2 * 2 + b] = __builtin_amdgcn_perm(y[1], y[0], 0x06040200u);
        }
    out[tid] = v;
}

extern "C" int kmi_trans_layout_w4a8(void* out_i8, const void* qweight, int N, int K, void* stream) {
    const char* fn = "kmi_trans_layout_w4a8";
    if (!out_i8 || !qweight) return kmi_set_error(KMI_E_NULL, "%s: NULL pointer argument", fn);
    if (!kmi_aligned16(out_i8) || !kmi_aligned16(qweight))
        return kmi_set_error(KMI_E_ALIGN, "%s: out_i8 and qweight must be 16-byte aligned", fn);
    if (N <= 0 || K <= 0 || (N & 31) || (K & 63))
        return kmi_set_error(KMI_E_SHAPE, "%s: need N%%32==0 and K%%64==0, got N=%d K=%d", fn, N, K);
    const long total = (long)N * K / 32;                   // 16-byte pieces of the output
    hipLaunchKernelGGL(trans_layout_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<u4_t*>(out_i8), static_cast<const u2_t*>(qweight), K,
                       total);
    return kmi_check_launch(fn);
}

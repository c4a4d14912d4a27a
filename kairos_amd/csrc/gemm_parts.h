// Parts shared by the MFMA GEMM kernels of the library: argument block, accumulator epilogues, the split-K reduce
// kernel, scheduling hints and the workgroup -> tile order.  Included by gemm_mfma.hip and gemm_w4a8.hip.
#pragma once
#include "kmi_common.h"
#include <type_traits>

enum { KIND_F16 = 0, KIND_W4A16 = 1, KIND_W8A16 = 2, KIND_W8A8 = 3, KIND_W8A8_ACC = 4 };

struct GemmArgs {
    void* out;
    const void* a;
    const void* b;
    const half_t* scales;     // W4A16: [Gp, N]
    const half_t* szeros;     // W4A16: [Gp, N]
    const half_t* wscales;    // W8A16 / W8A8: [N]
    const half_t* ascales;    // W8A8: [M]
    const half_t* bias;       // [N] or null
    int M, N, K;
    void* partial;            // split-K: [splits][M][N] fp32 / int32 partial sums, else null
    int splits;               // number of K splits (1 = none)
    int n_begin, n_cols;      // output columns this launch covers (a multiple of the tile width unless it ends at N)
    int group_m;              // tile rows per column-major group of the workgroup -> tile order (0 = the default, 8)
};


__device__ __forceinline__ int lds_off(int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); }

// int8 x4 -> two fp16 pairs, exactly: flip the sign bit (b+128 in 0..255), splice each byte under
// the exponent of 1024.0, subtract 1152.
__device__ __forceinline__ void i8x4_to_h2x2(uint32_t w, h2_t& lo, h2_t& hi) {
    const h2_t k1152 = {(half_t)1152.0f, (half_t)1152.0f};
    const uint32_t u = w ^ 0x80808080u;
    lo = as_h2(__builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - k1152;
    hi = as_h2(__builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - k1152;
}

// One accumulator element, for the epilogues.  The 256 accumulator registers of a 256x256 tile live in
// AGPRs; left to itself the register allocator copies all of them to VGPRs where the main loop ends and
// spills over a hundred to scratch.  An explicit read at the point of use keeps each one in place until
// it is needed.  (The caller leaves >= 18 wait states between the last MFMA and the first read.)
template <bool FROM_AGPR, typename T>
__device__ __forceinline__ T acc_elem(T a) {
    if constexpr (FROM_AGPR) {
        T v;
        asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
        return v;
    } else {
        return a;
    }
}

// Split-K: a workgroup that only covers part of K writes its raw accumulators (fp32 or int32, 4 bytes
// each) to slice `split` of the partial buffer; splitk_reduce_kernel adds the slices in a fixed order
// and applies the epilogue arithmetic.  Lane layout as in gemm_epilogue below.
template <int BM, int BN, int FM, int FN, typename acc_t>
__device__ __forceinline__ void store_partial(const GemmArgs& p, acc_t (&acc)[FM][FN], int split, int m0, int n0,
                                              int wave, int lane) {
    const int M = p.M, N = p.N;
    const int wm = wave >> 1, wn = wave & 1;
    const int c = lane & 31, hl = lane >> 5;
    const int mw = m0 + wm * (BM / 2), nw = n0 + wn * (BN / 2);
    uint32_t* dst = static_cast<uint32_t*>(p.partial) + (long)split * M * N;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        const int m = mw + i * 32 + c;
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = nw + j * 32 + 8 * g + 4 * hl;       // four consecutive columns, N % 4 == 0
                if (m < M && n < N) {
                    u4_t v;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const auto elem = acc_elem<(FM * FN >= 12)>(acc[i][j][4 * g + r]);   // a scalar copy:
                        v[r] = __builtin_bit_cast(uint32_t, elem);       // bit_cast needs an addressable scalar
                    }
                    *reinterpret_cast<u4_t*>(dst + (long)m * N + n) = v;
                }
            }
    }
}

template <int KIND>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(GemmArgs p) {
    const long quad = (long)blockIdx.x * 256 + threadIdx.x;       // one thread = four consecutive columns
    const long total = (long)p.M * p.N / 4;
    if (quad >= total) return;
    const long e0 = quad * 4;
    const int m = (int)(e0 / p.N), n = (int)(e0 - (long)m * p.N);
    constexpr bool I8 = (KIND == KIND_W8A8 || KIND == KIND_W8A8_ACC);
    int isum[4] = {0, 0, 0, 0};
    float fsum[4] = {0.f, 0.f, 0.f, 0.f};
    const uint32_t* part = static_cast<const uint32_t*>(p.partial);
    for (int s = 0; s < p.splits; ++s) {
        const u4_t v = *reinterpret_cast<const u4_t*>(part + (long)s * p.M * p.N + e0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t w = v[r];                         // scalar copy: bit_cast of a vector element misreads
            if constexpr (I8) isum[r] += (int)w;
            else fsum[r] += __builtin_bit_cast(float, w);
        }
    }
    if constexpr (KIND == KIND_W8A8_ACC) {
        int* o = static_cast<int*>(p.out) + e0;
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = isum[r];
    } else {
        half_t h[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float v;
            if constexpr (KIND == KIND_W8A8) {
                v = (float)isum[r] * ((float)p.wscales[n + r] * (float)p.ascales[m]);
                asm volatile("" : "+v"(v));                  // two roundings, as in gemm_epilogue
            } else if constexpr (KIND == KIND_W8A16) {
                v = fsum[r] * (float)p.wscales[n + r];
            } else {
                v = fsum[r];
            }
            h[r] = (half_t)v;
            if (p.bias) h[r] = (half_t)((float)h[r] + (float)p.bias[n + r]);
        }
        *reinterpret_cast<h4_t*>(static_cast<half_t*>(p.out) + e0) = h4_t{h[0], h[1], h[2], h[3]};
    }
}

// Epilogue shared by the GEMM kernels.  The MFMAs are issued with the weight fragment as the first
// operand, so an accumulator tile is D^T: lane (c = lane&31, hl = lane>>5) holds, for activation row
// m = c, the output columns n = 8g + 4hl + r (e = 4g + r) -- four consecutive columns per g.
// A wave converts one 32-row block at a time, writes it to its private LDS patch as fp16 [32][BN/2]
// (8-byte writes, pitch padded by 8 bytes -> conflict free), and streams it out with 16-byte stores
// in which 16 consecutive lanes cover 256 contiguous bytes of one output row.
//
// With one wave per SIMD every instruction of the epilogue, scalar or vector, costs an issue slot that nothing
// else fills, so the instruction count is the cost.  Three things keep it down:
//   * W8A8: the factor of element (m, n) is wscale[n] * ascale[m], exact in fp32 (two 11-bit significands).  One
//     32x32x8 fp16 MFMA per accumulator tile, fed with the wave's 32 column factors and 32 row factors in its k = 0
//     slice and zeros elsewhere, writes those 1024 products in the accumulator's own lane layout; the matrix pipe is
//     idle here anyway.  Element work is then read, int -> float, one multiply, pack.
//   * a tile that lies inside the matrix stores through a buffer resource at the tile's origin: a per-lane
//     offset fixed for the kernel, a scalar offset per store, no masks and no 64-bit address arithmetic;
//   * accumulators are read four at a time, so no read is followed by its own use (a wait state otherwise).
struct NoHook {
    __device__ __forceinline__ void operator()() const {}
    __device__ __forceinline__ void operator()(int) const {}
};

// This lane's entries of the per-column and per-row factors of a W8A8 tile: ws[j] belongs to column
// nw + 32j + lane%32 of the wave's block, as[i] to row mw + 32i + lane%32.
template <int FM, int FN>
struct EpiFactors {
    half_t ws[FN];
    half_t as[FM];
};
template <int BM, int BN, int FM, int FN>
__device__ __forceinline__ void epilogue_factors(const GemmArgs& p, int m0, int n0, int wave, int lane, EpiFactors<FM, FN>& f) {
    const int c = lane & 31;
    const int mw = m0 + (wave >> 1) * (BM / 2) + c, nw = n0 + (wave & 1) * (BN / 2) + c;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const int n = nw + j * 32;
        f.ws[j] = p.wscales[n < p.N ? n : p.N - 1];
    }
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        const int m = mw + i * 32;
        f.as[i] = p.ascales[m < p.M ? m : p.M - 1];
    }
}

// `before_block(i)` runs in front of the conversion of every 32-row block, the first time once the per-column and
// per-row factors have arrived and before the first result leaves: a persistent kernel issues the next tile's first
// operand loads there, a few per block (a burst of them would queue up in the address path while the wave waits),
// behind every load this epilogue waits for.
// `pre`: W8A8 factors the caller loaded ahead of time (else they are loaded here).
template <int KIND, int BM, int BN, bool HAS_BIAS, int FM, int FN, typename acc_t, typename Hook = NoHook>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& p, acc_t (&acc)[FM][FN], char* smem, int m0, int n0,
                                              int wave, int lane, Hook before_block = Hook{},
                                              const EpiFactors<FM, FN>* pre = nullptr
                                              ) {
    const int M = p.M, N = p.N;
    const int wm = wave >> 1, wn = wave & 1;
    const int c = lane & 31, hl = lane >> 5;
    const int mw = m0 + wm * (BM / 2), nw = n0 + wn * (BN / 2);
    if constexpr (KIND == KIND_W8A8_ACC) {
        // raw accumulators (verification tier): plain element stores
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            const int m = mw + i * 32 + c;
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int n = nw + j * 32 + 8 * (e >> 2) + 4 * hl + (e & 3);
                    if (m < M && n < N) static_cast<int*>(p.out)[(long)m * N + n] = acc[i][j][e];
                }
        }
    } else {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass knows neither the buffer resource type nor the MFMA
        constexpr int WN = BN / 2;                       // columns per wave
        constexpr bool BIG = FM * FN >= 12;              // accumulators in AGPRs, read explicitly
        constexpr int PITCH = WN * 2 + 8;                // bytes
        constexpr int CPR = WN * 2 / 16;                 // 16-byte chunks per row
        char* patch = smem + wave * (32 * PITCH);
        // per-column factors of this lane: columns nw + j*32 + 8g + 4hl + (0..3), one 8-byte load each
        // (N % 4 == 0, so a group of four columns is entirely inside or outside the matrix)
        h4_t ws4[FN][4], bs4[FN][4];
        (void)ws4; (void)bs4;
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                int n = nw + j * 32 + 8 * g + 4 * hl;
                n = n < N ? n : N - 4;
                if constexpr (KIND == KIND_W8A16) ws4[j][g] = *reinterpret_cast<const h4_t*>(p.wscales + n);
                if constexpr (HAS_BIAS) bs4[j][g] = *reinterpret_cast<const h4_t*>(p.bias + n);
            }
        float wsf[FN][4][4];                              // fp32 once, not once per row block
        (void)wsf;
        if constexpr (KIND == KIND_W8A16) {
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int r = 0; r < 4; ++r) wsf[j][g][r] = (float)ws4[j][g][r];
        }
        // W8A8: the operands of the factor tiles.  Weight side first, as in the main loop, so the product tile has
        // the accumulators' layout; only the k = 0..3 slice (lanes 0..31) carries a value, in its first element.
        h4_t wop[FN], aop[FM];
        (void)wop; (void)aop;
        if constexpr (KIND == KIND_W8A8) {
            EpiFactors<FM, FN> f;
            if (pre) f = *pre;
            else epilogue_factors<BM, BN, FM, FN>(p, m0, n0, wave, lane, f);
            const half_t zero = (half_t)0.f;
#pragma unroll
            for (int j = 0; j < FN; ++j) wop[j] = h4_t{hl == 0 ? f.ws[j] : zero, zero, zero, zero};
#pragma unroll
            for (int i = 0; i < FM; ++i) aop[i] = h4_t{hl == 0 ? f.as[i] : zero, zero, zero, zero};
            // built here, once: the statements that use them must find them in registers, not rebuild them on the spot
#pragma unroll
            for (int j = 0; j < FN; ++j) asm volatile("" : "+v"(wop[j]));
#pragma unroll
            for (int i = 0; i < FM; ++i) asm volatile("" : "+v"(aop[i]));
        }
        if constexpr (!std::is_same<Hook, NoHook>::value) {
            // name every loaded factor as an operand, so the compiler places its waits for them here and
            // none of its later waits can fall behind the loads that the hook starts
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                if constexpr (KIND == KIND_W8A8) asm volatile("" : "+v"(wop[j]));
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    if constexpr (KIND == KIND_W8A16) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) asm volatile("" : "+v"(wsf[j][g][r]));
                    }
                    if constexpr (HAS_BIAS) asm volatile("" : "+v"(bs4[j][g]));
                }
            }
            if constexpr (KIND == KIND_W8A8) {
#pragma unroll
                for (int i = 0; i < FM; ++i) asm volatile("" : "+v"(aop[i]));
            }
            asm volatile("" ::: "memory");
        }
        half_t* outp = static_cast<half_t*>(p.out);
        const bool wide = (N & 7) == 0;                  // 16-byte row segments stay aligned
        // a tile inside the matrix: stores relative to the tile's origin, 32-bit offsets (256 rows of N fp16)
        const bool inside = wide && m0 + BM <= M && n0 + BN <= N && (64 % CPR) == 0 && (long)N * BM * 2 < (1L << 32);
        const __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(outp + ((long)m0 * N + n0), 0, -1, 0x00020000);
        const uint32_t ovoff = (uint32_t)(((wm * (BM / 2) + lane / CPR) * N + wn * WN + (lane % CPR) * 8) * 2);
        // Factor tiles, two in flight: tile t+1 is issued before tile t is converted.  Written as asm with a VGPR
        // destination: the compiler would place the result in AGPRs, and every element would cost a read again.
        // The compiler knows nothing of the latency of such a statement, so the distance between a product and its
        // first use is built from ordered statements: the first tile carries its wait states itself; every later
        // tile is handed to its users (`settled`) only behind the 64 multiplies of the tile before it, each a
        // statement of its own, in program order: far more than the 19 wait states a 16-pass MFMA asks for.
        f16_t fac[2];
        (void)fac;
        auto factor_tile = [&](int t) {
            if constexpr (KIND == KIND_W8A8) {
                if (t == 0)
                    asm volatile("s_nop 3\n\tv_mfma_f32_32x32x8_f16 %0, %1, %2, 0\n\ts_nop 15\n\ts_nop 7"
                                 : "=&v"(fac[0]) : "v"(wop[0]), "v"(aop[0]));
                else if (t < FM * FN)   // the wait state in front: the compiler may have copied an operand just before
                    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x8_f16 %0, %1, %2, 0" : "=&v"(fac[t & 1]) : "v"(wop[t % FN]), "v"(aop[t / FN]));
            }
        };
        auto settled = [&](int t) {
            if constexpr (KIND == KIND_W8A8) asm volatile("" : "+v"(fac[t & 1]));
        };
        // A row block leaves in two steps, one block apart: its 16-byte chunks are read back from the patch right
        // behind its last write, and stored while the next block is being converted (after that block's first tile),
        // so neither the LDS round trip nor the store issue stands between two conversions.
        constexpr int NK = 32 * CPR / 64;                    // 16-byte chunks per lane and 32-row block
        static_assert((32 * CPR) % 64 == 0, "whole 16-byte chunks per lane");
        u4_t v[NK];
        auto read_block = [&]() {
#pragma unroll
            for (int k = 0; k < NK; ++k) {
                const int idx = k * 64 + lane;
                v[k] = *reinterpret_cast<const u4_t*>(patch + (idx / CPR) * PITCH + (idx % CPR) * 16);
            }
        };
        auto store_block = [&](int i) {
            if constexpr (64 % CPR != 0) {                   // 96 columns per wave: the column changes with k
#pragma unroll
                for (int k = 0; k < NK; ++k) {
                    const int idx = k * 64 + lane;
                    const int m = mw + i * 32 + idx / CPR, n = nw + (idx % CPR) * 8;
                    half_t* d = outp + (long)m * N + n;
                    if (wide) {
                        if (m < M && n < N) __builtin_nontemporal_store(v[k], reinterpret_cast<u4_t*>(d));
                    } else {
                        if (m < M && n < N) *reinterpret_cast<u2_t*>(d) = u2_t{v[k][0], v[k][1]};
                        if (m < M && n + 4 < N) *reinterpret_cast<u2_t*>(d + 4) = u2_t{v[k][2], v[k][3]};
                    }
                }
                return;
            }
            if (inside) {
#pragma unroll
                for (int k = 0; k < NK; ++k)
                    __builtin_amdgcn_raw_buffer_store_b128(v[k], orsrc, ovoff, (uint32_t)((i * 32 + k * (64 / CPR)) * N * 2), 2 /* nt */);
                return;
            }
            const int n = nw + (lane % CPR) * 8;             // CPR divides 64: the column is the same for every k
            half_t* dst = outp + (long)(mw + i * 32 + lane / CPR) * N + n;
            if (wide) {
#pragma unroll
                for (int k = 0; k < NK; ++k) {
                    const int m = mw + i * 32 + (k * 64 + lane) / CPR;
                    if (m < M && n < N) __builtin_nontemporal_store(v[k], reinterpret_cast<u4_t*>(dst + (long)k * (64 / CPR) * N));
                }
            } else {                                         // N % 8 == 4: two 8-byte halves, each whole or absent
#pragma unroll
                for (int k = 0; k < NK; ++k) {
                    const int m = mw + i * 32 + (k * 64 + lane) / CPR;
                    half_t* d = dst + (long)k * (64 / CPR) * N;
                    if (m < M && n < N) *reinterpret_cast<u2_t*>(d) = u2_t{v[k][0], v[k][1]};
                    if (m < M && n + 4 < N) *reinterpret_cast<u2_t*>(d + 4) = u2_t{v[k][2], v[k][3]};
                }
            }
        };
        factor_tile(0);
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            if constexpr (!std::is_same<Hook, NoHook>::value) {
                before_block(i);
                asm volatile("" ::: "memory");
            }
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                if (j == (FN > 1 ? 1 : 0) && i > 0) {         // the block before: its chunks have arrived by now
                    store_block(i - 1);
                    asm volatile("" ::: "memory");
                }
                settled(i * FN + j);
                factor_tile(i * FN + j + 1);
                if constexpr (KIND == KIND_W8A8 && BIG && !HAS_BIAS) {
                    // One wave per SIMD: a dependent instruction issued right behind its producer waits about one
                    // more issue slot, and nothing else fills it.  Eight elements at a time, every step a statement
                    // of its own in the order written, keep producer and user at least four instructions apart.
#pragma unroll
                    for (int gg = 0; gg < 2; ++gg) {
                        int ai[8];
                        float af[8], pr[8];
                        uint32_t pk[4];
#pragma unroll
                        for (int e = 0; e < 8; ++e) asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(ai[e]) : "a"(acc[i][j][8 * gg + e]));
#pragma unroll
                        for (int e = 0; e < 8; ++e) asm volatile("v_cvt_f32_i32 %0, %1" : "=v"(af[e]) : "v"(ai[e]));
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const float s = fac[(i * FN + j) & 1][8 * gg + e];
                            asm volatile("v_mul_f32 %0, %1, %2" : "=v"(pr[e]) : "v"(af[e]), "v"(s));
                        }
#pragma unroll
                        for (int q = 0; q < 4; ++q) asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(pk[q]) : "v"(pr[2 * q]), "v"(pr[2 * q + 1]));
#pragma unroll
                        for (int h = 0; h < 2; ++h)
                            *reinterpret_cast<u2_t*>(patch + c * PITCH + (j * 32 + 8 * (2 * gg + h) + 4 * hl) * 2) = u2_t{pk[2 * h], pk[2 * h + 1]};
                    }
                } else {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        decltype(acc_elem<BIG>(acc[i][j][0])) a[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) a[r] = acc_elem<BIG>(acc[i][j][4 * g + r]);
                        half_t h[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            float v;
                            if constexpr (KIND == KIND_W8A8) {
                                // product rounded to fp32 first, then to fp16 (two roundings, as the
                                // reference epilogue): keep the compiler from fusing them into one
                                // (the multiply is a statement of its own, which also makes it one of the ordered
                                // instructions that stand between a factor tile and its users)
                                const float s = fac[(i * FN + j) & 1][4 * g + r];
                                const float fa = (float)a[r];
                                asm volatile("v_mul_f32 %0, %1, %2" : "=v"(v) : "v"(fa), "v"(s));
                            } else if constexpr (KIND == KIND_W8A16) {
                                v = a[r] * wsf[j][g][r];
                            } else {
                                v = a[r];
                            }
                            h[r] = (half_t)v;
                            if constexpr (HAS_BIAS) h[r] = (half_t)((float)h[r] + (float)bs4[j][g][r]);
                        }
                        h4_t pk = {h[0], h[1], h[2], h[3]};
                        *reinterpret_cast<h4_t*>(patch + c * PITCH + (j * 32 + 8 * g + 4 * hl) * 2) = pk;
                    }
                }
            }
            // The patch is private to the wave and LDS serves a wave's requests in order: these reads see the writes
            // above without a wait, and the next block's writes cannot overtake them.
            asm volatile("" ::: "memory");
            read_block();
        }
        store_block(FM - 1);
#endif
    }
}

// Scheduling hints: spread WRITES LDS writes evenly between the NMFMA MFMAs of one k-step, READS LDS
// reads between those of its first half (their results are needed by the next block) and LOADS global
// loads between those of its second half (a direct-to-LDS load counts as an LDS store, so the compiler
// keeps it behind every LDS read that precedes it in program order), so that the matrix pipe never
// waits behind a burst of memory issue.
template <int NMFMA, int READS, int WRITES, int LOADS, int K = 0>
__device__ __forceinline__ void sched_interleave() {
    if constexpr (NMFMA >= 4 && K < NMFMA) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        constexpr int H = NMFMA / 2;                     // LDS reads go behind the first half of the MFMAs
        constexpr int r = K < H ? (K + 1) * READS / H - K * READS / H : 0;
        constexpr int w = (K + 1) * WRITES / NMFMA - K * WRITES / NMFMA;
        constexpr int l = K >= H ? (K - H + 1) * LOADS / (NMFMA - H) - (K - H) * LOADS / (NMFMA - H) : 0;
        if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(0x100, r, 0);
        if constexpr (w > 0) __builtin_amdgcn_sched_group_barrier(0x200, w, 0);
        if constexpr (l > 0) __builtin_amdgcn_sched_group_barrier(0x010, l, 0);   // any VMEM: a direct-to-LDS load is not a plain read
        sched_interleave<NMFMA, READS, WRITES, LOADS, K + 1>();
    }
}

// Workgroup -> output tile.  Hardware deals workgroups round-robin over the 8 XCDs (id % 8), each
// with a private L2.  Give every XCD a contiguous run of the tile sequence, and order that sequence
// in column-major groups of GROUP_M tile rows, so the tiles resident on one XCD at a time form a
// compact block that shares A row-panels and B column-panels in that XCD's L2.
__device__ __forceinline__ void tile_of_block(int wg, int TM, int TN, int& tm, int& tn, int group_m = 0) {
    constexpr int XCDS = 8;
    const int GROUP_M = group_m > 0 ? group_m : 8;
    const int total = TM * TN;
    const int xcd = wg % XCDS, q = wg / XCDS;
    const int base = total / XCDS, rem = total % XCDS;
    const int L = xcd * base + (xcd < rem ? xcd : rem) + q;
    const int per_group = GROUP_M * TN;
    const int g = L / per_group, in_g = L - g * per_group;
    const int rows = (TM - g * GROUP_M) < GROUP_M ? (TM - g * GROUP_M) : GROUP_M;
    tn = in_g / rows;
    tm = g * GROUP_M + (in_g - tn * rows);
}

// ---- host side, defined in gemm_mfma.hip ---------------------------------------------------------------------------
// Scratch for split-K partial sums: every GEMM entry point takes a caller-owned device buffer (pointer and size)
// and uses it only for the duration of the call's launches on the given stream.  Without one (NULL or too small
// for two slices) no split is used.  Nothing about it is remembered between calls.
struct Workspace { void* ptr; size_t bytes; };
int kmi_pick_splits(int M, int N, int K, int BM, int BN, int ktiles, const Workspace& ws);
int kmi_gemm_args_check(const char* fn, const GemmArgs& a, bool tiled);
int kmi_workspace_check(const char* fn, const void* workspace, size_t bytes, Workspace& ws);
int kmi_pick_tile_rows(int M, int N, long row_bytes);
int kmi_forced_tile();       // test hook of the calling thread, 0 = automatic
int kmi_forced_group_m();    // test hook of the calling thread, 0 = the default tile order

// LDS-staged MFMA GEMMs of the switched linear path:  out[M,N] = A[M,K] . B[N,K]^T  with
//   KIND_F16    A fp16, B fp16 row-major                       v_mfma_f32_32x32x16_f16
//   KIND_W4A16  A fp16, B packed uint4, decoded while staging   v_mfma_f32_32x32x16_f16
//   KIND_W8A16  A fp16, B int8, widened while staging           v_mfma_f32_32x32x16_f16
//   KIND_W8A8   A int8, B int8, int32 accumulators              v_mfma_i32_32x32x32_i8
//
// Both operands are K-contiguous, so one k-tile of either operand is `rows x 128 bytes` (64 fp16 or
// 128 int8).  In LDS a row is eight 16-byte chunks; chunk c of row r is stored at c ^ ((r>>1)&7),
// which makes both the 16-byte staging writes and the MFMA fragment reads (32 consecutive rows, one
// logical chunk) bank-conflict free.  256 threads = 2x2 waves; each wave owns a (BM/2)x(BN/2) block
// of 32x32 accumulator tiles.  Global loads for k-tile t+1 are issued before the MFMAs of k-tile t
// and written to the other LDS stage afterwards: one barrier per k-tile.
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

template <int KIND, int BM, int BN, bool TILED_B>
__global__ __launch_bounds__(256) void gemm_kernel(GemmArgs p) {
    constexpr bool I8 = (KIND == KIND_W8A8 || KIND == KIND_W8A8_ACC);
    constexpr int FM = BM / 64, FN = BN / 64;              // 32x32 accumulator tiles per wave
    constexpr int A_CH = BM * 8 / 256;                      // 16-byte chunks per thread, A tile
    constexpr int B_CH = (KIND == KIND_W4A16) ? BN * 2 / 256 : (KIND == KIND_W8A16) ? BN * 4 / 256 : BN * 8 / 256;
    constexpr int STAGE = (BM + BN) * 128;
    static_assert(B_CH >= 1, "tile too small for the staging scheme");
    using acc_t = typename std::conditional<I8, i16_t, f16_t>::type;

    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int M = p.M, N = p.N, K = p.K;
    const long a_row_bytes = I8 ? (long)K : (long)K * 2;
    const int KT = (int)(a_row_bytes >> 7);
    const char* A = static_cast<const char*>(p.a);
    const char* B = static_cast<const char*>(p.b);

    acc_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    u4_t ra[A_CH];
    u4_t rb[B_CH];
    half_t rs[B_CH], rz[B_CH];
    (void)rs; (void)rz;

    auto load_tile = [&](int kt) {
#pragma unroll
        for (int i = 0; i < A_CH; ++i) {
            const int q = tid + i * 256, row = q >> 3, c = q & 7;
            const int m = m0 + row;
            ra[i] = (m < M) ? *reinterpret_cast<const u4_t*>(A + (long)m * a_row_bytes + (long)kt * 128 + c * 16)
                            : u4_t{0, 0, 0, 0};
        }
        if constexpr (KIND == KIND_W4A16) {
#pragma unroll
            for (int i = 0; i < B_CH; ++i) {
                const int q = tid + i * 256, row = q >> 1, h = q & 1;
                int n = n0 + row;
                n = n < N ? n : N - 1;
                rb[i] = *reinterpret_cast<const u4_t*>(B + (long)(n >> 2) * K * 2 + (long)kt * 128 + (n & 3) * 32 + h * 16);
                rs[i] = p.scales[(long)(kt >> 1) * N + n];
                rz[i] = p.szeros[(long)(kt >> 1) * N + n];
            }
        } else if constexpr (TILED_B && KIND == KIND_W8A16) {
            // int8 tiles are 128 K wide: this 64-wide k-tile is one half of every row of tile kt/2
#pragma unroll
            for (int i = 0; i < B_CH; ++i) {
                const int q = tid + i * 256, row = q >> 2, c4 = q & 3;
                const int strip = row >> 7, rin = row & 127;
                if (n0 + strip * KMI_TILE_N < N) {
                    const long tile = ((long)(n0 / KMI_TILE_N) + strip) * (K >> 7) + (kt >> 1);
                    const int src_c = ((kt & 1) * 4 + c4) ^ ((rin >> 1) & 7);
                    rb[i] = *reinterpret_cast<const u4_t*>(B + tile * (KMI_TILE_N * 128) + rin * 128 + src_c * 16);
                } else {
                    rb[i] = u4_t{0, 0, 0, 0};
                }
            }
        } else if constexpr (TILED_B) {
            // the k-tile of a 128-row strip is one contiguous, already swizzled 16 KiB block
#pragma unroll
            for (int i = 0; i < B_CH; ++i) {
                const int q = tid + i * 256;                 // chunk index inside the BN x 128B tile
                const int strip = q >> 10, inner = q & 1023;
                if (n0 + strip * KMI_TILE_N < N) {
                    const long tile = ((long)(n0 / KMI_TILE_N) + strip) * KT + kt;
                    rb[i] = *reinterpret_cast<const u4_t*>(B + tile * (KMI_TILE_N * 128) + inner * 16);
                } else {
                    rb[i] = u4_t{0, 0, 0, 0};
                }
            }
        } else if constexpr (KIND == KIND_W8A16) {
#pragma unroll
            for (int i = 0; i < B_CH; ++i) {
                const int q = tid + i * 256, row = q >> 2, c = q & 3;
                int n = n0 + row;
                n = n < N ? n : N - 1;
                rb[i] = *reinterpret_cast<const u4_t*>(B + (long)n * K + (long)kt * 64 + c * 16);
            }
        } else {
#pragma unroll
            for (int i = 0; i < B_CH; ++i) {
                const int q = tid + i * 256, row = q >> 3, c = q & 7;
                int n = n0 + row;
                n = n < N ? n : N - 1;
                rb[i] = *reinterpret_cast<const u4_t*>(B + (long)n * a_row_bytes + (long)kt * 128 + c * 16);
            }
        }
    };

    auto store_tile = [&](int stage) {
        char* sa = smem + stage * STAGE;
        char* sb = sa + BM * 128;
#pragma unroll
        for (int i = 0; i < A_CH; ++i) {
            const int q = tid + i * 256;
            *reinterpret_cast<u4_t*>(sa + lds_off(q >> 3, q & 7)) = ra[i];
        }
        if constexpr (KIND == KIND_W4A16) {
#pragma unroll
            for (int i = 0; i < B_CH; ++i) {
                const int q = tid + i * 256, row = q >> 1, h = q & 1;
                const h2_t s2 = {rs[i], rs[i]}, z2 = {rz[i], rz[i]};
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 4 * h + 0)) = dequant_nibble<0>(rb[i], s2, z2);
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 4 * h + 1)) = dequant_nibble<1>(rb[i], s2, z2);
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 4 * h + 2)) = dequant_nibble<2>(rb[i], s2, z2);
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 4 * h + 3)) = dequant_nibble<3>(rb[i], s2, z2);
            }
        } else if constexpr (KIND == KIND_W8A16) {
#pragma unroll
            for (int i = 0; i < B_CH; ++i) {
                const int q = tid + i * 256, row = q >> 2, c = q & 3;
                h2_t v[8];
#pragma unroll
                for (int w = 0; w < 4; ++w) i8x4_to_h2x2(rb[i][w], v[2 * w], v[2 * w + 1]);
                h8_t lo, hi;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    lo[2 * e] = v[e][0]; lo[2 * e + 1] = v[e][1];
                    hi[2 * e] = v[4 + e][0]; hi[2 * e + 1] = v[4 + e][1];
                }
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 2 * c)) = lo;
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 2 * c + 1)) = hi;
            }
        } else if constexpr (TILED_B) {
#pragma unroll
            for (int i = 0; i < B_CH; ++i) *reinterpret_cast<u4_t*>(sb + (tid + i * 256) * 16) = rb[i];
        } else {
#pragma unroll
            for (int i = 0; i < B_CH; ++i) {
                const int q = tid + i * 256;
                *reinterpret_cast<u4_t*>(sb + lds_off(q >> 3, q & 7)) = rb[i];
            }
        }
    };

    auto compute = [&](int stage) {
        const char* sa = smem + stage * STAGE + (wm * (BM / 2)) * 128;
        const char* sb = smem + stage * STAGE + BM * 128 + (wn * (BN / 2)) * 128;
        const int r = lane & 31, kh = lane >> 5;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            u4_t fa[FM], fb[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) fa[i] = *reinterpret_cast<const u4_t*>(sa + lds_off(i * 32 + r, 2 * s + kh));
#pragma unroll
            for (int j = 0; j < FN; ++j) fb[j] = *reinterpret_cast<const u4_t*>(sb + lds_off(j * 32 + r, 2 * s + kh));
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    if constexpr (I8)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i4_t, fa[i]),
                                                                          __builtin_bit_cast(i4_t, fb[j]), acc[i][j], 0, 0, 0);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8_t, fa[i]),
                                                                           __builtin_bit_cast(h8_t, fb[j]), acc[i][j], 0, 0, 0);
                }
        }
    };

    load_tile(0);
    store_tile(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const bool more = (kt + 1 < KT);
        if (more) load_tile(kt + 1);
        compute(kt & 1);
        if (more) store_tile((kt + 1) & 1);
        __syncthreads();
    }

    // ---- epilogue: lane holds, per 32x32 tile, column (lane&31) and rows 8*(e/4) + 4*(lane>>5) + e%4
    const int col_in = lane & 31, row_in = (lane >> 5) * 4;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const int n = n0 + wn * (BN / 2) + j * 32 + col_in;
        if (n >= N) continue;
        float ws = 1.0f, bv = 0.0f;
        if constexpr (KIND == KIND_W8A16 || KIND == KIND_W8A8) ws = (float)p.wscales[n];
        if (p.bias) bv = (float)p.bias[n];
#pragma unroll
        for (int i = 0; i < FM; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * (BM / 2) + i * 32 + 8 * (e >> 2) + row_in + (e & 3);
                if (m >= M) continue;
                if constexpr (KIND == KIND_W8A8_ACC) {
                    static_cast<int*>(p.out)[(long)m * N + n] = acc[i][j][e];
                } else {
                    float v;
                    if constexpr (KIND == KIND_W8A8) {
                        // product rounded to fp32 first, then to fp16 (two roundings, as the
                        // reference epilogue): keep the compiler from fusing them into one
                        v = (float)acc[i][j][e] * (ws * (float)p.ascales[m]);
                        asm volatile("" : "+v"(v));
                    }
                    else if constexpr (KIND == KIND_W8A16) v = acc[i][j][e] * ws;
                    else v = acc[i][j][e];
                    half_t h = (half_t)v;
                    if (p.bias) h = (half_t)((float)h + bv);
                    static_cast<half_t*>(p.out)[(long)m * N + n] = h;
                }
            }
        }
    }
}

// ---- host side ---------------------------------------------------------------------------------
template <int KIND, int BM, int BN, bool TILED>
static int launch_gemm(const GemmArgs& a, hipStream_t st) {
    constexpr size_t lds = 2 * (size_t)(BM + BN) * 128;
    auto fn = gemm_kernel<KIND, BM, BN, TILED>;
    if (lds > 64 * 1024) {
        static thread_local bool raised = false;   // per kernel instantiation, per thread
        if (!raised) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
                return kmi_set_error(KMI_E_LAUNCH, "gemm: cannot raise the dynamic LDS limit to %zu bytes", lds);
            raised = true;
        }
    }
    const dim3 grid((a.N + BN - 1) / BN, (a.M + BM - 1) / BM), block(256);
    hipLaunchKernelGGL(fn, grid, block, lds, st, a);
    return KMI_OK;
}

// Tile choice: the largest tile that still yields about one workgroup per CU.
static int pick_tile(int M, int N) {
    auto wgs = [&](int bm, int bn) { return (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    if (M > 128 && wgs(256, 256) >= 200) return 256;
    if (M > 64 && wgs(128, 128) >= 128) return 128;
    return 64;
}
extern "C" int kmi_gemm_pick_tile(int M, int N) { return pick_tile(M, N); }

template <int KIND, bool TILED>
static int dispatch_gemm(const GemmArgs& a, hipStream_t st, int force_tile) {
    const int tile = force_tile > 0 ? force_tile : pick_tile(a.M, a.N);
    switch (tile) {
        case 256: return launch_gemm<KIND, 256, 256, TILED>(a, st);
        case 128: return launch_gemm<KIND, 128, 128, TILED>(a, st);
        case 64: return launch_gemm<KIND, 64, 128, TILED>(a, st);
    }
    return kmi_set_error(KMI_E_SHAPE, "gemm: unknown tile selector %d", tile);
}

static int gemm_check(const char* fn, const GemmArgs& a, bool tiled) {
    if (!a.out || !a.a || !a.b) return kmi_set_error(KMI_E_NULL, "%s: NULL pointer argument", fn);
    if (!kmi_aligned16(a.a) || !kmi_aligned16(a.b)) return kmi_set_error(KMI_E_ALIGN, "%s: operands must be 16-byte aligned", fn);
    if (a.M < 0 || a.N <= 0 || a.K <= 0 || (a.K & 127) || (a.N & 3))
        return kmi_set_error(KMI_E_SHAPE, "%s: need M>=0, N%%4==0, K%%128==0 (M=%d N=%d K=%d)", fn, a.M, a.N, a.K);
    if (tiled && (a.N % KMI_TILE_N)) return kmi_set_error(KMI_E_SHAPE, "%s: tiled operand needs N%%%d==0 (N=%d)", fn, KMI_TILE_N, a.N);
    return KMI_OK;
}

static thread_local int g_force_tile = 0;
extern "C" void kmi_gemm_force_tile(int tile) { g_force_tile = tile; }

#define KMI_GEMM_BODY(NAME, KIND, TILED)                                      \
    int rc = gemm_check(NAME, a, TILED);                                      \
    if (rc != KMI_OK) return rc;                                              \
    if (a.M == 0) return KMI_OK;                                              \
    rc = dispatch_gemm<KIND, TILED>(a, static_cast<hipStream_t>(stream), g_force_tile); \
    if (rc != KMI_OK) return rc;                                              \
    return kmi_check_launch(NAME);

extern "C" int kmi_gemm_w4a16(void* out, const void* x, const void* qweight, const void* scales, const void* szeros,
                              const void* bias, int M, int N, int K, int G, void* stream) {
    if (G != 128) return kmi_set_error(KMI_E_GROUP, "kmi_gemm_w4a16: group size %d unsupported (128 only)", G);
    if (!scales || !szeros) return kmi_set_error(KMI_E_NULL, "kmi_gemm_w4a16: NULL scale table");
    GemmArgs a{out, x, qweight, (const half_t*)scales, (const half_t*)szeros, nullptr, nullptr, (const half_t*)bias, M, N, K};
    KMI_GEMM_BODY("kmi_gemm_w4a16", KIND_W4A16, false)
}

extern "C" int kmi_gemm_w8a16(void* out, const void* x, const void* w8, const void* wscales, const void* bias,
                              int M, int N, int K, void* stream) {
    if (!wscales) return kmi_set_error(KMI_E_NULL, "kmi_gemm_w8a16: NULL wscales");
    GemmArgs a{out, x, w8, nullptr, nullptr, (const half_t*)wscales, nullptr, (const half_t*)bias, M, N, K};
    KMI_GEMM_BODY("kmi_gemm_w8a16", KIND_W8A16, false)
}

extern "C" int kmi_gemm_w8a8(void* out, const void* a8, const void* w8, const void* wscales, const void* ascales,
                             const void* bias, int M, int N, int K, void* stream) {
    if (!wscales || !ascales) return kmi_set_error(KMI_E_NULL, "kmi_gemm_w8a8: NULL scale vector");
    GemmArgs a{out, a8, w8, nullptr, nullptr, (const half_t*)wscales, (const half_t*)ascales, (const half_t*)bias, M, N, K};
    KMI_GEMM_BODY("kmi_gemm_w8a8", KIND_W8A8, false)
}

extern "C" int kmi_gemm_w8a8_acc_i32(void* acc, const void* a8, const void* w8, int M, int N, int K, void* stream) {
    GemmArgs a{acc, a8, w8, nullptr, nullptr, nullptr, nullptr, nullptr, M, N, K};
    KMI_GEMM_BODY("kmi_gemm_w8a8_acc_i32", KIND_W8A8_ACC, false)
}

extern "C" int kmi_gemm_f16(void* out, const void* x, const void* w16, const void* bias, int M, int N, int K, void* stream) {
    GemmArgs a{out, x, w16, nullptr, nullptr, nullptr, nullptr, (const half_t*)bias, M, N, K};
    KMI_GEMM_BODY("kmi_gemm_f16", KIND_F16, false)
}

extern "C" int kmi_gemm_w8a8_tiled(void* out, const void* a8, const void* w8t, const void* wscales, const void* ascales,
                                   const void* bias, int M, int N, int K, void* stream) {
    if (!wscales || !ascales) return kmi_set_error(KMI_E_NULL, "kmi_gemm_w8a8_tiled: NULL scale vector");
    GemmArgs a{out, a8, w8t, nullptr, nullptr, (const half_t*)wscales, (const half_t*)ascales, (const half_t*)bias, M, N, K};
    KMI_GEMM_BODY("kmi_gemm_w8a8_tiled", KIND_W8A8, true)
}

extern "C" int kmi_gemm_w8a16_tiled(void* out, const void* x, const void* w8t, const void* wscales, const void* bias,
                                    int M, int N, int K, void* stream) {
    if (!wscales) return kmi_set_error(KMI_E_NULL, "kmi_gemm_w8a16_tiled: NULL wscales");
    GemmArgs a{out, x, w8t, nullptr, nullptr, (const half_t*)wscales, nullptr, (const half_t*)bias, M, N, K};
    KMI_GEMM_BODY("kmi_gemm_w8a16_tiled", KIND_W8A16, true)
}

extern "C" int kmi_gemm_f16_tiled(void* out, const void* x, const void* w16t, const void* bias, int M, int N, int K, void* stream) {
    GemmArgs a{out, x, w16t, nullptr, nullptr, nullptr, nullptr, (const half_t*)bias, M, N, K};
    KMI_GEMM_BODY("kmi_gemm_f16_tiled", KIND_F16, true)
}

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
// of 32x32 accumulator tiles.  That is the register-staged kernel (gemm_kernel: W4A16, W8A16), which
// keeps two k-tiles in flight in two register sets and writes them to the other of two LDS stages:
// one barrier per k-tile.  The operand-copy kinds (F16, W8A8) use gemm_direct_kernel further down:
// direct-to-LDS loads, four 64-byte stages.
// W4A16 products of up to ~1000 rows run gemm_w4a16_wp_kernel instead (weights decoded in registers by the wave
// that owns their columns, never written to LDS); the host side at the end of the file picks kernel and tile.
#include "gemm_parts.h"
#include <atomic>
#include <mutex>

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
    const int M = p.M, N = p.N, K = p.K;
    int tm, tn;
    const int TM_ = (M + BM - 1) / BM, TN_ = (p.n_cols + BN - 1) / BN;
    const int split = blockIdx.x / (TM_ * TN_);
    tile_of_block(blockIdx.x - split * (TM_ * TN_), TM_, TN_, tm, tn, p.group_m);
    const int m0 = tm * BM, n0 = p.n_begin + tn * BN;
    const long a_row_bytes = I8 ? (long)K : (long)K * 2;
    const int KT_all = (int)(a_row_bytes >> 7);
    const int kt_per = (KT_all + p.splits - 1) / p.splits;
    const int kt0 = split * kt_per;                          // this workgroup covers k-tiles kt0 .. kt0+KT-1
    const int KT = (kt0 + kt_per <= KT_all) ? kt_per : KT_all - kt0;

    acc_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    // ---- per-thread global sources (rows beyond M / N are clamped: their products are never stored)
    const char* pa[A_CH];
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
        const int q = tid + i * 256, row = q >> 3, c = q & 7;
        int m = m0 + row;
        m = m < M ? m : M - 1;
        pa[i] = static_cast<const char*>(p.a) + (long)m * a_row_bytes + c * 16;
    }
    const char* pb[B_CH];
    long b_step;                                              // bytes between consecutive k-tiles
    int scale_col[B_CH];
    (void)scale_col;
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
        const int q = tid + i * 256;
        const char* B = static_cast<const char*>(p.b);
        if constexpr (KIND == KIND_W4A16) {
            const int row = q >> 1, h = q & 1;
            int n = n0 + row;
            n = n < N ? n : N - 1;
            pb[i] = B + (long)(n >> 2) * K * 2 + (n & 3) * 32 + h * 16;
            scale_col[i] = n;
        } else if constexpr (KIND == KIND_W8A16) {
            const int row = q >> 2, c = q & 3;
            int n = n0 + row;
            n = n < N ? n : N - 1;
            pb[i] = B + (long)n * K + c * 16;
        } else {
            const int row = q >> 3, c = q & 7;
            int n = n0 + row;
            n = n < N ? n : N - 1;
            pb[i] = B + (long)n * a_row_bytes + c * 16;
        }
    }
    static_assert(!TILED_B, "the register-staged kernel reads row-major / packed operands only");
    if constexpr (KIND == KIND_W8A16) b_step = 64;
    else b_step = 128;

    // Two register sets hold k-tiles in flight between global memory and LDS: tile t travels in set
    // t & 1, is loaded about two iterations before it is written to LDS, and the set index is a
    // compile-time constant everywhere (the main loop is unrolled by two), so the compiler can count
    // exactly how many newer loads may stay outstanding at each use.
    u4_t ra[2][A_CH];
    u4_t rb[2][B_CH];
    half_t rs[2][B_CH], rz[2][B_CH];
    (void)rs; (void)rz;
    using set0 = std::integral_constant<int, 0>;
    using set1 = std::integral_constant<int, 1>;

    auto load_tile = [&](auto set, int kt_req) {
        constexpr int S = decltype(set)::value;
        const int kt = kt_req < KT ? kt_req : KT - 1;        // past the end: a harmless reload, never stored
#pragma unroll
        for (int i = 0; i < A_CH; ++i) ra[S][i] = *reinterpret_cast<const u4_t*>(pa[i] + (long)(kt0 + kt) * 128);
#pragma unroll
        for (int i = 0; i < B_CH; ++i) {
            rb[S][i] = *reinterpret_cast<const u4_t*>(pb[i] + (long)(kt0 + kt) * b_step);
            if constexpr (KIND == KIND_W4A16) {
                rs[S][i] = p.scales[(long)((kt0 + kt) >> 1) * N + scale_col[i]];
                rz[S][i] = p.szeros[(long)((kt0 + kt) >> 1) * N + scale_col[i]];
            }
        }
    };

    auto store_tile = [&](auto set, int stage) {
        constexpr int S = decltype(set)::value;
        char* sa = smem + stage * STAGE;
        char* sb = sa + BM * 128;
#pragma unroll
        for (int i = 0; i < A_CH; ++i) {
            const int q = tid + i * 256;
            *reinterpret_cast<u4_t*>(sa + lds_off(q >> 3, q & 7)) = ra[S][i];
        }
        if constexpr (KIND == KIND_W4A16) {
#pragma unroll
            for (int i = 0; i < B_CH; ++i) {
                const int q = tid + i * 256, row = q >> 1, h = q & 1;
                const h2_t s2 = {rs[S][i], rs[S][i]}, z2 = {rz[S][i], rz[S][i]};
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 4 * h + 0)) = dequant_nibble<0>(rb[S][i], s2, z2);
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 4 * h + 1)) = dequant_nibble<1>(rb[S][i], s2, z2);
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 4 * h + 2)) = dequant_nibble<2>(rb[S][i], s2, z2);
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 4 * h + 3)) = dequant_nibble<3>(rb[S][i], s2, z2);
            }
        } else if constexpr (KIND == KIND_W8A16) {
#pragma unroll
            for (int i = 0; i < B_CH; ++i) {
                const int q = tid + i * 256, row = q >> 2, c = q & 3;
                h2_t v[8];
#pragma unroll
                for (int w = 0; w < 4; ++w) i8x4_to_h2x2(rb[S][i][w], v[2 * w], v[2 * w + 1]);
                h8_t lo, hi;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    lo[2 * e] = v[e][0]; lo[2 * e + 1] = v[e][1];
                    hi[2 * e] = v[4 + e][0]; hi[2 * e + 1] = v[4 + e][1];
                }
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 2 * c)) = lo;
                *reinterpret_cast<h8_t*>(sb + lds_off(row, 2 * c + 1)) = hi;
            }
        } else {
#pragma unroll
            for (int i = 0; i < B_CH; ++i) {
                const int q = tid + i * 256;
                *reinterpret_cast<u4_t*>(sb + lds_off(q >> 3, q & 7)) = rb[S][i];
            }
        }
    };

    // ---- fragments: two register sets, read one k-step ahead of the MFMAs that consume them
    u4_t fa[2][FM], fb[2][FN];
    const int fr = lane & 31, fkh = lane >> 5;
    auto read_frags = [&](int stage, int s, int set) {
        const char* sa = smem + stage * STAGE + (wm * (BM / 2)) * 128;
        const char* sb = smem + stage * STAGE + BM * 128 + (wn * (BN / 2)) * 128;
#pragma unroll
        for (int i = 0; i < FM; ++i) fa[set][i] = *reinterpret_cast<const u4_t*>(sa + lds_off(i * 32 + fr, 2 * s + fkh));
#pragma unroll
        for (int j = 0; j < FN; ++j) fb[set][j] = *reinterpret_cast<const u4_t*>(sb + lds_off(j * 32 + fr, 2 * s + fkh));
    };
    auto mfma_step = [&](int set) {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                if constexpr (I8)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i4_t, fb[set][j]),
                                                                      __builtin_bit_cast(i4_t, fa[set][i]), acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8_t, fb[set][j]),
                                                                       __builtin_bit_cast(h8_t, fa[set][i]), acc[i][j], 0, 0, 0);
            }
    };
    constexpr bool PURE_COPY = (KIND == KIND_F16 || I8);     // staging without conversion ALU work
    constexpr int NMF = FM * FN, NRD = FM + FN, NWR = PURE_COPY ? A_CH + B_CH : 0, NLD = A_CH + B_CH;

    // ---- software pipeline.  LDS stage t&1 holds k-tile t.  Per k-tile kt:
    //   steps 0,1: MFMAs + fragment reads of the next step
    //   step 2   : MFMAs + fragment reads of step 3 + write k-tile kt+1 (in registers since iteration kt-2)
    //              to the other stage
    //   barrier  : the other stage is complete, this stage is no longer read
    //   step 3   : MFMAs + fragment reads of step 0 of k-tile kt+1 + global loads of k-tile kt+3 into the
    //              register set just emptied
    load_tile(set0{}, 0);
    store_tile(set0{}, 0);
    // the loads of the two tiles must be issued in the loop's own order (all of k-tile 1, then all of
    // k-tile 2): the wait counts inside the loop are the merge of this state and the back edge's
    __builtin_amdgcn_sched_barrier(0);
    load_tile(set1{}, 1);
    __builtin_amdgcn_sched_barrier(0);
    load_tile(set0{}, 2);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    read_frags(0, 0, 0);
    auto body = [&](auto set, int kt) {                       // `set` holds k-tile kt+1
        const int cur = kt & 1, nxt = cur ^ 1;
        read_frags(cur, 1, 1);
        mfma_step(0);
        sched_interleave<NMF, NRD, 0, 0>();
        __builtin_amdgcn_sched_barrier(0);
        read_frags(cur, 2, 0);
        mfma_step(1);
        sched_interleave<NMF, NRD, 0, 0>();
        __builtin_amdgcn_sched_barrier(0);
        read_frags(cur, 3, 1);
        store_tile(set, nxt);
        mfma_step(0);
        sched_interleave<NMF, NRD, NWR, 0>();
        __syncthreads();
        read_frags(nxt, 0, 0);
        load_tile(set, kt + 3);
        mfma_step(1);
        sched_interleave<NMF, NRD, 0, NLD>();
        __builtin_amdgcn_sched_barrier(0);
    };
    int kt = 0;
    for (; kt + 2 <= KT - 1; kt += 2) {
        body(set1{}, kt);
        body(set0{}, kt + 1);
    }
    if (kt < KT - 1) body(set1{}, kt);
    {   // last k-tile: nothing left to stage
        const int cur = (KT - 1) & 1;
        read_frags(cur, 1, 1);
        mfma_step(0);
        sched_interleave<NMF, NRD, 0, 0>();
        __builtin_amdgcn_sched_barrier(0);
        read_frags(cur, 2, 0);
        mfma_step(1);
        sched_interleave<NMF, NRD, 0, 0>();
        __builtin_amdgcn_sched_barrier(0);
        read_frags(cur, 3, 1);
        mfma_step(0);
        sched_interleave<NMF, NRD, 0, 0>();
        __builtin_amdgcn_sched_barrier(0);
        mfma_step(1);
    }

    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();                                         // staging LDS is reused by the epilogue
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");       // MFMA results settle before explicit AGPR reads
    if (p.splits > 1) store_partial<BM, BN, FM, FN>(p, acc, split, m0, n0, wave, lane);
    else if (p.bias) gemm_epilogue<KIND, BM, BN, true, FM, FN>(p, acc, smem, m0, n0, wave, lane);
    else gemm_epilogue<KIND, BM, BN, false, FM, FN>(p, acc, smem, m0, n0, wave, lane);
}

// dequant_nibble with the masks and the exponent pattern held in registers, so that mask-and-splice is one
// v_and_or_b32 instead of two literal-operand instructions (a VOP3 cannot take literals on gfx9).  Same
// arithmetic, same bits.
struct NibConsts { uint32_t mask_lo, mask_hi, magic; };
__device__ __forceinline__ NibConsts nib_consts() {
    NibConsts c{0x000F000Fu, 0x00F000F0u, 0x64006400u};
    asm volatile("" : "+s"(c.mask_lo), "+s"(c.mask_hi), "+v"(c.magic));      // opaque: keeps them out of the instructions
    return c;
}
template <int A>
__device__ __forceinline__ h8_t dequant_nibble_r(const u4_t& u, h2_t s2, h2_t z2, const NibConsts& c) {
    const h2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    const h2_t k16th = {(half_t)0.0625f, (half_t)0.0625f};
    const h2_t km64 = {(half_t)-64.0f, (half_t)-64.0f};
    h2_t r[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const uint32_t w = (A >= 2) ? (u[t] >> 8) : u[t];
        h2_t q;
        if constexpr (A & 1) q = pk_fma(as_h2((w & c.mask_hi) | c.magic), k16th, km64);
        else q = as_h2((w & c.mask_lo) | c.magic) - k1024;
        r[t] = pk_fma(q, s2, z2);
    }
    h8_t o;
    o[0] = r[0][0]; o[1] = r[0][1]; o[2] = r[1][0]; o[3] = r[1][1];
    o[4] = r[2][0]; o[5] = r[2][1]; o[6] = r[3][0]; o[7] = r[3][1];
    return o;
}

// f(integral_constant<int, B>) ... f(integral_constant<int, E - 1>), unrolled at compile time
template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// =================================================================================================
// W4A16 for M up to a few hundred rows: wave-private weights.
//
// With so few rows the register-staged kernel above is bound by instruction issue, not by MFMA or
// memory: every weight passes through LDS (a write and two fragment reads) and one wave per SIMD
// serialises decode, LDS and load issue.  Here a workgroup tile is BM rows x 128 columns and each
// wave owns 32 of the columns for itself, so its weights never touch LDS: lane (n = lane%32,
// h = lane/32) loads the 16-byte chunk h of row n of the 64-wide k-tile (32 weights) and decodes its four
// 8-weight planes exactly as the converters do; plane p is k 32h + 8p .. + 7 of the k-tile.  Which sixteen k
// an MFMA sums is free as long as both operands agree, so MFMA p of the four per k-tile takes plane p as it
// lies -- k 8p..8p+7 in the lower half-wave, 32+8p..32+8p+7 in the upper -- and the activation fragment is
// read from LDS at those k (chunk 4h + p of the row): no lane of the wave ever hands a weight to another
// (a v_permlane32_swap costs 13-16 cycles of the vector ALU, three ordinary instructions; sixteen of them per
// k-tile were 40 % of the decode).  Only the activations are staged (direct-to-LDS loads, PF+1 stages),
// shared by the four column waves.  The workgroup has KH such wave quartets; quartet q takes k-tiles
// q, q+KH, ... and the quartets' accumulators meet in LDS at the end (fixed order).  A scale and a
// scaled zero arrive in ONE load (lower lanes fetch the scale, upper lanes the zero of the same column)
// and are spread with one more swap.  Per wave and k-tile: BM/32 + 2 load instructions, no LDS write.
template <int BM, int KH, int PF>
__global__ __launch_bounds__(256 * KH) void gemm_w4a16_wp_kernel(GemmArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int FM = BM / 32;
    constexpr int NSA = PF + 1;                      // activation stages per quartet
    constexpr int A_STAGE = BM * 128;                // bytes: BM rows x 64 fp16
    constexpr int A_LD = BM / 32;                    // direct loads per wave and k-tile
    constexpr int OPS = A_LD + 2;                    // load instructions per wave and k-tile
    static_assert(BM == 32 || BM == 64 || BM == 128, "row tiles of 32, 64 or 128");
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wc = wave & 3, kq = wave >> 2;
    const int M = p.M, N = p.N, K = p.K;
    const int TM_ = (M + BM - 1) / BM, TN_ = (p.n_cols + 127) / 128;
    const int split = blockIdx.x / (TM_ * TN_);
    int tm, tn;
    tile_of_block(blockIdx.x - split * (TM_ * TN_), TM_, TN_, tm, tn, p.group_m);
    const int m0 = tm * BM, n0 = p.n_begin + tn * 128;
    const int KT_all = K >> 6;                       // 64-wide k-tiles
    const int kt_per = (((KT_all + p.splits - 1) / p.splits) + KH - 1) / KH * KH;
    const int kt0 = split * kt_per;
    const int KT = (kt0 + kt_per <= KT_all) ? kt_per : KT_all - kt0;     // multiple of KH (host checks K)
    const int T = KT / KH;                           // k-tiles of this quartet: kt0 + kq + j*KH

    f16_t acc[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;

    // ---- sources
    char* ring = smem + kq * (NSA * A_STAGE);
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.a), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.b), 0, -1, 0x00020000);
    uint32_t voff_a[A_LD];
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
        const int row = 8 * (wc + 4 * i) + (lane >> 3), pc = lane & 7;
        const int c = pc ^ ((row >> 1) & 7);
        int m = m0 + row;
        m = m < M ? m : M - 1;
        voff_a[i] = (uint32_t)((long)m * K * 2 + c * 16);
    }
    const int hl = lane >> 5;
    int ncol = n0 + wc * 32 + (lane & 31);
    ncol = ncol < N ? ncol : N - 1;                  // ragged last strip: clamp loads, stores are masked
    const uint32_t voff_b = (uint32_t)((long)(ncol >> 2) * K * 2 + (ncol & 3) * 32 + hl * 16);
    const half_t* szp = (hl ? p.szeros : p.scales) + ncol;

    u4_t rb[PF];
    half_t rsz[PF];
    auto issue = [&](auto set, int j_req) {          // loads of this quartet's j-th k-tile
        constexpr int S = decltype(set)::value;
        const int j = j_req < T ? j_req : T - 1;     // past the end: harmless reloads, never used
        const int g = kt0 + kq + j * KH;
        char* dst = ring + (j_req % NSA) * A_STAGE + wc * 1024;
#pragma unroll
        for (int i = 0; i < A_LD; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(dst + i * 4096), 16, voff_a[i], (uint32_t)g * 128u, 0, 0);
        rb[S] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, voff_b, (uint32_t)g * 128u, 0);
        rsz[S] = szp[(long)(g >> 1) * N];
    };

    // Software pipeline inside the wave: iteration j runs the MFMAs of k-tile j on weights decoded during
    // iteration j-1 and meanwhile decodes k-tile j+1, so the decode's VALU work is spread between the MFMAs
    // instead of standing in front of them.  At the top of iteration j every load of k-tile j+1 must have
    // landed -- its weights and scales for the decode, its activations for the fragment reads issued during
    // k-step 3 -- while the PF-2 younger k-tiles may stay in flight (OPS instructions each, issued in whole
    // groups); the barrier also frees the LDS stage of k-tile j-1 for the loads of k-tile j+PF.
    auto tile_barrier = [&](auto keep_tiles) {
        constexpr int KEEP = decltype(keep_tiles)::value * OPS;
        static_assert(KEEP >= 0 && KEEP < 64, "vmcnt is a six-bit count");
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(KEEP) : "memory");
    };

    const int fr = lane & 31;
    const NibConsts nc = nib_consts();
    u4_t pl[2][4];                                   // decoded weights: [parity of the k-tile][MFMA of the k-tile]
    u4_t fa[2][FM];                                  // activation fragments: [parity of the k-step]
    // pl[.][jj] is plane jj of the lane's own chunk: k 32*hl + 8*jj .. + 7; the activations of the same k
    auto read_frags = [&](int j, int jj, int set) {
        const char* st = ring + (j % NSA) * A_STAGE;
#pragma unroll
        for (int i = 0; i < FM; ++i) fa[set][i] = *reinterpret_cast<const u4_t*>(st + lds_off(i * 32 + fr, 4 * hl + jj));
    };
    // planes 2*half, 2*half+1 of k-tile set S -> pl[par][2*half .. 2*half+1]
    auto decode_half = [&](auto set, auto half, int par, h2_t s2, h2_t z2) {
        constexpr int S = decltype(set)::value, H = decltype(half)::value;
        const u4_t raw = rb[S];
        pl[par][2 * H] = __builtin_bit_cast(u4_t, dequant_nibble_r<2 * H>(raw, s2, z2, nc));
        pl[par][2 * H + 1] = __builtin_bit_cast(u4_t, dequant_nibble_r<2 * H + 1>(raw, s2, z2, nc));
    };
    auto scales_of = [&](auto set, h2_t& s2, h2_t& z2) {
        constexpr int S = decltype(set)::value;
        const uint32_t own = (uint32_t)__builtin_bit_cast(unsigned short, rsz[S]);
        const auto sw = __builtin_amdgcn_permlane32_swap(own, own, false, false);
        const uint32_t sbits = sw[0], zbits = sw[1];          // scale / scaled zero in every lane
        s2 = as_h2(sbits | (sbits << 16));
        z2 = as_h2(zbits | (zbits << 16));
    };
    auto mfma_block = [&](int par, int jj, int set) {
#pragma unroll
        for (int i = 0; i < FM; ++i)
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8_t, pl[par][jj]), __builtin_bit_cast(h8_t, fa[set][i]),
                                                            acc[i], 0, 0, 0);
    };
    // one MFMA, then a share of the other work of the block
    auto interleave = [&](auto valu, auto ds, auto vmem) {
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if constexpr (decltype(valu)::value > 0) __builtin_amdgcn_sched_group_barrier(0x002, (decltype(valu)::value + FM - 1) / FM, 0);
            if constexpr (decltype(ds)::value > 0) __builtin_amdgcn_sched_group_barrier(0x100, (decltype(ds)::value + FM - 1) / FM, 0);
            if constexpr (decltype(vmem)::value > 0) __builtin_amdgcn_sched_group_barrier(0x010, (decltype(vmem)::value + FM - 1) / FM, 0);
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    // iteration j: S = j % PF (compile time); weights of k-tile j are in pl[S & 1], fa[0] holds its k-step 0
    auto body = [&](auto set, int j) {
        constexpr int S = decltype(set)::value, SN = (S + 1) % PF, par = S & 1;
        using SetN = std::integral_constant<int, SN>;
        tile_barrier(std::integral_constant<int, PF - 2>{});
        h2_t s2, z2;
        scales_of(SetN{}, s2, z2);
        // k-step 0 under the first half of the next decode
        read_frags(j, 1, 1);
        mfma_block(par, 0, 0);
        decode_half(SetN{}, I0{}, par ^ 1, s2, z2);
        interleave(std::integral_constant<int, 28>{}, std::integral_constant<int, FM>{}, I0{});
        __builtin_amdgcn_sched_barrier(0);
        // k-step 1 under the second half
        read_frags(j, 2, 0);
        mfma_block(par, 1, 1);
        decode_half(SetN{}, I1{}, par ^ 1, s2, z2);
        interleave(std::integral_constant<int, 36>{}, std::integral_constant<int, FM>{}, I0{});
        __builtin_amdgcn_sched_barrier(0);
        // k-step 2 under the loads of k-tile j+PF (their registers and their LDS stage are free now)
        read_frags(j, 3, 1);
        mfma_block(par, 2, 0);
        issue(set, j + PF);
        interleave(I0{}, std::integral_constant<int, FM>{}, std::integral_constant<int, OPS>{});
        __builtin_amdgcn_sched_barrier(0);
        // k-step 3 under the first fragment reads of k-tile j+1
        read_frags(j + 1, 0, 0);
        mfma_block(par, 3, 1);
        interleave(I0{}, std::integral_constant<int, FM>{}, I0{});
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- pipeline: PF k-tiles in flight per wave (register set = k-tile index modulo PF, a compile-time constant)
    static_assert(PF % 2 == 0 && PF >= 4, "the parity of a k-tile must follow from its register set");
    static_for<0, PF>([&](auto set) { issue(set, decltype(set)::value); __builtin_amdgcn_sched_barrier(0); });
    {   // k-tile 0: decoded in the open
        tile_barrier(std::integral_constant<int, PF - 1>{});
        h2_t s2, z2;
        scales_of(I0{}, s2, z2);
        decode_half(I0{}, I0{}, 0, s2, z2);
        decode_half(I0{}, I1{}, 0, s2, z2);
        read_frags(0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
    int j = 0;
    for (; j + PF <= T; j += PF) static_for<0, PF>([&](auto set) { body(set, j + decltype(set)::value); });
    static_for<0, PF - 1>([&](auto set) {
        if (j < T) { body(set, j); ++j; }
    });
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");   // no load outlives its stage

    // ---- the quartets' partial sums meet in LDS, added to quartet 0 in quartet order
    if constexpr (KH > 1) {
        float* red = reinterpret_cast<float*>(smem);
#pragma unroll
        for (int q = 1; q < KH; ++q) {
            if (kq == q) {
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e) red[((wc * FM + i) * 16 + e) * 64 + lane] = acc[i][e];
            }
            __syncthreads();
            if (kq == 0) {
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[i][e] += red[((wc * FM + i) * 16 + e) * 64 + lane];
            }
            __syncthreads();
        }
        if (kq != 0) return;
    }

    // ---- output: lane (row = lane%32, hl) holds columns 8g + 4hl + (0..3) of its wave's 32
    const int nw = n0 + wc * 32;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        const int m = m0 + i * 32 + fr;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int n = nw + 8 * g + 4 * hl;
            if (m < M && n < N) {
                if (p.splits > 1) {
                    u4_t v;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float f = acc[i][4 * g + r];
                        v[r] = __builtin_bit_cast(uint32_t, f);
                    }
                    *reinterpret_cast<u4_t*>(static_cast<uint32_t*>(p.partial) + (long)split * M * N + (long)m * N + n) = v;
                } else {
                    half_t h[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        h[r] = (half_t)acc[i][4 * g + r];
                        if (p.bias) h[r] = (half_t)((float)h[r] + (float)p.bias[n + r]);
                    }
                    *reinterpret_cast<h4_t*>(static_cast<half_t*>(p.out) + (long)m * N + n) = h4_t{h[0], h[1], h[2], h[3]};
                }
            }
        }
    }
#endif
}

// =================================================================================================
// Direct-to-LDS variant for the operand-copy kinds (KIND_F16, KIND_W8A8, KIND_W8A8_ACC).
//
// With one workgroup per CU (a 256x256 tile needs all 512 VGPRs) only LDS can hold enough bytes in
// flight to cover the global-load latency: registers cannot hold several k-tiles.  Here global loads
// write LDS directly (buffer_load_dwordx4 ... lds: the 64 lanes of a wave fill one contiguous KiB), so
// the spare LDS stages ARE the in-flight buffer: NS stages of (BM+BN) rows x 64 bytes, loads issued
// NS-1 stages ahead, one barrier per stage.
//
// Stage layout: row r (A rows first, then B rows) at r*64; its four 16-byte chunks are stored at
// c ^ ((r>>2)&3), which spreads the fragment reads of 16 consecutive rows over all 64 banks.  Since a
// direct load puts lane l's data at slot l, the swizzle is applied on the global side: lane l
// fetches the chunk that belongs in slot l.  The tiled weight layout ([N/128][K-stages][128][64 B],
// already swizzled) makes the B side a straight 8 KiB copy per 128-row strip.

// Wait until at most KEEP direct loads of this thread are outstanding, then meet the other waves.
// A plain barrier instruction (no fence): the fence of __syncthreads would drain every load.
template <int KEEP>
__device__ __forceinline__ void direct_stage_barrier() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(KEEP) : "memory");
}

template <int KIND, int BM, int BN, bool TILED_B, int NS, bool PERSIST = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((NS == 3 && BM == 256 && BN == 128) ? 2 : 1)))
void gemm_direct_kernel(GemmArgs p) {   // the 256 x 128 instance is built for two workgroups per CU: <= 256 registers, 72 KiB of LDS
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass cannot instantiate code that uses the buffer resource type
    constexpr bool I8 = (KIND == KIND_W8A8 || KIND == KIND_W8A8_ACC);
    static_assert(KIND == KIND_F16 || I8, "direct staging copies operands verbatim");
    constexpr int FM = BM / 64, FN = BN / 64;
    constexpr int ROWS = BM + BN;
    constexpr int STAGE = ROWS * 64;
    constexpr int NLD = ROWS * 4 / 256;                     // direct loads per thread per stage
    static_assert(BM % 64 == 0 && BN % 64 == 0 && NLD * 64 == ROWS, "each wave-load fills 16 rows");
    static_assert(!PERSIST || NS == 4, "the persistent form keeps two stages of the next tile beside the epilogue's patches");
    using acc_t = typename std::conditional<I8, i16_t, f16_t>::type;

    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: feeds M0
    const int wm = wave >> 1, wn = wave & 1;
    const int M = p.M, N = p.N, K = p.K;
    const int TM_ = (M + BM - 1) / BM, TN_ = (p.n_cols + BN - 1) / BN;
    const int nvirt = TM_ * TN_ * p.splits;                  // tiles x splits: the units of work
    const long row_bytes = I8 ? (long)K : (long)K * 2;
    const int T_all = (int)(row_bytes >> 6);                // 64-byte stages along K
    const int t_per = (T_all + p.splits - 1) / p.splits;

    // ---- global sources.  Load i of wave w fills the KiB region R = 4*i + w = rows 16R .. 16R+15.
    // Addresses are a wave-uniform base (advanced per k-stage with scalar adds) plus a per-lane
    // 32-bit offset that never changes within a tile, so the loop carries no vector address arithmetic.
    // A unit of work: its place in the output, its K range and the per-lane offsets of its loads.  The
    // persistent form folds the weight strip of the tile into the offsets (the host checks that they fit
    // 32 bits); the one-tile form moves the base pointer instead.
    struct Unit { int split, m0, n0, t0, T; uint32_t voff[NLD]; };
    auto setup = [&](int vb, Unit& u) {
        int tm, tn;
        u.split = vb / (TM_ * TN_);
        tile_of_block(vb - u.split * (TM_ * TN_), TM_, TN_, tm, tn, p.group_m);
        u.m0 = tm * BM;
        u.n0 = p.n_begin + tn * BN;
        u.t0 = u.split * t_per;                              // this unit covers stages t0 .. t0+T-1
        u.T = (u.t0 + t_per <= T_all) ? t_per : T_all - u.t0;
        // FOLD: the weight strip of the tile goes into the per-lane offsets (several tiles per workgroup, or tiles
        // whose width is not a whole number of 128-row strips, so that a tile may start in the middle of one)
        constexpr bool FOLD = TILED_B && (PERSIST || (BN % KMI_TILE_N) != 0);
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int row = 16 * (4 * i + wave) + (lane >> 2);
            const int pc = lane & 3;
            const int c = pc ^ ((row >> 2) & 3);
            if (16 * (4 * i) < BM) {                         // region lies in the A part (BM % 64 == 0)
                int m = u.m0 + row;
                m = m < M ? m : M - 1;
                u.voff[i] = (uint32_t)((long)m * row_bytes + c * 16);
            } else if constexpr (TILED_B) {
                // 16-row groups never straddle a strip (tiles start at multiples of 64 columns); the stored swizzle
                // depends on the row inside the strip, which equals the row inside the tile modulo 16
                const int rb = row - BM;
                const int base_n = FOLD ? 0 : (u.n0 / KMI_TILE_N) * KMI_TILE_N;   // first column of the strip at the resource's base
                int nrel = u.n0 - base_n + rb;                                     // this row's column relative to it
                if (base_n + nrel >= N) nrel = ((u.n0 - base_n) & ~(KMI_TILE_N - 1)) + (rb & (KMI_TILE_N - 1));   // ragged last tile: the (valid) strip of n0; stores are masked
                u.voff[i] = (uint32_t)((long)(nrel >> 7) * T_all * (KMI_TILE_N * 64) + (nrel & 127) * 64 + pc * 16);
            } else {
                int n = u.n0 + row - BM;
                n = n < N ? n : N - 1;
                u.voff[i] = (uint32_t)((long)n * row_bytes + c * 16);
            }
        }
    };
    Unit cur;
    setup(blockIdx.x, cur);

    const char* a_base = static_cast<const char*>(p.a);
    const char* b_base = static_cast<const char*>(p.b);
    if constexpr (TILED_B && !(PERSIST || (BN % KMI_TILE_N) != 0)) b_base += (long)(cur.n0 / KMI_TILE_N) * T_all * (KMI_TILE_N * 64);
    constexpr long B_STEP = TILED_B ? KMI_TILE_N * 64 : 64;
    // k-stage t -> LDS stage t % NS; the loads of a stage are issued in two halves (h = 0, 1)
    constexpr int NLD0 = (NLD + 1) / 2;
    // Buffer addressing: a resource per operand (base pointer, no stride, no range limit), the per-lane
    // 32-bit offset and a scalar offset that advances with the k-stage, so a load reads one address VGPR
    // per lane and the loop carries no vector address arithmetic at all.
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a_base), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(b_base), 0, -1, 0x00020000);
    auto issue_half = [&](const Unit& u, int t, int h) {
        const int tt = u.t0 + (t < u.T ? t : u.T - 1);       // past the end: harmless reload into a free stage
        char* dst = smem + (t % NS) * STAGE + wave * 1024;
        const uint32_t sa = (uint32_t)tt * 64u, sb = (uint32_t)tt * (uint32_t)B_STEP;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            if ((i < NLD0) != (h == 0)) continue;
            if (16 * (4 * i) < BM)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(dst + i * 4096), 16, u.voff[i], sa, 0, 0);
            else
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_ptr)(dst + i * 4096), 16, u.voff[i], sb, 0, 0);
        }
    };
    auto issue_stage = [&](const Unit& u, int t) { issue_half(u, t, 0); issue_half(u, t, 1); };

    // ---- fragment addressing: lane (r = lane&31, kh = lane>>5) reads chunk 2s+kh of row base+r
    const int fr = lane & 31, fkh = lane >> 5;
    const int fsw = (fr >> 2) & 3;
    int off_a[2], off_b[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        off_a[s] = (wm * (BM / 2) + fr) * 64 + (((2 * s + fkh) ^ fsw) << 4);
        off_b[s] = (BM + wn * (BN / 2) + fr) * 64 + (((2 * s + fkh) ^ fsw) << 4);
    }
    acc_t acc[FM][FN];
    u4_t fa[2][FM], fb[2][FN];
    auto read_frags = [&](int t, int s, int set) {
        const char* st = smem + (t % NS) * STAGE;
#pragma unroll
        for (int i = 0; i < FM; ++i) fa[set][i] = *reinterpret_cast<const u4_t*>(st + off_a[s] + i * 2048);
#pragma unroll
        for (int j = 0; j < FN; ++j) fb[set][j] = *reinterpret_cast<const u4_t*>(st + off_b[s] + j * 2048);
    };
    // `fresh`: the tile's first k-step, which starts from a zero operand instead of cleared accumulators
    auto mfma_step = [&](int set, auto fresh) {
        constexpr bool FRESH = decltype(fresh)::value;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const acc_t c = FRESH ? acc_t{} : acc[i][j];
                if constexpr (I8)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i4_t, fb[set][j]),
                                                                      __builtin_bit_cast(i4_t, fa[set][i]), c, 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8_t, fb[set][j]),
                                                                       __builtin_bit_cast(h8_t, fa[set][i]), c, 0, 0, 0);
            }
    };
    constexpr int NMF = FM * FN, NRD = FM + FN;

    // ---- pipeline: stage t is computed while stages t+1 .. t+NS-1 are in flight.  Every MFMA block
    // (one k-step) issues, between its first MFMAs, the fragment reads of the NEXT k-step into the
    // other register set, so LDS latency hides behind the block and nothing is read after it.
    // Between the two blocks of a stage the wave waits until stage t+1 has landed (at most `keep` younger direct
    // loads of this thread outstanding: loads retire in issue order) and meets the other waves; see
    // direct_stage_barrier.  One iteration, `left` = stages after t, known at compile time when below NS:
    // the last NS iterations issue only loads that exist and wait for exactly what is still on its way.
    static_assert(NS == 4 || NS == 3, "three or four stages");
    static_assert(NLD * (NS - 2) <= 48, "wait immediates stay well below the counter's range");
    using Yes = std::integral_constant<bool, true>;
    using I0 = std::integral_constant<int, 0>;
    using No = std::integral_constant<bool, false>;
    auto stage_body = [&](const Unit& u, int t, auto fresh, auto left_, auto extra_, auto&& after_last_load) {
        constexpr int LEFT = decltype(left_)::value;            // NS stands for "NS or more"
        constexpr int EXTRA = decltype(extra_)::value;          // other loads of this thread, younger than every stage load
        constexpr bool LD1 = LEFT >= NS - 1, LD0 = LEFT >= NS;   // stages t+NS-1 and t+NS exist
        constexpr int YOUNGER = LEFT - 1 < NS - 2 ? LEFT - 1 : NS - 2;   // whole stages issued after stage t+1
        // Slot (t-1) % NS was released by the previous barrier: it takes k-stage t+NS-1, half of the
        // loads in each of the two MFMA blocks that follow that barrier, so the memory pipe sees one
        // load per wave every few MFMAs instead of a burst.
        read_frags(t, 1, 1);
        if constexpr (LD1) issue_half(u, t + NS - 1, 1);
        if constexpr (LEFT == NS - 1) after_last_load();         // the last stage load of the unit is out
        mfma_step(0, fresh);                                     // (t, step 0)
        sched_interleave<NMF, NRD, 0, LD1 ? NLD - NLD0 : 0>();
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (LEFT >= 1) {
            // stage t+1 has landed for every wave and stage t is fully in registers
            direct_stage_barrier<NLD * YOUNGER + EXTRA>();
            read_frags(t + 1, 0, 0);
        }
        if constexpr (LD0) issue_half(u, t + NS, 0);
        mfma_step(1, No{});                                      // (t, step 1)
        sched_interleave<NMF, LEFT >= 1 ? NRD : 0, 0, LD0 ? NLD0 : 0>();
        __builtin_amdgcn_sched_barrier(0);
    };
    // The epilogue's per-wave patches: the start of LDS in the one-tile form; the END of LDS in the
    // persistent form (stage 3 and the last KiB of stage 2), which leaves stages 0 and 1 free to receive
    // the next unit's first k-stages while this unit's results are written out.
    constexpr int PATCH_BYTES = 4 * 32 * ((BN / 2) * 2 + 8);
    constexpr int PATCH_OFF = PERSIST ? NS * STAGE - PATCH_BYTES : 0;
    static_assert(!PERSIST || PATCH_OFF >= 2 * STAGE, "patches must stay clear of stages 0 and 1");

    bool ahead = false;                                      // stages 0 and 1 of `cur` are already on their way
    for (int vb = blockIdx.x;;) {
        // Stages past the end of a short K range (fewer than NS-1 stages) are clamped reloads into free slots; the
        // waits of the last iterations then cover them too, which is harmless.
        if (PERSIST && ahead) {
            // every wave has left the previous epilogue before stage 2 (whose end holds a patch) is refilled
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
            for (int t = 2; t < NS - 1; ++t) issue_stage(cur, t);
        } else {
#pragma unroll
            for (int t = 0; t < NS - 1; ++t) issue_stage(cur, t);
        }
        // loads retire in issue order and the stores of a previous epilogue are older than every load
        // counted here, so the same immediate holds for the first and for later units
        direct_stage_barrier<NLD * (NS - 2)>();
        if (cur.T >= NS) issue_half(cur, NS - 1, 0);
        read_frags(0, 0, 0);
        int t = 0;
        Unit nxt;
        bool more = false, nxt_ready = false;
        if (cur.T > NS) {
            if constexpr (PERSIST) {
                // the next unit's place and load offsets: integer work for the issue slots between the first MFMAs
                // (no branch in it, so that it can be scheduled into the block: past the last unit it describes the
                // last unit again and is not used)
                const int nb = vb + (int)gridDim.x;
                more = nb < nvirt;
                setup(more ? nb : nvirt - 1, nxt);
                nxt_ready = true;
            }
            stage_body(cur, 0, Yes{}, std::integral_constant<int, NS>{}, I0{}, NoHook{});
            t = 1;
        } else {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
        }
        for (; t + NS < cur.T; ++t) stage_body(cur, t, No{}, std::integral_constant<int, NS>{}, I0{}, NoHook{});
        // W8A8: this lane's row and column factors travel under the last stages: FM + FN two-byte loads, issued right
        // behind the unit's last stage load, so they are the youngest loads of the thread and the waits below make
        // room for exactly them.
        constexpr int NF = (KIND == KIND_W8A8) ? FM + FN : 0;
        EpiFactors<FM, FN> fac;
        auto load_factors = [&]() {
            if constexpr (KIND == KIND_W8A8) {
                asm volatile("" ::: "memory");
                epilogue_factors<BM, BN, FM, FN>(p, cur.m0, cur.n0, wave, lane, fac);
                asm volatile("" ::: "memory");
            }
        };
        if (cur.T < NS) load_factors();                          // no iteration below issues a stage load
        static_for<0, NS>([&](auto back) {                       // left = NS-1 .. 0
            constexpr int LEFT = NS - 1 - decltype(back)::value;
            if (t < cur.T && cur.T - 1 - t == LEFT) {
                stage_body(cur, t, No{}, std::integral_constant<int, LEFT>{}, std::integral_constant<int, NF>{}, load_factors);
                ++t;
            }
        });

        if constexpr (PERSIST) {
            if (!nxt_ready) {                                    // a short K range: no first iteration to hide it in
                more = vb + (int)gridDim.x < nvirt;
                if (more) setup(vb + (int)gridDim.x, nxt);
            }
        }
        // no direct load may outlive the workgroup or land in LDS that the epilogue reuses
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier\n\ts_nop 15\n\ts_nop 15" ::: "memory");

        if constexpr (PERSIST) {
            // the host uses this form without a split over K only
            // stages 0 and 1 of the next unit, spread over the first three row blocks of this unit's epilogue; all of
            // them are older than the last block's stores, which is what the wait at the top of the next unit counts on
            static_assert(FM >= 4, "the next unit's first loads are dealt over three row blocks");
            auto start_next = [&](int i) {
                if (more) {
                    if (i == 0) issue_stage(nxt, 0);
                    else if (i == 1) issue_half(nxt, 1, 0);
                    else if (i == 2) issue_half(nxt, 1, 1);
                }
            };
            const EpiFactors<FM, FN>* pre = (KIND == KIND_W8A8) ? &fac : nullptr;
            if (p.bias) gemm_epilogue<KIND, BM, BN, true, FM, FN>(p, acc, smem + PATCH_OFF, cur.m0, cur.n0, wave, lane, start_next, pre);
            else gemm_epilogue<KIND, BM, BN, false, FM, FN>(p, acc, smem + PATCH_OFF, cur.m0, cur.n0, wave, lane, start_next, pre);
            if (!more) break;
            cur = nxt;
            ahead = true;
            vb += (int)gridDim.x;
        } else {
            if (p.splits > 1) store_partial<BM, BN, FM, FN>(p, acc, cur.split, cur.m0, cur.n0, wave, lane);
            else {
                const EpiFactors<FM, FN>* pre = (KIND == KIND_W8A8) ? &fac : nullptr;
                if (p.bias) gemm_epilogue<KIND, BM, BN, true, FM, FN>(p, acc, smem, cur.m0, cur.n0, wave, lane, NoHook{}, pre);
                else gemm_epilogue<KIND, BM, BN, false, FM, FN>(p, acc, smem, cur.m0, cur.n0, wave, lane, NoHook{}, pre);
            }
            break;
        }
    }
#endif
}

// ---- host side ---------------------------------------------------------------------------------
// Test and tuning hooks of the calling host thread (0 = automatic): they change speed and, for the fp16 lanes, the
// order of the fp32 sums, never which entry point runs.
static thread_local int g_force_splits = 0;
extern "C" void kmi_gemm_force_splits(int splits) { g_force_splits = splits; }

// Number of K splits: only while the split workgroups still fit one round over the 256 CUs (a second
// round costs more than the idle CUs of the first), every split keeps at least eight 128-byte k-tiles,
// and the partial sums fit the registered workspace.  Measured on MI355X: splitting 192 or 224 tiles in
// two is 1.3-2x slower than running them as they are.
int kmi_pick_splits(int M, int N, int K, int BM, int BN, int ktiles, const Workspace& ws) {
    const long tiles = (long)((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    if (tiles <= 0) return 1;                                 // empty product (M or N not positive): nothing to split
    int s = 1;
    if (g_force_splits > 0) {
        s = g_force_splits;
        if (s > ktiles / 4) s = ktiles / 4;
    } else {
        s = (int)(256 / tiles);
        if (s > 8) s = 8;
        if (s > ktiles / 8) s = ktiles / 8;
    }
    const size_t per = (size_t)M * N * 4;
    if (per == 0 || ws.ptr == nullptr) return 1;
    if ((size_t)s * per > ws.bytes) s = (int)(ws.bytes / per);
    if (s > 1) {                                              // no empty split
        const int per_split = (ktiles + s - 1) / s;
        s = (ktiles + per_split - 1) / per_split;
    }
    return s < 2 ? 1 : s;
}

// Compute units of the current device (0 if the query fails), asked once per device.
static int cu_count() {
    static std::atomic<int> cached[KMI_NOALLOC_MAX_DEVICES];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= KMI_NOALLOC_MAX_DEVICES) return 0;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

template <int KIND, int BM, int BN, bool TILED, int NS_ = 4>
static int launch_gemm(const GemmArgs& a_in, const Workspace& ws, hipStream_t st, int n_begin = 0, int n_cols = -1) {
    GemmArgs a = a_in;
    a.group_m = kmi_forced_group_m();
    a.n_begin = n_begin;
    a.n_cols = n_cols < 0 ? a.N - n_begin : n_cols;
    const bool whole = (a.n_begin == 0 && a.n_cols == a.N);
    constexpr bool DIRECT = (KIND == KIND_F16 || KIND == KIND_W8A8 || KIND == KIND_W8A8_ACC);
    constexpr int NS = NS_;
    constexpr size_t lds = DIRECT ? (size_t)NS * (BM + BN) * 64 : 2 * (size_t)(BM + BN) * 128;
    void (*fn)(GemmArgs);
    if constexpr (DIRECT) fn = gemm_direct_kernel<KIND, BM, BN, TILED, NS>;
    else fn = gemm_kernel<KIND, BM, BN, false>;
    if (lds > 64 * 1024) {
        static thread_local bool raised = false;   // per kernel instantiation, per thread
        if (!raised) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
                return kmi_set_error(KMI_E_LAUNCH, "gemm: cannot raise the dynamic LDS limit to %zu bytes", lds);
            raised = true;
        }
    }
    const bool i8 = (KIND == KIND_W8A8 || KIND == KIND_W8A8_ACC);
    // units the kernels split K in: 128-byte k-tiles (register-staged) or 64-byte stages (direct)
    const int units = (int)(((long)a.K * (i8 ? 1 : 2)) >> (DIRECT ? 6 : 7));
    a.splits = whole ? kmi_pick_splits(a.M, a.N, a.K, BM, BN, DIRECT ? units / 2 : units, ws) : 1;
    a.partial = a.splits > 1 ? ws.ptr : nullptr;
    dim3 grid(((a.n_cols + BN - 1) / BN) * ((a.M + BM - 1) / BM) * a.splits), block(256);
    if constexpr (DIRECT && TILED && BM == 256 && (BN == 256 || BN == 192) && NS == 4) {
        // More tiles than CUs: one workgroup per CU walks the tiles (same order, same XCD per tile) and starts
        // the next tile's loads before it writes the current one out.  Its weight offsets are 32-bit.
        const int cus = cu_count();
        if (a.splits == 1 && cus > 0 && (long)grid.x > cus && (long)a.N * a.K * (i8 ? 1 : 2) < (1L << 32)) {
            void (*pfn)(GemmArgs) = gemm_direct_kernel<KIND, BM, BN, TILED, NS, true>;
            static thread_local bool praised = false;
            if (!praised) {
                if (hipFuncSetAttribute(reinterpret_cast<const void*>(pfn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
                    return kmi_set_error(KMI_E_LAUNCH, "gemm: cannot raise the dynamic LDS limit to %zu bytes", lds);
                praised = true;
            }
            fn = pfn;
            grid.x = (unsigned)cus;
        }
    }
    hipLaunchKernelGGL(fn, grid, block, lds, st, a);
    if (a.splits > 1) {
        const long quads = (long)a.M * a.N / 4;
        hipLaunchKernelGGL(splitk_reduce_kernel<KIND>, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, st, a);
    }
    return KMI_OK;
}

// Launch of the wave-private-weights kernel (W4A16, small M).  K is split over KH wave quartets inside the
// workgroup and, when the tiles alone leave CUs idle, over workgroups as well (partials + reduce kernel).
template <int BM, int KH = 2>
static int launch_w4a16_wp(const GemmArgs& a_in, const Workspace& ws, hipStream_t st) {
    GemmArgs a = a_in;
    a.group_m = kmi_forced_group_m();
    constexpr int PF = 4;                                        // k-tiles in flight per wave (8 measured 3-5 % slower at 32 / 64 rows)
    constexpr size_t lds = (size_t)KH * (PF + 1) * BM * 128;
    static_assert(lds <= 160 * 1024, "the activation ring must fit the LDS of a CU");
    void (*fn)(GemmArgs) = gemm_w4a16_wp_kernel<BM, KH, PF>;
    static thread_local bool raised = false;
    if (lds > 64 * 1024 && !raised) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return kmi_set_error(KMI_E_LAUNCH, "gemm: cannot raise the dynamic LDS limit to %zu bytes", lds);
        raised = true;
    }
    a.n_begin = 0;
    a.n_cols = a.N;
    const int tiles = ((a.M + BM - 1) / BM) * ((a.N + 127) / 128);
    const int kt_all = a.K / 64;
    int s = g_force_splits > 0 ? g_force_splits : 256 / tiles;
    if (s > 8) s = 8;
    if (s > kt_all / 16) s = kt_all / 16;                       // at least 16 k-tiles (8 per quartet) per split
    const size_t per = (size_t)a.M * a.N * 4;
    if (ws.ptr == nullptr || per == 0) s = 1;
    else if ((size_t)s * per > ws.bytes) s = (int)(ws.bytes / per);
    if (s < 1) s = 1;
    if (s > 1) {                                                 // whole quartet rounds per split, no empty split
        const int per_split = ((kt_all + s - 1) / s + KH - 1) / KH * KH;
        s = (kt_all + per_split - 1) / per_split;
    }
    a.splits = s;
    a.partial = s > 1 ? ws.ptr : nullptr;
    hipLaunchKernelGGL(fn, dim3(tiles * s), dim3(256 * KH), lds, st, a);
    if (s > 1) {
        const long quads = (long)a.M * a.N / 4;
        hipLaunchKernelGGL(splitk_reduce_kernel<KIND_W4A16>, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, st, a);
    }
    return KMI_OK;
}

// Tile choice: the largest tile that still yields about one workgroup per CU.  row_bytes = K for the int8-operand
// kinds (0 for the others, which keep the plain rule: 256-row tiles from 180 workgroups, 128-row tiles from 128).
// Measured on MI355X (W8A8, tiled weights, Llama-3-8B / -70B and Qwen2.5-7B shapes):
//   * the 256 tile pays from ~144 workgroups on (256 x 37888 x 3584: 50 against 68 us with the 128 tile), and on
//     long rows already when a split over K brings it there, provided every split keeps ~9000 bytes of K
//     (768 x 8192 x 28672: 96 tiles x 2 splits, 189 against 284 us; 2048 x 4096 x 14336 split in two loses);
//   * with short rows 128 workgroups of the 128 tile lose to 256 of the 64-row tile (512 x 4096 x 4096: 21.1
//     against 15.9 us) and win from ~144 on; with long rows the 128 tile wins from ~48 workgroups
//     (384 x 4096 x 14336: 36.0 against 43.7 us);
//   * where 128-row tiles pad M further than 64-row tiles and would not fill the GPU while the 64-row tiles do,
//     the latter win (192 x 10240 x 8192: 28.8 against 31.9 us; not at 192 x 28672 x 4096: 52.5 against 43.7 us).
static int pick_tile(int M, int N, long row_bytes) {
    if (M <= 0 || N <= 0) return 64;                          // empty product: the entry points return before any launch
    auto wgs = [&](int bm, int bn) { return (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    if (row_bytes <= 0) {
        if (M > 128 && wgs(256, 256) >= 180) return 256;
        if (M > 64 && wgs(128, 128) >= 128) return 128;
        return 64;
    }
    long split = 256 / wgs(256, 256);
    if (split > row_bytes / 9000) split = row_bytes / 9000;
    if (split < 1) split = 1;
    if (M > 128 && wgs(256, 256) * split >= 144) {
        // One round either way: 256 x 192 tiles (N a multiple of 192 and of the 128-row weight strips; selector 320,
        // tiled weights only) put the same output on more CUs with less work each.  The narrower tile is less efficient
        // per MFMA, so the gain is small: 2048 x 6144 x 4096 51.9 against 54.9 us, 2048 x 4608 x 3584 37.9 against 45.1.
        // The same holds for whole rounds of them where the wider tile leaves a ragged one (4096 x 6144 x 4096: two
        // rounds, 88.1 against 93.7 us for 1.5 rounds of 256 x 256 with a 128 x 128 tail).
        const long w192 = wgs(256, 192), w256 = wgs(256, 256);
        if (split == 1 && N % 384 == 0 && w256 < w192 && (w192 <= 256 || (w192 % 256 == 0 && w256 % 256 != 0))) return 320;
        return 256;
    }
    // too few 256 x 256 tiles for the CUs, yet the rows are too short to split: 256 x 128 tiles, two workgroups per CU
    // (selector 192), when they come to 192..256 (2048 x 4096 x 14336: 119 against 130 us with 128 x 128 tiles and 134
    // with 256 x 256; 1536 x 4096 x 14336: 95 against 106; on long rows the split 256 tile wins: 1024 x 8192 x 28672)
    if (M >= 1024 && row_bytes <= 20000 && wgs(256, 256) < 144 && wgs(256, 128) >= 192 && wgs(256, 128) <= 256) return 192;
    const bool pad128 = (M + 127) / 128 * 2 > (M + 63) / 64;
    if (pad128 && wgs(64, 128) >= 200 && wgs(128, 128) < 256) return 64;
    if (M > 64 && wgs(128, 128) >= (row_bytes >= 8192 ? 48 : 144)) return 128;
    return 64;
}
extern "C" int kmi_gemm_pick_tile(int M, int N, int K) { return pick_tile(M, N, K); }
int kmi_pick_tile_rows(int M, int N, long row_bytes) { return pick_tile(M, N, row_bytes); }

// Variant of the wave-private-weights W4A16 kernel for an M x N x K product: rows per tile (0 = run the
// register-staged kernel instead) and wave quartets per workgroup.  Measured on MI355X (Llama-3-8B and -70B
// shapes): the wave-private kernel wins while its tiles fit one or two rounds over the CUs; 64-row tiles while
// they fit one round, 128-row tiles beyond that or when K is long and there are at least 64 of them (the decode of
// a weight is then shared by twice as many rows: 10240 x 8192 at M=128 37 against 44 us), a single quartet per
// workgroup once there are more tiles than CUs.  Beyond two rounds the register-staged kernel takes over only
// where it runs its 256-row tile without more row padding than 128-row tiles would have (28672 x 4096: M=512
// 131 against 141 us for the staged kernel, M=384 126 against 109 us).  Very few tiles: 32-row tiles up to M=64
// (4096 x 4096 at M=64: 12.5 against 13.7 us).  Where 128-row tiles would pad M further than 64-row tiles (M = 192,
// 320, ...) the 64-row variants are preferred (37888 x 3584 at M=192: 71 against 84 us).
struct WpChoice { int rows, quartets; };
static WpChoice pick_wp(int M, int N, int K) {
    if (M > 1024) return {0, 0};
    const long strips = (N + 127) / 128;
    const long tiles32 = ((M + 31) / 32) * strips, tiles64 = ((M + 63) / 64) * strips, tiles128 = ((M + 127) / 128) * strips;
    const bool pad128 = (M + 127) / 128 * 2 > (M + 63) / 64;      // 128-row tiles pad M further than 64-row tiles
    if (M <= 32) return {32, 2};
    if (M <= 64) return (tiles32 <= 80 && K <= 8192) ? WpChoice{32, 2} : WpChoice{64, 2};
    // long K: 128-row tiles from 64 tiles on, unless they pad more, cannot be split over K and 64-row tiles fit a round
    if (K >= 8192 && tiles128 >= 64 && tiles128 <= 256 && !(pad128 && tiles128 > 128 && tiles64 <= 256)) return {128, 2};
    if (tiles64 <= 256) return {64, 2};
    if (tiles128 <= 256) return {128, 2};
    if (pad128 && tiles64 <= 2048) return {64, 1};
    if (tiles128 <= 512) return {128, 1};
    const bool staged256 = pick_tile(M, N, 0) == 256 && (M + 255) / 256 * 2 == (M + 127) / 128;
    return staged256 ? WpChoice{0, 0} : WpChoice{128, 1};
}
extern "C" int kmi_gemm_w4a16_wp_rows(int M, int N, int K) { return pick_wp(M, N, K).rows; }

template <int KIND, bool TILED>
static int dispatch_gemm(const GemmArgs& a, const Workspace& ws, hipStream_t st, int force_tile) {
    int tile = force_tile > 0 ? force_tile : pick_tile(a.M, a.N, (KIND == KIND_W8A8 || KIND == KIND_W8A8_ACC) ? (long)a.K : 0);
    if constexpr (KIND == KIND_W4A16) {
        // selectors 1032 / 1064 / 1128 force the wave-private-weights kernel with 32 / 64 / 128 rows per tile
        if (tile == 1032) return launch_w4a16_wp<32>(a, ws, st);
        if (tile == 1064) return launch_w4a16_wp<64>(a, ws, st);
        if (tile == 1128) return launch_w4a16_wp<128>(a, ws, st);
        if (tile == 2032) return launch_w4a16_wp<32, 1>(a, ws, st);      // 2xxx: one wave quartet per workgroup
        if (tile == 2064) return launch_w4a16_wp<64, 1>(a, ws, st);
        if (tile == 2128) return launch_w4a16_wp<128, 1>(a, ws, st);
        if (force_tile == 0) {
            const WpChoice c = pick_wp(a.M, a.N, a.K);
            if (c.rows == 32) return launch_w4a16_wp<32>(a, ws, st);
            if (c.rows == 64 && c.quartets == 2) return launch_w4a16_wp<64>(a, ws, st);
            if (c.rows == 64) return launch_w4a16_wp<64, 1>(a, ws, st);
            if (c.rows == 128 && c.quartets == 2) return launch_w4a16_wp<128>(a, ws, st);
            if (c.rows == 128) return launch_w4a16_wp<128, 1>(a, ws, st);
        }
    }
    if (tile == 320 && !(TILED && (KIND == KIND_W8A8 || KIND == KIND_W8A8_ACC || KIND == KIND_F16)))
        tile = 256;                                          // row-major operands and the other kinds: 256 x 256 as before
    if (tile == 256 && force_tile == 0) {
        // Round quantisation: TM x TN tiles run in rounds of 256 (one workgroup per CU).  When the last
        // round would be at most ~60 % full, the columns it would cover are run with the 128x128 tile
        // instead (four times as many workgroups of a quarter of the work, two per CU), so the tail costs
        // about half a round; the two launches cover disjoint column ranges split at a multiple of 256.
        const int TM = (a.M + 255) / 256, TN = (a.N + 255) / 256;
        const int tiles = TM * TN, rem = tiles % 256;
        const int head_cols = ((tiles - rem) / TM);          // column tiles that make up whole rounds
        if (tiles > 256 && rem > 0 && head_cols > 0 && (TN - head_cols) * TM <= 160) {
            const int rc = launch_gemm<KIND, 256, 256, TILED>(a, ws, st, 0, head_cols * 256);
            if (rc != KMI_OK) return rc;
            return launch_gemm<KIND, 128, 128, TILED>(a, ws, st, head_cols * 256, a.N - head_cols * 256);
        }
    }
    switch (tile) {
        case 256: return launch_gemm<KIND, 256, 256, TILED>(a, ws, st);
        case 320:                                        // 256 rows x 192 columns (tiled weights): N = 6144 in whole tiles
            if constexpr (TILED && (KIND == KIND_W8A8 || KIND == KIND_W8A8_ACC || KIND == KIND_F16)) return launch_gemm<KIND, 256, 192, TILED>(a, ws, st);
            break;
        case 192:                                        // 256 rows x 128 columns, three stages, two workgroups per CU
            if constexpr (KIND == KIND_W8A8 || KIND == KIND_W8A8_ACC || KIND == KIND_F16) return launch_gemm<KIND, 256, 128, TILED, 3>(a, ws, st);
            break;
        case 128: return launch_gemm<KIND, 128, 128, TILED>(a, ws, st);
        case 64: return launch_gemm<KIND, 64, 128, TILED>(a, ws, st);
    }
    return kmi_set_error(KMI_E_SHAPE, "gemm: unknown tile selector %d", tile);
}

int kmi_gemm_args_check(const char* fn, const GemmArgs& a, bool tiled) {
    if (!a.out || !a.a || !a.b) return kmi_set_error(KMI_E_NULL, "%s: NULL pointer argument", fn);
    if (!kmi_aligned16(a.a) || !kmi_aligned16(a.b)) return kmi_set_error(KMI_E_ALIGN, "%s: operands must be 16-byte aligned", fn);
    if (a.M < 0 || a.N <= 0 || a.K <= 0 || (a.K & 127) || (a.N & 3))
        return kmi_set_error(KMI_E_SHAPE, "%s: need M>=0, N%%4==0, K%%128==0 (M=%d N=%d K=%d)", fn, a.M, a.N, a.K);
    if (tiled && (a.N % KMI_TILE_N)) return kmi_set_error(KMI_E_SHAPE, "%s: tiled operand needs N%%%d==0 (N=%d)", fn, KMI_TILE_N, a.N);
    if ((long)a.M * a.K * 2 >= (1L << 32) || (long)a.N * a.K * 2 >= (1L << 32))
        return kmi_set_error(KMI_E_SHAPE, "%s: an operand of 4 GiB or more is not supported (M=%d N=%d K=%d)", fn, a.M, a.N, a.K);
    return KMI_OK;
}

static thread_local int g_force_tile = 0;
extern "C" void kmi_gemm_force_tile(int tile) { g_force_tile = tile; }
int kmi_forced_tile() { return g_force_tile; }
static thread_local int g_force_group_m = 0;
extern "C" void kmi_gemm_force_group_m(int group_m) { g_force_group_m = group_m; }
int kmi_forced_group_m() { return g_force_group_m; }

int kmi_workspace_check(const char* fn, const void* workspace, size_t bytes, Workspace& ws) {
    if (workspace && !kmi_aligned16(workspace)) return kmi_set_error(KMI_E_ALIGN, "%s: workspace must be 16-byte aligned", fn);
    ws.ptr = const_cast<void*>(workspace);
    ws.bytes = workspace ? bytes : 0;
    return KMI_OK;
}

#define KMI_GEMM_BODY(NAME, KIND, TILED)                                      \
    Workspace ws;                                                             \
    int rc = kmi_gemm_args_check(NAME, a, TILED);                                      \
    if (rc != KMI_OK) return rc;                                              \
    rc = kmi_workspace_check(NAME, workspace, workspace_bytes, ws);               \
    if (rc != KMI_OK) return rc;                                              \
    if (a.M == 0) return KMI_OK;                                              \
    rc = dispatch_gemm<KIND, TILED>(a, ws, static_cast<hipStream_t>(stream), g_force_tile); \
    if (rc != KMI_OK) return rc;                                              \
    return kmi_check_launch(NAME);

extern "C" int kmi_gemm_w4a16(void* out, const void* x, const void* qweight, const void* scales, const void* szeros,
                              const void* bias, int M, int N, int K, int G, void* workspace, size_t workspace_bytes,
                              void* stream) {
    if (G != 128) return kmi_set_error(KMI_E_GROUP, "kmi_gemm_w4a16: group size %d unsupported (128 only)", G);
    if (!scales || !szeros) return kmi_set_error(KMI_E_NULL, "kmi_gemm_w4a16: NULL scale table");
    GemmArgs a{out, x, qweight, (const half_t*)scales, (const half_t*)szeros, nullptr, nullptr, (const half_t*)bias, M, N, K, nullptr, 1, 0, N};
    KMI_GEMM_BODY("kmi_gemm_w4a16", KIND_W4A16, false)
}

extern "C" int kmi_gemm_w8a16(void* out, const void* x, const void* w8, const void* wscales, const void* bias,
                              int M, int N, int K, void* workspace, size_t workspace_bytes, void* stream) {
    if (!wscales) return kmi_set_error(KMI_E_NULL, "kmi_gemm_w8a16: NULL wscales");
    GemmArgs a{out, x, w8, nullptr, nullptr, (const half_t*)wscales, nullptr, (const half_t*)bias, M, N, K, nullptr, 1, 0, N};
    KMI_GEMM_BODY("kmi_gemm_w8a16", KIND_W8A16, false)
}

extern "C" int kmi_gemm_w8a8(void* out, const void* a8, const void* w8, const void* wscales, const void* ascales,
                             const void* bias, int M, int N, int K, void* workspace, size_t workspace_bytes, void* stream) {
    if (!wscales || !ascales) return kmi_set_error(KMI_E_NULL, "kmi_gemm_w8a8: NULL scale vector");
    GemmArgs a{out, a8, w8, nullptr, nullptr, (const half_t*)wscales, (const half_t*)ascales, (const half_t*)bias, M, N, K, nullptr, 1, 0, N};
    KMI_GEMM_BODY("kmi_gemm_w8a8", KIND_W8A8, false)
}

extern "C" int kmi_gemm_w8a8_acc_i32(void* acc, const void* a8, const void* w8, int M, int N, int K, void* workspace,
                                     size_t workspace_bytes, void* stream) {
    GemmArgs a{acc, a8, w8, nullptr, nullptr, nullptr, nullptr, nullptr, M, N, K, nullptr, 1, 0, N};
    KMI_GEMM_BODY("kmi_gemm_w8a8_acc_i32", KIND_W8A8_ACC, false)
}

extern "C" int kmi_gemm_f16(void* out, const void* x, const void* w16, const void* bias, int M, int N, int K,
                            void* workspace, size_t workspace_bytes, void* stream) {
    GemmArgs a{out, x, w16, nullptr, nullptr, nullptr, nullptr, (const half_t*)bias, M, N, K, nullptr, 1, 0, N};
    KMI_GEMM_BODY("kmi_gemm_f16", KIND_F16, false)
}

extern "C" int kmi_gemm_w8a8_tiled(void* out, const void* a8, const void* w8t, const void* wscales, const void* ascales,
                                   const void* bias, int M, int N, int K, void* workspace, size_t workspace_bytes,
                                   void* stream) {
    if (!wscales || !ascales) return kmi_set_error(KMI_E_NULL, "kmi_gemm_w8a8_tiled: NULL scale vector");
    GemmArgs a{out, a8, w8t, nullptr, nullptr, (const half_t*)wscales, (const half_t*)ascales, (const half_t*)bias, M, N, K, nullptr, 1, 0, N};
    KMI_GEMM_BODY("kmi_gemm_w8a8_tiled", KIND_W8A8, true)
}

extern "C" int kmi_gemm_f16_tiled(void* out, const void* x, const void* w16t, const void* bias, int M, int N, int K,
                                  void* workspace, size_t workspace_bytes, void* stream) {
    GemmArgs a{out, x, w16t, nullptr, nullptr, nullptr, nullptr, (const half_t*)bias, M, N, K, nullptr, 1, 0, N};
    KMI_GEMM_BODY("kmi_gemm_f16_tiled", KIND_F16, true)
}

// ---- the W4A16 GEMM for callers that cannot allocate --------------------------------------------------------------
// Same kernels as kmi_gemm_w4a16; the split-K partial sums live in a file-scope device array instead of a buffer the
// caller brings.  Every GPU the library's code object is loaded on holds its own copy of the array until the process
// ends, at its own address: that address is looked up once per device and is what the kernels receive.
#define KMI_NOALLOC_SCRATCH_BYTES (16u << 20)
static __device__ __align__(256) unsigned char scratch[KMI_NOALLOC_SCRATCH_BYTES];
static void* g_scratch_ptr[KMI_NOALLOC_MAX_DEVICES] = {};      // device address of `scratch`, per device ordinal
static std::mutex g_scratch_mutex;

static int scratch_of_current_device(const char* fn, void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= KMI_NOALLOC_MAX_DEVICES)
        return kmi_set_error(KMI_E_LAUNCH, "%s: cannot identify the current device (ordinal %d)", fn, dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            return kmi_set_error(KMI_E_LAUNCH, "%s: hipGetSymbolAddress failed on device %d: %s", fn, dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return KMI_OK;
}

extern "C" int kmi_gemm_w4a16_noalloc(void* out, const void* x, const void* qweight, const void* scales, const void* szeros,
                                      const void* bias, int M, int N, int K, int G, void* stream) {
    const char* fn = "kmi_gemm_w4a16_noalloc";
    if (G != 128) return kmi_set_error(KMI_E_GROUP, "%s: group size %d unsupported (128 only)", fn, G);
    if (!scales || !szeros) return kmi_set_error(KMI_E_NULL, "%s: NULL scale table", fn);
    GemmArgs a{out, x, qweight, (const half_t*)scales, (const half_t*)szeros, nullptr, nullptr, (const half_t*)bias, M, N, K, nullptr, 1, 0, N};
    int rc = kmi_gemm_args_check(fn, a, false);
    if (rc != KMI_OK) return rc;
    if ((long)M * N > KMI_NOALLOC_MAX_OUTPUTS)
        return kmi_set_error(KMI_E_M_RANGE, "%s: M*N = %ld outputs exceed the %d this entry point's built-in scratch serves "
                             "(use kmi_gemm_w4a16 with a workspace)", fn, (long)M * N, KMI_NOALLOC_MAX_OUTPUTS);
    if (a.M == 0) return KMI_OK;
    static_assert((size_t)KMI_NOALLOC_MAX_OUTPUTS * 4 * 8 <= KMI_NOALLOC_SCRATCH_BYTES, "eight fp32 slices of the largest output");
    Workspace ws{nullptr, KMI_NOALLOC_SCRATCH_BYTES};
    rc = scratch_of_current_device(fn, &ws.ptr);
    if (rc != KMI_OK) return rc;
    rc = dispatch_gemm<KIND_W4A16, false>(a, ws, static_cast<hipStream_t>(stream), g_force_tile);
    if (rc != KMI_OK) return rc;
    return kmi_check_launch(fn);
}

// Host-only query: the number of K splits a call of the given lane would use with a workspace of that size
// (1 = none).  lane: 0 W4A16, 1 W8A16, 2 W8A8, 3 fp16; tiled as in the *_tiled entry points.
extern "C" int kmi_gemm_splits_for(int lane, int M, int N, int K, size_t workspace_bytes) {
    if (lane < 0 || lane > 3 || M <= 0 || N <= 0 || K <= 0 || (K & 127))
        return kmi_set_error(KMI_E_SHAPE, "kmi_gemm_splits_for: bad arguments (lane=%d M=%d N=%d K=%d)", lane, M, N, K);
    const Workspace ws{workspace_bytes ? reinterpret_cast<void*>(16) : nullptr, workspace_bytes};
    const size_t per = (size_t)M * N * 4;
    if (lane == 0) {
        const WpChoice c = pick_wp(M, N, K);
        if (c.rows) {                                         // mirrors launch_w4a16_wp
            const int tiles = ((M + c.rows - 1) / c.rows) * ((N + 127) / 128), kt_all = K / 64, KH = c.quartets;
            int s = g_force_splits > 0 ? g_force_splits : 256 / tiles;
            if (s > 8) s = 8;
            if (s > kt_all / 16) s = kt_all / 16;
            if (ws.ptr == nullptr) s = 1;
            else if ((size_t)s * per > ws.bytes) s = (int)(ws.bytes / per);
            if (s < 1) s = 1;
            if (s > 1) {
                const int per_split = ((kt_all + s - 1) / s + KH - 1) / KH * KH;
                s = (kt_all + per_split - 1) / per_split;
            }
            return s;
        }
    }
    const bool i8 = lane == 2;
    const int tile = g_force_tile > 0 ? g_force_tile : pick_tile(M, N, i8 ? (long)K : 0);
    if (tile == 256 && g_force_tile == 0) {                   // mirrors the head/tail rule of dispatch_gemm: no split
        const int TM = (M + 255) / 256, TN = (N + 255) / 256, tiles = TM * TN, rem = tiles % 256;
        const int head_cols = (tiles - rem) / TM;
        if (tiles > 256 && rem > 0 && head_cols > 0 && (TN - head_cols) * TM <= 160) return 1;
    }
    const int BM = tile == 64 ? 64 : tile == 128 ? 128 : 256, BN = (tile == 256) ? 256 : (tile == 320) ? 192 : 128;
    const int ktiles = (int)(((long)K * (i8 ? 1 : 2)) >> 7);
    return kmi_pick_splits(M, N, K, BM, BN, ktiles, ws);
}

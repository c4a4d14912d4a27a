// W4A8: int8 activations x packed uint4 weights on v_mfma_i32_32x32x32_i8, without a converted copy of the weight.
//
//   acc[m,n] = sum_k a8[m,k] * W8[n,k],   W8[n,k] = (int8) fma_f16(q[n,k], scales_to8[k/128,n], scaled_zeros_to8[k/128,n])
//
// i.e. exactly the int8 weight the int4 -> int8 converter would write (truncation toward zero, clipped), decoded on
// the way from HBM to LDS, so accumulators and fp16 outputs are bit-identical to converter + W8A8 GEMM while the
// conversion pass (N*K/2 bytes read, N*K written, N*K read again) disappears.
//
// Decoding by table.  For one row n and one 128-wide group g the converted value depends on the nibble only: sixteen
// possible bytes.  The thread that stages row n builds that 16-byte table once per group (eight packed fp16 FMAs and
// the converter's own clip-and-truncate) into four registers and then looks nibbles up with v_perm_b32, four at a
// time: the low three bits of four nibbles select from either half of the table (two v_perm), bit 3 picks between the
// two results (a third v_perm whose selector is 0x03020100 | 4*bit3).  One more v_perm per output word puts the bytes
// into K order (a packed word holds k = 2t, 16+2t, 2t+1, 17+2t, ...).  About 1.9 VALU operations per weight.
//
// Pipeline.  256 threads = 2x2 waves, 32x32 MFMA tiles, workgroup tile BM x BN, NS LDS stages of (BM+BN) rows x
// 64 bytes of K, rows XOR-swizzled as in the operand-copy kernel.  Activations travel global -> LDS directly
// (buffer_load ... lds), four stages ahead.  A thread owns one weight row of the tile (BN = 256: both 16-byte chunks
// of the row per stage; BN = 128: one chunk): its packed chunks are loaded into registers four stages ahead, decoded
// two stages ahead between the MFMAs of the current stage, and written to the stage's LDS rows with 16-byte stores.
// Iteration t: wait for everything issued up to two iterations ago; [MFMA block of k-step 0 | table of the next
// group (even t), decode of chunk 0 of stage t+2, second half of the activation loads of stage t+3]; barrier;
// [MFMA block of k-step 1 | decode of chunk 1, first half of the activation loads and the packed chunks of stage
// t+4, scale and zero of the group of stage t+4 (even t)].
#include "gemm_parts.h"
#include "prep_bodies.h"

template <int N>
__device__ __forceinline__ void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// The converter's arithmetic for the nibble values 4J .. 4J+3: table byte q = (int8) clip(fma_f16(q, s, z)).
template <int J>
__device__ __forceinline__ uint32_t w4a8_table_word(half_t s, half_t z) {
    const h2_t s2 = {s, s}, z2 = {z, z};
    const h2_t q01 = {(half_t)(float)(4 * J), (half_t)(float)(4 * J + 1)};
    const h2_t q23 = {(half_t)(float)(4 * J + 2), (half_t)(float)(4 * J + 3)};
    return pack_i8x4(pk_fma(q01, s2, z2), pk_fma(q23, s2, z2));
}

// The same for the nibble values held in q01 / q23 (four consecutive values as fp16 pairs): the form used when two
// threads share a weight row and each builds half of the row's table.
__device__ __forceinline__ uint32_t w4a8_table_word_of(h2_t q01, h2_t q23, half_t s, half_t z) {
    const h2_t s2 = {s, s}, z2 = {z, z};
    return pack_i8x4(pk_fma(q01, s2, z2), pk_fma(q23, s2, z2));
}

// Integer factors (the form a per-group integer dequantiser uses): table byte q = (q * scale + zero) modulo 256 read as
// int8, `scale` an unsigned byte, `zero` the pre-multiplied (negated) zero point as a byte.  `wbase` holds the four nibble
// values of the word, one per byte.  The products are taken per byte pair so that no carry crosses a byte, whatever the
// scale; the add wraps per byte.
__device__ __forceinline__ uint32_t w4a8_table_word_int(uint32_t wbase, uint32_t scale, uint32_t zero) {
    const uint32_t even = ((wbase & 0x00FF00FFu) * (scale & 0xFFu)) & 0x00FF00FFu;
    const uint32_t odd = (((wbase >> 8) & 0x00FF00FFu) * (scale & 0xFFu)) & 0x00FF00FFu;
    const uint32_t prod = even | (odd << 8);
    const uint32_t z4 = zero * 0x01010101u;
    return ((prod & 0x7F7F7F7Fu) + (z4 & 0x7F7F7F7Fu)) ^ ((prod ^ z4) & 0x80808080u);
}

// Four nibbles (`idx3`: their low three bits, one per byte; `sel_hi`: 0x03020100 + 4 * bit 3, one per byte) -> four
// table bytes.
__device__ __forceinline__ uint32_t w4a8_lookup(const uint32_t (&L)[4], uint32_t idx3, uint32_t sel_hi) {
    const uint32_t lo = __builtin_amdgcn_perm(L[1], L[0], idx3);
    const uint32_t hi = __builtin_amdgcn_perm(L[3], L[2], idx3);
    return __builtin_amdgcn_perm(hi, lo, sel_hi);
}

// One 16-byte chunk (32 weights of one row; word t, nibble a, half c is k = 8a + 2t + c) -> 32 int8 in K order, in
// small steps that the caller places between its MFMAs.  First the bytes of two words are gathered so that the nibbles
// of four consecutive k share a register (byte 2c + a/2 of word t holds nibble a of half c):
//   x[h] = bytes 0, 2 of words 2h, 2h+1: low nibbles a = 0 (k = 4h .. 4h+3), high nibbles a = 1 (k = 8 + 4h ..)
//   y[h] = bytes 1, 3 of words 2h, 2h+1: low nibbles a = 2 (k = 16 + 4h ..), high nibbles a = 3 (k = 24 + 4h ..)
// then output word j (k = 4j .. 4j+3) is one table lookup of the low or the high nibbles of one of them.
struct W4a8Masks { uint32_t m7, m4, ident; };
__device__ __forceinline__ W4a8Masks w4a8_masks() {
    W4a8Masks c{0x07070707u, 0x04040404u, 0x03020100u};
    asm volatile("" : "+s"(c.m7), "+s"(c.m4), "+v"(c.ident));   // held in registers: v_and_or_b32 takes no literal
    return c;
}
__device__ __forceinline__ void w4a8_gather_nibbles(const u4_t& u, uint32_t (&xy)[4]) {    // xy = x[0], x[1], y[0], y[1]
    xy[0] = __builtin_amdgcn_perm(u[1], u[0], 0x06040200u);
    xy[1] = __builtin_amdgcn_perm(u[3], u[2], 0x06040200u);
    xy[2] = __builtin_amdgcn_perm(u[1], u[0], 0x07050301u);
    xy[3] = __builtin_amdgcn_perm(u[3], u[2], 0x07050301u);
}
template <int J>      // output word J of the chunk: k = 4J .. 4J+3
__device__ __forceinline__ uint32_t w4a8_decode_word(const uint32_t (&xy)[4], const uint32_t (&L)[4], const W4a8Masks& c) {
    static_assert(J >= 0 && J < 8, "eight output words per chunk");
    const uint32_t w = xy[(J & 1) + 2 * (J >> 2)];             // x[J&1] for k < 16, y[J&1] beyond
    if constexpr (((J >> 1) & 1) == 0) return w4a8_lookup(L, w & c.m7, ((w >> 1) & c.m4) | c.ident);       // low nibbles
    else return w4a8_lookup(L, (w >> 4) & c.m7, ((w >> 5) & c.m4) | c.ident);                                // high nibbles
}

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// KH = 2: two wave quartets per workgroup.  Each is the whole pipeline below on its own half of the workgroup's K range
// with its own LDS ring; they share nothing but the barriers, so on every SIMD one wave's decode instructions issue under
// the other's MFMAs -- what two workgroups per CU do for each other, without a second output tile or partial sums in
// memory.  Their int32 accumulators meet in LDS at the end (integers: the order does not matter).  Small tiles only:
// two waves per SIMD leave 256 registers each.
//
// MW = 2: two wave quartets on ONE pipeline.  Quartet h multiplies rows h*BM/2 .. of the tile against all BN columns and
// both read the same LDS stages, but the staging is divided: quartet 0 loads, decodes and stores the weights, quartet 1
// brings in all the activation rows.  With one wave per SIMD every instruction of the stage -- some 200 against 32
// MFMAs -- queues on that wave's own issue port, which the MFMAs cannot cover, and a 64-lane load holds the port far
// longer than a vector instruction; with the roles apart the decoding wave never waits behind a load, and the second
// wave of the SIMD issues its MFMAs, fragment reads and loads into the gaps of the first.
//
// INTF: the per-group factors are integers -- `p.scales` / `p.szeros` point to int8 tables [K/128][N] (scale byte and
// pre-multiplied negated zero byte) and the table of a group is (q * scale + zero) modulo 256; everything else is the same.
template <int KIND, int BM, int BN, int KH = 1, int MW = 1, bool INTF = false>
__global__ __launch_bounds__(256 * KH * MW) void gemm_w4a8_kernel(GemmArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
    static_assert(KIND == KIND_W8A8 || KIND == KIND_W8A8_ACC, "int8 accumulation");
    constexpr int NS = 4;
    static_assert(MW == 1 || (MW == 2 && KH == 1), "two quartets share either the K range or the tile's rows");
    constexpr int BMW = BM / MW;                            // tile rows of one quartet
    constexpr int FM = BMW / 64, FN = BN / 64;
    constexpr int ROWS = BM + BN;
    constexpr int STAGE = ROWS * 64;
    constexpr int NLA = BM * 4 / 256;                       // direct activation loads per thread and stage, of the quartet that issues them
    constexpr int CPT = BN * 2 / 256;                       // packed 16-byte chunks per thread and stage
    static_assert(BM % 64 == 0 && (BN == 128 || BN == 256) && NLA >= 2, "tile shapes this staging scheme covers");
    using acc_t = i16_t;

    static_assert(KH * MW == 1 || FM * FN < 16, "two quartets: 256 registers per wave");
    extern __shared__ __attribute__((aligned(16))) char smem_all[];

    const int tid = threadIdx.x & 255;                       // index inside the quartet
    const int quartet = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8);
    const int kq = MW == 1 ? quartet : 0;                    // KH = 2: which half of the K range
    const int mh = MW == 2 ? quartet : 0;                    // MW = 2: which half of the tile's rows
    char* const smem = smem_all + kq * (NS * STAGE);         // this quartet's ring (MW = 2: the one ring)
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int M = p.M, N = p.N, K = p.K;
    int tm, tn;
    const int TM_ = (M + BM - 1) / BM, TN_ = (p.n_cols + BN - 1) / BN;
    const int split = blockIdx.x / (TM_ * TN_);
    tile_of_block(blockIdx.x - split * (TM_ * TN_), TM_, TN_, tm, tn, p.group_m);
    const int m0 = tm * BM, n0 = p.n_begin + tn * BN;
    const int T_all = K >> 6;                                // 64-byte stages along K (K % 128 == 0: even)
    const int t_per = (((T_all + p.splits - 1) / p.splits) + 2 * KH - 1) / (2 * KH) * (2 * KH);   // whole groups per split and quartet
    const int t_split = (split * t_per + t_per <= T_all) ? t_per : T_all - split * t_per;   // even, >= 2 (no empty split)
    const int T = t_split / KH;                              // two quartets: the host keeps this even as well
    const int t0 = split * t_per + kq * T;

    acc_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    // ---- activation side: load i of wave w fills the KiB region R = 4*i + w = tile rows 16R .. 16R+15 (MW = 2: the
    // waves of the second quartet, which stage no weights, bring in all the rows of the tile)
    uint32_t voff_a[NLA];
#pragma unroll
    for (int i = 0; i < NLA; ++i) {
        const int row = 16 * (4 * i + wave) + (lane >> 2);
        const int c = (lane & 3) ^ ((row >> 2) & 3);
        int m = m0 + row;
        m = m < M ? m : M - 1;
        voff_a[i] = (uint32_t)((long)m * K + c * 16);
    }
    // ---- weight side: this thread's row of the tile
    const int brow = CPT == 2 ? tid : (tid >> 1);
    int ncol = n0 + brow;
    ncol = ncol < N ? ncol : N - 1;                          // ragged last tile: clamp loads, stores are masked
    const uint32_t voff_b = (uint32_t)((long)(ncol >> 2) * K * 2 + (ncol & 3) * 32 + (CPT == 2 ? 0 : (tid & 1) * 16));
    const uint32_t voff_s = (uint32_t)ncol * (INTF ? 1u : 2u);
    constexpr uint32_t SZB = INTF ? 1u : 2u;                // bytes per table entry
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.a), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.b), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(p.scales), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_z = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(p.szeros), 0, -1, 0x00020000);
    // where this thread's decoded bytes go inside a stage: row BM + brow, 16-byte slot s at s ^ ((row >> 2) & 3)
    const int bsw = (brow >> 2) & 3;
    const int bdst = (BM + brow) * 64;
    const int hsel = CPT == 2 ? 0 : (tid & 1);              // BN = 128: which half of the row this thread decodes

    u4_t raw[2][2][CPT];                                     // [stage parity][group parity][chunk]
    unsigned short sraw[2], zraw[2];                         // [group parity]
    uint32_t L[4];

    auto clamp_stage = [&](int u) { return t0 + (u < T ? u : T - 1); };   // past the end: harmless reloads
    auto load_factor = [&](__amdgpu_buffer_rsrc_t rsrc, uint32_t so) -> unsigned short {
        if constexpr (INTF) return (unsigned short)__builtin_amdgcn_raw_buffer_load_b8(rsrc, voff_s, so, 0);
        else return (unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rsrc, voff_s, so, 0);
    };
    auto issue_raw = [&](int u, auto sp, auto gp) {
        const uint32_t sb = (uint32_t)clamp_stage(u) * 128u;
#pragma unroll
        for (int j = 0; j < CPT; ++j)
            raw[decltype(sp)::value][decltype(gp)::value][j] =
                __builtin_bit_cast(u4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, voff_b + 16u * j, sb, 0));
    };
    auto issue_sz = [&](int u, auto gp) {                    // scale and scaled zero of the group of (even) stage u
        const uint32_t so = (uint32_t)(clamp_stage(u) >> 1) * (uint32_t)N * SZB;
        sraw[decltype(gp)::value] = load_factor(rsrc_s, so);
        zraw[decltype(gp)::value] = load_factor(rsrc_z, so);
    };
    // ---- the decode work of one iteration as a list of small items (compile-time index), placed one by one between
    // the MFMAs.  Items of an iteration that decodes stage u (stage parity SP, group parity GN of u):
    //   [table words 0..3 of the group, only when u is the first stage of its group]
    //   per chunk J of this thread: the nibble gather, then output words 0..7 (words 3 and 7 complete a 16-byte
    //   slot of the LDS row and store it).
    const W4a8Masks wm4 = w4a8_masks();
    uint32_t xy[4];
    u4_t dq;
    // BN = 128: the two threads of a row (lanes 2r, 2r+1) need the same table; each builds the half for the nibble
    // values 8*hsel .. 8*hsel+7 and gets the other half from its neighbour with a lane swap inside the quad.
    h2_t tq[4];                                              // the eight nibble values of this thread's half, as fp16 pairs
    uint32_t town[2], tnbr[2];
    uint32_t wb[2];                                          // INTF: the same eight values, one per byte
    if constexpr (CPT == 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) tq[i] = h2_t{(half_t)(float)(8 * hsel + 2 * i), (half_t)(float)(8 * hsel + 2 * i + 1)};
        wb[0] = 0x03020100u + 0x08080808u * (uint32_t)hsel;
        wb[1] = 0x07060504u + 0x08080808u * (uint32_t)hsel;
    }
    auto work_item = [&](auto sp, auto gn, auto with_table, auto item, int slot) {
        constexpr int SPv = decltype(sp)::value, GNv = decltype(gn)::value, IT = decltype(item)::value;
        constexpr int NT = decltype(with_table)::value ? 4 : 0;
        if constexpr (IT < NT) {
            const half_t sc = __builtin_bit_cast(half_t, sraw[GNv]), zc = __builtin_bit_cast(half_t, zraw[GNv]);
            if constexpr (CPT == 2) {
                if constexpr (INTF) L[IT] = w4a8_table_word_int(0x03020100u + 0x04040404u * IT, sraw[GNv], zraw[GNv]);
                else L[IT] = w4a8_table_word<IT>(sc, zc);
            } else if constexpr (IT < 2) {
                if constexpr (INTF) town[IT] = w4a8_table_word_int(wb[IT], sraw[GNv], zraw[GNv]);
                else town[IT] = w4a8_table_word_of(tq[2 * IT], tq[2 * IT + 1], sc, zc);
            } else if constexpr (IT == 2) {                  // quad_perm [1, 0, 3, 2]: the other thread of the row
                tnbr[0] = (uint32_t)__builtin_amdgcn_mov_dpp((int)town[0], 0xB1, 0xF, 0xF, true);
                tnbr[1] = (uint32_t)__builtin_amdgcn_mov_dpp((int)town[1], 0xB1, 0xF, 0xF, true);
            } else {
                L[0] = hsel ? tnbr[0] : town[0];
                L[1] = hsel ? tnbr[1] : town[1];
                L[2] = hsel ? town[0] : tnbr[0];
                L[3] = hsel ? town[1] : tnbr[1];
            }
        } else if constexpr (IT < NT + 9 * CPT) {
            constexpr int J = (IT - NT) / 9, ST = (IT - NT) % 9;
            if constexpr (ST == 0) {
                w4a8_gather_nibbles(raw[SPv][GNv][J], xy);
            } else {
                constexpr int W = ST - 1;
                dq[W & 3] = w4a8_decode_word<W>(xy, L, wm4);
                if constexpr ((W & 3) == 3) {
                    char* row = smem + slot * STAGE + bdst;
                    const int h = CPT == 2 ? J : hsel;       // 32-wide half of the 64-wide stage
                    *reinterpret_cast<u4_t*>(row + (((2 * h + (W >> 2)) ^ bsw) << 4)) = dq;
                }
            }
        }
    };

    // ---- fragments: lane (r = lane&31, kh = lane>>5) reads 16-byte slot 2s+kh of row base+r
    const int fr = lane & 31, fkh = lane >> 5;
    const int fsw = (fr >> 2) & 3;
    int off_a[2], off_b[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        off_a[s] = (mh * BMW + wm * (BMW / 2) + fr) * 64 + (((2 * s + fkh) ^ fsw) << 4);
        off_b[s] = (BM + wn * (BN / 2) + fr) * 64 + (((2 * s + fkh) ^ fsw) << 4);
    }
    u4_t fa[2][FM], fb[2][FN];
    auto read_frags = [&](int slot, int s, int set) {
        const char* st = smem + slot * STAGE;
#pragma unroll
        for (int i = 0; i < FM; ++i) fa[set][i] = *reinterpret_cast<const u4_t*>(st + off_a[s] + i * 2048);
#pragma unroll
        for (int j = 0; j < FN; ++j) fb[set][j] = *reinterpret_cast<const u4_t*>(st + off_b[s] + j * 2048);
    };
    constexpr int NMF = FM * FN, NRD = FM + FN;
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;

    // ---- prologue.  Issue order mirrors the loop's, so that the loop's wait counts hold from iteration 0 on:
    //   [A0, packed 0, packed 1, scale/zero of group 0] [A1] [A2 first half, packed 2, scale/zero of group 1]
    //   [A2 second half] [A3 first half, packed 3]
    // DEC: this wave stages weights (always, except the second quartet of MW = 2); the others issue the same
    // barriers and only the activation loads, so their wait counts leave the weight-side loads out.
    auto pipeline = [&](auto dec_) {
    constexpr bool DEC = decltype(dec_)::value;
    constexpr int CPE = DEC ? CPT : 0, SZ = DEC ? 2 : 0;     // weight-side loads of this wave: packed chunks, scale + zero
    constexpr int ALD = (MW == 1 || !DEC) ? NLA : 0;         // activation loads of this wave per stage
    constexpr int NLA0 = (ALD + 1) / 2, NLA1 = ALD - NLA0;   // issued behind the barrier / in front of it
    auto issue_a_half = [&](int u, int slot, int h) {        // h = 0: loads 0 .. NLA0-1, h = 1: the rest
        char* dst = smem + slot * STAGE + wave * 1024;
        const uint32_t sa = (uint32_t)clamp_stage(u) * 64u;
#pragma unroll
        for (int i = 0; i < ALD; ++i) {
            if ((i < NLA0) != (h == 0)) continue;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(dst + i * 4096), 16, voff_a[i], sa, 0, 0);
        }
    };
    issue_a_half(0, 0, 0); issue_a_half(0, 0, 1);
    if constexpr (DEC) {
        issue_raw(0, I0{}, I0{});
        issue_raw(1, I1{}, I0{});
        issue_sz(0, I0{});
    }
    __builtin_amdgcn_sched_barrier(0);
    issue_a_half(1, 1, 0); issue_a_half(1, 1, 1);
    issue_a_half(2, 2, 0);
    if constexpr (DEC) {
        issue_raw(2, I0{}, I1{});
        issue_sz(2, I1{});
    }
    __builtin_amdgcn_sched_barrier(0);
    issue_a_half(2, 2, 1);
    issue_a_half(3, 3, 0);
    if constexpr (DEC) issue_raw(3, I1{}, I1{});
    __builtin_amdgcn_sched_barrier(0);
    wait_vmcnt<ALD + (NLA0 + CPE + SZ) + NLA1 + (NLA0 + CPE)>();
    if constexpr (DEC) {
        static_for<0, 4 + 9 * CPT>([&](auto it) { work_item(I0{}, I0{}, I1{}, it, 0); });       // stage 0 (builds the table)
        static_for<0, 9 * CPT>([&](auto it) { work_item(I1{}, I0{}, I0{}, it, 1); });           // stage 1
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    read_frags(0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);

    // ---- iteration t (stage parity SP = t & 1, group parity GP = (t >> 1) & 1, LDS slot t & 3: all compile time).
    // 2 * NMF slots, one MFMA each, scheduled by hand (a scheduling barrier closes every slot): slot q of the first
    // block also takes the q-th fragment read of k-step 1 (first slots) or one of the loads issued in front of the
    // barrier (last slots); the second block likewise with the reads of k-step 0 of stage t+1 and the loads issued
    // behind the barrier; the decode items of stage t+2 are dealt evenly over all slots.
    auto iteration = [&](auto sp, auto gp, int t) {
        constexpr int SP = decltype(sp)::value, GP = decltype(gp)::value;
        constexpr int SLOT = 2 * GP + SP;                    // t % 4
        using GN = std::integral_constant<int, GP ^ 1>;      // group parity of stage t+2
        using WT = std::integral_constant<int, SP == 0 ? 1 : 0>;   // stage t+2 opens a group: build its table first
        constexpr int NTAB = SP == 0 ? 4 : 0, NITEMS = DEC ? NTAB + 9 * CPT : 0;
        constexpr int COST = 2 * NTAB + 9 * CPT;            // a table word costs about two lookups
        constexpr int NSLOTS = 2 * NMF;
        constexpr int NP1 = NLA1, NP2 = NLA0 + CPE + (SP == 0 ? SZ : 0);  // loads in front of / behind the barrier
        constexpr int RD_SLOTS = NMF >= 8 ? NMF / 2 : NMF;   // fragment reads go to the first slots of a block,
        constexpr int LD_FROM = NMF >= 8 ? NMF / 2 : 0;      // loads to the last ones (small tiles: everywhere)
        // everything issued up to two iterations ago has landed: activations of stage t+1, the packed chunks of
        // stage t+2 and, on even t, scale and zero of its group.  Younger: second half of A(t+2), [first half of
        // A(t+3), packed t+3, and on odd t the scale/zero pair issued by the even iteration before].
        wait_vmcnt<NLA1 + NLA0 + CPE + (SP == 1 ? SZ : 0)>();
        const uint32_t sa3 = (uint32_t)clamp_stage(t + 3) * 64u, sa4 = (uint32_t)clamp_stage(t + 4) * 64u;
        const uint32_t sb4 = (uint32_t)clamp_stage(t + 4) * 128u;
        const uint32_t so4 = (uint32_t)(clamp_stage(t + 4) >> 1) * (uint32_t)N * SZB;
        static_for<0, NSLOTS>([&](auto q_) {
            constexpr int Q = decltype(q_)::value, BLK = Q / NMF, q = Q % NMF;
            if constexpr (Q == NMF)      // stage t+1 is complete for every wave and stage t is in registers
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            // fragment reads of the next k-step: set 1 <- (stage t, k-step 1) / set 0 <- (stage t+1, k-step 0)
            constexpr int r0 = q < RD_SLOTS ? q * NRD / RD_SLOTS : NRD, r1 = q < RD_SLOTS ? (q + 1) * NRD / RD_SLOTS : NRD;
            static_for<r0, r1>([&](auto r_) {
                constexpr int r = decltype(r_)::value;
                const char* st = smem + ((SLOT + BLK) & 3) * STAGE;
                const int s = 1 - BLK;
                if constexpr (r < FM) fa[1 - BLK][r] = *reinterpret_cast<const u4_t*>(st + off_a[s] + r * 2048);
                else fb[1 - BLK][r - FM] = *reinterpret_cast<const u4_t*>(st + off_b[s] + (r - FM) * 2048);
            });
            // loads
            constexpr int NP = BLK == 0 ? NP1 : NP2;
            constexpr int l0 = q >= LD_FROM ? (q - LD_FROM) * NP / (NMF - LD_FROM) : NP;
            constexpr int l1 = q >= LD_FROM ? (q - LD_FROM + 1) * NP / (NMF - LD_FROM) : NP;
            static_for<l0, l1>([&](auto l_) {
                constexpr int l = decltype(l_)::value;
                if constexpr (BLK == 0) {                    // second half of the activation rows of stage t+3
                    char* dst = smem + ((SLOT + 3) & 3) * STAGE + wave * 1024;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(dst + (NLA0 + l) * 4096), 16, voff_a[NLA0 + l], sa3, 0, 0);
                } else if constexpr (l < NLA0) {             // first half of the activation rows of stage t+4
                    char* dst = smem + SLOT * STAGE + wave * 1024;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(dst + l * 4096), 16, voff_a[l], sa4, 0, 0);
                } else if constexpr (l < NLA0 + CPE) {       // packed chunks of stage t+4
                    raw[SP][GP][l - NLA0] = __builtin_bit_cast(u4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, voff_b + 16u * (l - NLA0), sb4, 0));
                } else if constexpr (l == NLA0 + CPE) {      // scale / scaled zero of the group stage t+4 opens
                    sraw[GP] = load_factor(rsrc_s, so4);
                } else {
                    zraw[GP] = load_factor(rsrc_z, so4);
                }
            });
            // the slot's MFMA
            {
                constexpr int i = q / FN, j = q % FN;
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i4_t, fb[BLK][j]),
                                                                  __builtin_bit_cast(i4_t, fa[BLK][i]), acc[i][j], 0, 0, 0);
            }
            // its share of the decode of stage t+2
            static_for<0, NITEMS>([&](auto it) {
                constexpr int IT = decltype(it)::value;
                constexpr int before = IT < NTAB ? 2 * IT : 2 * NTAB + (IT - NTAB);      // cost of the items in front
                if constexpr (before * NSLOTS / COST == Q) work_item(sp, GN{}, WT{}, it, (SLOT + 2) & 3);
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    int t = 0;
    for (; t + 4 <= T; t += 4) {
        iteration(I0{}, I0{}, t);
        iteration(I1{}, I0{}, t + 1);
        iteration(I0{}, I1{}, t + 2);
        iteration(I1{}, I1{}, t + 3);
    }
    if (t < T) {                                             // T is even: two stages left
        iteration(I0{}, I0{}, t);
        iteration(I1{}, I0{}, t + 1);
    }
    };
    if constexpr (MW == 1) {
        pipeline(std::true_type{});
    } else {
        if (mh == 0) pipeline(std::true_type{});
        else pipeline(std::false_type{});
    }
    // no direct load may outlive the workgroup or land in LDS that the epilogue reuses
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier\n\ts_nop 15\n\ts_nop 15" ::: "memory");

    if constexpr (KH > 1) {                                  // quartet 1 hands its accumulators to quartet 0 and leaves
        constexpr int RED_OFF = 32 * 1024;                   // clear of the epilogue's patches at the start of LDS
        static_assert(4 * 32 * ((BN / 2) * 2 + 8) <= RED_OFF && RED_OFF + FM * FN * 16 * 256 * 4 <= KH * NS * STAGE, "LDS layout of the hand-over");
        int* red = reinterpret_cast<int*>(smem_all + RED_OFF);
        if (kq == 1) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) red[((i * FN + j) * 16 + e) * 256 + tid] = acc[i][j][e];
        }
        __syncthreads();
        if (kq == 1) return;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] += red[((i * FN + j) * 16 + e) * 256 + tid];
    }
    // each quartet of MW = 2 writes its half of the tile's rows out, with patches of its own
    constexpr int EPI_LDS = 4 * 32 * ((BN / 2) * 2 + 8);
    char* const epi = smem + mh * EPI_LDS;
    const int me = m0 + mh * BMW;
    if (p.splits > 1) store_partial<BMW, BN, FM, FN>(p, acc, split, me, n0, wave, lane);
    else if (p.bias) gemm_epilogue<KIND, BMW, BN, true, FM, FN>(p, acc, epi, me, n0, wave, lane);
    else gemm_epilogue<KIND, BMW, BN, false, FM, FN>(p, acc, epi, me, n0, wave, lane);
#endif
}

// ---- host side ---------------------------------------------------------------------------------
template <int KIND, bool INTF, int BM, int BN, int KH = 1, int MW = 1>
static int launch_w4a8(const GemmArgs& a_in, const Workspace& ws_in, hipStream_t st, int n_begin = 0, int n_cols = -1) {
    GemmArgs a = a_in;
    a.group_m = kmi_forced_group_m();
    a.n_begin = n_begin;
    a.n_cols = n_cols < 0 ? a.N - n_begin : n_cols;
    const Workspace ws = (a.n_begin == 0 && a.n_cols == a.N) ? ws_in : Workspace{nullptr, 0};   // column ranges: no split over K
    constexpr size_t lds = (size_t)KH * 4 * (BM + BN) * 64;
    void (*fn)(GemmArgs) = gemm_w4a8_kernel<KIND, BM, BN, KH, MW, INTF>;
    static thread_local bool raised = false;                 // per instantiation, per thread
    if (lds > 64 * 1024 && !raised) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return kmi_set_error(KMI_E_LAUNCH, "gemm_w4a8: cannot raise the dynamic LDS limit to %zu bytes", lds);
        raised = true;
    }
    // K splits as for the W8A8 lane, in whole 128-wide groups (two stages), no empty split
    const int stages = a.K >> 6;
    int s = kmi_pick_splits(a.M, a.N, a.K, BM, BN, a.K >> 7, ws);
    constexpr int UNIT = 2 * KH;                             // stages per split: whole groups for every quartet
    if (s > 1) {
        const int per = (((stages + s - 1) / s) + UNIT - 1) / UNIT * UNIT;
        s = (stages + per - 1) / per;
    }
    if (KH == 2 && (stages % UNIT != 0)) return kmi_set_error(KMI_E_SHAPE, "gemm_w4a8: two quartets need K %% 256 == 0 (K=%d)", a.K);
    a.splits = s < 2 ? 1 : s;
    a.partial = a.splits > 1 ? ws.ptr : nullptr;
    const dim3 grid(((a.n_cols + BN - 1) / BN) * ((a.M + BM - 1) / BM) * a.splits), block(256 * KH * MW);
    hipLaunchKernelGGL(fn, grid, block, lds, st, a);
    if (a.splits > 1) {
        const long quads = (long)a.M * a.N / 4;
        hipLaunchKernelGGL(splitk_reduce_kernel<KIND>, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, st, a);
    }
    return KMI_OK;
}

// Tile choice by a small cost model fitted to MI355X timings (microseconds).  A 256 x 256 tile over K = 4096 takes
// about 69.5 us with one workgroup per CU (0.40 of the int8 peak with the decode between the MFMAs); a 256 x 128 tile
// (selector 192; eight waves, roles divided as in the 512 x 128 tile) 0.56 of that (0.50 on a single round), a 128 x 128 tile 0.50 alone on a CU and 0.67 per pair when two share one (its decode
// makes it VALU-bound).  Workgroups run in rounds over the CUs; a split over K divides the tile time and adds the
// partial-sum traffic and the reduce kernel.  Checked against sweeps of the Llama-3-8B shapes, M = 128 .. 4096:
// 6144 columns M = 1024 -> 256 x 128 (41.7 us against 48.8 with 128 x 128 and 58.4 with 256 x 256), 28672 columns
// M = 256 -> 256 x 128 (42.0 / 51.2 / 62.6), M = 512 -> 256 x 256 (70.9 against 83.1 / 96.8), 4096 x 14336 M = 1024
// -> 256 x 128 (84.6 / 105.5 / 93.8).
// Column tiles (256 wide) that make up whole rounds of 256 workgroups of 256 x 256 tiles; 0 when the tiles are whole
// rounds already, fewer than a round, or the rest would not be thin (more than ~60 % of a round).
static int w4a8_head_cols(int M, int N) {
    const int TM = (M + 255) / 256, TN = (N + 255) / 256;
    const int tiles = TM * TN, rem = tiles % 256;
    const int head = (tiles - rem) / TM;
    if (tiles <= 256 || rem == 0 || head <= 0 || (TN - head) * TM > 160 || (N % 256) != 0) return 0;
    return head;
}

// The same for 512 x 128 tiles (selector 640): column tiles (128 wide) of the whole rounds, when the last round would be
// at most ~55 % full; the rest runs as 256 x 128 tiles in a second launch.
static int w4a8_head_cols_512(int M, int N) {
    const int TM = (M + 511) / 512, TN = (N + 127) / 128;
    const int tiles = TM * TN, rem = tiles % 256;
    const int head = (tiles - rem) / TM;
    if (M < 512 || tiles <= 256 || rem == 0 || head <= 0 || (TN - head) * TM > 140 || (N % 128) != 0) return 0;
    return head;
}

static int w4a8_tile(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 128;              // empty product: the entry points return before any launch
    const int forced = kmi_forced_tile();
    if (forced == 128 || forced == 192 || forced == 256 || forced == 512) return forced;
    if (forced == 130) return (K % 256 == 0) ? 130 : 128;    // 128 x 128 tile, two wave quartets per workgroup
    if (forced == 448) return w4a8_head_cols(M, N) > 0 ? 448 : 256;
    if (forced == 640) return w4a8_head_cols_512(M, N) > 0 ? 640 : 512;
    const Workspace roomy{reinterpret_cast<void*>(16), (size_t)64 << 20};
    const double fixed = 6.0;                                // launch, pipeline fill, epilogue: paid once per launch, split or not
    const double t256 = 63.5 * (double)K / 4096.0;           // + fixed = 69.5 us at K = 4096
    // unit_alone: one round with every CU busy; a round that leaves CUs idle runs faster per workgroup (clock, shared
    // caches), by `idle_gain` for an empty GPU
    auto cost = [&](int bm, int bn, double unit_alone, double unit_shared, int shared_cap, double idle_gain = 0.0) {
        const long tiles = (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
        const int s = kmi_pick_splits(M, N, K, bm, bn, K >> 7, roomy);
        const long w = tiles * s;
        const double rounds_t = w <= 256 ? unit_alone - idle_gain * (1.0 - (double)w / 256.0)
                                         : (double)((w + shared_cap - 1) / shared_cap) * unit_shared;
        double us = fixed + rounds_t * t256 / s;
        if (s > 1) us += (double)(s + 1) * (double)M * (double)N * 4.0 / 4.0e6 + 3.0;
        return us;
    };
    // 128 x 128 alone on a CU: 0.45 with one wave quartet.  With two (selector 130, needs K % 256 == 0, at most one
    // workgroup per CU) the time is a fixed ~7 us + 0.265 us per 64-byte stage, rising to 0.315 as the last CUs fill
    // (4096 x 4096 M=128: 17.7 us, M=1024: 26.4; 4096 x 14336 M=1024: 77.3 against 91.8 with split 256 x 256 tiles).
    const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    const int s128 = kmi_pick_splits(M, N, K, 128, 128, K >> 7, roomy);
    const bool two_quartets = (K % 256 == 0) && tiles128 * s128 <= 256;
    const double c256 = cost(256, 256, 1.0, 1.0, 256), c192 = cost(256, 128, 0.50, 0.56, 256, 0.25);
    double c128 = cost(128, 128, 0.45, 0.67, 512);
    if (two_quartets) {
        const double w = (double)(tiles128 * s128);
        c128 = 7.0 + (0.265 + (w > 192.0 ? 0.05 * (w - 192.0) / 64.0 : 0.0)) * (double)(K >> 6) / s128;
        if (s128 > 1) c128 += (double)(s128 + 1) * (double)M * (double)N * 4.0 / 4.0e6 + 3.0;
    }
    // 256 x 256 tiles in whole rounds of 256 and the columns of the thin last round as 256 x 128 tiles in a second
    // launch (selector 448): 2048 x 28672 is 896 tiles = 3.5 rounds -> 3 rounds + one round of half-size tiles.
    double c448 = 1e30;
    if (w4a8_head_cols(M, N) > 0) {
        const int TM = (M + 255) / 256, TN = (N + 255) / 256, head = w4a8_head_cols(M, N);
        const long tail = (long)(TN - head) * TM * 2;
        c448 = 2.0 * fixed + ((double)((head * TM + 255) / 256) + (double)((tail + 255) / 256) * 0.55) * t256;
    }
    if (c128 <= c192 && c128 <= c256 && c128 <= c448 && (M < 512 || c128 <= cost(512, 128, 0.90, 0.90, 256))) {
        // At most one workgroup per CU: two wave quartets per workgroup, each on half of the workgroup's K range
        // (28672 columns M=128: 28.0 against 32.5 us; 6144 columns M=512: 24.8 against 29.6; 4096 x 14336 M=256 with
        // four splits: 33.1 against 35.5; level elsewhere).  More workgroups than CUs overlap each other already.
        return two_quartets ? 130 : 128;
    }
    // 512 x 128 on eight waves (two quartets, 256 rows each): as many accumulators per SIMD as a 256 x 256 tile, but one
    // decoded weight serves 512 activation rows, i.e. half the decode instructions per MFMA (28672 columns M=1024: 123.7
    // against 134.7 us; M=4096: 471 against 488; 6144 columns M=2048: 55.8 against 61.9; four waves of 256 x 64 each on
    // the same tile: 127.5 / 475 / 58.3).  Not below 512 rows, where half of the tile would be padding.
    const double c512 = M >= 512 ? cost(512, 128, 0.90, 0.90, 256) : 1e30;
    // whole rounds of 512 x 128 tiles + the columns of a thin last round as 256 x 128 tiles (selector 640): 2048 x 28672 is
    // 3.5 rounds -> 3 rounds + 256 half-size workgroups
    double c640 = 1e30;
    if (w4a8_head_cols_512(M, N) > 0) {
        const int TM = (M + 511) / 512, TN = (N + 127) / 128, head = w4a8_head_cols_512(M, N);
        const long tail = (long)(TN - head) * ((M + 255) / 256);
        const double tail_unit = tail <= 256 ? 0.50 - 0.25 * (1.0 - (double)tail / 256.0) : (double)((tail + 255) / 256) * 0.56;
        c640 = 2.0 * fixed + ((double)((head * TM + 255) / 256) * 0.90 + tail_unit) * t256;
    }
    if (c640 < c512 && c640 < c448 && c640 < c192 && c640 < c256) return 640;
    if (c512 < c448 && c512 < c192 && c512 < c256) return 512;
    if (c448 <= c192 && c448 <= c256) return 448;
    return c192 <= c256 ? 192 : 256;
}
extern "C" int kmi_gemm_w4a8_pick_tile(int M, int N, int K) { return w4a8_tile(M, N, K); }

template <int KIND, bool INTF = false>
static int w4a8_entry(const char* fn, GemmArgs& a, int G, const void* workspace, size_t workspace_bytes, void* stream) {
    if (G != 128) return kmi_set_error(KMI_E_GROUP, "%s: group size %d unsupported (128 only)", fn, G);
    if (!a.scales || !a.szeros) return kmi_set_error(KMI_E_NULL, "%s: NULL scale table", fn);
    if (KIND == KIND_W8A8 && (!a.wscales || !a.ascales)) return kmi_set_error(KMI_E_NULL, "%s: NULL scale vector", fn);
    int rc = kmi_gemm_args_check(fn, a, false);
    if (rc != KMI_OK) return rc;
    Workspace ws;
    rc = kmi_workspace_check(fn, workspace, workspace_bytes, ws);
    if (rc != KMI_OK) return rc;
    if (a.M == 0) return KMI_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int tile = w4a8_tile(a.M, a.N, a.K);
    if (tile == 640) {
        const int head = w4a8_head_cols_512(a.M, a.N) * 128;
        rc = launch_w4a8<KIND, INTF, 512, 128, 1, 2>(a, ws, st, 0, head);
        if (rc == KMI_OK) rc = launch_w4a8<KIND, INTF, 256, 128, 1, 2>(a, ws, st, head, a.N - head);
    } else if (tile == 448) {
        const int head = w4a8_head_cols(a.M, a.N) * 256;
        rc = launch_w4a8<KIND, INTF, 256, 256>(a, ws, st, 0, head);
        if (rc == KMI_OK) rc = launch_w4a8<KIND, INTF, 256, 128, 1, 2>(a, ws, st, head, a.N - head);
    } else {
        rc = tile == 256 ? launch_w4a8<KIND, INTF, 256, 256>(a, ws, st)
           : tile == 192 ? launch_w4a8<KIND, INTF, 256, 128, 1, 2>(a, ws, st)
           : tile == 130 ? launch_w4a8<KIND, INTF, 128, 128, 2>(a, ws, st)
           : tile == 512 ? launch_w4a8<KIND, INTF, 512, 128, 1, 2>(a, ws, st) : launch_w4a8<KIND, INTF, 128, 128>(a, ws, st);
    }
    if (rc != KMI_OK) return rc;
    return kmi_check_launch(fn);
}

extern "C" int kmi_gemm_w4a8(void* out, const void* a8, const void* qweight, const void* scales_to8, const void* szeros_to8,
                             const void* wscales, const void* ascales, const void* bias, int M, int N, int K, int G,
                             void* workspace, size_t workspace_bytes, void* stream) {
    GemmArgs a{out, a8, qweight, (const half_t*)scales_to8, (const half_t*)szeros_to8, (const half_t*)wscales,
               (const half_t*)ascales, (const half_t*)bias, M, N, K, nullptr, 1, 0, N};
    return w4a8_entry<KIND_W8A8>("kmi_gemm_w4a8", a, G, workspace, workspace_bytes, stream);
}

extern "C" int kmi_gemm_w4a8_acc_i32(void* acc, const void* a8, const void* qweight, const void* scales_to8,
                                     const void* szeros_to8, int M, int N, int K, int G, void* workspace,
                                     size_t workspace_bytes, void* stream) {
    GemmArgs a{acc, a8, qweight, (const half_t*)scales_to8, (const half_t*)szeros_to8, nullptr, nullptr, nullptr, M, N, K,
               nullptr, 1, 0, N};
    return w4a8_entry<KIND_W8A8_ACC>("kmi_gemm_w4a8_acc_i32", a, G, workspace, workspace_bytes, stream);
}

// The same product with integer per-group factors: int8 tables [K/128][N] in plain column order, weight byte =
// (q * scale + zero) modulo 256 read as int8.
extern "C" int kmi_gemm_w4a8_int(void* out, const void* a8, const void* qweight, const void* s2_scales_i8, const void* s2_zeros_i8,
                                 const void* wscales, const void* ascales, const void* bias, int M, int N, int K, int G,
                                 void* workspace, size_t workspace_bytes, void* stream) {
    GemmArgs a{out, a8, qweight, (const half_t*)s2_scales_i8, (const half_t*)s2_zeros_i8, (const half_t*)wscales,
               (const half_t*)ascales, (const half_t*)bias, M, N, K, nullptr, 1, 0, N};
    return w4a8_entry<KIND_W8A8, true>("kmi_gemm_w4a8_int", a, G, workspace, workspace_bytes, stream);
}

extern "C" int kmi_gemm_w4a8_int_acc_i32(void* acc, const void* a8, const void* qweight, const void* s2_scales_i8,
                                         const void* s2_zeros_i8, int M, int N, int K, int G, void* workspace,
                                         size_t workspace_bytes, void* stream) {
    GemmArgs a{acc, a8, qweight, (const half_t*)s2_scales_i8, (const half_t*)s2_zeros_i8, nullptr, nullptr, nullptr, M, N, K,
               nullptr, 1, 0, N};
    return w4a8_entry<KIND_W8A8_ACC, true>("kmi_gemm_w4a8_int_acc_i32", a, G, workspace, workspace_bytes, stream);
}

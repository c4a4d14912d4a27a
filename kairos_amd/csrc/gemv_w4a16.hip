// W4A16 product for decode-sized M (1..64): the packed uint4 weights are streamed from HBM exactly
// once with 16-byte loads and fed to v_mfma_f32_16x16x32_f16 with fp32 accumulation.
//
// Decoding costs no arithmetic: an fp16 whose exponent field is zero is the subnormal m * 2^-24, and
// the MFMA unit honours subnormal inputs, so a nibble masked in place IS the number q * 2^-24 (low
// nibble of a byte) or 16q * 2^-24 (high nibble).  Per 128-wide K group g and output column n the
// kernel therefore accumulates P = sum_k x[m,k] * q[n,k] exactly (activations for the high-nibble
// planes are pre-multiplied by 1/16), obtains X = sum_k x[m,k] from one extra MFMA against a tile of
// ones, and adds  scales[g,n] * P + scaled_zeros[g,n] * X  in fp32.  That is the dequantise-then-
// multiply product with the weights kept at full precision instead of rounded to fp16 first (the
// difference to the fp16 converter's weights is below 2^-11 relative per weight).
//
// Work split.  A workgroup owns 16*NT output columns; its NW waves interleave over the K groups
// (wave w takes groups w, w+NW, ...), so the workgroup as a whole walks contiguous memory: the
// four-row interleave makes a 16-row strip one contiguous K*8-byte region.  Partial sums meet in
// LDS and are added in a fixed order (deterministic output).
//
// Long, narrow weights (K much larger than N: 4096 x 14336, 8192 x 28672) have too few column strips to keep enough
// loads in flight and make every workgroup read the whole activation matrix.  There K is also split over KS
// workgroups per column strip (grid.y): each writes its fp32 partial sums to caller-owned scratch and bumps a per-strip
// counter; whichever workgroup arrives last adds the KS partial sums in split order (deterministic), applies bias and
// writes the output.  Nobody ever waits for another workgroup.  Partial sums and the counter travel through
// agent-scope atomic stores, loads and one atomic add (coherent across the XCDs' L2 caches without cache
// write-backs); a thread waits for its own stores to complete before the workgroup's arrival is counted.
//
// Lane roles inside a wave, for one K group and one 16-column tile: lane = (r16, j), r16 = lane&15,
// j = lane>>4.  The lane loads the 16-byte chunk of row n = tile*16 + r16 that covers
// k = 128c + 32j .. +31; nibble plane a of its four words holds the eight K-contiguous weights
// k = 128c + 32j + 8a .. +7, which is exactly the MFMA B fragment of lane (col r16, k-block j).  The
// matching A fragment is x[m = r16][same eight k], one 16-byte load.  Four MFMAs (a = 0..3) per tile
// consume the group.
#include "kmi_common.h"
#include <mutex>
#include <set>

// Row spread.  With at most four activation rows the kernels place row m in row 4m of the 16-row MFMA operand
// (RS = 4; RS = 2 for up to eight rows), so that the rows that count land in accumulator element 0 (elements 0 and 2)
// of the lanes: the per-group scale-and-add then touches one (two) of the four accumulator registers of a tile, and
// the reduction moves a quarter (half) of the data.  RS = 1 is the plain layout.
//
// Tail shared by the kernels of this file: the waves' partial tiles meet in LDS (`red`, nw * MT*NT*(4/RS) * 64 floats)
// and are added in wave order; with a split over K (gridDim.y > 1) the workgroup's sums go to `partial`, the
// strip's arrival counter is bumped and whichever workgroup arrives last adds the slices in split order.
template <int MT, int NT, int RS>
__device__ __forceinline__ void gemv_finish(const f4_t (&acc)[MT][NT], float* red, int NW, int wave, int lane, int strip, int n0,
                                            half_t* __restrict__ out, const half_t* __restrict__ bias, int M, int N,
                                            float* __restrict__ partial, uint32_t* __restrict__ counters) {
    const int KS = gridDim.y, ks = blockIdx.y;
    constexpr int E = 4 / RS;                                // live accumulator elements per tile
    constexpr int R = MT * NT * E;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int e = 0; e < E; ++e) red[(wave * R + (mt * NT + nt) * E + e) * 64 + lane] = acc[mt][nt][e * RS];
    __syncthreads();
    // idx -> (lane l, live element e of tile (mt, nt)); MFMA row 4*(l>>4) + e*RS holds activation row (that row) / RS
    auto place = [&](int idx, int& m, int& n) {
        const int l = idx & 63, reg = idx >> 6;
        const int e = reg % E, t = reg / E;
        const int nt = t % NT, mt = t / NT;
        m = mt * 16 + (4 * (l >> 4) + e * RS) / RS;
        n = n0 + nt * 16 + (l & 15);
    };

    if (KS == 1) {
        for (int idx = threadIdx.x; idx < R * 64; idx += NW * 64) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) v += red[w * R * 64 + idx];
            int m, n;
            place(idx, m, n);
            if (m < M && n < N) {
                half_t h = (half_t)v;
                if (bias) h = (half_t)((float)h + (float)bias[n]);
                out[(long)m * N + n] = h;
            }
        }
        return;
    }
    // ---- K split over workgroups: publish this workgroup's partial sums, count the arrival, last one finishes
    for (int idx = threadIdx.x; idx < R * 64; idx += NW * 64) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) v += red[w * R * 64 + idx];
        int m, n;
        place(idx, m, n);
        if (m < M && n < N)
            __hip_atomic_store(partial + ((long)ks * M + m) * N + n, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // Hand-off without fences.  Every partial sum travels by an agent-scope atomic store (performed at the memory side
    // that all XCDs share, not in this XCD's L2); `s_waitcnt vmcnt(0)` holds the thread until its stores have been
    // performed, the barrier until every thread's have; only then is the arrival counted, by an agent-scope atomic add
    // at the same memory side.  A workgroup that reads KS-1 from the counter therefore runs after every other
    // workgroup's stores were performed, and its agent-scope atomic loads read them from that memory side.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // this thread's partial sums have been performed
    __shared__ uint32_t arrived;
    __syncthreads();                                         // ... and everybody else's in the workgroup
    if (threadIdx.x == 0) arrived = __hip_atomic_fetch_add(counters + strip, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (arrived != (uint32_t)(KS - 1)) return;               // workgroup-uniform
    for (int idx = threadIdx.x; idx < R * 64; idx += NW * 64) {
        int m, n;
        place(idx, m, n);
        if (m < M && n < N) {
            float v = 0.f;
            for (int q = 0; q < KS; ++q)                     // split order: the same sum whoever arrives last
                v += __hip_atomic_load(partial + ((long)q * M + m) * N + n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            half_t h = (half_t)v;
            if (bias) h = (half_t)((float)h + (float)bias[n]);
            out[(long)m * N + n] = h;
        }
    }
    if (threadIdx.x == 0) __hip_atomic_store(counters + strip, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next call
}

template <int MT, int NT, int NW, int RS>
__global__ __launch_bounds__(NW * 64) void gemv_w4a16_kernel(half_t* __restrict__ out, const half_t* __restrict__ x,
                                                             const u4_t* __restrict__ qw,
                                                             const half_t* __restrict__ scales,
                                                             const half_t* __restrict__ szeros,
                                                             const half_t* __restrict__ bias, int M, int N, int K,
                                                             float* __restrict__ partial, uint32_t* __restrict__ counters) {
    static_assert(RS == 1 || MT == 1, "rows are spread over the operand only when one row tile holds them all");
    extern __shared__ float red[];               // [NW][MT*NT*(4/RS)][64]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int j = lane >> 4;
    // Workgroup ids are dealt round-robin over the 8 XCDs, each with its own L2.  Neighbouring column strips share
    // 128-byte lines of the scale tables (a strip of 16*NT columns is 32*NT bytes of a table row), so every XCD takes
    // a contiguous run of strips: a table line is then fetched by one L2, not by up to four.
    const int nblk = gridDim.x, xcd = blockIdx.x & 7;
    const int strip = xcd * (nblk >> 3) + min(xcd, nblk & 7) + (blockIdx.x >> 3);
    const int n0 = strip * (16 * NT);
    const int KS = gridDim.y, ks = blockIdx.y;              // K split over workgroups: this one covers groups [g0, g1)
    const int all_groups = K >> 7;
    const int g0 = (int)((long)ks * all_groups / KS), ngroups = (int)((long)(ks + 1) * all_groups / KS);
    const int kq = K >> 3;                       // 16-byte units per fp16 row of x / per four-row weight block

    f4_t acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f4_t{0.f, 0.f, 0.f, 0.f};

    const u4_t* wp[NT];
    int ncol[NT];
    const half_t* szp[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int n = n0 + nt * 16 + r16;
        n = n < N ? n : N - 1;                   // partial last strip: clamp loads, stores are masked
        ncol[nt] = n;
        szp[nt] = ((lane >> 5) ? szeros : scales) + n;
        wp[nt] = qw + (long)(n >> 2) * kq + (n & 3) * 2 + (j & 1) + (j >> 1) * 8;
    }
    // Rows beyond M are not loaded at all (their lanes feed zeros): the texture path spends time per
    // active lane quad, so a decode step with one token costs a quarter of a full tile.
    const h8_t* xp[MT];
    bool xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r16 / RS;                    // operand row r16 carries activation row r16 / RS ...
        xrow[mt] = m < M && (r16 % RS) == 0;                 // ... if it is a multiple of the spread
        xp[mt] = reinterpret_cast<const h8_t*>(x) + (long)(xrow[mt] ? m : 0) * kq + j * 4;
    }

    // U K-groups per trip: all loads of the trip are issued before the first MFMA.  Two is the measured
    // optimum for narrow waves; deeper batching costs more in occupancy (VGPRs) than it gains.
    constexpr int U = (MT == 1 && NT <= 2) ? 2 : 1;
    const h8_t ones = {(half_t)1, (half_t)1, (half_t)1, (half_t)1, (half_t)1, (half_t)1, (half_t)1, (half_t)1};
    const h8_t sixteenth = ones * (half_t)0.0625f;
    for (int c0 = g0 + wave; c0 < ngroups; c0 += NW * U) {
        u4_t u[U][NT];
        half_t sz[U][NT];
        h8_t xa[U][MT][4];
#pragma unroll
        for (int t = 0; t < U; ++t) {
            int c = c0 + t * NW;
            c = c < ngroups ? c : ngroups - 1;               // ragged last trip: reload, result unused
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                u[t][nt] = __builtin_nontemporal_load(wp[nt] + c * 16);
                sz[t][nt] = szp[nt][(long)c * N];              // lower half-wave: scale, upper: scaled zero
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (xrow[mt]) {
#pragma unroll
                    for (int a = 0; a < 4; ++a) xa[t][mt][a] = xp[mt][c * 16 + a];
                } else {
#pragma unroll
                    for (int a = 0; a < 4; ++a) xa[t][mt][a] = ones * (half_t)0.0f;
                }
            }
        }
#pragma unroll
        for (int t = 0; t < U; ++t) {
            if (c0 + t * NW < ngroups) {                     // wave-uniform
                f4_t xsum[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    xsum[mt] = f4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int a = 0; a < 4; ++a)
                        xsum[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t][mt][a], ones, xsum[mt], 0, 0, 0);
                    xa[t][mt][1] *= sixteenth;               // planes 1 and 3 carry 16q
                    xa[t][mt][3] *= sixteenth;
                }
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    u4_t lo, hi, lo8, hi8;                   // nibble planes 0, 1, 2, 3 as fp16 subnormals
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const uint32_t v = u[t][nt][w], v8 = v >> 8;
                        lo[w] = v & 0x000F000Fu;
                        hi[w] = v & 0x00F000F0u;
                        lo8[w] = v8 & 0x000F000Fu;
                        hi8[w] = v8 & 0x00F000F0u;
                    }
                    // one load brought the scale to lanes 0-31 and the scaled zero to lanes 32-63 (same column:
                    // it depends on lane%16 only); one swap gives every lane both
                    const uint32_t own = (uint32_t)__builtin_bit_cast(unsigned short, sz[t][nt]);
                    const auto both = __builtin_amdgcn_permlane32_swap(own, own, false, false);
                    const float sc = (float)__builtin_bit_cast(half_t, (unsigned short)both[0]) * 16777216.0f;   // undo the 2^-24 of the subnormal encoding
                    const float zc = (float)__builtin_bit_cast(half_t, (unsigned short)both[1]);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        f4_t pg = {0.f, 0.f, 0.f, 0.f};
                        pg = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t][mt][0], __builtin_bit_cast(h8_t, lo), pg, 0, 0, 0);
                        pg = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t][mt][1], __builtin_bit_cast(h8_t, hi), pg, 0, 0, 0);
                        pg = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t][mt][2], __builtin_bit_cast(h8_t, lo8), pg, 0, 0, 0);
                        pg = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t][mt][3], __builtin_bit_cast(h8_t, hi8), pg, 0, 0, 0);
#pragma unroll
                        for (int i = 0; i < 4; i += RS)          // the rows that count (see the row spread above)
                            acc[mt][nt][i] = __builtin_fmaf(pg[i], sc, __builtin_fmaf(xsum[mt][i], zc, acc[mt][nt][i]));
                    }
                }
            }
        }
    }

    gemv_finish<MT, NT, RS>(acc, red, NW, wave, lane, strip, n0, out, bias, M, N, partial, counters);
}

// =====================================================================================================================
// Ring form of the same product.  Registers cannot hold more than one or two K groups per wave in flight, so the
// kernel above alternates between waiting for HBM and computing.  Here every operand of a K group -- NT KiB of packed
// weights, the activation rows, the group's scale-table entries -- travels global -> LDS by buffer loads that write
// LDS directly (no destination registers), into a ring of D slots that is private to the wave: the wave keeps D groups
// in flight, waits with `s_waitcnt vmcnt` for the oldest (loads retire in issue order), copies it to registers,
// re-issues the slot for the group D trips ahead and only then computes.  No barrier until the final reduction.
//   slot = [NT x 1 KiB weights: lane l's 16-byte chunk at l*16][XI x 1 KiB activations][256 B scales][256 B scaled zeros]
//   activations: 16-byte unit `ch` (0..15) of row r of the group's [rows][128] block sits at unit r*16 + (ch ^ (r & 15)),
//   so the 16 lanes that read one plane of 16 different rows hit 16 different bank quads; XI loads cover 4*XI rows
//   (rows >= M repeat row M-1: their products land in output rows that are never stored).
template <int L, int KMAX>
__device__ __forceinline__ void gemv_wait_slots(int k) {         // until at most k slots' loads (L each) are outstanding
    if constexpr (KMAX > 0) {
        if (k >= KMAX) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(KMAX * L) : "memory");
            return;
        }
        gemv_wait_slots<L, KMAX - 1>(k);
    } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
}

template <int XI, int NT>
static constexpr int gemv_ring_max_depth() {                        // vmcnt counts up to 63
    constexpr int L = NT + XI + 2;
    return (63 / L + 1) < 8 ? (63 / L + 1) : 8;
}

template <int XI, int NT>
__global__ __launch_bounds__(512) void gemv_ring_kernel(half_t* __restrict__ out, const half_t* __restrict__ x,
                                                        const u4_t* __restrict__ qw, const half_t* __restrict__ scales,
                                                        const half_t* __restrict__ szeros, const half_t* __restrict__ bias,
                                                        int M, int N, int K, int D, float* __restrict__ partial,
                                                        uint32_t* __restrict__ counters) {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass cannot instantiate code that uses the buffer resource type
    constexpr int MT = (XI + 3) / 4;
    constexpr int RS = XI == 1 ? 4 : XI == 2 ? 2 : 1;              // row spread: at most 4 / 8 rows sit in operand rows 4m / 2m
    constexpr int L = NT + XI + 2;                                 // direct loads per slot
    constexpr int X_OFF = NT * 1024, S_OFF = X_OFF + XI * 1024, SLOT = S_OFF + 512;
    constexpr int KMAX = gemv_ring_max_depth<XI, NT>() - 1;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // scalar: feeds M0
    const int NW = blockDim.x >> 6;
    const int r16 = lane & 15, j = lane >> 4;
    const int nblk = gridDim.x, xcd = blockIdx.x & 7;               // contiguous run of strips per XCD, as above
    const int strip = xcd * (nblk >> 3) + min(xcd, nblk & 7) + (blockIdx.x >> 3);
    const int n0 = strip * (16 * NT);
    const int KS = gridDim.y, ks = blockIdx.y;
    const int all_groups = K >> 7;
    const int g0 = (int)((long)ks * all_groups / KS), g1 = (int)((long)(ks + 1) * all_groups / KS);
    const int kq = K >> 3;
    const int mine = g0 + wave < g1 ? (g1 - g0 - wave + NW - 1) / NW : 0;   // groups g0 + wave + i*NW, i < mine

    // ---- global sources: a resource per tensor, a per-lane byte offset that never changes, a scalar offset per group
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<u4_t*>(qw), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_s = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(scales), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_z = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(szeros), 0, -1, 0x00020000);
    uint32_t voff_w[NT], voff_x[XI];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int n = n0 + nt * 16 + r16;
        n = n < N ? n : N - 1;                                     // partial last strip: clamp loads, stores are masked
        voff_w[nt] = (uint32_t)(((long)(n >> 2) * kq + (n & 3) * 2 + (j & 1) + (j >> 1) * 8) * 16);
    }
#pragma unroll
    for (int i = 0; i < XI; ++i) {
        const int p = i * 64 + lane, row = p >> 4, ch = (p & 15) ^ (row & 15);
        const int m = row < M ? row : M - 1;
        voff_x[i] = (uint32_t)(((long)m * K + ch * 8) * 2);
    }
    uint32_t voff_s;
    {
        int n = n0 + 2 * (lane < 8 * NT ? lane : 8 * NT - 1);
        n = n < N ? n : N - 2;
        voff_s = (uint32_t)(n * 2);
    }
    char* ring = smem + wave * (D * SLOT);
    auto issue = [&](int slot, int i) {                             // the wave's i-th group into ring slot `slot`
        const uint32_t c = (uint32_t)(g0 + wave + i * NW);
        char* dst = ring + slot * SLOT;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_void_ptr)(dst + nt * 1024), 16, voff_w[nt], c * 256u, 0, 0);
#pragma unroll
        for (int t = 0; t < XI; ++t)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lds_void_ptr)(dst + X_OFF + t * 1024), 16, voff_x[t], c * 256u, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_s, (lds_void_ptr)(dst + S_OFF), 4, voff_s, c * (uint32_t)(N * 2), 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_z, (lds_void_ptr)(dst + S_OFF + 256), 4, voff_s, c * (uint32_t)(N * 2), 0, 0);
    };

    // ---- LDS read addresses of this lane inside a slot
    int xoff[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int row = mt * 16 + r16 / RS;                              // operand row r16 carries activation row r16 / RS
        row = row < 4 * XI ? row : 4 * XI - 1;
#pragma unroll
        for (int a = 0; a < 4; ++a) xoff[mt][a] = X_OFF + (row * 16 + ((4 * j + a) ^ (row & 15))) * 16;
    }

    f4_t acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f4_t{0.f, 0.f, 0.f, 0.f};
    const h8_t ones = {(half_t)1, (half_t)1, (half_t)1, (half_t)1, (half_t)1, (half_t)1, (half_t)1, (half_t)1};
    const h8_t sixteenth = ones * (half_t)0.0625f;

    const int pre = mine < D ? mine : D;
    for (int i = 0; i < pre; ++i) issue(i, i);
    int slot = 0;
    for (int i = 0; i < mine; ++i) {
        const int behind = mine - 1 - i;                            // slots issued after this one and still wanted
        gemv_wait_slots<L, KMAX>(behind < D - 1 ? behind : D - 1);
        const char* src = ring + slot * SLOT;
        u4_t u[NT];
        half_t sc_h[NT], zc_h[NT];
        h8_t xa[MT][4];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            u[nt] = *reinterpret_cast<const u4_t*>(src + nt * 1024 + lane * 16);
            sc_h[nt] = *reinterpret_cast<const half_t*>(src + S_OFF + (nt * 16 + r16) * 2);
            zc_h[nt] = *reinterpret_cast<const half_t*>(src + S_OFF + 256 + (nt * 16 + r16) * 2);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int a = 0; a < 4; ++a) xa[mt][a] = *reinterpret_cast<const h8_t*>(src + xoff[mt][a]);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");         // the slot is in registers: hand it back
        if (i + D < mine) issue(slot, i + D);
        slot = slot + 1 == D ? 0 : slot + 1;

        f4_t xsum[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            xsum[mt] = f4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int a = 0; a < 4; ++a)
                xsum[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt][a], ones, xsum[mt], 0, 0, 0);
            xa[mt][1] *= sixteenth;                                 // planes 1 and 3 carry 16q
            xa[mt][3] *= sixteenth;
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            u4_t lo, hi, lo8, hi8;                                  // nibble planes 0, 1, 2, 3 as fp16 subnormals
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t v = u[nt][w], v8 = v >> 8;
                lo[w] = v & 0x000F000Fu;
                hi[w] = v & 0x00F000F0u;
                lo8[w] = v8 & 0x000F000Fu;
                hi8[w] = v8 & 0x00F000F0u;
            }
            const float sc = (float)sc_h[nt] * 16777216.0f;         // undo the 2^-24 of the subnormal encoding
            const float zc = (float)zc_h[nt];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                f4_t pg = {0.f, 0.f, 0.f, 0.f};
                pg = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt][0], __builtin_bit_cast(h8_t, lo), pg, 0, 0, 0);
                pg = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt][1], __builtin_bit_cast(h8_t, hi), pg, 0, 0, 0);
                pg = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt][2], __builtin_bit_cast(h8_t, lo8), pg, 0, 0, 0);
                pg = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt][3], __builtin_bit_cast(h8_t, hi8), pg, 0, 0, 0);
#pragma unroll
                for (int e = 0; e < 4; e += RS)                     // the rows that count
                    acc[mt][nt][e] = __builtin_fmaf(pg[e], sc, __builtin_fmaf(xsum[mt][e], zc, acc[mt][nt][e]));
            }
        }
    }
    // every wave has emptied its ring (and no direct load is outstanding) before the rings become the reduction buffer
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    gemv_finish<MT, NT, RS>(acc, reinterpret_cast<float*>(smem), NW, wave, lane, strip, n0, out, bias, M, N, partial, counters);
#endif
}

typedef void (*gemv_fn)(half_t*, const half_t*, const u4_t*, const half_t*, const half_t*, const half_t*, int, int, int, float*, uint32_t*);

template <int MT, int NT, int NW>
static constexpr bool gemv_cfg_ok() {
    return MT * NT <= 8 && NW * MT * NT <= 64 && (NW < 16 || MT * NT <= 2);
}

static int gemv_row_spread(int M) { return M <= 4 ? 4 : M <= 8 ? 2 : 1; }

template <int MT, int NT, int NW>
static gemv_fn gemv_pick(int rs) {
    if constexpr (gemv_cfg_ok<MT, NT, NW>()) {
        if constexpr (MT == 1) {
            if (rs == 4) return gemv_w4a16_kernel<MT, NT, NW, 4>;
            if (rs == 2) return gemv_w4a16_kernel<MT, NT, NW, 2>;
        }
        return gemv_w4a16_kernel<MT, NT, NW, 1>;
    } else {
        return nullptr;
    }
}

template <int MT, int NT>
static gemv_fn gemv_pick_nw(int nw, int rs) {
    switch (nw) {
        case 4: return gemv_pick<MT, NT, 4>(rs);
        case 8: return gemv_pick<MT, NT, 8>(rs);
        case 16: return gemv_pick<MT, NT, 16>(rs);
    }
    return nullptr;
}

template <int MT>
static gemv_fn gemv_pick_nt(int nt, int nw, int rs) {
    switch (nt) {
        case 1: return gemv_pick_nw<MT, 1>(nw, rs);
        case 2: return gemv_pick_nw<MT, 2>(nw, rs);
        case 3: return gemv_pick_nw<MT, 3>(nw, rs);
        case 4: return gemv_pick_nw<MT, 4>(nw, rs);
        case 5: return gemv_pick_nw<MT, 5>(nw, rs);
        case 6: return gemv_pick_nw<MT, 6>(nw, rs);
        case 7: return gemv_pick_nw<MT, 7>(nw, rs);
        case 8: return gemv_pick_nw<MT, 8>(nw, rs);
    }
    return nullptr;
}

// rs: row spread of the kernel (gemv_row_spread(M)); the existence of a kernel does not depend on it
static gemv_fn gemv_lookup(int mt, int nt, int nw, int rs = 1) {
    switch (mt) {
        case 1: return gemv_pick_nt<1>(nt, nw, rs);
        case 2: return gemv_pick_nt<2>(nt, nw, 1);
        case 3: return gemv_pick_nt<3>(nt, nw, 1);
        case 4: return gemv_pick_nt<4>(nt, nw, 1);
    }
    return nullptr;
}

// Default split, from sweeps on MI355X over the Llama-3-8B / -70B and Qwen2.5-7B shapes.
//   Column tiles per wave (nt).  All workgroups of these grids are resident at once (up to four per CU), so the
//   kernel ends when the CU with the most column strips ends: ceil(workgroups / 256) * nt strips.  More tiles per
//   wave reuse every activation fragment more often (the whole activation matrix is read by every workgroup), less
//   so at small M; measured times follow  busiest * (1 + c / nt)  with c = 0.6 (M <= 4), 1.0 (M <= 8), 1.7 (M <= 16),
//   2.5 beyond.  The nt with the smallest estimate wins: 1792 strips (28672 columns) -> 7 tiles, 256 workgroups
//   (M=16: 14.0 against 16.4 us with 4); 640 strips -> 3 (11.5 against 12.5 us); 2368 -> 5 (14.2 against 15.5);
//   288 -> 2 (5.1 against 5.9 us with 1).
//   Waves per workgroup over K (nw): eight; sixteen for a single column tile at the smallest M, where the kernel is
//   a pure latency chain (4096 x 14336 at M=1: 10.4 against 11.9 us); four from three row tiles on (M > 32), and for
//   seven or eight column tiles when more than one workgroup shares a CU (57344 x 8192 at M=16: 45.3 against 48.5 us).
static void gemv_default_cfg(int M, int mt, int N, int K, int* nt_out, int* nw_out, int* ks_out) {
    const int strips = (N + 15) / 16, groups = K / 128;
    const double c = M <= 4 ? 0.6 : M <= 8 ? 1.0 : M <= 16 ? 1.7 : 2.5;
    int nt = 1, wgs = strips;
    double best = 1e30;
    for (int cand = 1; cand <= 8; ++cand) {
        if (gemv_lookup(mt, cand, 8) == nullptr) continue;           // row tiles x column tiles <= 8 (registers)
        const int w = (strips + cand - 1) / cand;
        const double est = (double)((w + 255) / 256) * (cand + c);    // busiest * (1 + c / nt), busiest = rounds * nt
        if (est < best - 1e-9) { best = est; nt = cand; wgs = w; }
    }
    if (M <= 4 && strips > 3072 && gemv_lookup(mt, 2, 8) != nullptr) {   // many rounds at the smallest M: two tiles stream best
        nt = 2;                                                         // (128256 x 4096 at M=1: 49.2 against 51.4 us)
        wgs = (strips + 1) / 2;
    }
    int nw = 8;
    if (nt == 1 && (M <= 4 || (M <= 8 && K <= 4096)) && groups >= 16 && gemv_lookup(mt, nt, 16) != nullptr) nw = 16;
    if (mt >= 3 && nt >= 2 && gemv_lookup(mt, nt, 4) != nullptr) nw = 4;
    if (nt >= 7 && wgs > 256 && gemv_lookup(mt, nt, 4) != nullptr) nw = 4;
    while (nw > 4 && (groups < nw || gemv_lookup(mt, nt, nw) == nullptr)) nw >>= 1;
    *nt_out = nt;
    *nw_out = nw;
    *ks_out = 1;
    // Long, narrow weights: few column strips, each a long walk over K.  A wave then runs several load-wait-compute
    // trips in a row and every workgroup reads the whole activation matrix.  Split K over ks workgroups per strip
    // so that strips / nt * ks stays near 256, with wider column tiles as M grows.  Measured (us, before -> after):
    // 4096 x 14336  M=1 10.8 -> 9.5, M=8 13.6 -> 10.6, M=16 16.7 -> 12.0, M=32 29.0 -> 17.4;  8192 x 28672  M=16
    // 36.3 -> 29.1, M=32 58.2 -> 42.5;  4096 x 4096  M=32 10.2 -> 9.4;  8192 x 8192  M=32 18.7 -> 17.1.  Short rows
    // (K = 4096 at M <= 16, K = 8192 at M <= 16) lose to the unsplit kernel and keep it.
    if (mt <= 2 && strips <= 512 && ((mt == 1 && groups >= 96) || (mt == 2 && groups >= 32))) {
        int want_nt = M <= 4 ? 2 : M <= 8 ? (strips > 256 ? 4 : 2) : (mt == 2 && groups < 64) ? 2 : 4;
        while (want_nt > 1 && gemv_lookup(mt, want_nt, 8) == nullptr) want_nt >>= 1;
        int ks = (256 * want_nt + strips / 2) / strips;
        if (ks > 8) ks = 8;
        int want_nw = (M <= 4 && gemv_lookup(mt, want_nt, 16) != nullptr) ? 16 : 8;
        while (ks > 1 && groups / ks < want_nw) --ks;
        if (ks >= 2) {
            *nt_out = want_nt;
            *nw_out = want_nw;
            *ks_out = ks;
        }
    }
}

// ---- ring form: dispatch over (activation loads per group, column tiles per wave) -------------------------------------
typedef void (*gemv_ring_fn)(half_t*, const half_t*, const u4_t*, const half_t*, const half_t*, const half_t*, int, int, int, int,
                             float*, uint32_t*);
struct GemvRingKernel { gemv_ring_fn fn; int slot_bytes, max_depth; };

template <int XI, int NT>
static GemvRingKernel gemv_ring_pick() {
    if constexpr (((XI + 3) / 4) * NT <= 8) return {gemv_ring_kernel<XI, NT>, NT * 1024 + XI * 1024 + 512, gemv_ring_max_depth<XI, NT>()};
    else return {nullptr, 0, 0};
}

template <int XI>
static GemvRingKernel gemv_ring_pick_nt(int nt) {
    switch (nt) {
        case 1: return gemv_ring_pick<XI, 1>();
        case 2: return gemv_ring_pick<XI, 2>();
        case 3: return gemv_ring_pick<XI, 3>();
        case 4: return gemv_ring_pick<XI, 4>();
        case 5: return gemv_ring_pick<XI, 5>();
        case 6: return gemv_ring_pick<XI, 6>();
        case 7: return gemv_ring_pick<XI, 7>();
        case 8: return gemv_ring_pick<XI, 8>();
    }
    return {nullptr, 0, 0};
}

static int gemv_ring_xi(int M) { return M <= 4 ? 1 : M <= 8 ? 2 : M <= 16 ? 4 : M <= 32 ? 8 : M <= 48 ? 12 : 16; }

static GemvRingKernel gemv_ring_lookup(int M, int nt) {
    switch (gemv_ring_xi(M)) {
        case 1: return gemv_ring_pick_nt<1>(nt);
        case 2: return gemv_ring_pick_nt<2>(nt);
        case 4: return gemv_ring_pick_nt<4>(nt);
        case 8: return gemv_ring_pick_nt<8>(nt);
        case 12: return gemv_ring_pick_nt<12>(nt);
        case 16: return gemv_ring_pick_nt<16>(nt);
    }
    return {nullptr, 0, 0};
}

// When the ring form runs, and with which split (graph-replay timings on MI355X, us, register form -> ring form;
// weights rotated through 700 MB):
//   M > 16 (two or more row tiles): always.  4096 x 4096 M=32 9.8 -> 8.1, 6144 x 4096 11.0 -> 9.0, 28672 x 4096 24.6 ->
//   23.2, 4096 x 14336 18.5 -> 16.6, 10240 x 8192 20.5 -> 17.2, 57344 x 8192 80 -> 72, 8192 x 28672 41.7 -> 38.4,
//   3584 x 18944 31.1 -> 19.4.  Column tiles per wave: one per 256 strips (so that about one workgroup lands on each
//   CU), as many as the accumulators allow beyond.
//   M <= 16 on narrow weights: from M = 9 up to 640 column strips (6144 x 4096 M=16 7.3 -> 6.1, 10240 x 8192 13.7 ->
//   13.3), from M = 5 up to 384 (4096 x 4096 M=8 5.4 -> 4.9, M=16 6.9 -> 5.5; 4608 x 3584 M=8 5.8 -> 5.2, M=16 7.4 -> 5.7),
//   from M = 1 up to 320 where K is long (>= 96 groups: 4096 x 14336 M=1 9.9 -> 9.4, M=16 13.2 -> 12.4; 3584 x 18944
//   M=16 15.0 -> 14.2).  Wide weights (28672, 37888, 57344 columns) stay with the register form there (12.2 against
//   13.6 us at 28672 x 4096), as do long, fairly wide ones (8192 x 28672 up to M = 16: 22.5 against 24.9 us at M = 4):
//   their trips are long enough to cover the wait, and the ring's extra hop through LDS costs more than it hides.
//   Long K (>= 96 groups) at M >= 8: two workgroups share a strip's K range and the waves take twice the column tiles,
//   which halves the activation bytes every CU pulls through its L1.
static bool gemv_ring_default(int M, int N, int K, bool can_split, int* nt, int* nw, int* ks, int* depth) {
    const int strips = N / 16, groups = K / 128, mt = (M + 15) / 16, cap = 8 / mt;
    int per_round = (strips + 255) / 256;
    if (per_round > cap) per_round = cap;
    *nw = 8;
    *depth = 2;
    *ks = 1;
    *nt = per_round;
    const bool long_k = can_split && groups >= 96 && strips <= 512;    // without scratch for a split: the unsplit ring
    if (M > 16) {
        if (long_k) {
            *nt = 2 * per_round < cap ? 2 * per_round : cap;
            *ks = 2;
        }
        return true;
    }
    // up to 16 rows: narrow weights only, and the narrower the fewer rows it takes for the ring to win
    const int widest = M >= 9 ? ((groups >= 96) ? 320 : 640) : M >= 5 ? 384 : 320;
    if (strips > widest || !(M >= 5 || groups >= 96)) return false;
    if (M >= 8 && long_k && strips <= 320) {
        *nt = 2;
        *ks = 2;
    }
    return true;
}

#define KMI_GEMV_RING_LDS (160 * 1024 - 256)   // dynamic LDS a workgroup may ask for: the CU's 160 KiB less the static part (arrival flag)

static int gemv_check_args(const void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                           const void* scaled_zeros, int M, int N, int K, int G, const void* workspace) {
    if (!out_f16 || !x_f16 || !qweight || !scales || !scaled_zeros)
        return kmi_set_error(KMI_E_NULL, "kmi_gemv_w4a16: NULL pointer argument");
    if (!kmi_aligned16(x_f16) || !kmi_aligned16(qweight) || (workspace && !kmi_aligned16(workspace)))
        return kmi_set_error(KMI_E_ALIGN, "kmi_gemv_w4a16: x, qweight and workspace must be 16-byte aligned");
    if (G != 128) return kmi_set_error(KMI_E_GROUP, "kmi_gemv_w4a16: group size %d unsupported (128 only)", G);
    if (M < 1 || M > KMI_GEMV_MAX_M)
        return kmi_set_error(KMI_E_M_RANGE, "kmi_gemv_w4a16: M=%d outside 1..%d", M, KMI_GEMV_MAX_M);
    if (N <= 0 || K <= 0 || (N & 15) || (K & 127))
        return kmi_set_error(KMI_E_SHAPE, "kmi_gemv_w4a16: need N%%16==0 and K%%128==0, got N=%d K=%d", N, K);
    return KMI_OK;
}

// The ring form addresses its operands with 32-bit buffer offsets and loads table entries as dwords.
static bool gemv_ring_eligible(const void* scales, const void* scaled_zeros, int M, int N, int K) {
    return !(reinterpret_cast<uintptr_t>(scales) & 3u) && !(reinterpret_cast<uintptr_t>(scaled_zeros) & 3u) &&
           (long)N * K / 2 < (1L << 32) && (long)M * K * 2 < (1L << 32) && (long)(K / 128) * N * 2 < (1L << 32);
}

static int gemv_ring_launch(void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                            const void* scaled_zeros, const void* bias, int M, int N, int K,
                            int nt, int nw, int ks, int depth, void* workspace, size_t workspace_bytes, void* stream) {
    if (!gemv_ring_eligible(scales, scaled_zeros, M, N, K))
        return kmi_set_error(KMI_E_ALIGN, "kmi_gemv_w4a16: the ring form needs 4-byte aligned tables and operands below 4 GiB");
    const GemvRingKernel kn = gemv_ring_lookup(M, nt);
    if (!kn.fn || (nw != 1 && nw != 2 && nw != 4 && nw != 8))
        return kmi_set_error(KMI_E_SHAPE, "kmi_gemv_w4a16: no ring kernel for M=%d nt=%d nw=%d", M, nt, nw);
    const int strips = N / 16, wg_x = (strips + nt - 1) / nt, groups = K / 128;
    if (ks < 1) ks = 1;
    if (ks > groups) ks = groups;
    const size_t need = (size_t)KMI_GEMV_WS_HEADER + (size_t)ks * M * N * sizeof(float);
    if (ks > 1 && (workspace == nullptr || workspace_bytes < need || (size_t)wg_x * sizeof(uint32_t) > KMI_GEMV_WS_HEADER))
        return kmi_set_error(KMI_E_SHAPE, "kmi_gemv_w4a16: %d K splits need %zu bytes of workspace", ks, need);
    // ring depth: what the wave's share of K can use, what vmcnt can count, what LDS holds
    const int per_wave = (groups / ks + nw - 1) / nw;
    if (depth <= 0 || depth > per_wave) depth = per_wave > 0 ? per_wave : 1;
    if (depth > kn.max_depth) depth = kn.max_depth;
    while (depth > 1 && (size_t)nw * depth * kn.slot_bytes > KMI_GEMV_RING_LDS) --depth;
    const int mt = (M + 15) / 16;
    size_t lds = (size_t)nw * depth * kn.slot_bytes;
    const size_t red = (size_t)nw * mt * nt * 4 * 64 * sizeof(float);
    if (red > lds) lds = red;
    if (lds > KMI_GEMV_RING_LDS) return kmi_set_error(KMI_E_SHAPE, "kmi_gemv_w4a16: nt=%d nw=%d needs %zu bytes of LDS", nt, nw, lds);
    if (lds > 64 * 1024) {                                          // opt in to more than 64 KiB of dynamic LDS, once per kernel
        static std::mutex mu;
        static std::set<const void*> raised;
        std::lock_guard<std::mutex> g(mu);
        if (!raised.count(reinterpret_cast<const void*>(kn.fn))) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kn.fn), hipFuncAttributeMaxDynamicSharedMemorySize, KMI_GEMV_RING_LDS) != hipSuccess)
                return kmi_set_error(KMI_E_LAUNCH, "kmi_gemv_w4a16: cannot raise the dynamic LDS limit");
            raised.insert(reinterpret_cast<const void*>(kn.fn));
        }
    }
    uint32_t* counters = static_cast<uint32_t*>(workspace);
    float* partial = workspace ? reinterpret_cast<float*>(static_cast<char*>(workspace) + KMI_GEMV_WS_HEADER) : nullptr;
    hipLaunchKernelGGL(kn.fn, dim3(wg_x, ks), dim3(nw * 64), lds, static_cast<hipStream_t>(stream), static_cast<half_t*>(out_f16),
                       static_cast<const half_t*>(x_f16), static_cast<const u4_t*>(qweight),
                       static_cast<const half_t*>(scales), static_cast<const half_t*>(scaled_zeros),
                       static_cast<const half_t*>(bias), M, N, K, depth, partial, counters);
    return kmi_check_launch("kmi_gemv_w4a16");
}

extern "C" int kmi_gemv_w4a16_ring_cfg(void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                                       const void* scaled_zeros, const void* bias, int M, int N, int K, int G,
                                       int nt, int nw, int ks, int depth, void* workspace, size_t workspace_bytes, void* stream) {
    const int rc = gemv_check_args(out_f16, x_f16, qweight, scales, scaled_zeros, M, N, K, G, workspace);
    if (rc != KMI_OK) return rc;
    return gemv_ring_launch(out_f16, x_f16, qweight, scales, scaled_zeros, bias, M, N, K, nt, nw, ks, depth, workspace,
                            workspace_bytes, stream);
}

// What an automatic call does with a workspace of that many bytes: *form 0 = register form, 1 = ring form.
static void gemv_plan(const void* scales, const void* scaled_zeros, int M, int N, int K, size_t workspace_bytes, bool have_ws,
                      int* form, int* nt, int* nw, int* ks, int* depth) {
    const int mt = (M + 15) / 16, groups = K / 128;
    auto fits = [&](int nt_, int ks_) {                      // scratch of a split: counters of every strip + ks fp32 slices
        const size_t need = (size_t)KMI_GEMV_WS_HEADER + (size_t)ks_ * M * N * sizeof(float);
        const int wg_x = (N / 16 + nt_ - 1) / nt_;
        return have_ws && workspace_bytes >= need && (size_t)wg_x * sizeof(uint32_t) <= KMI_GEMV_WS_HEADER;
    };
    *form = 0;
    *depth = 0;
    if (gemv_ring_eligible(scales, scaled_zeros, M, N, K)) {
        bool ring = gemv_ring_default(M, N, K, true, nt, nw, ks, depth);
        if (ring && *ks > 1 && !fits(*nt, *ks)) ring = gemv_ring_default(M, N, K, false, nt, nw, ks, depth);
        if (ring && gemv_ring_lookup(M, *nt).fn != nullptr) {
            *form = 1;
            return;
        }
    }
    gemv_default_cfg(M, mt, N, K, nt, nw, ks);
    if (*ks > groups) *ks = groups;
    if (*ks > 1 && !fits(*nt, *ks)) *ks = 1;
    *depth = 0;
}

extern "C" int kmi_gemv_w4a16_plan(int M, int N, int K, size_t workspace_bytes, int* form, int* nt, int* nw, int* ks, int* depth) {
    if (M < 1 || M > KMI_GEMV_MAX_M) return kmi_set_error(KMI_E_M_RANGE, "kmi_gemv_w4a16_plan: M=%d outside 1..%d", M, KMI_GEMV_MAX_M);
    if (N <= 0 || K <= 0 || (N & 15) || (K & 127))
        return kmi_set_error(KMI_E_SHAPE, "kmi_gemv_w4a16_plan: need N%%16==0 and K%%128==0, got N=%d K=%d", N, K);
    int f, a, b, c, d;
    gemv_plan(nullptr, nullptr, M, N, K, workspace_bytes, workspace_bytes > 0, &f, &a, &b, &c, &d);
    if (form) *form = f;
    if (nt) *nt = a;
    if (nw) *nw = b;
    if (ks) *ks = c;
    if (depth) *depth = d;
    return KMI_OK;
}

extern "C" int kmi_gemv_w4a16_cfg(void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                                  const void* scaled_zeros, const void* bias, int M, int N, int K, int G,
                                  int nt, int nw, int ks, void* workspace, size_t workspace_bytes, void* stream) {
    const int rc = gemv_check_args(out_f16, x_f16, qweight, scales, scaled_zeros, M, N, K, G, workspace);
    if (rc != KMI_OK) return rc;
    const int mt = (M + 15) / 16;
    const bool automatic = nt <= 0 || nw <= 0;
    if (automatic) {
        int form, depth;
        gemv_plan(scales, scaled_zeros, M, N, K, workspace_bytes, workspace != nullptr, &form, &nt, &nw, &ks, &depth);
        if (form == 1)
            return gemv_ring_launch(out_f16, x_f16, qweight, scales, scaled_zeros, bias, M, N, K, nt, nw, ks, depth, workspace,
                                    workspace_bytes, stream);
    }
    if (ks < 1) ks = 1;
    const int rs = mt == 1 ? gemv_row_spread(M) : 1;
    gemv_fn fn = gemv_lookup(mt, nt, nw, rs);
    if (!fn) return kmi_set_error(KMI_E_SHAPE, "kmi_gemv_w4a16: no kernel for m-tiles=%d nt=%d nw=%d", mt, nt, nw);
    const int strips = N / 16, wg_x = (strips + nt - 1) / nt, groups = K / 128;
    // a split over K needs scratch: [KMI_GEMV_WS_HEADER bytes of per-strip arrival counters, zero between calls]
    // [ks x M x N fp32 partial sums]; without it (or with too little) the call runs unsplit
    if (ks > groups) ks = groups;
    const size_t need = (size_t)KMI_GEMV_WS_HEADER + (size_t)ks * M * N * sizeof(float);
    if (ks > 1 && (workspace == nullptr || workspace_bytes < need || (size_t)wg_x * sizeof(uint32_t) > KMI_GEMV_WS_HEADER)) {
        if (!automatic) return kmi_set_error(KMI_E_SHAPE, "kmi_gemv_w4a16: %d K splits need %zu bytes of workspace", ks, need);
        ks = 1;
    }
    const dim3 grid(wg_x, ks), block(nw * 64);
    const size_t lds = (size_t)nw * mt * nt * (4 / rs) * 64 * sizeof(float);
    uint32_t* counters = static_cast<uint32_t*>(workspace);
    float* partial = workspace ? reinterpret_cast<float*>(static_cast<char*>(workspace) + KMI_GEMV_WS_HEADER) : nullptr;
    hipLaunchKernelGGL(fn, grid, block, lds, static_cast<hipStream_t>(stream), static_cast<half_t*>(out_f16),
                       static_cast<const half_t*>(x_f16), static_cast<const u4_t*>(qweight),
                       static_cast<const half_t*>(scales), static_cast<const half_t*>(scaled_zeros),
                       static_cast<const half_t*>(bias), M, N, K, partial, counters);
    return kmi_check_launch("kmi_gemv_w4a16");
}

// Arrival counters back to zero.  The kernels leave them zero themselves; this is for a buffer whose history is
// unknown (a launch that failed or was abandoned half-way).  A plain fill kernel, so that it can be captured
// into a graph where a memset node cannot.
__global__ __launch_bounds__(256) void gemv_ws_reset_kernel(uint32_t* counters, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) counters[i] = 0u;
}

extern "C" int kmi_gemv_ws_reset(void* workspace, size_t workspace_bytes, void* stream) {
    if (!workspace) return kmi_set_error(KMI_E_NULL, "kmi_gemv_ws_reset: workspace is NULL");
    if (!kmi_aligned16(workspace)) return kmi_set_error(KMI_E_ALIGN, "kmi_gemv_ws_reset: workspace is not 16-byte aligned");
    if (workspace_bytes < KMI_GEMV_WS_HEADER)
        return kmi_set_error(KMI_E_SHAPE, "kmi_gemv_ws_reset: a workspace holds at least its %d-byte counter header", KMI_GEMV_WS_HEADER);
    const int n = KMI_GEMV_WS_HEADER / (int)sizeof(uint32_t);
    hipLaunchKernelGGL(gemv_ws_reset_kernel, dim3((n + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint32_t*>(workspace), n);
    return kmi_check_launch("kmi_gemv_ws_reset");
}

extern "C" int kmi_gemv_w4a16(void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                              const void* scaled_zeros, const void* bias, int M, int N, int K, int G,
                              void* workspace, size_t workspace_bytes, void* stream) {
    return kmi_gemv_w4a16_cfg(out_f16, x_f16, qweight, scales, scaled_zeros, bias, M, N, K, G, 0, 0, 0, workspace,
                              workspace_bytes, stream);
}

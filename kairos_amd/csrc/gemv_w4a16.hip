// W4A16 product for decode-sized M (1..64): the packed uint4 weights are streamed from HBM exactly
// once with 16-byte loads, decoded to fp16 in registers (bit-identical to the fp16 converter) and fed
// to v_mfma_f32_16x16x32_f16 with fp32 accumulation.
//
// Work split.  A workgroup owns 16*NT output columns; its NW waves interleave over the 128-wide K
// groups (wave w takes groups w, w+NW, ...), so the workgroup as a whole walks contiguous memory:
// the four-row interleave makes a 16-row strip one contiguous K*8-byte region.  Partial sums meet in
// LDS and are added in a fixed order (deterministic output).
//
// Lane roles inside a wave, for one K group and one 16-column tile: lane = (r16, j), r16 = lane&15,
// j = lane>>4.  The lane loads the 16-byte chunk of row n = tile*16 + r16 that covers
// k = 128c + 32j .. +31; nibble plane a of its four words decodes to the eight K-contiguous weights
// k = 128c + 32j + 8a .. +7, which is exactly the MFMA B fragment of lane (col r16, k-block j).  The
// matching A fragment is x[m = r16][same eight k], one 16-byte load.  Four MFMAs (a = 0..3) per tile
// consume the group.
#include "kmi_common.h"

template <int MT, int NT, int NW>
__global__ __launch_bounds__(NW * 64) void gemv_w4a16_kernel(half_t* __restrict__ out, const half_t* __restrict__ x,
                                                             const u4_t* __restrict__ qw,
                                                             const half_t* __restrict__ scales,
                                                             const half_t* __restrict__ szeros,
                                                             const half_t* __restrict__ bias, int M, int N, int K) {
    extern __shared__ float red[];               // [NW][MT*NT*4][64]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int j = lane >> 4;
    const int n0 = blockIdx.x * (16 * NT);
    const int ngroups = K >> 7;
    const int kq = K >> 3;                       // 16-byte units per fp16 row of x / per four-row weight block

    f4_t acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f4_t{0.f, 0.f, 0.f, 0.f};

    const u4_t* wp[NT];
    int ncol[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int n = n0 + nt * 16 + r16;
        n = n < N ? n : N - 1;                   // partial last strip: clamp loads, stores are masked
        ncol[nt] = n;
        wp[nt] = qw + (long)(n >> 2) * kq + (n & 3) * 2 + (j & 1) + (j >> 1) * 8;
    }
    const h8_t* xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int m = mt * 16 + r16;
        m = m < M ? m : M - 1;
        xp[mt] = reinterpret_cast<const h8_t*>(x) + (long)m * kq + j * 4;
    }

    for (int c = wave; c < ngroups; c += NW) {
        u4_t u[NT];
        half_t s[NT], z[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            u[nt] = __builtin_nontemporal_load(wp[nt] + c * 16);
            s[nt] = scales[(long)c * N + ncol[nt]];
            z[nt] = szeros[(long)c * N + ncol[nt]];
        }
        h8_t xa[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int a = 0; a < 4; ++a) xa[mt][a] = xp[mt][c * 16 + a];

#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const h2_t s2 = {s[nt], s[nt]};
            const h2_t z2 = {z[nt], z[nt]};
            h8_t b[4];
            b[0] = dequant_nibble<0>(u[nt], s2, z2);
            b[1] = dequant_nibble<1>(u[nt], s2, z2);
            b[2] = dequant_nibble<2>(u[nt], s2, z2);
            b[3] = dequant_nibble<3>(u[nt], s2, z2);
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt][a], b[a], acc[mt][nt], 0, 0, 0);
        }
    }

    constexpr int R = MT * NT * 4;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[(wave * R + (mt * NT + nt) * 4 + i) * 64 + lane] = acc[mt][nt][i];
    __syncthreads();

    for (int idx = threadIdx.x; idx < R * 64; idx += NW * 64) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) v += red[w * R * 64 + idx];
        const int l = idx & 63, reg = idx >> 6;
        const int i = reg & 3, t = reg >> 2;
        const int nt = t % NT, mt = t / NT;
        const int m = mt * 16 + 4 * (l >> 4) + i;
        const int n = n0 + nt * 16 + (l & 15);
        if (m < M && n < N) {
            half_t h = (half_t)v;
            if (bias) h = (half_t)((float)h + (float)bias[n]);
            out[(long)m * N + n] = h;
        }
    }
}

typedef void (*gemv_fn)(half_t*, const half_t*, const u4_t*, const half_t*, const half_t*, const half_t*, int, int, int);

template <int MT, int NT, int NW>
static constexpr bool gemv_cfg_ok() {
    return MT * NT <= 8 && NW * MT * NT <= 64 && (NW < 16 || MT * NT <= 2);
}

template <int MT, int NT, int NW>
static gemv_fn gemv_pick() {
    if constexpr (gemv_cfg_ok<MT, NT, NW>()) return gemv_w4a16_kernel<MT, NT, NW>;
    else return nullptr;
}

template <int MT, int NT>
static gemv_fn gemv_pick_nw(int nw) {
    switch (nw) {
        case 4: return gemv_pick<MT, NT, 4>();
        case 8: return gemv_pick<MT, NT, 8>();
        case 16: return gemv_pick<MT, NT, 16>();
    }
    return nullptr;
}

template <int MT>
static gemv_fn gemv_pick_nt(int nt, int nw) {
    switch (nt) {
        case 1: return gemv_pick_nw<MT, 1>(nw);
        case 2: return gemv_pick_nw<MT, 2>(nw);
        case 4: return gemv_pick_nw<MT, 4>(nw);
    }
    return nullptr;
}

static gemv_fn gemv_lookup(int mt, int nt, int nw) {
    switch (mt) {
        case 1: return gemv_pick_nt<1>(nt, nw);
        case 2: return gemv_pick_nt<2>(nt, nw);
        case 3: return gemv_pick_nt<3>(nt, nw);
        case 4: return gemv_pick_nt<4>(nt, nw);
    }
    return nullptr;
}

// Default split: enough waves to keep every SIMD streaming (>= 8 per CU) while each wave still owns
// at least two K groups.
static void gemv_default_cfg(int mt, int N, int K, int* nt_out, int* nw_out) {
    const int strips = (N + 15) / 16, groups = K / 128;
    const int want_waves = 2048;
    int nt = 4, nw = 4;
    while (nt > 1 && ((strips + nt - 1) / nt * nw < want_waves || mt * nt > 8)) nt >>= 1;
    while (nw < 16 && (strips + nt - 1) / nt * nw < want_waves && groups / (nw * 2) >= 2 &&
           gemv_lookup(mt, nt, nw * 2) != nullptr)
        nw <<= 1;
    *nt_out = nt;
    *nw_out = nw;
}

extern "C" int kmi_gemv_w4a16_cfg(void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                                  const void* scaled_zeros, const void* bias, int M, int N, int K, int G,
                                  int nt, int nw, void* stream) {
    if (!out_f16 || !x_f16 || !qweight || !scales || !scaled_zeros)
        return kmi_set_error(KMI_E_NULL, "kmi_gemv_w4a16: NULL pointer argument");
    if (!kmi_aligned16(x_f16) || !kmi_aligned16(qweight))
        return kmi_set_error(KMI_E_ALIGN, "kmi_gemv_w4a16: x and qweight must be 16-byte aligned");
    if (G != 128) return kmi_set_error(KMI_E_GROUP, "kmi_gemv_w4a16: group size %d unsupported (128 only)", G);
    if (M < 1 || M > KMI_GEMV_MAX_M)
        return kmi_set_error(KMI_E_M_RANGE, "kmi_gemv_w4a16: M=%d outside 1..%d", M, KMI_GEMV_MAX_M);
    if (N <= 0 || K <= 0 || (N & 15) || (K & 127))
        return kmi_set_error(KMI_E_SHAPE, "kmi_gemv_w4a16: need N%%16==0 and K%%128==0, got N=%d K=%d", N, K);
    const int mt = (M + 15) / 16;
    if (nt <= 0 || nw <= 0) gemv_default_cfg(mt, N, K, &nt, &nw);
    gemv_fn fn = gemv_lookup(mt, nt, nw);
    if (!fn) return kmi_set_error(KMI_E_SHAPE, "kmi_gemv_w4a16: no kernel for m-tiles=%d nt=%d nw=%d", mt, nt, nw);
    const int strips = N / 16;
    const dim3 grid((strips + nt - 1) / nt), block(nw * 64);
    const size_t lds = (size_t)nw * mt * nt * 4 * 64 * sizeof(float);
    hipLaunchKernelGGL(fn, grid, block, lds, static_cast<hipStream_t>(stream), static_cast<half_t*>(out_f16),
                       static_cast<const half_t*>(x_f16), static_cast<const u4_t*>(qweight),
                       static_cast<const half_t*>(scales), static_cast<const half_t*>(scaled_zeros),
                       static_cast<const half_t*>(bias), M, N, K);
    return kmi_check_launch("kmi_gemv_w4a16");
}

extern "C" int kmi_gemv_w4a16(void* out_f16, const void* x_f16, const void* qweight, const void* scales,
                              const void* scaled_zeros, const void* bias, int M, int N, int K, int G, void* stream) {
    return kmi_gemv_w4a16_cfg(out_f16, x_f16, qweight, scales, scaled_zeros, bias, M, N, K, G, 0, 0, stream);
}

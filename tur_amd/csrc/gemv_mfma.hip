// Skinny quantized matmul (decode / small batches, m <= 32) on the tiled layout.
//
// One workgroup owns one 16-row tile of the weight; its waves split the 256-column tiles of that
// row tile between them (wave w takes b = w, w + W, ...), so at any moment the workgroup streams one
// contiguous stretch of HBM.  For every tile a wave issues lane-linear 16-byte loads of the packed
// quants, turns them into exact integer-valued f16 B operands with v_and_or_b32 / v_pk_fma_f16
// (mfma_common.h), and feeds v_mfma_f32_16x16x32_f16 with the prepared activations as A operand.
// Block scales that are not integers (d, dmin) are applied in f32 on the 16x16 result of each
// tile.  Waves reduce their partial tiles through LDS; wave 0 adds the bias and stores.
//
// HBM traffic per launch = the weight once (+ activations and outputs, tiny): the kernel is bound
// by HBM bandwidth, the VALU unpack (about 2 to 3 instructions per weight byte) rides along.
#include "layout.h"
#include "mfma_common.h"

namespace {

constexpr uint32_t kMagic1024 = 0x64006400u;  // 1024.0 in both halves
constexpr uint32_t kMagic256 = 0x5C005C00u;   // 256.0
constexpr uint32_t kMagic16 = 0x4C004C00u;    // 16.0
constexpr uint32_t kMagic4 = 0x44004400u;     // 4.0

__device__ inline float h2f_bits(uint32_t bits16) {
    const uint16_t u = (uint16_t)bits16;
    _Float16 h;
    __builtin_memcpy(&h, &u, 2);
    return (float)h;
}

// activation fragment of step q for this lane (zero for rows beyond the prepared height)
__device__ inline half8v load_afrag(const half8v *__restrict__ tile_frags, int q, int g, int r, int mpad) {
    half8v z = {0, 0, 0, 0, 0, 0, 0, 0};
    if (r < mpad) z = tile_frags[(q * 4 + g) * mpad + r];
    return z;
}

// The 6-bit scales and mins of the two sub-blocks a lane owns, as packed f16 constants.
struct K4Consts {
    half2v s_lo, s16_lo, c1_lo, c2_lo;  // sub-block 2g:   scale, scale/16, -1024*scale, -64*scale
    half2v s_hi, s16_hi, c1_hi, c2_hi;  // sub-block 2g+1
    half8v bmin;                        // (m_lo x4, m_hi x4) against the group-sum fragment
    float d, dmin;
};

__device__ inline K4Consts k4_consts(uint4v hd, int g) {
    // 24-bit group g of the 96-bit field in hd.y, hd.z, hd.w
    const uint32_t lo = g < 2 ? hd.y : (g == 2 ? hd.z : hd.w);
    const uint32_t hi = g == 1 ? hd.z : hd.w;
    const uint32_t G = __builtin_amdgcn_alignbit(hi, lo, (uint32_t)((24 * g) & 31));
    const half2v k1024 = splat2((_Float16)1024.0f);
    // (sc_lo, sc_hi) and (m_lo, m_hi) through the 1024 + v trick
    const half2v sc = as_half2((G & 0x3Fu) | ((G << 4) & 0x003F0000u) | kMagic1024) - k1024;
    const half2v mn = as_half2(((G >> 6) & 0x3Fu) | ((G >> 2) & 0x003F0000u) | kMagic1024) - k1024;
    K4Consts c;
    c.s_lo = splat2(sc.x);
    c.s_hi = splat2(sc.y);
    c.s16_lo = c.s_lo * splat2((_Float16)0.0625f);
    c.s16_hi = c.s_hi * splat2((_Float16)0.0625f);
    c.c1_lo = c.s_lo * splat2((_Float16)-1024.0f);
    c.c1_hi = c.s_hi * splat2((_Float16)-1024.0f);
    c.c2_lo = c.s_lo * splat2((_Float16)-64.0f);
    c.c2_hi = c.s_hi * splat2((_Float16)-64.0f);
    c.bmin = half8v{mn.x, mn.x, mn.x, mn.x, mn.y, mn.y, mn.y, mn.y};
    c.d = h2f_bits(hd.x & 0xFFFFu);
    c.dmin = h2f_bits(hd.x >> 16);
    return c;
}

// eight nibbles of a Q4_K / Q5_K step dword -> exact (nibble [+16*high]) * scale as f16 B operand
template <bool HIGH>
__device__ inline half8v k45_operand(uint32_t w, half2v s, half2v s16, half2v c1, half2v c2, uint32_t h0, uint32_t h1,
                                     int u0) {
    const uint32_t w8 = w >> 8;
    uint32_t t0 = (w & 0x000F000Fu) | kMagic1024;
    uint32_t t1 = (w & 0x00F000F0u) | kMagic1024;
    uint32_t t2 = (w8 & 0x000F000Fu) | kMagic1024;
    uint32_t t3 = (w8 & 0x00F000F0u) | kMagic1024;
    if (HIGH) {  // fifth bit: +16 on top of the nibble (bit 4 / 20, or bit 8 / 24 for the x16 form)
        t0 |= rotr32(h0, (uint32_t)u0) & 0x00100010u;
        t1 |= rotr32(h1, (uint32_t)u0) & 0x01000100u;
        t2 |= rotr32(h0, (uint32_t)(u0 + 1)) & 0x00100010u;
        t3 |= rotr32(h1, (uint32_t)(u0 + 1)) & 0x01000100u;
    }
    return make_half8(pk_fma(as_half2(t0), s, c1), pk_fma(as_half2(t1), s16, c2), pk_fma(as_half2(t2), s, c1),
                      pk_fma(as_half2(t3), s16, c2));
}

template <int DT, int MT> struct TileOp;

// ---- Q4_K and Q5_K ----
template <int DT, int MT> struct TileOpK45 {
    using F = TiledFmt<DT>;
    static constexpr bool HIGH = DT == TURQ_Q5_K;
    __device__ static void run(const uint8_t *__restrict__ tile, const half8v *__restrict__ fr, int64_t mt_stride,
                               int mpad, int lane, float4v *acc) {
        const int r = lane & 15, g = lane >> 4;
        const uint4v qa = *(const uint4v *)(tile + F::kQA + 16 * lane);
        const uint4v qb = *(const uint4v *)(tile + F::kQB + 16 * lane);
        const uint4v hd = *(const uint4v *)(tile + F::kHDR + 16 * r);
        uint2v hh = {0, 0};
        if constexpr (HIGH) hh = *(const uint2v *)(tile + TiledFmt<TURQ_Q5_K>::kQH + 8 * lane);
        const K4Consts c = k4_consts(hd, g);
        const uint32_t wq[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        float4v tmp[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) tmp[mt] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const half8v bop = i < 4 ? k45_operand<HIGH>(wq[i], c.s_lo, c.s16_lo, c.c1_lo, c.c2_lo, hh.x, hh.y, 2 * i)
                                     : k45_operand<HIGH>(wq[i], c.s_hi, c.s16_hi, c.c1_hi, c.c2_hi, hh.x, hh.y, 2 * i);
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
                tmp[mt] = mfma16x16x32(load_afrag(fr + mt * mt_stride, i, g, r, mpad), bop, tmp[mt]);
        }
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            const float4v tmin =
                mfma16x16x32(load_afrag(fr + mt * mt_stride, 8, g, r, mpad), c.bmin, float4v{0.f, 0.f, 0.f, 0.f});
            acc[mt] += c.d * tmp[mt] - c.dmin * tmin;
        }
    }
};
template <int MT> struct TileOp<TURQ_Q4_K, MT> : TileOpK45<TURQ_Q4_K, MT> {};
template <int MT> struct TileOp<TURQ_Q5_K, MT> : TileOpK45<TURQ_Q5_K, MT> {};

// ---- Q6_K ----
template <int MT> struct TileOp<TURQ_Q6_K, MT> {
    using F = TiledFmt<TURQ_Q6_K>;
    __device__ static void run(const uint8_t *__restrict__ tile, const half8v *__restrict__ fr, int64_t mt_stride,
                               int mpad, int lane, float4v *acc) {
        const int r = lane & 15, g = lane >> 4;
        const uint4v qla = *(const uint4v *)(tile + F::kQLA + 16 * lane);
        const uint4v qlb = *(const uint4v *)(tile + F::kQLB + 16 * lane);
        const uint4v qh = *(const uint4v *)(tile + F::kQH + 16 * lane);
        const uint32_t scw = *(const uint32_t *)(tile + F::kSC + 4 * lane);
        const float d = h2f_bits(*(const uint16_t *)(tile + F::kD + 2 * r));
        const uint32_t wl[8] = {qla.x, qla.y, qla.z, qla.w, qlb.x, qlb.y, qlb.z, qlb.w};
        const uint32_t wh[4] = {qh.x, qh.y, qh.z, qh.w};
        float4v tmp[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) tmp[mt] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sg = 0; sg < 4; sg++) {  // scale group sg covers steps 2sg, 2sg+1
            const _Float16 sc = (_Float16)(float)(int)(int8_t)(scw >> (8 * sg));
            const half2v s1 = splat2(sc);
            const half2v c256 = s1 * splat2((_Float16)-256.0f);
            const half2v c16 = s1 * splat2((_Float16)-16.0f);
            const half2v s16 = s1 * splat2((_Float16)16.0f);
            const half2v c288 = s1 * splat2((_Float16)-288.0f);
            const half2v c96 = s1 * splat2((_Float16)-96.0f);
#pragma unroll
            for (int ii = 0; ii < 2; ii++) {
                const int i = 2 * sg + ii;
                // low nibbles: n * sc
                const uint32_t w = wl[i];
                const uint32_t w8 = rotr32(w, 8);
                const half8v b1 = make_half8(pk_fma(and_or_h2(w, 0x003C003Cu, kMagic256), s1, c256),
                                             pk_fma(and_or_h2(w, 0x03C003C0u, kMagic16), s1, c16),
                                             pk_fma(and_or_h2(w8, 0x003C003Cu, kMagic256), s1, c256),
                                             pk_fma(and_or_h2(w8, 0x03C003C0u, kMagic16), s1, c16));
                // high two bits: 16 * (h - 2) * sc   (the "- 32" of the 6-bit value lives here)
                const uint32_t hA = ii == 0 ? wh[sg] : rotr32(wh[sg], 8);
                const uint32_t hB = rotr32(hA, 4);
                const half8v b2 = make_half8(pk_fma(and_or_h2(hA, 0x00C000C0u, kMagic16), s16, c288),
                                             pk_fma(and_or_h2(hA, 0x03000300u, kMagic4), s16, c96),
                                             pk_fma(and_or_h2(hB, 0x00C000C0u, kMagic16), s16, c288),
                                             pk_fma(and_or_h2(hB, 0x03000300u, kMagic4), s16, c96));
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    const half8v a = load_afrag(fr + mt * mt_stride, i, g, r, mpad);
                    tmp[mt] = mfma16x16x32(a, b1, tmp[mt]);
                    tmp[mt] = mfma16x16x32(a, b2, tmp[mt]);
                }
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[mt] += d * tmp[mt];
    }
};

// ---- Q8_0 ----
template <int MT> struct TileOp<TURQ_Q8_0, MT> {
    using F = TiledFmt<TURQ_Q8_0>;
    __device__ static void run(const uint8_t *__restrict__ tile, const half8v *__restrict__ fr, int64_t mt_stride,
                               int mpad, int lane, float4v *acc) {
        const int r = lane & 15, g = lane >> 4;
        uint4v p[4];
#pragma unroll
        for (int i = 0; i < 4; i++) p[i] = *(const uint4v *)(tile + 1024 * i + 16 * lane);
        const uint4v dd = *(const uint4v *)(tile + F::kD + 16 * r);
        const uint32_t dw[4] = {dd.x, dd.y, dd.z, dd.w};
        const half2v k1152 = splat2((_Float16)-1152.0f);  // 1024 + the 128 the bytes were offset by
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const uint32_t w0 = (q & 1) ? p[q >> 1].z : p[q >> 1].x;
            const uint32_t w1 = (q & 1) ? p[q >> 1].w : p[q >> 1].y;
            const half8v bop = make_half8(and_or_h2(w0, 0x00FF00FFu, kMagic1024) + k1152,
                                          and_or_h2(w0 >> 8, 0x00FF00FFu, kMagic1024) + k1152,
                                          and_or_h2(w1, 0x00FF00FFu, kMagic1024) + k1152,
                                          and_or_h2(w1 >> 8, 0x00FF00FFu, kMagic1024) + k1152);
            const float d = h2f_bits((q & 1) ? (dw[q >> 1] >> 16) : (dw[q >> 1] & 0xFFFFu));
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                const float4v t = mfma16x16x32(load_afrag(fr + mt * mt_stride, q, g, r, mpad), bop,
                                               float4v{0.f, 0.f, 0.f, 0.f});
                acc[mt] += d * t;
            }
        }
    }
};

template <int DT, int MT, int YT>
__global__ void __launch_bounds__(512) gemv_mfma_kernel(const uint8_t *__restrict__ w, int64_t n, int64_t ntc,
                                                         const half8v *__restrict__ frags, int64_t m, int mpad,
                                                         void *__restrict__ y, int64_t ldy,
                                                         const float *__restrict__ bias) {
    extern __shared__ float4v red[];  // [wave][mt][lane]
    constexpr int NQ = DT == TURQ_Q8_0 ? TURQ_NQ_Q8_0 : TURQ_NQ_KQUANT;
    constexpr int TB = TiledFmt<DT>::kTileBytes;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const int64_t rt = blockIdx.x;
    const int64_t tile_chunks = (int64_t)NQ * 4 * mpad;  // 16-byte chunks of one (mt, b) fragment set
    const int64_t mt_stride = ntc * tile_chunks;
    float4v acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[mt] = float4v{0.f, 0.f, 0.f, 0.f};
    const uint8_t *wrow = w + rt * ntc * TB;
    for (int64_t b = wave; b < ntc; b += nwaves)
        TileOp<DT, MT>::run(wrow + b * TB, frags + b * tile_chunks, mt_stride, mpad, lane, acc);

    if (nwaves > 1) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) red[(wave * MT + mt) * 64 + lane] = acc[mt];
        __syncthreads();
        if (wave != 0) return;
        for (int wv = 1; wv < nwaves; wv++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[mt] += red[(wv * MT + mt) * 64 + lane];
    }
    // lane (nn, g) holds y[16 mt + 4 g + i][16 rt + nn], i = 0..3
    const int nn = lane & 15, g = lane >> 4;
    const int64_t col = rt * 16 + nn;
    if (col >= n) return;
    const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int64_t row = 16 * mt + 4 * g + i;
            if (row < m) turq_store_out<YT>(y, row * ldy + col, acc[mt][i] + bv);
        }
}

template <int DT, int MT>
hipError_t launch2(int yt, const void *w, int64_t n, int64_t k, const void *frags, int64_t m, void *y, int64_t ldy,
                   const float *bias, int nwaves, hipStream_t s) {
    const int64_t ntc = turq_tile_cols(k);
    const int mpad = MT > 1 ? 16 : turq_mpad(m);
    const unsigned grid = (unsigned)turq_tile_rows(n);
    const size_t lds = nwaves > 1 ? (size_t)nwaves * MT * 64 * sizeof(float4v) : 0;
    const dim3 block((unsigned)(64 * nwaves));
#define TURQ_GO(YT)                                                                                            \
    gemv_mfma_kernel<DT, MT, YT><<<grid, block, lds, s>>>((const uint8_t *)w, n, ntc, (const half8v *)frags, m, \
                                                           mpad, y, ldy, bias)
    switch (yt) {
    case TURQ_ACT_F32: TURQ_GO(TURQ_ACT_F32); break;
    case TURQ_ACT_BF16: TURQ_GO(TURQ_ACT_BF16); break;
    case TURQ_ACT_F16: TURQ_GO(TURQ_ACT_F16); break;
    default: return hipErrorInvalidValue;
    }
#undef TURQ_GO
    return hipGetLastError();
}

template <int DT>
hipError_t launch1(int yt, const void *w, int64_t n, int64_t k, const void *frags, int64_t m, void *y, int64_t ldy,
                   const float *bias, int nwaves, hipStream_t s) {
    if (m <= 16) return launch2<DT, 1>(yt, w, n, k, frags, m, y, ldy, bias, nwaves, s);
    return launch2<DT, 2>(yt, w, n, k, frags, m, y, ldy, bias, nwaves, s);
}

}  // namespace

hipError_t turq_launch_gemv_mfma(int dtype, const void *w, int64_t n, int64_t k, const void *frags, int64_t m, void *y,
                                 int y_dtype, int64_t ldy, const float *bias, int nwaves, hipStream_t stream) {
    if (n == 0 || m == 0) return hipSuccess;
    if (m > TURQ_GEMV_MAX_M || nwaves < 1 || nwaves > 8) return hipErrorInvalidValue;
    switch (dtype) {
    case TURQ_Q4_K: return launch1<TURQ_Q4_K>(y_dtype, w, n, k, frags, m, y, ldy, bias, nwaves, stream);
    case TURQ_Q5_K: return launch1<TURQ_Q5_K>(y_dtype, w, n, k, frags, m, y, ldy, bias, nwaves, stream);
    case TURQ_Q6_K: return launch1<TURQ_Q6_K>(y_dtype, w, n, k, frags, m, y, ldy, bias, nwaves, stream);
    case TURQ_Q8_0: return launch1<TURQ_Q8_0>(y_dtype, w, n, k, frags, m, y, ldy, bias, nwaves, stream);
    default: return hipErrorInvalidValue;
    }
}

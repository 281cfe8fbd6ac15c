// Quantized matmul for prefill chunks (m > 32) on the tiled layout: the only shape of this path that
// is a dense contraction, so this kernel is priced against the MFMA peak, not HBM.
//
// Workgroup tile 256 (m) x 96 (n), 4 waves stacked along m, wave tile 64 x 96 = 4 x 6 MFMA tiles of
// v_mfma_f32_16x16x32_f16 (96 accumulator registers): every A fragment read from LDS feeds 6 MFMAs,
// which keeps the LDS traffic (about 64 KiB per 64-column stage and workgroup) under the LDS bandwidth.  Activations arrive prepared in A-fragment
// order (act_prep.hip) and are staged through LDS, two operand steps (64 columns) per stage, double
// buffered, one barrier per stage.  Weights do NOT go through LDS: each wave loads the packed tiles
// of its three row tiles straight into registers (lane-linear 16-byte loads) and unpacks them with
// the same and_or / pk_fma arithmetic as the GEMV kernel; one unpacked B operand feeds 8 MFMAs.
//
// Block scales.  The GEMV kernel keeps the weights as exact integers and applies d / dmin in f32 on
// each tile result; with 96 accumulators that would need a second accumulator set.  Here the f16
// super-block scale is folded into the packed-f16 constants instead: B = nibble * f16(d * sc) (two
// roundings of 2^-12 relative), and the "- dmin * m" term is one extra MFMA per super-block against
// the activation group sums with B = -f16(dmin * m).  Measured against the f32 matmul on dequantized
// weights this costs about 2e-4 relative L2 (bar: 1e-3).
#include <hip/hip_ext.h>

#include "layout.h"
#include "mfma_common.h"

namespace {

constexpr uint32_t kMagic1024 = 0x64006400u;
constexpr int BM = 256, BN = 96;            // workgroup tile
constexpr int WM_TILES = 4, WN_TILES = 6;   // MFMA tiles per wave: 64 x 96
constexpr uint32_t kMagic64 = 0x54005400u;  // 64.0: a nibble in mantissa bits 4..7 reads as 64 + n
constexpr int STAGE_BLOCKS = 32;            // 2 operand steps x 16 m-tiles of 1 KiB per LDS stage

__device__ inline _Float16 h_from_bits(uint32_t bits16) {
    const uint16_t u = (uint16_t)bits16;
    _Float16 h;
    __builtin_memcpy(&h, &u, 2);
    return h;
}

// Per (row tile, super-block) constants of a lane for Q4_K: lane (n, g) owns sub-blocks 2g, 2g+1.
struct Q4Consts {
    half2v s[2], c1[2], c2[2];  // [0] sub-block 2g, [1] sub-block 2g+1: d*sc, -1024*d*sc, -64*d*sc
    half2v dmn;                 // -(dmin*m_lo, dmin*m_hi)
};

__device__ inline Q4Consts q4_consts(uint4v hd, int g) {
    const uint32_t lo = g < 2 ? hd.y : (g == 2 ? hd.z : hd.w);
    const uint32_t hi = g == 1 ? hd.z : hd.w;
    const uint32_t G = __builtin_amdgcn_alignbit(hi, lo, (uint32_t)((24 * g) & 31));
    const half2v k1024 = splat2((_Float16)1024.0f);
    const half2v sc = as_half2((G & 0x3Fu) | ((G << 4) & 0x003F0000u) | kMagic1024) - k1024;
    const half2v mn = as_half2(((G >> 6) & 0x3Fu) | ((G >> 2) & 0x003F0000u) | kMagic1024) - k1024;
    const half2v dsc = sc * splat2(h_from_bits(hd.x & 0xFFFFu));          // (d*sc_lo, d*sc_hi), rounded to f16
    const half2v dmn = mn * splat2((_Float16)(-(float)h_from_bits(hd.x >> 16)));  // -(dmin*m_lo, dmin*m_hi)
    Q4Consts c;
    c.s[0] = splat2(dsc.x);
    c.s[1] = splat2(dsc.y);
#pragma unroll
    for (int h = 0; h < 2; h++) {
        c.c1[h] = c.s[h] * splat2((_Float16)-1024.0f);
        c.c2[h] = c.s[h] * splat2((_Float16)-64.0f);
    }
    c.dmn = dmn;
    return c;
}

// low nibbles read as 1024 + n, high nibbles (mantissa bits 4..7 of 64.0) as 64 + n: one scale, two offsets
__device__ inline half8v q4_operand(uint32_t w, half2v s, half2v c1, half2v c2) {
    const uint32_t w8 = w >> 8;
    return make_half8(pk_fma(and_or_h2(w, 0x000F000Fu, kMagic1024), s, c1), pk_fma(and_or_h2(w, 0x00F000F0u, kMagic64), s, c2),
                      pk_fma(and_or_h2(w8, 0x000F000Fu, kMagic1024), s, c1), pk_fma(and_or_h2(w8, 0x00F000F0u, kMagic64), s, c2));
}

struct Q4Tile { uint4v qa, qb, hd; };

__device__ inline Q4Tile q4_load(const uint8_t *__restrict__ tile, int lane) {
    using F = TiledFmt<TURQ_Q4_K>;
    Q4Tile t;
    t.qa = *(const uint4v *)(tile + F::kQA + 16 * lane);
    t.qb = *(const uint4v *)(tile + F::kQB + 16 * lane);
    t.hd = *(const uint4v *)(tile + F::kHDR + 16 * (lane & 15));
    return t;
}

// frags: prepared activations, chunk (16 B) index (((mt * ntc + b) * 9 + q) * 64 + lane); mtiles = ceil(m / 16)
__global__ void __launch_bounds__(256) gemm_q4k_kernel(const uint8_t *__restrict__ w, int64_t n, int64_t k,
                                                       const uint4v *__restrict__ frags, int64_t m, void *__restrict__ y,
                                                       int yt, int64_t ldy, const float *__restrict__ bias, int nblocks_n,
                                                       int nblocks_m) {
    __shared__ uint4v lds[2][STAGE_BLOCKS * 64];  // 2 x 32 KiB
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave, wn = 0;
    const int g = lane >> 4;
    // Workgroups of one XCD (blockIdx % 8) get consecutive logical ids, and the m-blocks of one n-block are
    // consecutive in that order: the packed weights they share stay in that XCD's L2.
    const int nwg = nblocks_n * nblocks_m;
    int lid = blockIdx.x;
    if ((nwg & 7) == 0) lid = (blockIdx.x & 7) * (nwg >> 3) + (blockIdx.x >> 3);
    const int nb = lid / nblocks_m, mb = lid - nb * nblocks_m;
    const int64_t ntc = turq_tile_cols(k);
    const int64_t mtiles = (m + 15) / 16;
    const int64_t nrt = turq_tile_rows(n);
    constexpr int TB = TiledFmt<TURQ_Q4_K>::kTileBytes;

    // this wave's three row tiles (clamped: results of tiles past the end are never stored)
    int64_t rt[WN_TILES];
#pragma unroll
    for (int j = 0; j < WN_TILES; j++) {
        const int64_t r = (int64_t)nb * (BN / 16) + wn * WN_TILES + j;
        rt[j] = r < nrt ? r : nrt - 1;
    }

    float4v acc[WM_TILES][WN_TILES];
#pragma unroll
    for (int i = 0; i < WM_TILES; i++)
#pragma unroll
        for (int j = 0; j < WN_TILES; j++) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

    // stage s = 5 * b + ks: ks < 4 copies operand steps (2ks, 2ks+1) of super-block b for 16 m-tiles,
    // ks == 4 copies the group-sum fragment (q = 8); each thread moves 8 (or 4) chunks of 16 B
    const int64_t nstages = ntc * 5;
    uint4v stage_regs[8];
    auto stage_load = [&](int64_t s) {
        const int64_t b = s / 5;
        const int ks = (int)(s - b * 5);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int c = tid + 256 * i;          // chunk within the stage
            const int blk = c >> 6;               // 0..31: (qq, mt)
            const int qq = blk >> 4, mt = blk & 15;
            const int q = ks < 4 ? 2 * ks + qq : 8;
            const int64_t mtg = (int64_t)mb * (BM / 16) + mt;
            uint4v v = {0, 0, 0, 0};
            if (mtg < mtiles && (ks < 4 || qq == 0)) v = frags[((mtg * ntc + b) * 9 + q) * 64 + (c & 63)];
            stage_regs[i] = v;
        }
    };
    auto stage_store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 8; i++) lds[buf][tid + 256 * i] = stage_regs[i];
    };

    Q4Tile wt[WN_TILES], wnext[WN_TILES];  // weights of this super-block, and the next one in flight
    Q4Consts cs[WN_TILES];
    stage_load(0);
#pragma unroll
    for (int j = 0; j < WN_TILES; j++) wt[j] = q4_load(w + (rt[j] * ntc) * TB, lane);
    stage_store(0);
    __syncthreads();

    for (int64_t b = 0; b < ntc; b++) {
#pragma unroll
        for (int ks = 0; ks < 5; ks++) {  // fully unrolled: ks selects registers at compile time
            const int64_t s = b * 5 + ks;
            const int buf = (int)(s & 1);
            if (s + 1 < nstages) stage_load(s + 1);
            if (ks == 0) {
#pragma unroll
                for (int j = 0; j < WN_TILES; j++) cs[j] = q4_consts(wt[j].hd, g);
                const int64_t bn = b + 1 < ntc ? b + 1 : b;  // last super-block: harmless re-read
#pragma unroll
                for (int j = 0; j < WN_TILES; j++) wnext[j] = q4_load(w + (rt[j] * ntc + bn) * TB, lane);
            }
            const uint4v *abase = &lds[buf][0];
            if (ks < 4) {
#pragma unroll
                for (int qq = 0; qq < 2; qq++) {
                    half8v bop[WN_TILES];
#pragma unroll
                    for (int j = 0; j < WN_TILES; j++) {
                        // operand step q = 2*ks + qq: dword q of the lane; sub-block half h = q >> 2
                        const uint4v src = ks < 2 ? wt[j].qa : wt[j].qb;
                        const uint32_t wd = (ks & 1) ? (qq ? src.w : src.z) : (qq ? src.y : src.x);
                        const int h = ks >> 1;
                        bop[j] = q4_operand(wd, cs[j].s[h], cs[j].c1[h], cs[j].c2[h]);
                    }
#pragma unroll
                    for (int i = 0; i < WM_TILES; i++) {
                        const half8v a = __builtin_bit_cast(half8v, abase[(qq * 16 + wm * WM_TILES + i) * 64 + lane]);
#pragma unroll
                        for (int j = 0; j < WN_TILES; j++) acc[i][j] = mfma16x16x32(a, bop[j], acc[i][j]);
                    }
                }
            } else {
                // "- dmin * m" term against the group sums; then the prefetched weights of the next super-block take over
#pragma unroll
                for (int i = 0; i < WM_TILES; i++) {
                    const half8v a = __builtin_bit_cast(half8v, abase[(wm * WM_TILES + i) * 64 + lane]);
#pragma unroll
                    for (int j = 0; j < WN_TILES; j++) {
                        const half2v d2 = cs[j].dmn;
                        acc[i][j] = mfma16x16x32(a, half8v{d2.x, d2.x, d2.x, d2.x, d2.y, d2.y, d2.y, d2.y}, acc[i][j]);
                    }
                }
#pragma unroll
                for (int j = 0; j < WN_TILES; j++) wt[j] = wnext[j];
            }
            if (s + 1 < nstages) stage_store(buf ^ 1);
            __syncthreads();
        }
    }

    // lane (nn, G) of tile (i, j) holds y[row0 + 16 i + 4 G + r][col0 + 16 j + nn]
    const int nn = lane & 15;
#pragma unroll
    for (int j = 0; j < WN_TILES; j++) {
        const int64_t col = ((int64_t)nb * (BN / 16) + wn * WN_TILES + j) * 16 + nn;
        if (col >= n) continue;
        const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
        for (int i = 0; i < WM_TILES; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int64_t row = (int64_t)mb * BM + (wm * WM_TILES + i) * 16 + 4 * g + r;
                if (row < m) {
                    const float v = acc[i][j][r] + bv;
                    if (yt == TURQ_ACT_F32) turq_store_out<TURQ_ACT_F32>(y, row * ldy + col, v);
                    else if (yt == TURQ_ACT_BF16) turq_store_out<TURQ_ACT_BF16>(y, row * ldy + col, v);
                    else turq_store_out<TURQ_ACT_F16>(y, row * ldy + col, v);
                }
            }
    }
}

}  // namespace

// frags: activations prepared by turq_launch_act_prep for all m rows (16-row tiles, mpad = 16)
hipError_t turq_launch_gemm_mfma(int dtype, const void *w, int64_t n, int64_t k, const void *frags, int64_t m, void *y,
                                 int y_dtype, int64_t ldy, const float *bias, hipStream_t stream, hipEvent_t ev_start,
                                 hipEvent_t ev_stop) {
    if (n == 0 || m == 0) return hipSuccess;
    if (dtype != TURQ_Q4_K || m <= 16) return hipErrorInvalidValue;
    const int nbn = (int)((n + BN - 1) / BN), nbm = (int)((m + BM - 1) / BM);
    const dim3 grid((unsigned)(nbn * nbm)), block(256);
    if (ev_start) {
        hipExtLaunchKernelGGL(gemm_q4k_kernel, grid, block, 0, stream, ev_start, ev_stop, 0, (const uint8_t *)w, n, k,
                              (const uint4v *)frags, m, y, y_dtype, ldy, bias, nbn, nbm);
    } else {
        gemm_q4k_kernel<<<grid, block, 0, stream>>>((const uint8_t *)w, n, k, (const uint4v *)frags, m, y, y_dtype, ldy, bias,
                                                    nbn, nbm);
    }
    return hipGetLastError();
}

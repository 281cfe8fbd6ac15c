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
#include <hip/hip_ext.h>

#include "gemv_tileop.h"

namespace {

// ---- fused activation preparation (small m): the wave converts its own slice of x ----
// Raw activations of one tile for one lane: 4 consecutive columns of each of MP rows.
template <int XT, int MP> struct XRegs { float v[MP][4]; };

template <int XT, int MP>
__device__ inline XRegs<XT, MP> load_x(const void *__restrict__ x, int64_t ldx, int64_t m, int64_t k, int64_t b,
                                       int lane) {
    XRegs<XT, MP> xr;
    const int64_t col = b * 256 + 4 * lane;
#pragma unroll
    for (int rr = 0; rr < MP; rr++) {
        const bool ok = rr < m && col < k;  // k is a multiple of 32, so 4 columns are in or out together
        const int64_t off = ok ? rr * ldx + col : 0;
        if (XT == TURQ_ACT_F32) {
            const float4 t = *(const float4 *)((const float *)x + off);
            xr.v[rr][0] = t.x; xr.v[rr][1] = t.y; xr.v[rr][2] = t.z; xr.v[rr][3] = t.w;
        } else {
            const uint2 t = *(const uint2 *)((const uint16_t *)x + off);
            const uint32_t u[2] = {t.x, t.y};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t bits = (u[j >> 1] >> (16 * (j & 1))) & 0xFFFFu;
                xr.v[rr][j] = XT == TURQ_ACT_BF16 ? __uint_as_float(bits << 16) : h2f_bits(bits);
            }
        }
        if (!ok) { xr.v[rr][0] = 0.f; xr.v[rr][1] = 0.f; xr.v[rr][2] = 0.f; xr.v[rr][3] = 0.f; }
    }
    return xr;
}

// Write the wave's slice to its LDS region as f16 (+ group sums), then read the fragments back.
// Region layout: MP rows of 256 f16 (512 B each), then MP rows of 16 (hi, lo) sum pairs (64 B each).
template <int DT, int XT, int MP>
__device__ inline AFrags<DT, 1> stage_frags_lds(const XRegs<XT, MP> &xr, uint8_t *region, int lane) {
    constexpr bool KQ = DT != TURQ_Q8_0;
    const int g = lane >> 4, r = (lane & 15) & (MP - 1);
#pragma unroll
    for (int rr = 0; rr < MP; rr++) {
        const half2v h01 = {(_Float16)xr.v[rr][0], (_Float16)xr.v[rr][1]};
        const half2v h23 = {(_Float16)xr.v[rr][2], (_Float16)xr.v[rr][3]};
        *(uint2v *)(region + rr * 512 + 8 * lane) = uint2v{as_u32(h01), as_u32(h23)};
        if (KQ) {  // sum of the 16 f16-rounded values of a group = 4 lanes
            float s = ((float)h01.x + (float)h01.y) + ((float)h23.x + (float)h23.y);
            s += __shfl_xor(s, 1, 64);
            s += __shfl_xor(s, 2, 64);
            const _Float16 hi = (_Float16)s;
            const _Float16 lo = (_Float16)(s - (float)hi);
            if ((lane & 3) == 0) *(uint32_t *)(region + MP * 512 + rr * 64 + lane) = as_u32(half2v{hi, lo});
        }
    }
    // same-wave LDS traffic is processed in order; the fences keep the compiler from reordering
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    AFrags<DT, 1> f;
#pragma unroll
    for (int q = 0; q < 8; q++) {
        const int col = KQ ? 64 * g + 8 * q : 32 * q + 8 * g;
        f.a[0][q] = *(const half8v *)(region + r * 512 + 2 * col);
    }
    if constexpr (KQ) f.a[0][8] = *(const half8v *)(region + MP * 512 + r * 64 + 16 * g);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    return f;
}

// ---- the kernel ----
// FUSED: activations come raw from x (m <= MP <= 4) and are prepared per wave through LDS;
// otherwise they come from the fragment buffer written by the activation preparation kernel.
// P = tiles whose loads a wave keeps in flight together.
// MAXT = largest workgroup the instantiation is launched with (bounds the registers per lane).
// the work of one workgroup: row tile rt of one weight
template <int DT, int MT, int XT, bool FUSED, int MP, int P>
__device__ __forceinline__ void gemv_body(const uint8_t *__restrict__ w, int64_t n, int64_t k, const void *__restrict__ xin,
                                          int64_t ldx, int64_t m, int mpad, void *__restrict__ y, int yt, int64_t ldy,
                                          const float *__restrict__ bias, int64_t rt) {
    extern __shared__ uint8_t smem[];
    constexpr int NQ = DT == TURQ_Q8_0 ? TURQ_NQ_Q8_0 : TURQ_NQ_KQUANT;
    constexpr int TB = TiledFmt<DT>::kTileBytes;
    constexpr int REGION = FUSED ? MP * (512 + 64) : 0;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // wave-uniform: scalar address math
    const int nwaves = blockDim.x >> 6;
    const int64_t ntc = turq_tile_cols(k);
    const int64_t tile_chunks = (int64_t)NQ * 4 * mpad;  // 16-byte chunks of one (mt, b) fragment set
    const int64_t mt_stride = ntc * tile_chunks;
    float4v *red = (float4v *)(smem + (size_t)nwaves * REGION);
    uint8_t *region = smem + (size_t)wave * REGION;
    float4v acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[mt] = float4v{0.f, 0.f, 0.f, 0.f};
    const uint8_t *wrow = w + rt * ntc * TB;
    GOff go = lane_offsets(lane, mpad);
    for (int64_t b0 = wave; b0 < ntc; b0 += (int64_t)nwaves * P) {
        WRegs<DT> wr[P];
        XRegs<XT, MP> xr[P];
        go.touch();
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t b = b0 + (int64_t)p * nwaves;
            const int64_t bc = b < ntc ? b : b0;  // keep the address in bounds; the result is not used
            wr[p] = load_tile<DT>(wrow + bc * TB, go);
            if constexpr (FUSED) xr[p] = load_x<XT, MP>(xin, ldx, m, k, bc, lane);
        }
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t b = b0 + (int64_t)p * nwaves;
            if (b < ntc) {  // uniform per wave
                if constexpr (FUSED) {
                    const AFrags<DT, 1> f = stage_frags_lds<DT, XT, MP>(xr[p], region, lane);
                    TileOp<DT, 1, 4>::run(wr[p], f, lane, acc);
                } else {
                    const AFrags<DT, MT> f =
                        load_frags_global<DT, MT>((const half8v *)xin + b * tile_chunks, mt_stride, mpad, go);
                    TileOp<DT, MT, 4>::run(wr[p], f, lane, acc);
                }
            }
        }
    }

    const int nn = lane & 15, g = lane >> 4;
    const int64_t col = rt * 16 + nn;
    if constexpr (FUSED) {
        // only rows 0..MP-1 exist: lanes 0..15 hold them in components 0..MP-1.
        // partial sums go to LDS as ps[row][n][wave]; wave 0 adds them up four waves per lane.
        float *ps = (float *)red;
        if (nwaves > 1) {
            if (lane < 16)
#pragma unroll
                for (int i = 0; i < MP; i++) ps[(i * 16 + nn) * 16 + wave] = acc[0][i];
            __syncthreads();
            if (wave != 0) return;
            const int n4 = lane >> 2, w4 = (lane & 3) * 4;  // lane sums waves w4..w4+3 of column n4
#pragma unroll
            for (int i = 0; i < MP; i++) {
                float s = 0.f;
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (w4 + j < nwaves) s += ps[(i * 16 + n4) * 16 + w4 + j];
                s += __shfl_xor(s, 1, 64);
                s += __shfl_xor(s, 2, 64);
                acc[0][i] = s;  // every lane of the quad holds column n4's total
            }
            const int64_t c4 = rt * 16 + n4;
            if ((lane & 3) == 0 && c4 < n) {
                const float bv = bias ? bias[c4] : 0.0f;
#pragma unroll
                for (int i = 0; i < MP; i++)
                    if (i < m) turq_store_any(y, yt, (int64_t)i * ldy + c4, acc[0][i] + bv);
            }
            return;
        }
        if (lane < 16 && col < n) {
            const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
            for (int i = 0; i < MP; i++)
                if (i < m) turq_store_any(y, yt, (int64_t)i * ldy + col, acc[0][i] + bv);
        }
        return;
    }
    if (nwaves > 1) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) red[(wave * MT + mt) * 64 + lane] = acc[mt];
        __syncthreads();
        if (wave != 0) return;
        float4v extra[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) extra[mt] = float4v{0.f, 0.f, 0.f, 0.f};
        int wv = 1;
        for (; wv + 1 < nwaves; wv += 2)  // two independent chains so the LDS reads overlap
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                acc[mt] += red[(wv * MT + mt) * 64 + lane];
                extra[mt] += red[((wv + 1) * MT + mt) * 64 + lane];
            }
        if (wv < nwaves)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[mt] += red[(wv * MT + mt) * 64 + lane];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[mt] += extra[mt];
    }
    // lane (nn, g) holds y[16 mt + 4 g + i][16 rt + nn], i = 0..3
    if (col >= n) return;
    const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
    for (int mt = 0; mt < MT; mt++) turq_store_col4(y, yt, 16 * mt + 4 * g, m, ldy, col, acc[mt] + float4v{bv, bv, bv, bv});
}

template <int DT, int MT, int XT, bool FUSED, int MP, int P, int MAXT>
__global__ void __launch_bounds__(MAXT) gemv_mfma_kernel(const uint8_t *__restrict__ w, int64_t n, int64_t k,
                                                          const void *__restrict__ xin, int64_t ldx, int64_t m,
                                                          int mpad, void *__restrict__ y, int yt, int64_t ldy,
                                                          const float *__restrict__ bias) {
    gemv_body<DT, MT, XT, FUSED, MP, P>(w, n, k, xin, ldx, m, mpad, y, yt, ldy, bias, (int64_t)blockIdx.x);
}

template <int DT, int XT, int MP, int P, int MAXT>
__global__ void __launch_bounds__(MAXT) gemv_multi_kernel(MultiArgs a, int64_t k, const void *__restrict__ x, int64_t ldx,
                                                           int64_t m, int yt) {
    // wave-uniform selection without indexing the argument block dynamically
    const int blk = (int)blockIdx.x;
    const uint8_t *w = a.w[0];
    void *y = a.y[0];
    const float *bias = a.bias[0];
    int64_t n = a.n[0], ldy = a.ldy[0];
    int first = 0;
#pragma unroll
    for (int i = 1; i < kMaxMulti; i++)
        if (i < a.count && blk >= a.first[i]) {
            w = a.w[i], y = a.y[i], bias = a.bias[i], n = a.n[i], ldy = a.ldy[i], first = a.first[i];
        }
    gemv_body<DT, 1, XT, true, MP, P>(w, n, k, x, ldx, m, MP, y, yt, ldy, bias, (int64_t)(blk - first));
}

// Prepared fragments, R row tiles per workgroup: a wave applies the fragments of a column tile, once fetched, to R weight
// tiles, which divides the fragment traffic through L2 (9 - 18 KiB per column tile against 2 - 4 KiB per weight tile) by R.
// GU (R = 2): the two row tiles are row tile rtg of a gate weight (w) and of an up weight (w2) of one shape, and what is stored
// is silu(gate) * up (src/models/qwen3.rs:161-167).
template <int DT, int MT, int P, int R, bool GU = false>
__device__ __forceinline__ void gemv_frag_body(const uint8_t *__restrict__ w, int64_t n, int64_t k, const void *__restrict__ frags,
                                               int64_t m, int mpad, void *__restrict__ y, int yt, int64_t ldy,
                                               const float *__restrict__ bias, int64_t rtg, const uint8_t *__restrict__ w2 = nullptr,
                                               const float *__restrict__ bias2 = nullptr) {
    static_assert(!GU || R == 2, "gate and up take the places of two row tiles");
    extern __shared__ uint8_t smem[];
    constexpr int NQ = DT == TURQ_Q8_0 ? TURQ_NQ_Q8_0 : TURQ_NQ_KQUANT;
    constexpr int TB = TiledFmt<DT>::kTileBytes;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nwaves = blockDim.x >> 6;
    const int64_t ntc = turq_tile_cols(k), nrt = turq_tile_rows(n);
    const int64_t rt0 = GU ? rtg : rtg * R;
    const int64_t tile_chunks = (int64_t)NQ * 4 * mpad;
    const int64_t mt_stride = ntc * tile_chunks;
    float4v *red = (float4v *)smem;
    float4v acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[r][mt] = float4v{0.f, 0.f, 0.f, 0.f};
    const uint8_t *wrow[R];  // row tiles past the end re-read the last one; their results are not stored
#pragma unroll
    for (int r = 0; r < R; r++) {
        if constexpr (GU) wrow[r] = (r == 0 ? w : w2) + rt0 * ntc * TB;
        else wrow[r] = w + (rt0 + r < nrt ? rt0 + r : nrt - 1) * ntc * TB;
    }
    GOff go = lane_offsets(lane, mpad);
    for (int64_t b0 = wave; b0 < ntc; b0 += (int64_t)nwaves * P) {
        WRegs<DT> wr[P][R];
        go.touch();
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t b = b0 + (int64_t)p * nwaves;
            const int64_t bc = b < ntc ? b : b0;
#pragma unroll
            for (int r = 0; r < R; r++) wr[p][r] = load_tile<DT>(wrow[r] + bc * TB, go);
        }
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t b = b0 + (int64_t)p * nwaves;
            if (b < ntc) {  // uniform per wave
                const AFrags<DT, MT> f = load_frags_global<DT, MT>((const half8v *)frags + b * tile_chunks, mt_stride, mpad, go);
#pragma unroll
                for (int r = 0; r < R; r++) TileOp<DT, MT, 4>::run(wr[p][r], f, lane, acc[r]);
            }
        }
    }
    if (nwaves > 1) {
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) red[((wave * R + r) * MT + mt) * 64 + lane] = acc[r][mt];
        __syncthreads();
        if (wave != 0) return;
        for (int wv = 1; wv < nwaves; wv++)
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int mt = 0; mt < MT; mt++) acc[r][mt] += red[((wv * R + r) * MT + mt) * 64 + lane];
    }
    // lane (nn, g) holds y[16 mt + 4 g + i][16 (rt0 + r) + nn], i = 0..3
    const int nn = lane & 15, g = lane >> 4;
    if constexpr (GU) {
        const int64_t col = rt0 * 16 + nn;
        if (col >= n) return;
        const float bg = bias ? bias[col] : 0.0f, bu = bias2 ? bias2[col] : 0.0f;
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int64_t row = 16 * mt + 4 * g + i;
                const float gate = acc[0][mt][i] + bg, up = acc[1][mt][i] + bu;
                if (row < m) turq_store_any(y, yt, row * ldy + col, gate / (1.0f + expf(-gate)) * up);
            }
        return;
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int64_t col = (rt0 + r) * 16 + nn;
        if (rt0 + r >= nrt || col >= n) continue;
        const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
        for (int mt = 0; mt < MT; mt++) turq_store_col4(y, yt, 16 * mt + 4 * g, m, ldy, col, acc[r][mt] + float4v{bv, bv, bv, bv});
    }
}

// the same with activation fragments prepared once by act_prep_kernel and shared by all the weights
template <int DT, int MT, int P, int MAXT, int R>
__global__ void __launch_bounds__(MAXT) gemv_multi_frag_kernel(MultiArgs a, int64_t k, const void *__restrict__ frags, int64_t m,
                                                                int mpad, int yt) {
    const int blk = (int)blockIdx.x;
    const uint8_t *w = a.w[0];
    void *y = a.y[0];
    const float *bias = a.bias[0];
    int64_t n = a.n[0], ldy = a.ldy[0];
    int first = 0;
#pragma unroll
    for (int i = 1; i < kMaxMulti; i++)
        if (i < a.count && blk >= a.first[i]) {
            w = a.w[i], y = a.y[i], bias = a.bias[i], n = a.n[i], ldy = a.ldy[i], first = a.first[i];
        }
    if constexpr (R == 1) gemv_body<DT, MT, TURQ_ACT_F16, false, 1, P>(w, n, k, frags, 0, m, mpad, y, yt, ldy, bias, (int64_t)(blk - first));
    else gemv_frag_body<DT, MT, P, R>(w, n, k, frags, m, mpad, y, yt, ldy, bias, (int64_t)(blk - first));
}

// gate_proj and up_proj of one MLP against prepared fragments, SiLU and the product applied before the store: workgroup b takes
// row tile b of both weights
template <int DT, int MT, int P, int MAXT>
__global__ void __launch_bounds__(MAXT) gemv_gateup_frag_kernel(const uint8_t *__restrict__ wg, const uint8_t *__restrict__ wu,
                                                                 const float *__restrict__ bg, const float *__restrict__ bu, int64_t n,
                                                                 int64_t k, const void *__restrict__ frags, int64_t m, int mpad,
                                                                 void *__restrict__ y, int64_t ldy, int yt) {
    gemv_frag_body<DT, MT, P, 2, true>(wg, n, k, frags, m, mpad, y, yt, ldy, bg, (int64_t)blockIdx.x, wu, bu);
}

// prepared fragments, weights of two formats with the same fragment order (Q4_K weights followed by Q6_K ones: q, k and v of a
// Q4_K_M file): the workgroup's weight decides which body runs.  One row tile per workgroup.
template <int DTA, int DTB, int MT, int P, int MAXT>
__global__ void __launch_bounds__(MAXT) gemv_multi_frag_mixed_kernel(MultiArgs a, int64_t k, const void *__restrict__ frags, int64_t m,
                                                                      int mpad, int yt) {
    const int blk = (int)blockIdx.x;
    const uint8_t *w = a.w[0];
    void *y = a.y[0];
    const float *bias = a.bias[0];
    int64_t n = a.n[0], ldy = a.ldy[0];
    int first = 0, index = 0;
#pragma unroll
    for (int i = 1; i < kMaxMulti; i++)
        if (i < a.count && blk >= a.first[i]) {
            w = a.w[i], y = a.y[i], bias = a.bias[i], n = a.n[i], ldy = a.ldy[i], first = a.first[i], index = i;
        }
    if (index < a.second) gemv_body<DTA, MT, TURQ_ACT_F16, false, 1, P>(w, n, k, frags, 0, m, mpad, y, yt, ldy, bias, (int64_t)(blk - first));
    else gemv_body<DTB, MT, TURQ_ACT_F16, false, 1, P>(w, n, k, frags, 0, m, mpad, y, yt, ldy, bias, (int64_t)(blk - first));
}

struct GemvArgs {
    const void *w; int64_t n, k; const void *xin; int64_t ldx, m; void *y; int yt; int64_t ldy; const float *bias;
    int nwaves; hipStream_t s;
    hipEvent_t ev_start, ev_stop;  // kernel timing: the dispatch's own begin / end timestamps (or null)
};

template <int DT, int MT, int XT, bool FUSED, int MP, int P, int MAXT>
hipError_t launch_final(const GemvArgs &a) {
    const int mpad = FUSED ? MP : (MT > 1 ? 16 : turq_mpad(a.m));
    const unsigned grid = (unsigned)turq_tile_rows(a.n);
    const size_t region = FUSED ? (size_t)MP * (512 + 64) : 0;
    // reduction buffer: full 16x16 tiles per wave, or (fused) MP rows x 16 columns x 16 wave slots
    const size_t red = FUSED ? (size_t)MP * 16 * 16 * sizeof(float) : (size_t)a.nwaves * MT * 64 * sizeof(float4v);
    const size_t lds = (size_t)a.nwaves * region + (a.nwaves > 1 ? red : 0);
    if (a.ev_start) {
        hipExtLaunchKernelGGL((gemv_mfma_kernel<DT, MT, XT, FUSED, MP, P, MAXT>), dim3(grid), dim3((unsigned)(64 * a.nwaves)),
                              (unsigned)lds, a.s, a.ev_start, a.ev_stop, 0, (const uint8_t *)a.w, a.n, a.k, a.xin, a.ldx, a.m,
                              mpad, a.y, a.yt, a.ldy, a.bias);
        return hipGetLastError();
    }
    gemv_mfma_kernel<DT, MT, XT, FUSED, MP, P, MAXT><<<grid, dim3((unsigned)(64 * a.nwaves)), lds, a.s>>>(
        (const uint8_t *)a.w, a.n, a.k, a.xin, a.ldx, a.m, mpad, a.y, a.yt, a.ldy, a.bias);
    return hipGetLastError();
}

// Prefetch depth by workgroup size: small groups (<= 4 waves) may use up to 512 registers per lane
// and keep four tiles in flight; 16-wave groups are held to 128 registers and keep at most two.
template <int DT, int MT, int XT, bool FUSED, int MP>
hipError_t launch_p(const GemvArgs &a) {
    const int64_t per_wave = (turq_tile_cols(a.k) + a.nwaves - 1) / a.nwaves;
    if (a.nwaves <= 4) {
        if (per_wave <= 1) return launch_final<DT, MT, XT, FUSED, MP, 1, 256>(a);
        if (per_wave <= 2) return launch_final<DT, MT, XT, FUSED, MP, 2, 256>(a);
        return launch_final<DT, MT, XT, FUSED, MP, 4, 256>(a);
    }
    if (per_wave <= 1 || MT > 1) return launch_final<DT, MT, XT, FUSED, MP, 1, 1024>(a);
    return launch_final<DT, MT, XT, FUSED, MP, 2, 1024>(a);
}

template <int DT, int XT>
hipError_t launch_fused(const GemvArgs &a) {
    if (a.m <= 1) return launch_p<DT, 1, XT, true, 1>(a);
    if (a.m <= 2) return launch_p<DT, 1, XT, true, 2>(a);
    return launch_p<DT, 1, XT, true, 4>(a);
}

template <int DT>
hipError_t launch_x(int xt, bool fused, const GemvArgs &a) {
    if (!fused) {
        if (a.m <= 16) return launch_p<DT, 1, TURQ_ACT_F16, false, 1>(a);
        return launch_p<DT, 2, TURQ_ACT_F16, false, 1>(a);
    }
    switch (xt) {
    case TURQ_ACT_F32: return launch_fused<DT, TURQ_ACT_F32>(a);
    case TURQ_ACT_BF16: return launch_fused<DT, TURQ_ACT_BF16>(a);
    case TURQ_ACT_F16: return launch_fused<DT, TURQ_ACT_F16>(a);
    default: return hipErrorInvalidValue;
    }
}

template <int DT, int XT, int MP, int P, int MAXT>
hipError_t launch_multi_final(const MultiArgs &ma, int total_blocks, int64_t k, const void *x, int64_t ldx, int64_t m, int yt,
                              int nwaves, hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    const size_t region = (size_t)MP * (512 + 64);
    const size_t red = (size_t)MP * 16 * 16 * sizeof(float);
    const size_t lds = (size_t)nwaves * region + (nwaves > 1 ? red : 0);
    if (ev0) {
        hipExtLaunchKernelGGL((gemv_multi_kernel<DT, XT, MP, P, MAXT>), dim3((unsigned)total_blocks), dim3((unsigned)(64 * nwaves)),
                              (unsigned)lds, s, ev0, ev1, 0, ma, k, x, ldx, m, yt);
        return hipGetLastError();
    }
    gemv_multi_kernel<DT, XT, MP, P, MAXT><<<(unsigned)total_blocks, dim3((unsigned)(64 * nwaves)), lds, s>>>(ma, k, x, ldx, m, yt);
    return hipGetLastError();
}

template <int DT, int XT, int MP>
hipError_t launch_multi_p(const MultiArgs &ma, int total_blocks, int64_t k, const void *x, int64_t ldx, int64_t m, int yt,
                          int nwaves, hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    const int64_t per_wave = (turq_tile_cols(k) + nwaves - 1) / nwaves;
    if (nwaves <= 4) {
        if (per_wave <= 1) return launch_multi_final<DT, XT, MP, 1, 256>(ma, total_blocks, k, x, ldx, m, yt, nwaves, s, ev0, ev1);
        if (per_wave <= 2) return launch_multi_final<DT, XT, MP, 2, 256>(ma, total_blocks, k, x, ldx, m, yt, nwaves, s, ev0, ev1);
        return launch_multi_final<DT, XT, MP, 4, 256>(ma, total_blocks, k, x, ldx, m, yt, nwaves, s, ev0, ev1);
    }
    if (per_wave <= 1) return launch_multi_final<DT, XT, MP, 1, 1024>(ma, total_blocks, k, x, ldx, m, yt, nwaves, s, ev0, ev1);
    return launch_multi_final<DT, XT, MP, 2, 1024>(ma, total_blocks, k, x, ldx, m, yt, nwaves, s, ev0, ev1);
}

template <int DT, int XT>
hipError_t launch_multi_m(const MultiArgs &ma, int total_blocks, int64_t k, const void *x, int64_t ldx, int64_t m, int yt,
                          int nwaves, hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    if (m <= 1) return launch_multi_p<DT, XT, 1>(ma, total_blocks, k, x, ldx, m, yt, nwaves, s, ev0, ev1);
    if (m <= 2) return launch_multi_p<DT, XT, 2>(ma, total_blocks, k, x, ldx, m, yt, nwaves, s, ev0, ev1);
    return launch_multi_p<DT, XT, 4>(ma, total_blocks, k, x, ldx, m, yt, nwaves, s, ev0, ev1);
}

template <int DT, int MT, int P, int MAXT, int R>
hipError_t launch_multi_frag_final(const MultiArgs &ma, int total_blocks, int64_t k, const void *frags, int64_t m, int yt, int nwaves,
                                   hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    const int mpad = MT > 1 ? 16 : turq_mpad(m);
    const size_t lds = nwaves > 1 ? (size_t)nwaves * R * MT * 64 * sizeof(float4v) : 0;
    if (ev0) {
        hipExtLaunchKernelGGL((gemv_multi_frag_kernel<DT, MT, P, MAXT, R>), dim3((unsigned)total_blocks), dim3((unsigned)(64 * nwaves)),
                              (unsigned)lds, s, ev0, ev1, 0, ma, k, frags, m, mpad, yt);
        return hipGetLastError();
    }
    gemv_multi_frag_kernel<DT, MT, P, MAXT, R><<<(unsigned)total_blocks, dim3((unsigned)(64 * nwaves)), lds, s>>>(ma, k, frags, m, mpad, yt);
    return hipGetLastError();
}

template <int DT, int MT>
hipError_t launch_multi_frag_p(const MultiArgs &ma, int total_blocks, int64_t k, const void *frags, int64_t m, int yt, int nwaves,
                               int rtiles, hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    const int64_t per_wave = (turq_tile_cols(k) + nwaves - 1) / nwaves;
    if (rtiles == 2) {  // two row tiles per workgroup, at most four waves: four weight tiles in flight per wave where there are that many
        if (per_wave <= 1) return launch_multi_frag_final<DT, MT, 1, 256, 2>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
        return launch_multi_frag_final<DT, MT, 2, 256, 2>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
    }
    if (nwaves <= 4) {
        if (per_wave <= 1) return launch_multi_frag_final<DT, MT, 1, 256, 1>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
        if (per_wave <= 2) return launch_multi_frag_final<DT, MT, 2, 256, 1>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
        return launch_multi_frag_final<DT, MT, 4, 256, 1>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
    }
    if (per_wave <= 1 || MT > 1) return launch_multi_frag_final<DT, MT, 1, 1024, 1>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
    return launch_multi_frag_final<DT, MT, 2, 1024, 1>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
}

template <int DT>
hipError_t launch_multi_frag(const MultiArgs &ma, int total_blocks, int64_t k, const void *frags, int64_t m, int yt, int nwaves,
                             int rtiles, hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    if (m <= 16) return launch_multi_frag_p<DT, 1>(ma, total_blocks, k, frags, m, yt, nwaves, rtiles, s, ev0, ev1);
    return launch_multi_frag_p<DT, 2>(ma, total_blocks, k, frags, m, yt, nwaves, rtiles, s, ev0, ev1);
}

template <int DT>
hipError_t launch_multi_x(int xt, const MultiArgs &ma, int total_blocks, int64_t k, const void *x, int64_t ldx, int64_t m,
                          int yt, int nwaves, hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    switch (xt) {
    case TURQ_ACT_F32: return launch_multi_m<DT, TURQ_ACT_F32>(ma, total_blocks, k, x, ldx, m, yt, nwaves, s, ev0, ev1);
    case TURQ_ACT_BF16: return launch_multi_m<DT, TURQ_ACT_BF16>(ma, total_blocks, k, x, ldx, m, yt, nwaves, s, ev0, ev1);
    case TURQ_ACT_F16: return launch_multi_m<DT, TURQ_ACT_F16>(ma, total_blocks, k, x, ldx, m, yt, nwaves, s, ev0, ev1);
    default: return hipErrorInvalidValue;
    }
}

template <int DTA, int DTB, int MT, int P, int MAXT>
hipError_t launch_multi_frag_mixed_final(const MultiArgs &ma, int total_blocks, int64_t k, const void *frags, int64_t m, int yt,
                                         int nwaves, hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    const int mpad = MT > 1 ? 16 : turq_mpad(m);
    const size_t lds = nwaves > 1 ? (size_t)nwaves * MT * 64 * sizeof(float4v) : 0;
    if (ev0) {
        hipExtLaunchKernelGGL((gemv_multi_frag_mixed_kernel<DTA, DTB, MT, P, MAXT>), dim3((unsigned)total_blocks),
                              dim3((unsigned)(64 * nwaves)), (unsigned)lds, s, ev0, ev1, 0, ma, k, frags, m, mpad, yt);
        return hipGetLastError();
    }
    gemv_multi_frag_mixed_kernel<DTA, DTB, MT, P, MAXT><<<(unsigned)total_blocks, dim3((unsigned)(64 * nwaves)), lds, s>>>(ma, k, frags, m,
                                                                                                                        mpad, yt);
    return hipGetLastError();
}

// the launch shapes of launch_multi_frag_p with one row tile per workgroup
template <int DTA, int DTB, int MT>
hipError_t launch_multi_frag_mixed_p(const MultiArgs &ma, int total_blocks, int64_t k, const void *frags, int64_t m, int yt, int nwaves,
                                     hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    const int64_t per_wave = (turq_tile_cols(k) + nwaves - 1) / nwaves;
    if (nwaves <= 4) {
        if (per_wave <= 1) return launch_multi_frag_mixed_final<DTA, DTB, MT, 1, 256>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
        if (per_wave <= 2) return launch_multi_frag_mixed_final<DTA, DTB, MT, 2, 256>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
        return launch_multi_frag_mixed_final<DTA, DTB, MT, 4, 256>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
    }
    if (per_wave <= 1 || MT > 1) return launch_multi_frag_mixed_final<DTA, DTB, MT, 1, 1024>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
    return launch_multi_frag_mixed_final<DTA, DTB, MT, 2, 1024>(ma, total_blocks, k, frags, m, yt, nwaves, s, ev0, ev1);
}

}  // namespace

// count (2..4) weights of one format and one k.  fused: `x` are the raw activations (m <= TURQ_GEMV_FUSED_MAX_M, rows 16-byte
// aligned); otherwise `x` is the fragment buffer prepared for this format (m <= TURQ_GEMV_MAX_M; x_dtype and ldx unused).
hipError_t turq_launch_gemv_multi(int dtype, int count, const void *const *w, const int64_t *n, int64_t k, const void *x,
                                  int x_dtype, int64_t ldx, int64_t m, bool fused, void *const *y, int y_dtype, const int64_t *ldy,
                                  const float *const *bias, int nwaves, int row_tiles, hipStream_t stream, hipEvent_t ev_start,
                                  hipEvent_t ev_stop) {
    if (count < 1 || count > kMaxMulti || m < 1 || m > (fused ? TURQ_GEMV_FUSED_MAX_M : TURQ_GEMV_MAX_M) || nwaves < 1 || nwaves > 16)
        return hipErrorInvalidValue;
    if (!turq_yt_ok(y_dtype, true)) return hipErrorInvalidValue;
    if (row_tiles != 1 && !(row_tiles == 2 && !fused && nwaves <= 4)) return hipErrorInvalidValue;
    MultiArgs ma{};
    int64_t blocks = 0;
    for (int i = 0; i < count; i++) {
        ma.w[i] = (const uint8_t *)w[i];
        ma.y[i] = y[i];
        ma.bias[i] = bias ? bias[i] : nullptr;
        ma.n[i] = n[i];
        ma.ldy[i] = ldy[i];
        ma.first[i] = (int)blocks;
        blocks += (turq_tile_rows(n[i]) + row_tiles - 1) / row_tiles;
    }
    ma.count = count;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFF) return hipErrorInvalidValue;
    if (!fused) {
        switch (dtype) {
        case TURQ_Q4_K: return launch_multi_frag<TURQ_Q4_K>(ma, (int)blocks, k, x, m, y_dtype, nwaves, row_tiles, stream, ev_start, ev_stop);
        case TURQ_Q5_K: return launch_multi_frag<TURQ_Q5_K>(ma, (int)blocks, k, x, m, y_dtype, nwaves, row_tiles, stream, ev_start, ev_stop);
        case TURQ_Q6_K: return launch_multi_frag<TURQ_Q6_K>(ma, (int)blocks, k, x, m, y_dtype, nwaves, row_tiles, stream, ev_start, ev_stop);
        case TURQ_Q8_0: return launch_multi_frag<TURQ_Q8_0>(ma, (int)blocks, k, x, m, y_dtype, nwaves, row_tiles, stream, ev_start, ev_stop);
        default: return hipErrorInvalidValue;
        }
    }
    switch (dtype) {
    case TURQ_Q4_K: return launch_multi_x<TURQ_Q4_K>(x_dtype, ma, (int)blocks, k, x, ldx, m, y_dtype, nwaves, stream, ev_start, ev_stop);
    case TURQ_Q5_K: return launch_multi_x<TURQ_Q5_K>(x_dtype, ma, (int)blocks, k, x, ldx, m, y_dtype, nwaves, stream, ev_start, ev_stop);
    case TURQ_Q6_K: return launch_multi_x<TURQ_Q6_K>(x_dtype, ma, (int)blocks, k, x, ldx, m, y_dtype, nwaves, stream, ev_start, ev_stop);
    case TURQ_Q8_0: return launch_multi_x<TURQ_Q8_0>(x_dtype, ma, (int)blocks, k, x, ldx, m, y_dtype, nwaves, stream, ev_start, ev_stop);
    default: return hipErrorInvalidValue;
    }
}

// the pairs of a Q4_K_M and of a Q5_K_M file
bool turq_gemv_multi_mixed_supports(int dtype_a, int dtype_b) {
    return (dtype_a == TURQ_Q4_K || dtype_a == TURQ_Q5_K) && dtype_b == TURQ_Q6_K;
}

// count (2..4) weights of one k against prepared fragments (K-quant order) of m <= TURQ_GEMV_MAX_M rows: the first `second` of
// format dtype_a, the others of dtype_b (a pair turq_gemv_multi_mixed_supports accepts); one row tile per workgroup.
hipError_t turq_launch_gemv_multi_mixed(int dtype_a, int dtype_b, int count, int second, const void *const *w, const int64_t *n,
                                        int64_t k, const void *frags, int64_t m, void *const *y, int y_dtype, const int64_t *ldy,
                                        const float *const *bias, int nwaves, hipStream_t stream, hipEvent_t ev_start,
                                        hipEvent_t ev_stop) {
    if (!turq_gemv_multi_mixed_supports(dtype_a, dtype_b) || count < 2 || count > kMaxMulti || second < 1 || second >= count || m < 1 ||
        m > TURQ_GEMV_MAX_M || nwaves < 1 || nwaves > 16)
        return hipErrorInvalidValue;
    if (!turq_yt_ok(y_dtype, true)) return hipErrorInvalidValue;
    MultiArgs ma{};
    int64_t blocks = 0;
    for (int i = 0; i < count; i++) {
        ma.w[i] = (const uint8_t *)w[i];
        ma.y[i] = y[i];
        ma.bias[i] = bias ? bias[i] : nullptr;
        ma.n[i] = n[i];
        ma.ldy[i] = ldy[i];
        ma.first[i] = (int)blocks;
        blocks += turq_tile_rows(n[i]);
    }
    ma.count = count;
    ma.second = second;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFF) return hipErrorInvalidValue;
    if (dtype_a == TURQ_Q5_K) {
        if (m <= 16)
            return launch_multi_frag_mixed_p<TURQ_Q5_K, TURQ_Q6_K, 1>(ma, (int)blocks, k, frags, m, y_dtype, nwaves, stream, ev_start, ev_stop);
        return launch_multi_frag_mixed_p<TURQ_Q5_K, TURQ_Q6_K, 2>(ma, (int)blocks, k, frags, m, y_dtype, nwaves, stream, ev_start, ev_stop);
    }
    if (m <= 16)
        return launch_multi_frag_mixed_p<TURQ_Q4_K, TURQ_Q6_K, 1>(ma, (int)blocks, k, frags, m, y_dtype, nwaves, stream, ev_start, ev_stop);
    return launch_multi_frag_mixed_p<TURQ_Q4_K, TURQ_Q6_K, 2>(ma, (int)blocks, k, frags, m, y_dtype, nwaves, stream, ev_start, ev_stop);
}

// `xin` is the prepared fragment buffer (fused == false; ldx and x_dtype unused) or the raw
// activations (fused == true, m <= TURQ_GEMV_FUSED_MAX_M).
hipError_t turq_launch_gemv_mfma(int dtype, const void *w, int64_t n, int64_t k, const void *xin, int x_dtype,
                                 int64_t ldx, int64_t m, bool fused, void *y, int y_dtype, int64_t ldy,
                                 const float *bias, int nwaves, hipStream_t stream, hipEvent_t ev_start,
                                 hipEvent_t ev_stop) {
    if (n == 0 || m == 0) return hipSuccess;
    if (m > TURQ_GEMV_MAX_M || nwaves < 1 || nwaves > 16) return hipErrorInvalidValue;
    if (fused && m > TURQ_GEMV_FUSED_MAX_M) return hipErrorInvalidValue;
    if (!turq_yt_ok(y_dtype, true)) return hipErrorInvalidValue;
    const GemvArgs a{w, n, k, xin, ldx, m, y, y_dtype, ldy, bias, nwaves, stream, ev_start, ev_stop};
    switch (dtype) {
    case TURQ_Q4_K: return launch_x<TURQ_Q4_K>(x_dtype, fused, a);
    case TURQ_Q5_K: return launch_x<TURQ_Q5_K>(x_dtype, fused, a);
    case TURQ_Q6_K: return launch_x<TURQ_Q6_K>(x_dtype, fused, a);
    case TURQ_Q8_0: return launch_x<TURQ_Q8_0>(x_dtype, fused, a);
    default: return hipErrorInvalidValue;
    }
}

namespace {
template <int DT, int MT, int P>
hipError_t launch_gateup_frag_final(const void *wg, const void *wu, const float *bg, const float *bu, int64_t n, int64_t k,
                                    const void *frags, int64_t m, void *y, int64_t ldy, int yt, int nwaves, hipStream_t s,
                                    hipEvent_t ev0, hipEvent_t ev1) {
    const int mpad = MT > 1 ? 16 : turq_mpad(m);
    const size_t lds = nwaves > 1 ? (size_t)nwaves * 2 * MT * 64 * sizeof(float4v) : 0;
    const dim3 grid((unsigned)turq_tile_rows(n)), block((unsigned)(64 * nwaves));
    if (ev0) {
        hipExtLaunchKernelGGL((gemv_gateup_frag_kernel<DT, MT, P, 256>), grid, block, (unsigned)lds, s, ev0, ev1, 0, (const uint8_t *)wg,
                              (const uint8_t *)wu, bg, bu, n, k, frags, m, mpad, y, ldy, yt);
        return hipGetLastError();
    }
    gemv_gateup_frag_kernel<DT, MT, P, 256><<<grid, block, lds, s>>>((const uint8_t *)wg, (const uint8_t *)wu, bg, bu, n, k, frags, m, mpad,
                                                                      y, ldy, yt);
    return hipGetLastError();
}

template <int DT>
hipError_t launch_gateup_frag(const void *wg, const void *wu, const float *bg, const float *bu, int64_t n, int64_t k, const void *frags,
                              int64_t m, void *y, int64_t ldy, int yt, int nwaves, hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    const int64_t per_wave = (turq_tile_cols(k) + nwaves - 1) / nwaves;
    if (m <= 16) {
        if (per_wave <= 1) return launch_gateup_frag_final<DT, 1, 1>(wg, wu, bg, bu, n, k, frags, m, y, ldy, yt, nwaves, s, ev0, ev1);
        return launch_gateup_frag_final<DT, 1, 2>(wg, wu, bg, bu, n, k, frags, m, y, ldy, yt, nwaves, s, ev0, ev1);
    }
    if (per_wave <= 1) return launch_gateup_frag_final<DT, 2, 1>(wg, wu, bg, bu, n, k, frags, m, y, ldy, yt, nwaves, s, ev0, ev1);
    return launch_gateup_frag_final<DT, 2, 2>(wg, wu, bg, bu, n, k, frags, m, y, ldy, yt, nwaves, s, ev0, ev1);
}
}  // namespace

// y[r][c] = silu(x[r] . gate[c] + bias_gate[c]) * (x[r] . up[c] + bias_up[c]) for m <= TURQ_GEMV_MAX_M rows whose fragments
// turq_launch_act_prep prepared for this format; gate and up: two tiled weights of one format and shape [n, k]; up to four waves
hipError_t turq_launch_gemv_gateup_frag(int dtype, const void *w_gate, const void *w_up, int64_t n, int64_t k, const void *frags,
                                        int64_t m, void *y, int y_dtype, int64_t ldy, const float *bias_gate, const float *bias_up,
                                        int nwaves, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop) {
    if (nwaves < 1 || nwaves > 4 || m < 1 || m > TURQ_GEMV_MAX_M || k <= 0 || k % turq_dt_block_elems(dtype) != 0) return hipErrorInvalidValue;
    if (!turq_yt_ok(y_dtype, true)) return hipErrorInvalidValue;
    if (n == 0) return hipSuccess;
    switch (dtype) {
    case TURQ_Q4_K: return launch_gateup_frag<TURQ_Q4_K>(w_gate, w_up, bias_gate, bias_up, n, k, frags, m, y, ldy, y_dtype, nwaves, stream, ev_start, ev_stop);
    case TURQ_Q5_K: return launch_gateup_frag<TURQ_Q5_K>(w_gate, w_up, bias_gate, bias_up, n, k, frags, m, y, ldy, y_dtype, nwaves, stream, ev_start, ev_stop);
    case TURQ_Q6_K: return launch_gateup_frag<TURQ_Q6_K>(w_gate, w_up, bias_gate, bias_up, n, k, frags, m, y, ldy, y_dtype, nwaves, stream, ev_start, ev_stop);
    case TURQ_Q8_0: return launch_gateup_frag<TURQ_Q8_0>(w_gate, w_up, bias_gate, bias_up, n, k, frags, m, y, ldy, y_dtype, nwaves, stream, ev_start, ev_stop);
    default: return hipErrorInvalidValue;
    }
}

TURQ_NONFINITE_READER(turq_nonfinite_gemv_mfma)

// Skinny quantized matmul, 2 <= m <= 32 activation rows, for weights with several 16-row tiles per compute unit.
//
// A workgroup owns RG neighbouring row tiles of a weight and all of its columns; its waves split the 256-column tiles.  A wave
// builds the activation fragments of its column tile ONCE, in registers, straight from the caller's rows (f32 / bf16 / f16 ->
// f16, with the 16-element group sums the K-quants need: each lane reads exactly the values of its own A-operand slots, so
// there is no LDS pass, no cross-lane traffic and no preparation launch), and then streams the RG weight tiles of that column
// tile past them: the weights of a tile are requested D tiles ahead, across column-tile boundaries, so the stream from HBM
// never drains.  Every weight byte is read once and every activation once per workgroup.  The partial 16 x 16 results of the
// waves meet in the LDS at the end, in a fixed order.
//
// The tile arithmetic is the one of the other skinny kernels (gemv_tileop.h).
#include <hip/hip_ext.h>

#include <cstdlib>

#include "gemv_tileop.h"

namespace {

// one workgroup: row tiles grp * RG .. + RG - 1 of one weight, all column tiles, m <= 16 MT activation rows
template <int DT, int MT, int XT, int RG, int D>
__device__ __forceinline__ void cs_body(const uint8_t *__restrict__ w, int64_t n, int64_t k, const void *__restrict__ x, int64_t ldx,
                                        int64_t m, void *__restrict__ y, int yt, int64_t ldy, const float *__restrict__ bias,
                                        int64_t grp) {
    static_assert(RG % D == 0, "the ring of weight tiles repeats per column tile");
    extern __shared__ uint8_t smem[];
    constexpr int TB = TiledFmt<DT>::kTileBytes;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nwaves = blockDim.x >> 6;
    const int64_t ntc = turq_tile_cols(k), nrt = turq_tile_rows(n);
    const int64_t rt0 = grp * RG;
    float4v acc[RG][MT];
    const uint8_t *wrow[RG];  // row tiles past the weight's last one re-read it; their results are not stored
#pragma unroll
    for (int r = 0; r < RG; r++) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[r][mt] = float4v{0.f, 0.f, 0.f, 0.f};
        wrow[r] = w + (rt0 + r < nrt ? rt0 + r : nrt - 1) * ntc * TB;
    }
    GOff go = lane_offsets(lane, 16);
    WRegs<DT> wr[D];
    if (wave < ntc) {
#pragma unroll
        for (int d = 0; d < D; d++) wr[d] = load_tile<DT>(wrow[d] + (int64_t)wave * TB, go);
    }
    for (int64_t b = wave; b < ntc; b += nwaves) {
        go.touch();
        AFrags<DT, MT> f;
#pragma unroll
        for (int mt = 0; mt < MT; mt++) frags_from_rows<DT, XT>(x, ldx, m, k, b, lane, mt, f.a[mt]);
        const int64_t bn = b + nwaves;  // the wave's next column tile
#pragma unroll
        for (int r = 0; r < RG; r++) {
            TileOp<DT, MT, 4>::run(wr[r % D], f, lane, acc[r]);
            // the slot is free: request the tile D steps ahead
            if (r + D < RG) wr[r % D] = load_tile<DT>(wrow[r + D] + b * TB, go);
            else if (bn < ntc) wr[r % D] = load_tile<DT>(wrow[r + D - RG] + bn * TB, go);
        }
    }
    // the waves' partial tiles meet in the LDS; wave i adds up the i-th (row tile, m-tile) pair in wave order
    float4v *red = (float4v *)smem;
    if (nwaves > 1) {
#pragma unroll
        for (int r = 0; r < RG; r++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) red[((r * MT + mt) * nwaves + wave) * 64 + lane] = acc[r][mt];
        __syncthreads();
    }
    const int nn = lane & 15, g = lane >> 4;
    for (int i = wave; i < RG * MT; i += nwaves) {
        const int r = i / MT, mt = i - r * MT;
        float4v s;
        if (nwaves > 1) {
            s = red[(i * nwaves) * 64 + lane];
            for (int wv = 1; wv < nwaves; wv++) s += red[(i * nwaves + wv) * 64 + lane];
        } else {
            s = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int rr = 0; rr < RG; rr++)
#pragma unroll
                for (int mm = 0; mm < MT; mm++)
                    if (rr == r && mm == mt) s = acc[rr][mm];
        }
        const int64_t col = (rt0 + r) * 16 + nn;
        if (rt0 + r >= nrt || col >= n) continue;
        const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int64_t row = 16 * mt + 4 * g + j;
            if (row < m) turq_store_any(y, yt, row * ldy + col, s[j] + bv);
        }
    }
}

// The same workgroup, written out for a wave that owns exactly CPW column tiles.  In the loop above the compiler sizes its
// waits (s_waitcnt vmcnt) for the worst path through the conditions and schedules the header arithmetic of a tile ahead of the
// tiles before it, so a tile requested D steps ahead is in fact waited for at once, and the activations of a column tile, which
// are requested after the weights, drain the whole ring before they can be used.  Here every load sits in straight-line code,
// the tiles are kept apart by scheduling barriers, and the next column tile's activations are requested BEFORE the last D
// weight tiles of the current one - loads return in order, so waiting for them leaves the ring in flight - and converted after
// those D tiles, when they have long arrived.  Results are those of cs_body bit for bit.
template <int DT, int MT, int XT, int RG, int D, int CPW>
__device__ __forceinline__ void cs_body_unrolled(const uint8_t *__restrict__ w, int64_t n, int64_t k, const void *__restrict__ x, int64_t ldx,
                                                 int64_t m, void *__restrict__ y, int yt, int64_t ldy, const float *__restrict__ bias,
                                                 int64_t grp) {
    static_assert(RG % D == 0 && RG >= D, "the ring of weight tiles repeats per column tile");
    extern __shared__ uint8_t smem[];
    constexpr int TB = TiledFmt<DT>::kTileBytes;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nwaves = blockDim.x >> 6;  // ntc == CPW * nwaves
    const int64_t ntc = turq_tile_cols(k), nrt = turq_tile_rows(n);
    const int64_t rt0 = grp * RG;
    float4v acc[RG][MT];
    const uint8_t *wrow[RG];  // row tiles past the weight's last one re-read it; their results are not stored
#pragma unroll
    for (int r = 0; r < RG; r++) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[r][mt] = float4v{0.f, 0.f, 0.f, 0.f};
        wrow[r] = w + (rt0 + r < nrt ? rt0 + r : nrt - 1) * ntc * TB;
    }
    GOff go = lane_offsets(lane, 16);
    // the first column tile's activations go out first, the first D weight tiles right behind them
    RawRows<XT> raw[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) raw[mt] = load_rows_raw<DT, XT>(x, ldx, m, k, wave, lane, mt);
    WRegs<DT> wr[D];
#pragma unroll
    for (int d = 0; d < D; d++) wr[d] = load_tile<DT>(wrow[d] + (int64_t)wave * TB, go);
    AFrags<DT, MT> f;
#pragma unroll
    for (int mt = 0; mt < MT; mt++) frags_from_raw<DT, XT>(raw[mt], f.a[mt]);
#pragma unroll
    for (int c = 0; c < CPW; c++) {
        const int64_t b = wave + (int64_t)c * nwaves, bn = b + nwaves;
#pragma unroll
        for (int r = 0; r < RG; r++) {
            if (r == RG - D && c + 1 < CPW) {
#pragma unroll
                for (int mt = 0; mt < MT; mt++) raw[mt] = load_rows_raw<DT, XT>(x, ldx, m, k, bn, lane, mt);
            }
            TileOp<DT, MT, 4>::run(wr[r % D], f, lane, acc[r]);
            __builtin_amdgcn_sched_barrier(0);
            // the slot is free: request the tile D steps ahead
            if (r + D < RG) wr[r % D] = load_tile<DT>(wrow[r + D] + b * TB, go);
            else if (c + 1 < CPW) wr[r % D] = load_tile<DT>(wrow[r + D - RG] + bn * TB, go);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (c + 1 < CPW) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++) frags_from_raw<DT, XT>(raw[mt], f.a[mt]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // the waves' partial tiles meet in the LDS; wave i adds up the i-th (row tile, m-tile) pair in wave order
    float4v *red = (float4v *)smem;
#pragma unroll
    for (int r = 0; r < RG; r++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) red[((r * MT + mt) * nwaves + wave) * 64 + lane] = acc[r][mt];
    __syncthreads();
    const int nn = lane & 15, g = lane >> 4;
    for (int i = wave; i < RG * MT; i += nwaves) {
        const int r = i / MT, mt = i - r * MT;
        float4v s = red[(i * nwaves) * 64 + lane];
        for (int wv = 1; wv < nwaves; wv++) s += red[(i * nwaves + wv) * 64 + lane];
        const int64_t col = (rt0 + r) * 16 + nn;
        if (rt0 + r >= nrt || col >= n) continue;
        const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int64_t row = 16 * mt + 4 * g + j;
            if (row < m) turq_store_any(y, yt, row * ldy + col, s[j] + bv);
        }
    }
}

template <int DT, int MT, int XT, int RG, int D, int CPW, int MAXT>
__global__ void __launch_bounds__(MAXT) gemv_cs_unrolled_kernel(MultiArgs a, int64_t k, const void *__restrict__ x, int64_t ldx, int64_t m,
                                                                 int yt) {
    const MultiPick p = multi_pick(a, (int)blockIdx.x);
    cs_body_unrolled<DT, MT, XT, RG, D, CPW>(p.w, p.n, k, x, ldx, m, p.y, yt, p.ldy, p.bias, (int64_t)p.block);
}

template <int DT, int MT, int XT, int RG, int D, int MAXT>
__global__ void __launch_bounds__(MAXT) gemv_cs_kernel(MultiArgs a, int64_t k, const void *__restrict__ x, int64_t ldx, int64_t m, int yt) {
    const MultiPick p = multi_pick(a, (int)blockIdx.x);
    cs_body<DT, MT, XT, RG, D>(p.w, p.n, k, x, ldx, m, p.y, yt, p.ldy, p.bias, (int64_t)p.block);
}

struct CsLaunch {
    MultiArgs a;
    int blocks;
    int64_t k;
    const void *x;
    int64_t ldx, m;
    int yt, nwaves;
    hipStream_t s;
    hipEvent_t ev0, ev1;
};

template <int DT, int MT, int XT, int RG, int D>
hipError_t launch_final(const CsLaunch &l) {
    constexpr int MAXT = 512;
    const size_t lds = l.nwaves > 1 ? (size_t)l.nwaves * RG * MT * 64 * sizeof(float4v) : 0;
    if (lds > (64u << 10)) {
        static const hipError_t raised = hipFuncSetAttribute((const void *)gemv_cs_kernel<DT, MT, XT, RG, D, MAXT>,
                                                             hipFuncAttributeMaxDynamicSharedMemorySize, 128 << 10);
        if (raised != hipSuccess) return raised;
    }
    const dim3 grid((unsigned)l.blocks), block((unsigned)(64 * l.nwaves));
    // a wave that owns exactly two column tiles (K = 4096 with eight waves): the written-out form
    static const bool generic = [] { const char *e = getenv("TURQ_CS_GENERIC"); return e && atoi(e) != 0; }();
    if constexpr (MT == 1 && RG == 6) {
        if (!generic && l.nwaves > 1 && turq_tile_cols(l.k) == 2 * (int64_t)l.nwaves && lds <= (64u << 10)) {
            if (l.ev0) {
                hipExtLaunchKernelGGL((gemv_cs_unrolled_kernel<DT, MT, XT, RG, D, 2, MAXT>), grid, block, (unsigned)lds, l.s, l.ev0, l.ev1, 0,
                                      l.a, l.k, l.x, l.ldx, l.m, l.yt);
                return hipGetLastError();
            }
            gemv_cs_unrolled_kernel<DT, MT, XT, RG, D, 2, MAXT><<<grid, block, lds, l.s>>>(l.a, l.k, l.x, l.ldx, l.m, l.yt);
            return hipGetLastError();
        }
    }
    if (l.ev0) {
        hipExtLaunchKernelGGL((gemv_cs_kernel<DT, MT, XT, RG, D, MAXT>), grid, block, (unsigned)lds, l.s, l.ev0, l.ev1, 0, l.a, l.k, l.x,
                              l.ldx, l.m, l.yt);
        return hipGetLastError();
    }
    gemv_cs_kernel<DT, MT, XT, RG, D, MAXT><<<grid, block, lds, l.s>>>(l.a, l.k, l.x, l.ldx, l.m, l.yt);
    return hipGetLastError();
}

template <int DT, int MT, int XT>
hipError_t launch_rg(int rg, const CsLaunch &l) {
    switch (rg) {
    case 2: return launch_final<DT, MT, XT, 2, 2>(l);
    case 3: return launch_final<DT, MT, XT, 3, 3>(l);
    case 6: return launch_final<DT, MT, XT, 6, 3>(l);
    default: return hipErrorInvalidValue;
    }
}

template <int DT, int XT>
hipError_t launch_mt(int rg, const CsLaunch &l) {
    return l.m <= 16 ? launch_rg<DT, 1, XT>(rg, l) : launch_rg<DT, 2, XT>(rg, l);
}

template <int DT>
hipError_t launch_xt(int xt, int rg, const CsLaunch &l) {
    switch (xt) {
    case TURQ_ACT_F32: return launch_mt<DT, TURQ_ACT_F32>(rg, l);
    case TURQ_ACT_BF16: return launch_mt<DT, TURQ_ACT_BF16>(rg, l);
    case TURQ_ACT_F16: return launch_mt<DT, TURQ_ACT_F16>(rg, l);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

// row tiles per workgroup this kernel is built for
bool turq_gemv_cs_rows_ok(int row_tiles_per_group) { return row_tiles_per_group == 2 || row_tiles_per_group == 3 || row_tiles_per_group == 6; }

// count (1..4) tiled weights of one format and one k against m (2..32) activation rows of stride ldx (rows 16-byte aligned);
// row_tiles (2, 3 or 6) per workgroup, nwaves (1..8) waves that split the column tiles
hipError_t turq_launch_gemv_cs(int dtype, int count, const void *const *w, const int64_t *n, int64_t k, const void *x, int x_dtype,
                               int64_t ldx, int64_t m, void *const *y, int y_dtype, const int64_t *ldy, const float *const *bias,
                               int nwaves, int row_tiles, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop) {
    if (count < 1 || count > kMaxMulti || m < 1 || m > TURQ_GEMV_MAX_M || nwaves < 1 || nwaves > 8 || !turq_gemv_cs_rows_ok(row_tiles))
        return hipErrorInvalidValue;
    if (k <= 0 || k % turq_dt_block_elems(dtype) != 0) return hipErrorInvalidValue;
    if (y_dtype != TURQ_ACT_F32 && y_dtype != TURQ_ACT_BF16 && y_dtype != TURQ_ACT_F16) return hipErrorInvalidValue;
    CsLaunch l{};
    int64_t blocks = 0;
    for (int i = 0; i < count; i++) {
        l.a.w[i] = (const uint8_t *)w[i];
        l.a.y[i] = y[i];
        l.a.bias[i] = bias ? bias[i] : nullptr;
        l.a.n[i] = n[i];
        l.a.ldy[i] = ldy ? ldy[i] : n[i];
        l.a.first[i] = (int)blocks;
        blocks += (turq_tile_rows(n[i]) + row_tiles - 1) / row_tiles;
    }
    l.a.count = count;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFF) return hipErrorInvalidValue;
    l.blocks = (int)blocks, l.k = k, l.x = x, l.ldx = ldx, l.m = m, l.yt = y_dtype, l.nwaves = nwaves;
    l.s = stream, l.ev0 = ev_start, l.ev1 = ev_stop;
    switch (dtype) {
    case TURQ_Q4_K: return launch_xt<TURQ_Q4_K>(x_dtype, row_tiles, l);
    case TURQ_Q5_K: return launch_xt<TURQ_Q5_K>(x_dtype, row_tiles, l);
    case TURQ_Q6_K: return launch_xt<TURQ_Q6_K>(x_dtype, row_tiles, l);
    case TURQ_Q8_0: return launch_xt<TURQ_Q8_0>(x_dtype, row_tiles, l);
    default: return hipErrorInvalidValue;
    }
}

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
// This file holds that form as a loop over single column tiles (any k), and the entry points of the faster form that stages the
// activation rows through the LDS (gemv_cs_staged.h: k a multiple of 512), which the dispatcher prefers wherever it applies.
//
// The tile arithmetic is the one of the other skinny kernels (gemv_tileop.h).
#include <hip/hip_ext.h>

#include <cstdlib>

#include "gemv_cs_staged.h"

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
        turq_store_col4(y, yt, 16 * mt + 4 * g, m, ldy, col, s + float4v{bv, bv, bv, bv});
    }
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
        const hipError_t raised = turq_raise_lds_limit((const void *)gemv_cs_kernel<DT, MT, XT, RG, D, MAXT>, 128 << 10);
        if (raised != hipSuccess) return raised;
    }
    const dim3 grid((unsigned)l.blocks), block((unsigned)(64 * l.nwaves));
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
    // (not instantiated: the group sizes that do not fit the register file - six row tiles with two activation tiles or with
    // Q8_0's 4352-byte tiles, three with both; cs_row_tiles() in mfma_dispatch.cpp never asks for them)
    switch (rg) {
    case 2: return launch_final<DT, MT, XT, 2, 2>(l);
    case 3:
        if constexpr (DT == TURQ_Q8_0 && MT == 2) return hipErrorInvalidValue;
        else return launch_final<DT, MT, XT, 3, 3>(l);
    case 6:
        if constexpr (DT == TURQ_Q8_0 || MT == 2) return hipErrorInvalidValue;
        else return launch_final<DT, MT, XT, 6, 3>(l);
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
    if (!turq_yt_ok(y_dtype, true)) return hipErrorInvalidValue;
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

// ---- activations staged through the LDS (gemv_cs_staged.h; one translation unit per activation type) ----
// k a multiple of 512; up to 32 rows
hipError_t turq_launch_gemv_cs_staged_f32(TURQ_STAGED_LAUNCH_ARGS);
hipError_t turq_launch_gemv_cs_staged_bf16(TURQ_STAGED_LAUNCH_ARGS);
hipError_t turq_launch_gemv_cs_staged_f16(TURQ_STAGED_LAUNCH_ARGS);

// whether the staged form has this case: formats (dtype_b = dtype_a for one format, else a K-quant pair with Q6_K second),
// k, m and row tiles per workgroup (1, 2; 3 up to 16 rows; 6 up to 16 rows and, in the four-wave form, from 17)
bool turq_gemv_cs_staged_takes(int dtype_a, int dtype_b, int64_t k, int64_t m, int row_tiles) {
    if (!turq_gemv_cs_staged_waves(k) || m < 1 || m > 32) return false;
    if (dtype_a != dtype_b && !((dtype_a == TURQ_Q4_K || dtype_a == TURQ_Q5_K) && dtype_b == TURQ_Q6_K)) return false;
    if (dtype_a != TURQ_Q4_K && dtype_a != TURQ_Q5_K && dtype_a != TURQ_Q6_K && dtype_a != TURQ_Q8_0) return false;
    if (m > 16 && row_tiles != 6 && k > 4096) return false;  // the two passes of 16 rows are only built with one pair per wave
    return row_tiles == 1 || row_tiles == 2 || (row_tiles == 3 && m <= 16) || row_tiles == 6;
}

int turq_gemv_cs_staged_second_rows(int row_tiles) { return staged_second_rows(row_tiles); }

// count (1..4) tiled weights of one k against m (1..32) activation rows of stride ldx (rows 16-byte aligned); the first `second`
// weights are of format dtype_a, the others of dtype_b (second = count and dtype_b = dtype_a: one format); row_tiles per
// workgroup as turq_gemv_cs_staged_takes accepts (the weights of a second format: turq_gemv_cs_staged_second_rows of it)
hipError_t turq_launch_gemv_cs_staged(int dtype_a, int dtype_b, int count, int second, const void *const *w, const int64_t *n, int64_t k,
                                      const void *x, int x_dtype, int64_t ldx, int64_t m, void *const *y, int y_dtype, const int64_t *ldy,
                                      const float *const *bias, int row_tiles, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop) {
    if (count < 1 || count > kMaxMulti || second < 1 || second > count || (second == count) != (dtype_a == dtype_b) ||
        !turq_gemv_cs_staged_takes(dtype_a, dtype_b, k, m, row_tiles))
        return hipErrorInvalidValue;
    if (!turq_yt_ok(y_dtype, true)) return hipErrorInvalidValue;
    switch (x_dtype) {
    case TURQ_ACT_F32: return turq_launch_gemv_cs_staged_f32(TURQ_STAGED_LAUNCH_PASS);
    case TURQ_ACT_BF16: return turq_launch_gemv_cs_staged_bf16(TURQ_STAGED_LAUNCH_PASS);
    case TURQ_ACT_F16: return turq_launch_gemv_cs_staged_f16(TURQ_STAGED_LAUNCH_PASS);
    default: return hipErrorInvalidValue;
    }
}

// ---- gate and up of an MLP with the activation and the product in the staged kernel ----
hipError_t turq_launch_gemv_cs_staged_gateup_f32(TURQ_STAGED_GATEUP_ARGS);
hipError_t turq_launch_gemv_cs_staged_gateup_bf16(TURQ_STAGED_GATEUP_ARGS);
hipError_t turq_launch_gemv_cs_staged_gateup_f16(TURQ_STAGED_GATEUP_ARGS);

// tiles per workgroup (gate and up together: 2 or 6) for n output columns on `units` compute units, 0: not this case
// (17 .. 32 rows: the four-wave form, which has groups of 6, on up to 4096 columns)
int turq_gemv_cs_staged_gateup_tiles(int dtype, int64_t n, int64_t k, int64_t m, int64_t units) {
    if (dtype != TURQ_Q4_K && dtype != TURQ_Q5_K && dtype != TURQ_Q6_K && dtype != TURQ_Q8_0) return 0;
    if (!turq_gemv_cs_staged_waves(k) || m < 1 || m > 32) return 0;
    if (m > 16) return (turq_tile_rows(n) > 2 * units && k <= 4096) ? 6 : 0;
    return turq_tile_rows(n) > 2 * units ? 6 : 2;
}

// y[r][c] = silu(x[r] . gate[c] + bias_gate[c]) * (x[r] . up[c] + bias_up[c]); tiled weights of one format, n and k; m (1..32)
// activation rows of stride ldx (rows 16-byte aligned); tiles as turq_gemv_cs_staged_gateup_tiles says
hipError_t turq_launch_gemv_cs_staged_gateup(int dtype, const void *w_gate, const void *w_up, int64_t n, int64_t k, const void *x, int x_dtype,
                                             int64_t ldx, int64_t m, void *y, int y_dtype, int64_t ldy, const float *bias_gate,
                                             const float *bias_up, int tiles, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop) {
    if (!turq_gemv_cs_staged_waves(k) || m < 1 || m > 32 || (tiles != 2 && tiles != 6) || (m > 16 && tiles != 6)) return hipErrorInvalidValue;
    if (!turq_yt_ok(y_dtype, true)) return hipErrorInvalidValue;
    switch (x_dtype) {
    case TURQ_ACT_F32: return turq_launch_gemv_cs_staged_gateup_f32(TURQ_STAGED_GATEUP_PASS);
    case TURQ_ACT_BF16: return turq_launch_gemv_cs_staged_gateup_bf16(TURQ_STAGED_GATEUP_PASS);
    case TURQ_ACT_F16: return turq_launch_gemv_cs_staged_gateup_f16(TURQ_STAGED_GATEUP_PASS);
    default: return hipErrorInvalidValue;
    }
}

TURQ_NONFINITE_READER(turq_nonfinite_gemv_cs)

// The skinny kernel that splits the columns over the waves of a workgroup, in the form that stages the activation rows through
// the LDS (see gemv_cs.hip for the decomposition).  One translation unit per activation type instantiates it (the kernels are
// many and large), each through staged_launch<XT>.
#pragma once

#include <hip/hip_ext.h>

#include <algorithm>
#include <type_traits>

#include "gemv_tileop.h"

namespace {

// ---- a workgroup owns RG row tiles and all columns; a wave walks its column tiles in PAIRS ----
//
// Two things hold back the form of this decomposition whose lanes load their own A-operand slots from the caller's rows in a loop
// over single column tiles (gemv_cs.hip).  (1) A lane that loads exactly its own A-operand slots reads 16 bytes from each of 32
// different cache lines per instruction (rows are a row stride apart, lane groups 256 bytes), and half of that twice when there
// are no more than 8 rows: the address unit of the CU works through four to eight times the lines the data needs, the loads of
// the second wave of every SIMD queue behind those of the first, and for microseconds half of the waves have no activations and
// request no weights.  (2) The compiler sizes its waits (s_waitcnt vmcnt) for the worst path through the loop's conditions and
// schedules the header arithmetic of a tile ahead of the tiles before it, so a tile requested D steps ahead is waited for at once.
//
// Here a wave loads the rows of its column tile as they lie in memory (one KiB per instruction: a whole f32 row, or two rows of
// 16-bit values), converts them to f16, writes them to its own few KiB of the LDS and reads its A-operand slots back from there
// (LDS operations of one wave complete in order: no barrier).  The column tiles of a weight are taken in pairs (2 p, 2 p + 1),
// wave w of the workgroup takes pairs w, w + waves, ...; the code of a pair is straight-line - every load unconditional, the
// tiles kept apart by scheduling barriers, the next column tile's rows requested as soon as the current ones have been written to
// the LDS, the weight ring reaching into the next pair - and exists twice: as the body of a loop over all pairs but the last,
// and once more without the requests for a next pair.  With every path through the loop issuing the same loads in the same
// order the compiler's wait counts are exact, and any even number of column tiles goes (k a multiple of 512).  Results are
// those of cs_body bit for bit where both apply (same conversions, sums and tile order).
constexpr int kXRow = 512 + 16;  // bytes per staged activation row: 256 f16 and a pad that spreads the rows over the banks

template <int XT, int MR> struct XRows {
    uint4v v[XT == TURQ_ACT_F32 ? MR : MR / 2];
};
// rows row0 .. row0 + MR - 1 (rows past m repeat row m - 1) of column tile b
template <int XT, int MR>
__device__ inline XRows<XT, MR> load_x_rows(const void *__restrict__ x, int64_t ldx, int64_t m, int row0, int64_t b, int lane) {
    XRows<XT, MR> raw;
    if constexpr (XT == TURQ_ACT_F32) {
#pragma unroll
        for (int j = 0; j < MR; j++) {
            const int64_t row = row0 + j < m ? row0 + j : m - 1;
            raw.v[j] = *(const uint4v *)((const uint8_t *)x + (row * ldx + b * 256) * 4 + 16 * lane);
        }
    } else {
#pragma unroll
        for (int i = 0; i < MR / 2; i++) {
            const int64_t j = row0 + 2 * i + (lane >> 5), row = j < m ? j : m - 1;
            raw.v[i] = *(const uint4v *)((const uint8_t *)x + (row * ldx + b * 256) * 2 + 16 * (lane & 31));
        }
    }
    return raw;
}
// ... as f16 into the wave's LDS rows
template <int XT, int MR> __device__ inline void stage_x_rows(const XRows<XT, MR> &raw, uint8_t *__restrict__ rows, int lane) {
    if constexpr (XT == TURQ_ACT_F32) {
#pragma unroll
        for (int j = 0; j < MR; j++) {
            const uint4v a = raw.v[j];
            const half2v h0 = __builtin_convertvector(float2v{__uint_as_float(a.x), __uint_as_float(a.y)}, half2v);
            const half2v h1 = __builtin_convertvector(float2v{__uint_as_float(a.z), __uint_as_float(a.w)}, half2v);
            *(uint2v *)(rows + j * kXRow + 8 * lane) = uint2v{__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1)};
        }
    } else {
#pragma unroll
        for (int i = 0; i < MR / 2; i++) {
            uint8_t *p = rows + (2 * i + (lane >> 5)) * kXRow + 16 * (lane & 31);
            if constexpr (XT == TURQ_ACT_BF16) *(half8v *)p = bf16x8_to_half8(raw.v[i]);
            else *(uint4v *)p = raw.v[i];
        }
    }
}
// the A fragments of the staged column tile: lane (r, g) holds row r (rows past m repeat row m - 1);
// K-quants: step q = columns 64 g + 8 q .. + 7, step 8 = the (hi, lo) sums of its four 16-column groups; Q8_0: step q = columns 32 q + 8 g .. + 7
template <int DT> __device__ inline void frags_from_staged(const uint8_t *__restrict__ rows, int m, int lane, half8v *__restrict__ out) {
    const int r = lane & 15, g = lane >> 4;
    const uint8_t *p = rows + (r < m ? r : m - 1) * kXRow + (DT != TURQ_Q8_0 ? 128 : 16) * g;
#pragma unroll
    for (int q = 0; q < 8; q++) out[q] = *(const half8v *)(p + (DT != TURQ_Q8_0 ? 16 : 64) * q);
    if constexpr (DT != TURQ_Q8_0) out[8] = kq_group_sums(out);
}

// m <= MR rows (4, 8, 16 or 32), k a multiple of 512.  More than 16 rows are taken as two halves of 16, one after the other against
// the same weight tiles (HV = 2): the tiles of a column tile stay in their registers for both passes and are unpacked once per
// pass, which for these launches costs less than what holding the fragments of 32 rows next to the rows in flight would
// (registers), or a launch that prepares them.  D: weight tiles in flight; a ring slot holds the same tile of every pair, so D
// divides 2 RG (and with two passes is at least RG: a column tile's tiles stay for both).
// GU: the workgroup's row tiles are RG / 2 of a gate weight (w) and the same RG / 2 of an up weight (w2) of one shape, and what
// is stored is silu(gate) * up (src/models/qwen3.rs:161-167).
// CNT: pairs per wave when every wave has the same number and it is known at compile time (the loop is then written out, which
// is 1 - 5 % faster on the 4096-column weights), 0: counted at run time.
template <int DT, int XT, int MR, int RG, int D, int CNT, bool GU = false>
__device__ __forceinline__ void cs_body_staged(const uint8_t *__restrict__ w, int64_t n, int64_t k, const void *__restrict__ x, int64_t ldx,
                                               int64_t m, void *__restrict__ y, int yt, int64_t ldy, const float *__restrict__ bias,
                                               int64_t grp, const uint8_t *__restrict__ w2 = nullptr,
                                               const float *__restrict__ bias2 = nullptr) {
    static_assert(!GU || RG % 2 == 0, "gate and up tiles come in pairs");
    constexpr int RO = GU ? RG / 2 : RG;  // row tiles of the output per workgroup
    constexpr int HV = MR > 16 ? 2 : 1;   // passes of HR rows each
    constexpr int HR = MR / HV;
    static_assert(D >= 1 && D <= 2 * RG && (2 * RG) % D == 0 && (HV == 1 || D >= RG), "ring of weight tiles");
    extern __shared__ uint8_t smem[];
    constexpr int TB = TiledFmt<DT>::kTileBytes;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nwaves = blockDim.x >> 6;  // at most ntc / 2
    const int64_t ntc = turq_tile_cols(k), nrt = turq_tile_rows(n);
    const int cnt = __builtin_amdgcn_readfirstlane((int)((ntc / 2 - wave + nwaves - 1) / nwaves));  // the wave's pairs
    const int64_t rt0 = grp * RO;
    float4v acc[RG][HV];
    const uint8_t *wrow[RG];  // row tiles past the weight's last one re-read it; their results are not stored
#pragma unroll
    for (int r = 0; r < RG; r++) {
#pragma unroll
        for (int h = 0; h < HV; h++) acc[r][h] = float4v{0.f, 0.f, 0.f, 0.f};
        const int ro = r < RO ? r : r - RO;
        wrow[r] = (r < RO ? w : w2) + (rt0 + ro < nrt ? rt0 + ro : nrt - 1) * ntc * TB;
    }
    GOff go = lane_offsets(lane, 16);
    int64_t p = wave;  // the current pair: column tiles 2 p and 2 p + 1
    // the first column tile's rows go out first, the first D weight tiles right behind them
    XRows<XT, HR> raw = load_x_rows<XT, HR>(x, ldx, m, 0, 2 * p, lane);
    WRegs<DT> wr[D];
#pragma unroll
    for (int d = 0; d < D; d++) wr[d] = load_tile<DT>(wrow[d % RG] + (2 * p + d / RG) * TB, go);
    uint8_t *rows = smem + wave * (HR * kXRow);
    AFrags<DT, 1> f;
    auto pair = [&](auto last) {
        constexpr bool LAST = decltype(last)::value;
#pragma unroll
        for (int cc = 0; cc < 2; cc++) {
#pragma unroll
            for (int h = 0; h < HV; h++) {
                stage_x_rows<XT, HR>(raw, rows, lane);
                __builtin_amdgcn_sched_barrier(0);
                // the rows of the next pass: the other half of this column tile, the pair's second column tile, the next pair
                if (h + 1 < HV) raw = load_x_rows<XT, HR>(x, ldx, m, HR * (h + 1), 2 * p + cc, lane);
                else if (cc == 0) raw = load_x_rows<XT, HR>(x, ldx, m, 0, 2 * p + 1, lane);
                else if (!LAST) raw = load_x_rows<XT, HR>(x, ldx, m, 0, 2 * (p + nwaves), lane);
                __builtin_amdgcn_sched_barrier(0);
                frags_from_staged<DT>(rows, (int)m - HR * h, lane, f.a[0]);
#pragma unroll
                for (int r = 0; r < RG; r++) {
                    const int t = cc * RG + r;
                    // (second pass: unpacked again; what the compiler would keep of the first pass's operands does not fit the
                    // registers of more than one row tile)
                    if constexpr (RG > 1) {
                        if (h > 0) touch(wr[t % D]);
                    }
                    TileOp<DT, 1, 4>::run(wr[t % D], f, lane, &acc[r][h]);
                    __builtin_amdgcn_sched_barrier(0);
                    // after the last pass the slot is free: request the tile D steps ahead, in this pair or the next
                    if (h == HV - 1) {
                        if (t + D < 2 * RG) wr[t % D] = load_tile<DT>(wrow[(t + D) % RG] + (2 * p + (t + D) / RG) * TB, go);
                        else if (!LAST) wr[t % D] = load_tile<DT>(wrow[(t + D - 2 * RG) % RG] + (2 * (p + nwaves) + (t + D - 2 * RG) / RG) * TB, go);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };
    if constexpr (CNT > 0) {
#pragma unroll
        for (int i = 1; i < CNT; i++) {
            pair(std::false_type{});
            p += nwaves;
        }
    } else {
        for (int i = 1; i < cnt; i++) {
            pair(std::false_type{});
            p += nwaves;
        }
    }
    pair(std::true_type{});
    // the waves' partial tiles meet in the LDS (over the staged rows, once every wave is done with its own);
    // wave i adds up the i-th (row tile, pass) pair in wave order
    __syncthreads();
    float4v *red = (float4v *)smem;
#pragma unroll
    for (int r = 0; r < RG; r++)
#pragma unroll
        for (int h = 0; h < HV; h++) red[((r * HV + h) * nwaves + wave) * 64 + lane] = acc[r][h];
    __syncthreads();
    const int nn = lane & 15, g = lane >> 4;
    for (int i = wave; i < RO * HV; i += nwaves) {
        const int r = i / HV, h = i - r * HV;
        float4v s = red[(i * nwaves) * 64 + lane];
        for (int wv = 1; wv < nwaves; wv++) s += red[(i * nwaves + wv) * 64 + lane];
        float4v s2 = float4v{0.f, 0.f, 0.f, 0.f};
        if constexpr (GU) {
            const int i2 = i + RO * HV;  // the up tile of the pair
            s2 = red[(i2 * nwaves) * 64 + lane];
            for (int wv = 1; wv < nwaves; wv++) s2 += red[(i2 * nwaves + wv) * 64 + lane];
        }
        const int64_t col = (rt0 + r) * 16 + nn;
        if (rt0 + r >= nrt || col >= n) continue;
        const float bv = bias ? bias[col] : 0.0f, bv2 = (GU && bias2) ? bias2[col] : 0.0f;
        if constexpr (GU) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int64_t row = HR * h + 4 * g + j;
                if (row >= m) continue;
                const float gate = s[j] + bv, up = s2[j] + bv2;
                turq_store_any(y, yt, row * ldy + col, gate / (1.0f + expf(-gate)) * up);
            }
        } else {
            turq_store_col4(y, yt, HR * h + 4 * g, m, ldy, col, s + float4v{bv, bv, bv, bv});
        }
    }
}

// weight tiles in flight per wave for RG row tiles per workgroup (measured on 4096- and 12288-column weights: a deeper ring
// delays the activation rows behind it); with two passes per tile a column tile's tiles (a slot is requested again a whole pass
// before its next use; more does not fit the registers next to 16 f32 rows in flight)
constexpr int staged_ring(int dt, int rg, int mr, bool two_formats = false) {
    if (mr > 16) return rg == 1 ? 2 : rg;
    // (three tiles do not fit the registers next to 16 f32 rows: Q6_K, and the kernels that hold the code of two formats)
    if ((dt == TURQ_Q6_K || two_formats) && rg == 6 && mr == 16) return 2;
    return rg == 1 ? 2 : rg == 2 ? 4 : 3;
}
// row tiles per workgroup for the weights of the second format of a two-format launch: Q6_K tiles behind Q4_K / Q5_K ones are
// half as large again and cost half as much arithmetic again, so their workgroups take fewer of them
constexpr int staged_second_rows(int rg) { return (rg + 1) / 2; }

// weights [0, a.second) are of format DTA with RG row tiles per workgroup, the others of DTB with staged_second_rows(RG)
// (one format: DTA == DTB)
template <int DTA, int DTB, int XT, int MR, int RG, int CNT>
__global__ void __launch_bounds__(512) gemv_cs_staged_kernel(MultiArgs a, int64_t k, const void *__restrict__ x, int64_t ldx, int64_t m, int yt) {
    const MultiPick p = multi_pick(a, (int)blockIdx.x);
    constexpr int RGB = staged_second_rows(RG);
    if (DTA == DTB || p.index < a.second)
        cs_body_staged<DTA, XT, MR, RG, staged_ring(DTA, RG, MR, DTA != DTB), CNT>(p.w, p.n, k, x, ldx, m, p.y, yt, p.ldy, p.bias, (int64_t)p.block);
    else
        cs_body_staged<DTB, XT, MR, RGB, staged_ring(DTB, RGB, MR, DTA != DTB), CNT>(p.w, p.n, k, x, ldx, m, p.y, yt, p.ldy, p.bias, (int64_t)p.block);
}

// gate (a.w[0]) and up (a.w[1]) of one MLP, RG / 2 row tiles of each per workgroup, silu(gate) * up stored to a.y[0]
template <int DT, int XT, int MR, int RG, int CNT>
__global__ void __launch_bounds__(512) gemv_cs_staged_gateup_kernel(MultiArgs a, int64_t k, const void *__restrict__ x, int64_t ldx, int64_t m,
                                                                     int yt) {
    cs_body_staged<DT, XT, MR, RG, staged_ring(DT, RG, MR), CNT, true>(a.w[0], a.n[0], k, x, ldx, m, a.y[0], yt, a.ldy[0], a.bias[0],
                                                               (int64_t)blockIdx.x, a.w[1], a.bias[1]);
}

// ---- 17 .. 32 rows, both 16-row tiles against ONE unpack of a weight tile ----
// The fragments of 32 rows (72 registers) next to 32 f32 rows in flight (128) and the accumulators of six row tiles (48) do not
// fit 256 registers, which is what a wave gets with two waves per SIMD; with FOUR waves per workgroup (one per SIMD) a wave may
// use 512, and a weight tile is unpacked once for both 16-row tiles instead of once per pass.  That wins where there are several
// row tiles per set of fragments (gate / up at 32 rows: 25.3 us against 32.8 in two passes and 26.1 + 3.9 with prepared
// fragments); with one row tile per workgroup the two passes with eight waves are as fast, and with two row tiles of Q4_K next to
// one of Q6_K (q / k / v) faster (13.7 against 15.0 us), so only groups of six are built.
template <int DT, int XT, int RG, int D, int CNT, bool GU = false>
__device__ __forceinline__ void cs_body_staged_two(const uint8_t *__restrict__ w, int64_t n, int64_t k, const void *__restrict__ x, int64_t ldx,
                                                   int64_t m, void *__restrict__ y, int yt, int64_t ldy, const float *__restrict__ bias,
                                                   int64_t grp, const uint8_t *__restrict__ w2 = nullptr,
                                                   const float *__restrict__ bias2 = nullptr) {
    static_assert(!GU || RG % 2 == 0, "gate and up tiles come in pairs");
    constexpr int RO = GU ? RG / 2 : RG;  // row tiles of the output per workgroup
    static_assert(D >= 1 && D <= 2 * RG && (2 * RG) % D == 0, "ring of weight tiles");
    extern __shared__ uint8_t smem[];
    constexpr int TB = TiledFmt<DT>::kTileBytes;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nwaves = blockDim.x >> 6;  // at most ntc / 2
    const int64_t ntc = turq_tile_cols(k), nrt = turq_tile_rows(n);
    const int cnt = __builtin_amdgcn_readfirstlane((int)((ntc / 2 - wave + nwaves - 1) / nwaves));  // the wave's pairs
    const int64_t rt0 = grp * RO;
    float4v acc[RG][2];
    const uint8_t *wrow[RG];  // row tiles past the weight's last one re-read it; their results are not stored
#pragma unroll
    for (int r = 0; r < RG; r++) {
        acc[r][0] = acc[r][1] = float4v{0.f, 0.f, 0.f, 0.f};
        const int ro = r < RO ? r : r - RO;
        wrow[r] = (r < RO ? w : w2) + (rt0 + ro < nrt ? rt0 + ro : nrt - 1) * ntc * TB;
    }
    GOff go = lane_offsets(lane, 16);
    int64_t p = wave;
    XRows<XT, 16> raw[2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++) raw[mt] = load_x_rows<XT, 16>(x, ldx, m, 16 * mt, 2 * p, lane);
    WRegs<DT> wr[D];
#pragma unroll
    for (int d = 0; d < D; d++) wr[d] = load_tile<DT>(wrow[d % RG] + (2 * p + d / RG) * TB, go);
    uint8_t *rows = smem + wave * (32 * kXRow);
    AFrags<DT, 2> f;
    auto pair = [&](auto last) {
        constexpr bool LAST = decltype(last)::value;
#pragma unroll
        for (int cc = 0; cc < 2; cc++) {
#pragma unroll
            for (int mt = 0; mt < 2; mt++) stage_x_rows<XT, 16>(raw[mt], rows + mt * 16 * kXRow, lane);
            __builtin_amdgcn_sched_barrier(0);
            if (cc == 0 || !LAST) {
                const int64_t b = cc == 0 ? 2 * p + 1 : 2 * (p + nwaves);
#pragma unroll
                for (int mt = 0; mt < 2; mt++) raw[mt] = load_x_rows<XT, 16>(x, ldx, m, 16 * mt, b, lane);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int mt = 0; mt < 2; mt++) frags_from_staged<DT>(rows + mt * 16 * kXRow, (int)m - 16 * mt, lane, f.a[mt]);
#pragma unroll
            for (int r = 0; r < RG; r++) {
                const int t = cc * RG + r;
                TileOp<DT, 2, 4>::run(wr[t % D], f, lane, acc[r]);
                __builtin_amdgcn_sched_barrier(0);
                if (t + D < 2 * RG) wr[t % D] = load_tile<DT>(wrow[(t + D) % RG] + (2 * p + (t + D) / RG) * TB, go);
                else if (!LAST) wr[t % D] = load_tile<DT>(wrow[(t + D - 2 * RG) % RG] + (2 * (p + nwaves) + (t + D - 2 * RG) / RG) * TB, go);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    if constexpr (CNT > 0) {
#pragma unroll
        for (int i = 1; i < CNT; i++) {
            pair(std::false_type{});
            p += nwaves;
        }
    } else {
        for (int i = 1; i < cnt; i++) {
            pair(std::false_type{});
            p += nwaves;
        }
    }
    pair(std::true_type{});
    __syncthreads();
    float4v *red = (float4v *)smem;
#pragma unroll
    for (int r = 0; r < RG; r++)
#pragma unroll
        for (int mt = 0; mt < 2; mt++) red[((r * 2 + mt) * nwaves + wave) * 64 + lane] = acc[r][mt];
    __syncthreads();
    const int nn = lane & 15, g = lane >> 4;
    for (int i = wave; i < RO * 2; i += nwaves) {
        const int r = i / 2, mt = i - 2 * r;
        float4v s = red[(i * nwaves) * 64 + lane];
        for (int wv = 1; wv < nwaves; wv++) s += red[(i * nwaves + wv) * 64 + lane];
        float4v s2 = float4v{0.f, 0.f, 0.f, 0.f};
        if constexpr (GU) {
            const int i2 = i + RO * 2;  // the up tile of the pair
            s2 = red[(i2 * nwaves) * 64 + lane];
            for (int wv = 1; wv < nwaves; wv++) s2 += red[(i2 * nwaves + wv) * 64 + lane];
        }
        const int64_t col = (rt0 + r) * 16 + nn;
        if (rt0 + r >= nrt || col >= n) continue;
        const float bv = bias ? bias[col] : 0.0f, bv2 = (GU && bias2) ? bias2[col] : 0.0f;
        if constexpr (GU) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int64_t row = 16 * mt + 4 * g + j;
                if (row >= m) continue;
                const float gate = s[j] + bv, up = s2[j] + bv2;
                turq_store_any(y, yt, row * ldy + col, gate / (1.0f + expf(-gate)) * up);
            }
        } else {
            turq_store_col4(y, yt, 16 * mt + 4 * g, m, ldy, col, s + float4v{bv, bv, bv, bv});
        }
    }
}

// four waves; weights [0, a.second) of format DTA, the others of DTB with staged_second_rows(6) row tiles per workgroup
template <int DTA, int DTB, int XT, int CNT>
__global__ void __launch_bounds__(256) gemv_cs_staged_two_kernel(MultiArgs a, int64_t k, const void *__restrict__ x, int64_t ldx, int64_t m,
                                                                  int yt) {
    const MultiPick p = multi_pick(a, (int)blockIdx.x);
    constexpr int RGB = staged_second_rows(6);
    if (DTA == DTB || p.index < a.second) cs_body_staged_two<DTA, XT, 6, 3, CNT>(p.w, p.n, k, x, ldx, m, p.y, yt, p.ldy, p.bias, (int64_t)p.block);
    else cs_body_staged_two<DTB, XT, RGB, 3, CNT>(p.w, p.n, k, x, ldx, m, p.y, yt, p.ldy, p.bias, (int64_t)p.block);
}

// ... gate (a.w[0]) and up (a.w[1]) of one MLP, three row tiles of each per workgroup, silu(gate) * up stored to a.y[0]
template <int DT, int XT, int CNT>
__global__ void __launch_bounds__(256) gemv_cs_staged_two_gateup_kernel(MultiArgs a, int64_t k, const void *__restrict__ x, int64_t ldx,
                                                                         int64_t m, int yt) {
    cs_body_staged_two<DT, XT, 6, 3, CNT, true>(a.w[0], a.n[0], k, x, ldx, m, a.y[0], yt, a.ldy[0], a.bias[0], (int64_t)blockIdx.x, a.w[1],
                                           a.bias[1]);
}

struct StagedLaunch {
    MultiArgs a;
    int blocks;
    int64_t k;
    const void *x;
    int64_t ldx, m;
    int yt, nwaves;
    hipStream_t s;
    hipEvent_t ev0, ev1;
    bool two;  // the four-wave form for 17 .. 32 rows
    int cnt;   // pairs of column tiles per wave if that is the same number for every wave, else 0
};

// launches `kernel` with lds bytes of dynamic LDS (more than 64 KiB: raised once per kernel)
template <auto kernel>
hipError_t staged_go(size_t lds, const StagedLaunch &l) {
    if (lds > (64u << 10)) {
        const hipError_t raised = turq_raise_lds_limit((const void *)kernel, 144 << 10);
        if (raised != hipSuccess) return raised;
    }
    const dim3 grid((unsigned)l.blocks), block((unsigned)(64 * l.nwaves));
    if (l.ev0) {
        hipExtLaunchKernelGGL(kernel, grid, block, (unsigned)lds, l.s, l.ev0, l.ev1, 0, l.a, l.k, l.x, l.ldx, l.m, l.yt);
        return hipGetLastError();
    }
    kernel<<<grid, block, lds, l.s>>>(l.a, l.k, l.x, l.ldx, l.m, l.yt);
    return hipGetLastError();
}

template <int MR, int RG> size_t staged_lds(int nwaves) {
    constexpr int HV = MR > 16 ? 2 : 1;
    return std::max((size_t)nwaves * (MR / HV) * kXRow, (size_t)nwaves * RG * HV * 64 * sizeof(float4v));
}

// one pair per wave (up to 4096 columns) written out, anything else counted at run time; more than 16 rows are only taken on
// up to 4096 columns
template <int DTA, int DTB, int XT, int MR, int RG>
hipError_t staged_count(const StagedLaunch &l) {
    if (l.cnt == 1) return staged_go<gemv_cs_staged_kernel<DTA, DTB, XT, MR, RG, 1>>(staged_lds<MR, RG>(l.nwaves), l);
    if constexpr (MR <= 16) return staged_go<gemv_cs_staged_kernel<DTA, DTB, XT, MR, RG, 0>>(staged_lds<MR, RG>(l.nwaves), l);
    return hipErrorInvalidValue;
}

template <int DTA, int DTB, int XT, int MR>
hipError_t staged_shape(int rg, const StagedLaunch &l) {
    switch (rg) {
    case 1: return staged_count<DTA, DTB, XT, MR, 1>(l);
    case 2: return staged_count<DTA, DTB, XT, MR, 2>(l);
    case 3:
        if constexpr (MR <= 16) return staged_count<DTA, DTB, XT, MR, 3>(l);
        break;
    case 6:
        if constexpr (MR <= 16) return staged_count<DTA, DTB, XT, MR, 6>(l);
        break;
    }
    return hipErrorInvalidValue;
}

template <int DTA, int DTB, int XT>
hipError_t staged_rows(int rg, const StagedLaunch &l) {
    if (l.two) {
        const size_t lds = std::max((size_t)l.nwaves * 32 * kXRow, (size_t)l.nwaves * 12 * 1024);
        if (rg != 6) return hipErrorInvalidValue;
        return l.cnt == 2 ? staged_go<gemv_cs_staged_two_kernel<DTA, DTB, XT, 2>>(lds, l) : staged_go<gemv_cs_staged_two_kernel<DTA, DTB, XT, 0>>(lds, l);
    }
    if (l.m <= 4) return staged_shape<DTA, DTB, XT, 4>(rg, l);
    if (l.m <= 8) return staged_shape<DTA, DTB, XT, 8>(rg, l);
    if (l.m <= 16) return staged_shape<DTA, DTB, XT, 16>(rg, l);
    return staged_shape<DTA, DTB, XT, 32>(rg, l);
}

template <int DT, int XT, int MR, int RG>
hipError_t staged_gateup_count(const StagedLaunch &l) {
    if (l.cnt == 1) return staged_go<gemv_cs_staged_gateup_kernel<DT, XT, MR, RG, 1>>(staged_lds<MR, RG>(l.nwaves), l);
    return staged_go<gemv_cs_staged_gateup_kernel<DT, XT, MR, RG, 0>>(staged_lds<MR, RG>(l.nwaves), l);
}

// tiles per workgroup (both weights together): 2 or 6; 17 .. 32 rows: 6, four waves
template <int DT, int XT>
hipError_t staged_gateup_shape(int rg, const StagedLaunch &l) {
    if (l.two) {
        const size_t lds = std::max((size_t)l.nwaves * 32 * kXRow, (size_t)l.nwaves * 12 * 1024);
        if (rg != 6) return hipErrorInvalidValue;
        return l.cnt == 2 ? staged_go<gemv_cs_staged_two_gateup_kernel<DT, XT, 2>>(lds, l) : staged_go<gemv_cs_staged_two_gateup_kernel<DT, XT, 0>>(lds, l);
    }
    if (rg == 2) return l.m <= 4 ? staged_gateup_count<DT, XT, 4, 2>(l) : l.m <= 8 ? staged_gateup_count<DT, XT, 8, 2>(l) : staged_gateup_count<DT, XT, 16, 2>(l);
    if (rg == 6) return l.m <= 4 ? staged_gateup_count<DT, XT, 4, 6>(l) : l.m <= 8 ? staged_gateup_count<DT, XT, 8, 6>(l) : staged_gateup_count<DT, XT, 16, 6>(l);
    return hipErrorInvalidValue;
}

}  // namespace

// waves per workgroup of the staged form for this k (0: it does not take it): k a multiple of 512, one pair of column tiles per
// wave and round, at most eight waves
inline int turq_gemv_cs_staged_waves(int64_t k) {
    if (k <= 0 || k % 512 != 0) return 0;
    const int64_t pairs = k / 512;
    return (int)(pairs < 8 ? pairs : 8);
}

// the four-wave form for 17 .. 32 rows (0: not this case): groups of six row tiles
inline int turq_gemv_cs_staged_two_waves(int64_t k, int64_t m, int row_tiles) {
    if (k <= 0 || k % 512 != 0 || m <= 16 || m > 32 || row_tiles != 6) return 0;
    const int64_t pairs = k / 512;
    return (int)(pairs < 4 ? pairs : 4);
}

// the launch for activations of type XT; arguments as turq_launch_gemv_cs_staged, which has checked them
template <int XT>
hipError_t staged_launch(int dtype_a, int dtype_b, int count, int second, const void *const *w, const int64_t *n, int64_t k, const void *x,
                         int64_t ldx, int64_t m, void *const *y, int y_dtype, const int64_t *ldy, const float *const *bias, int row_tiles,
                         hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop) {
    const int two = turq_gemv_cs_staged_two_waves(k, m, row_tiles);
    StagedLaunch l{};
    l.two = two != 0;
    l.nwaves = two ? two : turq_gemv_cs_staged_waves(k);
    l.cnt = (k / 512) % l.nwaves == 0 ? (int)(k / 512 / l.nwaves) : 0;
    int64_t blocks = 0;
    for (int i = 0; i < count; i++) {
        l.a.w[i] = (const uint8_t *)w[i];
        l.a.y[i] = y[i];
        l.a.bias[i] = bias ? bias[i] : nullptr;
        l.a.n[i] = n[i];
        l.a.ldy[i] = ldy ? ldy[i] : n[i];
        l.a.first[i] = (int)blocks;
        const int rt = i < second ? row_tiles : staged_second_rows(row_tiles);
        blocks += (turq_tile_rows(n[i]) + rt - 1) / rt;
    }
    l.a.count = count;
    l.a.second = second;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFF) return hipErrorInvalidValue;
    l.blocks = (int)blocks, l.k = k, l.x = x, l.ldx = ldx, l.m = m, l.yt = y_dtype;
    l.s = stream, l.ev0 = ev_start, l.ev1 = ev_stop;
    if (dtype_a == TURQ_Q4_K && dtype_b == TURQ_Q6_K) return staged_rows<TURQ_Q4_K, TURQ_Q6_K, XT>(row_tiles, l);
    if (dtype_a == TURQ_Q5_K && dtype_b == TURQ_Q6_K) return staged_rows<TURQ_Q5_K, TURQ_Q6_K, XT>(row_tiles, l);
    switch (dtype_a) {
    case TURQ_Q4_K: return staged_rows<TURQ_Q4_K, TURQ_Q4_K, XT>(row_tiles, l);
    case TURQ_Q5_K: return staged_rows<TURQ_Q5_K, TURQ_Q5_K, XT>(row_tiles, l);
    case TURQ_Q6_K: return staged_rows<TURQ_Q6_K, TURQ_Q6_K, XT>(row_tiles, l);
    case TURQ_Q8_0: return staged_rows<TURQ_Q8_0, TURQ_Q8_0, XT>(row_tiles, l);
    default: return hipErrorInvalidValue;
    }
}

// gate and up of one MLP (same format, n and k) with silu(gate) * up stored: tiles per workgroup = 2 * (row tiles of the output)
template <int XT>
hipError_t staged_gateup_launch(int dtype, const void *w_gate, const void *w_up, int64_t n, int64_t k, const void *x, int64_t ldx, int64_t m,
                                void *y, int y_dtype, int64_t ldy, const float *bias_gate, const float *bias_up, int tiles,
                                hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop) {
    const int two = turq_gemv_cs_staged_two_waves(k, m, tiles);
    StagedLaunch l{};
    l.two = two != 0;
    l.nwaves = two ? two : turq_gemv_cs_staged_waves(k);
    l.cnt = (k / 512) % l.nwaves == 0 ? (int)(k / 512 / l.nwaves) : 0;
    l.a.w[0] = (const uint8_t *)w_gate, l.a.w[1] = (const uint8_t *)w_up;
    l.a.bias[0] = bias_gate, l.a.bias[1] = bias_up;
    l.a.y[0] = y, l.a.n[0] = l.a.n[1] = n, l.a.ldy[0] = ldy, l.a.count = 2, l.a.second = 2;
    const int64_t blocks = (turq_tile_rows(n) + tiles / 2 - 1) / (tiles / 2);
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFF) return hipErrorInvalidValue;
    l.blocks = (int)blocks, l.k = k, l.x = x, l.ldx = ldx, l.m = m, l.yt = y_dtype;
    l.s = stream, l.ev0 = ev_start, l.ev1 = ev_stop;
    switch (dtype) {
    case TURQ_Q4_K: return staged_gateup_shape<TURQ_Q4_K, XT>(tiles, l);
    case TURQ_Q5_K: return staged_gateup_shape<TURQ_Q5_K, XT>(tiles, l);
    case TURQ_Q6_K: return staged_gateup_shape<TURQ_Q6_K, XT>(tiles, l);
    case TURQ_Q8_0: return staged_gateup_shape<TURQ_Q8_0, XT>(tiles, l);
    default: return hipErrorInvalidValue;
    }
}

#define TURQ_STAGED_GATEUP_ARGS                                                                                                          \
    int dtype, const void *w_gate, const void *w_up, int64_t n, int64_t k, const void *x, int64_t ldx, int64_t m, void *y, int y_dtype,  \
        int64_t ldy, const float *bias_gate, const float *bias_up, int tiles, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop
#define TURQ_STAGED_GATEUP_PASS dtype, w_gate, w_up, n, k, x, ldx, m, y, y_dtype, ldy, bias_gate, bias_up, tiles, stream, ev_start, ev_stop

#define TURQ_STAGED_LAUNCH_ARGS                                                                                                          \
    int dtype_a, int dtype_b, int count, int second, const void *const *w, const int64_t *n, int64_t k, const void *x, int64_t ldx,      \
        int64_t m, void *const *y, int y_dtype, const int64_t *ldy, const float *const *bias, int row_tiles, hipStream_t stream,         \
        hipEvent_t ev_start, hipEvent_t ev_stop
#define TURQ_STAGED_LAUNCH_PASS dtype_a, dtype_b, count, second, w, n, k, x, ldx, m, y, y_dtype, ldy, bias, row_tiles, stream, ev_start, ev_stop

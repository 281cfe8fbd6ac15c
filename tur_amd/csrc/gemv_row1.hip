// One activation row (decode) against Q4_K / Q5_K weights on the tiled layout.
//
// With a single row fifteen of the sixteen A rows of v_mfma_f32_16x16x32_f16 are idle.  This kernel puts them to
// work as SUB-BLOCK selectors: A row R of MFMA step i holds the activations of the step's 32 columns where they belong
// to sub-block R's slot and zeros elsewhere, so after the eight steps of a 256-column tile the 16 x 16 result holds,
// per weight row n, the eight per-sub-block dot products apart instead of their sum.  That moves the 6-bit sub-block
// scales from the B operand (one v_pk_fma_f16 per two weights in the general kernel) to the result (one multiply-add per
// sub-block and weight row): the B operand is the raw "magic number" f16 (base + nibble), one v_and_or_b32 per two weights
// and nothing else.  The base is taken out through the accumulator: it starts at -sum(base * x) of the sub-block, which
// depends on the activations only.  The result rows that no step writes carry the plain sub-block sums of x for the
// "- dmin * m" term, so a lane finds all four factors of its four 6-bit header fields in its four result registers:
//   result row 4g     = sum over sub-block 2g   of q * x        (field sc[2g])
//   result row 4g + 1 = sum over sub-block 2g   of x            (field m[2g])
//   result row 4g + 2 = sum over sub-block 2g+1 of q * x        (field sc[2g+1])
//   result row 4g + 3 = sum over sub-block 2g+1 of x            (field m[2g+1])
// which is the order of the 24-bit group g of the tile header.  Lane (n, g) adds d * (sc*r0 + sc'*r2) - dmin * (m*r1 + m'*r3)
// to its partial y[n]; the four lane groups and the waves of the workgroup are summed through LDS at the end.
//
// Numerics: products are exact (integers below 2048 times f16), sums in f32.  The base term makes the partial sums about
// 1024 * |x| large where the result is about 30 * |x|, which costs 5 bits of the f32 accumulator: measured rel-L2 against
// the f32 matmul on dequantized weights stays below 3e-5 for bf16 activations.
//
// Per workgroup: one 16-row tile, the waves split the column tiles; every wave converts its own slice of x (256 columns
// per tile) to f16 through its own LDS region and computes the sub-block sums on the way.
#include <hip/hip_ext.h>

#include <cstdlib>

#include "layout.h"
#include "mfma_common.h"

namespace {

constexpr uint32_t kMagic1024 = 0x64006400u;  // 1024.0 in both halves: field at mantissa bit 0
constexpr uint32_t kMagic64 = 0x54005400u;    // 64.0: field at mantissa bit 4
constexpr uint32_t kMagicHdr = 0x64005400u;   // header fields: low half at bit 4 of 64.0, high half at bit 0 of 1024.0

// LDS region of one (wave, tile in flight): 256 f16 of x, 8 x (-base sum, plain sum), 64 bytes of zeros
constexpr int kX = 0, kInit = 512, kZero = 576, kRegion = 640;

template <int DT> struct W1Regs { uint4v qa, qb; uint2v hh; uint32_t hd, grp; };

template <int DT>
__device__ inline W1Regs<DT> load_tile1(const uint8_t *__restrict__ tile, int lane, int grp_off) {
    using F = TiledFmt<DT>;
    W1Regs<DT> w;
    w.qa = *(const uint4v *)(tile + F::kQA + 16 * lane);
    w.qb = *(const uint4v *)(tile + F::kQB + 16 * lane);
    if constexpr (DT == TURQ_Q5_K) w.hh = *(const uint2v *)(tile + F::kQH + 8 * lane);
    else w.hh = uint2v{0u, 0u};
    const uint8_t *h = tile + F::kHDR + 16 * (lane & 15);
    w.hd = *(const uint32_t *)h;                  // f16 d, f16 dmin
    __builtin_memcpy(&w.grp, h + grp_off, 4);     // the (unaligned) dword that holds this lane's 24-bit group
    return w;
}

// raw activations of one tile: 4 consecutive columns per lane, as two packed f16 registers
template <int XT> struct X1Regs { uint32_t r[XT == TURQ_ACT_F32 ? 4 : 2]; };

template <int XT>
__device__ inline X1Regs<XT> load_x1(const void *__restrict__ x, int64_t b, int lane) {
    X1Regs<XT> v;
    const int64_t col = b * 256 + 4 * lane;
    if constexpr (XT == TURQ_ACT_F32) {
        const uint4v t = *(const uint4v *)((const float *)x + col);
        v.r[0] = t.x; v.r[1] = t.y; v.r[2] = t.z; v.r[3] = t.w;
    } else {
        const uint2v t = *(const uint2v *)((const uint16_t *)x + col);
        v.r[0] = t.x; v.r[1] = t.y;
    }
    return v;
}

template <int XT>
__device__ inline void to_half4(const X1Regs<XT> &v, half2v &h01, half2v &h23) {
    if constexpr (XT == TURQ_ACT_F32) {
        h01 = half2v{(_Float16)__uint_as_float(v.r[0]), (_Float16)__uint_as_float(v.r[1])};
        h23 = half2v{(_Float16)__uint_as_float(v.r[2]), (_Float16)__uint_as_float(v.r[3])};
    } else if constexpr (XT == TURQ_ACT_BF16) {
        h01 = half2v{(_Float16)__uint_as_float(v.r[0] << 16), (_Float16)__uint_as_float(v.r[0] & 0xFFFF0000u)};
        h23 = half2v{(_Float16)__uint_as_float(v.r[1] << 16), (_Float16)__uint_as_float(v.r[1] & 0xFFFF0000u)};
    } else {
        h01 = as_half2(v.r[0]);
        h23 = as_half2(v.r[1]);
    }
}

// v + (the same value from the lane `ctrl` points at), inside a row of 16 lanes
template <int CTRL> __device__ inline float dpp_add(float v) {
    const int o = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false);
    return v + __int_as_float(o);
}
// sum over the 8 lanes that share a 32-column sub-block
__device__ inline float sum8(float v) {
    v = dpp_add<0xB1>(v);   // quad_perm [1, 0, 3, 2]
    v = dpp_add<0x4E>(v);   // quad_perm [2, 3, 0, 1]
    v = dpp_add<0x141>(v);  // row_half_mirror: lane i <- lane 7 - i of its half row
    return v;
}

// Stage one tile's activations: f16 values, and per sub-block (-sum(base * x), sum(x)).
// The slots of an MFMA step alternate in pairs between fields at mantissa bit 0 (base 1024) and bit 4 (base 64):
// of a lane's four columns the first two are of the first kind.
template <int XT>
__device__ inline void stage_x1(const X1Regs<XT> &v, uint8_t *region, int lane) {
    half2v h01, h23;
    to_half4<XT>(v, h01, h23);
    *(uint2v *)(region + kX + 8 * lane) = uint2v{as_u32(h01), as_u32(h23)};
    const half2v one = splat2((_Float16)1.0f), b0 = splat2((_Float16)-1024.0f), b1 = splat2((_Float16)-64.0f);
    const float s = sum8(__builtin_amdgcn_fdot2(h23, one, __builtin_amdgcn_fdot2(h01, one, 0.0f, false), false));
    const float nbsum = sum8(__builtin_amdgcn_fdot2(h23, b1, __builtin_amdgcn_fdot2(h01, b0, 0.0f, false), false));
    if ((lane & 7) == 0) *(float2 *)(region + kInit + lane) = float2{nbsum, s};  // sub-block lane / 8 at 8 bytes each
}

// eight raw f16 B values (base + nibble [+ 16 * high bit]) of one step dword
template <bool HIGH>
__device__ inline half8v raw_operand(uint32_t w, uint32_t h0, uint32_t h1, int u0) {
    const uint32_t w8 = w >> 8;
    uint32_t t0 = and_or_u32(w, 0x000F000Fu, kMagic1024);
    uint32_t t1 = and_or_u32(w, 0x00F000F0u, kMagic64);
    uint32_t t2 = and_or_u32(w8, 0x000F000Fu, kMagic1024);
    uint32_t t3 = and_or_u32(w8, 0x00F000F0u, kMagic64);
    if (HIGH) {  // fifth bit: + 16, i.e. mantissa bit 4 next to base 1024 and bit 8 next to base 64
        t0 = and_or_u32(rotr32(h0, (uint32_t)u0), 0x00100010u, t0);
        t1 = and_or_u32(rotr32(h1, (uint32_t)u0), 0x01000100u, t1);
        t2 = and_or_u32(rotr32(h0, (uint32_t)(u0 + 1)), 0x00100010u, t2);
        t3 = and_or_u32(rotr32(h1, (uint32_t)(u0 + 1)), 0x01000100u, t3);
    }
    return make_half8(as_half2(t0), as_half2(t1), as_half2(t2), as_half2(t3));
}

constexpr int kMaxRow1 = 4;
struct Row1Args {
    const uint8_t *w[kMaxRow1];
    void *y[kMaxRow1];
    const float *bias[kMaxRow1];
    int64_t n[kMaxRow1];
    int first[kMaxRow1];
    int count;
};

// P = tiles a wave keeps in flight; MAXT = largest workgroup of the instantiation
template <int DT, int XT, int P, int MAXT>
__global__ void __launch_bounds__(MAXT) gemv_row1_kernel(Row1Args a, int64_t k, const void *__restrict__ x, int yt) {
    extern __shared__ uint8_t smem[];
    constexpr bool HIGH = DT == TURQ_Q5_K;
    constexpr int TB = TiledFmt<DT>::kTileBytes;
    const int blk = (int)blockIdx.x;
    const uint8_t *w = a.w[0];
    void *y = a.y[0];
    const float *bias = a.bias[0];
    int64_t n = a.n[0];
    int first = 0;
#pragma unroll
    for (int i = 1; i < kMaxRow1; i++)
        if (i < a.count && blk >= a.first[i]) { w = a.w[i], y = a.y[i], bias = a.bias[i], n = a.n[i], first = a.first[i]; }
    const int64_t rt = blk - first;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nwaves = blockDim.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int64_t ntc = k / 256;
    uint8_t *region = smem + (size_t)wave * (P * kRegion);
    float *red = (float *)(smem + (size_t)nwaves * (P * kRegion));

    // the zeros that the idle A rows read
    if (lane < 16)
#pragma unroll
        for (int p = 0; p < P; p++) *(uint32_t *)(region + p * kRegion + kZero + 4 * lane) = 0u;
    // A operand: steps 0..3 carry the columns of sub-block 2g into result row 4g, steps 4..7 those of sub-block 2g+1 into
    // row 4g + 2; every other row reads zeros.  Byte offsets inside a region; step i adds 16 * (i % 4).
    const int offA = r == 4 * g ? kX + 128 * g : kZero;
    const int offB = r == 4 * g + 2 ? kX + 128 * g + 64 : kZero;
    // header group g sits at bit 24 g of the 12 bytes after (d, dmin): byte 3 g, except that group 3 is read one byte early
    // so that the load ends with the header.  Rotations that put (sc, sc') / (m, m') on bits 4..9 and 16..21.
    const int grp_off = 4 + 3 * g - (g == 3);
    const uint32_t rot_s = g == 3 ? 4u : 28u, rot_m = g == 3 ? 10u : 2u;

    float acc = 0.0f;
    const uint8_t *wrow = w + rt * ntc * TB;
    for (int64_t b0 = wave; b0 < ntc; b0 += (int64_t)nwaves * P) {
        X1Regs<XT> xr[P];
        W1Regs<DT> wr[P];
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t b = b0 + (int64_t)p * nwaves;
            xr[p] = load_x1<XT>(x, b < ntc ? b : b0, lane);
        }
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t b = b0 + (int64_t)p * nwaves;
            wr[p] = load_tile1<DT>(wrow + (b < ntc ? b : b0) * TB, lane, grp_off);
        }
#pragma unroll
        for (int p = 0; p < P; p++) stage_x1<XT>(xr[p], region + p * kRegion, lane);
        // same-wave LDS traffic is processed in order; the fences keep the compiler from reordering
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t b = b0 + (int64_t)p * nwaves;
            if (b >= ntc) continue;  // uniform per wave
            const uint8_t *reg = region + p * kRegion;
            float4v c = *(const float4v *)(reg + kInit + 16 * g);
            const uint32_t wq[8] = {wr[p].qa.x, wr[p].qa.y, wr[p].qa.z, wr[p].qa.w, wr[p].qb.x, wr[p].qb.y, wr[p].qb.z, wr[p].qb.w};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const half8v av = *(const half8v *)(reg + (i < 4 ? offA : offB) + 16 * (i & 3));
                c = mfma16x16x32(av, raw_operand<HIGH>(wq[i], wr[p].hh.x, wr[p].hh.y, 2 * i), c);
            }
            const half2v kb = {(_Float16)-64.0f, (_Float16)-1024.0f};
            const half2v sc = and_or_h2(rotr32(wr[p].grp, rot_s), 0x003F03F0u, kMagicHdr) + kb;
            const half2v mn = and_or_h2(rotr32(wr[p].grp, rot_m), 0x003F03F0u, kMagicHdr) + kb;
            const half2v dd = as_half2(wr[p].hd);
            const float u = (float)sc.x * c[0] + (float)sc.y * c[2];
            const float v = (float)mn.x * c[1] + (float)mn.y * c[3];
            acc += (float)dd.x * u - (float)dd.y * v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }

    // y[16 rt + n] = sum over lane groups and waves
    red[wave * 64 + lane] = acc;
    __syncthreads();
    if (wave != 0) return;
    const int n4 = lane >> 2, q = lane & 3;
    float s = 0.0f;
    for (int wv = 0; wv < nwaves; wv++) s += red[wv * 64 + n4 + 16 * q];
    s = dpp_add<0xB1>(s);
    s = dpp_add<0x4E>(s);
    const int64_t col = rt * 16 + n4;
    if (q == 0 && col < n) {
        const float out = s + (bias ? bias[col] : 0.0f);
        if (yt == TURQ_ACT_F32) turq_store_out<TURQ_ACT_F32>(y, col, out);
        else if (yt == TURQ_ACT_BF16) turq_store_out<TURQ_ACT_BF16>(y, col, out);
        else turq_store_out<TURQ_ACT_F16>(y, col, out);
    }
}

template <int DT, int XT, int P, int MAXT>
hipError_t launch_final(const Row1Args &a, int blocks, int64_t k, const void *x, int yt, int nwaves, hipStream_t s, hipEvent_t ev0,
                        hipEvent_t ev1) {
    const size_t lds = (size_t)nwaves * P * kRegion + (size_t)nwaves * 64 * sizeof(float);
    if (ev0) {
        hipExtLaunchKernelGGL((gemv_row1_kernel<DT, XT, P, MAXT>), dim3((unsigned)blocks), dim3((unsigned)(64 * nwaves)), (unsigned)lds, s,
                              ev0, ev1, 0, a, k, x, yt);
        return hipGetLastError();
    }
    gemv_row1_kernel<DT, XT, P, MAXT><<<(unsigned)blocks, dim3((unsigned)(64 * nwaves)), lds, s>>>(a, k, x, yt);
    return hipGetLastError();
}

template <int DT, int XT>
hipError_t launch_p(const Row1Args &a, int blocks, int64_t k, const void *x, int yt, int nwaves, hipStream_t s, hipEvent_t ev0,
                    hipEvent_t ev1) {
    static const int forced = [] { const char *e = getenv("TURQ_ROW1_P"); return e ? atoi(e) : 0; }();
    const int64_t per_wave = (k / 256 + nwaves - 1) / nwaves;
    int p = (int)(per_wave < 4 ? per_wave : 4);
    if (forced >= 1 && forced <= 4) p = forced;
    if (p == 1) return launch_final<DT, XT, 1, 1024>(a, blocks, k, x, yt, nwaves, s, ev0, ev1);
    if (p == 2) return launch_final<DT, XT, 2, 1024>(a, blocks, k, x, yt, nwaves, s, ev0, ev1);
    if (p == 3) return launch_final<DT, XT, 3, 1024>(a, blocks, k, x, yt, nwaves, s, ev0, ev1);
    return launch_final<DT, XT, 4, 1024>(a, blocks, k, x, yt, nwaves, s, ev0, ev1);
}

template <int DT>
hipError_t launch_x(int xt, const Row1Args &a, int blocks, int64_t k, const void *x, int yt, int nwaves, hipStream_t s, hipEvent_t ev0,
                    hipEvent_t ev1) {
    switch (xt) {
    case TURQ_ACT_F32: return launch_p<DT, TURQ_ACT_F32>(a, blocks, k, x, yt, nwaves, s, ev0, ev1);
    case TURQ_ACT_BF16: return launch_p<DT, TURQ_ACT_BF16>(a, blocks, k, x, yt, nwaves, s, ev0, ev1);
    case TURQ_ACT_F16: return launch_p<DT, TURQ_ACT_F16>(a, blocks, k, x, yt, nwaves, s, ev0, ev1);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

bool turq_gemv_row1_supports(int dtype) { return dtype == TURQ_Q4_K || dtype == TURQ_Q5_K; }

// count (1..4) weights of one format (Q4_K or Q5_K) and one k against ONE activation row x (16-byte aligned).
hipError_t turq_launch_gemv_row1(int dtype, int count, const void *const *w, const int64_t *n, int64_t k, const void *x, int x_dtype,
                                 void *const *y, int y_dtype, const float *const *bias, int nwaves, hipStream_t stream,
                                 hipEvent_t ev_start, hipEvent_t ev_stop) {
    if (count < 1 || count > kMaxRow1 || nwaves < 1 || nwaves > 16 || k % 256 != 0) return hipErrorInvalidValue;
    if (y_dtype != TURQ_ACT_F32 && y_dtype != TURQ_ACT_BF16 && y_dtype != TURQ_ACT_F16) return hipErrorInvalidValue;
    Row1Args a{};
    int64_t blocks = 0;
    for (int i = 0; i < count; i++) {
        a.w[i] = (const uint8_t *)w[i];
        a.y[i] = y[i];
        a.bias[i] = bias ? bias[i] : nullptr;
        a.n[i] = n[i];
        a.first[i] = (int)blocks;
        blocks += turq_tile_rows(n[i]);
    }
    a.count = count;
    if (blocks == 0 || k == 0) return blocks == 0 ? hipSuccess : hipErrorInvalidValue;
    if (blocks > 0x7FFFFFFF) return hipErrorInvalidValue;
    switch (dtype) {
    case TURQ_Q4_K: return launch_x<TURQ_Q4_K>(x_dtype, a, (int)blocks, k, x, y_dtype, nwaves, stream, ev_start, ev_stop);
    case TURQ_Q5_K: return launch_x<TURQ_Q5_K>(x_dtype, a, (int)blocks, k, x, y_dtype, nwaves, stream, ev_start, ev_stop);
    default: return hipErrorInvalidValue;
    }
}

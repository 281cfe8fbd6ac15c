// One activation row (decode) against quantized weights on the tiled layout.
//
// With a single row fifteen of the sixteen A rows of v_mfma_f32_16x16x32_f16 are idle.  This kernel puts them to
// work as SUB-BLOCK selectors: A row R of an MFMA step holds the activations of the step's 32 columns where they belong
// to the sub-block that result row R stands for and zeros elsewhere, so after the eight steps of a 256-column tile the
// 16 x 16 result holds, per weight row n, the per-sub-block dot products apart instead of their sum.  That moves the
// sub-block scales from the B operand (one v_pk_fma_f16 per two weights in the general kernel) to the result (one
// multiply-add per sub-block and weight row): the B operand is the raw "magic number" f16 (base + quant), one or two
// v_and_or_b32 per two weights and nothing else.  The base (and the format's zero point) is taken out through the
// accumulator: it starts at -sum(base * x) over the sub-block, which depends on the activations only.
//
//   Q4_K / Q5_K  8 sub-blocks of 32.  Result rows 4g, 4g + 2 collect sub-blocks 2g, 2g + 1; rows 4g + 1, 4g + 3 are
//                written by no step and carry the plain sums of x over those sub-blocks for the "- dmin * m" term.  A
//                lane's four result registers thus meet the four 6-bit fields (sc, m, sc', m') of header group g:
//                lane (n, g) adds d * (sc * r0 + sc' * r2) - dmin * (m * r1 + m' * r3) to its partial y[n].
//   Q6_K         16 sub-blocks of 16, result row = sub-block: lane (n, g) holds sub-blocks 4g .. 4g + 3, whose int8
//                scales are the dword it loads from the tile's scale plane.  Zero point 32: base 256 + 32.
//   Q8_0         8 blocks of 32, result row = block (rows 8 .. 15 stay zero), f16 scale per block.  The tile stores
//                the bytes offset by 128: base 1024 + 128.
// The four lane groups and the waves of the workgroup are summed through LDS at the end.
//
// Numerics: products are exact (integers below 2048 times f16), sums in f32.  The base term makes the partial sums
// up to 1024 * |x| large where the result is about 30 * |x|; measured rel-L2 against the f32 matmul on dequantized
// weights with the same f16-rounded activations stays below 2e-5.
//
// Per workgroup: one 16-row tile, the waves split the column tiles; every wave converts its own slice of x (256 columns
// per tile) to f16 through its own LDS region and computes the sub-block sums on the way.
#include <hip/hip_ext.h>

#include <cstdlib>

#include <algorithm>

#include "layout.h"
#include "mfma_common.h"

namespace {

constexpr uint32_t kMagic1024 = 0x64006400u;  // 1024.0 in both halves: field at mantissa bit 0
constexpr uint32_t kMagic256 = 0x5C005C00u;   // 256.0: field at mantissa bit 2
constexpr uint32_t kMagic64 = 0x54005400u;    // 64.0: field at mantissa bit 4
constexpr uint32_t kMagicHdr = 0x64005400u;   // header fields: low half at bit 4 of 64.0, high half at bit 0 of 1024.0

// LDS region of one (wave, tile in flight): 256 f16 of x, 16 floats the accumulator starts from, 64 bytes of zeros
constexpr int kX = 0, kInit = 512, kZero = 576, kRegion = 640;
// LDS region of one (wave, tile in flight, PAIR of activation rows) in the packed form, where the sixteen A rows of an MFMA are
// eight sub-blocks x two activation rows: 2 x 256 f16 of x, 16 start values, 16 sums of x (for the mins), 64 bytes of zeros
constexpr int kPX = 0, kPInit = 1024, kPSum = 1088, kPZero = 1152, kPairRegion = 1216;

// v + (the same value from the lane `CTRL` points at), inside a row of 16 lanes
template <int CTRL> __device__ inline float dpp_add(float v) {
    const int o = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false);
    return v + __int_as_float(o);
}
__device__ inline float sum4(float v) {
    v = dpp_add<0xB1>(v);  // quad_perm [1, 0, 3, 2]
    return dpp_add<0x4E>(v);  // quad_perm [2, 3, 0, 1]
}
// row_half_mirror: lane i <- lane 7 - i of its half row.  The result is pinned here: the callers store it from one lane in eight,
// and an add that the compiler sinks into that branch no longer merges with its DPP move.
__device__ inline float sum8(float v) {
    float r = dpp_add<0x141>(sum4(v));
    asm volatile("" : "+v"(r));
    return r;
}

__device__ inline float dot2(half2v a, _Float16 b0, float c) { return __builtin_amdgcn_fdot2(a, splat2(b0), c, false); }

// raw activations of one tile: 4 consecutive columns per lane
template <int XT> struct X1Regs { uint32_t r[XT == TURQ_ACT_F32 ? 4 : 2]; };

// RAGGED: k may end inside the tile (Q8_0: a multiple of 32, four columns are in or out together); the K-quants' k is a
// multiple of 256 and needs no test
template <int XT, bool RAGGED>
__device__ inline X1Regs<XT> load_x1(const void *__restrict__ x, int64_t k, int64_t b, int lane, const GOff &o) {
    // x: the activation row (wave-uniform pointer)
    X1Regs<XT> v;
    constexpr int ES = XT == TURQ_ACT_F32 ? 4 : 2;
    const bool ok = !RAGGED || b * 256 + 4 * lane < k;
    const uint32_t off = XT == TURQ_ACT_F32 ? o.o16 : o.o8;
    const uint8_t *src = (const uint8_t *)x + b * (256 * ES) + (ok ? off : 0u);
    if (RAGGED && !ok) src = (const uint8_t *)x;
    if constexpr (XT == TURQ_ACT_F32) {
        const uint4v t = *(const uint4v *)src;
        v.r[0] = ok ? t.x : 0u; v.r[1] = ok ? t.y : 0u; v.r[2] = ok ? t.z : 0u; v.r[3] = ok ? t.w : 0u;
    } else {
        const uint2v t = *(const uint2v *)src;
        v.r[0] = ok ? t.x : 0u; v.r[1] = ok ? t.y : 0u;
    }
    return v;
}

template <int XT>
__device__ inline void to_half4(const X1Regs<XT> &v, half2v &h01, half2v &h23) {
    if constexpr (XT == TURQ_ACT_F32) {
        h01 = __builtin_convertvector(float2v{__uint_as_float(v.r[0]), __uint_as_float(v.r[1])}, half2v);
        h23 = __builtin_convertvector(float2v{__uint_as_float(v.r[2]), __uint_as_float(v.r[3])}, half2v);
    } else if constexpr (XT == TURQ_ACT_BF16) {
        h01 = half2v{(_Float16)__uint_as_float(v.r[0] << 16), (_Float16)__uint_as_float(v.r[0] & 0xFFFF0000u)};
        h23 = half2v{(_Float16)__uint_as_float(v.r[1] << 16), (_Float16)__uint_as_float(v.r[1] & 0xFFFF0000u)};
    } else {
        h01 = as_half2(v.r[0]);
        h23 = as_half2(v.r[1]);
    }
}

// ---- per-format pieces ----
//   Lane:   per-lane constants (LDS offsets of the A operand, header addressing)
//   W:      what a lane loads from HBM for one tile
//   sums(): what the accumulator starts from, from a lane's four staged columns (h01, h23), written to region + kInit
//   chain(): the eight MFMA steps of a tile;  scales(): the tile's scale factors;
//   finish(): the scales on the result of the chain = the lane's contribution to its partial y
template <int DT> struct Row1Fmt;

template <int DT> struct Row1K45 {
    static constexpr bool HIGH = DT == TURQ_Q5_K;
    using F = TiledFmt<DT>;
    struct Lane {
        int offA, offB;   // steps 0..3 feed result row 4g (sub-block 2g), steps 4..7 row 4g + 2; other rows read zeros
        uint32_t rot_s, rot_m;  // rotations that put (sc, sc') / (m, m') of the lane's header group on bits 4..9 and 16..21
    };
    struct W { uint4v qa, qb; uint2v hh; uint32_t hd, grp; };
    __device__ static Lane lane_init(int r, int g) {
        Lane l;
        l.offA = r == 4 * g ? kX + 128 * g : kZero;
        l.offB = r == 4 * g + 2 ? kX + 128 * g + 64 : kZero;
        l.rot_s = g == 3 ? 4u : 28u;
        l.rot_m = g == 3 ? 10u : 2u;
        return l;
    }
    // header group g sits at bit 24 g of the 12 bytes after (d, dmin) = byte 3 g; group 3 is read one byte early so that the
    // load ends with the header
    __device__ static uint32_t aux_off(int r, int g) { return 16u * (uint32_t)r + 4u + 3u * (uint32_t)g - (g == 3 ? 1u : 0u); }
    // (non-temporal loads for everything that is read once per launch: see load_tile in gemv_tileop.h)
    __device__ static W load(const uint8_t *__restrict__ tile, const GOff &o) {
        W w;
        w.qa = __builtin_nontemporal_load((const uint4v *)(tile + F::kQA + o.o16));
        w.qb = __builtin_nontemporal_load((const uint4v *)(tile + F::kQB + o.o16));
        if constexpr (HIGH) w.hh = __builtin_nontemporal_load((const uint2v *)(tile + F::kQH + o.o8));
        else w.hh = uint2v{0u, 0u};
        w.hd = __builtin_nontemporal_load((const uint32_t *)(tile + F::kHDR + o.hdr));  // f16 d, f16 dmin
        __builtin_memcpy(&w.grp, tile + F::kHDR + o.aux, 4);  // the (unaligned) dword that holds this lane's 24-bit group
        return w;
    }
    // The slots of a step alternate in pairs between fields at mantissa bit 0 (base 1024) and bit 4 (base 64): of a lane's
    // four columns the first two are of the first kind.  Per sub-block (8 lanes): (-sum(base * x), sum(x)).
    __device__ static void sums(half2v h01, half2v h23, uint8_t *region, int lane) {
        const float s = sum8(dot2(h23, (_Float16)1.0f, dot2(h01, (_Float16)1.0f, 0.0f)));
        const float nb = sum8(dot2(h23, (_Float16)-64.0f, dot2(h01, (_Float16)-1024.0f, 0.0f)));
        if ((lane & 7) == 0) *(float2 *)(region + kInit + lane) = float2{nb, s};
    }
    __device__ static half8v operand(uint32_t w, uint32_t h0, uint32_t h1, int u0) {
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
    // M activation rows: their regions follow each other; every operand is unpacked once and used for all of them
    template <int M> __device__ static void chain(const W &w, const uint8_t *reg, const Lane &l, int g, float4v *c) {
#pragma unroll
        for (int mm = 0; mm < M; mm++) c[mm] = *(const float4v *)(reg + mm * kRegion + kInit + 16 * g);
        const uint32_t wq[8] = {w.qa.x, w.qa.y, w.qa.z, w.qa.w, w.qb.x, w.qb.y, w.qb.z, w.qb.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const half8v bop = operand(wq[i], w.hh.x, w.hh.y, 2 * i);
#pragma unroll
            for (int mm = 0; mm < M; mm++) {
                const half8v av = *(const half8v *)(reg + mm * kRegion + (i < 4 ? l.offA : l.offB) + 16 * (i & 3));
                c[mm] = mfma16x16x32(av, bop, c[mm]);
            }
        }
    }
    // ---- packed form: two activation rows per chain.  A row R = 4 g' + 2 s + a carries sub-block 2 g' + s of activation row
    // a of the pair, so lane (n, g) of the result finds (sub-block 2g, row 0), (2g, row 1), (2g + 1, row 0), (2g + 1, row 1) in
    // its four registers; no row is left for sum(x), which the staging keeps in the LDS instead (kPSum, same index).
    static constexpr bool kPacked = true;
    struct LanePK { int offA, offB; };
    __device__ static LanePK lane_init_pk(int r, int g) {
        const int gq = r >> 2, s = (r >> 1) & 1, a = r & 1;
        LanePK l;
        l.offA = (g == gq && s == 0) ? kPX + 512 * a + 128 * g : kPZero;
        l.offB = (g == gq && s == 1) ? kPX + 512 * a + 128 * g + 64 : kPZero;
        return l;
    }
    __device__ static void sums_pk(half2v h01, half2v h23, uint8_t *pr, int lane, int a) {
        const float s = sum8(dot2(h23, (_Float16)1.0f, dot2(h01, (_Float16)1.0f, 0.0f)));
        const float nb = sum8(dot2(h23, (_Float16)-64.0f, dot2(h01, (_Float16)-1024.0f, 0.0f)));
        if ((lane & 7) == 0) {
            const int at = 4 * (2 * (lane >> 3) + a);  // sub-block lane / 8
            *(float *)(pr + kPInit + at) = nb;
            *(float *)(pr + kPSum + at) = s;
        }
    }
    template <int NP> __device__ static void chain_pk(const W &w, const uint8_t *pr, const LanePK &l, int g, float4v *c) {
#pragma unroll
        for (int np = 0; np < NP; np++) c[np] = *(const float4v *)(pr + np * kPairRegion + kPInit + 16 * g);
        const uint32_t wq[8] = {w.qa.x, w.qa.y, w.qa.z, w.qa.w, w.qb.x, w.qb.y, w.qb.z, w.qb.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const half8v bop = operand(wq[i], w.hh.x, w.hh.y, 2 * i);
#pragma unroll
            for (int np = 0; np < NP; np++) {
                const half8v av = *(const half8v *)(pr + np * kPairRegion + (i < 4 ? l.offA : l.offB) + 16 * (i & 3));
                c[np] = mfma16x16x32(av, bop, c[np]);
            }
        }
    }
    struct Sc { half2v sc, mn, dd; };  // (sc, sc'), (m, m'), (d, dmin)
    __device__ static Sc scales(const W &w, const Lane &l) {
        const half2v kb = {(_Float16)-64.0f, (_Float16)-1024.0f};
        Sc s;
        s.sc = and_or_h2(rotr32(w.grp, l.rot_s), 0x003F03F0u, kMagicHdr) + kb;
        s.mn = and_or_h2(rotr32(w.grp, l.rot_m), 0x003F03F0u, kMagicHdr) + kb;
        s.dd = as_half2(w.hd);
        return s;
    }
    __device__ static float finish(const Sc &s, const float4v &c) {
        const float u = (float)s.sc.x * c[0] + (float)s.sc.y * c[2];
        const float v = (float)s.mn.x * c[1] + (float)s.mn.y * c[3];
        return (float)s.dd.x * u - (float)s.dd.y * v;
    }
    // sx: the sums of x in the order of c
    __device__ static void finish_pk(const Sc &s, const float4v &c, const float4v &sx, float &y0, float &y1) {
        const float sc0 = (float)s.sc.x, sc1 = (float)s.sc.y, m0 = (float)s.mn.x, m1 = (float)s.mn.y;
        const float d = (float)s.dd.x, dmin = (float)s.dd.y;
        y0 += d * (sc0 * c[0] + sc1 * c[2]) - dmin * (m0 * sx[0] + m1 * sx[2]);
        y1 += d * (sc0 * c[1] + sc1 * c[3]) - dmin * (m0 * sx[1] + m1 * sx[3]);
    }
};
template <> struct Row1Fmt<TURQ_Q4_K> : Row1K45<TURQ_Q4_K> {};
template <> struct Row1Fmt<TURQ_Q5_K> : Row1K45<TURQ_Q5_K> {};

template <> struct Row1Fmt<TURQ_Q6_K> {
    using F = TiledFmt<TURQ_Q6_K>;
    struct Lane { int off[4]; };  // steps 2s, 2s + 1 feed result row 4g + s (sub-block 4g + s)
    static constexpr bool kPacked = false;  // no packed form: rows are handled one MFMA chain each
    struct W { uint4v qla, qlb, qh; uint32_t scw, d16; };
    __device__ static Lane lane_init(int r, int g) {
        Lane l;
#pragma unroll
        for (int s = 0; s < 4; s++) l.off[s] = r == 4 * g + s ? kX + 128 * g + 32 * s : kZero;
        return l;
    }
    __device__ static uint32_t aux_off(int r, int) { return 2u * (uint32_t)r; }  // the row's d
    __device__ static W load(const uint8_t *__restrict__ tile, const GOff &o) {
        W w;
        w.qla = __builtin_nontemporal_load((const uint4v *)(tile + F::kQLA + o.o16));
        w.qlb = __builtin_nontemporal_load((const uint4v *)(tile + F::kQLB + o.o16));
        w.qh = __builtin_nontemporal_load((const uint4v *)(tile + F::kQH + o.o16));
        w.scw = __builtin_nontemporal_load((const uint32_t *)(tile + F::kSC + o.o4));
        w.d16 = __builtin_nontemporal_load((const uint16_t *)(tile + F::kD + o.aux));
        return w;
    }
    // every value is built in the mantissa of 256.0 and stands for q - 32: per sub-block (4 lanes) -288 * sum(x)
    __device__ static void sums(half2v h01, half2v h23, uint8_t *region, int lane) {
        const float nb = sum4(dot2(h23, (_Float16)-288.0f, dot2(h01, (_Float16)-288.0f, 0.0f)));
        if ((lane & 3) == 0) *(float *)(region + kInit + lane) = nb;
    }
    template <int M> __device__ static void chain(const W &w, const uint8_t *reg, const Lane &l, int g, float4v *c) {
#pragma unroll
        for (int mm = 0; mm < M; mm++) c[mm] = *(const float4v *)(reg + mm * kRegion + kInit + 16 * g);
        const uint32_t wl[8] = {w.qla.x, w.qla.y, w.qla.z, w.qla.w, w.qlb.x, w.qlb.y, w.qlb.z, w.qlb.w};
        const uint32_t wh[4] = {w.qh.x, w.qh.y, w.qh.z, w.qh.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            // pair t of the step: the nibbles sit 4 t bits above mantissa bits 2..5, the two high bits 2 t + 8 (i % 2)
            // bits above mantissa bits 6..7; together the 6-bit quant in the mantissa of 256.0 (ulp 1/4)
            uint32_t v[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const uint32_t lo = t ? rotr32(wl[i], 4u * t) : wl[i];
                const uint32_t rh = 2u * t + 8u * (i & 1);
                const uint32_t hi = rh ? rotr32(wh[i >> 1], rh) : wh[i >> 1];
                v[t] = and_or_u32(hi, 0x00C000C0u, and_or_u32(lo, 0x003C003Cu, kMagic256));
            }
            const half8v bop = make_half8(as_half2(v[0]), as_half2(v[1]), as_half2(v[2]), as_half2(v[3]));
#pragma unroll
            for (int mm = 0; mm < M; mm++) {
                const half8v av = *(const half8v *)(reg + mm * kRegion + l.off[i >> 1] + 16 * (i & 1));
                c[mm] = mfma16x16x32(av, bop, c[mm]);
            }
        }
    }
    struct Sc { float s[4]; float d; };
    __device__ static Sc scales(const W &w, const Lane &) {
        Sc s;
#pragma unroll
        for (int i = 0; i < 4; i++) s.s[i] = (float)(int)(int8_t)(w.scw >> (8 * i));
        _Float16 d;
        const uint16_t db = (uint16_t)w.d16;
        __builtin_memcpy(&d, &db, 2);
        s.d = (float)d;
        return s;
    }
    __device__ static float finish(const Sc &s, const float4v &c) {
        return s.d * ((s.s[0] * c[0] + s.s[1] * c[1]) + (s.s[2] * c[2] + s.s[3] * c[3]));
    }
};

template <> struct Row1Fmt<TURQ_Q8_0> {
    using F = TiledFmt<TURQ_Q8_0>;
    struct Lane { int off[8]; };  // step q feeds result row q (block q); rows 8..15 stay zero
    static constexpr bool kPacked = false;  // no packed form: rows are handled one MFMA chain each
    struct W { uint4v p[4]; uint2v dd; };
    __device__ static Lane lane_init(int r, int g) {
        Lane l;
#pragma unroll
        for (int q = 0; q < 8; q++) l.off[q] = r == q ? kX + 64 * q + 16 * g : kZero;
        return l;
    }
    // the four block scales that belong to result rows 4 (g % 2) .. 4 (g % 2) + 3
    __device__ static uint32_t aux_off(int r, int g) { return (uint32_t)F::kD + 16u * (uint32_t)r + 8u * (uint32_t)(g & 1); }
    __device__ static W load(const uint8_t *__restrict__ tile, const GOff &o) {
        W w;
#pragma unroll
        for (int i = 0; i < 4; i++) w.p[i] = __builtin_nontemporal_load((const uint4v *)(tile + 1024 * i + o.o16));
        w.dd = __builtin_nontemporal_load((const uint2v *)(tile + o.aux));
        return w;
    }
    // bytes are stored as q + 128 and unpacked into the mantissa of 1024.0: per block (8 lanes) -1152 * sum(x).
    // Lane groups 2 and 3 read the second half of the init area, which stays zero.
    __device__ static void sums(half2v h01, half2v h23, uint8_t *region, int lane) {
        const float nb = sum8(dot2(h23, (_Float16)-1152.0f, dot2(h01, (_Float16)-1152.0f, 0.0f)));
        if ((lane & 7) == 0) *(float *)(region + kInit + (lane >> 1)) = nb;
    }
    template <int M> __device__ static void chain(const W &w, const uint8_t *reg, const Lane &l, int g, float4v *c) {
#pragma unroll
        for (int mm = 0; mm < M; mm++) c[mm] = *(const float4v *)(reg + mm * kRegion + kInit + 16 * g);
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const uint32_t w0 = (q & 1) ? w.p[q >> 1].z : w.p[q >> 1].x;
            const uint32_t w1 = (q & 1) ? w.p[q >> 1].w : w.p[q >> 1].y;
            const half8v bop = make_half8(as_half2(and_or_u32(w0, 0x00FF00FFu, kMagic1024)), as_half2(and_or_u32(w0 >> 8, 0x00FF00FFu, kMagic1024)),
                                          as_half2(and_or_u32(w1, 0x00FF00FFu, kMagic1024)), as_half2(and_or_u32(w1 >> 8, 0x00FF00FFu, kMagic1024)));
#pragma unroll
            for (int mm = 0; mm < M; mm++) {
                const half8v av = *(const half8v *)(reg + mm * kRegion + l.off[q]);
                c[mm] = mfma16x16x32(av, bop, c[mm]);
            }
        }
    }
    struct Sc { half2v d01, d23; };
    __device__ static Sc scales(const W &w, const Lane &) { return Sc{as_half2(w.dd.x), as_half2(w.dd.y)}; }
    __device__ static float finish(const Sc &s, const float4v &c) {
        return ((float)s.d01.x * c[0] + (float)s.d01.y * c[1]) + ((float)s.d23.x * c[2] + (float)s.d23.y * c[3]);
    }
};

// Stage one tile's activations: f16 values at kX, the accumulator start values at kInit.
template <int DT, int XT>
__device__ inline void stage_x1(const X1Regs<XT> &v, uint8_t *region, int lane) {
    half2v h01, h23;
    to_half4<XT>(v, h01, h23);
    *(uint2v *)(region + kX + 8 * lane) = uint2v{as_u32(h01), as_u32(h23)};
    Row1Fmt<DT>::sums(h01, h23, region, lane);
}

constexpr int kMaxRow1 = 4;
struct Row1Args {
    const uint8_t *w[kMaxRow1];
    void *y[kMaxRow1];
    const float *bias[kMaxRow1];
    int64_t n[kMaxRow1], ldy[kMaxRow1];
    int first[kMaxRow1];
    int count;
    int second;  // two-format launches: weights [0, second) are of the first format, [second, count) of the second
};

// the work of one workgroup: row tiles rtb * R .. rtb * R + R - 1 of one weight, against m <= M activation rows.
// P = column tiles a wave keeps in flight; R = row tiles per workgroup (a wave stages the activations of a column tile once and
// uses them for R weight tiles); M = activation rows the instantiation holds (rows past m repeat row 0 and are not stored)
// GU (R = 2): the two "row tiles" are row tile rtb of a gate weight (w) and of an up weight (w2) of the same shape, and
// what is stored is act(gate) * up (src/models/qwen3.rs:161-167 computes that product from the two projections' outputs)
// NORM (M = 1): the activation row is RmsNorm(x) with weight gw (src/models/layers/norm.rs:81-93, applied in front of q / k / v,
// gate / up and the LM head): a lane multiplies its columns by gw when it stages them and adds up their squares, and the row's
// 1 / sqrt(mean(x^2) + eps), which is the same for every column, multiplies the results - the separate launch of the norm and
// the round trip of its output go away.
template <int DT, int XT, int P, int R, int M, bool GU = false, bool NORM = false, bool ACC = false>
__device__ __forceinline__ void row1_body(const uint8_t *__restrict__ w, void *__restrict__ y, int64_t ldy, const float *__restrict__ bias,
                                          int64_t n, int64_t rtb, int64_t k, const void *__restrict__ x, int64_t ldx, int m, int yt,
                                          const uint8_t *__restrict__ w2 = nullptr, const float *__restrict__ bias2 = nullptr,
                                          const float *__restrict__ gw = nullptr, float eps = 0.0f) {
    static_assert(!GU || R == 2, "gate and up take the places of two row tiles");
    static_assert(!NORM || M == 1, "the norm is taken into the kernel for one activation row");
    extern __shared__ uint8_t smem[];
    using Fmt = Row1Fmt<DT>;
    constexpr int TB = TiledFmt<DT>::kTileBytes;
    constexpr int ES = XT == TURQ_ACT_F32 ? 4 : 2;
    const int64_t rt0 = GU ? rtb : rtb * R, nrt = turq_tile_rows(n);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nwaves = blockDim.x >> 6;
    const int g = lane >> 4;
    const int64_t ntc = turq_tile_cols(k);
    // several rows of a format that has the packed form: two rows per MFMA chain, regions per pair of rows
    constexpr bool PK = Fmt::kPacked && M > 1;
    constexpr int NP = M / 2;
    constexpr int PSTRIDE = PK ? NP * kPairRegion : M * kRegion;  // LDS of one tile in flight
    static_assert(!PK || M % 2 == 0, "packed pairs");
    uint8_t *region = smem + (size_t)wave * (P * PSTRIDE);  // [p][activation row] or [p][pair]
    float *red = (float *)(smem + (size_t)nwaves * (P * PSTRIDE));
    float *red_ss = red + (size_t)nwaves * (R * M * 64);  // NORM: a sum of squares per wave
    float ss = 0.0f;

    // the zeros that the idle A rows read, and start values that no format overwrites
    if constexpr (PK) {
        if (lane < 48)
#pragma unroll
            for (int p = 0; p < P * NP; p++) *(float *)(region + p * kPairRegion + kPInit + 4 * lane) = 0.0f;
    } else {
        if (lane < 32)
#pragma unroll
            for (int p = 0; p < P * M; p++) *(float *)(region + p * kRegion + kInit + 4 * lane) = 0.0f;  // float like the later writes
    }
    const typename Fmt::Lane lc = Fmt::lane_init(lane & 15, g);
    GOff go{16u * (uint32_t)lane, 8u * (uint32_t)lane, 4u * (uint32_t)lane, 16u * (uint32_t)(lane & 15), Fmt::aux_off(lane & 15, g), 0u};

    float acc[R][M];
    const uint8_t *wrow[R];  // row tiles past the weight's last one re-read it; their results are not stored
    const uint8_t *xrow[M];
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int mm = 0; mm < M; mm++) acc[r][mm] = 0.0f;
        if constexpr (GU) wrow[r] = (r == 0 ? w : w2) + rt0 * ntc * TB;
        else wrow[r] = w + (rt0 + r < nrt ? rt0 + r : nrt - 1) * ntc * TB;
    }
#pragma unroll
    for (int mm = 0; mm < M; mm++) xrow[mm] = (const uint8_t *)x + (mm < m ? mm : 0) * ldx * ES;
    // ACC (TURQ_OUT_ACCUMULATE in yt; an instantiation of its own, since even the untaken branch cost the plain launches 2 %):
    // the element this lane will add its first result to, requested now so that it has long arrived when the sums are done (a
    // load at the end of the kernel is a whole memory round trip on the critical path)
    float old_first = 0.0f;
    if constexpr (ACC && !GU) {
        if (wave < R * M) {
            const int r = wave / M, mm = wave - r * M;
            const int64_t col = (rt0 + r) * 16 + (lane >> 2);
            if ((lane & 3) == 0 && rt0 + r < nrt && col < n && mm < m) {
                const int64_t at = (int64_t)mm * ldy + col;
                const int base = yt & 0xFF;
                old_first = base == TURQ_ACT_F32 ? turq_load_out<TURQ_ACT_F32>(y, at) : base == TURQ_ACT_BF16 ? turq_load_out<TURQ_ACT_BF16>(y, at) : turq_load_out<TURQ_ACT_F16>(y, at);
            }
        }
    }
    for (int64_t b0 = wave; b0 < ntc; b0 += (int64_t)nwaves * P) {
        X1Regs<XT> xr[P][M];
        float4v gv[NORM ? P : 1];
        typename Fmt::W wr[P][R];
        go.touch();
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t b = b0 + (int64_t)p * nwaves;
#pragma unroll
            for (int mm = 0; mm < M; mm++) xr[p][mm] = load_x1<XT, DT == TURQ_Q8_0>(xrow[mm], k, b < ntc ? b : b0, lane, go);
            if constexpr (NORM) {
                const int64_t bb = b < ntc ? b : b0;
                const bool ok = DT != TURQ_Q8_0 || bb * 256 + 4 * lane < k;  // (Q8_0: k may end inside the tile; the columns are zeros then)
                gv[p] = *(const float4v *)(gw + (ok ? bb * 256 + 4 * lane : 0));
            }
        }
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t b = b0 + (int64_t)p * nwaves;
#pragma unroll
            for (int r = 0; r < R; r++) wr[p][r] = Fmt::load(wrow[r] + (b < ntc ? b : b0) * TB, go);
        }
#pragma unroll
        for (int p = 0; p < P; p++)
#pragma unroll
            for (int mm = 0; mm < M; mm++) {
                if constexpr (PK) {
                    uint8_t *pr = region + p * PSTRIDE + (mm >> 1) * kPairRegion;
                    half2v h01, h23;
                    to_half4<XT>(xr[p][mm], h01, h23);
                    *(uint2v *)(pr + kPX + 512 * (mm & 1) + 8 * lane) = uint2v{as_u32(h01), as_u32(h23)};
                    Fmt::sums_pk(h01, h23, pr, lane, mm & 1);
                } else if constexpr (NORM) {
                    float f[4];
                    if constexpr (XT == TURQ_ACT_F32) {
#pragma unroll
                        for (int e = 0; e < 4; e++) f[e] = __uint_as_float(xr[p][mm].r[e]);
                    } else if constexpr (XT == TURQ_ACT_BF16) {
                        f[0] = __uint_as_float(xr[p][mm].r[0] << 16), f[1] = __uint_as_float(xr[p][mm].r[0] & 0xFFFF0000u);
                        f[2] = __uint_as_float(xr[p][mm].r[1] << 16), f[3] = __uint_as_float(xr[p][mm].r[1] & 0xFFFF0000u);
                    } else {
                        const half2v a = as_half2(xr[p][mm].r[0]), c = as_half2(xr[p][mm].r[1]);
                        f[0] = (float)a.x, f[1] = (float)a.y, f[2] = (float)c.x, f[3] = (float)c.y;
                    }
                    if (b0 + (int64_t)p * nwaves < ntc) ss += (f[0] * f[0] + f[1] * f[1]) + (f[2] * f[2] + f[3] * f[3]);  // (a tile past the end repeats another)
                    const half2v h01 = __builtin_convertvector(float2v{f[0] * gv[p].x, f[1] * gv[p].y}, half2v);
                    const half2v h23 = __builtin_convertvector(float2v{f[2] * gv[p].z, f[3] * gv[p].w}, half2v);
                    uint8_t *rg = region + p * PSTRIDE + mm * kRegion;
                    *(uint2v *)(rg + kX + 8 * lane) = uint2v{as_u32(h01), as_u32(h23)};
                    Fmt::sums(h01, h23, rg, lane);
                } else {
                    stage_x1<DT, XT>(xr[p][mm], region + p * PSTRIDE + mm * kRegion, lane);
                }
            }
        // same-wave LDS traffic is processed in order; the fences keep the compiler from reordering
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int64_t b = b0 + (int64_t)p * nwaves;
            if (b >= ntc) continue;  // uniform per wave
#pragma unroll
            for (int r = 0; r < R; r++) {
                if constexpr (PK) {
                    const typename Fmt::LanePK lpk = Fmt::lane_init_pk(lane & 15, g);
                    float4v c[NP];
                    Fmt::template chain_pk<NP>(wr[p][r], region + p * PSTRIDE, lpk, g, c);
#pragma unroll
                    for (int np = 0; np < NP; np++) asm volatile("" : "+v"(c[np]));
                    __builtin_amdgcn_sched_barrier(0x10 | 0x80 | 0x4);
                    const typename Fmt::Sc sc = Fmt::scales(wr[p][r], lc);
#pragma unroll
                    for (int np = 0; np < NP; np++) {
                        const float4v sx = *(const float4v *)(region + p * PSTRIDE + np * kPairRegion + kPSum + 16 * g);
                        Fmt::finish_pk(sc, c[np], sx, acc[r][2 * np], acc[r][2 * np + 1]);
                    }
                    continue;
                }
                float4v c[M];
                Fmt::template chain<M>(wr[p][r], region + p * PSTRIDE, lc, g, c);
                // One tile after the other.  Left free, the scheduler interleaves the tiles' chains and scale arithmetic, the
                // unpacked operands of several tiles are live at once and the 128 registers a wave of a 16-wave workgroup may
                // use overflow (spills in the instantiations with four tiles per workgroup pass; the 510 MB LM head lost
                // 20 %).  The empty asm consumes the chains' results; vector and matrix instructions may not cross the barrier.
#pragma unroll
                for (int mm = 0; mm < M; mm++) asm volatile("" : "+v"(c[mm]));
                __builtin_amdgcn_sched_barrier(0x10 | 0x80 | 0x4);
                const typename Fmt::Sc sc = Fmt::scales(wr[p][r], lc);
#pragma unroll
                for (int mm = 0; mm < M; mm++) acc[r][mm] += Fmt::finish(sc, c[mm]);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }

    // y[mm][16 rt + n] = sum over lane groups and waves; wave i adds up the i-th (row tile, activation row) pair
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int mm = 0; mm < M; mm++) red[((r * M + mm) * nwaves + wave) * 64 + lane] = acc[r][mm];
    if constexpr (NORM) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) ss += __shfl_xor(ss, off, 64);
        if (lane == 0) red_ss[wave] = ss;
    }
    __syncthreads();
    float inv_rms = 1.0f;
    if constexpr (NORM) {
        float tot = 0.0f;
        for (int wv = 0; wv < nwaves; wv++) tot += red_ss[wv];
        inv_rms = 1.0f / sqrtf(tot / (float)k + eps);
    }
    const int n4 = lane >> 2, q = lane & 3;
    if constexpr (GU) {
        for (int mm = wave; mm < M; mm += nwaves) {
            float sg = 0.0f, su = 0.0f;
            for (int wv = 0; wv < nwaves; wv++) {
                sg += red[(mm * nwaves + wv) * 64 + n4 + 16 * q];
                su += red[((M + mm) * nwaves + wv) * 64 + n4 + 16 * q];
            }
            sg = sum4(sg);
            su = sum4(su);
            const int64_t col = rt0 * 16 + n4;
            if (q == 0 && col < n && mm < m) {
                const float gate = sg * inv_rms + (bias ? bias[col] : 0.0f), up = su * inv_rms + (bias2 ? bias2[col] : 0.0f);
                const float out = gate / (1.0f + expf(-gate)) * up;  // SiLU
                const int64_t at = (int64_t)mm * ldy + col;
                turq_store_any(y, yt, at, out);
            }
        }
        return;
    }
    for (int i = wave; i < R * M; i += nwaves) {
        const int r = i / M, mm = i - r * M;
        float s = 0.0f;
        for (int wv = 0; wv < nwaves; wv++) s += red[(i * nwaves + wv) * 64 + n4 + 16 * q];
        s = sum4(s);
        const int64_t col = (rt0 + r) * 16 + n4;
        if (q == 0 && rt0 + r < nrt && col < n && mm < m) {
            const float out = s * inv_rms + (bias ? bias[col] : 0.0f);
            const int64_t at = (int64_t)mm * ldy + col;
            if (ACC && i == wave) turq_store_any(y, yt & 0xFF, at, out + old_first);  // (what y held was requested before the main loop)
            else turq_store_any(y, yt, at, out);
        }
    }
}

// which weight of the launch this workgroup works on
struct Row1Pick { const uint8_t *w; void *y; const float *bias; int64_t n, ldy; int first; int index; };
__device__ inline Row1Pick row1_pick(const Row1Args &a, int blk) {
    Row1Pick p{a.w[0], a.y[0], a.bias[0], a.n[0], a.ldy[0], 0, 0};
#pragma unroll
    for (int i = 1; i < kMaxRow1; i++)
        if (i < a.count && blk >= a.first[i]) p = Row1Pick{a.w[i], a.y[i], a.bias[i], a.n[i], a.ldy[i], a.first[i], i};
    return p;
}

// m <= M activation rows of stride ldx; MAXT = largest workgroup of the instantiation
template <int DT, int XT, int P, int R, int M, int MAXT, bool NORM = false, bool ACC = false>
__global__ void __launch_bounds__(MAXT) gemv_row1_kernel(Row1Args a, int64_t k, const void *__restrict__ x, int64_t ldx, int m, int yt,
                                                         const float *__restrict__ gw, float eps) {
    const Row1Pick p = row1_pick(a, (int)blockIdx.x);
    row1_body<DT, XT, P, R, M, false, NORM, ACC>(p.w, p.y, p.ldy, p.bias, p.n, (int64_t)((int)blockIdx.x - p.first), k, x, ldx, m, yt, nullptr,
                                            nullptr, gw, eps);
}

// gate_proj and up_proj of one MLP in one launch, the activation and the product applied before the store: workgroup b
// takes row tile b of both weights
template <int DT, int XT, int P, int M, int MAXT, bool NORM = false>
__global__ void __launch_bounds__(MAXT) gemv_row1_gateup_kernel(const uint8_t *__restrict__ wg, const uint8_t *__restrict__ wu,
                                                                 const float *__restrict__ bg, const float *__restrict__ bu, int64_t n,
                                                                 int64_t k, const void *__restrict__ x, int64_t ldx, int m,
                                                                 void *__restrict__ y, int64_t ldy, int yt, const float *__restrict__ gw,
                                                                 float eps) {
    row1_body<DT, XT, P, 2, M, true, NORM>(wg, y, ldy, bg, n, (int64_t)blockIdx.x, k, x, ldx, m, yt, wu, bu, gw, eps);
}

// weights of two formats that share an input (q, k Q4_K and v Q6_K of a Q4_K_M file) in one launch: the workgroup's weight
// decides which body runs
template <int DTA, int DTB, int XT, int P, int M, int MAXT, bool NORM = false>
__global__ void __launch_bounds__(MAXT) gemv_row1_mixed_kernel(Row1Args a, int64_t k, const void *__restrict__ x, int64_t ldx, int m,
                                                                int yt, const float *__restrict__ gw, float eps) {
    const Row1Pick p = row1_pick(a, (int)blockIdx.x);
    const int64_t rtb = (int64_t)((int)blockIdx.x - p.first);
    if (p.index < a.second) row1_body<DTA, XT, P, 1, M, false, NORM>(p.w, p.y, p.ldy, p.bias, p.n, rtb, k, x, ldx, m, yt, nullptr, nullptr, gw, eps);
    else row1_body<DTB, XT, P, 1, M, false, NORM>(p.w, p.y, p.ldy, p.bias, p.n, rtb, k, x, ldx, m, yt, nullptr, nullptr, gw, eps);
}

struct Row1Launch {
    Row1Args a;
    int blocks;
    int64_t k;
    const void *x;
    int64_t ldx;
    int m, yt, nwaves, rtiles;
    hipStream_t s;
    hipEvent_t ev0, ev1;
    const float *gw;  // RmsNorm weight (null: the activations are taken as they are) and eps
    float eps;
};

template <int DT, int P, int R, int M> size_t row1_lds(int nwaves) {
    const size_t tile = (Row1Fmt<DT>::kPacked && M > 1) ? (size_t)(M / 2) * kPairRegion : (size_t)M * kRegion;
    return (size_t)nwaves * P * tile + (size_t)nwaves * R * M * 64 * sizeof(float) + 64;  // (+ a sum of squares per wave)
}

template <int DT, int XT, int P, int R, int M, bool NORM, bool ACC>
hipError_t launch_final_n(const Row1Launch &l) {
    const size_t lds = row1_lds<DT, P, R, M>(l.nwaves);
    const dim3 grid((unsigned)l.blocks), block((unsigned)(64 * l.nwaves));
    if (lds > (64u << 10)) {  // 16 waves x two tiles in flight x two pairs of rows: 94 KiB
        const hipError_t raised = turq_raise_lds_limit((const void *)gemv_row1_kernel<DT, XT, P, R, M, 1024, NORM, ACC>, 128 << 10);
        if (raised != hipSuccess) return raised;
    }
    if (l.ev0) {
        hipExtLaunchKernelGGL((gemv_row1_kernel<DT, XT, P, R, M, 1024, NORM, ACC>), grid, block, (unsigned)lds, l.s, l.ev0, l.ev1, 0, l.a, l.k,
                              l.x, l.ldx, l.m, l.yt, l.gw, l.eps);
        return hipGetLastError();
    }
    gemv_row1_kernel<DT, XT, P, R, M, 1024, NORM, ACC><<<grid, block, lds, l.s>>>(l.a, l.k, l.x, l.ldx, l.m, l.yt, l.gw, l.eps);
    return hipGetLastError();
}
template <int DT, int XT, int P, int R, int M>
hipError_t launch_final(const Row1Launch &l) {
    if constexpr (M == 1) {
        // (with the norm weights held next to the weights, three column tiles in flight spill registers for Q5_K and Q6_K: two)
        if (l.gw) return launch_final_n<DT, XT, (P > 2 ? 2 : P), R, M, true, false>(l);
    }
    if (l.gw) return hipErrorInvalidValue;  // (the norm inside the kernel: one activation row)
    // the residual additions behind o_proj and down_proj: one row tile per workgroup (the tall matrices that take two are LM
    // heads; they would add through the store's own load of y)
    if constexpr (R == 1) {
        if (l.yt & TURQ_OUT_ACCUMULATE) return launch_final_n<DT, XT, P, R, M, false, true>(l);
    }
    return launch_final_n<DT, XT, P, R, M, false, false>(l);
}

// Column tiles in flight per wave: ONE.  The kernels exist with up to three for one activation row (four do not fit the
// registers of every format) and up to two for several rows, and while the weights were read with plain loads two or three
// were ahead; with the non-temporal loads a wave that takes its tiles one after the other is ahead on every shape measured
// (down_proj 12288 columns: 8.0 -> 7.5 us; MLP step at 1 / 2 / 3 / 4 rows + 2.5 / 3.6 / 4.9 / 4.1 %; LM head Q6_K / Q5_K + 7 / + 15 %;
// 4096 columns, two tiles per wave: level): the waves of a workgroup are at different tiles at any moment, which spreads
// their requests, and a wave holds fewer registers and less LDS.  TURQ_ROW1_P = 2 / 3 asks for the other forms.
inline int row1_in_flight(int64_t k, int nwaves, int m) {
    (void)k, (void)nwaves;
    const int forced = turq_tuning().row1_p;
    const int most = m > 1 ? 2 : 3;
    return forced >= 1 && forced <= most ? forced : 1;
}

template <int DT, int XT>
hipError_t launch_p(const Row1Launch &l) {
    const int p = row1_in_flight(l.k, l.nwaves, l.m);
    static_assert(TURQ_ROW1_MAX_M == 4, "instantiations for one, two and (packed formats) four activation rows");
    if (l.m > 2) {
        if constexpr (Row1Fmt<DT>::kPacked) return p == 1 ? launch_final<DT, XT, 1, 1, 4>(l) : launch_final<DT, XT, 2, 1, 4>(l);
        else return hipErrorInvalidValue;  // turq_gemv_row1_rows() says so
    }
    if (l.m == 2) return p == 1 ? launch_final<DT, XT, 1, 1, 2>(l) : launch_final<DT, XT, 2, 1, 2>(l);
    if (l.rtiles == 2)  // two row tiles double the weights a wave holds: at most two column tiles in flight
        return p == 1 ? launch_final<DT, XT, 1, 2, 1>(l) : launch_final<DT, XT, 2, 2, 1>(l);
    if (p == 1) return launch_final<DT, XT, 1, 1, 1>(l);
    if (p == 2) return launch_final<DT, XT, 2, 1, 1>(l);
    return launch_final<DT, XT, 3, 1, 1>(l);
}

template <int DT>
hipError_t launch_x(int xt, const Row1Launch &l) {
    switch (xt) {
    case TURQ_ACT_F32: return launch_p<DT, TURQ_ACT_F32>(l);
    case TURQ_ACT_BF16: return launch_p<DT, TURQ_ACT_BF16>(l);
    case TURQ_ACT_F16: return launch_p<DT, TURQ_ACT_F16>(l);
    default: return hipErrorInvalidValue;
    }
}

template <int DTA, int DTB, int XT, int P, int M, bool NORM>
hipError_t launch_mixed_final_n(const Row1Launch &l) {
    const size_t lds = std::max(row1_lds<DTA, P, 1, M>(l.nwaves), row1_lds<DTB, P, 1, M>(l.nwaves));
    const dim3 grid((unsigned)l.blocks), block((unsigned)(64 * l.nwaves));
    if (l.ev0) {
        hipExtLaunchKernelGGL((gemv_row1_mixed_kernel<DTA, DTB, XT, P, M, 1024, NORM>), grid, block, (unsigned)lds, l.s, l.ev0, l.ev1, 0,
                              l.a, l.k, l.x, l.ldx, l.m, l.yt, l.gw, l.eps);
        return hipGetLastError();
    }
    gemv_row1_mixed_kernel<DTA, DTB, XT, P, M, 1024, NORM><<<grid, block, lds, l.s>>>(l.a, l.k, l.x, l.ldx, l.m, l.yt, l.gw, l.eps);
    return hipGetLastError();
}
template <int DTA, int DTB, int XT, int P, int M>
hipError_t launch_mixed_final(const Row1Launch &l) {
    if constexpr (M == 1) {
        if (l.gw) return launch_mixed_final_n<DTA, DTB, XT, (P > 2 ? 2 : P), M, true>(l);  // (as in launch_final)
    }
    if (l.gw) return hipErrorInvalidValue;
    return launch_mixed_final_n<DTA, DTB, XT, P, M, false>(l);
}

template <int DTA, int DTB, int XT>
hipError_t launch_mixed_p(const Row1Launch &l) {
    const int p = row1_in_flight(l.k, l.nwaves, l.m);
    if (l.m > 2) return hipErrorInvalidValue;
    if (l.m == 2) return p == 1 ? launch_mixed_final<DTA, DTB, XT, 1, 2>(l) : launch_mixed_final<DTA, DTB, XT, 2, 2>(l);
    if (p == 1) return launch_mixed_final<DTA, DTB, XT, 1, 1>(l);
    if (p == 2) return launch_mixed_final<DTA, DTB, XT, 2, 1>(l);
    return launch_mixed_final<DTA, DTB, XT, 3, 1>(l);
}

// fills the argument block; returns false for arguments no launch accepts
bool row1_args(Row1Launch &l, int count, const void *const *w, const int64_t *n, void *const *y, const int64_t *ldy,
               const float *const *bias, int row_tiles) {
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
    if (blocks > 0x7FFFFFFF) return false;
    l.blocks = (int)blocks;
    return true;
}

}  // namespace

bool turq_gemv_row1_supports(int dtype) {
    return dtype == TURQ_Q4_K || dtype == TURQ_Q5_K || dtype == TURQ_Q6_K || dtype == TURQ_Q8_0;
}
// activation rows one launch takes for this format: four where two rows share an MFMA chain, else two
int turq_gemv_row1_rows(int dtype) {
    switch (dtype) {
    case TURQ_Q4_K: return Row1Fmt<TURQ_Q4_K>::kPacked ? 4 : 2;
    case TURQ_Q5_K: return Row1Fmt<TURQ_Q5_K>::kPacked ? 4 : 2;
    case TURQ_Q6_K: return Row1Fmt<TURQ_Q6_K>::kPacked ? 4 : 2;
    case TURQ_Q8_0: return Row1Fmt<TURQ_Q8_0>::kPacked ? 4 : 2;
    default: return 0;
    }
}

// count (1..4) weights of one format and one k against m (1..TURQ_ROW1_MAX_M) activation rows of stride ldx (rows 16-byte
// aligned); results to y[i] with row stride ldy[i] (null: n[i]); row_tiles (1 or 2; 2 with one activation row only) per workgroup.
hipError_t turq_launch_gemv_row1(int dtype, int count, const void *const *w, const int64_t *n, int64_t k, const void *x, int x_dtype,
                                 int64_t ldx, int64_t m, void *const *y, int y_dtype, const int64_t *ldy, const float *const *bias,
                                 int nwaves, int row_tiles, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop, const float *norm_weight,
                                 float norm_eps) {
    if (count < 1 || count > kMaxRow1 || nwaves < 1 || nwaves > 16 || k % turq_dt_block_elems(dtype) != 0) return hipErrorInvalidValue;
    if (m < 1 || m > TURQ_ROW1_MAX_M || (row_tiles != 1 && !(row_tiles == 2 && m == 1))) return hipErrorInvalidValue;
    if (!turq_yt_ok(y_dtype, true)) return hipErrorInvalidValue;
    Row1Launch l{};
    if (!row1_args(l, count, w, n, y, ldy, bias, row_tiles)) return hipErrorInvalidValue;
    if (l.blocks == 0) return hipSuccess;
    if (k == 0) return hipErrorInvalidValue;
    l.k = k, l.x = x, l.ldx = ldx, l.m = (int)m, l.yt = y_dtype, l.nwaves = nwaves, l.rtiles = row_tiles;
    l.s = stream, l.ev0 = ev_start, l.ev1 = ev_stop, l.gw = norm_weight, l.eps = norm_eps;
    switch (dtype) {
    case TURQ_Q4_K: return launch_x<TURQ_Q4_K>(x_dtype, l);
    case TURQ_Q5_K: return launch_x<TURQ_Q5_K>(x_dtype, l);
    case TURQ_Q6_K: return launch_x<TURQ_Q6_K>(x_dtype, l);
    case TURQ_Q8_0: return launch_x<TURQ_Q8_0>(x_dtype, l);
    default: return hipErrorInvalidValue;
    }
}

// the pairs of a Q4_K_M and of a Q5_K_M file
bool turq_gemv_row1_mixed_supports(int dtype_a, int dtype_b) {
    return (dtype_a == TURQ_Q4_K || dtype_a == TURQ_Q5_K) && dtype_b == TURQ_Q6_K;
}

// count (2..4) weights of one k against m activation rows: the first `second` of format dtype_a, the others of dtype_b
// (a pair turq_gemv_row1_mixed_supports accepts); one row tile per workgroup.
hipError_t turq_launch_gemv_row1_mixed(int dtype_a, int dtype_b, int count, int second, const void *const *w, const int64_t *n,
                                       int64_t k, const void *x, int x_dtype, int64_t ldx, int64_t m, void *const *y, int y_dtype,
                                       const int64_t *ldy, const float *const *bias, int nwaves, hipStream_t stream,
                                       hipEvent_t ev_start, hipEvent_t ev_stop, const float *norm_weight, float norm_eps) {
    if (!turq_gemv_row1_mixed_supports(dtype_a, dtype_b) || count < 2 || count > kMaxRow1 || second < 1 || second >= count ||
        nwaves < 1 || nwaves > 16 || k % 256 != 0 || m < 1 || m > TURQ_ROW1_MAX_M)
        return hipErrorInvalidValue;
    if (!turq_yt_ok(y_dtype, true)) return hipErrorInvalidValue;
    Row1Launch l{};
    if (!row1_args(l, count, w, n, y, ldy, bias, 1)) return hipErrorInvalidValue;
    l.a.second = second;
    if (l.blocks == 0) return hipSuccess;
    if (k == 0) return hipErrorInvalidValue;
    l.k = k, l.x = x, l.ldx = ldx, l.m = (int)m, l.yt = y_dtype, l.nwaves = nwaves, l.rtiles = 1;
    l.s = stream, l.ev0 = ev_start, l.ev1 = ev_stop, l.gw = norm_weight, l.eps = norm_eps;
    if (dtype_a == TURQ_Q5_K) {
        switch (x_dtype) {
        case TURQ_ACT_F32: return launch_mixed_p<TURQ_Q5_K, TURQ_Q6_K, TURQ_ACT_F32>(l);
        case TURQ_ACT_BF16: return launch_mixed_p<TURQ_Q5_K, TURQ_Q6_K, TURQ_ACT_BF16>(l);
        case TURQ_ACT_F16: return launch_mixed_p<TURQ_Q5_K, TURQ_Q6_K, TURQ_ACT_F16>(l);
        default: return hipErrorInvalidValue;
        }
    }
    switch (x_dtype) {
    case TURQ_ACT_F32: return launch_mixed_p<TURQ_Q4_K, TURQ_Q6_K, TURQ_ACT_F32>(l);
    case TURQ_ACT_BF16: return launch_mixed_p<TURQ_Q4_K, TURQ_Q6_K, TURQ_ACT_BF16>(l);
    case TURQ_ACT_F16: return launch_mixed_p<TURQ_Q4_K, TURQ_Q6_K, TURQ_ACT_F16>(l);
    default: return hipErrorInvalidValue;
    }
}

namespace {
struct GateUpLaunch {
    const void *wg, *wu;
    const float *bg, *bu;
    int64_t n, k;
    const void *x;
    int64_t ldx;
    int m;
    void *y;
    int64_t ldy;
    int yt, nwaves;
    hipStream_t s;
    hipEvent_t ev0, ev1;
    const float *gw;  // RmsNorm weight (null: none) and eps
    float eps;
};

template <int DT, int XT, int P, int M, bool NORM>
hipError_t launch_gateup_final(const GateUpLaunch &l) {
    const size_t lds = row1_lds<DT, P, 2, M>(l.nwaves);
    const dim3 grid((unsigned)turq_tile_rows(l.n)), block((unsigned)(64 * l.nwaves));
    if (l.ev0) {
        hipExtLaunchKernelGGL((gemv_row1_gateup_kernel<DT, XT, P, M, 1024, NORM>), grid, block, (unsigned)lds, l.s, l.ev0, l.ev1, 0,
                              (const uint8_t *)l.wg, (const uint8_t *)l.wu, l.bg, l.bu, l.n, l.k, l.x, l.ldx, l.m, l.y, l.ldy, l.yt, l.gw, l.eps);
        return hipGetLastError();
    }
    gemv_row1_gateup_kernel<DT, XT, P, M, 1024, NORM><<<grid, block, lds, l.s>>>((const uint8_t *)l.wg, (const uint8_t *)l.wu, l.bg, l.bu, l.n,
                                                                                l.k, l.x, l.ldx, l.m, l.y, l.ldy, l.yt, l.gw, l.eps);
    return hipGetLastError();
}

template <int DT, int XT>
hipError_t launch_gateup_p(const GateUpLaunch &l) {
    // one column tile in flight, as in row1_in_flight (two weights double what a wave holds per column tile: two at most,
    // on request, where a wave has two tiles to take)
    const int64_t per_wave = (turq_tile_cols(l.k) + l.nwaves - 1) / l.nwaves;
    const bool one = per_wave <= 1 || turq_tuning().row1_p != 2;
    if (l.m == 2) {
        if (l.gw) return hipErrorInvalidValue;  // (the norm inside the kernel: one activation row)
        return one ? launch_gateup_final<DT, XT, 1, 2, false>(l) : launch_gateup_final<DT, XT, 2, 2, false>(l);
    }
    if (l.gw) return one ? launch_gateup_final<DT, XT, 1, 1, true>(l) : launch_gateup_final<DT, XT, 2, 1, true>(l);
    return one ? launch_gateup_final<DT, XT, 1, 1, false>(l) : launch_gateup_final<DT, XT, 2, 1, false>(l);
}

template <int DT>
hipError_t launch_gateup_x(int xt, const GateUpLaunch &l) {
    switch (xt) {
    case TURQ_ACT_F32: return launch_gateup_p<DT, TURQ_ACT_F32>(l);
    case TURQ_ACT_BF16: return launch_gateup_p<DT, TURQ_ACT_BF16>(l);
    case TURQ_ACT_F16: return launch_gateup_p<DT, TURQ_ACT_F16>(l);
    default: return hipErrorInvalidValue;
    }
}
}  // namespace

// y[mm][c] = silu(x[mm] . gate[c] + bias_gate[c]) * (x[mm] . up[c] + bias_up[c]) for m = 1 or 2 activation rows: gate and up are
// two tiled weights of one format and one shape [n, k]; rows of x 16-byte aligned.  norm_weight (m = 1): x stands for RmsNorm(x)
hipError_t turq_launch_gemv_row1_gateup(int dtype, const void *w_gate, const void *w_up, int64_t n, int64_t k, const void *x,
                                        int x_dtype, int64_t ldx, int64_t m, void *y, int y_dtype, int64_t ldy, const float *bias_gate,
                                        const float *bias_up, int nwaves, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop,
                                        const float *norm_weight, float norm_eps) {
    if (nwaves < 1 || nwaves > 16 || m < 1 || m > 2 || k <= 0 || k % turq_dt_block_elems(dtype) != 0) return hipErrorInvalidValue;
    if (!turq_yt_ok(y_dtype, true)) return hipErrorInvalidValue;
    if (n == 0) return hipSuccess;
    const GateUpLaunch l{w_gate, w_up, bias_gate, bias_up, n, k, x, ldx, (int)m, y, ldy, y_dtype, nwaves, stream, ev_start, ev_stop, norm_weight, norm_eps};
    switch (dtype) {
    case TURQ_Q4_K: return launch_gateup_x<TURQ_Q4_K>(x_dtype, l);
    case TURQ_Q5_K: return launch_gateup_x<TURQ_Q5_K>(x_dtype, l);
    case TURQ_Q6_K: return launch_gateup_x<TURQ_Q6_K>(x_dtype, l);
    case TURQ_Q8_0: return launch_gateup_x<TURQ_Q8_0>(x_dtype, l);
    default: return hipErrorInvalidValue;
    }
}

TURQ_NONFINITE_READER(turq_nonfinite_gemv_row1)

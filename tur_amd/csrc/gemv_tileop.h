// Per-format pieces shared by the skinny MFMA kernels (gemv_mfma.hip, gemv_cs.hip): what a lane loads from HBM for one
// 16-row x 256-column weight tile, the activation fragments of a column tile, and the tile arithmetic
//   acc[mt] += x-fragments(mt) . unpacked weight tile        (v_mfma_f32_16x16x32_f16, exact integer-valued f16 B operands)
// with the f16 super-block scales applied in f32 on the 16 x 16 result.
#pragma once

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

// ---- weight registers of one tile (everything a lane loads from HBM for it) ----

template <int DT> struct WRegs;
template <> struct WRegs<TURQ_Q4_K> { uint4v qa, qb, hd; };
template <> struct WRegs<TURQ_Q5_K> { uint4v qa, qb, hd; uint2v hh; };
template <> struct WRegs<TURQ_Q6_K> { uint4v qla, qlb, qh; uint32_t scw; uint32_t d16; };
template <> struct WRegs<TURQ_Q8_0> { uint4v p[4]; uint4v dd; };

// o: the lane's byte offsets (aux = 2 bytes per weight row); `tile` is wave-uniform
// (non-temporal loads: every weight byte is read once per launch, and lines that are not kept in the L2 as if they would be
// read again leave the cache to the activations and make the end of a launch cheaper: + 5 % on the one-row MLP step)
template <int DT> __device__ inline WRegs<DT> load_tile(const uint8_t *__restrict__ tile, const GOff &o);
template <> __device__ inline WRegs<TURQ_Q4_K> load_tile<TURQ_Q4_K>(const uint8_t *__restrict__ tile, const GOff &o) {
    using F = TiledFmt<TURQ_Q4_K>;
    WRegs<TURQ_Q4_K> w;
    w.qa = __builtin_nontemporal_load((const uint4v *)(tile + F::kQA + o.o16));
    w.qb = __builtin_nontemporal_load((const uint4v *)(tile + F::kQB + o.o16));
    w.hd = __builtin_nontemporal_load((const uint4v *)(tile + F::kHDR + o.hdr));
    return w;
}
template <> __device__ inline WRegs<TURQ_Q5_K> load_tile<TURQ_Q5_K>(const uint8_t *__restrict__ tile, const GOff &o) {
    using F = TiledFmt<TURQ_Q5_K>;
    WRegs<TURQ_Q5_K> w;
    w.qa = __builtin_nontemporal_load((const uint4v *)(tile + F::kQA + o.o16));
    w.qb = __builtin_nontemporal_load((const uint4v *)(tile + F::kQB + o.o16));
    w.hh = __builtin_nontemporal_load((const uint2v *)(tile + F::kQH + o.o8));
    w.hd = __builtin_nontemporal_load((const uint4v *)(tile + F::kHDR + o.hdr));
    return w;
}
template <> __device__ inline WRegs<TURQ_Q6_K> load_tile<TURQ_Q6_K>(const uint8_t *__restrict__ tile, const GOff &o) {
    using F = TiledFmt<TURQ_Q6_K>;
    WRegs<TURQ_Q6_K> w;
    w.qla = __builtin_nontemporal_load((const uint4v *)(tile + F::kQLA + o.o16));
    w.qlb = __builtin_nontemporal_load((const uint4v *)(tile + F::kQLB + o.o16));
    w.qh = __builtin_nontemporal_load((const uint4v *)(tile + F::kQH + o.o16));
    w.scw = __builtin_nontemporal_load((const uint32_t *)(tile + F::kSC + o.o4));
    w.d16 = __builtin_nontemporal_load((const uint16_t *)(tile + F::kD + o.aux));
    return w;
}
template <> __device__ inline WRegs<TURQ_Q8_0> load_tile<TURQ_Q8_0>(const uint8_t *__restrict__ tile, const GOff &o) {
    using F = TiledFmt<TURQ_Q8_0>;
    WRegs<TURQ_Q8_0> w;
#pragma unroll
    for (int i = 0; i < 4; i++) w.p[i] = __builtin_nontemporal_load((const uint4v *)(tile + 1024 * i + o.o16));
    w.dd = __builtin_nontemporal_load((const uint4v *)(tile + F::kD + o.hdr));
    return w;
}
// makes the registers of a tile new values for the compiler (no instruction): what it derived from them before is not kept
__device__ inline void touch(uint4v &v) { asm volatile("" : "+v"(v)); }
__device__ inline void touch(uint2v &v) { asm volatile("" : "+v"(v)); }
__device__ inline void touch(uint32_t &v) { asm volatile("" : "+v"(v)); }
__device__ inline void touch(WRegs<TURQ_Q4_K> &w) { touch(w.qa), touch(w.qb), touch(w.hd); }
__device__ inline void touch(WRegs<TURQ_Q5_K> &w) { touch(w.qa), touch(w.qb), touch(w.hd), touch(w.hh); }
__device__ inline void touch(WRegs<TURQ_Q6_K> &w) { touch(w.qla), touch(w.qlb), touch(w.qh), touch(w.scw), touch(w.d16); }
__device__ inline void touch(WRegs<TURQ_Q8_0> &w) {
#pragma unroll
    for (int i = 0; i < 4; i++) touch(w.p[i]);
    touch(w.dd);
}
__device__ inline GOff lane_offsets(int lane, int mpad) {
    const uint32_t l = (uint32_t)lane, r = l & 15u;
    return GOff{16u * l, 8u * l, 4u * l, 16u * r, 2u * r, 16u * ((l >> 4) * (uint32_t)mpad + (r & (uint32_t)(mpad - 1)))};
}

// ---- activation fragments of one tile: NQ steps for each of MT m-tiles ----
// Rows of the A operand beyond the prepared height are never stored (every output row depends on
// its own A row only), so lanes of those rows simply re-read a valid row instead of zeros.
template <int DT, int MT> struct AFrags {
    static constexpr int NQ = DT == TURQ_Q8_0 ? TURQ_NQ_Q8_0 : TURQ_NQ_KQUANT;
    half8v a[MT][NQ];
};

// tile_frags (wave-uniform): the fragments of column tile b of m-tile 0; step q of m-tile mt starts mt * mt_stride + 4 q mpad
// chunks of 16 bytes further on, and lane (r, g) takes chunk g * mpad + r % mpad of it (o.frag)
template <int DT, int MT>
__device__ inline AFrags<DT, MT> load_frags_global(const half8v *__restrict__ tile_frags, int64_t mt_stride, int mpad,
                                                   const GOff &o) {
    AFrags<DT, MT> f;
    const uint8_t *base = (const uint8_t *)tile_frags;
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int q = 0; q < AFrags<DT, MT>::NQ; q++)
            f.a[mt][q] = *(const half8v *)(base + 16 * (mt * mt_stride + (int64_t)(q * 4) * mpad) + o.frag);
    return f;
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
    uint32_t t0 = and_or_u32(w, 0x000F000Fu, kMagic1024);
    uint32_t t1 = and_or_u32(w, 0x00F000F0u, kMagic1024);
    uint32_t t2 = and_or_u32(w8, 0x000F000Fu, kMagic1024);
    uint32_t t3 = and_or_u32(w8, 0x00F000F0u, kMagic1024);
    if (HIGH) {  // fifth bit: +16 on top of the nibble (bit 4 / 20, or bit 8 / 24 for the x16 form)
        t0 = and_or_u32(rotr32(h0, (uint32_t)u0), 0x00100010u, t0);
        t1 = and_or_u32(rotr32(h1, (uint32_t)u0), 0x01000100u, t1);
        t2 = and_or_u32(rotr32(h0, (uint32_t)(u0 + 1)), 0x00100010u, t2);
        t3 = and_or_u32(rotr32(h1, (uint32_t)(u0 + 1)), 0x01000100u, t3);
    }
    return make_half8(pk_fma(as_half2(t0), s, c1), pk_fma(as_half2(t1), s16, c2), pk_fma(as_half2(t2), s, c1),
                      pk_fma(as_half2(t3), s16, c2));
}

// ---- per-format tile arithmetic: acc[mt] += (this tile's contribution) ----
// NV = how many of a lane's four result rows get the f32 scale applied.  Always instantiated with 4.  (NV < 4 once
// returned garbage for Q8_0; that was at a time when the unpack's v_and_or_b32 was written as inline asm, which hides
// from the compiler the wait states between such an instruction and an MFMA whose registers it reuses, see
// mfma_common.h.  It has not been tried again since.)
template <int DT, int MT, int NV> struct TileOp;

template <int DT, int MT, int NV> struct TileOpK45 {
    static constexpr bool HIGH = DT == TURQ_Q5_K;
    __device__ static void run(const WRegs<DT> &w, const AFrags<DT, MT> &f, int lane, float4v *acc) {
        const int g = lane >> 4;
        uint32_t h0 = 0, h1 = 0;
        if constexpr (HIGH) { h0 = w.hh.x; h1 = w.hh.y; }
        const K4Consts c = k4_consts(w.hd, g);
        const uint32_t wq[8] = {w.qa.x, w.qa.y, w.qa.z, w.qa.w, w.qb.x, w.qb.y, w.qb.z, w.qb.w};
        float4v tmp[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) tmp[mt] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const half8v bop = i < 4 ? k45_operand<HIGH>(wq[i], c.s_lo, c.s16_lo, c.c1_lo, c.c2_lo, h0, h1, 2 * i)
                                     : k45_operand<HIGH>(wq[i], c.s_hi, c.s16_hi, c.c1_hi, c.c2_hi, h0, h1, 2 * i);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) tmp[mt] = mfma16x16x32(f.a[mt][i], bop, tmp[mt]);
        }
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            float4v tmin = mfma16x16x32(f.a[mt][8], c.bmin, float4v{0.f, 0.f, 0.f, 0.f});
#pragma unroll
            for (int i = 0; i < NV; i++) acc[mt][i] += c.d * tmp[mt][i] - c.dmin * tmin[i];
        }
    }
};
template <int MT, int NV> struct TileOp<TURQ_Q4_K, MT, NV> : TileOpK45<TURQ_Q4_K, MT, NV> {};
template <int MT, int NV> struct TileOp<TURQ_Q5_K, MT, NV> : TileOpK45<TURQ_Q5_K, MT, NV> {};

template <int MT, int NV> struct TileOp<TURQ_Q6_K, MT, NV> {
    __device__ static void run(const WRegs<TURQ_Q6_K> &w, const AFrags<TURQ_Q6_K, MT> &f, int lane, float4v *acc) {
        (void)lane;
        const float d = h2f_bits(w.d16);
        const uint32_t wl[8] = {w.qla.x, w.qla.y, w.qla.z, w.qla.w, w.qlb.x, w.qlb.y, w.qlb.z, w.qlb.w};
        const uint32_t wh[4] = {w.qh.x, w.qh.y, w.qh.z, w.qh.w};
        float4v tmp[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) tmp[mt] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sg = 0; sg < 4; sg++) {  // scale group sg covers steps 2sg, 2sg+1
            const _Float16 sc = (_Float16)(float)(int)(int8_t)(w.scw >> (8 * sg));
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
                const uint32_t wv = wl[i];
                const uint32_t w8 = rotr32(wv, 8);
                const half8v b1 = make_half8(pk_fma(and_or_h2(wv, 0x003C003Cu, kMagic256), s1, c256),
                                             pk_fma(and_or_h2(wv, 0x03C003C0u, kMagic16), s1, c16),
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
                    tmp[mt] = mfma16x16x32(f.a[mt][i], b1, tmp[mt]);
                    tmp[mt] = mfma16x16x32(f.a[mt][i], b2, tmp[mt]);
                }
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
#pragma unroll
            for (int i = 0; i < NV; i++) acc[mt][i] += d * tmp[mt][i];
        }
    }
};

template <int MT, int NV> struct TileOp<TURQ_Q8_0, MT, NV> {
    __device__ static void run(const WRegs<TURQ_Q8_0> &w, const AFrags<TURQ_Q8_0, MT> &f, int lane, float4v *acc) {
        (void)lane;
        const uint32_t dw[4] = {w.dd.x, w.dd.y, w.dd.z, w.dd.w};
        const half2v k1152 = splat2((_Float16)-1152.0f);  // 1024 + the 128 the bytes were offset by
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const uint32_t w0 = (q & 1) ? w.p[q >> 1].z : w.p[q >> 1].x;
            const uint32_t w1 = (q & 1) ? w.p[q >> 1].w : w.p[q >> 1].y;
            const half8v bop = make_half8(and_or_h2(w0, 0x00FF00FFu, kMagic1024) + k1152,
                                          and_or_h2(w0 >> 8, 0x00FF00FFu, kMagic1024) + k1152,
                                          and_or_h2(w1, 0x00FF00FFu, kMagic1024) + k1152,
                                          and_or_h2(w1 >> 8, 0x00FF00FFu, kMagic1024) + k1152);
            const float d = h2f_bits((q & 1) ? (dw[q >> 1] >> 16) : (dw[q >> 1] & 0xFFFFu));
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                float4v t = mfma16x16x32(f.a[mt][q], bop, float4v{0.f, 0.f, 0.f, 0.f});
#pragma unroll
                for (int i = 0; i < NV; i++) acc[mt][i] += d * t[i];
            }
        }
    }
};

// ---- activation fragments straight from the caller's rows ----
// The raw activations behind the A fragments of one column tile and m-tile: what frags_from_rows loads, kept apart from what it
// computes, for kernels that request the next column tile's activations while they still work on the current one.
template <int XT> struct RawRows {
    uint4v v[XT == TURQ_ACT_F32 ? 16 : 8];
};
template <int DT, int XT>
__device__ inline RawRows<XT> load_rows_raw(const void *__restrict__ x, int64_t ldx, int64_t m, int64_t k, int64_t b, int lane, int mt) {
    constexpr bool KQ = DT != TURQ_Q8_0;
    constexpr int ES = XT == TURQ_ACT_F32 ? 4 : 2;
    const int r = lane & 15, g = lane >> 4;
    int64_t row = 16 * mt + r;
    if (row >= m) row = m - 1;
    const uint8_t *base = (const uint8_t *)x + (row * ldx + b * 256) * ES;
    RawRows<XT> raw;
#pragma unroll
    for (int q = 0; q < 8; q++) {
        const int col = KQ ? 64 * g + 8 * q : 32 * q + 8 * g;
        const bool in = KQ || b * 256 + col < k;
        const uint8_t *p = base + (in ? col : 0) * ES;
        if constexpr (XT == TURQ_ACT_F32) {
            const uint4v a = *(const uint4v *)p, c = *(const uint4v *)(p + 16);
            raw.v[2 * q] = in ? a : uint4v{0u, 0u, 0u, 0u};
            raw.v[2 * q + 1] = in ? c : uint4v{0u, 0u, 0u, 0u};
        } else {
            const uint4v a = *(const uint4v *)p;
            raw.v[q] = in ? a : uint4v{0u, 0u, 0u, 0u};
        }
    }
    return raw;
}
// eight bf16 values -> f16 (through f32, round to nearest even)
__device__ inline half8v bf16x8_to_half8(uint4v u) {
    const uint32_t wd[4] = {u.x, u.y, u.z, u.w};
    half2v h[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
        h[j] = __builtin_convertvector(float2v{__uint_as_float(wd[j] << 16), __uint_as_float(wd[j] & 0xFFFF0000u)}, half2v);
    return make_half8(h[0], h[1], h[2], h[3]);
}
template <int XT> __device__ inline half8v raw_to_half8(const RawRows<XT> &raw, int q) {
    if constexpr (XT == TURQ_ACT_F32) {
        const uint4v a = raw.v[2 * q], b = raw.v[2 * q + 1];
        const half2v h0 = __builtin_convertvector(float2v{__uint_as_float(a.x), __uint_as_float(a.y)}, half2v);
        const half2v h1 = __builtin_convertvector(float2v{__uint_as_float(a.z), __uint_as_float(a.w)}, half2v);
        const half2v h2 = __builtin_convertvector(float2v{__uint_as_float(b.x), __uint_as_float(b.y)}, half2v);
        const half2v h3 = __builtin_convertvector(float2v{__uint_as_float(b.z), __uint_as_float(b.w)}, half2v);
        return make_half8(h0, h1, h2, h3);
    } else if constexpr (XT == TURQ_ACT_BF16) {
        return bf16x8_to_half8(raw.v[q]);
    } else {
        return __builtin_bit_cast(half8v, raw.v[q]);
    }
}
// step 8 of a K-quant column tile: the (hi, lo) f16 pairs of the sums of the lane's four 16-column groups (steps 2 j, 2 j + 1)
__device__ inline half8v kq_group_sums(const half8v *__restrict__ out) {
    half2v s[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float sum = 0.0f;
#pragma unroll
        for (int e = 0; e < 4; e++) sum = __builtin_amdgcn_fdot2(half2v{out[2 * j][2 * e], out[2 * j][2 * e + 1]}, splat2((_Float16)1.0f), sum, false);
#pragma unroll
        for (int e = 0; e < 4; e++) sum = __builtin_amdgcn_fdot2(half2v{out[2 * j + 1][2 * e], out[2 * j + 1][2 * e + 1]}, splat2((_Float16)1.0f), sum, false);
        const _Float16 hi = (_Float16)sum;
        s[j] = half2v{hi, (_Float16)(sum - (float)hi)};
    }
    return make_half8(s[0], s[1], s[2], s[3]);
}
// the fragments of those activations (the conversions and sums of frags_from_rows, value for value)
template <int DT, int XT> __device__ inline void frags_from_raw(const RawRows<XT> &raw, half8v *__restrict__ out) {
#pragma unroll
    for (int q = 0; q < 8; q++) out[q] = raw_to_half8<XT>(raw, q);
    if constexpr (DT != TURQ_Q8_0) out[8] = kq_group_sums(out);
}

// The A fragments of column tile b and m-tile mt, from the activation rows themselves.  Lane (r, g) holds row 16 mt + r:
// K-quants: step q = columns 256 b + 64 g + 8 q .. + 7, step 8 = the (hi, lo) sums of its four 16-column groups;
// Q8_0: step q = columns 256 b + 32 q + 8 g .. + 7 (zeros past k, which may end inside the tile).
// Rows past m repeat row m - 1: every output row depends on its own A row only and those rows are not stored.
template <int DT, int XT>
__device__ inline void frags_from_rows(const void *__restrict__ x, int64_t ldx, int64_t m, int64_t k, int64_t b, int lane, int mt,
                                       half8v *__restrict__ out) {
    const RawRows<XT> raw = load_rows_raw<DT, XT>(x, ldx, m, k, b, lane, mt);
    frags_from_raw<DT, XT>(raw, out);
}

// Several weights of one format and one k against the same activations in one launch (gate and up, or q and k,
// of a decoder layer): workgroups [first[i], first[i + 1]) work on weight i.  One launch instead of several
// spares the small matrices their start-up and tail, which at decode sizes is a third of a launch.
constexpr int kMaxMulti = 4;
struct MultiArgs {
    const uint8_t *w[kMaxMulti];
    void *y[kMaxMulti];
    const float *bias[kMaxMulti];
    int64_t n[kMaxMulti], ldy[kMaxMulti];
    int first[kMaxMulti];
    int count;
    int second;  // two-format launches: weights [0, second) are of the first format, [second, count) of the second
};

// the weight a workgroup of such a launch works on, and its index among the weight's workgroups
struct MultiPick { const uint8_t *w; void *y; const float *bias; int64_t n, ldy; int block; int index; };
__device__ inline MultiPick multi_pick(const MultiArgs &a, int blk) {
    MultiPick p{a.w[0], a.y[0], a.bias[0], a.n[0], a.ldy[0], blk, 0};
#pragma unroll
    for (int i = 1; i < kMaxMulti; i++)
        if (i < a.count && blk >= a.first[i]) p = MultiPick{a.w[i], a.y[i], a.bias[i], a.n[i], a.ldy[i], blk - a.first[i], i};
    return p;
}

}  // namespace

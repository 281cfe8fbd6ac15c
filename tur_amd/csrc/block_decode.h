// Element-wise decode of GGUF blocks kept in their native byte order (device code).
//
// decode8<DT>(row, e0, out) writes the eight consecutive dequantized elements e0..e0+7 (e0 % 8 == 0)
// of a row that starts at `row`.  The arithmetic is candle's `to_float`, operation for operation:
// every product and the subtraction are rounded separately, so the including translation unit must
// be compiled with -ffp-contract=off when bit-exact results are wanted.
#pragma once

#include "common.h"

__device__ inline float turq_h2f(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;  // exact, subnormals included
}
__device__ inline float turq_bf2f(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

__device__ inline uint16_t turq_ld_u16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

// 6-bit scale / min of sub-block j from the 12 packed bytes of a Q4_K / Q5_K block
__device__ inline void turq_scale_min_k4(int j, const uint8_t *q, uint32_t &sc, uint32_t &m) {
    if (j < 4) {
        sc = q[j] & 63u;
        m = q[j + 4] & 63u;
    } else {
        sc = (q[j + 4] & 0x0Fu) | ((uint32_t)(q[j - 4] >> 6) << 4);
        m = (uint32_t)(q[j + 4] >> 4) | ((uint32_t)(q[j] >> 6) << 4);
    }
}

template <int DT> struct Decode8;

template <> struct Decode8<TURQ_Q8_0> {
    __device__ static void run(const uint8_t *row, int64_t e0, float *out) {
#pragma clang fp contract(off)
        const uint8_t *b = row + (e0 >> 5) * 34;
        const float d = turq_h2f(turq_ld_u16(b));
        const int8_t *q = (const int8_t *)(b + 2 + (e0 & 31));
#pragma unroll
        for (int j = 0; j < 8; j++) out[j] = (float)q[j] * d;
    }
};

template <> struct Decode8<TURQ_Q4_K> {
    __device__ static void run(const uint8_t *row, int64_t e0, float *out) {
#pragma clang fp contract(off)
        const uint8_t *b = row + (e0 >> 8) * 144;
        const int e = (int)(e0 & 255);
        const int sub = e >> 5;          // sub-block 0..7
        const int l0 = e & 31;
        const float d = turq_h2f(turq_ld_u16(b));
        const float dmin = turq_h2f(turq_ld_u16(b + 2));
        uint32_t sc, m;
        turq_scale_min_k4(sub, b + 4, sc, m);
        const float dl = d * (float)sc;
        const float ml = dmin * (float)m;
        const uint8_t *q = b + 16 + 32 * (sub >> 1) + l0;
        const int shift = (sub & 1) * 4;
#pragma unroll
        for (int j = 0; j < 8; j++) out[j] = dl * (float)((q[j] >> shift) & 0xF) - ml;
    }
};

template <> struct Decode8<TURQ_Q5_K> {
    __device__ static void run(const uint8_t *row, int64_t e0, float *out) {
#pragma clang fp contract(off)
        const uint8_t *b = row + (e0 >> 8) * 176;
        const int e = (int)(e0 & 255);
        const int sub = e >> 5;
        const int l0 = e & 31;
        const float d = turq_h2f(turq_ld_u16(b));
        const float dmin = turq_h2f(turq_ld_u16(b + 2));
        uint32_t sc, m;
        turq_scale_min_k4(sub, b + 4, sc, m);
        const float dl = d * (float)sc;
        const float ml = dmin * (float)m;
        const uint8_t *qh = b + 16 + l0;
        const uint8_t *q = b + 48 + 32 * (sub >> 1) + l0;
        const int shift = (sub & 1) * 4;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float add = ((qh[j] >> sub) & 1) ? 16.0f : 0.0f;
            out[j] = dl * ((float)((q[j] >> shift) & 0xF) + add) - ml;
        }
    }
};

template <> struct Decode8<TURQ_Q6_K> {
    __device__ static void run(const uint8_t *row, int64_t e0, float *out) {
#pragma clang fp contract(off)
        const uint8_t *b = row + (e0 >> 8) * 210;
        const int e = (int)(e0 & 255);
        const int half = e >> 7;
        const int r = e & 127;
        const int quarter = r >> 5;
        const int l0 = r & 31;
        const float d = turq_h2f(turq_ld_u16(b + 208));
        const float sc = (float)((const int8_t *)(b + 192))[e >> 4];
        const float ds = d * sc;
        const uint8_t *ql = b + 64 * half + 32 * (quarter & 1) + l0;
        const uint8_t *qh = b + 128 + 32 * half + l0;
        const int lshift = (quarter >> 1) * 4;
        const int hshift = quarter * 2;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int q = (int)(((ql[j] >> lshift) & 0xF) | (((qh[j] >> hshift) & 3) << 4)) - 32;
            out[j] = ds * (float)q;
        }
    }
};

template <> struct Decode8<TURQ_F32> {
    __device__ static void run(const uint8_t *row, int64_t e0, float *out) {
        const float *p = (const float *)row + e0;
#pragma unroll
        for (int j = 0; j < 8; j++) out[j] = p[j];
    }
};
template <> struct Decode8<TURQ_F16> {
    __device__ static void run(const uint8_t *row, int64_t e0, float *out) {
        const uint16_t *p = (const uint16_t *)row + e0;
#pragma unroll
        for (int j = 0; j < 8; j++) out[j] = turq_h2f(p[j]);
    }
};
template <> struct Decode8<TURQ_BF16> {
    __device__ static void run(const uint8_t *row, int64_t e0, float *out) {
        const uint16_t *p = (const uint16_t *)row + e0;
#pragma unroll
        for (int j = 0; j < 8; j++) out[j] = turq_bf2f(p[j]);
    }
};

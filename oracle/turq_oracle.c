/*
 * turq_oracle.c — CPU restatement of the GGUF block-quantized matmul that the
 * reference runs for every linear layer (test infrastructure, NOT product code).
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load
 * this file's shared library.  The product path (tur_amd/, libturq.so) never
 * links, imports or calls it.
 *
 * What it restates.  The reference (danylokravchenko/tur) holds no quantized
 * arithmetic of its own; it calls candle-core 0.10.2 (pinned in the reference's
 * Cargo.lock:317-320), which is not vendored in the reference tree:
 *   - src/models/layers/linear.rs:19-31   LinearX::forward -> QMatMul::forward
 *   - src/models/layers/linear.rs:59-70   QMatMul::from_arc(qweight), bias dequantized
 *   - src/weights/gguf_varbuilder.rs:72-74 Content::tensor -> QTensor (raw blocks, shape (N,K))
 *   - src/weights/mod.rs:150,161; src/models/layers/mod.rs:37; norm.rs:84  QTensor::dequantize
 * Each function below restates the published candle / ggml algorithm
 * (candle-core quantized/k_quants.rs: BlockQ8_0, BlockQ4K, BlockQ5K, BlockQ6K,
 * BlockQ8K with to_float / from_float / vec_dot_unopt, and k_quants::matmul).
 *
 * PARITY UNPINNED (no executable candle, no golden vectors in the reference):
 *   - the f32 operation ORDER inside to_float for Q4_K/Q5_K/Q6_K (restated as
 *     unfused, left to right: (d*sc)*q - (dmin*m); (d*sc)*q for Q6_K),
 *   - the rounding / clamp details of BlockQ8K::from_float and BlockQ8_0::from_float
 *     (f32::round = half away from zero; Q8_K clamps with min(127)),
 *   - the f32 summation order of the SIMD vec_dot variants (scalar order is restated).
 * Everything else (byte layouts, bit-field unpacking, integer dot products) is
 * pinned by known-answer tests and by an independent NumPy restatement that must
 * agree bit for bit (tests/test_oracle_*.py).
 *
 * Build with -ffp-contract=off so that a*b-c stays two separately rounded ops
 * (Rust never contracts).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define QK8_0 32
#define QK_K 256
#define K_SCALE_SIZE 12

/* ggml dtype ids as stored in GGUF tensor infos */
enum {
    ORC_F32 = 0,
    ORC_F16 = 1,
    ORC_Q8_0 = 8,
    ORC_Q4_K = 12,
    ORC_Q5_K = 13,
    ORC_Q6_K = 14,
    ORC_Q8_K = 15,
    ORC_BF16 = 30
};

#pragma pack(push, 1)
typedef struct { uint16_t d; int8_t qs[QK8_0]; } block_q8_0;                                   /* 34 */
typedef struct { uint16_t d, dmin; uint8_t scales[K_SCALE_SIZE]; uint8_t qs[QK_K / 2]; } block_q4_K; /* 144 */
typedef struct { uint16_t d, dmin; uint8_t scales[K_SCALE_SIZE]; uint8_t qh[QK_K / 8]; uint8_t qs[QK_K / 2]; } block_q5_K; /* 176 */
typedef struct { uint8_t ql[QK_K / 2]; uint8_t qh[QK_K / 4]; int8_t scales[QK_K / 16]; uint16_t d; } block_q6_K; /* 210 */
typedef struct { float d; int8_t qs[QK_K]; int16_t bsums[QK_K / 16]; } block_q8_K;             /* 292 */
#pragma pack(pop)

_Static_assert(sizeof(block_q8_0) == 34, "q8_0");
_Static_assert(sizeof(block_q4_K) == 144, "q4_K");
_Static_assert(sizeof(block_q5_K) == 176, "q5_K");
_Static_assert(sizeof(block_q6_K) == 210, "q6_K");
_Static_assert(sizeof(block_q8_K) == 292, "q8_K");

/* ---------- scalar conversions (half::f16 semantics: to_f32 exact, from_f32 RNE) ---------- */

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while ((man & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((ax > 0x7F800000u) ? (0x200u | ((ax >> 13) & 0x3FFu)) : 0));
    }
    if (ax >= 0x477FF000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (ax < 0x33000001u) { /* <= 2^-25: rounds to zero (tie at exactly 2^-25 goes to even = 0) */
        return sign;
    }
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7FFFFFu) | 0x800000u;
    uint32_t shift;
    uint32_t base;
    if (e < -14) { /* subnormal half */
        shift = (uint32_t)(13 + (-14 - e));
        base = 0;
    } else {
        shift = 13;
        base = ((uint32_t)(e + 15) << 10) - 0x400u; /* implicit bit adds the 0x400 back */
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | (base + q));
}

float orc_bf16_to_f32(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t orc_f32_to_bf16(float f) { /* RNE, NaN kept quiet */
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x40u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7FFFu + lsb;
    return (uint16_t)(x >> 16);
}

/* ---------- geometry ---------- */

int orc_block_elems(int dtype) {
    switch (dtype) {
    case ORC_F32: case ORC_F16: case ORC_BF16: return 1;
    case ORC_Q8_0: return QK8_0;
    case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: case ORC_Q8_K: return QK_K;
    default: return 0;
    }
}

int orc_block_bytes(int dtype) {
    switch (dtype) {
    case ORC_F32: return 4;
    case ORC_F16: case ORC_BF16: return 2;
    case ORC_Q8_0: return 34;
    case ORC_Q4_K: return 144;
    case ORC_Q5_K: return 176;
    case ORC_Q6_K: return 210;
    case ORC_Q8_K: return 292;
    default: return 0;
    }
}

/* 6-bit scale/min unpack shared by Q4_K and Q5_K (candle k_quants get_scale_min_k4) */
static inline void get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* ---------- to_float (QTensor::dequantize) ---------- */

static void dequant_q8_0(const block_q8_0 *x, int64_t nb, float *y) {
    for (int64_t i = 0; i < nb; i++) {
        float d = orc_f16_to_f32(x[i].d);
        for (int j = 0; j < QK8_0; j++) y[i * QK8_0 + j] = (float)x[i].qs[j] * d;
    }
}

static void dequant_q4_K(const block_q4_K *x, int64_t nb, float *y) {
    for (int64_t i = 0; i < nb; i++) {
        const float d = orc_f16_to_f32(x[i].d);
        const float min = orc_f16_to_f32(x[i].dmin);
        const uint8_t *q = x[i].qs;
        int is = 0;
        for (int j = 0; j < QK_K; j += 64) {
            uint8_t sc, m;
            get_scale_min_k4(is, x[i].scales, &sc, &m);
            const float d1 = d * (float)sc, m1 = min * (float)m;
            get_scale_min_k4(is + 1, x[i].scales, &sc, &m);
            const float d2 = d * (float)sc, m2 = min * (float)m;
            for (int l = 0; l < 32; l++) *y++ = d1 * (float)(q[l] & 0xF) - m1;
            for (int l = 0; l < 32; l++) *y++ = d2 * (float)(q[l] >> 4) - m2;
            q += 32;
            is += 2;
        }
    }
}

static void dequant_q5_K(const block_q5_K *x, int64_t nb, float *y) {
    for (int64_t i = 0; i < nb; i++) {
        const float d = orc_f16_to_f32(x[i].d);
        const float min = orc_f16_to_f32(x[i].dmin);
        const uint8_t *ql = x[i].qs;
        const uint8_t *qh = x[i].qh;
        int is = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0; j < QK_K; j += 64) {
            uint8_t sc, m;
            get_scale_min_k4(is, x[i].scales, &sc, &m);
            const float d1 = d * (float)sc, m1 = min * (float)m;
            get_scale_min_k4(is + 1, x[i].scales, &sc, &m);
            const float d2 = d * (float)sc, m2 = min * (float)m;
            for (int l = 0; l < 32; l++) {
                float to_add = (qh[l] & u1) ? 16.0f : 0.0f;
                *y++ = d1 * ((float)(ql[l] & 0xF) + to_add) - m1;
            }
            for (int l = 0; l < 32; l++) {
                float to_add = (qh[l] & u2) ? 16.0f : 0.0f;
                *y++ = d2 * ((float)(ql[l] >> 4) + to_add) - m2;
            }
            ql += 32;
            is += 2;
            u1 <<= 2;
            u2 <<= 2;
        }
    }
}

static void dequant_q6_K(const block_q6_K *x, int64_t nb, float *y) {
    for (int64_t i = 0; i < nb; i++) {
        const float d = orc_f16_to_f32(x[i].d);
        const uint8_t *ql = x[i].ql;
        const uint8_t *qh = x[i].qh;
        const int8_t *sc = x[i].scales;
        for (int n = 0; n < QK_K; n += 128) {
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                const int8_t q1 = (int8_t)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                const int8_t q2 = (int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                const int8_t q3 = (int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                const int8_t q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                y[l] = d * (float)sc[is + 0] * (float)q1;
                y[l + 32] = d * (float)sc[is + 2] * (float)q2;
                y[l + 64] = d * (float)sc[is + 4] * (float)q3;
                y[l + 96] = d * (float)sc[is + 6] * (float)q4;
            }
            y += 128;
            ql += 64;
            qh += 32;
            sc += 8;
        }
    }
}

/* blocks -> f32; nelem must be a multiple of the block size. Returns 0 / -1. */
int orc_dequantize(int dtype, const void *blocks, int64_t nelem, float *out) {
    int be = orc_block_elems(dtype);
    if (be == 0 || nelem % be != 0) return -1;
    int64_t nb = nelem / be;
    switch (dtype) {
    case ORC_F32: memcpy(out, blocks, (size_t)nelem * 4); return 0;
    case ORC_F16: for (int64_t i = 0; i < nelem; i++) out[i] = orc_f16_to_f32(((const uint16_t *)blocks)[i]); return 0;
    case ORC_BF16: for (int64_t i = 0; i < nelem; i++) out[i] = orc_bf16_to_f32(((const uint16_t *)blocks)[i]); return 0;
    case ORC_Q8_0: dequant_q8_0((const block_q8_0 *)blocks, nb, out); return 0;
    case ORC_Q4_K: dequant_q4_K((const block_q4_K *)blocks, nb, out); return 0;
    case ORC_Q5_K: dequant_q5_K((const block_q5_K *)blocks, nb, out); return 0;
    case ORC_Q6_K: dequant_q6_K((const block_q6_K *)blocks, nb, out); return 0;
    default: return -1;
    }
}

/* ---------- from_float (activation quantisation) ---------- */

static inline int8_t sat_i8(float v) { /* Rust `as i8`: saturating, NaN -> 0 */
    if (v != v) return 0;
    if (v <= -128.0f) return -128;
    if (v >= 127.0f) return 127;
    return (int8_t)v;
}

/* BlockQ8_0::from_float */
int orc_quantize_q8_0(const float *x, int64_t k, void *out) {
    if (k % QK8_0 != 0) return -1;
    block_q8_0 *y = (block_q8_0 *)out;
    for (int64_t i = 0; i < k / QK8_0; i++) {
        const float *xs = x + i * QK8_0;
        float amax = 0.0f;
        for (int j = 0; j < QK8_0; j++) {
            float a = fabsf(xs[j]);
            if (a > amax) amax = a; /* f32::max */
        }
        const float d = amax / 127.0f;
        const float id = (d != 0.0f) ? 1.0f / d : 0.0f;
        y[i].d = orc_f32_to_f16(d);
        for (int j = 0; j < QK8_0; j++) y[i].qs[j] = sat_i8(roundf(xs[j] * id));
    }
    return 0;
}

/* BlockQ8K::from_float */
int orc_quantize_q8_K(const float *x, int64_t k, void *out) {
    if (k % QK_K != 0) return -1;
    block_q8_K *y = (block_q8_K *)out;
    for (int64_t i = 0; i < k / QK_K; i++) {
        const float *xs = x + i * QK_K;
        float max = 0.0f, amax = 0.0f;
        for (int j = 0; j < QK_K; j++) {
            float a = fabsf(xs[j]);
            if (amax < a) { amax = a; max = xs[j]; }
        }
        if (amax == 0.0f) {
            y[i].d = 0.0f;
            memset(y[i].qs, 0, QK_K);
            memset(y[i].bsums, 0, sizeof(y[i].bsums)); /* candle leaves the zero-initialised value */
            continue;
        }
        const float iscale = -128.0f / max;
        for (int j = 0; j < QK_K; j++) {
            float v = roundf(iscale * xs[j]);
            y[i].qs[j] = sat_i8(fminf(v, 127.0f));
        }
        for (int j = 0; j < QK_K / 16; j++) {
            int sum = 0;
            for (int ii = 0; ii < 16; ii++) sum += y[i].qs[j * 16 + ii];
            y[i].bsums[j] = (int16_t)sum;
        }
        y[i].d = 1.0f / iscale;
    }
    return 0;
}

/* ---------- vec_dot (scalar order of candle's vec_dot_unopt) ---------- */

static float vec_dot_q8_0_q8_0(int64_t k, const block_q8_0 *x, const block_q8_0 *y) {
    float sumf = 0.0f;
    for (int64_t i = 0; i < k / QK8_0; i++) {
        int32_t sumi = 0;
        for (int j = 0; j < QK8_0; j++) sumi += (int32_t)x[i].qs[j] * (int32_t)y[i].qs[j];
        sumf += (float)sumi * orc_f16_to_f32(x[i].d) * orc_f16_to_f32(y[i].d);
    }
    return sumf;
}

/* 6-bit unpack the way vec_dot does it (32-bit mask arithmetic); must equal get_scale_min_k4 */
static void unpack_scales_mins_u32(const uint8_t *packed, uint8_t *scales, uint8_t *mins) {
    const uint32_t kmask1 = 0x3f3f3f3fu, kmask2 = 0x0f0f0f0fu, kmask3 = 0x03030303u;
    uint32_t utmp[4];
    memcpy(utmp, packed, 12);
    utmp[3] = ((utmp[2] >> 4) & kmask2) | (((utmp[1] >> 6) & kmask3) << 4);
    const uint32_t uaux = utmp[1] & kmask1;
    utmp[1] = (utmp[2] & kmask2) | (((utmp[0] >> 6) & kmask3) << 4);
    utmp[2] = uaux;
    utmp[0] &= kmask1;
    memcpy(scales, &utmp[0], 8);
    memcpy(mins, &utmp[2], 8);
}

static float vec_dot_q4_K_q8_K(int64_t k, const block_q4_K *x, const block_q8_K *y) {
    uint8_t scales[8], mins[8];
    int8_t aux8[QK_K];
    int16_t aux16[8];
    float sums[8] = {0};
    int32_t aux32[8];
    float sumf = 0.0f;
    for (int64_t i = 0; i < k / QK_K; i++) {
        const uint8_t *q4 = x[i].qs;
        const int8_t *q8 = y[i].qs;
        memset(aux32, 0, sizeof(aux32));
        int8_t *a = aux8;
        for (int j = 0; j < QK_K / 64; j++) {
            for (int l = 0; l < 32; l++) a[l] = (int8_t)(q4[l] & 0xF);
            a += 32;
            for (int l = 0; l < 32; l++) a[l] = (int8_t)(q4[l] >> 4);
            a += 32;
            q4 += 32;
        }
        unpack_scales_mins_u32(x[i].scales, scales, mins);
        int32_t sumi = 0;
        for (int j = 0; j < QK_K / 16; j++) sumi += (int32_t)y[i].bsums[j] * (int32_t)mins[j / 2];
        a = aux8;
        for (int is = 0; is < 8; is++) {
            int32_t scale = scales[is];
            for (int g = 0; g < 4; g++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)(q8[l] * a[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * aux16[l];
                q8 += 8;
                a += 8;
            }
        }
        const float d = orc_f16_to_f32(x[i].d) * y[i].d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
        const float dmin = orc_f16_to_f32(x[i].dmin) * y[i].d;
        sumf -= dmin * (float)sumi;
    }
    float s = 0.0f;
    for (int l = 0; l < 8; l++) s += sums[l];
    return sumf + s;
}

static float vec_dot_q5_K_q8_K(int64_t k, const block_q5_K *x, const block_q8_K *y) {
    uint8_t scales[8], mins[8];
    int8_t aux8[QK_K];
    int16_t aux16[8];
    float sums[8] = {0};
    int32_t aux32[8];
    float sumf = 0.0f;
    for (int64_t i = 0; i < k / QK_K; i++) {
        const uint8_t *q4 = x[i].qs;
        const uint8_t *hm = x[i].qh;
        const int8_t *q8 = y[i].qs;
        memset(aux32, 0, sizeof(aux32));
        int8_t *a = aux8;
        uint8_t m = 1;
        for (int j = 0; j < QK_K / 64; j++) {
            for (int l = 0; l < 32; l++) a[l] = (int8_t)((q4[l] & 0xF) + ((hm[l] & m) ? 16 : 0));
            a += 32;
            m <<= 1;
            for (int l = 0; l < 32; l++) a[l] = (int8_t)((q4[l] >> 4) + ((hm[l] & m) ? 16 : 0));
            a += 32;
            m <<= 1;
            q4 += 32;
        }
        unpack_scales_mins_u32(x[i].scales, scales, mins);
        int32_t sumi = 0;
        for (int j = 0; j < QK_K / 16; j++) sumi += (int32_t)y[i].bsums[j] * (int32_t)mins[j / 2];
        a = aux8;
        for (int is = 0; is < 8; is++) {
            int32_t scale = scales[is];
            for (int g = 0; g < 4; g++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)(q8[l] * a[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * aux16[l];
                q8 += 8;
                a += 8;
            }
        }
        const float d = orc_f16_to_f32(x[i].d) * y[i].d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
        const float dmin = orc_f16_to_f32(x[i].dmin) * y[i].d;
        sumf -= dmin * (float)sumi;
    }
    float s = 0.0f;
    for (int l = 0; l < 8; l++) s += sums[l];
    return sumf + s;
}

static float vec_dot_q6_K_q8_K(int64_t k, const block_q6_K *x, const block_q8_K *y) {
    int8_t aux8[QK_K];
    int16_t aux16[8];
    float sums[8] = {0};
    int32_t aux32[8];
    for (int64_t i = 0; i < k / QK_K; i++) {
        const uint8_t *q4 = x[i].ql;
        const uint8_t *qh = x[i].qh;
        const int8_t *q8 = y[i].qs;
        memset(aux32, 0, sizeof(aux32));
        int8_t *a = aux8;
        for (int j = 0; j < QK_K; j += 128) {
            for (int l = 0; l < 32; l++) {
                a[l] = (int8_t)((q4[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                a[l + 32] = (int8_t)((q4[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                a[l + 64] = (int8_t)((q4[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                a[l + 96] = (int8_t)((q4[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            }
            a += 128;
            q4 += 64;
            qh += 32;
        }
        a = aux8;
        for (int is = 0; is < QK_K / 16; is++) {
            int32_t scale = x[i].scales[is];
            for (int g = 0; g < 2; g++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)(q8[l] * a[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * aux16[l];
                q8 += 8;
                a += 8;
            }
        }
        const float d = orc_f16_to_f32(x[i].d) * y[i].d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
    }
    float s = 0.0f;
    for (int l = 0; l < 8; l++) s += sums[l];
    return s;
}

/* dtype of the activation blocks a weight dtype is dotted with (GgmlType::VecDotType) */
int orc_vec_dot_type(int dtype) {
    switch (dtype) {
    case ORC_Q8_0: return ORC_Q8_0;
    case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: return ORC_Q8_K;
    default: return -1;
    }
}

/* one weight row (k elements) times one quantised activation row */
float orc_vec_dot(int dtype, int64_t k, const void *wrow, const void *actq) {
    switch (dtype) {
    case ORC_Q8_0: return vec_dot_q8_0_q8_0(k, (const block_q8_0 *)wrow, (const block_q8_0 *)actq);
    case ORC_Q4_K: return vec_dot_q4_K_q8_K(k, (const block_q4_K *)wrow, (const block_q8_K *)actq);
    case ORC_Q5_K: return vec_dot_q5_K_q8_K(k, (const block_q5_K *)wrow, (const block_q8_K *)actq);
    case ORC_Q6_K: return vec_dot_q6_K_q8_K(k, (const block_q6_K *)wrow, (const block_q8_K *)actq);
    default: return NAN;
    }
}

/* ---------- k_quants::matmul (QMatMul::forward on CPU) ----------
 * lhs f32 [m,k] row-major, rhs blocks [n, k/blk], dst f32 [m,n].
 * Activations are quantised row by row first, then rows are processed serially and
 * the n output columns in parallel (candle: rayon, here OpenMP with nthreads threads). */
int orc_qmatmul(int dtype, int64_t m, int64_t k, int64_t n, const float *lhs, const void *rhs,
                float *dst, int nthreads) {
    int vdt = orc_vec_dot_type(dtype);
    if (vdt < 0) return -1;
    int be = orc_block_elems(dtype), vbe = orc_block_elems(vdt);
    if (k % be != 0 || k % vbe != 0) return -1;
    size_t row_bytes = (size_t)(k / be) * (size_t)orc_block_bytes(dtype);
    size_t act_row_bytes = (size_t)(k / vbe) * (size_t)orc_block_bytes(vdt);
    uint8_t *lhs_q = (uint8_t *)calloc((size_t)m, act_row_bytes);
    if (!lhs_q) return -2;
    for (int64_t r = 0; r < m; r++) {
        if (vdt == ORC_Q8_0) orc_quantize_q8_0(lhs + r * k, k, lhs_q + (size_t)r * act_row_bytes);
        else orc_quantize_q8_K(lhs + r * k, k, lhs_q + (size_t)r * act_row_bytes);
    }
    if (nthreads < 1) nthreads = 1;
    for (int64_t r = 0; r < m; r++) {
        const uint8_t *arow = lhs_q + (size_t)r * act_row_bytes;
        float *drow = dst + r * n;
#pragma omp parallel for schedule(dynamic, 128) num_threads(nthreads)
        for (int64_t c = 0; c < n; c++) {
            drow[c] = orc_vec_dot(dtype, k, (const uint8_t *)rhs + (size_t)c * row_bytes, arow);
        }
    }
    free(lhs_q);
    return 0;
}

/* Dense comparator: y = x * dequantize(W)^T with f64 accumulation over the f32 dequantised
 * weights (the "f32 matmul on dequantised weights" of the parity bar, made order-independent). */
int orc_matmul_dequant(int dtype, int64_t m, int64_t k, int64_t n, const float *lhs,
                       const void *rhs, float *dst, int nthreads) {
    int be = orc_block_elems(dtype);
    if (be == 0 || k % be != 0) return -1;
    size_t row_bytes = (size_t)(k / be) * (size_t)orc_block_bytes(dtype);
    if (nthreads < 1) nthreads = 1;
    int err = 0;
#pragma omp parallel num_threads(nthreads)
    {
        float *w = (float *)malloc((size_t)k * sizeof(float));
        if (!w) {
#pragma omp atomic write
            err = -2;
        }
#pragma omp for schedule(dynamic, 64)
        for (int64_t c = 0; c < n; c++) {
            if (!w) continue;
            orc_dequantize(dtype, (const uint8_t *)rhs + (size_t)c * row_bytes, k, w);
            for (int64_t r = 0; r < m; r++) {
                const float *x = lhs + r * k;
                double acc = 0.0;
                for (int64_t i = 0; i < k; i++) acc += (double)x[i] * (double)w[i];
                dst[r * n + c] = (float)acc;
            }
        }
        free(w);
    }
    return err;
}

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

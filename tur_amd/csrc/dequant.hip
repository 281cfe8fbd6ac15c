// Bit-exact device counterparts of candle's `to_float` (QTensor::dequantize) and `from_float`
// (BlockQ8_0 / BlockQ8K activation quantisation).  This translation unit is compiled with
// -ffp-contract=off: every multiply and subtract is rounded on its own, as in the Rust code.
#include "block_decode.h"
#include "layout.h"

namespace {

template <int DT>
__global__ void __launch_bounds__(256) dequant_native_kernel(const uint8_t *__restrict__ w, int64_t k,
                                                             int64_t row_bytes, int64_t ngroups,
                                                             float *__restrict__ out) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= ngroups) return;
    const int64_t e = t * 8;
    const int64_t row = e / k;
    const int64_t e0 = e - row * k;
    float v[8];
    Decode8<DT>::run(w + row * row_bytes, e0, v);
    float4 *o = (float4 *)(out + e);
    o[0] = make_float4(v[0], v[1], v[2], v[3]);
    o[1] = make_float4(v[4], v[5], v[6], v[7]);
}

// Tiled layout: one thread rebuilds one native block in private memory and decodes it.  Load-time
// only, so clarity wins over speed here.
template <int DT>
__global__ void __launch_bounds__(64) dequant_tiled_kernel(const uint8_t *__restrict__ w, int64_t k,
                                                           int64_t nblocks_total, float *__restrict__ out) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= nblocks_total) return;
    constexpr int BE = TiledFmt<DT>::kBlockElems;
    constexpr int BB = TiledFmt<DT>::kBlockBytes;
    const int64_t bpr = k / BE;
    const int64_t row = t / bpr;
    const int64_t b = t - row * bpr;
    uint8_t blk[BB];
    for (int i = 0; i < BB; i++) blk[i] = 0;
    turq_untile_block<DT>(w, k, row, b, blk);
    float *o = out + row * k + b * BE;
    for (int e0 = 0; e0 < BE; e0 += 8) {
        float v[8];
        Decode8<DT>::run(blk, e0, v);
        float4 *o4 = (float4 *)(o + e0);
        o4[0] = make_float4(v[0], v[1], v[2], v[3]);
        o4[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
}

template <int DT>
__global__ void __launch_bounds__(256) dequant_dense_kernel(const uint8_t *__restrict__ w, int64_t nelem,
                                                            float *__restrict__ out) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= nelem) return;
    if (DT == TURQ_F32) out[t] = ((const float *)w)[t];
    else if (DT == TURQ_F16) out[t] = turq_h2f(((const uint16_t *)w)[t]);
    else out[t] = turq_bf2f(((const uint16_t *)w)[t]);
}

// ---- rows picked by index (the embedding lookup) ----
// out[i][:] = dequantize(W)[ids[i]][:], the same per-element arithmetic as the kernels above; an index past the table gives a
// row of NaN (the device cannot report it otherwise).  OT = output type.

__device__ inline void store_as(void *out, int ot, int64_t at, float v) {
    if (ot == TURQ_ACT_F32) ((float *)out)[at] = v;
    else if (ot == TURQ_ACT_BF16) {
        uint32_t u = __float_as_uint(v);
        uint16_t b;
        if ((u & 0x7FFFFFFFu) > 0x7F800000u) b = (uint16_t)((u >> 16) | 0x40u);
        else b = (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);  // round to nearest even
        ((uint16_t *)out)[at] = b;
    } else {
        const _Float16 h = (_Float16)v;
        uint16_t b;
        __builtin_memcpy(&b, &h, 2);
        ((uint16_t *)out)[at] = b;
    }
}

template <int DT>
__global__ void __launch_bounds__(256) gather_native_kernel(const uint8_t *__restrict__ w, int64_t n, int64_t k, int64_t row_bytes,
                                                            const uint32_t *__restrict__ ids, int64_t ngroups, void *__restrict__ out,
                                                            int ot, int64_t ldo, bool vec) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= ngroups) return;
    const int64_t gpr = k / 8;
    const int64_t i = t / gpr, e0 = (t - i * gpr) * 8;
    const int64_t row = ids[i];
    float v[8];
    if (row < n) Decode8<DT>::run(w + row * row_bytes, e0, v);
    else
        for (int j = 0; j < 8; j++) v[j] = __uint_as_float(0x7FC00000u);
    if (ot == TURQ_ACT_F32 && vec) {  // rows of 16-byte aligned f32: two 16-byte stores
        float4 *o = (float4 *)((float *)out + i * ldo + e0);
        o[0] = make_float4(v[0], v[1], v[2], v[3]);
        o[1] = make_float4(v[4], v[5], v[6], v[7]);
        return;
    }
    for (int j = 0; j < 8; j++) store_as(out, ot, i * ldo + e0 + j, v[j]);
}

template <int DT>
__global__ void __launch_bounds__(64) gather_tiled_kernel(const uint8_t *__restrict__ w, int64_t n, int64_t k,
                                                          const uint32_t *__restrict__ ids, int64_t nblocks_total,
                                                          void *__restrict__ out, int ot, int64_t ldo) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= nblocks_total) return;
    constexpr int BE = TiledFmt<DT>::kBlockElems;
    constexpr int BB = TiledFmt<DT>::kBlockBytes;
    const int64_t bpr = k / BE;
    const int64_t i = t / bpr, b = t - i * bpr;
    const int64_t row = ids[i];
    uint8_t blk[BB];
    for (int j = 0; j < BB; j++) blk[j] = 0;
    if (row < n) turq_untile_block<DT>(w, k, row, b, blk);
    for (int e0 = 0; e0 < BE; e0 += 8) {
        float v[8];
        Decode8<DT>::run(blk, e0, v);
        for (int j = 0; j < 8; j++) store_as(out, ot, i * ldo + b * BE + e0 + j, row < n ? v[j] : __uint_as_float(0x7FC00000u));
    }
}

template <int DT>
__global__ void __launch_bounds__(256) gather_dense_kernel(const uint8_t *__restrict__ w, int64_t n, int64_t k,
                                                           const uint32_t *__restrict__ ids, int64_t nelem, void *__restrict__ out,
                                                           int ot, int64_t ldo) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= nelem) return;
    const int64_t i = t / k, e = t - i * k;
    const int64_t row = ids[i];
    float v = __uint_as_float(0x7FC00000u);
    if (row < n) {
        const int64_t at = row * k + e;
        if (DT == TURQ_F32) v = ((const float *)w)[at];
        else if (DT == TURQ_F16) v = turq_h2f(((const uint16_t *)w)[at]);
        else v = turq_bf2f(((const uint16_t *)w)[at]);
    }
    store_as(out, ot, i * ldo + e, v);
}

template <int DT>
hipError_t launch_quant_gather(int layout, const void *w, int64_t n, int64_t k, const uint32_t *ids, int64_t count, void *out, int ot,
                               int64_t ldo, hipStream_t s) {
    if (layout == TURQ_LAYOUT_NATIVE) {
        const int64_t ngroups = count * (k / 8);
        const int64_t row_bytes = k / turq_dt_block_elems(DT) * turq_dt_block_bytes(DT);
        const bool vec = ((uintptr_t)out % 16 == 0) && ldo % 4 == 0;
        gather_native_kernel<DT><<<(unsigned)((ngroups + 255) / 256), 256, 0, s>>>((const uint8_t *)w, n, k, row_bytes, ids, ngroups, out,
                                                                                   ot, ldo, vec);
    } else {
        const int64_t nblk = count * (k / turq_dt_block_elems(DT));
        gather_tiled_kernel<DT><<<(unsigned)((nblk + 63) / 64), 64, 0, s>>>((const uint8_t *)w, n, k, ids, nblk, out, ot, ldo);
    }
    return hipGetLastError();
}

template <int DT>
hipError_t launch_dense_gather(const void *w, int64_t n, int64_t k, const uint32_t *ids, int64_t count, void *out, int ot, int64_t ldo,
                               hipStream_t s) {
    const int64_t nelem = count * k;
    gather_dense_kernel<DT><<<(unsigned)((nelem + 255) / 256), 256, 0, s>>>((const uint8_t *)w, n, k, ids, nelem, out, ot, ldo);
    return hipGetLastError();
}

// ---- activation quantisation ----

// Rust `as i8` on an f32 that is already integral: saturate.
__device__ inline int8_t sat_i8(float v) {
    if (!(v == v)) return 0;
    if (v <= -128.0f) return -128;
    if (v >= 127.0f) return 127;
    return (int8_t)v;
}

// One 32-lane half wave per Q8_0 block (two blocks per wave).
__global__ void __launch_bounds__(256) quantize_q8_0_kernel(const float *__restrict__ x, int64_t nblocks,
                                                            uint8_t *__restrict__ out) {
#pragma clang fp contract(off)
    const int64_t blk = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 5;
    const int j = threadIdx.x & 31;
    const bool live = blk < nblocks;
    const float v = live ? x[blk * 32 + j] : 0.0f;
    float amax = fabsf(v);
#pragma unroll
    for (int off = 16; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 32));
    const float d = amax / 127.0f;
    const float id = (d != 0.0f) ? 1.0f / d : 0.0f;
    if (!live) return;
    uint8_t *o = out + blk * 34;
    if (j == 0) {
        const _Float16 h = (_Float16)d;  // round to nearest even
        uint16_t bits;
        __builtin_memcpy(&bits, &h, 2);
        o[0] = (uint8_t)(bits & 0xFF);
        o[1] = (uint8_t)(bits >> 8);
    }
    o[2 + j] = (uint8_t)sat_i8(roundf(v * id));
}

// One wave per Q8_K block: lane j owns elements 4j..4j+3.
__global__ void __launch_bounds__(256) quantize_q8_k_kernel(const float *__restrict__ x, int64_t nblocks,
                                                            uint8_t *__restrict__ out) {
#pragma clang fp contract(off)
    const int64_t blk = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (blk >= nblocks) return;  // whole wave leaves together
    const float4 v4 = ((const float4 *)(x + blk * 256))[lane];
    const float v[4] = {v4.x, v4.y, v4.z, v4.w};
    // first element with the largest |x| (strictly greater wins, so ties keep the earlier index)
    float amax = 0.0f, mx = 0.0f;
    int idx = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float a = fabsf(v[i]);
        if (amax < a) { amax = a; mx = v[i]; idx = lane * 4 + i; }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float oa = __shfl_xor(amax, off, 64);
        const float om = __shfl_xor(mx, off, 64);
        const int oi = __shfl_xor(idx, off, 64);
        if (oa > amax || (oa == amax && oi < idx)) { amax = oa; mx = om; idx = oi; }
    }
    uint8_t *o = out + blk * 292;
    int q[4] = {0, 0, 0, 0};
    float d = 0.0f;
    if (amax != 0.0f) {
        const float iscale = -128.0f / mx;
#pragma unroll
        for (int i = 0; i < 4; i++) q[i] = (int)sat_i8(fminf(roundf(iscale * v[i]), 127.0f));
        d = 1.0f / iscale;
    }
    // bsums: 16 elements = 4 lanes
    int s = q[0] + q[1] + q[2] + q[3];
    s += __shfl_xor(s, 1, 64);
    s += __shfl_xor(s, 2, 64);
    uint32_t packed = (uint32_t)(uint8_t)q[0] | ((uint32_t)(uint8_t)q[1] << 8) | ((uint32_t)(uint8_t)q[2] << 16) |
                      ((uint32_t)(uint8_t)q[3] << 24);
    ((uint32_t *)(o + 4))[lane] = packed;  // 292-byte blocks keep 4-byte alignment
    if ((lane & 3) == 0) ((int16_t *)(o + 260))[lane >> 2] = (int16_t)s;
    if (lane == 0) *(float *)o = d;
}

template <int DT>
hipError_t launch_quant_dequant(int layout, const void *w, int64_t n, int64_t k, float *out, hipStream_t s) {
    const int64_t ngroups = n * k / 8;
    if (ngroups == 0) return hipSuccess;
    const unsigned grid = (unsigned)((ngroups + 255) / 256);
    if (layout == TURQ_LAYOUT_NATIVE) {
        const int64_t row_bytes = k / turq_dt_block_elems(DT) * turq_dt_block_bytes(DT);
        dequant_native_kernel<DT><<<grid, 256, 0, s>>>((const uint8_t *)w, k, row_bytes, ngroups, out);
    } else {
        const int64_t nblk = n * (k / turq_dt_block_elems(DT));
        dequant_tiled_kernel<DT><<<(unsigned)((nblk + 63) / 64), 64, 0, s>>>((const uint8_t *)w, k, nblk, out);
    }
    return hipGetLastError();
}

template <int DT>
hipError_t launch_dense_dequant(const void *w, int64_t nelem, float *out, hipStream_t s) {
    if (nelem == 0) return hipSuccess;
    dequant_dense_kernel<DT><<<(unsigned)((nelem + 255) / 256), 256, 0, s>>>((const uint8_t *)w, nelem, out);
    return hipGetLastError();
}

}  // namespace

hipError_t turq_launch_dequant(int dtype, int layout, const void *w, int64_t n, int64_t k, float *out,
                               hipStream_t stream) {
    switch (dtype) {
    case TURQ_Q8_0: return launch_quant_dequant<TURQ_Q8_0>(layout, w, n, k, out, stream);
    case TURQ_Q4_K: return launch_quant_dequant<TURQ_Q4_K>(layout, w, n, k, out, stream);
    case TURQ_Q5_K: return launch_quant_dequant<TURQ_Q5_K>(layout, w, n, k, out, stream);
    case TURQ_Q6_K: return launch_quant_dequant<TURQ_Q6_K>(layout, w, n, k, out, stream);
    case TURQ_F32: return launch_dense_dequant<TURQ_F32>(w, n * k, out, stream);
    case TURQ_F16: return launch_dense_dequant<TURQ_F16>(w, n * k, out, stream);
    case TURQ_BF16: return launch_dense_dequant<TURQ_BF16>(w, n * k, out, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t turq_launch_quantize_q8_0(const float *x, int64_t nblocks, void *out, hipStream_t stream) {
    if (nblocks == 0) return hipSuccess;
    const int64_t threads = nblocks * 32;
    quantize_q8_0_kernel<<<(unsigned)((threads + 255) / 256), 256, 0, stream>>>(x, nblocks, (uint8_t *)out);
    return hipGetLastError();
}

hipError_t turq_launch_quantize_q8_k(const float *x, int64_t nblocks, void *out, hipStream_t stream) {
    if (nblocks == 0) return hipSuccess;
    const int64_t threads = nblocks * 64;
    quantize_q8_k_kernel<<<(unsigned)((threads + 255) / 256), 256, 0, stream>>>(x, nblocks, (uint8_t *)out);
    return hipGetLastError();
}

// out[i][0..k) = dequantize(W)[ids[i]] for i < count, rows of `out` ldo elements apart, stored as out_dtype (TURQ_ACT_*)
hipError_t turq_launch_gather_rows(int dtype, int layout, const void *w, int64_t n, int64_t k, const uint32_t *ids, int64_t count,
                                   void *out, int out_dtype, int64_t ldo, hipStream_t stream) {
    if (count <= 0 || k <= 0) return hipSuccess;
    if (out_dtype != TURQ_ACT_F32 && out_dtype != TURQ_ACT_BF16 && out_dtype != TURQ_ACT_F16) return hipErrorInvalidValue;
    if (count * k / 8 > 0x7FFFFFFFLL * 64) return hipErrorInvalidValue;
    switch (dtype) {
    case TURQ_Q8_0: return launch_quant_gather<TURQ_Q8_0>(layout, w, n, k, ids, count, out, out_dtype, ldo, stream);
    case TURQ_Q4_K: return launch_quant_gather<TURQ_Q4_K>(layout, w, n, k, ids, count, out, out_dtype, ldo, stream);
    case TURQ_Q5_K: return launch_quant_gather<TURQ_Q5_K>(layout, w, n, k, ids, count, out, out_dtype, ldo, stream);
    case TURQ_Q6_K: return launch_quant_gather<TURQ_Q6_K>(layout, w, n, k, ids, count, out, out_dtype, ldo, stream);
    case TURQ_F32: return launch_dense_gather<TURQ_F32>(w, n, k, ids, count, out, out_dtype, ldo, stream);
    case TURQ_F16: return launch_dense_gather<TURQ_F16>(w, n, k, ids, count, out, out_dtype, ldo, stream);
    case TURQ_BF16: return launch_dense_gather<TURQ_BF16>(w, n, k, ids, count, out, out_dtype, ldo, stream);
    default: return hipErrorInvalidValue;
    }
}

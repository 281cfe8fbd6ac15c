// Activation preparation for the MFMA kernels: x (f32 / bf16 / f16, [m, k] with row stride ldx)
// is converted once to f16 and written in MFMA A-fragment order (see mfma_common.h), together with
// the per-16-element group sums the K-quant kernels need for the "- dmin * m" / "- 32 * sc" terms.
// Columns past k and rows past m are written as zeros.
#include "mfma_common.h"

namespace {

template <int XT> __device__ inline float ld_act(const void *x, int64_t i) {
    if (XT == TURQ_ACT_F32) return ((const float *)x)[i];
    if (XT == TURQ_ACT_BF16) return __uint_as_float((uint32_t)((const uint16_t *)x)[i] << 16);
    _Float16 h;
    const uint16_t u = ((const uint16_t *)x)[i];
    __builtin_memcpy(&h, &u, 2);
    return (float)h;
}

// One workgroup of 256 threads per (m-tile, column tile b): thread (r, pc) converts the 16 columns 16 pc .. 16 pc + 15 of
// row r (consecutive threads read consecutive columns), which are two 16-byte fragment pieces and, for the K-quants,
// exactly one of the 16-element groups whose sum the kernels need.
template <int XT, bool KQ>
__global__ void __launch_bounds__(256) act_prep_kernel(const void *__restrict__ x, int64_t m, int64_t k, int64_t ldx,
                                                       int64_t ntc, int mpad, half8v *__restrict__ frags) {
    constexpr int NQ = KQ ? TURQ_NQ_KQUANT : TURQ_NQ_Q8_0;
    const int r = (int)threadIdx.x >> 4, pc = (int)threadIdx.x & 15;
    if (r >= mpad) return;
    const int64_t tb = blockIdx.x;  // mt * ntc + b
    const int64_t b = tb % ntc, mt = tb / ntc;
    const int64_t row = mt * 16 + r, col0 = b * 256 + 16 * pc;
    float v[16];
    const char *src = (const char *)x + (row * ldx + col0) * (XT == TURQ_ACT_F32 ? 4 : 2);
    if (row < m && col0 + 16 <= k && ((uintptr_t)src & 15) == 0) {
        if (XT == TURQ_ACT_F32) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float4v t = ((const float4v *)src)[i];
                v[4 * i] = t.x, v[4 * i + 1] = t.y, v[4 * i + 2] = t.z, v[4 * i + 3] = t.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const uint4v u = ((const uint4v *)src)[i];
                const uint32_t wd[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if (XT == TURQ_ACT_BF16) {
                        v[8 * i + 2 * j] = __uint_as_float(wd[j] << 16);
                        v[8 * i + 2 * j + 1] = __uint_as_float(wd[j] & 0xFFFF0000u);
                    } else {
                        const half2v hh = as_half2(wd[j]);
                        v[8 * i + 2 * j] = (float)hh.x;
                        v[8 * i + 2 * j + 1] = (float)hh.y;
                    }
                }
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 16; j++) v[j] = (row < m && col0 + j < k) ? ld_act<XT>(x, row * ldx + col0 + j) : 0.0f;
    }
    half8v h0, h1;
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; j++) turq_note_result<TURQ_ACT_F16>(v[j]);
#pragma unroll
    for (int j = 0; j < 8; j++) {
        h0[j] = (_Float16)v[j];
        h1[j] = (_Float16)v[8 + j];
    }
#pragma unroll
    for (int j = 0; j < 8; j++) sum += (float)h0[j];
#pragma unroll
    for (int j = 0; j < 8; j++) sum += (float)h1[j];
    half8v *tile = frags + tb * (NQ * 4 * mpad);
    if (KQ) {
        // lane group g owns columns 64g..64g+63, step q its 8q..8q+7
        const int g = pc >> 2, q0 = 2 * (pc & 3);
        tile[(q0 * 4 + g) * mpad + r] = h0;
        tile[((q0 + 1) * 4 + g) * mpad + r] = h1;
        const _Float16 hi = (_Float16)sum;
        const _Float16 lo = (_Float16)(sum - (float)hi);
        ((half2v *)&tile[(8 * 4 + g) * mpad + r])[pc & 3] = half2v{hi, lo};
    } else {
        // step q is block q (32 columns), lane group g owns 8g..8g+7 of it
        const int q = pc >> 1, g0 = 2 * (pc & 1);
        tile[(q * 4 + g0) * mpad + r] = h0;
        tile[(q * 4 + g0 + 1) * mpad + r] = h1;
    }
}

template <int XT>
hipError_t launch(int dtype, const void *x, int64_t m, int64_t k, int64_t ldx, void *frags, hipStream_t s) {
    const int64_t mtiles = (m + 15) / 16;
    const int mpad = mtiles > 1 ? 16 : turq_mpad(m);
    const int64_t ntc = (k + 255) / 256;
    const unsigned grid = (unsigned)(mtiles * ntc);
    if (dtype == TURQ_Q8_0)
        act_prep_kernel<XT, false><<<grid, 256, 0, s>>>(x, m, k, ldx, ntc, mpad, (half8v *)frags);
    else
        act_prep_kernel<XT, true><<<grid, 256, 0, s>>>(x, m, k, ldx, ntc, mpad, (half8v *)frags);
    return hipGetLastError();
}

// ---- fragments for the prefill GEMM (v_mfma_f32_32x32x16_f16) ----
// 32-row m-tiles; per 256-column tile b there are 16 operand steps plus one group-sum step.  Lane
// (r, g32) = r + 32 * g32 of step q holds x[32 mt + r][256 b + 128 g32 + 8 q + j], j = 0..7; step 16
// holds for the four 32-column sub-blocks of the lane's 128 columns the sums of the f16-rounded
// activations as (hi, lo) f16 pairs.  chunk index = ((mt * ntc + b) * 17 + q) * 64 + lane.
// Q8_0 order (Q8 = true): step q holds x[32 mt + r][256 b + 32 (q / 2) + 16 g32 + 8 (q % 2) + j] — the lane takes lane
// slots 2 g32 and 2 g32 + 1 (8 elements each) of every 32-element block, block by block; step 16 is not used.
// One workgroup per (m-tile, 64 columns): thread (r, pc) reads the 8 columns 8 pc .. 8 pc + 7 of row r (8 threads one row
// piece of 64 columns), rounds them to f16 and stores its 16-byte fragment chunk straight from registers; the sub-block sums
// are added up between the four neighbouring lanes that hold a sub-block.  No LDS and no barrier: the kernel is a chain of
// load -> store latencies, and four times as many, smaller workgroups keep four times as many of them in flight per CU
// (6.3 -> 5.1 us at m = 512, K = 4096).
// GU: the rows are SiLU(x) * up of two f32 matrices (the MLP's intermediate, src/models/qwen3.rs:161-167), evaluated and
// rounded to f16 exactly as silu_mul_kernel stores it, so that down_proj's fragments come out of the two products directly.
template <int XT, bool Q8, bool GU = false>
__global__ void __launch_bounds__(256) act_prep32_kernel(const void *__restrict__ x, int64_t m, int64_t k, int64_t ldx,
                                                         int64_t ntc, half8v *__restrict__ frags, const float *__restrict__ up = nullptr) {
    const int tid = threadIdx.x;
    const int64_t wg = blockIdx.x;  // (mt * ntc + b) * 4 + quarter
    const int quarter = (int)(wg & 3);
    const int64_t tb = wg >> 2;
    const int64_t b = tb % ntc, mt = tb / ntc;
    const int r = tid >> 3, pc = tid & 7;
    const int cc = 8 * quarter + pc;  // piece of 8 columns inside the 256-column tile
    const int64_t row = mt * 32 + r, col0 = b * 256 + 8 * cc;
    float v[8];
    const char *src = (const char *)x + (row * ldx + col0) * (XT == TURQ_ACT_F32 ? 4 : 2);
    if (row < m && col0 + 8 <= k && ((uintptr_t)src & 15) == 0) {
        if (XT == TURQ_ACT_F32) {
            const float4v lo = ((const float4v *)src)[0], hi = ((const float4v *)src)[1];
            v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
        } else {
            const uint4v u = *(const uint4v *)src;
            const uint32_t wd[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (XT == TURQ_ACT_BF16) {
                    v[2 * j] = __uint_as_float(wd[j] << 16);
                    v[2 * j + 1] = __uint_as_float(wd[j] & 0xFFFF0000u);
                } else {
                    const half2v hh = as_half2(wd[j]);
                    v[2 * j] = (float)hh.x;
                    v[2 * j + 1] = (float)hh.y;
                }
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = (row < m && col0 + j < k) ? ld_act<XT>(x, row * ldx + col0 + j) : 0.0f;
    }
    if constexpr (GU) {
        static_assert(XT == TURQ_ACT_F32, "the two products are f32");
        float u[8];
        const float *us = up + row * ldx + col0;
        if (row < m && col0 + 8 <= k && ((uintptr_t)us & 15) == 0) {
            const float4v lo = ((const float4v *)us)[0], hi = ((const float4v *)us)[1];
            u[0] = lo.x, u[1] = lo.y, u[2] = lo.z, u[3] = lo.w, u[4] = hi.x, u[5] = hi.y, u[6] = hi.z, u[7] = hi.w;
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) u[j] = (row < m && col0 + j < k) ? us[j] : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = v[j] / (1.0f + expf(-v[j])) * u[j];
    }
    half8v h;
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        turq_note_result<TURQ_ACT_F16>(v[j]);
        h[j] = (_Float16)v[j];
        sum += (float)h[j];
    }
    half8v *dst = frags + tb * (17 * 64);
    const int g32 = Q8 ? (cc >> 1) & 1 : cc >> 4, q = Q8 ? 2 * (cc >> 2) + (cc & 1) : cc & 15;
    dst[q * 64 + r + 32 * g32] = h;
    if (!Q8) {
        // sub-block = 32 columns = pieces 4 s .. 4 s + 3: four neighbouring lanes; the same order of additions as a
        // pairwise tree over the pieces, (p0 + p1) + (p2 + p3)
        sum += __shfl_xor(sum, 1, 64);
        sum += __shfl_xor(sum, 2, 64);
        if ((pc & 3) == 0) {
            const int sb = (cc >> 2) & 3;  // sub-block inside the lane's 128 columns
            const _Float16 hi = (_Float16)sum;
            const _Float16 lo = (_Float16)(sum - (float)hi);
            ((half2v *)&dst[16 * 64 + r + 32 * g32])[sb] = half2v{hi, lo};
        }
    }
}

}  // namespace

hipError_t turq_launch_act_prep(int dtype, const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, void *frags,
                                hipStream_t stream) {
    if (m == 0 || k == 0) return hipSuccess;
    switch (x_dtype) {
    case TURQ_ACT_F32: return launch<TURQ_ACT_F32>(dtype, x, m, k, ldx, frags, stream);
    case TURQ_ACT_BF16: return launch<TURQ_ACT_BF16>(dtype, x, m, k, ldx, frags, stream);
    case TURQ_ACT_F16: return launch<TURQ_ACT_F16>(dtype, x, m, k, ldx, frags, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t turq_launch_act_prep32(int dtype, const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, void *frags,
                                  hipStream_t stream) {
    if (m == 0 || k == 0) return hipSuccess;
    const int64_t ntc = (k + 255) / 256;
    const unsigned grid = (unsigned)(((m + 31) / 32) * ntc * 4);
    const bool q8 = dtype == TURQ_Q8_0;
#define TURQ_PREP32(XT)                                                                                       \
    if (q8) act_prep32_kernel<XT, true><<<grid, 256, 0, stream>>>(x, m, k, ldx, ntc, (half8v *)frags);        \
    else act_prep32_kernel<XT, false><<<grid, 256, 0, stream>>>(x, m, k, ldx, ntc, (half8v *)frags);          \
    break
    switch (x_dtype) {
    case TURQ_ACT_F32: TURQ_PREP32(TURQ_ACT_F32);
    case TURQ_ACT_BF16: TURQ_PREP32(TURQ_ACT_BF16);
    case TURQ_ACT_F16: TURQ_PREP32(TURQ_ACT_F16);
    default: return hipErrorInvalidValue;
    }
#undef TURQ_PREP32
    return hipGetLastError();
}

// fragments of SiLU(gate) * up for the prefill GEMM of down_proj, from the two f32 products [m, n] (row stride n) that the
// gate / up GEMMs left in scratch memory: what silu_mul_kernel (f16 output) followed by turq_launch_act_prep32 would write
hipError_t turq_launch_silu_mul_prep32(int dtype, const float *gate, const float *up, int64_t m, int64_t n, void *frags,
                                       hipStream_t stream) {
    if (m == 0 || n == 0) return hipSuccess;
    const int64_t ntc = (n + 255) / 256;
    const unsigned grid = (unsigned)(((m + 31) / 32) * ntc * 4);
    if (dtype == TURQ_Q8_0) act_prep32_kernel<TURQ_ACT_F32, true, true><<<grid, 256, 0, stream>>>(gate, m, n, n, ntc, (half8v *)frags, up);
    else act_prep32_kernel<TURQ_ACT_F32, false, true><<<grid, 256, 0, stream>>>(gate, m, n, n, ntc, (half8v *)frags, up);
    return hipGetLastError();
}

TURQ_NONFINITE_READER(turq_nonfinite_act_prep)

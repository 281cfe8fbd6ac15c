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

// One thread per (m-tile, column tile b, lane group g, row r): 64 activations of one row.
template <int XT, bool KQ>
__global__ void __launch_bounds__(256) act_prep_kernel(const void *__restrict__ x, int64_t m, int64_t k, int64_t ldx,
                                                       int64_t ntc, int mpad, int64_t nthreads,
                                                       half8v *__restrict__ frags) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= nthreads) return;
    constexpr int NQ = KQ ? TURQ_NQ_KQUANT : TURQ_NQ_Q8_0;
    const int r = (int)(t % mpad);
    const int g = (int)((t / mpad) & 3);
    const int64_t tb = t / (4 * (int64_t)mpad);  // = mt * ntc + b
    const int64_t b = tb % ntc;
    const int64_t mt = tb / ntc;
    const int64_t row = mt * 16 + r;
    const bool row_ok = row < m;
    float gsum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q = 0; q < 8; q++) {
        // K-quants: lane group g owns columns 64g..64g+63, step q its 8q..8q+7
        // Q8_0:     step q is block q (32 columns), lane group g owns 8g..8g+7 of it
        const int64_t col0 = b * 256 + (KQ ? 64 * g + 8 * q : 32 * q + 8 * g);
        half8v h;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int64_t c = col0 + j;
            const float v = (row_ok && c < k) ? ld_act<XT>(x, row * ldx + c) : 0.0f;
            h[j] = (_Float16)v;
            if (KQ) gsum[q >> 1] += (float)h[j];
        }
        frags[((tb * NQ + q) * 4 + g) * mpad + r] = h;
    }
    if (KQ) {
        half8v s;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const _Float16 hi = (_Float16)gsum[i];
            const _Float16 lo = (_Float16)(gsum[i] - (float)hi);
            s[2 * i] = hi;
            s[2 * i + 1] = lo;
        }
        frags[((tb * NQ + 8) * 4 + g) * mpad + r] = s;
    }
}

template <int XT>
hipError_t launch(int dtype, const void *x, int64_t m, int64_t k, int64_t ldx, void *frags, hipStream_t s) {
    const int64_t mtiles = (m + 15) / 16;
    const int mpad = mtiles > 1 ? 16 : turq_mpad(m);
    const int64_t ntc = (k + 255) / 256;
    const int64_t nthreads = mtiles * ntc * 4 * mpad;
    const unsigned grid = (unsigned)((nthreads + 255) / 256);
    if (dtype == TURQ_Q8_0)
        act_prep_kernel<XT, false><<<grid, 256, 0, s>>>(x, m, k, ldx, ntc, mpad, nthreads, (half8v *)frags);
    else
        act_prep_kernel<XT, true><<<grid, 256, 0, s>>>(x, m, k, ldx, ntc, mpad, nthreads, (half8v *)frags);
    return hipGetLastError();
}

// ---- fragments for the prefill GEMM (v_mfma_f32_32x32x16_f16) ----
// 32-row m-tiles; per 256-column tile b there are 16 operand steps plus one group-sum step.  Lane
// (r, g32) = r + 32 * g32 of step q holds x[32 mt + r][256 b + 128 g32 + 8 q + j], j = 0..7; step 16
// holds for the four 32-column sub-blocks of the lane's 128 columns the sums of the f16-rounded
// activations as (hi, lo) f16 pairs.  chunk index = ((mt * ntc + b) * 17 + q) * 64 + lane.
template <int XT>
__global__ void __launch_bounds__(256) act_prep32_kernel(const void *__restrict__ x, int64_t m, int64_t k, int64_t ldx,
                                                         int64_t ntc, int64_t nchunks, half8v *__restrict__ frags) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= nchunks) return;
    const int lane = (int)(t & 63);
    const int64_t blk = t >> 6;            // (mt * ntc + b) * 17 + q
    const int q = (int)(blk % 17);
    const int64_t tb = blk / 17;
    const int64_t b = tb % ntc, mt = tb / ntc;
    const int r = lane & 31, g32 = lane >> 5;
    const int64_t row = mt * 32 + r;
    const bool row_ok = row < m;
    half8v h;
    if (q < 16) {
        const int64_t col0 = b * 256 + 128 * g32 + 8 * q;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int64_t c = col0 + j;
            h[j] = (_Float16)((row_ok && c < k) ? ld_act<XT>(x, row * ldx + c) : 0.0f);
        }
    } else {
#pragma unroll
        for (int sb = 0; sb < 4; sb++) {
            const int64_t col0 = b * 256 + 128 * g32 + 32 * sb;
            float sum = 0.0f;
            for (int j = 0; j < 32; j++) {
                const int64_t c = col0 + j;
                sum += (float)(_Float16)((row_ok && c < k) ? ld_act<XT>(x, row * ldx + c) : 0.0f);
            }
            const _Float16 hi = (_Float16)sum;
            h[2 * sb] = hi;
            h[2 * sb + 1] = (_Float16)(sum - (float)hi);
        }
    }
    frags[t] = h;
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

hipError_t turq_launch_act_prep32(const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, void *frags, hipStream_t stream) {
    if (m == 0 || k == 0) return hipSuccess;
    const int64_t ntc = (k + 255) / 256;
    const int64_t nchunks = ((m + 31) / 32) * ntc * 17 * 64;
    const unsigned grid = (unsigned)((nchunks + 255) / 256);
    switch (x_dtype) {
    case TURQ_ACT_F32: act_prep32_kernel<TURQ_ACT_F32><<<grid, 256, 0, stream>>>(x, m, k, ldx, ntc, nchunks, (half8v *)frags); break;
    case TURQ_ACT_BF16: act_prep32_kernel<TURQ_ACT_BF16><<<grid, 256, 0, stream>>>(x, m, k, ldx, ntc, nchunks, (half8v *)frags); break;
    case TURQ_ACT_F16: act_prep32_kernel<TURQ_ACT_F16><<<grid, 256, 0, stream>>>(x, m, k, ldx, ntc, nchunks, (half8v *)frags); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

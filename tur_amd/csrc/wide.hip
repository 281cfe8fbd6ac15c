// Activations of any finite f32 magnitude for the f16 matrix kernels.
//
// The MFMA kernels round the activations to f16, whose range ends at 65504 and whose precision fades below 6e-5, while the
// reference's contract is f32 activations (src/weights/mod.rs:84-99; candle's CPU path scales every 256-element block on its
// own, BlockQ8K::from_float).  The "wide" path brackets a matmul with two small kernels: before it, every row is multiplied by
// the power of two that puts its largest magnitude between 2^9 and 2^10 and written as f16 (exact apart from the rounding
// the kernels would do anyway; the headroom is for the sums over 16 and 32 neighbouring activations that the K-quant kernels
// keep as f16 pairs); after it, every output row is multiplied by the inverse power of two (exact) and the bias is
// added.  Rows of zeros and rows that hold an infinity or a NaN are left as they are, so non-finite inputs propagate.
#include "mfma_common.h"

namespace {

template <int XT> __device__ inline float ld_x(const void *x, int64_t i) {
    if (XT == TURQ_ACT_F32) return ((const float *)x)[i];
    return __uint_as_float((uint32_t)((const uint16_t *)x)[i] << 16);  // bf16
}

// one workgroup of 256 threads per row: the row's largest magnitude, then the scaled f16 copy
template <int XT>
__global__ void __launch_bounds__(256) wide_scale_kernel(const void *__restrict__ x, int64_t k, int64_t ldx, _Float16 *__restrict__ x16,
                                                         float *__restrict__ inv) {
    __shared__ float part[4];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    float amax = 0.0f;
    bool finite = true;
    for (int64_t c = tid; c < k; c += 256) {
        const float v = fabsf(ld_x<XT>(x, row * ldx + c));
        finite = finite && v <= 3.4028234e38f;  // false for an infinity and for a NaN
        amax = fmaxf(amax, v);
    }
    if (!finite) amax = __uint_as_float(0x7F800000u);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if ((tid & 63) == 0) part[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    // exponent of the scale: the largest magnitude lands in [2^9, 2^10); nothing to do for 0 and for non-finite rows
    int e = 0;
    if (amax > 0.0f && amax <= 3.4028234e38f) {
        int ex;
        (void)frexpf(amax, &ex);  // amax = f * 2^ex, f in [0.5, 1)
        e = 10 - ex;
        if (e > 126) e = 126;  // subnormal rows: as far as an f32 power of two reaches
    }
    const float s = ldexpf(1.0f, e);
    if (tid == 0) inv[row] = ldexpf(1.0f, -e);
    for (int64_t c = tid; c < k; c += 256) x16[row * k + c] = (_Float16)(ld_x<XT>(x, row * ldx + c) * s);
}

// y[r][c] = y32[r][c] * inv[r] + bias[c]
template <int YT>
__global__ void __launch_bounds__(256) wide_rescale_kernel(const float *__restrict__ y32, int64_t ld32, int64_t n, const float *__restrict__ inv,
                                                           const float *__restrict__ bias, void *__restrict__ y, int64_t ldy, int64_t m,
                                                           int accum) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= n) return;
    const float b = bias ? bias[c] : 0.0f;
    for (int64_t row = blockIdx.y; row < m; row += gridDim.y) {  // (a grid has at most 65535 rows of workgroups)
        const float v = y32[row * ld32 + c] * inv[row] + b + (accum ? turq_load_out<YT>(y, row * ldy + c) : 0.0f);
        turq_store_out<YT>(y, row * ldy + c, v);
    }
}

}  // namespace

hipError_t turq_launch_wide_scale(const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, void *x16, float *inv, hipStream_t stream) {
    if (m == 0 || k == 0) return hipSuccess;
    if (m > 0x7FFFFFFF) return hipErrorInvalidValue;
    if (x_dtype == TURQ_ACT_F32) wide_scale_kernel<TURQ_ACT_F32><<<(unsigned)m, 256, 0, stream>>>(x, k, ldx, (_Float16 *)x16, inv);
    else if (x_dtype == TURQ_ACT_BF16) wide_scale_kernel<TURQ_ACT_BF16><<<(unsigned)m, 256, 0, stream>>>(x, k, ldx, (_Float16 *)x16, inv);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t turq_launch_wide_rescale(const float *y32, int64_t ld32, int64_t m, int64_t n, const float *inv, const float *bias, void *y,
                                    int y_dtype, int64_t ldy, hipStream_t stream) {
    if (m == 0 || n == 0) return hipSuccess;
    const dim3 grid((unsigned)((n + 255) / 256), (unsigned)(m < 65535 ? m : 65535));
    const int accum = (y_dtype & TURQ_OUT_ACCUMULATE) != 0;
    switch (y_dtype & 0xFF) {
    case TURQ_ACT_F32: wide_rescale_kernel<TURQ_ACT_F32><<<grid, 256, 0, stream>>>(y32, ld32, n, inv, bias, y, ldy, m, accum); break;
    case TURQ_ACT_BF16: wide_rescale_kernel<TURQ_ACT_BF16><<<grid, 256, 0, stream>>>(y32, ld32, n, inv, bias, y, ldy, m, accum); break;
    case TURQ_ACT_F16: wide_rescale_kernel<TURQ_ACT_F16><<<grid, 256, 0, stream>>>(y32, ld32, n, inv, bias, y, ldy, m, accum); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

TURQ_NONFINITE_READER(turq_nonfinite_wide)

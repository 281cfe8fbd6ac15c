// RmsNorm, the layer in front of the q / k / v and gate / up projections (reference: src/models/layers/norm.rs:81-93 builds
// candle_nn::RmsNorm from the dequantized F32 `weight` of the GGUF file; src/models/qwen3.rs applies it before the attention and
// MLP blocks).  y[r][c] = x[r][c] / sqrt(mean_c(x[r][c]^2) + eps) * weight[c], computed in f32 in candle's order: the sum of
// squares of the row, one square root, then per element a division and a multiplication.
#include "mfma_common.h"

namespace {

template <int XT> __device__ inline float ld_elem(const void *x, int64_t i) {
    if (XT == TURQ_ACT_F32) return ((const float *)x)[i];
    if (XT == TURQ_ACT_BF16) return __uint_as_float((uint32_t)((const uint16_t *)x)[i] << 16);
    _Float16 h;
    const uint16_t u = ((const uint16_t *)x)[i];
    __builtin_memcpy(&h, &u, 2);
    return (float)h;
}

// one workgroup of 256 threads per row; a thread keeps up to PER of the row's elements in registers between the two passes
// (rows of up to 256 * PER elements are read once), longer rows are read again
template <int XT, int YT, int PER>
__global__ void __launch_bounds__(256) rms_norm_kernel(const void *__restrict__ x, int64_t k, int64_t ldx, const float *__restrict__ w,
                                                       float eps, void *__restrict__ y, int64_t ldy) {
    __shared__ float part[4];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int64_t xo = row * ldx, yo = row * ldy;
    float v[PER];
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int64_t c = (int64_t)j * 256 + tid;
        v[j] = c < k ? ld_elem<XT>(x, xo + c) : 0.0f;
        s += v[j] * v[j];
    }
    for (int64_t c = (int64_t)PER * 256 + tid; c < k; c += 256) {
        const float t = ld_elem<XT>(x, xo + c);
        s += t * t;
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
    if ((tid & 63) == 0) part[tid >> 6] = s;
    __syncthreads();
    const float total = (part[0] + part[1]) + (part[2] + part[3]);
    const float rms = sqrtf(total / (float)k + eps);
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int64_t c = (int64_t)j * 256 + tid;
        if (c < k) turq_store_out<YT>(y, yo + c, v[j] / rms * w[c]);
    }
    for (int64_t c = (int64_t)PER * 256 + tid; c < k; c += 256) turq_store_out<YT>(y, yo + c, ld_elem<XT>(x, xo + c) / rms * w[c]);
}

template <int XT, int YT>
hipError_t launch2(const void *x, int64_t m, int64_t k, int64_t ldx, const float *w, float eps, void *y, int64_t ldy, hipStream_t s) {
    if (k <= 4 * 256) rms_norm_kernel<XT, YT, 4><<<(unsigned)m, 256, 0, s>>>(x, k, ldx, w, eps, y, ldy);
    else rms_norm_kernel<XT, YT, 16><<<(unsigned)m, 256, 0, s>>>(x, k, ldx, w, eps, y, ldy);
    return hipGetLastError();
}

template <int XT>
hipError_t launch1(int yt, const void *x, int64_t m, int64_t k, int64_t ldx, const float *w, float eps, void *y, int64_t ldy, hipStream_t s) {
    switch (yt) {
    case TURQ_ACT_F32: return launch2<XT, TURQ_ACT_F32>(x, m, k, ldx, w, eps, y, ldy, s);
    case TURQ_ACT_BF16: return launch2<XT, TURQ_ACT_BF16>(x, m, k, ldx, w, eps, y, ldy, s);
    case TURQ_ACT_F16: return launch2<XT, TURQ_ACT_F16>(x, m, k, ldx, w, eps, y, ldy, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

hipError_t turq_launch_rms_norm(const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, const float *weight, float eps, void *y,
                                int y_dtype, int64_t ldy, hipStream_t stream) {
    if (m == 0 || k == 0) return hipSuccess;
    if (m > 0x7FFFFFFF) return hipErrorInvalidValue;
    switch (x_dtype) {
    case TURQ_ACT_F32: return launch1<TURQ_ACT_F32>(y_dtype, x, m, k, ldx, weight, eps, y, ldy, stream);
    case TURQ_ACT_BF16: return launch1<TURQ_ACT_BF16>(y_dtype, x, m, k, ldx, weight, eps, y, ldy, stream);
    case TURQ_ACT_F16: return launch1<TURQ_ACT_F16>(y_dtype, x, m, k, ldx, weight, eps, y, ldy, stream);
    default: return hipErrorInvalidValue;
    }
}

TURQ_NONFINITE_READER(turq_nonfinite_norm)

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

// the workgroup's part of sqrt(mean(x^2) + eps): s = what thread t added up of the squares of columns t, t + 256, ... (explicit
// fused multiply-adds in that order), then the waves their lanes and the workgroup its four waves - one fixed order, shared by
// the kernels below so that they agree to the bit
__device__ inline float rms_of(float s, int64_t k, float eps, float *part) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
    if ((tid & 63) == 0) part[tid >> 6] = s;
    __syncthreads();
    const float total = (part[0] + part[1]) + (part[2] + part[3]);
    return sqrtf(total / (float)k + eps);
}

// one workgroup of 256 threads per row; a thread keeps up to PER of the row's elements in registers between the two passes
// (rows of up to 256 * PER elements are read once, so y may be x whatever the two element types), longer rows are read again
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
        s = __builtin_fmaf(v[j], v[j], s);  // (columns past k add +0: the sum is that of the columns that exist)
    }
    for (int64_t c = (int64_t)PER * 256 + tid; c < k; c += 256) {
        const float t = ld_elem<XT>(x, xo + c);
        s = __builtin_fmaf(t, t, s);
    }
    const float rms = rms_of(s, k, eps, part);
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int64_t c = (int64_t)j * 256 + tid;
        if (c < k) turq_store_out<YT>(y, yo + c, v[j] / rms * w[c]);
    }
    for (int64_t c = (int64_t)PER * 256 + tid; c < k; c += 256) turq_store_out<YT>(y, yo + c, ld_elem<XT>(x, xo + c) / rms * w[c]);
}

// The same rows written straight into the fragments of the prefill GEMM (the order act_prep32_kernel writes, see there): what
// rms_norm_kernel with an f32 output followed by that kernel would leave - the same sums in the same order, the same one rounding
// to f16 - without the launch and the round trip in between.  One workgroup per row of the 32-row m-tiles (rows past m: zeros);
// thread t holds the pieces of 8 columns t, t + 256, ... (PER of them: k <= 2048 * PER); the sub-block sums of the fragments
// (32 columns) are added up between the four neighbouring lanes that hold a sub-block.
template <int XT, bool Q8, int PER>
__global__ void __launch_bounds__(256) rms_norm_prep32_kernel(const void *__restrict__ x, int64_t m, int64_t k, int64_t ldx,
                                                              const float *__restrict__ w, float eps, int64_t ntc, half8v *__restrict__ frags) {
    __shared__ float part[4];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int64_t mt = row >> 5;
    const int r = (int)(row & 31);
    const bool live = row < m;
    const int64_t xo = row * ldx;
    float s = 0.0f;  // the row's sum of squares, added up as rms_norm_kernel adds it up
    if (live)
        for (int64_t c = tid; c < k; c += 256) {
            const float t = ld_elem<XT>(x, xo + c);
            s = __builtin_fmaf(t, t, s);
        }
    const float rms = rms_of(s, k, eps, part);
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int64_t piece = (int64_t)j * 256 + tid, col0 = piece * 8;
        if (col0 >= k) continue;  // (k is a multiple of 256: whole pieces, and whole groups of four lanes)
        half8v h;
        float sum = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float f = live ? ld_elem<XT>(x, xo + col0 + e) / rms * w[col0 + e] : 0.0f;
            turq_note_result<TURQ_ACT_F16>(f);
            h[e] = (_Float16)f;
            sum += (float)h[e];
        }
        const int64_t b = piece >> 5;
        const int cc = (int)(piece & 31);
        half8v *dst = frags + (mt * ntc + b) * (17 * 64);
        const int g32 = Q8 ? (cc >> 1) & 1 : cc >> 4, q = Q8 ? 2 * (cc >> 2) + (cc & 1) : cc & 15;
        dst[q * 64 + r + 32 * g32] = h;
        if (!Q8) {
            sum += __shfl_xor(sum, 1, 64);
            sum += __shfl_xor(sum, 2, 64);
            if ((tid & 3) == 0) {
                const int sb = (cc >> 2) & 3;
                const _Float16 hi = (_Float16)sum;
                const _Float16 lo = (_Float16)(sum - (float)hi);
                ((half2v *)&dst[16 * 64 + r + 32 * g32])[sb] = half2v{hi, lo};
            }
        }
    }
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

// frags: turq_act_prep32_bytes(m, k) bytes; k a multiple of 256 and at most 16384; dtype picks the fragment order (Q8_0 / K-quants)
hipError_t turq_launch_rms_norm_prep32(int dtype, const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, const float *weight,
                                       float eps, void *frags, hipStream_t stream) {
    if (m == 0 || k == 0) return hipSuccess;
    if (k % 256 != 0 || k > 16384 || m > (1 << 26)) return hipErrorInvalidValue;
    const int64_t ntc = k / 256;
    const unsigned grid = (unsigned)(((m + 31) / 32) * 32);
    const bool q8 = dtype == TURQ_Q8_0;
#define TURQ_NP32(XT, PER)                                                                                                           \
    if (q8) rms_norm_prep32_kernel<XT, true, PER><<<grid, 256, 0, stream>>>(x, m, k, ldx, weight, eps, ntc, (half8v *)frags);       \
    else rms_norm_prep32_kernel<XT, false, PER><<<grid, 256, 0, stream>>>(x, m, k, ldx, weight, eps, ntc, (half8v *)frags)
#define TURQ_NP32_X(XT)                                  \
    if (k <= 2048 * 2) { TURQ_NP32(XT, 2); }             \
    else if (k <= 2048 * 6) { TURQ_NP32(XT, 6); }        \
    else { TURQ_NP32(XT, 8); }                           \
    break
    switch (x_dtype) {
    case TURQ_ACT_F32: TURQ_NP32_X(TURQ_ACT_F32);
    case TURQ_ACT_BF16: TURQ_NP32_X(TURQ_ACT_BF16);
    case TURQ_ACT_F16: TURQ_NP32_X(TURQ_ACT_F16);
    default: return hipErrorInvalidValue;
    }
#undef TURQ_NP32_X
#undef TURQ_NP32
    return hipGetLastError();
}

TURQ_NONFINITE_READER(turq_nonfinite_norm)

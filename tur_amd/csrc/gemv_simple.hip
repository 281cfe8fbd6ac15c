// Plain quantized matmul on the native GGUF layout: one wave per output row, weights dequantized
// to f32 in registers (same decode as the dequantize kernel), f32 FMA against the activations, and
// a wave-wide shuffle reduction.  It is the straightforward statement of y = x * dequant(W)^T for
// any shape and any m; the MFMA kernels on the tiled layout are the fast path.
// It is also the dense arm of the layer: F32 / F16 / BF16 weights (candle's `QMatMul::from_arc` turns those GGUF tensors,
// and every tensor under CANDLE_DEQUANTIZE_ALL, into a dense f32 matmul; src/models/layers/linear.rs:69), any k.
#include "block_decode.h"
#include "mfma_common.h"

namespace {

template <int XT> __device__ inline float load_act(const void *x, int64_t i) {
    if (XT == TURQ_ACT_F32) return ((const float *)x)[i];
    if (XT == TURQ_ACT_BF16) return turq_bf2f(((const uint16_t *)x)[i]);
    return turq_h2f(((const uint16_t *)x)[i]);
}


template <int YT> __device__ inline void store_out(void *y, int64_t i, float v) {
    turq_note_result<YT>(v);
    if (YT == TURQ_ACT_F32) ((float *)y)[i] = v;
    else if (YT == TURQ_ACT_BF16) ((uint16_t *)y)[i] = turq_f2bf(v);
    else {
        const _Float16 h = (_Float16)v;
        uint16_t b;
        __builtin_memcpy(&b, &h, 2);
        ((uint16_t *)y)[i] = b;
    }
}

constexpr int MT = 8;  // activation rows handled per pass over a weight row

template <int DT, int XT, int YT>
__global__ void __launch_bounds__(256) gemv_simple_kernel(const uint8_t *__restrict__ w, int64_t n, int64_t k,
                                                          int64_t row_bytes, const void *__restrict__ x, int64_t m,
                                                          int64_t ldx, void *__restrict__ y, int64_t ldy,
                                                          const float *__restrict__ bias, int accum) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n) return;  // uniform per wave
    const uint8_t *wr = w + row * row_bytes;
    const float b = bias ? bias[row] : 0.0f;
    for (int64_t m0 = 0; m0 < m; m0 += MT) {
        float acc[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) acc[i] = 0.0f;
        constexpr bool DENSE = DT == TURQ_F32 || DT == TURQ_F16 || DT == TURQ_BF16;
        for (int64_t e0 = (int64_t)lane * 8; e0 < k; e0 += 64 * 8) {
            float wv[8];
            if (DENSE && e0 + 8 > k) {  // a dense row may end inside the lane's eight columns
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    if (e0 + j >= k) wv[j] = 0.0f;
                    else if (DT == TURQ_F32) wv[j] = ((const float *)wr)[e0 + j];
                    else if (DT == TURQ_F16) wv[j] = turq_h2f(((const uint16_t *)wr)[e0 + j]);
                    else wv[j] = turq_bf2f(((const uint16_t *)wr)[e0 + j]);
                }
#pragma unroll
                for (int i = 0; i < MT; i++) {
                    if (m0 + i < m) {
                        const int64_t base = (m0 + i) * ldx + e0;
#pragma unroll
                        for (int j = 0; j < 8; j++)
                            if (e0 + j < k) acc[i] = fmaf(wv[j], load_act<XT>(x, base + j), acc[i]);
                    }
                }
                continue;
            }
            Decode8<DT>::run(wr, e0, wv);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                if (m0 + i < m) {
                    const int64_t base = (m0 + i) * ldx + e0;
#pragma unroll
                    for (int j = 0; j < 8; j++) acc[i] = fmaf(wv[j], load_act<XT>(x, base + j), acc[i]);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < MT; i++) {
            float v = acc[i];
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
            if (lane == 0 && m0 + i < m) store_out<YT>(y, (m0 + i) * ldy + row, v + b + (accum ? turq_load_out<YT>(y, (m0 + i) * ldy + row) : 0.0f));
        }
    }
}

template <int DT, int XT, int YT>
hipError_t launch3(const void *w, int64_t n, int64_t k, const void *x, int64_t m, int64_t ldx, void *y, int64_t ldy,
                   const float *bias, hipStream_t s, int accum) {
    const int64_t row_bytes = k / turq_dt_block_elems(DT) * turq_dt_block_bytes(DT);
    const unsigned grid = (unsigned)((n + 3) / 4);
    gemv_simple_kernel<DT, XT, YT><<<grid, 256, 0, s>>>((const uint8_t *)w, n, k, row_bytes, x, m, ldx, y, ldy, bias, accum);
    return hipGetLastError();
}

template <int DT, int XT>
hipError_t launch2(int yt, const void *w, int64_t n, int64_t k, const void *x, int64_t m, int64_t ldx, void *y,
                   int64_t ldy, const float *bias, hipStream_t s) {
    const int accum = (yt & TURQ_OUT_ACCUMULATE) != 0;
    switch (yt & 0xFF) {
    case TURQ_ACT_F32: return launch3<DT, XT, TURQ_ACT_F32>(w, n, k, x, m, ldx, y, ldy, bias, s, accum);
    case TURQ_ACT_BF16: return launch3<DT, XT, TURQ_ACT_BF16>(w, n, k, x, m, ldx, y, ldy, bias, s, accum);
    case TURQ_ACT_F16: return launch3<DT, XT, TURQ_ACT_F16>(w, n, k, x, m, ldx, y, ldy, bias, s, accum);
    default: return hipErrorInvalidValue;
    }
}

template <int DT>
hipError_t launch1(int xt, int yt, const void *w, int64_t n, int64_t k, const void *x, int64_t m, int64_t ldx,
                   void *y, int64_t ldy, const float *bias, hipStream_t s) {
    switch (xt) {
    case TURQ_ACT_F32: return launch2<DT, TURQ_ACT_F32>(yt, w, n, k, x, m, ldx, y, ldy, bias, s);
    case TURQ_ACT_BF16: return launch2<DT, TURQ_ACT_BF16>(yt, w, n, k, x, m, ldx, y, ldy, bias, s);
    case TURQ_ACT_F16: return launch2<DT, TURQ_ACT_F16>(yt, w, n, k, x, m, ldx, y, ldy, bias, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

hipError_t turq_launch_gemv_simple(int dtype, const void *w, int64_t n, int64_t k, const void *x, int x_dtype,
                                   int64_t m, int64_t ldx, void *y, int y_dtype, int64_t ldy, const float *bias,
                                   hipStream_t stream) {
    if (n == 0 || m == 0) return hipSuccess;
    switch (dtype) {
    case TURQ_Q8_0: return launch1<TURQ_Q8_0>(x_dtype, y_dtype, w, n, k, x, m, ldx, y, ldy, bias, stream);
    case TURQ_Q4_K: return launch1<TURQ_Q4_K>(x_dtype, y_dtype, w, n, k, x, m, ldx, y, ldy, bias, stream);
    case TURQ_Q5_K: return launch1<TURQ_Q5_K>(x_dtype, y_dtype, w, n, k, x, m, ldx, y, ldy, bias, stream);
    case TURQ_Q6_K: return launch1<TURQ_Q6_K>(x_dtype, y_dtype, w, n, k, x, m, ldx, y, ldy, bias, stream);
    case TURQ_F32: return launch1<TURQ_F32>(x_dtype, y_dtype, w, n, k, x, m, ldx, y, ldy, bias, stream);
    case TURQ_F16: return launch1<TURQ_F16>(x_dtype, y_dtype, w, n, k, x, m, ldx, y, ldy, bias, stream);
    case TURQ_BF16: return launch1<TURQ_BF16>(x_dtype, y_dtype, w, n, k, x, m, ldx, y, ldy, bias, stream);
    default: return hipErrorInvalidValue;
    }
}

TURQ_NONFINITE_READER(turq_nonfinite_gemv_simple)

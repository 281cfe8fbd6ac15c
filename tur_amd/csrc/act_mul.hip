// act(gate) * up on two f32 matrices [m, n] (row stride n) that a pair of matmuls left in scratch memory: the general path of
// turq_qmatmul_gate_up (the decode path applies the same expression inside the matmul kernel, gemv_row1.hip).
// Reference: src/models/qwen3.rs:161-167 (`x.apply(&gate_proj)?.apply(&act_fn)? * x.apply(&up_proj)?`).
#include "mfma_common.h"

namespace {

__global__ void __launch_bounds__(256) silu_mul_kernel(const float *__restrict__ gate, const float *__restrict__ up, int64_t m, int64_t n,
                                                       void *__restrict__ y, int yt, int64_t ldy) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= m * n) return;
    const int64_t row = i / n, col = i - row * n;
    const float g = gate[i];
    const float out = g / (1.0f + expf(-g)) * up[i];
    const int64_t at = row * ldy + col;
    if (yt == TURQ_ACT_F32) turq_store_out<TURQ_ACT_F32>(y, at, out);
    else if (yt == TURQ_ACT_BF16) turq_store_out<TURQ_ACT_BF16>(y, at, out);
    else turq_store_out<TURQ_ACT_F16>(y, at, out);
}

}  // namespace

hipError_t turq_launch_silu_mul(const float *gate, const float *up, int64_t m, int64_t n, void *y, int y_dtype, int64_t ldy,
                                hipStream_t stream) {
    if (m <= 0 || n <= 0) return hipSuccess;
    if (!turq_yt_ok(y_dtype, true)) return hipErrorInvalidValue;
    const int64_t blocks = (m * n + 255) / 256;
    if (blocks > 0x7FFFFFFF) return hipErrorInvalidValue;
    silu_mul_kernel<<<(unsigned)blocks, 256, 0, stream>>>(gate, up, m, n, y, y_dtype, ldy);
    return hipGetLastError();
}

TURQ_NONFINITE_READER(turq_nonfinite_act_mul)

// Internal definitions shared by the translation units of libturq (not part of the C ABI).
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "../../include/turq.h"
#include "tuning.h"

#define TURQ_QK_K 256
#define TURQ_QK8_0 32

// ---- dtype geometry (ggml block layouts) ----
__host__ __device__ inline int turq_dt_block_elems(int dt) {
    switch (dt) {
    case TURQ_F32: case TURQ_F16: case TURQ_BF16: return 1;
    case TURQ_Q8_0: return 32;
    case TURQ_Q4_K: case TURQ_Q5_K: case TURQ_Q6_K: return 256;
    default: return 0;
    }
}
__host__ __device__ inline int turq_dt_block_bytes(int dt) {
    switch (dt) {
    case TURQ_F32: return 4;
    case TURQ_F16: case TURQ_BF16: return 2;
    case TURQ_Q8_0: return 34;
    case TURQ_Q4_K: return 144;
    case TURQ_Q5_K: return 176;
    case TURQ_Q6_K: return 210;
    default: return 0;
    }
}
inline const char *turq_dt_name(int dt) {
    switch (dt) {
    case TURQ_F32: return "F32";
    case TURQ_F16: return "F16";
    case TURQ_BF16: return "BF16";
    case TURQ_Q8_0: return "Q8_0";
    case TURQ_Q4_K: return "Q4_K";
    case TURQ_Q5_K: return "Q5_K";
    case TURQ_Q6_K: return "Q6_K";
    default: return "?";
    }
}
inline bool turq_dt_is_quant(int dt) {
    return dt == TURQ_Q8_0 || dt == TURQ_Q4_K || dt == TURQ_Q5_K || dt == TURQ_Q6_K;
}
// an output type may carry TURQ_OUT_ACCUMULATE; its element type is the low byte
inline int turq_yt_base(int yt) { return yt & 0xFF; }
inline bool turq_yt_ok(int yt, bool accumulate_allowed) {
    const int b = yt & 0xFF, flags = yt & ~0xFF;
    return (b == TURQ_ACT_F32 || b == TURQ_ACT_BF16 || b == TURQ_ACT_F16) && (flags == 0 || (accumulate_allowed && flags == TURQ_OUT_ACCUMULATE));
}
inline int turq_act_bytes(int act) {
    switch (act & 0xFF) {
    case TURQ_ACT_F32: return 4;
    case TURQ_ACT_BF16: case TURQ_ACT_F16: return 2;
    default: return 0;
    }
}

// ---- objects behind the opaque handles ----
// Live graphs of a context, shared between the context and its graphs (either may be destroyed first).  While the count is
// above zero a scratch buffer that has to grow is retired instead of freed: a captured graph keeps the addresses it was
// recorded with.
struct turq_graph_tally {
    std::atomic<int> live{0};
};

struct turq_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    int compute_units = 0;
    char device_name[128] = {0};
    std::string err;
    // growable device scratch: host staging for TURQ_MEM_HOST calls and prepared activations
    void *stage_x = nullptr;  size_t stage_x_cap = 0;
    void *stage_y = nullptr;  size_t stage_y_cap = 0;
    void *stage_b = nullptr;  size_t stage_b_cap = 0;
    void *act_prep = nullptr; size_t act_prep_cap = 0;
    void *gate_up = nullptr;  size_t gate_up_cap = 0;  // the two f32 products of turq_qmatmul_gate_up's general path
    // the wide-activation path (wide.hip): scaled f16 copy of the activations, per-row inverse scales, f32 results before rescaling
    void *wide_x = nullptr;   size_t wide_x_cap = 0;
    void *wide_s = nullptr;   size_t wide_s_cap = 0;
    void *wide_y = nullptr;   size_t wide_y_cap = 0;
    bool wide = false;  // device-pointer calls take that path too (host-pointer calls always do)
    void *mlp_h = nullptr;    size_t mlp_h_cap = 0;  // turq_mlp: the f32 intermediate act(gate) * up
    void *norm_x = nullptr;   size_t norm_x_cap = 0;  // turq_norm_*: the normalised rows where the kernels do not apply the norm themselves
    // prefill GEMM launches that split their columns over several workgroups: kSplitSlots counter blocks (zero between
    // launches; launch i of a call uses block i), then the partial tiles of the call's launches one after the other
    static constexpr int kSplitSlots = 16;
    void *gemm_split = nullptr; size_t gemm_split_cap = 0;
    // scratch buffers that were outgrown while a captured graph still referred to them: freed once no graph of the context is
    // alive (at the next growth) or with the context
    std::vector<void *> retired;
    std::shared_ptr<turq_graph_tally> tally;
    // turq_qmatmul_noalloc: for the duration of such a call act_prep points at the device's static scratch array and nothing
    // may be allocated (turq_ctx_reserve fails instead of growing, no timing events are created)
    bool fixed_scratch = false;
    void *static_scratch = nullptr;       // this device's copy of the static array (hipGetSymbolAddress at context creation)
    size_t static_scratch_cap = 0;
    int static_scratch_err = 0;           // hipError_t of that lookup
    // further streams for small prefill GEMMs of one turq_qmatmul_multi call that run next to each other: forked from `stream`
    // where the first launch of a group starts and joined again before the call returns (created on first use)
    static constexpr int kSide = 2;
    hipStream_t side[kSide] = {nullptr, nullptr};
    hipEvent_t ev_fork = nullptr, ev_join[kSide] = {nullptr, nullptr};
    // turq_weight_prefetch: a stream of its own for the read-only passes, forked from `stream` where the call is made (ev_pf_fork)
    // and, inside a graph capture, joined to it again before the capture ends (ev_pf_join)
    hipStream_t pf_stream = nullptr;
    hipEvent_t ev_pf_fork = nullptr, ev_pf_join = nullptr;
    bool pf_in_capture = false;  // the running capture holds prefetch work that is not joined yet
    int pf_workgroups = 0, pf_depth = 4;
    // kernel timing (turq_profile_*): event pairs recorded around matmul kernels
    bool profiling = false;
    bool capturing = false;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> prof_events;
    size_t prof_used = 0;
};

struct turq_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    int device = 0;
    std::shared_ptr<turq_graph_tally> tally;  // of the context it was captured on
};

// Kernel timing: hands out the next event pair (both null unless turq_profile_begin is active).
// The launcher passes them to hipExtLaunchKernelGGL, which stamps them with the dispatch's own
// begin / end times, i.e. the kernel's execution time without launch gaps.
hipError_t turq_prof_next(turq_ctx *ctx, hipEvent_t *start, hipEvent_t *stop);

struct turq_weight {
    std::atomic<int> refs{1};
    int device = 0;
    int dtype = 0;
    int layout = TURQ_LAYOUT_NATIVE;
    int64_t n = 0, k = 0;
    void *dev = nullptr;      // weight bytes in HBM (native or tiled)
    size_t dev_bytes = 0;     // allocation size
    size_t native_bytes = 0;  // n * k / blk * block_bytes
    // largest |d| * (largest block scale) over the tensor: the prefill GEMM folds d into f16 constants
    // scaled by 1024 and is only used while that cannot overflow f16
    float max_scale = 0.0f;
};

// ---- error plumbing ----
std::string &turq_thread_error();  // last error of calls without a context

inline int turq_fail(turq_ctx *ctx, int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (ctx) ctx->err = buf; else turq_thread_error() = buf;
    return code;
}

#define TURQ_HIP(ctx, call)                                                                      \
    do {                                                                                         \
        hipError_t e_ = (call);                                                                  \
        if (e_ != hipSuccess)                                                                    \
            return turq_fail((ctx), e_ == hipErrorOutOfMemory ? TURQ_ERR_OOM : TURQ_ERR_HIP,     \
                             "%s failed: %s", #call, hipGetErrorString(e_));                     \
    } while (0)

// A forward call that fails while the context's stream is capturing ends the capture and discards what was recorded (api.cpp)
int turq_capture_guard(turq_ctx *ctx, int rc);
// grow-only scratch on the context's device
int turq_ctx_reserve(turq_ctx *ctx, void **buf, size_t *cap, size_t need);
// The static scratch array of the current device (noalloc.hip): its device address and size.  The device must be current.
hipError_t turq_static_scratch(void **ptr, size_t *cap);

// ---- kernel launchers implemented in the .hip translation units ----
// All are asynchronous on `stream` and return hipGetLastError() of the launch.
hipError_t turq_launch_gather_rows(int dtype, int layout, const void *w, int64_t n, int64_t k, const uint32_t *ids, int64_t count,
                                   void *out, int out_dtype, int64_t ldo, hipStream_t stream);
hipError_t turq_launch_dequant(int dtype, int layout, const void *w, int64_t n, int64_t k, float *out,
                               hipStream_t stream);
hipError_t turq_launch_wide_scale(const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, void *x16, float *inv, hipStream_t stream);
hipError_t turq_launch_wide_rescale(const float *y32, int64_t ld32, int64_t m, int64_t n, const float *inv, const float *bias, void *y,
                                    int y_dtype, int64_t ldy, hipStream_t stream);
hipError_t turq_launch_rms_norm(const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, const float *weight, float eps, void *y,
                                int y_dtype, int64_t ldy, hipStream_t stream);
hipError_t turq_launch_quantize_q8_0(const float *x, int64_t nblocks, void *out, hipStream_t stream);
hipError_t turq_launch_quantize_q8_k(const float *x, int64_t nblocks, void *out, hipStream_t stream);
hipError_t turq_launch_gemv_simple(int dtype, const void *w, int64_t n, int64_t k, const void *x, int x_dtype,
                                   int64_t m, int64_t ldx, void *y, int y_dtype, int64_t ldy, const float *bias,
                                   hipStream_t stream);

// per translation unit whose kernels store results: adds the current device's count of non-finite results to *sum (mfma_common.h)
#define TURQ_NONFINITE_UNITS(X)                                                                                                   \
    X(turq_nonfinite_gemv_mfma) X(turq_nonfinite_gemv_row1) X(turq_nonfinite_gemv_cs) X(turq_nonfinite_gemv_cs_staged_f32)         \
    X(turq_nonfinite_gemv_cs_staged_bf16) X(turq_nonfinite_gemv_cs_staged_f16) X(turq_nonfinite_gemm_mfma)                        \
    X(turq_nonfinite_gemv_simple) X(turq_nonfinite_act_mul) X(turq_nonfinite_wide) X(turq_nonfinite_norm) X(turq_nonfinite_act_prep)
#define TURQ_DECLARE_NONFINITE(fn) hipError_t fn(unsigned long long *sum, int reset);
TURQ_NONFINITE_UNITS(TURQ_DECLARE_NONFINITE)
#undef TURQ_DECLARE_NONFINITE

// RmsNorm taken into a forward call: x stands for x / sqrt(mean(x^2) + eps) * w (w: f32 [k] in device memory)
struct TurqNorm {
    const float *w;
    float eps;
};
// whether the kernels of a call with these weights and rows apply the norm themselves (one row: inside the matmul kernel; more
// than 32 rows: the norm writes the prefill GEMM's fragments); otherwise the caller normalises into scratch first
bool turq_norm_fuses(const turq_ctx *ctx, int count, const turq_weight *const *w, const void *x, int xt, int64_t ldx, int64_t m);

// largest m the skinny MFMA kernel takes; above it the LDS-tiled GEMM runs
#define TURQ_GEMV_MAX_M 32
// largest m for which the skinny kernel can prepare the activations itself (no separate launch);
// whether it does is decided per call in mfma_dispatch.cpp
#define TURQ_GEMV_FUSED_MAX_M 4
// MFMA paths on the tiled layout (activation preparation + kernel launch), see mfma_dispatch.cpp
int turq_qmatmul_mfma(turq_ctx *ctx, const turq_weight *w, const void *x, int xt, int64_t m, int64_t ldx, void *y,
                      int yt, int64_t ldy, const float *bias, int algo, const TurqNorm *norm = nullptr);
// act(gate) * up on two f32 matrices [m, n] of row stride n (act_mul.hip)
hipError_t turq_launch_read_yardstick(const void *buf, size_t nbytes, int workgroups, hipStream_t stream, hipEvent_t ev_start,
                                      hipEvent_t ev_stop);
hipError_t turq_launch_weight_prefetch(const void *buf, size_t nbytes, int workgroups, int depth, hipStream_t stream, hipEvent_t ev_start,
                                       hipEvent_t ev_stop);
hipError_t turq_launch_silu_mul(const float *gate, const float *up, int64_t m, int64_t n, void *y, int y_dtype, int64_t ldy,
                                hipStream_t stream);
// act(gate) * up inside the one-row kernel; *taken = false (and nothing launched) where that kernel does not apply
int turq_qmatmul_gate_up_mfma(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const void *x, int xt, int64_t m,
                              int64_t ldx, void *y, int yt, int64_t ldy, const float *bias_gate, const float *bias_up, bool *taken,
                              const TurqNorm *norm = nullptr);
// whether a call of 33 .. 64 rows on these weights goes through the kernels of up to 32 rows in two chunks
bool turq_rows_in_chunks(const turq_ctx *ctx, int count, const turq_weight *const *w, const void *x, int xt, int64_t ldx, int64_t m);
int turq_qmatmul_multi_gemm(turq_ctx *ctx, int count, const turq_weight *const *w, const void *x, int xt, int64_t m, int64_t ldx,
                            void *const *y, int yt, const int64_t *ldy, const float *const *bias, bool *taken, const TurqNorm *norm = nullptr);
// The whole MLP of a prompt chunk (more than 32 rows): gate / up GEMMs into f32 scratch, one kernel that turns the two products
// into down_proj's fragments, down_proj's GEMM on them; *taken = false (nothing launched) where that route does not apply
int turq_mlp_prefill(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const turq_weight *down, const void *x, int xt,
                     int64_t m, int64_t ldx, void *y, int yt, int64_t ldy, const float *bias_gate, const float *bias_up,
                     const float *bias_down, bool *taken, const TurqNorm *norm = nullptr);
int turq_qmatmul_multi_mfma(turq_ctx *ctx, int count, const turq_weight *const *w, const void *x, int xt, int64_t m,
                            int64_t ldx, void *const *y, int yt, const int64_t *ldy, const float *const *bias, const TurqNorm *norm = nullptr);

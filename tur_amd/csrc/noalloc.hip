// turq_qmatmul_noalloc: the forward call for hosts that cannot allocate device memory around it (code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc).  turq_qmatmul keeps the prepared activation fragments of calls with
// more than one row in a scratch buffer of the context that grows on demand; here that buffer is a static device array of a
// fixed size instead, and a call that would need more is refused.
#include "layout.h"
#include "mfma_common.h"

// Every GPU the library runs on holds its own copy of this array, at its own address, until the process ends.
static __device__ __align__(256) uint8_t scratch[TURQ_NOALLOC_SCRATCH_BYTES];

// Device address and size of the current device's copy.  In host code the array's name is only a handle for this lookup,
// never an address a kernel may be given.
hipError_t turq_static_scratch(void **ptr, size_t *cap) {
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) {
        *ptr = nullptr;
        *cap = 0;
        return e;
    }
    *ptr = p;
    *cap = (size_t)TURQ_NOALLOC_SCRATCH_BYTES;
    return hipSuccess;
}

namespace {
// scratch bytes turq_qmatmul would reserve for this call (mfma_dispatch.cpp): prepared fragments of one chunk of up to 32 rows
// for the skinny kernels, of all m rows for the prefill GEMM; a call with one row, or on the native layout, uses none
size_t scratch_need(const turq_weight *w, int64_t m) {
    if (w->layout != TURQ_LAYOUT_TILED || m <= 1) return 0;
    if (m <= TURQ_GEMV_MAX_M) return turq_act_prep_bytes(w->dtype, m, w->k);
    const size_t chunks = turq_act_prep_bytes(w->dtype, TURQ_GEMV_MAX_M, w->k);  // the GEMM's fallback walks m in chunks
    const size_t gemm = turq_act_prep32_bytes(m, w->k);
    return gemm > chunks ? gemm : chunks;
}

struct FixedScratch {  // the context's fragment buffer is the static array for the life of this object
    turq_ctx *ctx;
    void *buf;
    size_t cap;
    explicit FixedScratch(turq_ctx *c) : ctx(c), buf(c->act_prep), cap(c->act_prep_cap) {
        ctx->act_prep = ctx->static_scratch;
        ctx->act_prep_cap = ctx->static_scratch_cap;
        ctx->fixed_scratch = true;
    }
    ~FixedScratch() {
        ctx->act_prep = buf;
        ctx->act_prep_cap = cap;
        ctx->fixed_scratch = false;
    }
};
}  // namespace

static int noalloc_impl(turq_ctx *ctx, const turq_weight *w, const void *x, int x_dtype, int64_t m, int64_t ldx, void *y, int y_dtype,
                        int64_t ldy, const float *bias) {
    if (!w) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul_noalloc: null weight");
    if (!ctx->static_scratch)
        return turq_fail(ctx, TURQ_ERR_HIP, "turq_qmatmul_noalloc: the static scratch array of device %d could not be located: %s", ctx->device,
                         hipGetErrorString((hipError_t)ctx->static_scratch_err));
    // wide activations need scratch of their own (the scaled copy of the rows, their factors): rather than round f32 / bf16 rows to
    // f16 behind the back of a host that asked for the full range, the call says so
    if (ctx->wide && x_dtype != TURQ_ACT_F16 && w->layout == TURQ_LAYOUT_TILED)
        return turq_fail(ctx, TURQ_ERR_INVALID,
                         "turq_qmatmul_noalloc: wide activations are switched on for this context, and the call that allocates nothing cannot "
                         "scale rows; pass f16 activations, or use turq_qmatmul");
    if (m > 0 && w->k > 0) {
        const size_t need = scratch_need(w, m);
        if (need > ctx->static_scratch_cap)
            return turq_fail(ctx, TURQ_ERR_SHAPE,
                             "turq_qmatmul_noalloc: m=%lld rows of k=%lld columns need %zu bytes of prepared activations, the static scratch "
                             "array holds %zu; split the rows over several calls or use turq_qmatmul",
                             (long long)m, (long long)w->k, need, ctx->static_scratch_cap);
    }
    FixedScratch guard(ctx);
    return turq_qmatmul(ctx, w, x, x_dtype, m, ldx, y, y_dtype, ldy, bias, TURQ_MEM_DEVICE, TURQ_ALGO_AUTO);
}

extern "C" int turq_qmatmul_noalloc(turq_ctx *ctx, const turq_weight *w, const void *x, int x_dtype, int64_t m, int64_t ldx, void *y,
                                    int y_dtype, int64_t ldy, const float *bias) {
    if (!ctx) return turq_fail(nullptr, TURQ_ERR_INVALID, "turq_qmatmul_noalloc: null context");
    // (its own refusals end a running capture like those of every other forward call)
    return turq_capture_guard(ctx, noalloc_impl(ctx, w, x, x_dtype, m, ldx, y, y_dtype, ldy, bias));
}

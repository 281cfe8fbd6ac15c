// C ABI of libturq: contexts, device memory helpers, weight upload/export, dequantize, forward.
#include <algorithm>
#include <cmath>
#include <memory>
#include <new>
#include <vector>

#include "common.h"

std::string &turq_thread_error() {
    static thread_local std::string e;
    return e;
}

int turq_ctx_reserve(turq_ctx *ctx, void **buf, size_t *cap, size_t need) {
    if (need <= *cap) return TURQ_OK;
    if (ctx->fixed_scratch)
        return turq_fail(ctx, TURQ_ERR_INVALID, "this call needs %zu bytes of scratch memory, the static array it may use holds %zu", need, *cap);
    if (ctx->capturing)
        return turq_fail(ctx, TURQ_ERR_INVALID, "a scratch buffer would have to grow (%zu > %zu bytes) while a graph is being captured: run the same calls once before turq_graph_begin", need, *cap);
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));  // the old buffer may still be in use
    const bool graphs_alive = ctx->tally && ctx->tally->live.load(std::memory_order_acquire) > 0;
    if (!graphs_alive) {  // nothing refers to outgrown buffers any more
        for (void *p : ctx->retired) (void)hipFree(p);
        ctx->retired.clear();
    }
    if (*buf) {
        // a captured graph holds the addresses it was recorded with: while one is alive the old buffer stays allocated
        if (graphs_alive) {
            try {
                ctx->retired.push_back(*buf);
            } catch (const std::bad_alloc &) {
                return turq_fail(ctx, TURQ_ERR_OOM, "turq_ctx_reserve: out of host memory");
            }
        } else {
            TURQ_HIP(ctx, hipFree(*buf));
        }
        *buf = nullptr;
        *cap = 0;
    }
    size_t want = need + need / 4 + 4096;
    TURQ_HIP(ctx, hipMalloc(buf, want));
    *cap = want;
    return TURQ_OK;
}

hipError_t turq_prof_next(turq_ctx *ctx, hipEvent_t *start, hipEvent_t *stop) {
    *start = nullptr;
    *stop = nullptr;
    if (!ctx->profiling) return hipSuccess;
    if (ctx->prof_used == ctx->prof_events.size()) {
        if (ctx->fixed_scratch) return hipSuccess;  // a call that may not allocate: this launch goes untimed
        hipEvent_t a = nullptr, b = nullptr;
        hipError_t e = hipEventCreate(&a);
        if (e != hipSuccess) return e;
        e = hipEventCreate(&b);
        if (e != hipSuccess) { (void)hipEventDestroy(a); return e; }
        ctx->prof_events.emplace_back(a, b);
    }
    *start = ctx->prof_events[ctx->prof_used].first;
    *stop = ctx->prof_events[ctx->prof_used].second;
    ctx->prof_used++;
    return hipSuccess;
}

namespace {

float half_bits_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu, bits;
    if (exp == 0) {
        if (man == 0) bits = sign;
        else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) bits = sign | 0x7F800000u | (man << 13);
    else bits = sign | ((exp + 112u) << 23) | (man << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

struct DeviceGuard {  // make ctx's device current for the duration of a call
    int prev = -1;
    bool ok = true;
    explicit DeviceGuard(int dev) {
        if (hipGetDevice(&prev) != hipSuccess) prev = -1;
        if (prev != dev) ok = hipSetDevice(dev) == hipSuccess;
    }
    ~DeviceGuard() {
        int cur = -1;
        if (prev >= 0 && hipGetDevice(&cur) == hipSuccess && cur != prev) (void)hipSetDevice(prev);
    }
};

#define TURQ_ENTER(ctx)                                                                     \
    if (!(ctx)) return turq_fail(nullptr, TURQ_ERR_INVALID, "%s: null context", __func__); \
    DeviceGuard guard_((ctx)->device);                                                      \
    if (!guard_.ok) return turq_fail((ctx), TURQ_ERR_HIP, "%s: hipSetDevice(%d) failed", __func__, (ctx)->device)

}  // namespace

extern "C" {

const char *turq_version(void) { return "turq 0.1 (gfx950)"; }
int turq_block_elems(int dt) { return turq_dt_block_elems(dt); }
int turq_block_bytes(int dt) { return turq_dt_block_bytes(dt); }

size_t turq_weight_nbytes(int dt, int64_t n, int64_t k) {
    const int be = turq_dt_block_elems(dt);
    if (be == 0 || n < 0 || k < 0 || k % be) return 0;
    return (size_t)n * (size_t)(k / be) * (size_t)turq_dt_block_bytes(dt);
}

int turq_ctx_create(int device, turq_ctx **out) {
    if (!out) return turq_fail(nullptr, TURQ_ERR_INVALID, "turq_ctx_create: null out pointer");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess) return turq_fail(nullptr, TURQ_ERR_HIP, "hipGetDeviceCount failed: %s", hipGetErrorString(e));
    if (device < 0 || device >= count)
        return turq_fail(nullptr, TURQ_ERR_INVALID, "turq_ctx_create: device %d out of range (%d visible)", device, count);
    std::unique_ptr<turq_ctx> ctx(new (std::nothrow) turq_ctx);
    if (!ctx) return turq_fail(nullptr, TURQ_ERR_OOM, "turq_ctx_create: out of host memory");
    ctx->device = device;
    DeviceGuard guard(device);
    if (!guard.ok) return turq_fail(nullptr, TURQ_ERR_HIP, "turq_ctx_create: hipSetDevice(%d) failed", device);
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return turq_fail(nullptr, TURQ_ERR_HIP, "hipGetDeviceProperties failed: %s", hipGetErrorString(e));
    ctx->compute_units = prop.multiProcessorCount;
    snprintf(ctx->device_name, sizeof ctx->device_name, "%s (%s)", prop.name, prop.gcnArchName);
    try {
        ctx->tally = std::make_shared<turq_graph_tally>();
    } catch (const std::bad_alloc &) {
        return turq_fail(nullptr, TURQ_ERR_OOM, "turq_ctx_create: out of host memory");
    }
    // the device's copy of the static scratch array of turq_qmatmul_noalloc; a failure is reported by that entry point
    ctx->static_scratch_err = (int)turq_static_scratch(&ctx->static_scratch, &ctx->static_scratch_cap);
    if (ctx->static_scratch_err != (int)hipSuccess) { ctx->static_scratch = nullptr; ctx->static_scratch_cap = 0; }
    e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (e != hipSuccess) return turq_fail(nullptr, TURQ_ERR_HIP, "hipStreamCreate failed: %s", hipGetErrorString(e));
    // the prefetch stream and its events exist from the start: nothing can be created while a graph is being captured
    e = hipStreamCreateWithFlags(&ctx->pf_stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&ctx->ev_pf_fork, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&ctx->ev_pf_join, hipEventDisableTiming);
    if (e != hipSuccess) {
        turq_ctx *dead = ctx.release();
        turq_ctx_destroy(dead);
        return turq_fail(nullptr, TURQ_ERR_HIP, "turq_ctx_create: the prefetch stream could not be made: %s", hipGetErrorString(e));
    }
    ctx->pf_workgroups = ctx->compute_units > 0 ? ctx->compute_units : 256;
    const TurqTuning &tune = turq_tuning();  // (the first context of a process reads the environment here)
    if (tune.prefetch_wgs >= 1 && tune.prefetch_wgs <= 4096) ctx->pf_workgroups = tune.prefetch_wgs;
    if (tune.prefetch_depth >= 1 && tune.prefetch_depth <= 4) ctx->pf_depth = tune.prefetch_depth;
    *out = ctx.release();
    return TURQ_OK;
}

void turq_ctx_destroy(turq_ctx *ctx) {
    if (!ctx) return;
    DeviceGuard guard(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (ctx->stage_x) (void)hipFree(ctx->stage_x);
    if (ctx->stage_y) (void)hipFree(ctx->stage_y);
    if (ctx->act_prep) (void)hipFree(ctx->act_prep);
    if (ctx->gate_up) (void)hipFree(ctx->gate_up);
    if (ctx->mlp_h) (void)hipFree(ctx->mlp_h);
    if (ctx->norm_x) (void)hipFree(ctx->norm_x);
    if (ctx->gemm_split) (void)hipFree(ctx->gemm_split);
    if (ctx->wide_x) (void)hipFree(ctx->wide_x);
    if (ctx->wide_s) (void)hipFree(ctx->wide_s);
    if (ctx->wide_y) (void)hipFree(ctx->wide_y);
    if (ctx->stage_b) (void)hipFree(ctx->stage_b);
    for (void *p : ctx->retired) (void)hipFree(p);  // graphs that still refer to them can no longer be launched: that needs the context
    for (auto &p : ctx->prof_events) { (void)hipEventDestroy(p.first); (void)hipEventDestroy(p.second); }
    for (int i = 0; i < turq_ctx::kSide; i++) {
        if (ctx->side[i]) { (void)hipStreamSynchronize(ctx->side[i]); (void)hipStreamDestroy(ctx->side[i]); }
        if (ctx->ev_join[i]) (void)hipEventDestroy(ctx->ev_join[i]);
    }
    if (ctx->ev_fork) (void)hipEventDestroy(ctx->ev_fork);
    if (ctx->pf_stream) { (void)hipStreamSynchronize(ctx->pf_stream); (void)hipStreamDestroy(ctx->pf_stream); }
    if (ctx->ev_pf_fork) (void)hipEventDestroy(ctx->ev_pf_fork);
    if (ctx->ev_pf_join) (void)hipEventDestroy(ctx->ev_pf_join);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

const char *turq_last_error(const turq_ctx *ctx) { return ctx ? ctx->err.c_str() : turq_thread_error().c_str(); }

int turq_sync(turq_ctx *ctx) {
    TURQ_ENTER(ctx);
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (!ctx->capturing) TURQ_HIP(ctx, hipStreamSynchronize(ctx->pf_stream));
    return TURQ_OK;
}

void *turq_ctx_stream(turq_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int turq_ctx_device_info(turq_ctx *ctx, char *name, size_t cap, int *cus) {
    if (!ctx) return turq_fail(nullptr, TURQ_ERR_INVALID, "turq_ctx_device_info: null context");
    if (name && cap) snprintf(name, cap, "%s", ctx->device_name);
    if (cus) *cus = ctx->compute_units;
    return TURQ_OK;
}

int turq_dev_alloc(turq_ctx *ctx, size_t nbytes, void **out) {
    TURQ_ENTER(ctx);
    if (!out) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_dev_alloc: null out pointer");
    *out = nullptr;
    if (nbytes == 0) return TURQ_OK;
    TURQ_HIP(ctx, hipMalloc(out, nbytes));
    return TURQ_OK;
}

int turq_dev_free(turq_ctx *ctx, void *ptr) {
    TURQ_ENTER(ctx);
    if (!ptr) return TURQ_OK;
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    TURQ_HIP(ctx, hipFree(ptr));
    return TURQ_OK;
}

int turq_memcpy_h2d(turq_ctx *ctx, void *dst, const void *src, size_t nbytes) {
    TURQ_ENTER(ctx);
    if (nbytes == 0) return TURQ_OK;
    if (!dst || !src) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_memcpy_h2d: null pointer");
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    TURQ_HIP(ctx, hipMemcpy(dst, src, nbytes, hipMemcpyHostToDevice));
    return TURQ_OK;
}

int turq_memcpy_d2h(turq_ctx *ctx, void *dst, const void *src, size_t nbytes) {
    TURQ_ENTER(ctx);
    if (nbytes == 0) return TURQ_OK;
    if (!dst || !src) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_memcpy_d2h: null pointer");
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    TURQ_HIP(ctx, hipMemcpy(dst, src, nbytes, hipMemcpyDeviceToHost));
    return TURQ_OK;
}

// ---- weights ----

int turq_weight_upload(turq_ctx *ctx, int dt, int64_t n, int64_t k, const void *host_bytes, size_t nbytes,
                       int layout, turq_weight **out) {
    TURQ_ENTER(ctx);
    if (!out) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_weight_upload: null out pointer");
    *out = nullptr;
    const int be = turq_dt_block_elems(dt);
    if (be == 0) return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_weight_upload: unsupported ggml dtype %d", dt);
    if (n < 0 || k < 0) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_weight_upload: negative shape (%lld, %lld)", (long long)n, (long long)k);
    if (k % be)
        return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_weight_upload: k=%lld is not a multiple of the %s block size %d",
                         (long long)k, turq_dt_name(dt), be);
    const size_t expect = turq_weight_nbytes(dt, n, k);
    if (nbytes != expect)
        return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_weight_upload: got %zu bytes, a %s tensor of shape (%lld, %lld) has %zu",
                         nbytes, turq_dt_name(dt), (long long)n, (long long)k, expect);
    if (!host_bytes && nbytes) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_weight_upload: null data pointer");
    if (layout != TURQ_LAYOUT_NATIVE && layout != TURQ_LAYOUT_TILED)
        return turq_fail(ctx, TURQ_ERR_INVALID, "turq_weight_upload: unknown layout %d", layout);
    if (layout == TURQ_LAYOUT_TILED && !turq_dt_is_quant(dt))
        return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_weight_upload: the tiled layout holds quantized dtypes only, got %s", turq_dt_name(dt));

    std::unique_ptr<turq_weight> w(new (std::nothrow) turq_weight);
    if (!w) return turq_fail(ctx, TURQ_ERR_OOM, "turq_weight_upload: out of host memory");
    w->device = ctx->device;
    w->dtype = dt;
    w->layout = layout;
    w->n = n;
    w->k = k;
    w->native_bytes = nbytes;
    const uint8_t *src = (const uint8_t *)host_bytes;
    if (turq_dt_is_quant(dt)) {
        // bound on the scale a weight is multiplied by: |d * sc| for the K-quants (6-bit scales <= 63, Q6_K int8 scales <= 128
        // in magnitude), |d| for Q8_0; see turq_weight::max_scale.  Q4_K / Q5_K: dmin counts with 1 / 1024 of its size, which
        // is what its packed-f16 constant (dmin * m, no base of 1024 on it) needs next to those of d.
        const int bs = turq_block_bytes(dt), d_at = dt == TURQ_Q6_K ? 208 : 0;
        const bool has_min = dt == TURQ_Q4_K || dt == TURQ_Q5_K;
        float mx = 0.0f;
        const int64_t nblk = n * (k / turq_dt_block_elems(dt));
        for (int64_t i = 0; i < nblk; i++) {
            const uint8_t *b = src + i * bs + d_at;
            const float d = std::fabs(half_bits_to_float((uint16_t)(b[0] | (b[1] << 8))));
            if (d > mx || d != d) mx = d;
            if (has_min) {
                const float dm = std::fabs(half_bits_to_float((uint16_t)(b[2] | (b[3] << 8)))) * (1.0f / 1024.0f);
                if (dm > mx || dm != dm) mx = dm;
            }
        }
        w->max_scale = mx * (dt == TURQ_Q8_0 ? 1.0f : dt == TURQ_Q6_K ? 128.0f : 63.0f);
    }
    std::vector<uint8_t> tiled;
    if (layout == TURQ_LAYOUT_TILED) {
        w->dev_bytes = turq_tiled_nbytes(dt, n, k);
        try {
            tiled.resize(w->dev_bytes);
        } catch (const std::bad_alloc &) {
            return turq_fail(ctx, TURQ_ERR_OOM, "turq_weight_upload: out of host memory for the tiled copy (%zu bytes)", w->dev_bytes);
        }
        int rc = turq_tile_host(dt, n, k, host_bytes, tiled.data());
        if (rc != TURQ_OK) return turq_fail(ctx, rc, "%s", turq_thread_error().c_str());
        src = tiled.data();
    } else {
        w->dev_bytes = nbytes;
    }
    if (w->dev_bytes) {
        // a few bytes of slack so that vector loads at the tail of the last row stay in bounds
        TURQ_HIP(ctx, hipMalloc(&w->dev, w->dev_bytes + 64));
        hipError_t e = hipMemcpy(w->dev, src, w->dev_bytes, hipMemcpyHostToDevice);
        if (e == hipSuccess) e = hipMemset((uint8_t *)w->dev + w->dev_bytes, 0, 64);
        if (e != hipSuccess) {
            (void)hipFree(w->dev);
            return turq_fail(ctx, TURQ_ERR_HIP, "turq_weight_upload: copy to device failed: %s", hipGetErrorString(e));
        }
    }
    *out = w.release();
    return TURQ_OK;
}

int turq_weight_retain(turq_weight *w) {
    if (!w) return turq_fail(nullptr, TURQ_ERR_INVALID, "turq_weight_retain: null weight");
    w->refs.fetch_add(1, std::memory_order_relaxed);
    return TURQ_OK;
}

int turq_weight_release(turq_weight *w) {
    if (!w) return TURQ_OK;
    if (w->refs.fetch_sub(1, std::memory_order_acq_rel) == 1) {
        if (w->dev) {
            DeviceGuard guard(w->device);
            (void)hipDeviceSynchronize();
            (void)hipFree(w->dev);
        }
        delete w;
    }
    return TURQ_OK;
}

int turq_weight_info(const turq_weight *w, int *dt, int64_t *n, int64_t *k, int *layout, size_t *device_bytes) {
    if (!w) return turq_fail(nullptr, TURQ_ERR_INVALID, "turq_weight_info: null weight");
    if (dt) *dt = w->dtype;
    if (n) *n = w->n;
    if (k) *k = w->k;
    if (layout) *layout = w->layout;
    if (device_bytes) *device_bytes = w->dev_bytes;
    return TURQ_OK;
}

int turq_weight_export(turq_ctx *ctx, const turq_weight *w, void *host_bytes, size_t nbytes) {
    TURQ_ENTER(ctx);
    if (!w) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_weight_export: null weight");
    if (nbytes != w->native_bytes)
        return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_weight_export: buffer has %zu bytes, tensor has %zu", nbytes, w->native_bytes);
    if (nbytes == 0) return TURQ_OK;
    if (!host_bytes) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_weight_export: null buffer");
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (w->layout == TURQ_LAYOUT_NATIVE) {
        TURQ_HIP(ctx, hipMemcpy(host_bytes, w->dev, nbytes, hipMemcpyDeviceToHost));
        return TURQ_OK;
    }
    std::vector<uint8_t> tiled;
    try {
        tiled.resize(w->dev_bytes);
    } catch (const std::bad_alloc &) {
        return turq_fail(ctx, TURQ_ERR_OOM, "turq_weight_export: out of host memory");
    }
    TURQ_HIP(ctx, hipMemcpy(tiled.data(), w->dev, w->dev_bytes, hipMemcpyDeviceToHost));
    int rc = turq_untile_host(w->dtype, w->n, w->k, tiled.data(), host_bytes);
    if (rc != TURQ_OK) return turq_fail(ctx, rc, "%s", turq_thread_error().c_str());
    return TURQ_OK;
}

// ---- dequantize ----

static int impl_dequantize(turq_ctx *ctx, const turq_weight *w, float *out, int out_mem) {
    TURQ_ENTER(ctx);
    if (!w) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_dequantize: null weight");
    if (w->device != ctx->device) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_dequantize: weight lives on device %d, context on %d", w->device, ctx->device);
    const size_t nelem = (size_t)w->n * (size_t)w->k;
    if (nelem == 0) return TURQ_OK;
    if (!out) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_dequantize: null output");
    if (!turq_dt_is_quant(w->dtype) && w->dtype != TURQ_F32 && w->dtype != TURQ_F16 && w->dtype != TURQ_BF16)
        return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_dequantize: unsupported dtype %d", w->dtype);
    if (out_mem == TURQ_MEM_DEVICE) {
        TURQ_HIP(ctx, turq_launch_dequant(w->dtype, w->layout, w->dev, w->n, w->k, out, ctx->stream));
        return TURQ_OK;
    }
    if (out_mem != TURQ_MEM_HOST) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_dequantize: bad out_mem %d", out_mem);
    int rc = turq_ctx_reserve(ctx, &ctx->stage_y, &ctx->stage_y_cap, nelem * sizeof(float));
    if (rc != TURQ_OK) return rc;
    TURQ_HIP(ctx, turq_launch_dequant(w->dtype, w->layout, w->dev, w->n, w->k, (float *)ctx->stage_y, ctx->stream));
    TURQ_HIP(ctx, hipMemcpyAsync(out, ctx->stage_y, nelem * sizeof(float), hipMemcpyDeviceToHost, ctx->stream));
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return TURQ_OK;
}

static int impl_embedding_lookup(turq_ctx *ctx, const turq_weight *w, const uint32_t *ids, int64_t count, void *out, int out_dtype,
                          int64_t ldo, int mem) {
    TURQ_ENTER(ctx);
    if (!w) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_embedding_lookup: null weight");
    if (w->device != ctx->device) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_embedding_lookup: weight lives on device %d, context on %d", w->device, ctx->device);
    if (!turq_dt_is_quant(w->dtype) && w->dtype != TURQ_F32 && w->dtype != TURQ_F16 && w->dtype != TURQ_BF16)
        return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_embedding_lookup: unsupported dtype %d", w->dtype);
    const int ob = turq_act_bytes(out_dtype);
    if (!ob) return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_embedding_lookup: output dtype %d", out_dtype);
    if (count < 0) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_embedding_lookup: count=%lld is negative", (long long)count);
    if (ldo < w->k) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_embedding_lookup: ldo=%lld is smaller than the row length %lld", (long long)ldo, (long long)w->k);
    if (count == 0 || w->k == 0) return TURQ_OK;
    if (!ids || !out) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_embedding_lookup: null index or output pointer");
    if (mem == TURQ_MEM_DEVICE) {
        TURQ_HIP(ctx, turq_launch_gather_rows(w->dtype, w->layout, w->dev, w->n, w->k, ids, count, out, out_dtype, ldo, ctx->stream));
        return TURQ_OK;
    }
    if (mem != TURQ_MEM_HOST) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_embedding_lookup: bad mem %d", mem);
    for (int64_t i = 0; i < count; i++)  // host indices can be checked before anything runs (candle's index_select refuses them too)
        if ((int64_t)ids[i] >= w->n)
            return turq_fail(ctx, TURQ_ERR_INVALID, "turq_embedding_lookup: index %u at position %lld is outside the table of %lld rows",
                             ids[i], (long long)i, (long long)w->n);
    const size_t row = (size_t)w->k * (size_t)ob;
    int rc = turq_ctx_reserve(ctx, &ctx->stage_x, &ctx->stage_x_cap, (size_t)count * sizeof(uint32_t));
    if (rc != TURQ_OK) return rc;
    rc = turq_ctx_reserve(ctx, &ctx->stage_y, &ctx->stage_y_cap, row * (size_t)count);
    if (rc != TURQ_OK) return rc;
    TURQ_HIP(ctx, hipMemcpyAsync(ctx->stage_x, ids, (size_t)count * sizeof(uint32_t), hipMemcpyHostToDevice, ctx->stream));
    TURQ_HIP(ctx, turq_launch_gather_rows(w->dtype, w->layout, w->dev, w->n, w->k, (const uint32_t *)ctx->stage_x, count, ctx->stage_y,
                                          out_dtype, w->k, ctx->stream));
    TURQ_HIP(ctx, hipMemcpy2DAsync(out, (size_t)ldo * ob, ctx->stage_y, row, row, (size_t)count, hipMemcpyDeviceToHost, ctx->stream));
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return TURQ_OK;
}

// ---- RmsNorm ----

static int impl_rms_norm(turq_ctx *ctx, const void *x, int xt, int64_t m, int64_t k, int64_t ldx, const float *weight, float eps, void *y,
                         int yt, int64_t ldy, int mem) {
    TURQ_ENTER(ctx);
    const int xb = turq_act_bytes(xt), yb = turq_act_bytes(yt);
    if (!xb) return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_rms_norm: unsupported activation dtype %d", xt);
    if (!yb) return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_rms_norm: unsupported output dtype %d", yt);
    if (m < 0 || k < 0) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_rms_norm: negative shape (%lld, %lld)", (long long)m, (long long)k);
    if (ldx < k || ldy < k) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_rms_norm: a row stride (%lld, %lld) is smaller than k=%lld", (long long)ldx, (long long)ldy, (long long)k);
    if (m == 0 || k == 0) return TURQ_OK;
    if (!x || !y || !weight) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_rms_norm: null activation, weight or output pointer");
    if (mem == TURQ_MEM_DEVICE) {
        TURQ_HIP(ctx, turq_launch_rms_norm(x, xt, m, k, ldx, weight, eps, y, yt, ldy, ctx->stream));
        return TURQ_OK;
    }
    if (mem != TURQ_MEM_HOST) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_rms_norm: bad mem %d", mem);
    const size_t xrow = (size_t)k * xb, yrow = (size_t)k * yb;
    int rc = turq_ctx_reserve(ctx, &ctx->stage_x, &ctx->stage_x_cap, xrow * (size_t)m);
    if (rc != TURQ_OK) return rc;
    rc = turq_ctx_reserve(ctx, &ctx->stage_y, &ctx->stage_y_cap, yrow * (size_t)m);
    if (rc != TURQ_OK) return rc;
    rc = turq_ctx_reserve(ctx, &ctx->stage_b, &ctx->stage_b_cap, (size_t)k * sizeof(float));
    if (rc != TURQ_OK) return rc;
    TURQ_HIP(ctx, hipMemcpy2DAsync(ctx->stage_x, xrow, x, (size_t)ldx * xb, xrow, (size_t)m, hipMemcpyHostToDevice, ctx->stream));
    TURQ_HIP(ctx, hipMemcpyAsync(ctx->stage_b, weight, (size_t)k * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    TURQ_HIP(ctx, turq_launch_rms_norm(ctx->stage_x, xt, m, k, k, (const float *)ctx->stage_b, eps, ctx->stage_y, yt, k, ctx->stream));
    TURQ_HIP(ctx, hipMemcpy2DAsync(y, (size_t)ldy * yb, ctx->stage_y, yrow, yrow, (size_t)m, hipMemcpyDeviceToHost, ctx->stream));
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return TURQ_OK;
}

// ---- forward ----

// wide: activations of any finite f32 magnitude (wide.hip) where the kernel would round them to f16
static int qmatmul_device(turq_ctx *ctx, const turq_weight *w, const void *x, int xt, int64_t m, int64_t ldx, void *y,
                          int yt, int64_t ldy, const float *bias, int algo, bool wide) {
    if (algo == TURQ_ALGO_AUTO) {
        if (w->layout == TURQ_LAYOUT_NATIVE) algo = TURQ_ALGO_SIMPLE;
        else algo = (m <= TURQ_GEMV_MAX_M || turq_rows_in_chunks(ctx, 1, &w, x, xt, ldx, m)) ? TURQ_ALGO_GEMV : TURQ_ALGO_GEMM;
    }
    if (wide && !ctx->fixed_scratch && xt != TURQ_ACT_F16 && (algo == TURQ_ALGO_GEMV || algo == TURQ_ALGO_GEMM) &&
        w->layout == TURQ_LAYOUT_TILED) {
        // rows scaled by powers of two into the f16 range, the plain call on the f16 copy, rows scaled back (+ bias)
        int rc = turq_ctx_reserve(ctx, &ctx->wide_x, &ctx->wide_x_cap, (size_t)m * (size_t)w->k * 2);
        if (rc != TURQ_OK) return rc;
        rc = turq_ctx_reserve(ctx, &ctx->wide_s, &ctx->wide_s_cap, (size_t)m * sizeof(float));
        if (rc != TURQ_OK) return rc;
        float *y32 = (float *)y;
        int64_t ld32 = ldy;
        if (yt != TURQ_ACT_F32) {  // (also an f32 output that is added to: the product must not land on the residual stream)
            rc = turq_ctx_reserve(ctx, &ctx->wide_y, &ctx->wide_y_cap, (size_t)m * (size_t)w->n * sizeof(float));
            if (rc != TURQ_OK) return rc;
            y32 = (float *)ctx->wide_y;
            ld32 = w->n;
        }
        TURQ_HIP(ctx, turq_launch_wide_scale(x, xt, m, w->k, ldx, ctx->wide_x, (float *)ctx->wide_s, ctx->stream));
        rc = turq_qmatmul_mfma(ctx, w, ctx->wide_x, TURQ_ACT_F16, m, w->k, y32, TURQ_ACT_F32, ld32, nullptr, algo);
        if (rc != TURQ_OK) return rc;
        TURQ_HIP(ctx, turq_launch_wide_rescale(y32, ld32, m, w->n, (const float *)ctx->wide_s, bias, y, yt, ldy, ctx->stream));
        return TURQ_OK;
    }
    switch (algo) {
    case TURQ_ALGO_SIMPLE:
        if (w->layout != TURQ_LAYOUT_NATIVE)
            return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul: TURQ_ALGO_SIMPLE needs a weight in the native layout");
        TURQ_HIP(ctx, turq_launch_gemv_simple(w->dtype, w->dev, w->n, w->k, x, xt, m, ldx, y, yt, ldy, bias, ctx->stream));
        return TURQ_OK;
    case TURQ_ALGO_GEMV:
    case TURQ_ALGO_GEMM:
        if (w->layout != TURQ_LAYOUT_TILED)
            return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul: the MFMA kernels need a weight in the tiled layout");
        return turq_qmatmul_mfma(ctx, w, x, xt, m, ldx, y, yt, ldy, bias, algo);
    default:
        return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul: unknown algo %d", algo);
    }
}

static int impl_qmatmul(turq_ctx *ctx, const turq_weight *w, const void *x, int xt, int64_t m, int64_t ldx, void *y, int yt,
                 int64_t ldy, const float *bias, int mem, int algo) {
    TURQ_ENTER(ctx);
    if (!w) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul: null weight");
    if (w->device != ctx->device) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul: weight lives on device %d, context on %d", w->device, ctx->device);
    if (!turq_dt_is_quant(w->dtype) && w->dtype != TURQ_F32 && w->dtype != TURQ_F16 && w->dtype != TURQ_BF16)
        return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_qmatmul: unsupported weight dtype %d", w->dtype);
    const int xb = (xt & ~0xFF) ? 0 : turq_act_bytes(xt), yb = turq_yt_ok(yt, true) ? turq_act_bytes(yt) : 0;
    if (!xb) return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_qmatmul: unsupported activation dtype %d", xt);
    if (!yb) return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_qmatmul: unsupported output dtype %d", yt);
    if (m < 0) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_qmatmul: m=%lld is negative", (long long)m);
    if (ldx < w->k) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_qmatmul: ldx=%lld is smaller than k=%lld", (long long)ldx, (long long)w->k);
    if (ldy < w->n) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_qmatmul: ldy=%lld is smaller than n=%lld", (long long)ldy, (long long)w->n);
    if (m == 0 || w->n == 0) return TURQ_OK;
    if (!x || !y) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul: null activation or output pointer");
    if (w->k == 0) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_qmatmul: k=0");

    if (mem == TURQ_MEM_DEVICE) return qmatmul_device(ctx, w, x, xt, m, ldx, y, yt, ldy, bias, algo, ctx->wide);
    if (mem != TURQ_MEM_HOST) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul: bad mem %d", mem);

    // host pointers: stage rows densely (ld = k / n on the device side), run, copy back
    const size_t xrow = (size_t)w->k * xb, yrow = (size_t)w->n * yb;
    int rc = turq_ctx_reserve(ctx, &ctx->stage_x, &ctx->stage_x_cap, xrow * (size_t)m);
    if (rc != TURQ_OK) return rc;
    rc = turq_ctx_reserve(ctx, &ctx->stage_y, &ctx->stage_y_cap, yrow * (size_t)m);
    if (rc != TURQ_OK) return rc;
    TURQ_HIP(ctx, hipMemcpy2DAsync(ctx->stage_x, xrow, x, (size_t)ldx * xb, xrow, (size_t)m, hipMemcpyHostToDevice, ctx->stream));
    if (yt & TURQ_OUT_ACCUMULATE)  // the rows that the results are added to
        TURQ_HIP(ctx, hipMemcpy2DAsync(ctx->stage_y, yrow, y, (size_t)ldy * yb, yrow, (size_t)m, hipMemcpyHostToDevice, ctx->stream));
    if (bias) {  // with host pointers the bias is a host array too
        rc = turq_ctx_reserve(ctx, &ctx->stage_b, &ctx->stage_b_cap, (size_t)w->n * sizeof(float));
        if (rc != TURQ_OK) return rc;
        TURQ_HIP(ctx, hipMemcpyAsync(ctx->stage_b, bias, (size_t)w->n * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
        bias = (const float *)ctx->stage_b;
    }
    // host tensors are the reference's own contract (f32 activations of any magnitude, src/weights/mod.rs:84-99): always wide
    rc = qmatmul_device(ctx, w, ctx->stage_x, xt, m, w->k, ctx->stage_y, yt, w->n, bias, algo, true);
    if (rc != TURQ_OK) return rc;
    TURQ_HIP(ctx, hipMemcpy2DAsync(y, (size_t)ldy * yb, ctx->stage_y, yrow, yrow, (size_t)m, hipMemcpyDeviceToHost, ctx->stream));
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return TURQ_OK;
}

static int impl_qmatmul_multi(turq_ctx *ctx, int count, const turq_weight *const *weights, const void *x, int xt, int64_t m,
                       int64_t ldx, void *const *ys, int yt, const int64_t *ldys, const float *const *biases, int mem, int algo) {
    TURQ_ENTER(ctx);
    if (count < 0) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul_multi: count=%d is negative", count);
    if (count == 0) return TURQ_OK;
    if (!weights || !ys || !ldys) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul_multi: null weight, output or stride array");
    const bool many_rows = m > TURQ_GEMV_MAX_M && (algo == TURQ_ALGO_AUTO || algo == TURQ_ALGO_GEMM);
    bool one_launch = mem == TURQ_MEM_DEVICE && !(ctx->wide && xt != TURQ_ACT_F16) && count > 1 && x != nullptr &&
                      (many_rows || ((algo == TURQ_ALGO_AUTO || algo == TURQ_ALGO_GEMV) && m >= 1 && m <= TURQ_GEMV_MAX_M));
    for (int i = 0; i < count && one_launch; i++) {
        const turq_weight *w = weights[i];
        one_launch = w && ys[i] && w->device == ctx->device && turq_dt_is_quant(w->dtype) && w->layout == TURQ_LAYOUT_TILED &&
                     w->k == weights[0]->k && w->k > 0 && w->n > 0 && ldys[i] >= w->n;
    }
    if (yt & ~0xFF) return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_qmatmul_multi: output dtype %d (TURQ_OUT_ACCUMULATE is for turq_qmatmul and turq_mlp)", yt);
    const int xb = (xt & ~0xFF) ? 0 : turq_act_bytes(xt), yb = turq_act_bytes(yt);
    one_launch = one_launch && xb && yb && ldx >= weights[0]->k;
    if (one_launch && many_rows && turq_rows_in_chunks(ctx, count, weights, x, xt, ldx, m)) {
        void *yc[4];
        for (int64_t m0 = 0; m0 < m; m0 += TURQ_GEMV_MAX_M) {
            for (int i = 0; i < count; i++) yc[i] = (uint8_t *)ys[i] + (size_t)m0 * (size_t)ldys[i] * yb;
            const int rc = turq_qmatmul_multi_mfma(ctx, count, weights, (const uint8_t *)x + (size_t)m0 * (size_t)ldx * xb, xt,
                                                   std::min<int64_t>(TURQ_GEMV_MAX_M, m - m0), ldx, yc, yt, ldys, biases);
            if (rc != TURQ_OK) return rc;
        }
        return TURQ_OK;
    }
    if (one_launch && many_rows) {
        // prefill: one preparation of the activations for all the weights, then a GEMM each
        bool taken = false;
        const int rc = turq_qmatmul_multi_gemm(ctx, count, weights, x, xt, m, ldx, ys, yt, ldys, biases, &taken);
        if (rc != TURQ_OK || taken) return rc;
        one_launch = false;
    }
    if (!one_launch) {
        // anything else is the same as the calls one after the other (which also report what is wrong with an argument)
        for (int i = 0; i < count; i++) {
            const int rc = turq_qmatmul(ctx, weights[i], x, xt, m, ldx, ys[i], yt, ldys[i], biases ? biases[i] : nullptr, mem, algo);
            if (rc != TURQ_OK) return rc;
        }
        return TURQ_OK;
    }
    return turq_qmatmul_multi_mfma(ctx, count, weights, x, xt, m, ldx, ys, yt, ldys, biases);
}

namespace {
uint16_t host_bf16(float v) {  // round to nearest even, as the kernels store it
    uint32_t u;
    memcpy(&u, &v, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
}  // namespace

static int impl_qmatmul_gate_up(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const void *x, int xt, int64_t m, int64_t ldx,
                         void *y, int yt, int64_t ldy, const float *bias_gate, const float *bias_up, int act, int mem) {
    TURQ_ENTER(ctx);
    if (!gate || !up) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul_gate_up: null weight");
    if (act != TURQ_ACTFN_SILU) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul_gate_up: activation %d is not supported", act);
    if (gate->n != up->n || gate->k != up->k)
        return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_qmatmul_gate_up: gate is [%lld, %lld], up is [%lld, %lld]", (long long)gate->n,
                         (long long)gate->k, (long long)up->n, (long long)up->k);
    if (mem != TURQ_MEM_DEVICE && mem != TURQ_MEM_HOST) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul_gate_up: bad mem %d", mem);
    const int yb = (yt & ~0xFF) ? 0 : turq_act_bytes(yt);
    if (!yb) return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_qmatmul_gate_up: output dtype %d", yt);
    if (m < 0) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_qmatmul_gate_up: m=%lld is negative", (long long)m);
    if (ldy < gate->n) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_qmatmul_gate_up: ldy=%lld is smaller than n=%lld", (long long)ldy, (long long)gate->n);
    const int64_t n = gate->n;
    const turq_weight *ws[2] = {gate, up};
    const float *biases[2] = {bias_gate, bias_up};
    const int64_t ldys[2] = {n, n};
    if (mem == TURQ_MEM_HOST) {
        // the two products through the host path, the expression on the host (the remaining argument checks are turq_qmatmul's)
        std::vector<float> prod;
        try { prod.resize((size_t)(2 * m * n)); } catch (...) { return turq_fail(ctx, TURQ_ERR_OOM, "turq_qmatmul_gate_up: host scratch"); }
        for (int i = 0; i < 2; i++) {
            const int rc = turq_qmatmul(ctx, ws[i], x, xt, m, ldx, prod.data() + (size_t)i * m * n, TURQ_ACT_F32, n, biases[i], mem, TURQ_ALGO_AUTO);
            if (rc != TURQ_OK) return rc;
        }
        if (m == 0 || n == 0) return TURQ_OK;
        if (!y) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul_gate_up: null output pointer");
        for (int64_t r = 0; r < m; r++)
            for (int64_t c = 0; c < n; c++) {
                const float g = prod[(size_t)(r * n + c)], u = prod[(size_t)((m + r) * n + c)];
                const float out = g / (1.0f + expf(-g)) * u;
                const size_t at = (size_t)(r * ldy + c);
                if (yt == TURQ_ACT_F32) ((float *)y)[at] = out;
                else if (yt == TURQ_ACT_BF16) ((uint16_t *)y)[at] = host_bf16(out);
                else {
                    const _Float16 h = (_Float16)out;
                    memcpy((uint16_t *)y + at, &h, 2);
                }
            }
        return TURQ_OK;
    }
    if (m > 0 && n > 0 && x && y && gate->device == ctx->device && up->device == ctx->device && gate->k > 0 && ldx >= gate->k &&
        turq_act_bytes(xt) && !(ctx->wide && xt != TURQ_ACT_F16)) {
        bool taken = false;
        const int rc = turq_qmatmul_gate_up_mfma(ctx, gate, up, x, xt, m, ldx, y, yt, ldy, bias_gate, bias_up, &taken);
        if (rc != TURQ_OK || taken) return rc;
    }
    // general path: both products as f32 into scratch (one call, so they share a launch or an activation preparation where
    // turq_qmatmul_multi does that), then one elementwise pass
    const size_t half = (size_t)(m > 0 ? m : 0) * (size_t)n;
    int rc = turq_ctx_reserve(ctx, &ctx->gate_up, &ctx->gate_up_cap, 2 * half * sizeof(float) + 16);
    if (rc != TURQ_OK) return rc;
    void *ys[2] = {ctx->gate_up, (float *)ctx->gate_up + half};
    rc = turq_qmatmul_multi(ctx, 2, ws, x, xt, m, ldx, ys, TURQ_ACT_F32, ldys, biases, mem, TURQ_ALGO_AUTO);
    if (rc != TURQ_OK) return rc;
    if (m == 0 || n == 0) return TURQ_OK;
    if (!y) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul_gate_up: null output pointer");
    TURQ_HIP(ctx, turq_launch_silu_mul((const float *)ys[0], (const float *)ys[1], m, n, y, yt, ldy, ctx->stream));
    return TURQ_OK;
}

static int mlp_check(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const turq_weight *down, int64_t m, int yt, int act, int mem) {
    if (!gate || !up || !down) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_mlp: null weight");
    if (act != TURQ_ACTFN_SILU) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_mlp: activation %d is not supported", act);
    if (gate->n != up->n || gate->k != up->k)
        return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_mlp: gate is [%lld, %lld], up is [%lld, %lld]", (long long)gate->n, (long long)gate->k,
                         (long long)up->n, (long long)up->k);
    if (down->k != gate->n)
        return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_mlp: down takes %lld columns, gate and up give %lld", (long long)down->k, (long long)gate->n);
    if (mem != TURQ_MEM_DEVICE && mem != TURQ_MEM_HOST) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_mlp: bad mem %d", mem);
    if (!turq_yt_ok(yt, true)) return turq_fail(ctx, TURQ_ERR_DTYPE, "turq_mlp: output dtype %d", yt);
    if (m < 0) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_mlp: m=%lld is negative", (long long)m);
    return TURQ_OK;
}

static int impl_mlp(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const turq_weight *down, const void *x, int xt, int64_t m,
                    int64_t ldx, void *y, int yt, int64_t ldy, const float *bias_gate, const float *bias_up, const float *bias_down, int act,
                    int mem) {
    TURQ_ENTER(ctx);
    {
        const int rc = mlp_check(ctx, gate, up, down, m, yt, act, mem);
        if (rc != TURQ_OK) return rc;
    }
    const int64_t n_ff = gate->n;
    const size_t h_elems = (size_t)m * (size_t)n_ff;
    if (mem == TURQ_MEM_HOST) {
        std::vector<float> h;
        try { h.resize(h_elems ? h_elems : 1); } catch (...) { return turq_fail(ctx, TURQ_ERR_OOM, "turq_mlp: host scratch"); }
        int rc = impl_qmatmul_gate_up(ctx, gate, up, x, xt, m, ldx, h.data(), TURQ_ACT_F32, n_ff, bias_gate, bias_up, act, mem);
        if (rc != TURQ_OK) return rc;
        return impl_qmatmul(ctx, down, h.data(), TURQ_ACT_F32, m, n_ff, y, yt, ldy, bias_down, mem, TURQ_ALGO_AUTO);
    }
    // The MFMA kernels round their activations to f16 first thing, so where down_proj goes through them the intermediate is
    // kept as f16 to begin with: the same values reach the same multiplications, and the rows that every compute unit reads
    // for down_proj are half as long.  (Not with wide activations, which scale f32 rows before that rounding, and not for a
    // dense or native-layout down_proj, which multiplies in f32.)
    if (m > TURQ_GEMV_MAX_M && !ctx->wide && x && y && turq_dt_is_quant(gate->dtype) && turq_dt_is_quant(up->dtype) && turq_dt_is_quant(down->dtype)) {
        // a prompt chunk: the two products, one kernel from them to down_proj's fragments, down_proj's GEMM
        bool taken = false;
        const int rc = turq_mlp_prefill(ctx, gate, up, down, x, xt, m, ldx, y, yt, ldy, bias_gate, bias_up, bias_down, &taken);
        if (rc != TURQ_OK || taken) return rc;
    }
    const bool h16 = !ctx->wide && turq_dt_is_quant(down->dtype) && down->layout == TURQ_LAYOUT_TILED && n_ff % 8 == 0;
    const int ht = h16 ? TURQ_ACT_F16 : TURQ_ACT_F32;
    int rc = turq_ctx_reserve(ctx, &ctx->mlp_h, &ctx->mlp_h_cap, h_elems * (h16 ? sizeof(uint16_t) : sizeof(float)) + 16);
    if (rc != TURQ_OK) return rc;
    rc = impl_qmatmul_gate_up(ctx, gate, up, x, xt, m, ldx, ctx->mlp_h, ht, n_ff, bias_gate, bias_up, act, mem);
    if (rc != TURQ_OK) return rc;
    return impl_qmatmul(ctx, down, ctx->mlp_h, ht, m, n_ff, y, yt, ldy, bias_down, mem, TURQ_ALGO_AUTO);
}

// ---- RmsNorm taken into the forward calls ----

// the normalised rows in scratch memory of the context, for the calls whose kernels do not apply the norm themselves: f16 where
// the matmul kernels would round them to f16 first thing (the same values, half the bytes), f32 with wide activations
static int norm_to_scratch(turq_ctx *ctx, const void *x, int xt, int64_t m, int64_t k, int64_t ldx, const float *nw, float eps, int *ht) {
    *ht = ctx->wide ? TURQ_ACT_F32 : TURQ_ACT_F16;
    int rc = turq_ctx_reserve(ctx, &ctx->norm_x, &ctx->norm_x_cap, (size_t)m * (size_t)k * (size_t)turq_act_bytes(*ht) + 16);
    if (rc != TURQ_OK) return rc;
    TURQ_HIP(ctx, turq_launch_rms_norm(x, xt, m, k, ldx, nw, eps, ctx->norm_x, *ht, k, ctx->stream));
    return TURQ_OK;
}

static int norm_args(turq_ctx *ctx, const char *fn, const void *x, int xt, int64_t m, int64_t k, int64_t ldx, const float *nw) {
    if ((xt & ~0xFF) || !turq_act_bytes(xt)) return turq_fail(ctx, TURQ_ERR_DTYPE, "%s: unsupported activation dtype %d", fn, xt);
    if (m < 0) return turq_fail(ctx, TURQ_ERR_SHAPE, "%s: m=%lld is negative", fn, (long long)m);
    if (ldx < k) return turq_fail(ctx, TURQ_ERR_SHAPE, "%s: ldx=%lld is smaller than k=%lld", fn, (long long)ldx, (long long)k);
    if (m > 0 && k > 0 && (!x || !nw)) return turq_fail(ctx, TURQ_ERR_INVALID, "%s: null activation or norm weight pointer", fn);
    return TURQ_OK;
}

static int impl_norm_qmatmul_multi(turq_ctx *ctx, int count, const turq_weight *const *weights, const void *x, int xt, int64_t m, int64_t ldx,
                                   const float *nw, float eps, void *const *ys, int yt, const int64_t *ldys, const float *const *biases,
                                   int mem) {
    TURQ_ENTER(ctx);
    if (count < 0) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_norm_qmatmul_multi: count=%d is negative", count);
    if (count == 0) return TURQ_OK;
    if (!weights || !ys || !ldys || !weights[0]) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_norm_qmatmul_multi: null weight, output or stride array");
    if (mem != TURQ_MEM_DEVICE && mem != TURQ_MEM_HOST) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_norm_qmatmul_multi: bad mem %d", mem);
    const int64_t k = weights[0]->k;
    int rc = norm_args(ctx, "turq_norm_qmatmul_multi", x, xt, m, k, ldx, nw);
    if (rc != TURQ_OK) return rc;
    if (m == 0 || k == 0) return impl_qmatmul_multi(ctx, count, weights, x, xt, m, ldx, ys, yt, ldys, biases, mem, TURQ_ALGO_AUTO);
    if (mem == TURQ_MEM_HOST) {
        std::vector<float> xn;
        try { xn.resize((size_t)m * (size_t)k); } catch (...) { return turq_fail(ctx, TURQ_ERR_OOM, "turq_norm_qmatmul_multi: host scratch"); }
        rc = impl_rms_norm(ctx, x, xt, m, k, ldx, nw, eps, xn.data(), TURQ_ACT_F32, k, mem);
        if (rc != TURQ_OK) return rc;
        return impl_qmatmul_multi(ctx, count, weights, xn.data(), TURQ_ACT_F32, m, k, ys, yt, ldys, biases, mem, TURQ_ALGO_AUTO);
    }
    bool plain = !(yt & ~0xFF) && turq_act_bytes(yt) && count <= 16;
    for (int i = 0; i < count && plain; i++) plain = weights[i] && ys[i] && ldys[i] >= weights[i]->n;
    if (plain && turq_norm_fuses(ctx, count, weights, x, xt, ldx, m)) {
        const TurqNorm nm{nw, eps};
        if (m == 1) return turq_qmatmul_multi_mfma(ctx, count, weights, x, xt, m, ldx, ys, yt, ldys, biases, &nm);
        bool taken = false;
        rc = turq_qmatmul_multi_gemm(ctx, count, weights, x, xt, m, ldx, ys, yt, ldys, biases, &taken, &nm);
        if (rc != TURQ_OK || taken) return rc;
    }
    int ht = TURQ_ACT_F16;
    rc = norm_to_scratch(ctx, x, xt, m, k, ldx, nw, eps, &ht);
    if (rc != TURQ_OK) return rc;
    return impl_qmatmul_multi(ctx, count, weights, ctx->norm_x, ht, m, k, ys, yt, ldys, biases, mem, TURQ_ALGO_AUTO);
}

static int impl_norm_mlp(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const turq_weight *down, const void *x, int xt, int64_t m,
                         int64_t ldx, const float *nw, float eps, void *y, int yt, int64_t ldy, const float *bias_gate, const float *bias_up,
                         const float *bias_down, int act, int mem) {
    TURQ_ENTER(ctx);
    int rc = mlp_check(ctx, gate, up, down, m, yt, act, mem);
    if (rc != TURQ_OK) return rc;
    const int64_t k = gate->k, n_ff = gate->n;
    rc = norm_args(ctx, "turq_norm_mlp", x, xt, m, k, ldx, nw);
    if (rc != TURQ_OK) return rc;
    if (m == 0 || k == 0) return impl_mlp(ctx, gate, up, down, x, xt, m, ldx, y, yt, ldy, bias_gate, bias_up, bias_down, act, mem);
    if (mem == TURQ_MEM_HOST) {
        std::vector<float> xn;
        try { xn.resize((size_t)m * (size_t)k); } catch (...) { return turq_fail(ctx, TURQ_ERR_OOM, "turq_norm_mlp: host scratch"); }
        rc = impl_rms_norm(ctx, x, xt, m, k, ldx, nw, eps, xn.data(), TURQ_ACT_F32, k, mem);
        if (rc != TURQ_OK) return rc;
        return impl_mlp(ctx, gate, up, down, xn.data(), TURQ_ACT_F32, m, k, y, yt, ldy, bias_gate, bias_up, bias_down, act, mem);
    }
    const turq_weight *gu[2] = {gate, up};
    if (y && ldy >= down->n && turq_norm_fuses(ctx, 2, gu, x, xt, ldx, m)) {
        const TurqNorm nm{nw, eps};
        bool taken = false;
        if (m == 1 && gate->dtype == up->dtype) {
            // as turq_mlp's one-row route: the f16 intermediate where down_proj rounds its input to f16 anyway
            const bool h16 = turq_dt_is_quant(down->dtype) && down->layout == TURQ_LAYOUT_TILED && n_ff % 8 == 0;
            const int ht = h16 ? TURQ_ACT_F16 : TURQ_ACT_F32;
            rc = turq_ctx_reserve(ctx, &ctx->mlp_h, &ctx->mlp_h_cap, (size_t)m * (size_t)n_ff * (h16 ? sizeof(uint16_t) : sizeof(float)) + 16);
            if (rc != TURQ_OK) return rc;
            rc = turq_qmatmul_gate_up_mfma(ctx, gate, up, x, xt, m, ldx, ctx->mlp_h, ht, n_ff, bias_gate, bias_up, &taken, &nm);
            if (rc != TURQ_OK) return rc;
            if (taken) return impl_qmatmul(ctx, down, ctx->mlp_h, ht, m, n_ff, y, yt, ldy, bias_down, mem, TURQ_ALGO_AUTO);
        } else if (m > TURQ_GEMV_MAX_M) {
            rc = turq_mlp_prefill(ctx, gate, up, down, x, xt, m, ldx, y, yt, ldy, bias_gate, bias_up, bias_down, &taken, &nm);
            if (rc != TURQ_OK || taken) return rc;
        }
    }
    int ht = TURQ_ACT_F16;
    rc = norm_to_scratch(ctx, x, xt, m, k, ldx, nw, eps, &ht);
    if (rc != TURQ_OK) return rc;
    return impl_mlp(ctx, gate, up, down, ctx->norm_x, ht, m, k, y, yt, ldy, bias_gate, bias_up, bias_down, act, mem);
}

// ---- graphs and kernel timing ----

int turq_graph_begin(turq_ctx *ctx) {
    TURQ_ENTER(ctx);
    if (ctx->capturing) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_graph_begin: a capture is already running");
    if (ctx->profiling) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_graph_begin: kernel timing is on; events cannot be captured");
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->pf_stream));  // eager prefetch work stays outside the capture
    TURQ_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    ctx->pf_in_capture = false;
    return TURQ_OK;
}

int turq_graph_end(turq_ctx *ctx, turq_graph **out) {
    TURQ_ENTER(ctx);
    if (!out) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_graph_end: null out pointer");
    *out = nullptr;
    if (!ctx->capturing)
        return turq_fail(ctx, TURQ_ERR_INVALID, "turq_graph_end: no capture is running (a call that fails inside a capture ends and discards it)");
    hipError_t e = hipSuccess;
    if (ctx->pf_in_capture) {  // the prefetch branch joins the captured stream, or the capture could not end
        e = hipEventRecord(ctx->ev_pf_join, ctx->pf_stream);
        if (e == hipSuccess) e = hipStreamWaitEvent(ctx->stream, ctx->ev_pf_join, 0);
        ctx->pf_in_capture = false;
    }
    ctx->capturing = false;
    std::unique_ptr<turq_graph> g(new (std::nothrow) turq_graph);
    hipGraph_t graph = nullptr;
    const hipError_t e_end = hipStreamEndCapture(ctx->stream, &graph);
    if (e == hipSuccess) e = e_end;
    if (e != hipSuccess || !g) {
        if (graph) (void)hipGraphDestroy(graph);
        return turq_fail(ctx, g ? TURQ_ERR_HIP : TURQ_ERR_OOM, "hipStreamEndCapture failed: %s", hipGetErrorString(e));
    }
    g->graph = graph;
    g->device = ctx->device;
    e = hipGraphInstantiate(&g->exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        return turq_fail(ctx, TURQ_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    }
    // from here on the graph refers to the context's scratch buffers by address (see turq_ctx_reserve)
    g->tally = ctx->tally;
    g->tally->live.fetch_add(1, std::memory_order_acq_rel);
    *out = g.release();
    return TURQ_OK;
}

int turq_graph_launch(turq_ctx *ctx, turq_graph *g) {
    TURQ_ENTER(ctx);
    if (!g || !g->exec) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_graph_launch: null graph");
    if (g->device != ctx->device) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_graph_launch: graph was captured on device %d", g->device);
    TURQ_HIP(ctx, hipGraphLaunch(g->exec, ctx->stream));
    return TURQ_OK;
}

void turq_graph_destroy(turq_graph *g) {
    if (!g) return;
    DeviceGuard guard(g->device);
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    if (g->tally) g->tally->live.fetch_sub(1, std::memory_order_acq_rel);
    delete g;
}

static int impl_weight_prefetch(turq_ctx *ctx, const turq_weight *w) {
    TURQ_ENTER(ctx);
    if (!w) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_weight_prefetch: null weight");
    if (w->device != ctx->device) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_weight_prefetch: weight lives on device %d, context on %d", w->device, ctx->device);
    if (!w->dev || w->dev_bytes < 4096) return TURQ_OK;
    // starts where the context's stream stands now, i.e. next to whatever is queued on it after this call
    TURQ_HIP(ctx, hipEventRecord(ctx->ev_pf_fork, ctx->stream));
    TURQ_HIP(ctx, hipStreamWaitEvent(ctx->pf_stream, ctx->ev_pf_fork, 0));
    if (ctx->capturing) ctx->pf_in_capture = true;
    TURQ_HIP(ctx, turq_launch_weight_prefetch(w->dev, w->dev_bytes, ctx->pf_workgroups, ctx->pf_depth, ctx->pf_stream, nullptr, nullptr));
    return TURQ_OK;
}

int turq_read_yardstick(turq_ctx *ctx, const void *dev_ptr, size_t nbytes) {
    TURQ_ENTER(ctx);
    if (!dev_ptr && nbytes) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_read_yardstick: null pointer");
    if ((uintptr_t)dev_ptr % 16) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_read_yardstick: the pointer must be 16-byte aligned");
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
    TURQ_HIP(ctx, turq_launch_read_yardstick(dev_ptr, nbytes, ctx->compute_units > 0 ? ctx->compute_units : 256, ctx->stream, ev0, ev1));
    return TURQ_OK;
}

int turq_profile_begin(turq_ctx *ctx) {
    TURQ_ENTER(ctx);
    if (ctx->capturing) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_profile_begin: a graph capture is running");
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    ctx->profiling = true;
    ctx->prof_used = 0;
    return TURQ_OK;
}

int turq_profile_end(turq_ctx *ctx, int64_t *launches, double *total_ms) {
    TURQ_ENTER(ctx);
    if (!ctx->profiling) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_profile_end: timing was not started");
    ctx->profiling = false;
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    double sum = 0.0;
    for (size_t i = 0; i < ctx->prof_used; i++) {
        float ms = 0.0f;
        TURQ_HIP(ctx, hipEventElapsedTime(&ms, ctx->prof_events[i].first, ctx->prof_events[i].second));
        sum += ms;
    }
    if (launches) *launches = (int64_t)ctx->prof_used;
    if (total_ms) *total_ms = sum;
    ctx->prof_used = 0;
    return TURQ_OK;
}

// ---- activation quantisation ----

static int quantize_common(turq_ctx *ctx, const float *x, int64_t m, int64_t k, void *out, int mem, bool q8k) {
    const int be = q8k ? 256 : 32, bb = q8k ? 292 : 34;
    if (m < 0 || k < 0) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_quantize: negative shape");
    if (k % be) return turq_fail(ctx, TURQ_ERR_SHAPE, "turq_quantize: k=%lld is not a multiple of %d", (long long)k, be);
    const int64_t nblocks = m * (k / be);
    if (nblocks == 0) return TURQ_OK;
    if (!x || !out) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_quantize: null pointer");
    const size_t in_bytes = (size_t)m * (size_t)k * 4, out_bytes = (size_t)nblocks * bb;
    const float *dx = x;
    void *dout = out;
    if (mem == TURQ_MEM_HOST) {
        int rc = turq_ctx_reserve(ctx, &ctx->stage_x, &ctx->stage_x_cap, in_bytes);
        if (rc != TURQ_OK) return rc;
        rc = turq_ctx_reserve(ctx, &ctx->stage_y, &ctx->stage_y_cap, out_bytes);
        if (rc != TURQ_OK) return rc;
        TURQ_HIP(ctx, hipMemcpyAsync(ctx->stage_x, x, in_bytes, hipMemcpyHostToDevice, ctx->stream));
        dx = (const float *)ctx->stage_x;
        dout = ctx->stage_y;
    } else if (mem != TURQ_MEM_DEVICE) {
        return turq_fail(ctx, TURQ_ERR_INVALID, "turq_quantize: bad mem %d", mem);
    }
    if (q8k) TURQ_HIP(ctx, turq_launch_quantize_q8_k(dx, nblocks, dout, ctx->stream));
    else TURQ_HIP(ctx, turq_launch_quantize_q8_0(dx, nblocks, dout, ctx->stream));
    if (mem == TURQ_MEM_HOST) {
        TURQ_HIP(ctx, hipMemcpyAsync(out, dout, out_bytes, hipMemcpyDeviceToHost, ctx->stream));
        TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    }
    return TURQ_OK;
}

static int impl_quantize_q8_0(turq_ctx *ctx, const float *x, int64_t m, int64_t k, void *out, int mem) {
    TURQ_ENTER(ctx);
    return quantize_common(ctx, x, m, k, out, mem, false);
}

static int impl_quantize_q8_k(turq_ctx *ctx, const float *x, int64_t m, int64_t k, void *out, int mem) {
    TURQ_ENTER(ctx);
    return quantize_common(ctx, x, m, k, out, mem, true);
}


// ---- the entry points a graph capture may hold ----
// A call that fails while the context's stream is capturing ends the capture and discards what was recorded, so that the stream
// and the context are usable again (turq_graph_end then reports that no capture is running).
}  // extern "C"
int turq_capture_guard(turq_ctx *ctx, int rc) {
    if (rc != TURQ_OK && ctx && ctx->capturing) {
        hipGraph_t dead = nullptr;
        (void)hipStreamEndCapture(ctx->stream, &dead);
        if (dead) (void)hipGraphDestroy(dead);
        (void)hipGetLastError();  // ending an invalidated capture reports an error of its own
        ctx->capturing = false;
        ctx->err += " (the graph capture in progress was ended and discarded)";
    }
    return rc;
}
extern "C" {

int turq_dequantize(turq_ctx *ctx, const turq_weight *w, float *out, int out_mem) {
    return turq_capture_guard(ctx, impl_dequantize(ctx, w, out, out_mem));
}
int turq_embedding_lookup(turq_ctx *ctx, const turq_weight *w, const uint32_t *ids, int64_t count, void *out, int out_dtype,
                          int64_t ldo, int mem) {
    return turq_capture_guard(ctx, impl_embedding_lookup(ctx, w, ids, count, out, out_dtype, ldo, mem));
}
int turq_qmatmul(turq_ctx *ctx, const turq_weight *w, const void *x, int xt, int64_t m, int64_t ldx, void *y, int yt,
                 int64_t ldy, const float *bias, int mem, int algo) {
    return turq_capture_guard(ctx, impl_qmatmul(ctx, w, x, xt, m, ldx, y, yt, ldy, bias, mem, algo));
}
int turq_qmatmul_multi(turq_ctx *ctx, int count, const turq_weight *const *weights, const void *x, int xt, int64_t m,
                       int64_t ldx, void *const *ys, int yt, const int64_t *ldys, const float *const *biases, int mem, int algo) {
    return turq_capture_guard(ctx, impl_qmatmul_multi(ctx, count, weights, x, xt, m, ldx, ys, yt, ldys, biases, mem, algo));
}
int turq_qmatmul_gate_up(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const void *x, int xt, int64_t m, int64_t ldx,
                         void *y, int yt, int64_t ldy, const float *bias_gate, const float *bias_up, int act, int mem) {
    return turq_capture_guard(ctx, impl_qmatmul_gate_up(ctx, gate, up, x, xt, m, ldx, y, yt, ldy, bias_gate, bias_up, act, mem));
}
int turq_mlp(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const turq_weight *down, const void *x, int xt, int64_t m,
             int64_t ldx, void *y, int yt, int64_t ldy, const float *bias_gate, const float *bias_up, const float *bias_down, int act, int mem) {
    return turq_capture_guard(ctx, impl_mlp(ctx, gate, up, down, x, xt, m, ldx, y, yt, ldy, bias_gate, bias_up, bias_down, act, mem));
}
int turq_norm_qmatmul_multi(turq_ctx *ctx, int count, const turq_weight *const *weights, const void *x, int xt, int64_t m, int64_t ldx,
                            const float *norm_weight, float eps, void *const *ys, int yt, const int64_t *ldys, const float *const *biases,
                            int mem) {
    return turq_capture_guard(ctx, impl_norm_qmatmul_multi(ctx, count, weights, x, xt, m, ldx, norm_weight, eps, ys, yt, ldys, biases, mem));
}
int turq_norm_mlp(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const turq_weight *down, const void *x, int xt, int64_t m,
                  int64_t ldx, const float *norm_weight, float eps, void *y, int yt, int64_t ldy, const float *bias_gate, const float *bias_up,
                  const float *bias_down, int act, int mem) {
    return turq_capture_guard(ctx, impl_norm_mlp(ctx, gate, up, down, x, xt, m, ldx, norm_weight, eps, y, yt, ldy, bias_gate, bias_up, bias_down, act, mem));
}
int turq_quantize_q8_0(turq_ctx *ctx, const float *x, int64_t m, int64_t k, void *out, int mem) {
    return turq_capture_guard(ctx, impl_quantize_q8_0(ctx, x, m, k, out, mem));
}
int turq_quantize_q8_k(turq_ctx *ctx, const float *x, int64_t m, int64_t k, void *out, int mem) {
    return turq_capture_guard(ctx, impl_quantize_q8_k(ctx, x, m, k, out, mem));
}

int turq_weight_prefetch(turq_ctx *ctx, const turq_weight *w) { return turq_capture_guard(ctx, impl_weight_prefetch(ctx, w)); }

int turq_rms_norm(turq_ctx *ctx, const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, const float *weight, float eps, void *y,
                  int y_dtype, int64_t ldy, int mem) {
    return turq_capture_guard(ctx, impl_rms_norm(ctx, x, x_dtype, m, k, ldx, weight, eps, y, y_dtype, ldy, mem));
}

int turq_ctx_set_wide_activations(turq_ctx *ctx, int on) {
    if (!ctx) return turq_fail(nullptr, TURQ_ERR_INVALID, "turq_ctx_set_wide_activations: null context");
    if (ctx->capturing) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_ctx_set_wide_activations: a graph capture is running");
    ctx->wide = on != 0;
    return TURQ_OK;
}

int turq_ctx_nonfinite_count(turq_ctx *ctx, uint64_t *count, int reset) {
    TURQ_ENTER(ctx);
    if (ctx->capturing) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_ctx_nonfinite_count: a graph capture is running");
    TURQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    unsigned long long sum = 0;
#define TURQ_READ_NONFINITE(fn) TURQ_HIP(ctx, fn(&sum, reset));
    TURQ_NONFINITE_UNITS(TURQ_READ_NONFINITE)
#undef TURQ_READ_NONFINITE
    if (count) *count = (uint64_t)sum;
    return TURQ_OK;
}

int turq_ctx_scratch_info(const turq_ctx *ctx, int *live_graphs, int *retired_buffers, size_t *act_prep_bytes) {
    if (!ctx) return turq_fail(nullptr, TURQ_ERR_INVALID, "turq_ctx_scratch_info: null context");
    if (live_graphs) *live_graphs = ctx->tally ? ctx->tally->live.load(std::memory_order_acquire) : 0;
    if (retired_buffers) *retired_buffers = (int)ctx->retired.size();
    if (act_prep_bytes) *act_prep_bytes = ctx->act_prep_cap;
    return TURQ_OK;
}

}  // extern "C"

// Host side of the MFMA paths: prepare the activations, pick the launch shape, launch.
#include <algorithm>
#include <cstdlib>

#include "layout.h"
#include "mfma_common.h"

namespace {

// Waves per workgroup (= how many ways a row tile's columns are split).  Enough waves to cover the
// machine a few times over, never more than there are column tiles.
int pick_waves(const turq_ctx *ctx, int64_t n, int64_t k) {
    const int forced = turq_tuning().gemv_waves;
    if (forced >= 1 && forced <= 16) return (int)std::min<int64_t>(forced, turq_tile_cols(k));
    const int64_t row_tiles = turq_tile_rows(n);
    const int64_t col_tiles = turq_tile_cols(k);
    const int64_t want_waves = (int64_t)(ctx->compute_units > 0 ? ctx->compute_units : 256) * 12;
    int64_t w = (want_waves + row_tiles - 1) / row_tiles;
    w = std::max<int64_t>(1, std::min<int64_t>({w, col_tiles, 16}));
    return (int)w;
}

// The skinny kernel can convert up to TURQ_GEMV_FUSED_MAX_M activation rows itself (no preparation launch), but every wave
// then converts its own column tiles again for every row tile; measured, that pays for one row, and for two rows unless
// the matrix is large enough for the two-row-tile form of the prepared path (LM head).
// A matrix of a few MB is bound by the launch itself: there the extra preparation launch costs more than it saves.
bool use_fused(const turq_ctx *ctx, int64_t m, int64_t row_tiles, size_t weight_bytes) {
    const int64_t cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
    if (m > TURQ_GEMV_FUSED_MAX_M) return false;
    return m == 1 || weight_bytes < (8u << 20) || (m == 2 && row_tiles < 4 * cus);
}

// one activation row, formats the sub-block-row kernel covers (TURQ_GEMV_NO_ROW1 keeps the general kernel, for comparison)
bool use_row1(int dtype) {
    return !turq_tuning().gemv_no_row1 && turq_gemv_row1_supports(dtype);
}

// The one-row kernel stages the raw activations itself, once per wave and column tile, and needs no preparation launch.
// One activation row: always.  Two rows: where the weights of the call are large enough for its launch to beat the fused
// general kernel (+ 5 .. 12 % at 28 MB and more, - 10 % at 3 MB).  Three and four rows (formats whose kernel packs pairs of
// rows): the 16 MFMAs and LDS operand reads per tile then cost as much as the tile's bytes, so only up to a size where the
// general kernel's preparation launch and its tail still weigh more (Q4_K: + 6 .. 40 % up to 57 MB, - 4 % at 75 MB,
// - 19 % at 350 MB; Q5_K: + 7 % at 92 MB, - 12 % at 430 MB).  TURQ_ROW1_M lowers the row limit, for comparison.
bool row1_takes(int64_t m, size_t weight_bytes, int dtype) {
    const int most = std::min(std::max(turq_tuning().row1_m, 1), TURQ_ROW1_MAX_M);
    const size_t least = (size_t)8 << 20;  // below: the general kernel is level or up to 10 % ahead, for any number of rows
    if (m == 1) return true;
    if (m > most || m > turq_gemv_row1_rows(dtype) || weight_bytes < least) return false;
    if (m <= 2) return true;
    return weight_bytes <= ((size_t)(dtype == TURQ_Q4_K ? 64 : 128) << 20);
}

// Waves per workgroup of the one-row kernel: it is light on registers and on vector work, so what it wants is many waves
// with few column tiles each (two by default), up to the largest workgroup.
int pick_waves_row1(int64_t k) {
    const int forced = turq_tuning().gemv_waves;
    const int tpw_env = std::max(turq_tuning().row1_tpw, 0);
    const int64_t col_tiles = turq_tile_cols(k);
    // (up to four column tiles, K <= 1024: one per wave; the 3072 x 1024 Q8_0 matrix gains 5 %)
    const int tpw = tpw_env ? tpw_env : (col_tiles <= 4 ? 1 : 2);
    if (forced >= 1 && forced <= 16) return (int)std::min<int64_t>(forced, col_tiles);
    return (int)std::max<int64_t>(1, std::min<int64_t>((col_tiles + tpw - 1) / tpw, 16));
}

// Row tiles per workgroup of the one-row kernel (TURQ_ROW1_R forces it).
int pick_rows_row1(const turq_ctx *ctx, int64_t row_tiles) {
    const int forced = turq_tuning().row1_r;
    if (forced == 1 || forced == 2) return forced;
    // two row tiles share the staged activations where there are row tiles to spare (the LM head: + 10 %)
    const int64_t cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
    return row_tiles >= 16 * cus ? 2 : 1;
}

// Row tiles per workgroup of the kernel that keeps a column tile's activation fragments in registers and streams the row tiles
// past them (gemv_cs.hip), or 0 where it does not apply.  It needs no preparation launch and reads the activations once per
// workgroup, but runs one eight-wave workgroup per compute unit: measured against preparation + prepared-fragment kernel it
// wins where the launch is one to two such workgroups per unit (gate + up of an MLP: 5 .. 15 % for 5 <= m <= 16, Q4_K and Q6_K)
// and loses where there are many (the LM head: - 12 .. - 30 %) or 32 rows (registers).  TURQ_CS = 0 switches it off,
// TURQ_CS_RG forces the group size (2, 3 or 6).
int cs_row_tiles(const turq_ctx *ctx, int64_t m, int64_t row_tiles, int dtype, bool aligned) {
    const int mode = turq_tuning().cs, forced = turq_tuning().cs_rg;
    if (mode == 0 || !aligned || m < 2 || m > TURQ_GEMV_MAX_M) return 0;
    const int64_t cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
    int rg = (m <= 16 && dtype != TURQ_Q8_0 && row_tiles >= 6 * cus && row_tiles <= 12 * cus) ? 6 : 0;
    if (forced && turq_gemv_cs_rows_ok(forced)) {
        rg = forced;
        // instantiations that do not fit the register file
        if (rg == 6 && (m > 16 || dtype == TURQ_Q8_0)) rg = 3;
        if (rg == 3 && dtype == TURQ_Q8_0 && m > 16) rg = 2;
    }
    return rg;
}

// The staged form of that kernel (activation rows loaded as they lie in memory and turned into fragments through the LDS) also
// pays for small launches, where it replaces a preparation launch and a kernel that re-reads prepared fragments: row tiles per
// workgroup so that the launch is about one workgroup per compute unit.  0: not this call.  TURQ_CS_STAGED = 0 switches it off,
// TURQ_CS_RG forces the group size.
int staged_row_tiles(const turq_ctx *ctx, int dtype_a, int dtype_b, int64_t k, int64_t m, int64_t row_tiles, int64_t row_tiles_b,
                     bool aligned) {
    const TurqTuning &tune = turq_tuning();
    const int mode = tune.cs_staged, forced = tune.cs_rg, min_m = tune.cs_staged_min_m, max_m = tune.cs_staged_max_m;
    if (mode == 0 || !aligned || m < min_m || m > max_m || m > TURQ_GEMV_MAX_M) return 0;
    const int64_t cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
    if (row_tiles > 12 * cus && !forced) return 0;  // many rounds of workgroups (an LM head): the prepared fragments do better
    // the smallest group with which the launch is one round of workgroups (the weights of a second format go out in smaller
    // groups); beyond three row tiles per unit, two rounds of 2 or 3 or groups of 6
    const int64_t per = (row_tiles + cus - 1) / cus;
    int rg = per == 4 ? 2 : per == 5 ? 3 : 6;
    for (int g = 3; g >= 1; g--) {
        const int gb = turq_gemv_cs_staged_second_rows(g);
        if ((row_tiles - row_tiles_b + g - 1) / g + (row_tiles_b + gb - 1) / gb <= cus) rg = g;
    }
    // more than 16 rows: on weights of up to 4096 columns (beyond, the f32 rows that every unit reads outweigh the preparation
    // launch); up to two row tiles per unit as two passes of 16 rows, more in the four-wave form with groups of six
    if (m > 16 && !forced) {
        if (k > 4096) return 0;
        if (row_tiles > 2 * cus) rg = 6;  // the four-wave form
    }
    if (forced) rg = forced;
    while (rg > 1 && !turq_gemv_cs_staged_takes(dtype_a, dtype_b, k, m, rg)) rg = rg == 6 ? 3 : rg - 1;
    return turq_gemv_cs_staged_takes(dtype_a, dtype_b, k, m, rg) ? rg : 0;
}

// whether the prefill GEMM can take this weight (its largest packed value must fit f16), and the power of two by which the
// kernel multiplies the block scales
bool gemm_takes(const turq_weight *w, float *wscale) {
    const float top = w->dtype == TURQ_Q4_K ? 1039.0f : w->dtype == TURQ_Q5_K ? 1055.0f : w->dtype == TURQ_Q6_K ? 319.0f : 128.0f;
    const bool ok = turq_dt_is_quant(w->dtype) && w->k % 256 == 0 && w->max_scale * top < 60000.0f;
    float ws = 1.0f;
    if (ok && w->max_scale > 0.0f)
        while (ws < 32768.0f && w->max_scale * top * ws * 2.0f < 40000.0f) ws *= 2.0f;
    *wscale = ws;
    return ok;
}

}  // namespace

// More than 32 rows, several weights that take the same activations: the fragments are prepared once per fragment order
// (K-quants / Q8_0) and every weight runs its GEMM on them.  *taken = false (nothing launched) if one of the weights cannot
// go through the GEMM.
// The further streams and their events, made on first use.  Not while a graph is being captured (creating a stream is not a
// call to make in the middle of a capture): the caller then stays on one stream.
static bool side_ready(turq_ctx *ctx) {
    if (ctx->side[0]) return true;
    if (ctx->capturing) return false;
    hipStream_t s[turq_ctx::kSide] = {};
    hipEvent_t j[turq_ctx::kSide] = {}, f = nullptr;
    bool ok = hipEventCreateWithFlags(&f, hipEventDisableTiming) == hipSuccess;
    for (int i = 0; i < turq_ctx::kSide && ok; i++)
        ok = hipStreamCreateWithFlags(&s[i], hipStreamNonBlocking) == hipSuccess &&
             hipEventCreateWithFlags(&j[i], hipEventDisableTiming) == hipSuccess;
    if (!ok) {
        for (int i = 0; i < turq_ctx::kSide; i++) {
            if (j[i]) (void)hipEventDestroy(j[i]);
            if (s[i]) (void)hipStreamDestroy(s[i]);
        }
        if (f) (void)hipEventDestroy(f);
        return false;
    }
    ctx->ev_fork = f;
    for (int i = 0; i < turq_ctx::kSide; i++) { ctx->side[i] = s[i]; ctx->ev_join[i] = j[i]; }
    return true;
}

// Scratch for the prefill GEMM launches of one call that split their columns over several workgroups: launch i gets counter
// block i and its own stretch of partial tiles (launches of one call may run next to each other), counters[i] null where
// launch i does not split or the call may not allocate.  The counter blocks are cleared when the buffer is allocated and
// left at zero by every launch; calls on the context's stream follow each other, so they share the buffer.
struct GemmSplit {
    void *counters[turq_ctx::kSplitSlots] = {};
    void *partials[turq_ctx::kSplitSlots] = {};
    size_t bytes[turq_ctx::kSplitSlots] = {};
};
static int gemm_split_reserve(turq_ctx *ctx, int count, const turq_weight *const *w, int64_t m, GemmSplit *out) {
    *out = GemmSplit{};
    if (ctx->fixed_scratch || count > turq_ctx::kSplitSlots) return TURQ_OK;
    constexpr size_t kCounters = (size_t)turq_ctx::kSplitSlots * TURQ_GEMM_SPLIT_COUNTER_BYTES;
    size_t off[turq_ctx::kSplitSlots], total = kCounters;
    bool any = false;
    for (int i = 0; i < count; i++) {
        out->bytes[i] = turq_gemm_split_scratch(w[i]->dtype, w[i]->n, w[i]->k, m, ctx->compute_units, nullptr, nullptr);
        off[i] = total;
        total += (out->bytes[i] + 255) & ~(size_t)255;
        any = any || out->bytes[i] != 0;
    }
    if (!any) return TURQ_OK;
    if (total > ((size_t)512 << 20)) {  // (a call whose launches together want more than this runs them unsplit)
        *out = GemmSplit{};
        return TURQ_OK;
    }
    if (total > ctx->gemm_split_cap) {
        int rc = turq_ctx_reserve(ctx, &ctx->gemm_split, &ctx->gemm_split_cap, total);
        if (rc != TURQ_OK) return rc;
        TURQ_HIP(ctx, hipMemsetAsync(ctx->gemm_split, 0, kCounters, ctx->stream));  // (never inside a capture: growing is refused there)
    }
    for (int i = 0; i < count; i++) {
        if (out->bytes[i] == 0) continue;
        out->counters[i] = (uint8_t *)ctx->gemm_split + (size_t)i * TURQ_GEMM_SPLIT_COUNTER_BYTES;
        out->partials[i] = (uint8_t *)ctx->gemm_split + off[i];
    }
    return TURQ_OK;
}

// CUs that the GEMM launch for [m, n] takes: its workgroups, by the launcher's choice between the 64-row tile (two of those
// workgroups share a CU) and the 128-row tiles (one per CU; wide tiles counted as two).  Measured on the Q4_K_M layer: launches
// of 192 workgroups next to each other help with the 64-row tile (m = 128: +4.8 %) and hurt with the 128-row tile (m = 256: -2.7 %).
static int64_t gemm_cus_taken_shape(int compute_units, int dtype, int64_t n, int64_t k, int64_t m, bool may_split) {
    int form = 0, split = 1;
    if (may_split && turq_gemm_split_scratch(dtype, n, k, m, compute_units, &form, &split) != 0) {
        const int64_t tiles = form == 4 ? ((n + 127) / 128) * ((m + 63) / 64) : ((n + 255) / 256) * ((m + 127) / 128);
        const bool whole = form != 4 || turq_gemm_low_two_groups(n, k, m, split, compute_units);
        return whole ? tiles * split : (tiles * split + 1) / 2;
    }
    const int64_t nt = (n + 127) / 128, wgs128 = ((m + 127) / 128) * nt;
    const bool low = m <= 64 || 2 * wgs128 <= compute_units;
    if (!low) return wgs128;
    const int64_t tiles = ((m + 63) / 64) * nt;
    return turq_gemm_low_two_groups(n, k, m, 1, compute_units) ? tiles : (tiles + 1) / 2;
}
static int64_t gemm_cus_taken(const turq_ctx *ctx, const turq_weight *w, int64_t m, bool may_split) {
    return gemm_cus_taken_shape(ctx->compute_units, w->dtype, w->n, w->k, m, may_split);
}

// Whether `run` (2 .. 4) neighbouring weights of one K-quant format and one shape [n, k] go out as ONE launch of the prefill
// GEMM over the rows of all of them: each must take more than half of the machine alone, and the launch over all the rows
// must fill its rounds over the CUs better - each alone leaves CUs idle and all together still fit one round, or the tile
// chosen for all the rows keeps a larger share of its rounds busy (by 5 % at least).  taken_alone: CUs one of them takes.
static bool gemm_merge_rule(int dtype, int64_t n, int64_t k, int64_t m, int run, int compute_units, int64_t taken_alone) {
    const int64_t cus = compute_units;
    if (run < 2 || 2 * taken_alone <= cus || !turq_dt_is_quant(dtype) || dtype == TURQ_Q8_0 || n % 256 != 0) return false;
    int64_t wgs_one = 0, wgs_all = 0;
    const double fill_one = turq_gemm_fill(dtype, n, k, m, compute_units, &wgs_one);
    const double fill_all = turq_gemm_fill(dtype, n * run, k, m, compute_units, &wgs_all);
    return (wgs_one < cus && wgs_all <= cus) || fill_all > 1.05 * fill_one;
}

int turq_qmatmul_multi_gemm(turq_ctx *ctx, int count, const turq_weight *const *w, const void *x, int xt, int64_t m, int64_t ldx,
                            void *const *y, int yt, const int64_t *ldy, const float *const *bias, bool *taken, const TurqNorm *norm) {
    *taken = false;
    float ws[16];
    if (count > 16) return TURQ_OK;
    if (norm && (w[0]->k % 256 != 0 || w[0]->k > 16384)) return TURQ_OK;  // (the kernel that writes normalised fragments)
    for (int i = 0; i < count; i++)
        if (!gemm_takes(w[i], &ws[i])) return TURQ_OK;
    int rc = turq_ctx_reserve(ctx, &ctx->act_prep, &ctx->act_prep_cap, turq_act_prep32_bytes(m, w[0]->k));
    if (rc != TURQ_OK) return rc;
    GemmSplit sp;
    rc = gemm_split_reserve(ctx, count, w, m, &sp);
    if (rc != TURQ_OK) return rc;
    // k_proj / v_proj of a prompt chunk are launches of a quarter of the machine each.  Launches that leave half of the CUs free
    // run in groups, as many as fit the machine together (three at most): the first of a group on the context's stream, the
    // others on further streams that start where it starts (an event recorded there; behind the preparation, the only thing
    // they need) and are joined before the call returns.  Only when one preparation serves the whole call (a later
    // preparation would overwrite fragments that another stream still reads).
    const bool no_side = turq_tuning().gemm_no_side;
    const int64_t cus = ctx->compute_units;
    int n_small = 0;
    bool one_order = true;
    for (int i = 0; i < count; i++) {
        n_small += 2 * gemm_cus_taken(ctx, w[i], m, sp.counters[i] != nullptr) <= cus;
        one_order = one_order && (w[i]->dtype == TURQ_Q8_0) == (w[0]->dtype == TURQ_Q8_0);
    }
    const bool fork = !no_side && one_order && n_small >= 2 && side_ready(ctx);
    bool used[turq_ctx::kSide] = {};
    int group_n = 0;        // launches in the open group (0: none open)
    int64_t group_cus = 0;  // CUs they take together
    int prepared = 0;       // 1: K-quant order, 2: Q8_0 order
    hipError_t e = hipSuccess;
    const int merge_env = turq_tuning().gemm_merge;  // 0: never, 2: every run
    const bool no_merge = merge_env == 0, merge_all = merge_env == 2;
    for (int i = 0; i < count && e == hipSuccess; i++) {
        const int order = w[i]->dtype == TURQ_Q8_0 ? 2 : 1;
        if (order != prepared) {
            e = norm ? turq_launch_rms_norm_prep32(w[i]->dtype, x, xt, m, w[i]->k, ldx, norm->w, norm->eps, ctx->act_prep, ctx->stream)
                     : turq_launch_act_prep32(w[i]->dtype, x, xt, m, w[i]->k, ldx, ctx->act_prep, ctx->stream);
            if (e != hipSuccess) break;
            prepared = order;
        }
        hipStream_t st = ctx->stream;
        const int64_t c = gemm_cus_taken(ctx, w[i], m, sp.counters[i] != nullptr);
        // Neighbouring weights of one K-quant format and one shape that each take more than half of the machine (gate and up)
        // go out as ONE launch over the rows of all of them where that fills the rounds over the CUs better: where each alone
        // leaves CUs idle and all together still fit one round, or where the tile chosen for all the rows keeps a larger share
        // of its rounds busy (Q4_K 2 x 12288 x 4096, two launches -> one: 128 rows 50 -> 42 us, 256 rows 80 -> 67, 1024 rows
        // 257 -> 220; at 384 and 512 rows one launch is 3 % slower and the rule keeps two).  TURQ_GEMM_MERGE = 0: never, 2: every
        // such run whatever its size.
        if (!no_merge && (2 * c > cus || merge_all) && turq_dt_is_quant(w[i]->dtype) && w[i]->dtype != TURQ_Q8_0 && w[i]->n % 256 == 0) {
            int j = i + 1;
            while (j < count && j - i < 4 && w[j]->dtype == w[i]->dtype && w[j]->n == w[i]->n) j++;
            if (j - i >= 2) {
                if (merge_all || gemm_merge_rule(w[i]->dtype, w[i]->n, w[i]->k, m, j - i, ctx->compute_units, c)) {
                    TurqGemmWeights g{};
                    g.count = j - i;
                    for (int t = i; t < j; t++) {
                        g.w[t - i] = w[t]->dev;
                        g.y[t - i] = y[t];
                        g.bias[t - i] = bias ? bias[t] : nullptr;
                        g.n[t - i] = w[t]->n;
                        g.ldy[t - i] = ldy[t];
                        g.wscale[t - i] = ws[t];
                    }
                    group_n = 0;  // (such a launch closes a group of small ones)
                    hipEvent_t ev0 = nullptr, ev1 = nullptr;
                    e = turq_prof_next(ctx, &ev0, &ev1);
                    if (e == hipSuccess)
                        e = turq_launch_gemm_mfma_group(w[i]->dtype, g, w[i]->k, ctx->act_prep, m, yt, ctx->compute_units, st, ev0, ev1);
                    i = j - 1;
                    continue;
                }
            }
        }
        if (fork && 2 * c <= cus) {
            if (group_n == 0 || group_n > turq_ctx::kSide || group_cus + c > cus) {
                e = hipEventRecord(ctx->ev_fork, ctx->stream);  // opens a group
                group_n = 1;
                group_cus = c;
            } else {
                st = ctx->side[group_n - 1];
                e = hipStreamWaitEvent(st, ctx->ev_fork, 0);
                used[group_n - 1] = true;
                group_n++;
                group_cus += c;
            }
            if (e != hipSuccess) break;
        } else {
            group_n = 0;  // a launch that fills the machine closes the group
        }
        hipEvent_t ev0 = nullptr, ev1 = nullptr;
        e = turq_prof_next(ctx, &ev0, &ev1);
        if (e == hipSuccess)
            e = turq_launch_gemm_mfma(w[i]->dtype, w[i]->dev, w[i]->n, w[i]->k, ctx->act_prep, m, y[i], yt, ldy[i],
                                      bias ? bias[i] : nullptr, ws[i], ctx->compute_units, st, ev0, ev1, sp.counters[i], sp.partials[i],
                                      sp.bytes[i]);
    }
    for (int s = 0; s < turq_ctx::kSide; s++) {  // also after an error: nothing may stay behind on the other streams
        if (!used[s]) continue;
        hipError_t j = hipEventRecord(ctx->ev_join[s], ctx->side[s]);
        if (j == hipSuccess) j = hipStreamWaitEvent(ctx->stream, ctx->ev_join[s], 0);
        if (e == hipSuccess) e = j;
    }
    TURQ_HIP(ctx, e);
    *taken = true;
    return TURQ_OK;
}

bool turq_norm_fuses(const turq_ctx *ctx, int count, const turq_weight *const *w, const void *x, int xt, int64_t ldx, int64_t m) {
    const bool off = turq_tuning().norm_fused_off, no_fuse = turq_tuning().gemv_no_fuse;
    if (off || count < 1 || ctx->wide || ctx->fixed_scratch || !turq_act_bytes(xt)) return false;
    float ws = 1.0f;
    for (int i = 0; i < count; i++)
        if (!w[i] || w[i]->device != ctx->device || !turq_dt_is_quant(w[i]->dtype) || w[i]->layout != TURQ_LAYOUT_TILED || w[i]->k != w[0]->k ||
            w[i]->k <= 0 || w[i]->n <= 0)
            return false;
    const bool aligned = ((uintptr_t)x % 16 == 0) && ((size_t)ldx * turq_act_bytes(xt)) % 16 == 0;
    if (m == 1) {  // the one-row kernels (every quantized format has one), on rows they can load 16 bytes at a time
        for (int i = 0; i < count; i++)
            if (!use_row1(w[i]->dtype)) return false;
        return aligned && !no_fuse;
    }
    if (m <= TURQ_GEMV_MAX_M) return false;
    if (w[0]->k % 256 != 0 || w[0]->k > 16384 || turq_rows_in_chunks(ctx, count, w, x, xt, ldx, m)) return false;
    for (int i = 0; i < count; i++)
        if (!gemm_takes(w[i], &ws)) return false;
    return true;
}

// the prefill GEMM of one weight on fragments that already sit in ctx->act_prep
static int gemm_on_frags(turq_ctx *ctx, const turq_weight *w, int64_t m, void *y, int yt, int64_t ldy, const float *bias, float wscale) {
    GemmSplit sp;
    int rc = gemm_split_reserve(ctx, 1, &w, m, &sp);
    if (rc != TURQ_OK) return rc;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
    TURQ_HIP(ctx, turq_launch_gemm_mfma(w->dtype, w->dev, w->n, w->k, ctx->act_prep, m, y, yt, ldy, bias, wscale, ctx->compute_units,
                                        ctx->stream, ev0, ev1, sp.counters[0], sp.partials[0], sp.bytes[0]));
    return TURQ_OK;
}

// `Qwen3MLP::forward` (src/models/qwen3.rs:161-167) on a prompt chunk.  The separate calls write the two products (f32), read
// them back for SiLU(gate) * up, write that as f16, read it back for down_proj's fragment preparation: here one kernel reads
// the two products and writes the fragments (the same f16 values, so the results are those of the separate calls bit for bit),
// which saves a launch and a round trip of the intermediate per MLP.
int turq_mlp_prefill(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const turq_weight *down, const void *x, int xt,
                     int64_t m, int64_t ldx, void *y, int yt, int64_t ldy, const float *bias_gate, const float *bias_up,
                     const float *bias_down, bool *taken, const TurqNorm *norm) {
    *taken = false;
    const bool off = turq_tuning().mlp_prefill_off;
    const turq_weight *gu[2] = {gate, up};
    float ws_down = 1.0f, ws_tmp = 1.0f;
    if (off || m <= TURQ_GEMV_MAX_M || ctx->fixed_scratch) return TURQ_OK;
    for (const turq_weight *w : {gate, up, down})
        if (w->device != ctx->device || w->layout != TURQ_LAYOUT_TILED || w->n <= 0 || w->k <= 0 || !gemm_takes(w, &ws_tmp)) return TURQ_OK;
    if (!gemm_takes(down, &ws_down) || down->k != gate->n || gate->n != up->n || gate->k != up->k) return TURQ_OK;
    if (ldx < gate->k || ldy < down->n || !turq_act_bytes(xt) || !turq_act_bytes(yt)) return TURQ_OK;
    if (turq_rows_in_chunks(ctx, 2, gu, x, xt, ldx, m)) return TURQ_OK;  // gate / up through the kernels of up to 32 rows
    const int64_t n_ff = gate->n;
    const size_t half = (size_t)m * (size_t)n_ff;
    int rc = turq_ctx_reserve(ctx, &ctx->gate_up, &ctx->gate_up_cap, 2 * half * sizeof(float) + 16);
    if (rc != TURQ_OK) return rc;
    // one fragment buffer serves both preparations: sized for the larger before anything is queued
    rc = turq_ctx_reserve(ctx, &ctx->act_prep, &ctx->act_prep_cap, std::max(turq_act_prep32_bytes(m, gate->k), turq_act_prep32_bytes(m, n_ff)));
    if (rc != TURQ_OK) return rc;
    void *ys[2] = {ctx->gate_up, (float *)ctx->gate_up + half};
    const int64_t ldys[2] = {n_ff, n_ff};
    const float *biases[2] = {bias_gate, bias_up};
    bool gu_taken = false;
    rc = turq_qmatmul_multi_gemm(ctx, 2, gu, x, xt, m, ldx, ys, TURQ_ACT_F32, ldys, biases, &gu_taken, norm);
    if (rc != TURQ_OK || !gu_taken) return rc;
    TURQ_HIP(ctx, turq_launch_silu_mul_prep32(down->dtype, (const float *)ys[0], (const float *)ys[1], m, n_ff, ctx->act_prep, ctx->stream));
    rc = gemm_on_frags(ctx, down, m, y, yt, ldy, bias_down, ws_down);
    if (rc != TURQ_OK) return rc;
    *taken = true;
    return TURQ_OK;
}

int turq_qmatmul_mfma(turq_ctx *ctx, const turq_weight *w, const void *x, int xt, int64_t m, int64_t ldx, void *y,
                      int yt, int64_t ldy, const float *bias, int algo, const TurqNorm *norm) {
    const int xb = turq_act_bytes(xt), yb = turq_act_bytes(yt);
    if (norm && !turq_norm_fuses(ctx, 1, &w, x, xt, ldx, m))
        return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul: no kernel applies the norm for this call (internal)");
    // prefill chunks: LDS-tiled MFMA GEMM.  Its weights are packed f16 values (base + q) * d * sc (base 1024 for the nibbles of
    // Q4_K / Q5_K, 256 for the 6-bit values of Q6_K; q * d for Q8_0), the scales multiplied by a power of two that puts the
    // largest of them near 2^15 (small scales would otherwise lose bits in the f16 subnormals); a tensor whose largest value
    // does not fit f16 even unscaled goes through the exact skinny kernel instead
    float wscale = 1.0f;
    const bool gemm_ok = gemm_takes(w, &wscale);
    if (algo == TURQ_ALGO_GEMM && !gemm_ok && m > TURQ_GEMV_MAX_M)
        algo = TURQ_ALGO_GEMV;  // scales too large for f16 operands, ragged Q8_0 columns: walk m in chunks through the skinny kernel
    if (m > TURQ_GEMV_MAX_M && algo == TURQ_ALGO_GEMM) {
        int rc = turq_ctx_reserve(ctx, &ctx->act_prep, &ctx->act_prep_cap, turq_act_prep32_bytes(m, w->k));
        if (rc != TURQ_OK) return rc;
        GemmSplit sp;
        rc = gemm_split_reserve(ctx, 1, &w, m, &sp);
        if (rc != TURQ_OK) return rc;
        hipEvent_t ev0 = nullptr, ev1 = nullptr;
        if (norm) TURQ_HIP(ctx, turq_launch_rms_norm_prep32(w->dtype, x, xt, m, w->k, ldx, norm->w, norm->eps, ctx->act_prep, ctx->stream));
        else TURQ_HIP(ctx, turq_launch_act_prep32(w->dtype, x, xt, m, w->k, ldx, ctx->act_prep, ctx->stream));
        TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
        TURQ_HIP(ctx, turq_launch_gemm_mfma(w->dtype, w->dev, w->n, w->k, ctx->act_prep, m, y, yt, ldy, bias, wscale, ctx->compute_units,
                                            ctx->stream, ev0, ev1, sp.counters[0], sp.partials[0], sp.bytes[0]));
        return TURQ_OK;
    }
    const int nwaves = pick_waves(ctx, w->n, w->k);
    for (int64_t m0 = 0; m0 < m; m0 += TURQ_GEMV_MAX_M) {
        const int64_t mc = std::min<int64_t>(TURQ_GEMV_MAX_M, m - m0);
        const uint8_t *xc = (const uint8_t *)x + (size_t)m0 * (size_t)ldx * xb;
        uint8_t *yc = (uint8_t *)y + (size_t)m0 * (size_t)ldy * yb;
        const bool no_fuse = turq_tuning().gemv_no_fuse;
        // raw activation rows must be 16-byte (f32) / 8-byte (16-bit) aligned for the fused loads
        const bool aligned = ((uintptr_t)xc % 16 == 0) && ((size_t)ldx * xb) % 16 == 0;
        if (aligned && !no_fuse && use_row1(w->dtype) && row1_takes(mc, w->dev_bytes, w->dtype)) {
            hipEvent_t ev0 = nullptr, ev1 = nullptr;
            TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
            const void *wp = w->dev;
            void *yv = yc;
            TURQ_HIP(ctx, turq_launch_gemv_row1(w->dtype, 1, &wp, &w->n, w->k, xc, xt, ldx, mc, &yv, yt, &ldy, bias ? &bias : nullptr,
                                                pick_waves_row1(w->k), mc == 1 ? pick_rows_row1(ctx, turq_tile_rows(w->n)) : 1,
                                                ctx->stream, ev0, ev1, norm ? norm->w : nullptr, norm ? norm->eps : 0.0f));
            continue;
        }
        if (use_fused(ctx, mc, turq_tile_rows(w->n), w->dev_bytes) && aligned && !no_fuse) {
            hipEvent_t ev0 = nullptr, ev1 = nullptr;
            TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
            TURQ_HIP(ctx, turq_launch_gemv_mfma(w->dtype, w->dev, w->n, w->k, xc, xt, ldx, mc, true, yc, yt, ldy, bias,
                                                nwaves, ctx->stream, ev0, ev1));
            continue;
        }
        // prepared fragments: the same path as a group of one weight
        void *yv = yc;
        const int rc = turq_qmatmul_multi_mfma(ctx, 1, &w, xc, xt, mc, ldx, &yv, yt, &ldy, bias ? &bias : nullptr);
        if (rc != TURQ_OK) return rc;
    }
    return TURQ_OK;
}

// gate_proj and up_proj of an MLP with the activation and the product in the kernel: one or two activation rows (two: on
// weights large enough for the one-row kernel, as in row1_takes), tiled weights of one format, 16-byte aligned rows
// 33 .. 64 rows against weights of more than two row tiles per compute unit and up to 4096 columns (gate / up of an 8B model):
// two passes of the four-wave staged kernel (up to 32 rows each) stream the weights twice and still beat the prefill GEMM,
// which at these row counts makes few, half-empty tiles (gate + up 12288 x 4096 at 64 rows: 2 x 24 us against 62 us for
// two GEMM launches, plus the preparation launch and, fused, the elementwise pass that the staged kernel has in its epilogue).
// TURQ_ROWS_IN_CHUNKS = 0 switches it off.
bool turq_rows_in_chunks(const turq_ctx *ctx, int count, const turq_weight *const *w, const void *x, int xt, int64_t ldx, int64_t m) {
    const bool off = turq_tuning().rows_in_chunks_off;
    if (off || m <= TURQ_GEMV_MAX_M || m > 2 * TURQ_GEMV_MAX_M || count < 1 || count > 4) return false;
    const bool aligned = ((uintptr_t)x % 16 == 0) && ((size_t)ldx * turq_act_bytes(xt)) % 16 == 0;
    const int64_t cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
    int64_t row_tiles = 0;
    for (int i = 0; i < count; i++) {
        if (!turq_dt_is_quant(w[i]->dtype) || w[i]->dtype == TURQ_Q8_0 || w[i]->dtype != w[0]->dtype || w[i]->layout != TURQ_LAYOUT_TILED ||
            w[i]->k != w[0]->k)
            return false;
        row_tiles += turq_tile_rows(w[i]->n);
    }
    if (row_tiles <= 2 * cus) return false;
    return staged_row_tiles(ctx, w[0]->dtype, w[0]->dtype, w[0]->k, TURQ_GEMV_MAX_M, row_tiles, 0, aligned) == 6;
}

int turq_qmatmul_gate_up_mfma(turq_ctx *ctx, const turq_weight *gate, const turq_weight *up, const void *x, int xt, int64_t m,
                              int64_t ldx, void *y, int yt, int64_t ldy, const float *bias_gate, const float *bias_up, bool *taken,
                              const TurqNorm *norm) {
    const bool no_fuse = turq_tuning().gemv_no_fuse;
    *taken = false;
    if (norm && m != 1) return TURQ_OK;  // (the caller normalises into scratch first)
    {
        const turq_weight *pair[2] = {gate, up};
        if (m > TURQ_GEMV_MAX_M && gate->n == up->n && turq_rows_in_chunks(ctx, 2, pair, x, xt, ldx, m) &&
            turq_gemv_cs_staged_gateup_tiles(gate->dtype, gate->n, gate->k, TURQ_GEMV_MAX_M, ctx->compute_units > 0 ? ctx->compute_units : 256) == 6) {
            const int xb = turq_act_bytes(xt), yb = turq_act_bytes(yt);
            for (int64_t m0 = 0; m0 < m; m0 += TURQ_GEMV_MAX_M) {
                bool part = false;
                const int rc = turq_qmatmul_gate_up_mfma(ctx, gate, up, (const uint8_t *)x + (size_t)m0 * (size_t)ldx * xb, xt,
                                                         std::min<int64_t>(TURQ_GEMV_MAX_M, m - m0), ldx,
                                                         (uint8_t *)y + (size_t)m0 * (size_t)ldy * yb, yt, ldy, bias_gate, bias_up, &part);
                if (rc != TURQ_OK) return rc;
                if (!part) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul_gate_up: a chunk of rows was not taken by the kernel its call was planned for");
            }
            *taken = true;
            return TURQ_OK;
        }
    }
    const bool aligned = ((uintptr_t)x % 16 == 0) && ((size_t)ldx * turq_act_bytes(xt)) % 16 == 0;
    if (m < 1 || m > TURQ_GEMV_MAX_M || gate->dtype != up->dtype || !turq_dt_is_quant(gate->dtype) || gate->layout != TURQ_LAYOUT_TILED ||
        up->layout != TURQ_LAYOUT_TILED)
        return TURQ_OK;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    // 3 .. 16 rows: the kernel that makes its fragments from the rows themselves (no preparation launch), activation in its epilogue
    {
        const int staged = turq_tuning().cs_staged;
        const int64_t cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
        const int tiles = (staged != 0 && aligned && m >= 3 && gate->n == up->n && gate->k == up->k)
                              ? turq_gemv_cs_staged_gateup_tiles(gate->dtype, gate->n, gate->k, m, cus) : 0;
        if (tiles) {
            TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
            TURQ_HIP(ctx, turq_launch_gemv_cs_staged_gateup(gate->dtype, gate->dev, up->dev, gate->n, gate->k, x, xt, ldx, m, y, yt, ldy,
                                                            bias_gate, bias_up, tiles, ctx->stream, ev0, ev1));
            *taken = true;
            return TURQ_OK;
        }
    }
    if (norm && (no_fuse || !aligned || !use_row1(gate->dtype))) return TURQ_OK;
    if (no_fuse || !aligned || m > 2 || !use_row1(gate->dtype) || !row1_takes(m, gate->dev_bytes + up->dev_bytes, gate->dtype)) {
        // up to 32 rows: fragments prepared once, then one launch whose workgroups take row tile b of both weights (the shape
        // of the two-row-tile kernel: at most four waves) and store the product
        const bool no_frag = turq_tuning().gateup_no_frag;
        if (no_frag) return TURQ_OK;
        int rc = turq_ctx_reserve(ctx, &ctx->act_prep, &ctx->act_prep_cap, turq_act_prep_bytes(gate->dtype, m, gate->k));
        if (rc != TURQ_OK) return rc;
        TURQ_HIP(ctx, turq_launch_act_prep(gate->dtype, x, xt, m, gate->k, ldx, ctx->act_prep, ctx->stream));
        TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
        const int nw = std::min(pick_waves(ctx, gate->n, gate->k), 4);
        TURQ_HIP(ctx, turq_launch_gemv_gateup_frag(gate->dtype, gate->dev, up->dev, gate->n, gate->k, ctx->act_prep, m, y, yt, ldy,
                                                   bias_gate, bias_up, nw, ctx->stream, ev0, ev1));
        *taken = true;
        return TURQ_OK;
    }
    TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
    // a wave holds a tile of each weight per column tile: half as many column tiles per wave as in the plain launch, i.e. twice
    // the waves (K = 4096: 16 waves of one column tile; 8 waves of two cost the MLP step 2.7 %)
    const bool forced = turq_tuning().gemv_waves != 0;
    int nwaves = pick_waves_row1(gate->k);
    if (!forced) nwaves = (int)std::min<int64_t>({2 * (int64_t)nwaves, 16, turq_tile_cols(gate->k)});
    TURQ_HIP(ctx, turq_launch_gemv_row1_gateup(gate->dtype, gate->dev, up->dev, gate->n, gate->k, x, xt, ldx, m, y, yt, ldy, bias_gate,
                                               bias_up, nwaves, ctx->stream, ev0, ev1, norm ? norm->w : nullptr, norm ? norm->eps : 0.0f));
    *taken = true;
    return TURQ_OK;
}

// Runs of neighbouring weights with the same format go out as one launch of the skinny kernel; the caller has
// checked that all weights are tiled, share k and the device and that m <= TURQ_GEMV_MAX_M.  Up to
// TURQ_GEMV_FUSED_MAX_M rows with 16-byte aligned activation rows the kernel converts the activations itself; otherwise
// the activation fragments are prepared once per fragment order (K-quants / Q8_0) and shared by all the weights.
int turq_qmatmul_multi_mfma(turq_ctx *ctx, int count, const turq_weight *const *w, const void *x, int xt, int64_t m,
                            int64_t ldx, void *const *y, int yt, const int64_t *ldy, const float *const *bias, const TurqNorm *norm) {
    const bool no_fuse = turq_tuning().gemv_no_fuse;
    if (norm && !(m == 1 && turq_norm_fuses(ctx, count, w, x, xt, ldx, m)))
        return turq_fail(ctx, TURQ_ERR_INVALID, "turq_qmatmul_multi: no kernel applies the norm for this call (internal)");
    const bool aligned = ((uintptr_t)x % 16 == 0) && ((size_t)ldx * turq_act_bytes(xt)) % 16 == 0;
    int64_t all_tiles = 0;
    size_t all_bytes = 0;
    for (int t = 0; t < count; t++) {
        all_tiles += turq_tile_rows(w[t]->n);
        all_bytes += w[t]->dev_bytes;
    }
    const bool fused = use_fused(ctx, m, all_tiles, all_bytes) && aligned && !no_fuse;
    int prepared = 0;  // fragment order currently in ctx->act_prep: 0 none, 1 K-quants, 2 Q8_0
    int i = 0;
    while (i < count) {
        int j = i + 1;
        while (j < count && j - i < 4 && w[j]->dtype == w[i]->dtype) j++;
        // one activation row: a run of a second format joins the launch where the kernel has that pair (q, k Q4_K + v Q6_K)
        const bool no_mixed = turq_tuning().gemv_no_mixed;
        // 5 .. 16 rows: fragments made in the kernel from the rows themselves (staged through the LDS), a second format in the
        // same launch where the kernel has the pair
        {
            int j2 = j;
            if (!no_mixed && j < count) {
                j2 = j + 1;
                while (j2 < count && w[j2]->dtype == w[j]->dtype) j2++;
                if (j2 - i > 4) j2 = j;
            }
            for (int end = j2; end >= j; end = (end == j ? -1 : j)) {
                int64_t tiles = 0, tiles_b = 0;
                for (int t = i; t < end; t++) tiles += turq_tile_rows(w[t]->n);
                for (int t = j; t < end; t++) tiles_b += turq_tile_rows(w[t]->n);
                const int dtb = end > j ? w[j]->dtype : w[i]->dtype;
                const int rg = staged_row_tiles(ctx, w[i]->dtype, dtb, w[i]->k, m, tiles, tiles_b, aligned);
                if (!rg) continue;
                const void *wp[4];
                int64_t nn[4];
                for (int t = i; t < end; t++) {
                    wp[t - i] = w[t]->dev;
                    nn[t - i] = w[t]->n;
                }
                hipEvent_t ev0 = nullptr, ev1 = nullptr;
                TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
                TURQ_HIP(ctx, turq_launch_gemv_cs_staged(w[i]->dtype, dtb, end - i, end > j ? j - i : end - i, wp, nn, w[i]->k, x, xt, ldx, m,
                                                         y + i, yt, ldy + i, bias ? bias + i : nullptr, rg, ctx->stream, ev0, ev1));
                i = end;
                break;
            }
            if (i >= j) continue;
        }
        // (more than two rows: only a call of one format, which would otherwise lose the launch it shares with a second one)
        const bool row1_ok = aligned && !no_fuse && use_row1(w[i]->dtype) && row1_takes(m, all_bytes, w[i]->dtype) &&
                             (m <= 2 || (i == 0 && j == count));
        if (row1_ok && m <= 2 && !no_mixed && j < count && use_row1(w[j]->dtype) &&
            turq_gemv_row1_mixed_supports(w[i]->dtype, w[j]->dtype)) {
            int j2 = j + 1;
            while (j2 < count && w[j2]->dtype == w[j]->dtype) j2++;
            if (j2 - i <= 4) {
                const void *wp[4];
                int64_t nn[4];
                for (int t = i; t < j2; t++) {
                    wp[t - i] = w[t]->dev;
                    nn[t - i] = w[t]->n;
                }
                hipEvent_t ev0 = nullptr, ev1 = nullptr;
                TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
                TURQ_HIP(ctx, turq_launch_gemv_row1_mixed(w[i]->dtype, w[j]->dtype, j2 - i, j - i, wp, nn, w[i]->k, x, xt, ldx, m, y + i,
                                                          yt, ldy + i, bias ? bias + i : nullptr, pick_waves_row1(w[i]->k), ctx->stream,
                                                          ev0, ev1, norm ? norm->w : nullptr, norm ? norm->eps : 0.0f));
                i = j2;
                continue;
            }
        }
        if (!row1_ok) {
            // several row tiles per compute unit: fragments in registers, built from the rows themselves, no preparation
            int64_t tiles = 0;
            for (int t = i; t < j; t++) tiles += turq_tile_rows(w[t]->n);
            const int rg = cs_row_tiles(ctx, m, tiles, w[i]->dtype, aligned);
            if (rg) {
                const void *wp[4];
                int64_t nn[4];
                for (int t = i; t < j; t++) {
                    wp[t - i] = w[t]->dev;
                    nn[t - i] = w[t]->n;
                }
                const int cs_waves = turq_tuning().cs_waves;
                const int nw = (int)std::min<int64_t>(cs_waves >= 1 && cs_waves <= 8 ? cs_waves : 8, turq_tile_cols(w[i]->k));
                hipEvent_t ev0 = nullptr, ev1 = nullptr;
                TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
                TURQ_HIP(ctx, turq_launch_gemv_cs(w[i]->dtype, j - i, wp, nn, w[i]->k, x, xt, ldx, m, y + i, yt, ldy + i,
                                                  bias ? bias + i : nullptr, nw, rg, ctx->stream, ev0, ev1));
                i = j;
                continue;
            }
        }
        if (row1_ok) {
            const void *wp[4];
            int64_t nn[4];
            int64_t rows = 0;
            for (int t = i; t < j; t++) {
                wp[t - i] = w[t]->dev;
                nn[t - i] = w[t]->n;
                rows += w[t]->n;
            }
            hipEvent_t ev0 = nullptr, ev1 = nullptr;
            TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
            TURQ_HIP(ctx, turq_launch_gemv_row1(w[i]->dtype, j - i, wp, nn, w[i]->k, x, xt, ldx, m, y + i, yt, ldy + i,
                                                bias ? bias + i : nullptr, pick_waves_row1(w[i]->k),
                                                m == 1 ? pick_rows_row1(ctx, turq_tile_rows(rows)) : 1, ctx->stream, ev0, ev1,
                                                norm ? norm->w : nullptr, norm ? norm->eps : 0.0f));
            i = j;
            continue;
        }
        if (!fused) {
            const int order = w[i]->dtype == TURQ_Q8_0 ? 2 : 1;
            if (prepared != order) {
                int rc = turq_ctx_reserve(ctx, &ctx->act_prep, &ctx->act_prep_cap, turq_act_prep_bytes(w[i]->dtype, m, w[i]->k));
                if (rc != TURQ_OK) return rc;
                TURQ_HIP(ctx, turq_launch_act_prep(w[i]->dtype, x, xt, m, w[i]->k, ldx, ctx->act_prep, ctx->stream));
                prepared = order;
            }
        }
        // prepared fragments: the same for a second format of the same fragment order, while one row tile per workgroup is the
        // launch shape anyway
        if (!fused && !no_mixed && j < count && turq_gemv_multi_mixed_supports(w[i]->dtype, w[j]->dtype)) {
            int j2 = j + 1;
            while (j2 < count && w[j2]->dtype == w[j]->dtype) j2++;
            int64_t rows2 = 0;
            for (int t = i; t < j2; t++) rows2 += w[t]->n;
            const int64_t cus2 = ctx->compute_units > 0 ? ctx->compute_units : 256;
            if (j2 - i <= 4 && turq_tile_rows(rows2) < 4 * cus2) {
                const void *wp2[4];
                int64_t nn2[4];
                for (int t = i; t < j2; t++) {
                    wp2[t - i] = w[t]->dev;
                    nn2[t - i] = w[t]->n;
                }
                hipEvent_t e0 = nullptr, e1 = nullptr;
                TURQ_HIP(ctx, turq_prof_next(ctx, &e0, &e1));
                TURQ_HIP(ctx, turq_launch_gemv_multi_mixed(w[i]->dtype, w[j]->dtype, j2 - i, j - i, wp2, nn2, w[i]->k, ctx->act_prep, m,
                                                           y + i, yt, ldy + i, bias ? bias + i : nullptr,
                                                           pick_waves(ctx, rows2, w[i]->k), ctx->stream, e0, e1));
                i = j2;
                continue;
            }
        }
        const void *wp[4];
        int64_t nn[4];
        int64_t rows = 0;
        for (int t = i; t < j; t++) {
            wp[t - i] = w[t]->dev;
            nn[t - i] = w[t]->n;
            rows += w[t]->n;
        }
        // prepared fragments are the larger stream (9 - 18 KiB per column tile against 2 - 4 KiB per weight tile): with enough
        // row tiles to keep every CU busy a workgroup takes two of them per set of fragments
        const int forced_r = turq_tuning().gemv_rowtiles;
        const int64_t cus = ctx->compute_units > 0 ? ctx->compute_units : 256;
        int rtiles = (!fused && turq_tile_rows(rows) >= 4 * cus) ? 2 : 1;
        if (!fused && (forced_r == 1 || forced_r == 2)) rtiles = forced_r;
        int nwaves = pick_waves(ctx, rows / rtiles, w[i]->k);
        if (rtiles == 2) nwaves = std::min(nwaves, 4);
        hipEvent_t ev0 = nullptr, ev1 = nullptr;
        TURQ_HIP(ctx, turq_prof_next(ctx, &ev0, &ev1));
        TURQ_HIP(ctx, turq_launch_gemv_multi(w[i]->dtype, j - i, wp, nn, w[i]->k, fused ? x : ctx->act_prep, xt, ldx, m, fused, y + i, yt,
                                             ldy + i, bias ? bias + i : nullptr, nwaves, rtiles, ctx->stream, ev0, ev1));
        i = j;
    }
    return TURQ_OK;
}

// whether turq_qmatmul_multi sends `count` neighbouring weights of this format and shape out as one prefill launch (no GPU needed)
extern "C" int turq_prefill_plan_multi(int dtype, int64_t n, int64_t k, int64_t m, int count, int compute_units, int *merged) {
    if (merged) *merged = 0;
    if (!turq_dt_is_quant(dtype)) return turq_fail(nullptr, TURQ_ERR_DTYPE, "turq_prefill_plan_multi: dtype %d has no prefill kernel", dtype);
    if (n <= 0 || k <= 0 || k % 256 != 0 || m <= TURQ_GEMV_MAX_M || compute_units <= 0 || count < 1 || count > 4)
        return turq_fail(nullptr, TURQ_ERR_SHAPE, "turq_prefill_plan_multi: n=%lld k=%lld m=%lld count=%d on %d compute units", (long long)n,
                         (long long)k, (long long)m, count, compute_units);
    const int64_t alone = gemm_cus_taken_shape(compute_units, dtype, n, k, m, true);
    if (merged) *merged = gemm_merge_rule(dtype, n, k, m, count, compute_units, alone) ? 1 : 0;
    return TURQ_OK;
}

// which launch the rules above and in gemm_mfma.hip make for a prompt chunk (no GPU needed)
extern "C" int turq_prefill_plan(int dtype, int64_t n, int64_t k, int64_t m, int compute_units, int *tile, int *split, int *wave_groups) {
    if (tile) *tile = 0;
    if (split) *split = 1;
    if (wave_groups) *wave_groups = 1;
    if (!turq_dt_is_quant(dtype)) return turq_fail(nullptr, TURQ_ERR_DTYPE, "turq_prefill_plan: dtype %d has no prefill kernel", dtype);
    if (n <= 0 || k <= 0 || k % 256 != 0 || m <= TURQ_GEMV_MAX_M || compute_units <= 0)
        return turq_fail(nullptr, TURQ_ERR_SHAPE, "turq_prefill_plan: n=%lld k=%lld m=%lld on %d compute units", (long long)n, (long long)k,
                         (long long)m, compute_units);
    int form = turq_gemm_form(dtype, n, k, m, compute_units), parts = 1, sform = 0;
    if (turq_gemm_split_scratch(dtype, n, k, m, compute_units, &sform, &parts) != 0) form = sform;
    else parts = 1;
    if (tile) *tile = form;
    if (split) *split = parts;
    if (wave_groups) *wave_groups = form == 4 && turq_gemm_low_two_groups(n, k, m, parts, compute_units) ? 2 : 1;
    return TURQ_OK;
}


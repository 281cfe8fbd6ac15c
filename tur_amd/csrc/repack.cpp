// Host-side transforms between GGUF byte order and the tiled HBM layout (layout.h).
// Pure CPU code: used by upload / export and callable without a GPU.
#include <algorithm>
#include <thread>
#include <vector>

#include "layout.h"

namespace {

template <int DT>
void tile_rows(int64_t n, int64_t k, const uint8_t *nat, uint8_t *tiled, int64_t rt0, int64_t rt1) {
    constexpr int BE = TiledFmt<DT>::kBlockElems, BB = TiledFmt<DT>::kBlockBytes;
    const int64_t bpr = k / BE;
    for (int64_t row = rt0 * 16; row < std::min<int64_t>(rt1 * 16, n); row++)
        for (int64_t b = 0; b < bpr; b++) turq_tile_block<DT>(nat + (row * bpr + b) * BB, tiled, k, row, b);
}

template <int DT>
void untile_rows(int64_t n, int64_t k, const uint8_t *tiled, uint8_t *nat, int64_t rt0, int64_t rt1) {
    constexpr int BE = TiledFmt<DT>::kBlockElems, BB = TiledFmt<DT>::kBlockBytes;
    const int64_t bpr = k / BE;
    for (int64_t row = rt0 * 16; row < std::min<int64_t>(rt1 * 16, n); row++)
        for (int64_t b = 0; b < bpr; b++) {
            uint8_t *dst = nat + (row * bpr + b) * BB;
            memset(dst, 0, BB);
            turq_untile_block<DT>(tiled, k, row, b, dst);
        }
}

template <typename Fn>
void parallel_row_tiles(int64_t nrt, Fn fn) {
    unsigned hw = std::thread::hardware_concurrency();
    int64_t nthreads = std::max<int64_t>(1, std::min<int64_t>({(int64_t)(hw ? hw : 1), 16, nrt / 64}));
    if (nthreads <= 1) { fn(0, nrt); return; }
    std::vector<std::thread> pool;
    const int64_t per = (nrt + nthreads - 1) / nthreads;
    for (int64_t t = 0; t < nthreads; t++) {
        const int64_t a = t * per, b = std::min(nrt, a + per);
        if (a >= b) break;
        pool.emplace_back([=] { fn(a, b); });
    }
    for (auto &th : pool) th.join();
}

bool shape_ok(int dt, int64_t n, int64_t k) {
    return turq_dt_is_quant(dt) && n >= 0 && k >= 0 && k % turq_dt_block_elems(dt) == 0;
}

}  // namespace

extern "C" size_t turq_tiled_nbytes(int dt, int64_t n, int64_t k) {
    if (!shape_ok(dt, n, k)) return 0;
    return (size_t)(turq_tile_rows(n) * turq_tile_cols(k)) * (size_t)turq_tile_bytes(dt);
}

extern "C" int turq_tile_host(int dt, int64_t n, int64_t k, const void *native, void *tiled) {
    if (!shape_ok(dt, n, k)) return turq_fail(nullptr, TURQ_ERR_SHAPE, "turq_tile_host: bad dtype/shape (%d, %lld, %lld)", dt, (long long)n, (long long)k);
    if ((!native || !tiled) && n * k > 0) return turq_fail(nullptr, TURQ_ERR_INVALID, "turq_tile_host: null pointer");
    memset(tiled, 0, turq_tiled_nbytes(dt, n, k));
    const uint8_t *src = (const uint8_t *)native;
    uint8_t *dst = (uint8_t *)tiled;
    const int64_t nrt = turq_tile_rows(n);
    switch (dt) {
    case TURQ_Q4_K: parallel_row_tiles(nrt, [=](int64_t a, int64_t b) { tile_rows<TURQ_Q4_K>(n, k, src, dst, a, b); }); break;
    case TURQ_Q5_K: parallel_row_tiles(nrt, [=](int64_t a, int64_t b) { tile_rows<TURQ_Q5_K>(n, k, src, dst, a, b); }); break;
    case TURQ_Q6_K: parallel_row_tiles(nrt, [=](int64_t a, int64_t b) { tile_rows<TURQ_Q6_K>(n, k, src, dst, a, b); }); break;
    case TURQ_Q8_0: parallel_row_tiles(nrt, [=](int64_t a, int64_t b) { tile_rows<TURQ_Q8_0>(n, k, src, dst, a, b); }); break;
    }
    return TURQ_OK;
}

extern "C" int turq_untile_host(int dt, int64_t n, int64_t k, const void *tiled, void *native) {
    if (!shape_ok(dt, n, k)) return turq_fail(nullptr, TURQ_ERR_SHAPE, "turq_untile_host: bad dtype/shape (%d, %lld, %lld)", dt, (long long)n, (long long)k);
    if ((!native || !tiled) && n * k > 0) return turq_fail(nullptr, TURQ_ERR_INVALID, "turq_untile_host: null pointer");
    const uint8_t *src = (const uint8_t *)tiled;
    uint8_t *dst = (uint8_t *)native;
    const int64_t nrt = turq_tile_rows(n);
    switch (dt) {
    case TURQ_Q4_K: parallel_row_tiles(nrt, [=](int64_t a, int64_t b) { untile_rows<TURQ_Q4_K>(n, k, src, dst, a, b); }); break;
    case TURQ_Q5_K: parallel_row_tiles(nrt, [=](int64_t a, int64_t b) { untile_rows<TURQ_Q5_K>(n, k, src, dst, a, b); }); break;
    case TURQ_Q6_K: parallel_row_tiles(nrt, [=](int64_t a, int64_t b) { untile_rows<TURQ_Q6_K>(n, k, src, dst, a, b); }); break;
    case TURQ_Q8_0: parallel_row_tiles(nrt, [=](int64_t a, int64_t b) { untile_rows<TURQ_Q8_0>(n, k, src, dst, a, b); }); break;
    }
    return TURQ_OK;
}

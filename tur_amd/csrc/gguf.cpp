// GGUF container reader: header, metadata, tensor infos, lazy per-tensor reads and upload.
// Follows the published GGUF layout (versions 1..3) the way candle's `gguf_file::Content::read`
// consumes it for `QVarBuilder::from_gguf` (reference: src/weights/gguf_varbuilder.rs:20-30) and
// `Content::tensor` for `QVarBuilder::get` (src/weights/gguf_varbuilder.rs:52-94).
#include <cerrno>
#include <map>
#include <memory>
#include <mutex>
#include <vector>

#include "common.h"

namespace {

enum ValueType : uint32_t {
    VT_U8 = 0, VT_I8 = 1, VT_U16 = 2, VT_I16 = 3, VT_U32 = 4, VT_I32 = 5, VT_F32 = 6, VT_BOOL = 7,
    VT_STRING = 8, VT_ARRAY = 9, VT_U64 = 10, VT_I64 = 11, VT_F64 = 12
};

struct MetaValue {
    uint32_t type = 0;
    uint64_t u = 0;     // unsigned / bool / array length
    int64_t i = 0;      // signed
    double f = 0.0;     // floats
    std::string s;      // strings
    uint32_t elem_type = 0;  // arrays: element type (elements themselves are skipped)
};

struct TensorInfo {
    int dtype = 0;
    int n_dims = 0;
    int64_t dims[4] = {1, 1, 1, 1};  // outermost first (GGUF order reversed)
    uint64_t offset = 0;             // relative to the data section
    size_t nbytes = 0;
};

}  // namespace

struct turq_gguf {
    FILE *fp = nullptr;
    std::mutex mu;  // one seek+read at a time (the reference keeps the File behind a Mutex)
    std::string path;
    uint32_t version = 0;
    uint64_t alignment = 32;
    uint64_t data_offset = 0;
    uint64_t file_size = 0;
    std::map<std::string, MetaValue> meta;
    std::vector<std::string> names;  // file order
    std::map<std::string, TensorInfo> tensors;
    mutable std::string err;
};

namespace {

struct Reader {
    FILE *fp;
    uint32_t version;
    uint64_t file_size = 0;  // lengths read from the file are checked against what is left of it
    bool ok = true;
    std::string why;
    void fail(const std::string &m) { if (ok) { ok = false; why = m; } }
    bool raw(void *dst, size_t n) {
        if (!ok) return false;
        if (n && fread(dst, 1, n, fp) != n) { fail("unexpected end of file"); return false; }
        return true;
    }
    template <typename T> T num() { T v{}; raw(&v, sizeof v); return v; }  // little-endian host assumed
    uint64_t count() { return version == 1 ? (uint64_t)num<uint32_t>() : num<uint64_t>(); }
    uint64_t left() {
        const off_t at = ftello(fp);
        return at < 0 || (uint64_t)at > file_size ? 0 : file_size - (uint64_t)at;
    }
    std::string str() {
        const uint64_t len = count();
        if (!ok) return {};
        if (len > (1ull << 30) || len > left()) { fail("string length " + std::to_string(len) + " runs past the end of the file"); return {}; }
        std::string s((size_t)len, '\0');
        raw(s.data(), (size_t)len);
        while (!s.empty() && s.back() == '\0') s.pop_back();  // GGUF v1 strings may carry a terminator
        return s;
    }
    void skip(uint64_t n) {
        if (!ok) return;
        if (n > left()) { fail("a value of " + std::to_string(n) + " bytes runs past the end of the file"); return; }
        if (fseeko(fp, (off_t)n, SEEK_CUR) != 0) fail("seek failed");
    }
    static size_t scalar_size(uint32_t t) {
        switch (t) {
        case VT_U8: case VT_I8: case VT_BOOL: return 1;
        case VT_U16: case VT_I16: return 2;
        case VT_U32: case VT_I32: case VT_F32: return 4;
        case VT_U64: case VT_I64: case VT_F64: return 8;
        default: return 0;
        }
    }
    MetaValue value(uint32_t t) {
        MetaValue v;
        v.type = t;
        switch (t) {
        case VT_U8: v.u = num<uint8_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
        case VT_I8: v.i = num<int8_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
        case VT_U16: v.u = num<uint16_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
        case VT_I16: v.i = num<int16_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
        case VT_U32: v.u = num<uint32_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
        case VT_I32: v.i = num<int32_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
        case VT_U64: v.u = num<uint64_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
        case VT_I64: v.i = num<int64_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
        case VT_F32: v.f = num<float>(); break;
        case VT_F64: v.f = num<double>(); break;
        case VT_BOOL: v.u = num<uint8_t>() != 0; v.i = (int64_t)v.u; v.f = (double)v.u; break;
        case VT_STRING: v.s = str(); break;
        case VT_ARRAY: {
            v.elem_type = num<uint32_t>();
            v.u = count();
            if (!ok) break;
            if (v.elem_type == VT_STRING) {
                for (uint64_t i = 0; i < v.u && ok; i++) skip(count());
            } else if (v.elem_type == VT_ARRAY) {
                fail("nested arrays in metadata are not supported");
            } else {
                const size_t sz = scalar_size(v.elem_type);
                if (!sz) fail("unknown array element type " + std::to_string(v.elem_type));
                else if (v.u > left() / sz) fail("array of " + std::to_string(v.u) + " elements runs past the end of the file");
                else skip(v.u * sz);
            }
            break;
        }
        default: fail("unknown metadata value type " + std::to_string(t));
        }
        return v;
    }
};

int gfail(turq_gguf *g, int code, const std::string &msg) {
    if (g) g->err = msg;
    turq_thread_error() = msg;
    return code;
}

const TensorInfo *find(const turq_gguf *g, const char *name) {
    auto it = g->tensors.find(name);
    return it == g->tensors.end() ? nullptr : &it->second;
}

}  // namespace

extern "C" {

static int gguf_open_impl(const char *path, turq_gguf **out);

int turq_gguf_open(const char *path, turq_gguf **out) {
    if (!out) return gfail(nullptr, TURQ_ERR_INVALID, "turq_gguf_open: null out pointer");
    *out = nullptr;
    if (!path) return gfail(nullptr, TURQ_ERR_INVALID, "turq_gguf_open: null path");
    try {  // strings, maps and vectors sized by the file: nothing may unwind through the C boundary
        return gguf_open_impl(path, out);
    } catch (const std::bad_alloc &) {
        return gfail(nullptr, TURQ_ERR_OOM, std::string(path) + ": out of memory while reading the header");
    } catch (const std::exception &e) {
        return gfail(nullptr, TURQ_ERR_IO, std::string(path) + ": " + e.what());
    }
}

static int gguf_open_impl(const char *path, turq_gguf **out) {
    std::unique_ptr<turq_gguf> g(new (std::nothrow) turq_gguf);
    if (!g) return gfail(nullptr, TURQ_ERR_OOM, "turq_gguf_open: out of memory");
    g->path = path;
    g->fp = fopen(path, "rb");
    if (!g->fp) return gfail(nullptr, TURQ_ERR_IO, std::string("cannot open ") + path + ": " + strerror(errno));
    auto bail = [&](int code, const std::string &m) {
        fclose(g->fp);
        g->fp = nullptr;
        return gfail(nullptr, code, std::string(path) + ": " + m);
    };
    fseeko(g->fp, 0, SEEK_END);
    g->file_size = (uint64_t)ftello(g->fp);
    fseeko(g->fp, 0, SEEK_SET);

    Reader rd{g->fp, 0, g->file_size};
    const uint32_t magic = rd.num<uint32_t>();
    if (!rd.ok || magic != 0x46554747u) return bail(TURQ_ERR_IO, "not a GGUF file (bad magic)");
    g->version = rd.num<uint32_t>();
    if (!rd.ok || g->version < 1 || g->version > 3) return bail(TURQ_ERR_IO, "unsupported GGUF version " + std::to_string(g->version));
    rd.version = g->version;
    const uint64_t tensor_count = rd.count();
    const uint64_t kv_count = rd.count();
    if (!rd.ok) return bail(TURQ_ERR_IO, rd.why);
    if (tensor_count > (1ull << 24) || kv_count > (1ull << 24)) return bail(TURQ_ERR_IO, "implausible tensor / metadata count");
    for (uint64_t i = 0; i < kv_count && rd.ok; i++) {
        std::string key = rd.str();
        const uint32_t vt = rd.num<uint32_t>();
        MetaValue v = rd.value(vt);
        if (rd.ok) g->meta.emplace(std::move(key), std::move(v));
    }
    if (!rd.ok) return bail(TURQ_ERR_IO, "metadata: " + rd.why);
    for (uint64_t i = 0; i < tensor_count && rd.ok; i++) {
        std::string name = rd.str();
        TensorInfo ti;
        const uint32_t nd = rd.num<uint32_t>();
        if (!rd.ok) break;
        if (nd < 1 || nd > 4) { rd.fail("tensor " + name + " has " + std::to_string(nd) + " dimensions"); break; }
        ti.n_dims = (int)nd;
        uint64_t ne[4] = {1, 1, 1, 1};
        for (uint32_t d = 0; d < nd; d++) ne[d] = g->version == 1 ? (uint64_t)rd.num<uint32_t>() : rd.num<uint64_t>();
        ti.dtype = (int)rd.num<uint32_t>();
        ti.offset = rd.num<uint64_t>();
        if (!rd.ok) break;
        uint64_t nelem = 1;
        for (uint32_t d = 0; d < nd; d++) {
            ti.dims[nd - 1 - d] = (int64_t)ne[d];  // reversed: outermost first
            if (ne[d] && nelem > (1ull << 62) / ne[d]) { rd.fail("tensor " + name + " is too large"); break; }
            nelem *= ne[d];
        }
        const int be = turq_dt_block_elems(ti.dtype);
        if (be) {
            if (ne[0] % (uint64_t)be) {
                rd.fail("tensor " + name + ": innermost dimension " + std::to_string(ne[0]) +
                        " is not divisible by the block size " + std::to_string(be));
                break;
            }
            ti.nbytes = (size_t)(nelem / (uint64_t)be) * (size_t)turq_dt_block_bytes(ti.dtype);
        }  // dtypes this library cannot hold stay listed with nbytes == 0 and fail on load
        if (g->tensors.count(name)) { rd.fail("tensor " + name + " is listed twice"); break; }
        g->names.push_back(name);
        g->tensors.emplace(std::move(name), ti);
    }
    if (!rd.ok) return bail(TURQ_ERR_IO, "tensor infos: " + rd.why);
    auto al = g->meta.find("general.alignment");
    if (al != g->meta.end()) {
        if (al->second.type == VT_STRING || al->second.type == VT_ARRAY || al->second.u == 0)
            return bail(TURQ_ERR_IO, "general.alignment is not a positive integer");
        g->alignment = al->second.u;
    }
    const uint64_t pos = (uint64_t)ftello(g->fp);
    g->data_offset = (pos + g->alignment - 1) / g->alignment * g->alignment;
    *out = g.release();
    return TURQ_OK;
}

void turq_gguf_close(turq_gguf *g) {
    if (!g) return;
    if (g->fp) fclose(g->fp);
    delete g;
}

const char *turq_gguf_last_error(const turq_gguf *g) { return g ? g->err.c_str() : turq_thread_error().c_str(); }

int64_t turq_gguf_tensor_count(const turq_gguf *g) { return g ? (int64_t)g->names.size() : 0; }

const char *turq_gguf_tensor_name(const turq_gguf *g, int64_t index) {
    if (!g || index < 0 || index >= (int64_t)g->names.size()) return nullptr;
    return g->names[(size_t)index].c_str();
}

int turq_gguf_tensor_info(const turq_gguf *g, const char *name, int *dt, int *n_dims, int64_t dims[4], uint64_t *file_offset,
                          size_t *nbytes) {
    if (!g || !name) return gfail(nullptr, TURQ_ERR_INVALID, "turq_gguf_tensor_info: null argument");
    const TensorInfo *ti = find(g, name);
    if (!ti) return gfail(const_cast<turq_gguf *>(g), TURQ_ERR_NOT_FOUND, std::string("cannot find tensor info for ") + name);
    if (dt) *dt = ti->dtype;
    if (n_dims) *n_dims = ti->n_dims;
    if (dims) for (int i = 0; i < 4; i++) dims[i] = i < ti->n_dims ? ti->dims[i] : 1;
    if (file_offset) *file_offset = g->data_offset + ti->offset;
    if (nbytes) *nbytes = ti->nbytes;
    return TURQ_OK;
}

static const MetaValue *meta_find(const turq_gguf *g, const char *key, int *rc) {
    if (!g || !key) { *rc = gfail(nullptr, TURQ_ERR_INVALID, "gguf metadata lookup: null argument"); return nullptr; }
    auto it = g->meta.find(key);
    if (it == g->meta.end()) {
        *rc = gfail(const_cast<turq_gguf *>(g), TURQ_ERR_NOT_FOUND, std::string("cannot find ") + key + " in metadata");
        return nullptr;
    }
    return &it->second;
}

int turq_gguf_meta_u64(const turq_gguf *g, const char *key, uint64_t *out) {
    int rc = TURQ_OK;
    const MetaValue *v = meta_find(g, key, &rc);
    if (!v) return rc;
    if (v->type == VT_STRING || v->type == VT_F32 || v->type == VT_F64)
        return gfail(const_cast<turq_gguf *>(g), TURQ_ERR_DTYPE, std::string(key) + " is not an integer value");
    if (out) *out = v->u;  // arrays report their length
    return TURQ_OK;
}

int turq_gguf_meta_f64(const turq_gguf *g, const char *key, double *out) {
    int rc = TURQ_OK;
    const MetaValue *v = meta_find(g, key, &rc);
    if (!v) return rc;
    if (v->type == VT_STRING || v->type == VT_ARRAY)
        return gfail(const_cast<turq_gguf *>(g), TURQ_ERR_DTYPE, std::string(key) + " is not a numeric value");
    if (out) *out = v->f;
    return TURQ_OK;
}

int turq_gguf_meta_str(const turq_gguf *g, const char *key, char *out, size_t cap) {
    int rc = TURQ_OK;
    const MetaValue *v = meta_find(g, key, &rc);
    if (!v) return rc;
    if (v->type != VT_STRING) return gfail(const_cast<turq_gguf *>(g), TURQ_ERR_DTYPE, std::string(key) + " is not a string value");
    if (out && cap) snprintf(out, cap, "%s", v->s.c_str());
    return TURQ_OK;
}

int turq_gguf_read_tensor(turq_gguf *g, const char *name, void *host_bytes, size_t nbytes) {
    if (!g || !name) return gfail(nullptr, TURQ_ERR_INVALID, "turq_gguf_read_tensor: null argument");
    const TensorInfo *ti = find(g, name);
    if (!ti) return gfail(g, TURQ_ERR_NOT_FOUND, std::string("cannot find tensor info for ") + name);
    if (!turq_dt_block_elems(ti->dtype))
        return gfail(g, TURQ_ERR_DTYPE, std::string("tensor ") + name + " has unsupported ggml dtype " + std::to_string(ti->dtype));
    if (nbytes != ti->nbytes)
        return gfail(g, TURQ_ERR_SHAPE, std::string("tensor ") + name + " has " + std::to_string(ti->nbytes) + " bytes, buffer has " + std::to_string(nbytes));
    if (nbytes == 0) return TURQ_OK;
    if (!host_bytes) return gfail(g, TURQ_ERR_INVALID, "turq_gguf_read_tensor: null buffer");
    // (checked without forming data_offset + offset + nbytes, which a hostile offset could wrap)
    if (g->data_offset > g->file_size || ti->offset > g->file_size - g->data_offset || nbytes > g->file_size - g->data_offset - ti->offset)
        return gfail(g, TURQ_ERR_IO, std::string("tensor ") + name + " runs past the end of " + g->path);
    const uint64_t off = g->data_offset + ti->offset;
    std::lock_guard<std::mutex> lock(g->mu);
    if (fseeko(g->fp, (off_t)off, SEEK_SET) != 0) return gfail(g, TURQ_ERR_IO, std::string("seek failed in ") + g->path);
    if (fread(host_bytes, 1, nbytes, g->fp) != nbytes) return gfail(g, TURQ_ERR_IO, std::string("short read in ") + g->path);
    return TURQ_OK;
}

int turq_gguf_load_weight(turq_ctx *ctx, turq_gguf *g, const char *name, int64_t expect_n, int64_t expect_k, int layout,
                          turq_weight **out) {
    if (!ctx) return turq_fail(nullptr, TURQ_ERR_INVALID, "turq_gguf_load_weight: null context");
    if (!out) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_gguf_load_weight: null out pointer");
    *out = nullptr;
    if (!g || !name) return turq_fail(ctx, TURQ_ERR_INVALID, "turq_gguf_load_weight: null argument");
    const TensorInfo *ti = find(g, name);
    if (!ti) return turq_fail(ctx, TURQ_ERR_NOT_FOUND, "cannot find tensor info for %s", name);
    if (ti->n_dims > 2) return turq_fail(ctx, TURQ_ERR_SHAPE, "tensor %s has %d dimensions, a linear weight has at most 2", name, ti->n_dims);
    const int64_t n = ti->n_dims == 2 ? ti->dims[0] : 1;
    const int64_t k = ti->n_dims == 2 ? ti->dims[1] : ti->dims[0];
    if ((expect_n >= 0 && expect_n != n) || (expect_k >= 0 && expect_k != k))
        return turq_fail(ctx, TURQ_ERR_SHAPE, "shape mismatch for %s, got [%lld, %lld], expected [%lld, %lld]", name,
                         (long long)n, (long long)k, (long long)expect_n, (long long)expect_k);
    std::vector<uint8_t> buf;
    try {
        buf.resize(ti->nbytes);
    } catch (const std::bad_alloc &) {
        return turq_fail(ctx, TURQ_ERR_OOM, "out of host memory reading %s (%zu bytes)", name, ti->nbytes);
    }
    int rc = turq_gguf_read_tensor(g, name, buf.data(), buf.size());
    if (rc != TURQ_OK) return turq_fail(ctx, rc, "%s", g->err.c_str());
    return turq_weight_upload(ctx, ti->dtype, n, k, buf.data(), buf.size(), layout, out);
}

}  // extern "C"

// C++ host-side mirror of the reference's quantized-linear interface over the libturq C ABI.
//
// The reference is Rust; its toolchain is not part of this build, so the host side above the C ABI
// is given in C++ with the reference's names, argument meaning and error behaviour:
//   turq::Device        the candle `Device` passed to `QVarBuilder::from_gguf`
//   turq::QTensor       `Arc<QTensor>` (shared, reference counted device copy; shape, dtype, dequantize)
//   turq::QMatMul       `QMatMul::from_arc` / `forward`
//   turq::LinearX       src/models/layers/linear.rs:8-31 (Quantized arm: matmul, then the bias)
//   turq::QVarBuilder   src/weights/gguf_varbuilder.rs (from_gguf, pp, get, get_no_shape, contains_key,
//                       tensor_shape, all_keys, one-entry last-tensor cache)
//   turq::linear()      src/models/layers/linear.rs:50-70 (GGUF arm)
// Failures throw turq::Error (the reference returns candle_core::Error through Result).
// Tensors here are device pointers (turq::DeviceBuffer) or host vectors; nothing computes on the CPU.
#pragma once

#include <cstdint>
#include <memory>
#include <mutex>
#include <cstdlib>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../../include/turq.h"

namespace turq {

struct Error : std::runtime_error {
    int code;
    Error(int c, const std::string &m) : std::runtime_error(m), code(c) {}
};

class Device {
public:
    explicit Device(int ordinal = 0) {
        turq_ctx *c = nullptr;
        int rc = turq_ctx_create(ordinal, &c);
        if (rc != TURQ_OK) throw Error(rc, turq_last_error(nullptr));
        ctx_ = std::shared_ptr<turq_ctx>(c, turq_ctx_destroy);
    }
    static Device new_hip(int ordinal) { return Device(ordinal); }
    turq_ctx *ctx() const { return ctx_.get(); }
    void check(int rc) const { if (rc != TURQ_OK) throw Error(rc, turq_last_error(ctx_.get())); }
    void synchronize() const { check(turq_sync(ctx_.get())); }

private:
    std::shared_ptr<turq_ctx> ctx_;
};

// RAII device allocation for callers without HIP bindings of their own
class DeviceBuffer {
public:
    DeviceBuffer(const Device &d, size_t nbytes) : dev_(d), nbytes_(nbytes) { dev_.check(turq_dev_alloc(dev_.ctx(), nbytes, &p_)); }
    ~DeviceBuffer() { if (p_) turq_dev_free(dev_.ctx(), p_); }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    void *ptr() const { return p_; }
    size_t nbytes() const { return nbytes_; }
    void upload(const void *src, size_t n) { dev_.check(turq_memcpy_h2d(dev_.ctx(), p_, src, n)); }
    void download(void *dst, size_t n) const { dev_.check(turq_memcpy_d2h(dev_.ctx(), dst, p_, n)); }

private:
    Device dev_;
    void *p_ = nullptr;
    size_t nbytes_ = 0;
};

class QTensor {
public:
    QTensor(const Device &d, turq_weight *w, bool one_dim) : dev_(d), w_(w, turq_weight_release), one_dim_(one_dim) {
        d.check(turq_weight_info(w, &dtype_, &n_, &k_, &layout_, &device_bytes_));
    }
    // raw GGUF block bytes of a tensor of shape (n, k)
    static QTensor from_blocks(const Device &d, int ggml_dtype, int64_t n, int64_t k, const void *bytes, size_t nbytes,
                               int layout = TURQ_LAYOUT_TILED) {
        turq_weight *w = nullptr;
        d.check(turq_weight_upload(d.ctx(), ggml_dtype, n, k, bytes, nbytes, layout, &w));
        return QTensor(d, w, false);
    }
    std::vector<int64_t> shape() const { return one_dim_ ? std::vector<int64_t>{k_} : std::vector<int64_t>{n_, k_}; }
    int dtype() const { return dtype_; }
    int64_t rows() const { return n_; }
    int64_t cols() const { return k_; }
    int layout() const { return layout_; }
    turq_weight *handle() const { return w_.get(); }
    const Device &device() const { return dev_; }
    // `QTensor::dequantize(device)`: f32 values, bit-exact with candle's to_float
    std::vector<float> dequantize() const {
        std::vector<float> out((size_t)n_ * (size_t)k_);
        dev_.check(turq_dequantize(dev_.ctx(), w_.get(), out.data(), TURQ_MEM_HOST));
        return out;
    }
    void dequantize_to(DeviceBuffer &out) const { dev_.check(turq_dequantize(dev_.ctx(), w_.get(), (float *)out.ptr(), TURQ_MEM_DEVICE)); }

private:
    Device dev_;
    std::shared_ptr<turq_weight> w_;  // copies share the device weight, like Arc<QTensor>
    bool one_dim_;
    int dtype_ = 0, layout_ = 0;
    int64_t n_ = 0, k_ = 0;
    size_t device_bytes_ = 0;
};

// As in candle, a block-quantized tensor gives the quantized matmul (QMatMul::QTensor) and an F32 / F16 / BF16 tensor - or any
// tensor while CANDLE_DEQUANTIZE_ALL / CANDLE_DEQUANTIZE_ALL_F16 is set - the dense one (QMatMul::Tensor): f32 arithmetic on
// the dequantized weights, activations not rounded (the plain kernel on the tensor's GGUF bytes; a tiled tensor is uploaded
// once more in GGUF order for it).
class QMatMul {
public:
    static bool dequantize_all() {
        const char *a = std::getenv("CANDLE_DEQUANTIZE_ALL"), *b = std::getenv("CANDLE_DEQUANTIZE_ALL_F16");
        return (a && *a) || (b && *b);
    }
    static QMatMul from_arc(const QTensor &t) {
        const int dt = t.dtype();
        const bool quant = dt == TURQ_Q8_0 || dt == TURQ_Q4_K || dt == TURQ_Q5_K || dt == TURQ_Q6_K;
        if (!quant && dt != TURQ_F32 && dt != TURQ_F16 && dt != TURQ_BF16) throw Error(TURQ_ERR_DTYPE, "QMatMul: unsupported ggml dtype");
        const bool dense = !quant || dequantize_all();
        if (dense && t.layout() != TURQ_LAYOUT_NATIVE) {
            std::vector<uint8_t> raw(turq_weight_nbytes(dt, t.rows(), t.cols()));
            t.device().check(turq_weight_export(t.device().ctx(), t.handle(), raw.data(), raw.size()));
            return QMatMul(QTensor::from_blocks(t.device(), dt, t.rows(), t.cols(), raw.data(), raw.size(), TURQ_LAYOUT_NATIVE), true);
        }
        return QMatMul(t, dense);
    }
    bool dense() const { return dense_; }
    // host tensors: xs is [m, k] row-major f32, returns [m, n]
    std::vector<float> forward(const std::vector<float> &xs, int64_t m, const float *bias = nullptr) const {
        if (m < 0 || (int64_t)xs.size() != m * t_.cols()) throw Error(TURQ_ERR_SHAPE, "shape mismatch in matmul: input is not [m, k]");
        std::vector<float> y((size_t)m * (size_t)t_.rows());
        t_.device().check(turq_qmatmul(t_.device().ctx(), t_.handle(), xs.data(), TURQ_ACT_F32, m, t_.cols(), y.data(), TURQ_ACT_F32,
                                       t_.rows(), bias, TURQ_MEM_HOST, dense_ ? TURQ_ALGO_SIMPLE : TURQ_ALGO_AUTO));
        return y;
    }
    // y += x W^T on device tensors: the residual connection taken into the matmul's store (`x + h`, src/models/qwen3.rs:635)
    void forward_add(const void *x_dev, int x_dtype, int64_t m, int64_t ldx, void *y_dev, int y_dtype, int64_t ldy,
                     const float *bias_dev = nullptr) const {
        forward(x_dev, x_dtype, m, ldx, y_dev, y_dtype | TURQ_OUT_ACCUMULATE, ldy, bias_dev);
    }
    // device tensors: asynchronous on the device's stream
    void forward(const void *x_dev, int x_dtype, int64_t m, int64_t ldx, void *y_dev, int y_dtype, int64_t ldy,
                 const float *bias_dev = nullptr) const {
        t_.device().check(turq_qmatmul(t_.device().ctx(), t_.handle(), x_dev, x_dtype, m, ldx, y_dev, y_dtype, ldy, bias_dev,
                                       TURQ_MEM_DEVICE, dense_ ? TURQ_ALGO_SIMPLE : TURQ_ALGO_AUTO));
    }
    // Several projections of one device tensor (q / k / v, gate / up: src/models/qwen3.rs:161-167, 272-274), ys[i] is
    // [m, n_i] with row stride n_i: one kernel launch per run of equal formats for m <= 32, the single calls otherwise.
    static void forward_multi(const std::vector<const QMatMul *> &layers, const void *x_dev, int x_dtype, int64_t m, int64_t ldx,
                              const std::vector<void *> &ys_dev, int y_dtype) {
        if (layers.empty()) return;
        if (layers.size() != ys_dev.size()) throw Error(TURQ_ERR_SHAPE, "forward_multi: one output per layer");
        std::vector<const turq_weight *> w;
        std::vector<int64_t> ldy;
        for (const QMatMul *l : layers) {
            w.push_back(l->t_.handle());
            ldy.push_back(l->t_.rows());
        }
        const Device &d = layers[0]->t_.device();
        d.check(turq_qmatmul_multi(d.ctx(), (int)w.size(), w.data(), x_dev, x_dtype, m, ldx, ys_dev.data(), y_dtype, ldy.data(), nullptr,
                                   TURQ_MEM_DEVICE, TURQ_ALGO_AUTO));
    }
    // silu(x gate^T) * (x up^T) of a device tensor, the first half of Qwen3MLP::forward (src/models/qwen3.rs:161-167): for one
    // or two rows one kernel launch that writes the product, otherwise two products and an elementwise pass
    static void forward_gate_up(const QMatMul &gate, const QMatMul &up, const void *x_dev, int x_dtype, int64_t m, int64_t ldx,
                                void *y_dev, int y_dtype, int64_t ldy) {
        const Device &d = gate.t_.device();
        d.check(turq_qmatmul_gate_up(d.ctx(), gate.t_.handle(), up.t_.handle(), x_dev, x_dtype, m, ldx, y_dev, y_dtype, ldy, nullptr,
                                     nullptr, TURQ_ACTFN_SILU, TURQ_MEM_DEVICE));
    }
    // (silu(x gate^T) * (x up^T)) down^T of a device tensor, the whole of Qwen3MLP::forward (src/models/qwen3.rs:161-167); the
    // f32 intermediate lives in the context's scratch memory
    static void forward_mlp(const QMatMul &gate, const QMatMul &up, const QMatMul &down, const void *x_dev, int x_dtype, int64_t m,
                            int64_t ldx, void *y_dev, int y_dtype, int64_t ldy) {
        const Device &d = gate.t_.device();
        d.check(turq_mlp(d.ctx(), gate.t_.handle(), up.t_.handle(), down.t_.handle(), x_dev, x_dtype, m, ldx, y_dev, y_dtype, ldy, nullptr,
                         nullptr, nullptr, TURQ_ACTFN_SILU, TURQ_MEM_DEVICE));
    }
    const QTensor &qtensor() const { return t_; }

private:
    explicit QMatMul(const QTensor &t, bool dense = false) : t_(t), dense_(dense) {}
    QTensor t_;
    bool dense_ = false;
};

// LinearX::Quantized { qmatmul, bias }: forward = qmatmul.forward(x), then broadcast_add(bias)
class LinearX {
public:
    LinearX(QMatMul q, std::optional<std::vector<float>> bias) : q_(std::move(q)), bias_(std::move(bias)) {}
    std::vector<float> forward(const std::vector<float> &x, int64_t m) const {
        return q_.forward(x, m, bias_ ? bias_->data() : nullptr);
    }
    const QMatMul &qmatmul() const { return q_; }
    const std::optional<std::vector<float>> &bias() const { return bias_; }
    static const char *name() { return "LinearX::Quantized"; }

private:
    QMatMul q_;
    std::optional<std::vector<float>> bias_;
};

// NormX over candle_nn's RmsNorm (src/models/layers/norm.rs:9-41), GGUF arm: f32 weight, f32 arithmetic, output in the input's type
class NormX {
public:
    NormX(const Device &d, std::vector<float> weight, float eps)
        : dev_(d), w_(std::move(weight)), eps_(eps), wdev_(std::make_shared<DeviceBuffer>(d, w_.size() * sizeof(float))) {
        wdev_->upload(w_.data(), w_.size() * sizeof(float));
    }
    // host tensor [m, k] f32
    std::vector<float> forward(const std::vector<float> &xs, int64_t m) const {
        const int64_t k = (int64_t)w_.size();
        if (m < 0 || (int64_t)xs.size() != m * k) throw Error(TURQ_ERR_SHAPE, "shape mismatch in rms-norm: input is not [m, k]");
        std::vector<float> y(xs.size());
        dev_.check(turq_rms_norm(dev_.ctx(), xs.data(), TURQ_ACT_F32, m, k, k, w_.data(), eps_, y.data(), TURQ_ACT_F32, k, TURQ_MEM_HOST));
        return y;
    }
    // device tensors, asynchronous on the device's stream; y may be x
    void forward(const void *x_dev, int x_dtype, int64_t m, int64_t ldx, void *y_dev, int y_dtype, int64_t ldy) const {
        dev_.check(turq_rms_norm(dev_.ctx(), x_dev, x_dtype, m, (int64_t)w_.size(), ldx, (const float *)wdev_->ptr(), eps_, y_dev, y_dtype, ldy,
                                 TURQ_MEM_DEVICE));
    }
    // forward_multi(layers, forward(x)) on a device tensor in one call: ln1 -> q / k / v (src/models/qwen3.rs:633-634, 272-274),
    // the final norm -> lm_head; the norm is applied inside the matmul kernels where they can (turq_norm_qmatmul_multi)
    void forward_then(const std::vector<const QMatMul *> &layers, const void *x_dev, int x_dtype, int64_t m, int64_t ldx,
                      const std::vector<void *> &ys_dev, int y_dtype) const {
        if (layers.empty()) return;
        if (layers.size() != ys_dev.size()) throw Error(TURQ_ERR_SHAPE, "forward_then: one output per layer");
        std::vector<const turq_weight *> w;
        std::vector<int64_t> ldy;
        for (const QMatMul *l : layers) {
            w.push_back(l->qtensor().handle());
            ldy.push_back(l->qtensor().rows());
        }
        dev_.check(turq_norm_qmatmul_multi(dev_.ctx(), (int)w.size(), w.data(), x_dev, x_dtype, m, ldx, (const float *)wdev_->ptr(), eps_,
                                           ys_dev.data(), y_dtype, ldy.data(), nullptr, TURQ_MEM_DEVICE));
    }
    // y += mlp(forward(x)) on device tensors, the second half of the decoder layer (src/models/qwen3.rs:637-640): y is the residual
    // stream (it may be x); accumulate = false writes the MLP's output instead
    void forward_mlp(const QMatMul &gate, const QMatMul &up, const QMatMul &down, const void *x_dev, int x_dtype, int64_t m, int64_t ldx,
                     void *y_dev, int y_dtype, int64_t ldy, bool accumulate = true) const {
        dev_.check(turq_norm_mlp(dev_.ctx(), gate.qtensor().handle(), up.qtensor().handle(), down.qtensor().handle(), x_dev, x_dtype, m, ldx,
                                 (const float *)wdev_->ptr(), eps_, y_dev, y_dtype | (accumulate ? TURQ_OUT_ACCUMULATE : 0), ldy, nullptr,
                                 nullptr, nullptr, TURQ_ACTFN_SILU, TURQ_MEM_DEVICE));
    }
    const std::vector<float> &weight() const { return w_; }
    static const char *name() { return "RmsNorm"; }

private:
    Device dev_;
    std::vector<float> w_;
    float eps_;
    std::shared_ptr<DeviceBuffer> wdev_;  // clones share the device copy of the weight
};

// candle's Embedding over a table that stays quantized: forward gathers and dequantizes the rows of the given token ids where
// the reference dequantizes the whole table at load (src/models/layers/mod.rs:30-37)
class Embedding {
public:
    Embedding(QTensor table, int64_t hidden_size) : t_(std::move(table)) {
        if (t_.cols() != hidden_size) throw Error(TURQ_ERR_SHAPE, "shape mismatch for weight: row length is not the hidden size");
    }
    // host ids -> host rows [ids.size(), hidden]
    std::vector<float> forward(const std::vector<uint32_t> &ids) const {
        std::vector<float> out(ids.size() * (size_t)t_.cols());
        t_.device().check(turq_embedding_lookup(t_.device().ctx(), t_.handle(), ids.data(), (int64_t)ids.size(), out.data(), TURQ_ACT_F32,
                                                t_.cols(), TURQ_MEM_HOST));
        return out;
    }
    // device ids -> device rows, asynchronous on the device's stream
    void forward(const uint32_t *ids_dev, int64_t count, void *out_dev, int out_dtype, int64_t ldo) const {
        t_.device().check(turq_embedding_lookup(t_.device().ctx(), t_.handle(), ids_dev, count, out_dev, out_dtype, ldo, TURQ_MEM_DEVICE));
    }
    int64_t vocab_size() const { return t_.rows(); }

private:
    QTensor t_;
};

class QVarBuilder {
public:
    static QVarBuilder from_gguf(const std::string &path, const Device &d, int layout = TURQ_LAYOUT_TILED) {
        turq_gguf *g = nullptr;
        int rc = turq_gguf_open(path.c_str(), &g);
        if (rc != TURQ_OK) throw Error(rc, turq_gguf_last_error(nullptr));
        QVarBuilder vb(d, layout);
        vb.g_ = std::shared_ptr<turq_gguf>(g, turq_gguf_close);
        vb.cache_ = std::make_shared<Cache>();
        return vb;
    }
    QVarBuilder pp(const std::string &s) const {
        QVarBuilder vb(*this);
        vb.path_.push_back(s);
        return vb;
    }
    QVarBuilder pp(int64_t i) const { return pp(std::to_string(i)); }
    std::string path(const std::string &tensor_name) const {
        std::string p;
        for (const auto &s : path_) p += s + ".";
        return p + tensor_name;
    }
    const Device &device() const { return dev_; }
    bool contains_key(const std::string &key) const {
        return turq_gguf_tensor_info(g_.get(), path(key).c_str(), nullptr, nullptr, nullptr, nullptr, nullptr) == TURQ_OK;
    }
    std::optional<std::vector<int64_t>> tensor_shape(const std::string &key) const {
        int nd = 0;
        int64_t dims[4];
        if (turq_gguf_tensor_info(g_.get(), path(key).c_str(), nullptr, &nd, dims, nullptr, nullptr) != TURQ_OK) return std::nullopt;
        return std::vector<int64_t>(dims, dims + nd);
    }
    std::vector<std::string> all_keys() const {
        std::vector<std::string> keys;
        for (int64_t i = 0; i < turq_gguf_tensor_count(g_.get()); i++) keys.emplace_back(turq_gguf_tensor_name(g_.get(), i));
        return keys;
    }
    // get((n, k), name) / get((k), name): shape-checked, served from the one-entry cache when the name repeats
    QTensor get(const std::vector<int64_t> &shape, const std::string &name) const {
        const std::string full = path(name);
        std::lock_guard<std::mutex> lock(cache_->mu);
        if (!cache_->tensor || cache_->name != full) {
            cache_->tensor = std::make_shared<QTensor>(load(full));
            cache_->name = full;
        }
        if (cache_->tensor->shape() != shape) throw Error(TURQ_ERR_SHAPE, "shape mismatch for " + name + ", got " + fmt(cache_->tensor->shape()) + ", expected " + fmt(shape));
        return *cache_->tensor;
    }
    QTensor get_no_shape(const std::string &name) const { return load(path(name)); }

private:
    struct Cache { std::mutex mu; std::string name; std::shared_ptr<QTensor> tensor; };
    QVarBuilder(const Device &d, int layout) : dev_(d), layout_(layout) {}
    static std::string fmt(const std::vector<int64_t> &s) {
        std::string r = "[";
        for (size_t i = 0; i < s.size(); i++) r += (i ? ", " : "") + std::to_string(s[i]);
        return r + "]";
    }
    QTensor load(const std::string &full) const {
        int dt = 0, nd = 0;
        if (turq_gguf_tensor_info(g_.get(), full.c_str(), &dt, &nd, nullptr, nullptr, nullptr) != TURQ_OK)
            throw Error(TURQ_ERR_NOT_FOUND, turq_gguf_last_error(g_.get()));
        const bool quant = dt == TURQ_Q8_0 || dt == TURQ_Q4_K || dt == TURQ_Q5_K || dt == TURQ_Q6_K;
        turq_weight *w = nullptr;
        dev_.check(turq_gguf_load_weight(dev_.ctx(), g_.get(), full.c_str(), -1, -1, quant ? layout_ : TURQ_LAYOUT_NATIVE, &w));
        return QTensor(dev_, w, nd == 1);
    }
    Device dev_;
    int layout_;
    std::shared_ptr<turq_gguf> g_;
    std::shared_ptr<Cache> cache_;
    std::vector<std::string> path_;
};

// GGUF arm of layers::linear: the weight stays quantized; the bias is looked up with `.ok()` (absent or mis-shaped: none) and
// dequantized at load, where a failure is an error (`.transpose()?`)
inline LinearX linear(int64_t in_dim, int64_t out_dim, const QVarBuilder &vb) {
    QTensor qweight = vb.get({out_dim, in_dim}, "weight");
    std::optional<QTensor> qbias;
    try {
        qbias = vb.get({out_dim}, "bias");
    } catch (const Error &) {
        qbias.reset();
    }
    std::optional<std::vector<float>> bias;
    if (qbias) bias = qbias->dequantize();
    return LinearX(QMatMul::from_arc(qweight), std::move(bias));
}

// GGUF arm of layers::norm::rms_norm (src/models/layers/norm.rs:52-94): the `weight` tensor dequantized to f32, plus one for the
// Gemma family
inline NormX rms_norm(int64_t size, double eps, const QVarBuilder &vb, bool is_gemma = false) {
    std::vector<float> w = vb.get({size}, "weight").dequantize();
    if (is_gemma)
        for (float &v : w) v += 1.0f;
    return NormX(vb.device(), std::move(w), (float)eps);
}

}  // namespace turq

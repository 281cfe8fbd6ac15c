// Exercises the C++ host mirror (tur_amd/csrc/host/turq.hpp) against a GGUF file written by the
// Python test that launches this program.  Usage: test_host FILE.gguf
// Prints "name n k checksum" lines the Python side compares with the oracle; exits non-zero on error.
#include <cmath>
#include <cstdio>
#include <cstring>

#include "../../tur_amd/csrc/host/turq.hpp"

static int fail(const char *what) {
    std::fprintf(stderr, "FAIL: %s\n", what);
    return 1;
}

int main(int argc, char **argv) {
    if (argc < 2) return fail("usage: test_host FILE.gguf");
    try {
        turq::Device dev = turq::Device::new_hip(0);
        turq::QVarBuilder vb = turq::QVarBuilder::from_gguf(argv[1], dev);
        if (vb.all_keys().empty()) return fail("no tensors");
        turq::QVarBuilder b0 = vb.pp("blk").pp(0);
        if (b0.path("ffn_gate.weight") != "blk.0.ffn_gate.weight") return fail("path");
        if (!b0.contains_key("ffn_gate.weight") || b0.contains_key("ffn_gate.bias")) return fail("contains_key");
        auto shp = b0.tensor_shape("ffn_gate.weight");
        if (!shp || shp->size() != 2) return fail("tensor_shape");
        const int64_t n = (*shp)[0], k = (*shp)[1];
        // shape mismatch must be an error with the reference's wording
        bool threw = false;
        try { b0.pp("ffn_gate").get({n + 1, k}, "weight"); } catch (const turq::Error &e) { threw = std::strstr(e.what(), "shape mismatch for weight") != nullptr; }
        if (!threw) return fail("shape mismatch not reported");
        threw = false;
        try { b0.pp("nope").get({n, k}, "weight"); } catch (const turq::Error &e) { threw = e.code == TURQ_ERR_NOT_FOUND; }
        if (!threw) return fail("missing tensor not reported");

        turq::LinearX gate = turq::linear(k, n, b0.pp("ffn_gate"));
        turq::LinearX biased = turq::linear(k, 96, b0.pp("biased"));
        if (gate.bias() || !biased.bias() || biased.bias()->size() != 96) return fail("bias handling");
        turq::LinearX copy = gate;  // Clone: shares the device weight

        // x[i, j] = deterministic pattern the Python side reproduces
        const int64_t m = 3;
        std::vector<float> x((size_t)m * k);
        for (int64_t i = 0; i < m; i++)
            for (int64_t j = 0; j < k; j++) x[i * k + j] = std::sin(0.37f * (float)(i * k + j)) * 2.0f;
        std::vector<float> y = copy.forward(x, m);
        std::vector<float> yb = biased.forward(x, m);
        if ((int64_t)y.size() != m * n || (int64_t)yb.size() != m * 96) return fail("output shape");
        std::printf("gate %lld %lld\n", (long long)n, (long long)k);
        for (float v : y) std::printf("%.9g\n", v);
        std::printf("biased 96 %lld\n", (long long)k);
        for (float v : yb) std::printf("%.9g\n", v);

        // device-pointer forward (bf16 output) through QMatMul
        turq::DeviceBuffer xd(dev, x.size() * 4), yd(dev, (size_t)m * n * 4);
        xd.upload(x.data(), x.size() * 4);
        copy.qmatmul().forward(xd.ptr(), TURQ_ACT_F32, m, k, yd.ptr(), TURQ_ACT_F32, n);
        dev.synchronize();
        std::vector<float> y2((size_t)m * n);
        yd.download(y2.data(), y2.size() * 4);
        for (size_t i = 0; i < y.size(); i++)
            if (y[i] != y2[i]) return fail("host-pointer and device-pointer forward differ");

        // two projections of the same device tensor in one call: equal to the single calls
        {
            turq::DeviceBuffer ya(dev, (size_t)m * n * 4), yc(dev, (size_t)m * 96 * 4);
            turq::QMatMul::forward_multi({&copy.qmatmul(), &biased.qmatmul()}, xd.ptr(), TURQ_ACT_F32, m, k, {ya.ptr(), yc.ptr()},
                                         TURQ_ACT_F32);
            dev.synchronize();
            std::vector<float> y3((size_t)m * n), y4((size_t)m * 96);
            ya.download(y3.data(), y3.size() * 4);
            yc.download(y4.data(), y4.size() * 4);
            for (size_t i = 0; i < y.size(); i++)
                if (std::fabs(y3[i] - y[i]) > 1e-4f * (1.0f + std::fabs(y[i]))) return fail("forward_multi differs from forward (first layer)");
            turq::DeviceBuffer ys(dev, (size_t)m * 96 * 4);
            biased.qmatmul().forward(xd.ptr(), TURQ_ACT_F32, m, k, ys.ptr(), TURQ_ACT_F32, 96);
            dev.synchronize();
            std::vector<float> y5((size_t)m * 96);
            ys.download(y5.data(), y5.size() * 4);
            for (size_t i = 0; i < y5.size(); i++)
                if (std::fabs(y4[i] - y5[i]) > 1e-4f * (1.0f + std::fabs(y5[i]))) return fail("forward_multi differs from forward (second layer)");
        }

        // silu(gate(x)) * up(x) in one call (same weight in both places): equal to the expression on the single call's result
        {
            turq::DeviceBuffer yg(dev, (size_t)m * n * 4);
            turq::QMatMul::forward_gate_up(copy.qmatmul(), copy.qmatmul(), xd.ptr(), TURQ_ACT_F32, m, k, yg.ptr(), TURQ_ACT_F32, n);
            dev.synchronize();
            std::vector<float> y6((size_t)m * n);
            yg.download(y6.data(), y6.size() * 4);
            for (size_t i = 0; i < y.size(); i++) {
                const double v = y[i], want = v / (1.0 + std::exp(-v)) * v;
                if (std::fabs(y6[i] - want) > 1e-4 * (1.0 + std::fabs(want))) return fail("forward_gate_up differs from silu(forward) * forward");
            }
            // the whole MLP in one call = down_proj of that product, bit for bit
            turq::LinearX down = turq::linear(n, 64, b0.pp("ffn_down"));
            turq::DeviceBuffer z1(dev, (size_t)m * 64 * 4), z2(dev, (size_t)m * 64 * 4);
            down.qmatmul().forward(yg.ptr(), TURQ_ACT_F32, m, n, z1.ptr(), TURQ_ACT_F32, 64);
            turq::QMatMul::forward_mlp(copy.qmatmul(), copy.qmatmul(), down.qmatmul(), xd.ptr(), TURQ_ACT_F32, m, k, z2.ptr(), TURQ_ACT_F32, 64);
            dev.synchronize();
            std::vector<float> a1((size_t)m * 64), a2((size_t)m * 64);
            z1.download(a1.data(), a1.size() * 4);
            z2.download(a2.data(), a2.size() * 4);
            if (std::memcmp(a1.data(), a2.data(), a1.size() * 4) != 0) return fail("forward_mlp differs from forward_gate_up + forward");
        }

        // embedding rows of the quantized table = rows of its full dequantize
        {
            turq::QTensor table = b0.pp("ffn_gate").get({n, k}, "weight");
            const std::vector<float> full = table.dequantize();
            turq::Embedding emb(table, k);
            const std::vector<uint32_t> ids = {0, (uint32_t)(n - 1), 5, 5};
            const std::vector<float> rows = emb.forward(ids);
            for (size_t i = 0; i < ids.size(); i++)
                if (std::memcmp(rows.data() + i * k, full.data() + (size_t)ids[i] * k, (size_t)k * 4) != 0) return fail("embedding row differs from dequantize");
            try { emb.forward({(uint32_t)n}); return fail("index outside the table accepted"); } catch (const turq::Error &) {}
        }

        // dequantize of the norm weight (F32 tensor) is a copy
        std::vector<float> norm = b0.pp("attn_norm").get({k}, "weight").dequantize();
        std::printf("norm %zu %.9g %.9g\n", norm.size(), norm.front(), norm.back());
        // a dense tensor takes the dense arm of QMatMul::from_arc: a [1, k] weight against one row is the dot product
        {
            turq::QMatMul dense = turq::QMatMul::from_arc(b0.pp("attn_norm").get({k}, "weight"));
            if (!dense.dense()) return fail("dense tensor did not take the dense arm");
            const std::vector<float> one = dense.forward(std::vector<float>(norm.begin(), norm.end()), 1);
            double want = 0.0;
            for (float v : norm) want += (double)v * (double)v;
            if (one.size() != 1 || std::fabs((double)one[0] - want) > 1e-5 * want) return fail("dense arm: wrong dot product");
        }
        // RmsNorm from the same tensor, then checked against the formula
        {
            turq::NormX nx = turq::rms_norm(k, 1e-6, b0.pp("attn_norm"));
            turq::NormX copy = nx;  // NormX is Clone in the reference
            std::vector<float> xs((size_t)2 * k);
            for (size_t i = 0; i < xs.size(); i++) xs[i] = std::cos(0.11f * (float)i) * 3.0f;
            const std::vector<float> ys = copy.forward(xs, 2);
            for (int r = 0; r < 2; r++) {
                double ss = 0.0;
                for (int64_t c = 0; c < k; c++) ss += (double)xs[r * k + c] * (double)xs[r * k + c];
                const double rms = std::sqrt(ss / (double)k + 1e-6);
                for (int64_t c = 0; c < k; c++) {
                    const double w = (double)xs[r * k + c] / rms * (double)norm[c];
                    if (std::fabs((double)ys[r * k + c] - w) > 1e-5 * (std::fabs(w) + 1e-3)) return fail("rms norm differs from the formula");
                }
            }
        }
        // the decoder layer's glue on device tensors: norm -> projection in one call (three rows: the norm runs into scratch, the
        // results are those of the two calls bit for bit; one row: the kernel applies the norm, within 5e-4) and y += x W^T
        {
            turq::NormX nx = turq::rms_norm(k, 1e-6, b0.pp("attn_norm"));
            for (int64_t rows : {(int64_t)3, (int64_t)1}) {
                turq::DeviceBuffer xn(dev, (size_t)rows * k * 4), y1(dev, (size_t)rows * n * 4), y2(dev, (size_t)rows * n * 4);
                nx.forward(xd.ptr(), TURQ_ACT_F32, rows, k, xn.ptr(), TURQ_ACT_F32, k);
                copy.qmatmul().forward(xn.ptr(), TURQ_ACT_F32, rows, k, y1.ptr(), TURQ_ACT_F32, n);
                nx.forward_then({&copy.qmatmul()}, xd.ptr(), TURQ_ACT_F32, rows, k, {y2.ptr()}, TURQ_ACT_F32);
                dev.synchronize();
                std::vector<float> a((size_t)rows * n), b((size_t)rows * n);
                y1.download(a.data(), a.size() * 4);
                y2.download(b.data(), b.size() * 4);
                double num = 0.0, den = 0.0;
                for (size_t i = 0; i < a.size(); i++) {
                    num += ((double)a[i] - b[i]) * ((double)a[i] - b[i]);
                    den += (double)a[i] * a[i];
                }
                if (rows > 1 && std::memcmp(a.data(), b.data(), a.size() * 4) != 0) return fail("forward_then differs from norm + forward");
                if (std::sqrt(num / den) > 5e-4) return fail("forward_then (one row) is not within 5e-4 of norm + forward");
                // y2 += x W^T on top of what it holds
                copy.qmatmul().forward_add(xn.ptr(), TURQ_ACT_F32, rows, k, y2.ptr(), TURQ_ACT_F32, n);
                dev.synchronize();
                std::vector<float> c((size_t)rows * n);
                y2.download(c.data(), c.size() * 4);
                for (size_t i = 0; i < c.size(); i++)
                    if (c[i] != b[i] + a[i]) return fail("forward_add is not the sum of what y held and forward");
            }
        }
    } catch (const std::exception &e) {
        std::fprintf(stderr, "FAIL: exception: %s\n", e.what());
        return 1;
    }
    std::printf("OK\n");
    return 0;
}

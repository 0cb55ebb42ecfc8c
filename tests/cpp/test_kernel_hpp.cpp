// Exercises include/rmi_hip_kernel.hpp (the C++ mirror of the reference's Kernel /
// Layer interface) on a GPU.  The cases are the reference's own unit tests:
// src/ops/kernel/q8_0/mod.rs:74-156 (closed forms, thread partition),
// tests/quantized_inference.rs:233-249 (Q4_K uniform block), plus eight
// std::threads calling one kernel at once, as pool.compute does.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <thread>
#include <vector>

#include "rmi_hip_kernel.hpp"

static int failures = 0;
#define EXPECT(cond)                                                     \
    do {                                                                 \
        if (!(cond)) {                                                   \
            std::printf("FAIL %s:%d %s\n", __FILE__, __LINE__, #cond);   \
            failures++;                                                  \
        }                                                                \
    } while (0)

static std::vector<uint8_t> q8_0_uniform_row(int8_t value, uint16_t scale_f16, int n_blocks = 1) {
    std::vector<uint8_t> row;
    for (int b = 0; b < n_blocks; b++) {
        row.push_back(uint8_t(scale_f16 & 0xff));
        row.push_back(uint8_t(scale_f16 >> 8));
        for (int i = 0; i < 32; i++) row.push_back(uint8_t(value));
    }
    return row;
}

int main() {
    if (rmi_hip_init(0) != RMI_HIP_OK) {
        std::printf("init failed: %s\n", rmi_hip_last_error());
        return 2;
    }
    const uint16_t one = 0x3c00, half = 0x3800;
    std::vector<uint8_t> ones_q(32, 1);
    float one_s = 1.0f;
    {
        auto w = q8_0_uniform_row(1, one);
        rmi::Q8Kernel k(w.data(), w.size(), 32, 1);
        float out = 0;
        k.forward_prequantized(ones_q.data(), &one_s, &out, 32, 1, 0, 1);
        EXPECT(out == 32.0f);
        std::vector<float> x(32, 1.0f);
        k.forward(x.data(), &out, 32, 1);
        EXPECT(std::fabs(out - 32.0f) < 5e-3f && out == 31.998047f);
    }
    {
        auto w = q8_0_uniform_row(1, half);
        rmi::Q8Kernel k(w.data(), w.size(), 32, 1);
        float out = 0;
        k.forward_prequantized(ones_q.data(), &one_s, &out, 32, 1, 0, 1);
        EXPECT(out == 16.0f);
    }
    {
        std::vector<uint8_t> w;
        for (int r = 0; r < 4; r++) {
            auto row = q8_0_uniform_row(1, one);
            w.insert(w.end(), row.begin(), row.end());
        }
        rmi::Q8Kernel k(w.data(), w.size(), 32, 4);
        float a[4] = {0, 0, 0, 0}, b[4] = {0, 0, 0, 0};
        k.forward_prequantized(ones_q.data(), &one_s, a, 32, 4, 0, 2);
        k.forward_prequantized(ones_q.data(), &one_s, b, 32, 4, 1, 2);
        EXPECT(a[0] == 32 && a[1] == 32 && a[2] == 0 && a[3] == 0);
        EXPECT(b[0] == 0 && b[1] == 0 && b[2] == 32 && b[3] == 32);
    }
    {
        // 8 threads, one full output, disjoint slices: every row must be written exactly once
        const size_t n_in = 1024, n_out = 7168, nth = 8;
        std::vector<uint8_t> w;
        for (size_t r = 0; r < n_out; r++) {
            auto row = q8_0_uniform_row(int8_t(r % 7 + 1), one, int(n_in / 32));
            w.insert(w.end(), row.begin(), row.end());
        }
        rmi::Q8Kernel k(w.data(), w.size(), n_in, n_out);
        std::vector<uint8_t> xq(n_in, 1);
        std::vector<float> xs(n_in / 32, 1.0f), out(n_out, -1.0f);
        std::vector<std::thread> pool;
        for (size_t ith = 0; ith < nth; ith++)
            pool.emplace_back([&, ith] { k.forward_prequantized(xq.data(), xs.data(), out.data(), n_in, n_out, ith, nth); });
        for (auto &t : pool) t.join();
        bool ok = true;
        for (size_t r = 0; r < n_out; r++) ok = ok && out[r] == float((r % 7 + 1) * n_in);
        EXPECT(ok);
        // fused == separate
        rmi::Q8Kernel k2(w.data(), w.size() / 2, n_in, n_out / 2);
        auto fused = rmi::fuse_vstack(k2, k2);
        EXPECT(fused.has_value());
        std::vector<float> of(n_out, 0.0f);
        fused->forward_prequantized(xq.data(), xs.data(), of.data(), n_in, n_out, 0, 1);
        ok = true;
        for (size_t r = 0; r < n_out; r++) ok = ok && of[r] == out[r % (n_out / 2)];
        EXPECT(ok);
    }
    {
        std::vector<uint8_t> w(144, 0);
        w[0] = 0x00;
        w[1] = 0x3c;
        const uint8_t sc[12] = {1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1};
        std::memcpy(&w[4], sc, 12);
        std::memset(&w[16], 0x11, 128);
        rmi::Q4_KKernel k(w.data(), w.size(), 256, 1);
        std::vector<uint8_t> xq(256, 1);
        std::vector<float> xs(8, 1.0f);
        float out = 0;
        k.forward_prequantized(xq.data(), xs.data(), &out, 256, 1, 0, 1);
        EXPECT(out == 256.0f);
        auto layer = rmi::QuantizedLinear::from_weight_slice(w.data(), w.size(), nullptr, 256, 1, "ffn");
        std::vector<float> x(256, 1.0f);
        rmi::ExecContext ctx{nullptr, 0, nullptr, 0, 0};
        layer.forward(x.data(), &out, ctx);
        EXPECT(out == 256.0f && layer.input_dim() == 256 && layer.output_dim() == 1);
        // integer path with the kernel quantizing the f32 input itself
        k.forward_prepared(x.data(), nullptr, nullptr, nullptr, &out, 256, 1, 0, 1);
        EXPECT(std::fabs(out - 256.0f) < 1e-3f);
    }
    {
        // error path: shape mismatch throws with the library's message
        auto w = q8_0_uniform_row(1, one);
        rmi::Q8Kernel k(w.data(), w.size(), 32, 1);
        float out;
        bool threw = false;
        try {
            k.forward_prequantized(ones_q.data(), &one_s, &out, 64, 1, 0, 1);
        } catch (const rmi::HipError &e) {
            threw = e.code == RMI_HIP_E_INVALID;
        }
        EXPECT(threw);
    }
    std::printf(failures ? "%d FAILED\n" : "all C++ interface checks passed\n", failures);
    return failures ? 1 : 0;
}

// Exercises include/rmi_hip_kernel.hpp (the C++ mirror of the reference's Kernel /
// Layer interface) on a GPU.  The cases are the reference's own unit tests:
// src/ops/kernel/q8_0/mod.rs:74-156 (closed forms, thread partition),
// tests/quantized_inference.rs:233-263 (Q4_K and Q6_K uniform blocks), plus eight
// std::threads calling one kernel at once, as pool.compute does, and a GGUF file written here and
// read through GGUFLoader (src/core/loader.rs:846-889 in miniature).
#include <unistd.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
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
    {  // tests/quantized_inference.rs:252-263: Q6_K uniform block, ql 0x11, qh 0xaa, scales 1, d 1.0
        std::vector<uint8_t> w(210, 0x11);
        std::memset(&w[128], 0xaa, 64);
        std::memset(&w[192], 1, 16);
        w[208] = uint8_t(one & 0xff);
        w[209] = uint8_t(one >> 8);
        rmi::Q6_KKernel k(w.data(), w.size(), 256, 1);
        std::vector<uint8_t> xq(256, 1);
        std::vector<float> xs(8, 1.0f), x(256, 1.0f);
        float out = 0;
        k.forward_prequantized(xq.data(), xs.data(), &out, 256, 1, 0, 1);
        EXPECT(out == 256.0f);
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
    {
        // device-resident decode of a one-layer toy model: runs, is deterministic, and the tokens it
        // generates are the argmax of the steps that produced them
        const uint32_t n_embd = 64, n_head = 2, n_kv = 1, hd = 32, n_ff = 96, vocab = 40, cap = 24;
        auto q8 = [](uint32_t rows, uint32_t cols, uint32_t seed) {
            std::vector<uint8_t> w(size_t(rows) * (cols / 32) * 34);
            uint32_t s = seed * 2654435761u + 1;
            for (size_t b = 0; b < w.size() / 34; b++) {
                w[b * 34] = 0x00;
                w[b * 34 + 1] = 0x1c;  // f16 0x1c00 = 2^-8
                for (int k = 0; k < 32; k++) {
                    s = s * 1664525u + 1013904223u;
                    w[b * 34 + 2 + k] = uint8_t(int8_t(int(s >> 24) % 100));
                }
            }
            return w;
        };
        auto embd = q8(vocab, n_embd, 1), wq = q8(n_head * hd, n_embd, 2), wk = q8(n_kv * hd, n_embd, 3),
             wv = q8(n_kv * hd, n_embd, 4), wo = q8(n_embd, n_head * hd, 5), wg = q8(n_ff, n_embd, 6),
             wu = q8(n_ff, n_embd, 7), wd = q8(n_embd, n_ff, 8);
        std::vector<float> ones(96, 1.0f);
        const float *norm = ones.data();
        const uint8_t *pq = wq.data(), *pk = wk.data(), *pv = wv.data(), *po = wo.data(), *pg = wg.data(),
                      *pu = wu.data(), *pd = wd.data();
        rmi_hip_qwen3_config cfg{n_embd, 1, n_head, n_kv, hd, hd, n_ff, vocab, cap, 1e-6f, 1e6f, 1, RMI_HIP_ROUND_TIES_EVEN};
        rmi_hip_qwen3_weights wt{embd.data(), nullptr, norm, &norm, &norm, &norm, &norm, &pq, &pk, &pv, &po, &pg, &pu, &pd};
        rmi::Qwen3Session sess(cfg, wt);
        std::vector<uint32_t> prompt = {3, 17, 5, 39, 0, 8}, am1, am2;
        std::vector<float> top;
        auto a = sess.generate(prompt, 10, &am1, &top);
        auto b = sess.generate(prompt, 10, &am2);
        EXPECT(a.size() == 10 && a == b && am1 == am2 && am1.size() == 15);
        bool greedy = true;
        for (size_t i = 0; i < a.size(); i++) greedy = greedy && a[i] == am1[prompt.size() - 1 + i] && a[i] < vocab;
        EXPECT(greedy);
        bool ordered = true;
        for (size_t i = 0; i < am1.size(); i++) ordered = ordered && top[2 * i] >= top[2 * i + 1];
        EXPECT(ordered);
        bool threw = false;
        try {
            sess.generate(prompt, 30);  // beyond the capacity
        } catch (const rmi::HipError &e) {
            threw = e.code == RMI_HIP_E_INVALID;
        }
        EXPECT(threw);
    }
    {
        // GGUFLoader over a file written here: one u32 key, one 32 x 4 Q8_0 tensor of ones (the closed form above),
        // read back through the mapping and uploaded from it
        std::string b = "GGUF";
        auto put = [&b](const void *p, size_t n) { b.append(static_cast<const char *>(p), n); };
        auto put_str = [&](const std::string &t) {
            const uint64_t n = t.size();
            put(&n, 8);
            b += t;
        };
        const uint32_t version = 3, u32_tag = 4, n_dims = 2, ctx = 4096;
        const uint64_t n_tensors = 1, n_kv = 1, dims[2] = {32, 4}, offset = 0;
        const int32_t q8_0 = 8;
        put(&version, 4), put(&n_tensors, 8), put(&n_kv, 8);
        put_str("qwen3.context_length"), put(&u32_tag, 4), put(&ctx, 4);
        put_str("blk.0.attn_q.weight"), put(&n_dims, 4), put(dims, 16), put(&q8_0, 4), put(&offset, 8);
        b.resize((b.size() + 31) / 32 * 32, '\0');
        for (int r = 0; r < 4; r++) {
            auto row = q8_0_uniform_row(1, one);
            b.append(reinterpret_cast<const char *>(row.data()), row.size());
        }
        char path[] = "/tmp/rmi_hip_cpp_XXXXXX";
        const int fd = mkstemp(path);
        EXPECT(fd >= 0 && write(fd, b.data(), b.size()) == ssize_t(b.size()));
        close(fd);
        {
            rmi::GGUFLoader g = rmi::GGUFLoader::from_file(path);
            uint64_t v = 0;
            double f = 0;
            std::string sv;
            EXPECT(g.version() == 3 && g.alignment() == 32 && g.n_tensors() == 1 && g.n_kv() == 1);
            EXPECT(g.to_u64("qwen3.context_length", &v) && v == 4096 && g.to_f64("qwen3.context_length", &f) && f == 4096.0);
            EXPECT(!g.to_u64("absent", &v) && !g.to_string_val("qwen3.context_length", &sv));
            rmi::GGUFLoader::TensorInfo t;
            EXPECT(g.tensor_info("blk.0.attn_q.weight", &t) && t.dims == std::vector<uint64_t>({32, 4}) &&
                   t.ggml_type == 8 && t.nbytes == 136);
            auto slice = g.tensor_slice("blk.0.attn_q.weight");
            EXPECT(slice.second == 136 && slice.first[2] == 1 && g.tensor_slice("absent").first == nullptr);
            rmi::Q8Kernel k(g.upload("blk.0.attn_q.weight"));
            float out[4] = {0, 0, 0, 0};
            k.forward_prequantized(ones_q.data(), &one_s, out, 32, 4, 0, 1);
            EXPECT(out[0] == 32 && out[1] == 32 && out[2] == 32 && out[3] == 32);
            rmi::Q8Kernel k2(g.upload_stack({"blk.0.attn_q.weight", "blk.0.attn_q.weight"}));
            float out8[8] = {0};
            k2.forward_prequantized(ones_q.data(), &one_s, out8, 32, 8, 0, 1);
            EXPECT(out8[0] == 32 && out8[7] == 32);
            bool threw = false;
            try {
                g.upload("absent");
            } catch (const rmi::HipError &e) {
                threw = std::strstr(e.what(), "Missing tensor: absent") != nullptr;
            }
            EXPECT(threw);
        }
        b[3] = 'L';
        FILE *fp = std::fopen(path, "wb");
        std::fwrite(b.data(), 1, b.size(), fp);
        std::fclose(fp);
        bool threw = false;
        try {
            rmi::GGUFLoader::from_file(path);
        } catch (const rmi::HipError &e) {
            threw = std::strstr(e.what(), "Invalid GGUF magic") != nullptr;
        }
        EXPECT(threw);
        std::remove(path);
    }
    std::printf(failures ? "%d FAILED\n" : "all C++ interface checks passed\n", failures);
    return failures ? 1 : 0;
}

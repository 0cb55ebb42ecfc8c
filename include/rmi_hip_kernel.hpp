// rmi_hip_kernel.hpp — C++ host-side mirror of the reference's operator
// interface for the quantized matmul path, header-only over the C ABI of
// rmi_hip.h.  Same method names, argument order and argument meaning as the
// Rust traits it stands in for:
//
//   Kernel            src/ops/kernel/trait_.rs:15-110
//   Q8Kernel          src/ops/kernel/q8_0/mod.rs:21-56
//   Q4_0Kernel        src/ops/kernel/q4_0/mod.rs:18-123
//   Q4_KKernel        src/ops/kernel/q4_k.rs:7-93
//   Q6_KKernel        src/ops/kernel/q6_k.rs:7-80
//   BlockQ8K          src/ops/quant/mod.rs:35-40
//   fuse_vstack       src/ops/kernel/qtensor_owned.rs:138-164
//   Layer, ExecContext, QuantizedLinear   src/core/traits.rs:45-74, src/core/model.rs:12-104
//
// Error behaviour follows the reference's GPU hook: a failing call throws
// (the Rust side panics through `.expect("GPU matmul failed")`,
// src/ops/kernel/q8_0/dispatch.rs:45-48); a failing rmi_hip_init is the
// signal to stay on the CPU kernels (src/ops/float.rs:51-57).
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "rmi_hip.h"

namespace rmi {

struct HipError : std::runtime_error {
    int code;
    HipError(int c, const std::string &what) : std::runtime_error(what), code(c) {}
};

inline void check(int rc) {
    if (rc != RMI_HIP_OK) throw HipError(rc, rmi_hip_last_error());
}

struct BlockQ8K {
    float d;
    int8_t qs[256];
    int16_t bsums[16];
};

// quantize_q8_0_into(input, n, q8, scales) on the device
inline void quantize_q8_0_into(const float *input, size_t n, uint8_t *q8, float *scales,
                               int rounding = RMI_HIP_ROUND_TIES_EVEN) {
    check(rmi_hip_quantize_q8_0(input, uint32_t(n), q8, scales, rounding));
}

// quantize_row_q8_k(x) -> Vec<BlockQ8K> on the device
inline std::vector<BlockQ8K> quantize_row_q8_k(const float *x, size_t n) {
    std::vector<float> d(n / 256);
    std::vector<int8_t> qs(n);
    std::vector<int16_t> bs(n / 16);
    check(rmi_hip_quantize_row_q8_k(x, uint32_t(n), d.data(), qs.data(), bs.data()));
    std::vector<BlockQ8K> out(n / 256);
    for (size_t i = 0; i < out.size(); i++) {
        out[i].d = d[i];
        for (int k = 0; k < 256; k++) out[i].qs[k] = qs[i * 256 + k];
        for (int k = 0; k < 16; k++) out[i].bsums[k] = bs[i * 16 + k];
    }
    return out;
}

// How forward_batched of the Q8_0 and Q4_K kernels multiplies a batch, for the whole process: RMI_HIP_BATCHED_X86_ORDER
// (default: an x86-64 host's bits for every token), RMI_HIP_BATCHED_AARCH64_ORDER, or RMI_HIP_BATCHED_FAST (the fastest
// kernel per product, within the reference's tolerance).  Chosen once at start-up; no call site changes.
inline void set_forward_batched_mode(int mode) {
    if (rmi_hip_set_forward_batched_mode(mode) != RMI_HIP_OK) throw HipError(RMI_HIP_E_INVALID, rmi_hip_last_error());
}

class Kernel {
  public:
    virtual ~Kernel() = default;

    virtual void forward_prequantized(const uint8_t *input_q8, const float *input_scales, float *output, size_t n_in,
                                      size_t n_out, size_t ith, size_t nth) const = 0;

    virtual void forward_prepared(const float *input_f32, const uint8_t *input_q8, const float *input_scales,
                                  const std::vector<BlockQ8K> *q8_k, float *output, size_t n_in, size_t n_out,
                                  size_t ith, size_t nth) const {
        (void)input_f32;
        (void)q8_k;
        forward_prequantized(input_q8, input_scales, output, n_in, n_out, ith, nth);
    }

    virtual void forward(const float *input, float *output, size_t n_in, size_t n_out) const {
        std::vector<uint8_t> q8(n_in);
        std::vector<float> scales((n_in + 31) / 32);
        quantize_q8_0_into(input, n_in, q8.data(), scales.data());
        forward_prepared(input, q8.data(), scales.data(), nullptr, output, n_in, n_out, 0, 1);
    }

    virtual void forward_batched(const float *input, size_t n_tokens, float *output, size_t n_in,
                                 size_t n_out) const {
        for (size_t t = 0; t < n_tokens; t++) forward(input + t * n_in, output + t * n_out, n_in, n_out);
    }
};

class DeviceWeight {
  public:
    explicit DeviceWeight(rmi_hip_weight *h) : h_(h) {
        if (!h_) throw HipError(RMI_HIP_E_INVALID, rmi_hip_last_error());
    }
    ~DeviceWeight() { rmi_hip_free_weight(h_); }
    DeviceWeight(const DeviceWeight &) = delete;
    DeviceWeight &operator=(const DeviceWeight &) = delete;
    rmi_hip_weight *get() const { return h_; }

  private:
    rmi_hip_weight *h_;
};

class Q8Kernel : public Kernel {
  public:
    // the weight slice is copied to HBM here and may be dropped afterwards
    Q8Kernel(const uint8_t *weight, size_t nbytes, size_t n_in, size_t n_out)
        : w_(std::make_shared<DeviceWeight>(rmi_hip_upload_q8_0(weight, nbytes, uint32_t(n_in), uint32_t(n_out)))) {}
    explicit Q8Kernel(std::shared_ptr<DeviceWeight> w) : w_(std::move(w)) {}

    void forward_prequantized(const uint8_t *input_q8, const float *input_scales, float *output, size_t n_in,
                              size_t n_out, size_t ith, size_t nth) const override {
        check(rmi_hip_q8_0_forward_prequantized(w_->get(), input_q8, input_scales, output, uint32_t(n_in),
                                                uint32_t(n_out), uint32_t(ith), uint32_t(nth)));
    }
    void forward(const float *input, float *output, size_t n_in, size_t n_out) const override {
        check(rmi_hip_q8_0_forward_batched(w_->get(), input, output, uint32_t(n_in), uint32_t(n_out), 1,
                                           RMI_HIP_ROUND_TIES_EVEN));
    }
    void forward_batched(const float *input, size_t n_tokens, float *output, size_t n_in,
                         size_t n_out) const override {
        check(rmi_hip_q8_0_forward_batched(w_->get(), input, output, uint32_t(n_in), uint32_t(n_out),
                                           uint32_t(n_tokens), RMI_HIP_ROUND_TIES_EVEN));
    }
    // the prefill path: the same product on the int8 matrix cores in the aarch64 kernel's accumulation order
    void forward_batched_matrix_cores(const float *input, size_t n_tokens, float *output, size_t n_in, size_t n_out,
                                      int rounding = RMI_HIP_ROUND_TIES_EVEN) const {
        check(rmi_hip_q8_0_forward_batched_neon(w_->get(), input, output, uint32_t(n_in), uint32_t(n_out),
                                                uint32_t(n_tokens), rounding));
    }
    const std::shared_ptr<DeviceWeight> &weight() const { return w_; }

  private:
    std::shared_ptr<DeviceWeight> w_;
};

class Q4_0Kernel : public Kernel {
  public:
    Q4_0Kernel(const uint8_t *data, size_t nbytes, size_t n_in, size_t n_out)
        : w_(std::make_shared<DeviceWeight>(rmi_hip_upload_q4_0(data, nbytes, uint32_t(n_in), uint32_t(n_out)))) {}
    explicit Q4_0Kernel(std::shared_ptr<DeviceWeight> w) : w_(std::move(w)) {}

    void forward_prequantized(const uint8_t *input_q8, const float *input_scales, float *output, size_t n_in,
                              size_t n_out, size_t ith, size_t nth) const override {
        check(rmi_hip_q4_0_forward_prequantized(w_->get(), input_q8, input_scales, output, uint32_t(n_in),
                                                uint32_t(n_out), uint32_t(ith), uint32_t(nth)));
    }
    const std::shared_ptr<DeviceWeight> &weight() const { return w_; }

  private:
    std::shared_ptr<DeviceWeight> w_;
};

class Q4_KKernel : public Kernel {
  public:
    Q4_KKernel(const uint8_t *data, size_t nbytes, size_t n_in, size_t n_out)
        : w_(std::make_shared<DeviceWeight>(rmi_hip_upload_q4_k(data, nbytes, uint32_t(n_in), uint32_t(n_out)))) {}
    explicit Q4_KKernel(std::shared_ptr<DeviceWeight> w) : w_(std::move(w)) {}

    void forward_prequantized(const uint8_t *input_q8, const float *input_scales, float *output, size_t n_in,
                              size_t n_out, size_t ith, size_t nth) const override {
        check(rmi_hip_q4_k_forward_prequantized(w_->get(), input_q8, input_scales, output, uint32_t(n_in),
                                                uint32_t(n_out), uint32_t(ith), uint32_t(nth)));
    }
    void forward_prepared(const float *input_f32, const uint8_t *, const float *, const std::vector<BlockQ8K> *q8_k,
                          float *output, size_t n_in, size_t n_out, size_t ith, size_t nth) const override {
        std::vector<BlockQ8K> owned;
        if (!q8_k) {  // q4_k.rs:77-84
            owned = quantize_row_q8_k(input_f32, n_in);
            q8_k = &owned;
        }
        std::vector<float> d(q8_k->size());
        std::vector<int8_t> qs(q8_k->size() * 256);
        std::vector<int16_t> bs(q8_k->size() * 16);
        for (size_t i = 0; i < q8_k->size(); i++) {
            d[i] = (*q8_k)[i].d;
            for (int k = 0; k < 256; k++) qs[i * 256 + k] = (*q8_k)[i].qs[k];
            for (int k = 0; k < 16; k++) bs[i * 16 + k] = (*q8_k)[i].bsums[k];
        }
        check(rmi_hip_q4_k_forward_prepared(w_->get(), d.data(), qs.data(), bs.data(), output, uint32_t(n_in),
                                            uint32_t(n_out), uint32_t(ith), uint32_t(nth)));
    }
    const std::shared_ptr<DeviceWeight> &weight() const { return w_; }

  private:
    std::shared_ptr<DeviceWeight> w_;
};

class Q6_KKernel : public Kernel {
  public:
    Q6_KKernel(const uint8_t *data, size_t nbytes, size_t n_in, size_t n_out)
        : w_(std::make_shared<DeviceWeight>(rmi_hip_upload_q6_k(data, nbytes, uint32_t(n_in), uint32_t(n_out)))) {}
    explicit Q6_KKernel(std::shared_ptr<DeviceWeight> w) : w_(std::move(w)) {}

    void forward_prequantized(const uint8_t *input_q8, const float *input_scales, float *output, size_t n_in,
                              size_t n_out, size_t ith, size_t nth) const override {
        check(rmi_hip_q6_k_forward_prequantized(w_->get(), input_q8, input_scales, output, uint32_t(n_in),
                                                uint32_t(n_out), uint32_t(ith), uint32_t(nth)));
    }
    void forward_prepared(const float *input_f32, const uint8_t *, const float *, const std::vector<BlockQ8K> *q8_k,
                          float *output, size_t n_in, size_t n_out, size_t ith, size_t nth) const override {
        std::vector<BlockQ8K> owned;
        if (!q8_k) {  // q6_k.rs:63-69
            owned = quantize_row_q8_k(input_f32, n_in);
            q8_k = &owned;
        }
        std::vector<float> d(q8_k->size());
        std::vector<int8_t> qs(q8_k->size() * 256);
        std::vector<int16_t> bs(q8_k->size() * 16);
        for (size_t i = 0; i < q8_k->size(); i++) {
            d[i] = (*q8_k)[i].d;
            for (int k = 0; k < 256; k++) qs[i * 256 + k] = (*q8_k)[i].qs[k];
            for (int k = 0; k < 16; k++) bs[i * 16 + k] = (*q8_k)[i].bsums[k];
        }
        check(rmi_hip_q6_k_forward_prepared(w_->get(), d.data(), qs.data(), bs.data(), output, uint32_t(n_in),
                                            uint32_t(n_out), uint32_t(ith), uint32_t(nth)));
    }
    const std::shared_ptr<DeviceWeight> &weight() const { return w_; }

  private:
    std::shared_ptr<DeviceWeight> w_;
};

// QTensorOwned::fuse_vstack: None (nullopt) when dtype or n_in differ
template <class K>
std::optional<K> fuse_vstack(const K &a, const K &b) {
    rmi_hip_weight *h = rmi_hip_fuse_vstack(a.weight()->get(), b.weight()->get());
    if (!h) return std::nullopt;
    return K(std::make_shared<DeviceWeight>(h));
}

struct ExecContext {
    float *scratch;        // accepted for signature parity; the GPU path dequantises in registers
    size_t scratch_len;
    void *kv_cache;
    uint32_t pos;
    uint32_t layer_idx;
};

class Layer {
  public:
    virtual ~Layer() = default;
    virtual void forward(const float *input, float *output, ExecContext &ctx) const = 0;
    virtual size_t input_dim() const = 0;
    virtual size_t output_dim() const = 0;
    virtual const char *name() const = 0;
};

class QuantizedLinear : public Layer {
  public:
    static QuantizedLinear from_weight_slice(const uint8_t *weight, size_t nbytes, const uint8_t *bias,
                                             size_t in_features, size_t out_features, std::string name) {
        (void)bias;  // ignored by the reference as well (src/core/model.rs:14-16)
        return QuantizedLinear(weight, nbytes, in_features, out_features, std::move(name));
    }
    void forward_dequant(const float *input, float *output) const {
        check(rmi_hip_quantized_linear_forward(w_.get(), input, output, uint32_t(in_), uint32_t(out_)));
    }
    void forward(const float *input, float *output, ExecContext &) const override { forward_dequant(input, output); }
    size_t input_dim() const override { return in_; }
    size_t output_dim() const override { return out_; }
    const char *name() const override { return name_.c_str(); }

  private:
    QuantizedLinear(const uint8_t *weight, size_t nbytes, size_t in_features, size_t out_features, std::string name)
        : w_(rmi_hip_upload_q4_k(weight, nbytes, uint32_t(in_features), uint32_t(out_features))),
          in_(in_features), out_(out_features), name_(std::move(name)) {}
    DeviceWeight w_;
    size_t in_, out_;
    std::string name_;
};

// GGUFLoader (src/core/loader.rs:187-372) over the library's parser: the TensorSource a model is built from,
// plus the uploads that take a tensor from the file's mapping to HBM.
class GGUFLoader {
  public:
    struct TensorInfo {  // src/core/tensor.rs:189-195
        std::string name;
        std::vector<uint64_t> dims;  // [columns, rows, ..]
        int ggml_type;
        uint64_t offset, nbytes;
    };
    // GGUFLoader::from_file; the message of a file the reference rejects is the reference's
    static GGUFLoader from_file(const std::string &path) {
        rmi_hip_gguf *g = rmi_hip_gguf_open(path.c_str());
        if (!g) throw HipError(RMI_HIP_E_INVALID, rmi_hip_last_error());
        return GGUFLoader(g);
    }
    GGUFLoader(GGUFLoader &&o) noexcept : g_(o.g_) { o.g_ = nullptr; }
    GGUFLoader(const GGUFLoader &) = delete;
    GGUFLoader &operator=(const GGUFLoader &) = delete;
    ~GGUFLoader() { rmi_hip_gguf_close(g_); }

    uint32_t version() const { return rmi_hip_gguf_version(g_); }
    uint64_t alignment() const { return rmi_hip_gguf_alignment(g_); }
    size_t data_offset() const { return size_t(rmi_hip_gguf_data_offset(g_)); }
    size_t n_tensors() const { return size_t(rmi_hip_gguf_n_tensors(g_)); }
    size_t n_kv() const { return size_t(rmi_hip_gguf_n_kv(g_)); }
    // metadata(key).and_then(MetaValue::to_u64) and its siblings: false where the reference gives None
    bool to_u64(const std::string &key, uint64_t *out) const { return rmi_hip_gguf_meta_u64(g_, key.c_str(), out) != 0; }
    bool to_f64(const std::string &key, double *out) const { return rmi_hip_gguf_meta_f64(g_, key.c_str(), out) != 0; }
    bool to_string_val(const std::string &key, std::string *out) const {
        const int64_t n = rmi_hip_gguf_meta_str(g_, key.c_str(), nullptr, 0);
        if (n < 0) return false;
        out->assign(size_t(n) + 1, '\0');
        rmi_hip_gguf_meta_str(g_, key.c_str(), &(*out)[0], size_t(n) + 1);
        out->resize(size_t(n));
        return true;
    }
    bool tensor_info(const std::string &name, TensorInfo *out) const {
        const int64_t i = rmi_hip_gguf_find_tensor(g_, name.c_str());
        if (i < 0) return false;
        const char *nm;
        uint32_t nd;
        uint64_t dims[8];
        check(rmi_hip_gguf_tensor_info(g_, uint64_t(i), &nm, &nd, dims, 8, &out->ggml_type, &out->offset, &out->nbytes));
        out->name = nm;
        out->dims.assign(dims, dims + nd);
        return true;
    }
    // tensor_slice: the bytes in the mapping, valid while the loader lives; {nullptr, 0} for an unknown name
    std::pair<const uint8_t *, size_t> tensor_slice(const std::string &name) const {
        TensorInfo t;
        if (!tensor_info(name, &t)) return {nullptr, 0};
        return {rmi_hip_gguf_tensor_data(g_, uint64_t(rmi_hip_gguf_find_tensor(g_, name.c_str()))), size_t(t.nbytes)};
    }
    // one matrix, or several of one type and width stacked row-wise ([q ; k ; v]), as a weight in HBM
    std::shared_ptr<DeviceWeight> upload_stack(const std::vector<std::string> &names) const {
        std::vector<const char *> p;
        for (const std::string &n : names) p.push_back(n.c_str());
        return std::make_shared<DeviceWeight>(rmi_hip_gguf_upload_stack(g_, p.data(), int(p.size())));
    }
    std::shared_ptr<DeviceWeight> upload(const std::string &name) const { return upload_stack({name}); }
    rmi_hip_qwen3_config qwen3_config(uint32_t capacity, int rounding = RMI_HIP_ROUND_TIES_EVEN) const {
        rmi_hip_qwen3_config c;
        check(rmi_hip_gguf_qwen3_config(g_, capacity, rounding, &c));
        return c;
    }
    rmi_hip_gguf *get() const { return g_; }

  private:
    explicit GGUFLoader(rmi_hip_gguf *g) : g_(g) {}
    rmi_hip_gguf *g_;
};

// Qwen3Session (src/models/qwen3.rs:581-1158) with the whole token step on the device.
class Qwen3Session {
  public:
    Qwen3Session(const rmi_hip_qwen3_config &cfg, const rmi_hip_qwen3_weights &weights)
        : cfg_(cfg), h_(rmi_hip_qwen3_create(&cfg, &weights)) {
        if (!h_) throw HipError(RMI_HIP_E_RUNTIME, rmi_hip_last_error());
    }
    // Qwen3Model::from_source + Qwen3Session::new over an open file: tensor bytes go from its mapping to HBM
    Qwen3Session(const GGUFLoader &source, uint32_t capacity, int rounding = RMI_HIP_ROUND_TIES_EVEN)
        : cfg_(source.qwen3_config(capacity, rounding)), h_(rmi_hip_qwen3_create_from_gguf(source.get(), capacity, rounding)) {
        if (!h_) throw HipError(RMI_HIP_E_RUNTIME, rmi_hip_last_error());
    }
    ~Qwen3Session() { rmi_hip_qwen3_destroy(h_); }
    Qwen3Session(const Qwen3Session &) = delete;
    Qwen3Session &operator=(const Qwen3Session &) = delete;
    // greedy generation; per step the argmax and the two largest logits if the vectors are given
    std::vector<uint32_t> generate(const std::vector<uint32_t> &prompt, uint32_t max_new,
                                   std::vector<uint32_t> *step_argmax = nullptr, std::vector<float> *step_top2 = nullptr,
                                   double *seconds = nullptr) {
        const size_t steps = prompt.size() + max_new - 1;
        std::vector<uint32_t> out(max_new);
        if (step_argmax) step_argmax->assign(steps, 0);
        if (step_top2) step_top2->assign(2 * steps, 0.0f);
        const int n = rmi_hip_qwen3_generate(h_, prompt.data(), uint32_t(prompt.size()), max_new, out.data(),
                                             step_argmax ? step_argmax->data() : nullptr,
                                             step_top2 ? step_top2->data() : nullptr, nullptr, 0, nullptr, seconds);
        check(n < 0 ? n : 0);
        out.resize(size_t(n));
        return out;
    }
    const rmi_hip_qwen3_config &config() const { return cfg_; }

  private:
    rmi_hip_qwen3_config cfg_;
    rmi_hip_qwen3 *h_;
};

}  // namespace rmi

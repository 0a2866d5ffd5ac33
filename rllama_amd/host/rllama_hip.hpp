// rllama_hip.hpp -- host-side mirror of the reference's model API over the C ABI (include/rllama_hip.h).
//
// The reference's host code is Rust (Noeda/rllama src/transformer.rs, src/tensor.rs); where no Rust toolchain
// is available this header plays its part: same type names, same method names and argument meaning, same
// failure behaviour (the reference panics / unwraps; these methods throw rllama::Error), no arithmetic of
// its own.  Header-only, C++17, links against librllama_hip.so.
//
//   rllama::OpenCL        <- OpenCL (src/tensor_opencl_support.rs:40-58): the device context (here a HIP device)
//   rllama::DataSettings  <- DataSettings (src/transformer.rs:38-109)
//   rllama::Transformer   <- Transformer (src/transformer.rs:17-34, 240-383)
//   rllama::TransformerCaches <- TransformerCaches (src/transformer.rs:111-113, 200-214)
//   rllama::Tensor        <- the device-resident subset of Tensor (src/tensor.rs:92-112; OpenCLTensor)
#pragma once

#include "../../include/rllama_hip.h"

#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace rllama {

using TokenId = int32_t; // src/tokenizer.rs

struct Error : std::runtime_error {
    int code;
    Error(int c, const std::string &what) : std::runtime_error(what), code(c) {}
};

inline void check(int rc) {
    if (rc != RLH_OK) throw Error(rc, rlh_last_error());
}

enum class TensorDType { Float16 = RLH_F16, Float32 = RLH_F32 }; // src/tensor.rs:50-54

// OpenCL::new(verbose, nth_device) (src/tensor_opencl_support.rs:86)
class OpenCL {
  public:
    OpenCL(bool verbose, size_t nth_device) { check(rlh_init((int)nth_device, verbose ? 1 : 0, &ctx_)); }
    ~OpenCL() { rlh_shutdown(ctx_); }
    OpenCL(const OpenCL &) = delete;
    OpenCL &operator=(const OpenCL &) = delete;
    void flush() { check(rlh_sync(ctx_)); } // src/tensor_opencl_support.rs:130
    rlh_ctx *raw() const { return ctx_; }

  private:
    rlh_ctx *ctx_ = nullptr;
};

// DataSettings (src/transformer.rs:38-109): builder-style, cheap to copy
class DataSettings {
  public:
    explicit DataSettings(std::shared_ptr<OpenCL> cl) : cl_(std::move(cl)) {}
    DataSettings force_f16() const {
        DataSettings d = *this;
        d.force_f16_ = true;
        return d;
    }
    DataSettings percentage_to_gpu(float percentage) const { // clamped by the library like :91-103
        DataSettings d = *this;
        d.percentage_to_gpu_ = percentage;
        return d;
    }
    const std::shared_ptr<OpenCL> &cl() const { return cl_; }
    bool is_force_f16() const { return force_f16_; }
    float get_percentage_to_gpu() const { return percentage_to_gpu_; }

  private:
    std::shared_ptr<OpenCL> cl_;
    bool force_f16_ = false;
    float percentage_to_gpu_ = 1.0f;
};

class Transformer;

// TransformerCaches (src/transformer.rs:111-113, 200-214); the KV cache lives in HBM
class TransformerCaches {
  public:
    ~TransformerCaches() { rlh_caches_free(h_); }
    TransformerCaches(TransformerCaches &&o) noexcept : cl_(std::move(o.cl_)), h_(o.h_) { o.h_ = nullptr; }
    TransformerCaches(const TransformerCaches &) = delete; // like the reference, copying is explicit: true_clone()
    TransformerCaches true_clone() const {
        rlh_caches *c = nullptr;
        check(rlh_caches_true_clone(h_, &c));
        return TransformerCaches(cl_, c);
    }
    void shift_left(size_t shifts) { check(rlh_caches_shift_left(h_, (int)shifts)); }
    rlh_caches *raw() const { return h_; }

  private:
    friend class Transformer;
    TransformerCaches(std::shared_ptr<OpenCL> cl, rlh_caches *h) : cl_(std::move(cl)), h_(h) {}
    std::shared_ptr<OpenCL> cl_; // keeps the context alive
    rlh_caches *h_ = nullptr;
};

// Transformer (src/transformer.rs:17-34).  from_unpickled's job -- reading params.json and the weight files --
// stays with the caller; this type receives the hyper-parameters and the tensors one by one.
class Transformer {
  public:
    Transformer(size_t dim, size_t n_layers, size_t n_heads, size_t ffn_hidden, size_t vocab_size, size_t max_seq_len, double eps,
                const DataSettings &data_settings)
        : cl_(data_settings.cl()), vocab_size_(vocab_size) {
        rlh_model_params p{};
        p.dim = (int32_t)dim;
        p.n_layers = (int32_t)n_layers;
        p.n_heads = (int32_t)n_heads;
        p.ffn_hidden = (int32_t)ffn_hidden;
        p.vocab_size = (int32_t)vocab_size;
        p.max_seq_len = (int32_t)max_seq_len;
        p.norm_eps = eps;
        p.force_f16 = data_settings.is_force_f16() ? 1 : 0;
        p.percentage_to_gpu = data_settings.get_percentage_to_gpu();
        check(rlh_model_create(cl_->raw(), &p, &h_));
    }
    ~Transformer() { rlh_model_free(h_); }
    Transformer(const Transformer &) = delete;
    Transformer &operator=(const Transformer &) = delete;

    // One weight, dense row-major; f16 sources are the raw bits of consolidated.NN/data/<k>
    void set_tensor(rlh_tensor_kind kind, int layer, const void *data, int rows, int cols, TensorDType src) {
        check(rlh_model_set_tensor(h_, kind, layer, data, rows, cols, (int)src));
    }
    void fill_synthetic(uint64_t seed, double std) { check(rlh_model_fill_synthetic(h_, seed, std)); }

    TransformerCaches make_caches() const { // src/transformer.rs:328-341
        rlh_caches *c = nullptr;
        check(rlh_caches_create(h_, &c));
        return TransformerCaches(cl_, c);
    }

    // forward(tokens, start_pos, caches) -> logits [vocab] (src/transformer.rs:343-383)
    std::vector<float> forward(const std::vector<TokenId> &tokens, size_t start_pos, TransformerCaches &caches) const {
        std::vector<float> logits(vocab_size_);
        check(rlh_forward(h_, caches.raw(), tokens.data(), (int)tokens.size(), (int)start_pos, logits.data()));
        return logits;
    }
    // forward + TokenSampler::sample at top_k = 1 (src/token_sampler.rs:83-174), argmax on the device
    TokenId forward_greedy(const std::vector<TokenId> &tokens, size_t start_pos, TransformerCaches &caches) const {
        TokenId next = 0;
        check(rlh_forward_greedy(h_, caches.raw(), tokens.data(), (int)tokens.size(), (int)start_pos, &next));
        return next;
    }
    // the token loop of command_line_inference (src/rllama_main.rs:821-897) at top_k = 1
    std::vector<TokenId> generate_greedy(const std::vector<TokenId> &prompt, size_t n_new, TransformerCaches &caches, float *ms_first = nullptr,
                                         float *ms_per_token = nullptr) const {
        std::vector<TokenId> out(n_new);
        check(rlh_generate_greedy(h_, caches.raw(), prompt.data(), (int)prompt.size(), (int)n_new, out.data(), ms_first, ms_per_token));
        return out;
    }
    // forward + TokenSampler::sample: the body of the token loop (src/rllama_main.rs:846-860)
    std::pair<TokenId, float> forward_sample(const std::vector<TokenId> &tokens, size_t start_pos, TransformerCaches &caches, const rlh_sampler_params &sampler,
                                             const std::vector<TokenId> &existing_tokens, float u) const {
        TokenId tok = 0;
        float prob = 0.0f;
        check(rlh_forward_sample(h_, caches.raw(), tokens.data(), (int)tokens.size(), (int)start_pos, &sampler, existing_tokens.data(),
                                 (int)existing_tokens.size(), u, &tok, &prob));
        return {tok, prob};
    }
    // The blocks first_layer..=last_layer on the rows of the residual stream x [n x dim] (the loop body of src/transformer.rs:361-376
    // for the layers percentage_to_gpu keeps on the device, :262-279); the host-side blocks, norm and head are the caller's.
    std::vector<float> forward_layers(const std::vector<float> &x, size_t n, size_t start_pos, TransformerCaches &caches, int first_layer,
                                      int last_layer) const {
        std::vector<float> out(x.size());
        check(rlh_forward_layers(h_, caches.raw(), x.data(), (int)n, (int)start_pos, first_layer, last_layer, out.data()));
        return out;
    }
    int last_layer_on_gpu() const { // src/transformer.rs:266-268
        int v = 0;
        check(rlh_model_layers_on_gpu(h_, &v));
        return v;
    }
    rlh_model *raw() const { return h_; }

  private:
    std::shared_ptr<OpenCL> cl_;
    rlh_model *h_ = nullptr;
    size_t vocab_size_;
};

// TokenSampler (src/token_sampler.rs:6-174): builder-style settings; the arithmetic is the library's (host code).
// The uniform variate of the draw comes from the caller (the reference uses rand::thread_rng).
class TokenSampler {
  public:
    TokenSampler() { rlh_sampler_default(&p_); } // TokenSampler::new(), :20-29
    TokenSampler temperature(float v) const { TokenSampler t = *this; t.p_.temperature = v; return t; }
    TokenSampler top_p(float v) const { TokenSampler t = *this; t.p_.top_p = v; return t; }
    TokenSampler top_k(size_t v) const { TokenSampler t = *this; t.p_.top_k = v > 0x7fffffffu ? 0x7fffffff : (int32_t)v; return t; }
    TokenSampler repetition_penalty(float v) const { TokenSampler t = *this; t.p_.repetition_penalty = v; return t; }
    float get_temperature() const { return p_.temperature; }
    float get_top_p() const { return p_.top_p; }
    size_t get_top_k() const { return (size_t)p_.top_k; }
    float get_repetition_penalty() const { return p_.repetition_penalty; }
    // sample(logits, tokenizer, existing_tokens) -> (token, probability) (:83-174); u in [0, 1]
    std::pair<TokenId, float> sample(const std::vector<float> &logits, const std::vector<TokenId> &existing_tokens, float u) const {
        TokenId tok = 0;
        float prob = 0.0f;
        check(rlh_sample(logits.data(), (int)logits.size(), &p_, existing_tokens.data(), (int)existing_tokens.size(), u, &tok, &prob));
        return {tok, prob};
    }
    const rlh_sampler_params &raw() const { return p_; }

  private:
    rlh_sampler_params p_;
};

// Device tensor with the op set of OpenCLTensor (src/tensor_opencl_support.rs:215-405)
class Tensor {
  public:
    // to_gpu_inplace (src/tensor.rs:2127-2147): host data [rows x cols], row stride cols_capacity elements
    Tensor(const std::shared_ptr<OpenCL> &cl, const void *host, int64_t rows, int64_t cols, int64_t cols_capacity, TensorDType dtype)
        : cl_(cl), rows_(rows), cols_(cols), dtype_(dtype) {
        check(rlh_tensor_upload(cl_->raw(), host, (int)rows, (int)cols, (int)cols_capacity, (int)dtype, &h_));
    }
    static Tensor zeros(const std::shared_ptr<OpenCL> &cl, int64_t rows, int64_t cols, TensorDType dtype) {
        rlh_tensor *t = nullptr;
        check(rlh_tensor_alloc(cl->raw(), (int)rows, (int)cols, (int)dtype, &t));
        return Tensor(cl, t, rows, cols, dtype);
    }
    ~Tensor() { rlh_tensor_free(h_); }
    Tensor(Tensor &&o) noexcept : cl_(std::move(o.cl_)), h_(o.h_), rows_(o.rows_), cols_(o.cols_), dtype_(o.dtype_) { o.h_ = nullptr; }
    Tensor(const Tensor &) = delete; // Tensor::clone of a GPU tensor panics in the reference (src/tensor.rs:126-129)

    int64_t rows() const { return rows_; }
    int64_t cols() const { return cols_; }
    TensorDType dtype() const { return dtype_; }

    void to_cpu(void *host, int64_t cols_capacity) const { check(rlh_tensor_download(h_, host, (int)cols_capacity, nullptr)); }
    Tensor transpose() const {
        Tensor out = zeros(cl_, cols_, rows_, dtype_);
        check(rlh_transpose_from(out.h_, h_));
        return out;
    }
    Tensor silu() const {
        Tensor out = zeros(cl_, rows_, cols_, dtype_);
        check(rlh_copy_inplace(out.h_, h_));
        check(rlh_silu_inplace(out.h_));
        return out;
    }
    Tensor hadamard_product(const Tensor &other) const {
        Tensor out = zeros(cl_, rows_, cols_, dtype_);
        check(rlh_copy_inplace(out.h_, h_));
        check(rlh_hadamard_product_inplace(out.h_, other.h_));
        return out;
    }
    Tensor matrix_mul_transposed(const Tensor &other) const { // src/tensor.rs:999-1025
        Tensor out = zeros(cl_, rows_, other.rows_, dtype_);
        check(rlh_matrix_mul_inplace_transposed(out.h_, h_, other.h_));
        return out;
    }

  private:
    Tensor(std::shared_ptr<OpenCL> cl, rlh_tensor *h, int64_t r, int64_t c, TensorDType d) : cl_(std::move(cl)), h_(h), rows_(r), cols_(c), dtype_(d) {}
    std::shared_ptr<OpenCL> cl_;
    rlh_tensor *h_ = nullptr;
    int64_t rows_ = 0, cols_ = 0;
    TensorDType dtype_ = TensorDType::Float16;
};

} // namespace rllama

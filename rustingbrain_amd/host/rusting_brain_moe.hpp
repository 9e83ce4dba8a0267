// C++ host-side mirror of RustingBrain's mixture-of-experts interface over the C ABI
// of librbmoe (include/rbmoe.h).  Header-only, C++17.
//
// Names, argument meaning and error behaviour follow the reference:
//   Matrix        reference src/matrix.rs:13-18          (row-major f32)
//   Layout        reference src/batch.rs:224-269
//   MoeConfig     reference src/moe.rs:25-87
//   MoeLayer      reference src/moe.rs:203-341, :348-489   (forward, forward_train, backward)
//   MoeCache      reference src/moe.rs:131-188
//   NetworkError  reference src/network.rs:19-83          (the variants this path raises)
//   TransformerBuilder (the methods that size the sparse layers) reference src/transformer.rs:278-447
// All arithmetic happens in the HIP library; this header only marshals host buffers.
#pragma once

#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/rbmoe.h"

namespace rusting_brain {

// ------------------------------------------------------------------ errors
struct NetworkError : std::runtime_error {
    using std::runtime_error::runtime_error;
};
struct InvalidInput : NetworkError {
    size_t expected, actual;
    InvalidInput(const std::string& m, size_t e = 0, size_t a = 0) : NetworkError(m), expected(e), actual(a) {}
};
struct InvalidConfig : NetworkError { using NetworkError::NetworkError; };
struct DeviceError : NetworkError { using NetworkError::NetworkError; };          // NetworkError::Cuda
struct BackendUnavailable : NetworkError { using NetworkError::NetworkError; };   // CudaFeatureDisabled
struct MemoryBudget : NetworkError { using NetworkError::NetworkError; };         // CudaMemoryBudget
struct OutOfMemory : NetworkError { using NetworkError::NetworkError; };          // CudaOutOfMemory
struct Unsupported : NetworkError { using NetworkError::NetworkError; };          // UnsupportedCuda

inline void check(int rc, const rbmoe_ctx* ctx = nullptr) {
    if (rc == RBMOE_OK) return;
    const char* m = ctx ? rbmoe_last_error(ctx) : rbmoe_last_global_error();
    const std::string msg = m && *m ? m : "rbmoe status " + std::to_string(rc);
    switch (rc) {
        case RBMOE_INVALID_INPUT:
        case RBMOE_NULL_POINTER: throw InvalidInput(msg);
        case RBMOE_INVALID_CONFIG: throw InvalidConfig(msg);
        case RBMOE_BACKEND_UNAVAILABLE: throw BackendUnavailable(msg);
        case RBMOE_MEMORY_BUDGET: throw MemoryBudget(msg);
        case RBMOE_OUT_OF_MEMORY: throw OutOfMemory(msg);
        case RBMOE_UNSUPPORTED: throw Unsupported(msg);
        default: throw DeviceError(msg);
    }
}

// ------------------------------------------------------------------ plain data
struct Matrix {
    size_t rows = 0, cols = 0;
    std::vector<float> data;
    Matrix() = default;
    Matrix(size_t r, size_t c) : rows(r), cols(c), data(r * c, 0.0f) {}
    static Matrix from_vec(size_t r, size_t c, std::vector<float> v) {
        if (v.size() != r * c) throw InvalidInput("data length does not match the shape", r * c, v.size());
        Matrix m;
        m.rows = r;
        m.cols = c;
        m.data = std::move(v);
        return m;
    }
    float* row_mut(size_t r) { return data.data() + r * cols; }
    const float* row(size_t r) const { return data.data() + r * cols; }
};

struct Layout {
    size_t seq_len = 0;              // 0 = the whole matrix is one sequence
    const std::vector<bool>* valid = nullptr;  // nullptr = every row is a real token
    bool is_valid(size_t row) const { return !valid || (*valid)[row]; }
    void check(size_t rows) const {
        const size_t s = seq_len ? seq_len : (rows ? rows : 1);
        if (rows % s != 0)
            throw InvalidConfig(std::to_string(rows) + " rows do not divide into sequences of " + std::to_string(s));
        if (valid && valid->size() != rows)
            throw InvalidConfig("padding mask covers " + std::to_string(valid->size()) + " rows, not " + std::to_string(rows));
    }
};

constexpr float DEFAULT_AUX_LOSS_WEIGHT = 0.01f;
constexpr float DEFAULT_ROUTER_Z_LOSS_WEIGHT = 1e-3f;
constexpr int UNROUTED = -1;  // usize::MAX in the reference

struct MoeConfig {
    size_t num_experts, experts_per_token, d_ff;
    bool shared_expert = false;
    float aux_loss_weight = DEFAULT_AUX_LOSS_WEIGHT;
    float router_z_loss_weight = DEFAULT_ROUTER_Z_LOSS_WEIGHT;

    MoeConfig(size_t n, size_t k, size_t f) : num_experts(n), experts_per_token(k), d_ff(f) {}
    MoeConfig with_shared_expert(bool b) const { MoeConfig c = *this; c.shared_expert = b; return c; }
    MoeConfig with_aux_loss_weight(float w) const { MoeConfig c = *this; c.aux_loss_weight = w; return c; }
    MoeConfig with_router_z_loss_weight(float w) const { MoeConfig c = *this; c.router_z_loss_weight = w; return c; }

    rbmoe_config raw(size_t d_model, int act = RBMOE_F32, int weight = RBMOE_F32, size_t max_tokens = 0,
                     size_t shared_d_ff = 0) const {
        rbmoe_config c;
        rbmoe_config_init(&c, (int32_t)d_model, (int32_t)num_experts, (int32_t)experts_per_token, (int32_t)d_ff);
        c.shared_expert = shared_expert ? 1 : 0;
        c.shared_d_ff = (int32_t)shared_d_ff;
        c.aux_loss_weight = aux_loss_weight;
        c.router_z_loss_weight = router_z_loss_weight;
        c.act_dtype = act;
        c.weight_dtype = weight;
        c.max_tokens = (int32_t)max_tokens;
        return c;
    }
    void validate() const {
        const rbmoe_config c = raw(1);
        char msg[256] = {0};
        const int rc = rbmoe_validate(&c, msg, sizeof msg);
        if (rc == RBMOE_OK) return;
        if (rc == RBMOE_INVALID_CONFIG) throw InvalidConfig(msg);
        throw Unsupported(msg);
    }
};

// ------------------------------------------------------------------ device
class Device {
  public:
    explicit Device(int index = 0, size_t budget_mib = 0) { check(rbmoe_ctx_create(index, budget_mib, &ctx_)); }
    static std::shared_ptr<Device> open(int index = 0, size_t budget_mib = 0) {
        return std::make_shared<Device>(index, budget_mib);
    }
    ~Device() { rbmoe_ctx_destroy(ctx_); }
    Device(const Device&) = delete;
    Device& operator=(const Device&) = delete;
    void synchronize() { check(rbmoe_synchronize(ctx_), ctx_); }
    rbmoe_ctx* raw() const { return ctx_; }

  private:
    rbmoe_ctx* ctx_ = nullptr;
};

// ------------------------------------------------------------------ cache
struct MoeCache {
    std::vector<std::pair<int, float>> assignments;  // slot = token * k + rank -> (expert or UNROUTED, gate)
    std::vector<std::vector<size_t>> expert_tokens, expert_slots;
    Matrix probabilities;
    std::vector<float> log_sum_exp;
    size_t valid_tokens = 0;
    float aux = 0.0f, z = 0.0f;

    float aux_loss() const { return aux; }
    float z_loss() const { return z; }
    float auxiliary_loss() const { return aux + z; }
    std::vector<float> load_fractions() const {
        size_t routed = 0;
        for (const auto& v : expert_tokens) routed += v.size();
        const float slots = (float)(routed ? routed : 1);
        std::vector<float> f;
        for (const auto& v : expert_tokens) f.push_back((float)v.size() / slots);
        return f;
    }
};

// ------------------------------------------------------------------ layer
class MoeLayer {
  public:
    MoeConfig config;

    // MoeLayer::new: validates, then creates the device layer (weights start at zero).
    MoeLayer(size_t d_model, const MoeConfig& cfg, std::shared_ptr<Device> device, size_t max_tokens = 1024,
             int act_dtype = RBMOE_F32, int weight_dtype = RBMOE_F32, size_t shared_d_ff = 0)
        : config(cfg), d_model_(d_model), device_(std::move(device)), act_(act_dtype), shared_d_ff_(shared_d_ff) {
        cfg.validate();
        const rbmoe_config c = cfg.raw(d_model, act_dtype, weight_dtype, max_tokens, shared_d_ff);
        check(rbmoe_layer_create(device_->raw(), &c, &layer_), device_->raw());
    }
    ~MoeLayer() { rbmoe_layer_destroy(layer_); }
    MoeLayer(const MoeLayer&) = delete;
    MoeLayer& operator=(const MoeLayer&) = delete;

    size_t d_model() const { return d_model_; }

    void set_router(const Matrix& w) { set(RBMOE_W_ROUTER, 0, w); }
    void set_expert(size_t e, const Matrix& gate, const Matrix& up, const Matrix& down) {
        set(RBMOE_W_GATE, (int)e, gate);
        set(RBMOE_W_UP, (int)e, up);
        set(RBMOE_W_DOWN, (int)e, down);
    }
    void set_shared(const Matrix& gate, const Matrix& up, const Matrix& down) {
        set(RBMOE_W_SHARED_GATE, 0, gate);
        set(RBMOE_W_SHARED_UP, 0, up);
        set(RBMOE_W_SHARED_DOWN, 0, down);
    }

    // One weight matrix by its id (RBMOE_W_*): f32 values, or the int8 values and per-row scales of a quantized
    // checkpoint as they are stored (DeviceParam::new, src/gpu_transformer.rs:471-490).
    void set_weight(int which, int expert, const Matrix& w) { set(which, expert, w); }
    void set_weight_q8(int which, int expert, const int8_t* q, const float* scales, size_t rows, size_t cols) {
        check(rbmoe_set_weight(layer_, which, expert, q, RBMOE_I8, scales, (int32_t)rows, (int32_t)cols), device_->raw());
    }

    // A quantized router as it is stored: int8 rows [num_experts, d_model] and one scale per row; the layer then
    // routes with the quantized product (src/quantized.rs:55-62).
    void set_router_q8(const int8_t* q, const float* scales) {
        set_weight_q8(RBMOE_W_ROUTER, 0, q, scales, config.num_experts, d_model_);
    }

    // What TransformerLm::quantize() (src/transformer.rs:899-910) does to this layer's Linears, applied to f32
    // weights as they are set from here on.  in_memory_rule: q = round(w * (1 / scale)) as Quantized::from_matrix
    // (src/quantized.rs:29-51), otherwise the .rbw writer's q = round(w / scale) (src/transformer.rs:512-519);
    // router: the router is quantized as well (src/moe.rs:491-500).  The experts follow only on a layer whose weight
    // dtype is RBMOE_I8.
    void quantize_on_upload(bool in_memory_rule = true, bool router = true) {
        set_option(RBMOE_OPT_QUANT_RULE, in_memory_rule ? 1 : 0);
        set_option(RBMOE_OPT_QUANTIZE_ROUTER, router ? 1 : 0);
    }

    Matrix forward(const Matrix& input) { return forward_train(input, Layout{}).first; }

    std::pair<Matrix, MoeCache> forward_train(const Matrix& input, const Layout& layout) {
        if (input.cols != d_model_)
            throw InvalidInput("input length " + std::to_string(input.cols) + " does not match expected length " +
                                   std::to_string(d_model_),
                               d_model_, input.cols);
        layout.check(input.rows);
        const size_t T = input.rows, E = config.num_experts, k = config.experts_per_token;
        std::vector<uint8_t> valid;
        size_t valid_tokens = T;
        if (layout.valid) {
            valid.resize(T);
            valid_tokens = 0;
            for (size_t t = 0; t < T; ++t) valid_tokens += (valid[t] = (*layout.valid)[t] ? 1 : 0);
        }
        Matrix out(T, d_model_);
        if (act_ == RBMOE_F32) {
            check(rbmoe_forward_host(layer_, input.data.data(), (int32_t)T, (int32_t)input.cols,
                                     layout.valid ? valid.data() : nullptr, nullptr, nullptr, out.data.data()),
                  device_->raw());
        } else {
            std::vector<uint16_t> xin(input.data.size()), xout(input.data.size());
            for (size_t i = 0; i < xin.size(); ++i) xin[i] = to_bf16(input.data[i]);
            check(rbmoe_forward_host(layer_, xin.data(), (int32_t)T, (int32_t)input.cols,
                                     layout.valid ? valid.data() : nullptr, nullptr, nullptr, xout.data()),
                  device_->raw());
            for (size_t i = 0; i < xout.size(); ++i) out.data[i] = from_bf16(xout[i]);
        }
        MoeCache cache;
        cache.valid_tokens = valid_tokens;
        check(rbmoe_get_losses(layer_, &cache.aux, &cache.z), device_->raw());
        std::vector<int32_t> expert_of(T * k), counts(E), offsets(E + 1), perm_slot(T * k), perm_token(T * k);
        std::vector<float> gate_of(T * k);
        cache.probabilities = Matrix(T, E);
        cache.log_sum_exp.assign(T, 0.0f);
        rbmoe_routing r{expert_of.data(), gate_of.data(), counts.data(), offsets.data(), perm_slot.data(),
                        perm_token.data(), cache.probabilities.data.data(), cache.log_sum_exp.data()};
        check(rbmoe_get_routing(layer_, &r), device_->raw());
        for (size_t s = 0; s < T * k; ++s) cache.assignments.emplace_back(expert_of[s], gate_of[s]);
        cache.expert_tokens.resize(E);
        cache.expert_slots.resize(E);
        for (size_t e = 0; e < E; ++e)
            for (int32_t p = offsets[e]; p < offsets[e + 1]; ++p) {
                cache.expert_tokens[e].push_back((size_t)perm_token[p]);
                cache.expert_slots[e].push_back((size_t)perm_slot[p]);
            }
        return {std::move(out), std::move(cache)};
    }

    // ---- training (MoeLayer::backward, src/moe.rs:348-489).  The reference takes the cache of the forward pass
    // as an argument; the device layer keeps that state itself, so backward differentiates the last forward.
    void enable_training() { check(rbmoe_layer_enable_training(layer_), device_->raw()); }

    // a behaviour switch of the layer (RBMOE_OPT_*); every default is the fast path
    void set_option(int option, int value) { check(rbmoe_layer_set_option(layer_, option, value), device_->raw()); }

    Matrix backward(const Matrix& grad_output) {
        if (grad_output.cols != d_model_)
            throw InvalidInput("grad_output length " + std::to_string(grad_output.cols) +
                                   " does not match expected length " + std::to_string(d_model_),
                               d_model_, grad_output.cols);
        Matrix grad_input(grad_output.rows, d_model_);
        if (act_ == RBMOE_F32) {
            check(rbmoe_backward_host(layer_, grad_output.data.data(), (int32_t)grad_output.rows, (int32_t)grad_output.cols,
                                      grad_input.data.data()),
                  device_->raw());
        } else {
            std::vector<uint16_t> gin(grad_output.data.size()), gout(grad_output.data.size());
            for (size_t i = 0; i < gin.size(); ++i) gin[i] = to_bf16(grad_output.data[i]);
            check(rbmoe_backward_host(layer_, gin.data(), (int32_t)grad_output.rows, (int32_t)grad_output.cols, gout.data()),
                  device_->raw());
            for (size_t i = 0; i < gout.size(); ++i) grad_input.data[i] = from_bf16(gout[i]);
        }
        return grad_input;
    }

    // ---- the block's steps either side of the layer (src/transformer_block.rs:216-222, :257-263)
    void set_feed_forward_norm(const std::vector<float>& weight, float eps) {
        check(rbmoe_set_feed_forward_norm(layer_, weight.data(), (int32_t)weight.size(), eps), device_->raw());
    }

    // input + forward(feed_forward_norm(input)); f32 boundary only (as forward_train's bf16 conversion is not repeated here)
    Matrix forward_block(const Matrix& residual) {
        if (residual.cols != d_model_)
            throw InvalidInput("input length " + std::to_string(residual.cols) + " does not match expected length " +
                                   std::to_string(d_model_),
                               d_model_, residual.cols);
        Matrix out(residual.rows, d_model_);
        if (act_ == RBMOE_F32) {
            check(rbmoe_forward_block_host(layer_, residual.data.data(), (int32_t)residual.rows, (int32_t)residual.cols,
                                           nullptr, nullptr, out.data.data()),
                  device_->raw());
        } else {
            std::vector<uint16_t> xin(residual.data.size()), xout(residual.data.size());
            for (size_t i = 0; i < xin.size(); ++i) xin[i] = to_bf16(residual.data[i]);
            check(rbmoe_forward_block_host(layer_, xin.data(), (int32_t)residual.rows, (int32_t)residual.cols, nullptr,
                                           nullptr, xout.data()),
                  device_->raw());
            for (size_t i = 0; i < xout.size(); ++i) out.data[i] = from_bf16(xout[i]);
        }
        return out;
    }

    // gradient of forward_block's input: through the layer, the norm and the residual
    Matrix backward_block(const Matrix& grad_output) {
        Matrix grad_input(grad_output.rows, d_model_);
        if (act_ == RBMOE_F32) {
            check(rbmoe_backward_block_host(layer_, grad_output.data.data(), (int32_t)grad_output.rows,
                                            (int32_t)grad_output.cols, grad_input.data.data()),
                  device_->raw());
        } else {
            std::vector<uint16_t> gin(grad_output.data.size()), gout(grad_output.data.size());
            for (size_t i = 0; i < gin.size(); ++i) gin[i] = to_bf16(grad_output.data[i]);
            check(rbmoe_backward_block_host(layer_, gin.data(), (int32_t)grad_output.rows, (int32_t)grad_output.cols,
                                            gout.data()),
                  device_->raw());
            for (size_t i = 0; i < gout.size(); ++i) grad_input.data[i] = from_bf16(gout[i]);
        }
        return grad_input;
    }

    // Param::zero_grad over the layer's parameters (src/param.rs)
    void zero_grads() { check(rbmoe_zero_grads(layer_), device_->raw()); }

    // accumulated gradient of one weight matrix (`which`: RBMOE_W_*), shaped like the weight
    Matrix weight_grad(int which, size_t expert = 0) {
        const size_t E = config.num_experts, F = config.d_ff, Fs = shared_d_ff_ ? shared_d_ff_ : config.d_ff;
        size_t rows = 0, cols = 0;
        switch (which) {
            case RBMOE_W_ROUTER: rows = E; cols = d_model_; break;
            case RBMOE_W_GATE: case RBMOE_W_UP: rows = F; cols = d_model_; break;
            case RBMOE_W_DOWN: rows = d_model_; cols = F; break;
            case RBMOE_W_SHARED_GATE: case RBMOE_W_SHARED_UP: rows = Fs; cols = d_model_; break;
            case RBMOE_W_SHARED_DOWN: rows = d_model_; cols = Fs; break;
            case RBMOE_W_NORM: rows = 1; cols = d_model_; break;
            default: throw InvalidConfig("unknown weight id");
        }
        Matrix g(rows, cols);
        check(rbmoe_get_weight_grad(layer_, which, (int32_t)expert, g.data.data(), (int32_t)rows, (int32_t)cols),
              device_->raw());
        return g;
    }

    uint64_t num_parameters() const { return counts().first; }
    uint64_t active_parameters() const { return counts().second; }
    std::string kernel_name() const { return rbmoe_expert_kernel_name(layer_); }

  private:
    static uint16_t to_bf16(float f) {
        uint32_t b;
        std::memcpy(&b, &f, 4);
        if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x40u);
        b += 0x7fffu + ((b >> 16) & 1u);
        return (uint16_t)(b >> 16);
    }
    static float from_bf16(uint16_t h) {
        const uint32_t b = (uint32_t)h << 16;
        float f;
        std::memcpy(&f, &b, 4);
        return f;
    }
    void set(int which, int expert, const Matrix& w) {
        check(rbmoe_set_weight(layer_, which, expert, w.data.data(), RBMOE_F32, nullptr, (int32_t)w.rows,
                               (int32_t)w.cols),
              device_->raw());
    }
    std::pair<uint64_t, uint64_t> counts() const {
        const rbmoe_config c = config.raw(d_model_);
        uint64_t total = 0, active = 0;
        check(rbmoe_parameter_counts(&c, &total, &active));
        return {total, active};
    }

    size_t d_model_;
    std::shared_ptr<Device> device_;
    int act_;
    size_t shared_d_ff_ = 0;
    rbmoe_layer* layer_ = nullptr;
};

// ------------------------------------------------------------------ builder surface
struct ParameterCounts {
    uint64_t total, active;
};

// The methods of `TransformerBuilder` that select and size the sparse layers; defaults
// are the reference's 55M-total / 36M-active model (src/transformer.rs:100-126).
class TransformerBuilder {
  public:
    TransformerBuilder& vocab_size(size_t v) { vocab_size_ = v; return *this; }
    TransformerBuilder& d_model(size_t v) { d_model_ = v; return *this; }
    TransformerBuilder& n_layers(size_t v) { n_layers_ = v; return *this; }
    TransformerBuilder& heads(size_t h, size_t kv, size_t dim) { n_heads_ = h; n_kv_heads_ = kv; head_dim_ = dim; return *this; }
    TransformerBuilder& d_ff(size_t v) { d_ff_ = v; return *this; }
    TransformerBuilder& moe_d_ff(size_t v) { moe_d_ff_ = v; return *this; }
    TransformerBuilder& experts(size_t n, size_t k) { num_experts_ = n; experts_per_token_ = k; return *this; }
    TransformerBuilder& moe_layers(std::vector<size_t> layers) { moe_layers_ = std::move(layers); return *this; }
    TransformerBuilder& shared_expert(bool b) { shared_expert_ = b; return *this; }
    TransformerBuilder& max_seq_len(size_t v) { max_seq_len_ = v; return *this; }
    TransformerBuilder& tie_embeddings(bool b) { tie_embeddings_ = b; return *this; }
    TransformerBuilder& aux_loss_weight(float w) { aux_loss_weight_ = w; return *this; }
    TransformerBuilder& router_z_loss_weight(float w) { router_z_loss_weight_ = w; return *this; }

    MoeConfig moe_config() const {
        return MoeConfig(num_experts_, experts_per_token_, moe_d_ff_)
            .with_shared_expert(shared_expert_)
            .with_aux_loss_weight(aux_loss_weight_)
            .with_router_z_loss_weight(router_z_loss_weight_);
    }
    bool is_moe_layer(size_t layer) const {
        for (size_t l : moe_layers_)
            if (l == layer) return true;
        return false;
    }
    void validate() const {  // TransformerConfig::validate, src/transformer.rs:129-175
        const std::pair<const char*, size_t> nonzero[] = {{"vocab_size", vocab_size_}, {"d_model", d_model_},
            {"n_layers", n_layers_}, {"n_heads", n_heads_}, {"n_kv_heads", n_kv_heads_}, {"head_dim", head_dim_},
            {"d_ff", d_ff_}, {"max_seq_len", max_seq_len_}};
        for (const auto& nv : nonzero)
            if (nv.second == 0) throw InvalidConfig(std::string(nv.first) + " must be non-zero");
        if (n_heads_ % n_kv_heads_ != 0 || n_kv_heads_ > n_heads_)
            throw InvalidConfig("n_heads (" + std::to_string(n_heads_) + ") must be a multiple of n_kv_heads (" +
                                std::to_string(n_kv_heads_) + ")");
        if (head_dim_ % 2 != 0)
            throw InvalidConfig("head_dim must be even for rotary embeddings, got " + std::to_string(head_dim_));
        for (size_t l : moe_layers_)
            if (l >= n_layers_)
                throw InvalidConfig("moe_layers names layer " + std::to_string(l) + ", but the model has " +
                                    std::to_string(n_layers_) + " layers");
        if (!moe_layers_.empty()) moe_config().validate();
    }
    ParameterCounts parameter_counts() const {  // src/transformer.rs:194-227
        const uint64_t query = d_model_ * n_heads_ * head_dim_, key_value = 2 * d_model_ * n_kv_heads_ * head_dim_;
        const uint64_t attention = 2 * query + key_value, norms = 2 * d_model_;
        const uint64_t dense_ffn = 3 * d_model_ * d_ff_, expert = 3 * d_model_ * moe_d_ff_;
        const uint64_t shared = shared_expert_ ? expert : 0, router = num_experts_ * d_model_;
        const uint64_t moe_total = router + num_experts_ * expert + shared;
        const uint64_t moe_active = router + experts_per_token_ * expert + shared;
        uint64_t total = vocab_size_ * d_model_ + d_model_;
        if (!tie_embeddings_) total += vocab_size_ * d_model_;
        uint64_t active = total;
        for (size_t layer = 0; layer < n_layers_; ++layer) {
            total += attention + norms;
            active += attention + norms;
            total += is_moe_layer(layer) ? moe_total : dense_ffn;
            active += is_moe_layer(layer) ? moe_active : dense_ffn;
        }
        return {total, active};
    }
    // Validates before any allocation, then builds one MoeLayer per index in moe_layers.
    std::map<size_t, std::unique_ptr<MoeLayer>> build_moe_layers(const std::shared_ptr<Device>& device,
                                                                 size_t max_tokens, int act_dtype = RBMOE_F32,
                                                                 int weight_dtype = RBMOE_F32) const {
        validate();
        std::map<size_t, std::unique_ptr<MoeLayer>> layers;
        for (size_t l : moe_layers_)
            layers[l] = std::make_unique<MoeLayer>(d_model_, moe_config(), device, max_tokens, act_dtype, weight_dtype);
        return layers;
    }

  private:
    size_t vocab_size_ = 32000, d_model_ = 512, n_layers_ = 8, n_heads_ = 8, n_kv_heads_ = 2, head_dim_ = 64;
    size_t d_ff_ = 1408, moe_d_ff_ = 352, num_experts_ = 8, experts_per_token_ = 2, max_seq_len_ = 2048;
    std::vector<size_t> moe_layers_ = {2, 3, 4, 5, 6, 7};
    bool shared_expert_ = true, tie_embeddings_ = true;
    float aux_loss_weight_ = DEFAULT_AUX_LOSS_WEIGHT, router_z_loss_weight_ = DEFAULT_ROUTER_Z_LOSS_WEIGHT;
};

}  // namespace rusting_brain

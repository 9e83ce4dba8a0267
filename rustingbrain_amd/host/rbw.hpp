// Reader of the reference's binary weight snapshot, `.rbw`, for the C++ host mirror.
//
// Format, from `TransformerLm::save_bin` / `load_bin` (reference src/transformer.rs:1806-1932; header struct
// :503-510; `quantize` :512-519):
//
//     8 bytes   magic "RBWTS001"                                            (:488)
//     u64 LE    length of the JSON header
//     bytes     JSON {"config": TransformerConfig, "optimizer": .., "optimizer_step": n, "precision": "F32" | "Q8"}
//     u64 LE    number of parameters
//     per parameter, in `TransformerLm::params_mut()` order (:1620-1630):
//         u64 LE rows, u64 LE cols
//         F32:  rows * cols little-endian f32, row-major
//         Q8:   per row: f32 scale (= absmax / 127), then cols int8
//
// Parameter order (src/transformer.rs:1620-1630, src/transformer_block.rs:286-292, src/attention.rs:911-917,
// src/moe.rs:516-525, src/ffn.rs:126-131): embedding; per block attention_norm, query, key, value, output,
// feed_forward_norm, then gate, up, down of a dense block or router, experts x (gate, up, down), shared (gate, up,
// down) of a sparse one; final_norm; lm_head unless the embeddings are tied.
//
// Only the sparse blocks are interpreted: their parameters go to `MoeLayer`s (a Q8 file's expert matrices as the
// int8 values and scales they are stored as, the router dequantised the way `load_bin` does), everything else is
// parsed so that the positions are right.  Snapshots of models with LoRA adapters are refused.
#pragma once

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "rusting_brain_moe.hpp"

namespace rusting_brain {
namespace rbw {

struct InvalidSnapshot : NetworkError { using NetworkError::NetworkError; };  // NetworkError::InvalidSnapshot

// ------------------------------------------------------------------ the header's JSON
struct Json {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    bool b = false;
    double number = 0.0;
    std::string text;
    std::vector<Json> items;
    std::map<std::string, Json> fields;

    bool has(const std::string& key) const { return kind == Object && fields.count(key) != 0; }
    const Json& at(const std::string& key) const {
        static const Json none;
        const auto it = fields.find(key);
        return it == fields.end() ? none : it->second;
    }
    bool is_null() const { return kind == Null; }
    size_t as_size(const std::string& what) const {
        if (kind != Number || number < 0 || number != (double)(uint64_t)number)
            throw InvalidSnapshot("weight file header: " + what + " is not a non-negative integer");
        return (size_t)number;
    }
    double as_number(double fallback) const { return kind == Number ? number : fallback; }
    bool as_bool(bool fallback) const { return kind == Bool ? b : fallback; }
};

class JsonParser {
  public:
    explicit JsonParser(const std::string& s) : s_(s) {}
    Json parse() {
        Json v = value();
        skip();
        if (pos_ != s_.size()) fail("trailing characters");
        return v;
    }

  private:
    [[noreturn]] void fail(const char* what) const {
        throw InvalidSnapshot(std::string("weight file header is not JSON: ") + what + " at byte " + std::to_string(pos_));
    }
    void skip() {
        while (pos_ < s_.size() && (s_[pos_] == ' ' || s_[pos_] == '\n' || s_[pos_] == '\t' || s_[pos_] == '\r')) ++pos_;
    }
    bool eat(char c) {
        skip();
        if (pos_ < s_.size() && s_[pos_] == c) {
            ++pos_;
            return true;
        }
        return false;
    }
    void word(const char* w) {
        const size_t n = std::strlen(w);
        if (s_.compare(pos_, n, w) != 0) fail("unknown literal");
        pos_ += n;
    }
    std::string string() {
        std::string out;
        while (true) {
            if (pos_ >= s_.size()) fail("unterminated string");
            const char c = s_[pos_++];
            if (c == '"') return out;
            if (c != '\\') {
                out.push_back(c);
                continue;
            }
            if (pos_ >= s_.size()) fail("unterminated escape");
            const char e = s_[pos_++];
            switch (e) {
                case '"': case '\\': case '/': out.push_back(e); break;
                case 'n': out.push_back('\n'); break;
                case 't': out.push_back('\t'); break;
                case 'r': out.push_back('\r'); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'u': {  // kept as UTF-8; the reference's header holds ASCII only
                    if (pos_ + 4 > s_.size()) fail("short \\u escape");
                    const unsigned cp = (unsigned)std::strtoul(s_.substr(pos_, 4).c_str(), nullptr, 16);
                    pos_ += 4;
                    if (cp < 0x80) {
                        out.push_back((char)cp);
                    } else if (cp < 0x800) {
                        out.push_back((char)(0xC0 | (cp >> 6)));
                        out.push_back((char)(0x80 | (cp & 0x3F)));
                    } else {
                        out.push_back((char)(0xE0 | (cp >> 12)));
                        out.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
                        out.push_back((char)(0x80 | (cp & 0x3F)));
                    }
                    break;
                }
                default: fail("unknown escape");
            }
        }
    }
    Json value() {
        skip();
        if (pos_ >= s_.size()) fail("unexpected end");
        Json v;
        const char c = s_[pos_];
        if (c == '{') {
            ++pos_;
            v.kind = Json::Object;
            if (eat('}')) return v;
            do {
                skip();
                if (pos_ >= s_.size() || s_[pos_] != '"') fail("expected a field name");
                ++pos_;
                const std::string key = string();
                if (!eat(':')) fail("expected ':'");
                v.fields[key] = value();
            } while (eat(','));
            if (!eat('}')) fail("expected '}'");
        } else if (c == '[') {
            ++pos_;
            v.kind = Json::Array;
            if (eat(']')) return v;
            do v.items.push_back(value());
            while (eat(','));
            if (!eat(']')) fail("expected ']'");
        } else if (c == '"') {
            ++pos_;
            v.kind = Json::String;
            v.text = string();
        } else if (c == 't') {
            word("true");
            v.kind = Json::Bool;
            v.b = true;
        } else if (c == 'f') {
            word("false");
            v.kind = Json::Bool;
        } else if (c == 'n') {
            word("null");
        } else {
            const char* begin = s_.c_str() + pos_;
            char* end = nullptr;
            v.number = std::strtod(begin, &end);
            if (end == begin) fail("expected a value");
            v.kind = Json::Number;
            pos_ += (size_t)(end - begin);
        }
        return v;
    }

    const std::string& s_;
    size_t pos_ = 0;
};

// ------------------------------------------------------------------ the file
struct Param {
    size_t rows = 0, cols = 0;
    std::vector<float> values;   // F32 files: [rows, cols]
    std::vector<int8_t> q;       // Q8 files:  [rows, cols]
    std::vector<float> scales;   // Q8 files:  [rows]

    // f32 values the way `load_bin` restores them: `q as f32 * scale`
    Matrix dequantized() const {
        Matrix m(rows, cols);
        if (q.empty()) {
            std::copy(values.begin(), values.end(), m.data.begin());
        } else {
            for (size_t r = 0; r < rows; ++r)
                for (size_t c = 0; c < cols; ++c) m.data[r * cols + c] = (float)q[r * cols + c] * scales[r];
        }
        return m;
    }
};

struct Snapshot {
    Json config;
    std::string precision;  // "F32" | "Q8"
    uint64_t optimizer_step = 0;
    std::vector<Param> params;
};

inline uint64_t le64(const unsigned char* p) {
    uint64_t v = 0;
    for (int i = 7; i >= 0; --i) v = (v << 8) | p[i];
    return v;
}
inline float le_f32(const unsigned char* p) {
    const uint32_t b = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
    float f;
    std::memcpy(&f, &b, 4);
    return f;
}

inline Snapshot read(const std::string& path) {
    std::FILE* f = std::fopen(path.c_str(), "rb");
    if (!f) throw InvalidSnapshot("cannot open " + path);
    std::vector<unsigned char> data;
    unsigned char buf[1 << 16];
    size_t n;
    while ((n = std::fread(buf, 1, sizeof buf, f)) > 0) data.insert(data.end(), buf, buf + n);
    std::fclose(f);
    if (data.size() < 16 || std::memcmp(data.data(), "RBWTS001", 8) != 0)
        throw InvalidSnapshot("not a RustingBrain weight file");
    size_t pos = 8;
    const uint64_t hlen = le64(&data[pos]);
    pos += 8;
    if (hlen > data.size() || pos + hlen + 8 > data.size())
        throw InvalidSnapshot("weight file is truncated inside its header");
    const std::string header_text(reinterpret_cast<const char*>(&data[pos]), (size_t)hlen);
    pos += (size_t)hlen;
    const Json header = JsonParser(header_text).parse();
    Snapshot snap;
    snap.config = header.at("config");
    snap.precision = header.at("precision").kind == Json::String ? header.at("precision").text : "";
    if (snap.precision != "F32" && snap.precision != "Q8") throw InvalidSnapshot("unknown precision '" + snap.precision + "'");
    snap.optimizer_step = (uint64_t)header.at("optimizer_step").as_number(0.0);
    const uint64_t count = le64(&data[pos]);
    pos += 8;
    const bool q8 = snap.precision == "Q8";
    for (uint64_t i = 0; i < count; ++i) {
        if (pos + 16 > data.size()) throw InvalidSnapshot("weight file is truncated between parameters");
        Param p;
        p.rows = (size_t)le64(&data[pos]);
        p.cols = (size_t)le64(&data[pos + 8]);
        pos += 16;
        const size_t bytes = q8 ? p.rows * (4 + p.cols) : p.rows * p.cols * 4;
        if (bytes > data.size() || pos + bytes > data.size()) throw InvalidSnapshot("weight file is truncated inside a parameter");
        if (q8) {
            p.q.resize(p.rows * p.cols);
            p.scales.resize(p.rows);
            for (size_t r = 0; r < p.rows; ++r) {
                const unsigned char* row = &data[pos + r * (4 + p.cols)];
                p.scales[r] = le_f32(row);
                std::memcpy(p.q.data() + r * p.cols, row + 4, p.cols);
            }
        } else {
            p.values.resize(p.rows * p.cols);
            for (size_t j = 0; j < p.values.size(); ++j) p.values[j] = le_f32(&data[pos + 4 * j]);
        }
        pos += bytes;
        snap.params.push_back(std::move(p));
    }
    if (pos != data.size()) throw InvalidSnapshot(std::to_string(data.size() - pos) + " bytes follow the last parameter");
    return snap;
}

// The parameters of one sparse block's feed-forward, in the reference's order (src/moe.rs:516-525).
struct Swiglu {
    const Param* gate = nullptr;
    const Param* up = nullptr;
    const Param* down = nullptr;
};
struct MoeBlock {
    size_t block = 0;
    const Param* norm = nullptr;  // feed_forward_norm.weight (src/norm.rs:30-35)
    const Param* router = nullptr;
    std::vector<Swiglu> experts;
    bool has_shared = false;
    Swiglu shared;
};

// Walks the parameter list in `params_mut()` order and picks out every sparse block.
inline std::vector<MoeBlock> moe_blocks(const Snapshot& snap) {
    const Json& c = snap.config;
    if (c.has("lora") && !c.at("lora").is_null())
        throw InvalidConfig("snapshots of models with LoRA adapters are not supported");
    const size_t d = c.at("d_model").as_size("d_model"), layers = c.at("n_layers").as_size("n_layers");
    const size_t heads = c.at("n_heads").as_size("n_heads"), kv_heads = c.at("n_kv_heads").as_size("n_kv_heads");
    const size_t head_dim = c.at("head_dim").as_size("head_dim");
    const size_t d_ff = c.at("d_ff").as_size("d_ff"), moe_d_ff = c.at("moe_d_ff").as_size("moe_d_ff");
    const size_t E = c.at("num_experts").as_size("num_experts"), vocab = c.at("vocab_size").as_size("vocab_size");
    std::vector<size_t> sparse;
    for (const Json& v : c.at("moe_layers").items) sparse.push_back(v.as_size("moe_layers entry"));
    const bool shared = c.at("shared_expert").as_bool(false);
    const std::vector<Param>& params = snap.params;
    size_t pos = 0;
    auto take = [&](size_t rows, size_t cols, const std::string& what) -> const Param* {
        if (pos >= params.size())
            throw InvalidSnapshot("weight file holds " + std::to_string(params.size()) + " parameters, this configuration builds more");
        const Param& p = params[pos];
        if (p.rows != rows || p.cols != cols)
            throw InvalidSnapshot("weight file has a " + std::to_string(p.rows) + "x" + std::to_string(p.cols) +
                                  " parameter where the model has " + std::to_string(rows) + "x" + std::to_string(cols) +
                                  " (" + what + ")");
        ++pos;
        return &p;
    };
    auto take_swiglu = [&](size_t f, const std::string& what) {
        Swiglu s;
        s.gate = take(f, d, what + ".gate");
        s.up = take(f, d, what + ".up");
        s.down = take(d, f, what + ".down");
        return s;
    };
    take(vocab, d, "embedding");
    std::vector<MoeBlock> out;
    for (size_t b = 0; b < layers; ++b) {
        const std::string name = "block " + std::to_string(b);
        ++pos;  // attention_norm (a vector; its orientation does not matter here)
        take(heads * head_dim, d, name + " query");
        take(kv_heads * head_dim, d, name + " key");
        take(kv_heads * head_dim, d, name + " value");
        take(d, heads * head_dim, name + " output");
        const Param* ff_norm = pos < params.size() ? &params[pos] : nullptr;
        ++pos;  // feed_forward_norm
        bool is_sparse = false;
        for (size_t s : sparse) is_sparse = is_sparse || s == b;
        if (is_sparse) {
            MoeBlock blk;
            blk.block = b;
            blk.norm = ff_norm;
            blk.router = take(E, d, name + " router");
            for (size_t e = 0; e < E; ++e) blk.experts.push_back(take_swiglu(moe_d_ff, name + " expert " + std::to_string(e)));
            blk.has_shared = shared;
            if (shared) blk.shared = take_swiglu(moe_d_ff, name + " shared expert");
            out.push_back(std::move(blk));
        } else {
            take_swiglu(d_ff, name + " feed-forward");
        }
    }
    ++pos;  // final_norm
    if (!c.at("tie_embeddings").as_bool(false)) take(vocab, d, "lm_head");
    if (pos != params.size())
        throw InvalidSnapshot("weight file holds " + std::to_string(params.size()) + " parameters, this configuration builds " +
                              std::to_string(pos));
    return out;
}

// One device `MoeLayer` per sparse block.  `weight_dtype` < 0: int8 for a Q8 file (the stored values and scales are
// used as they are), bf16 for an F32 file.
inline std::vector<std::unique_ptr<MoeLayer>> load_moe_layers(const std::string& path, std::shared_ptr<Device> device,
                                                              size_t max_tokens, int act_dtype = RBMOE_BF16,
                                                              int weight_dtype = -1) {
    const Snapshot snap = read(path);
    const Json& c = snap.config;
    const std::vector<MoeBlock> blocks = moe_blocks(snap);
    const bool q8 = snap.precision == "Q8";
    if (weight_dtype < 0) weight_dtype = q8 ? RBMOE_I8 : RBMOE_BF16;
    const size_t d = c.at("d_model").as_size("d_model");
    const MoeConfig cfg = MoeConfig(c.at("num_experts").as_size("num_experts"),
                                    c.at("experts_per_token").as_size("experts_per_token"),
                                    c.at("moe_d_ff").as_size("moe_d_ff"))
                              .with_shared_expert(c.at("shared_expert").as_bool(false))
                              .with_aux_loss_weight((float)c.at("aux_loss_weight").as_number(0.01))
                              .with_router_z_loss_weight((float)c.at("router_z_loss_weight").as_number(1e-3));
    const bool stored = q8 && weight_dtype == RBMOE_I8;
    std::vector<std::unique_ptr<MoeLayer>> layers;
    for (const MoeBlock& blk : blocks) {
        std::unique_ptr<MoeLayer> layer(new MoeLayer(d, cfg, device, max_tokens, act_dtype, weight_dtype));
        layer->set_router(blk.router->dequantized());
        if (blk.norm && blk.norm->rows * blk.norm->cols == d)  // the norm in front of the layer, for forward_block
            layer->set_feed_forward_norm(blk.norm->dequantized().data, (float)c.at("rmsnorm_eps").as_number(1e-6));
        auto put = [&](int gate_id, int expert, const Swiglu& s) {
            const int ids[3] = {gate_id, gate_id + 1, gate_id + 2};  // gate, up, down are consecutive weight ids
            const Param* ps[3] = {s.gate, s.up, s.down};
            for (int i = 0; i < 3; ++i) {
                if (stored) layer->set_weight_q8(ids[i], expert, ps[i]->q.data(), ps[i]->scales.data(), ps[i]->rows, ps[i]->cols);
                else layer->set_weight(ids[i], expert, ps[i]->dequantized());
            }
        };
        for (size_t e = 0; e < blk.experts.size(); ++e) put(RBMOE_W_GATE, (int)e, blk.experts[e]);
        if (blk.has_shared) put(RBMOE_W_SHARED_GATE, 0, blk.shared);
        layers.push_back(std::move(layer));
    }
    return layers;
}

}  // namespace rbw
}  // namespace rusting_brain

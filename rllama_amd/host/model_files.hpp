// model_files.hpp -- the reference's on-disk model format for the C++ host mirror: pickle reader, params.json,
// shard handling and the loader that feeds a rllama::Transformer.
//
//   rllama::unpickler::Value / unpickle   <- src/unpickler.rs:23-34, 317-675 (the same opcode subset, nothing executed)
//   rllama::TensorBuilder                 <- src/unpickler.rs:147-249, src/tensor.rs:2346-2546
//   rllama::ModelParams                   <- src/model_params.rs:3-14 (with its aliases)
//   rllama::DataSource                    <- src/data_source.rs:27-31, 166-210 (the LLaMA layout)
//   rllama::load_transformer              <- main + Transformer::from_unpickled (src/rllama_main.rs:235-283,
//                                            src/transformer.rs:242-326)
//
// Layout: <model>/params.json, <model>/consolidated.NN/data.pkl, <model>/consolidated.NN/data/<key> (raw
// little-endian f16, row-major).  Header-only, C++17.
#pragma once

#include "rllama_hip.hpp"

#include <cerrno>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <map>
#include <sstream>
#include <sys/stat.h>

namespace rllama {

namespace unpickler {

struct UnpicklingError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct Value;
using ValuePtr = std::shared_ptr<const Value>;

struct Value {
    enum Kind { Mark, String, Global, Integer64, Tuple, PersistentId, Bool, Reduce, Dict } kind = Mark;
    std::string str, attr;                                // String: str; Global: module name in str, attribute in attr
    int64_t integer = 0;
    bool boolean = false;
    std::vector<ValuePtr> items;                          // Tuple items; PersistentId: {value}; Reduce: {callable, args}
    std::map<std::string, ValuePtr> entries;              // Dict entries with string keys
    std::vector<std::pair<ValuePtr, ValuePtr>> other_entries; // Dict entries with any other key

    const Value *get_str_key(const std::string &key) const {
        auto it = entries.find(key);
        return kind == Dict && it != entries.end() ? it->second.get() : nullptr;
    }
    bool is_global(const char *module, const char *name) const { return kind == Global && str == module && attr == name; }
};

inline ValuePtr unpickle(const std::vector<uint8_t> &bytes) {
    if (bytes.size() < 2) throw UnpicklingError("Data is too short to be a pickle");
    if (bytes[0] != 0x80 || bytes[1] != 2) throw UnpicklingError("No magic header using Pickle 2 protocol");
    std::map<uint32_t, ValuePtr> memo;
    std::vector<ValuePtr> stack;
    size_t pos = 2;
    const size_t n = bytes.size();
    auto need = [&](size_t k, const char *what) {
        if (pos + k > n) throw UnpicklingError(std::string("Unexpected end of data while handling ") + what);
    };
    auto u32 = [&](size_t at) { return (uint32_t)bytes[at] | (uint32_t)bytes[at + 1] << 8 | (uint32_t)bytes[at + 2] << 16 | (uint32_t)bytes[at + 3] << 24; };
    auto make = [](Value::Kind k) {
        auto v = std::make_shared<Value>();
        v->kind = k;
        return v;
    };
    auto push_int = [&](int64_t i) {
        auto v = make(Value::Integer64);
        v->integer = i;
        stack.push_back(v);
    };
    auto pop_to_mark = [&](const char *what) {
        std::vector<ValuePtr> got;
        while (!stack.empty()) {
            ValuePtr top = stack.back();
            stack.pop_back();
            if (top->kind == Value::Mark) {
                std::vector<ValuePtr> in_order(got.rbegin(), got.rend());
                return in_order;
            }
            got.push_back(top);
        }
        throw UnpicklingError(std::string("No mark while handling ") + what);
    };
    auto top_needed = [&](size_t k, const char *what) {
        if (stack.size() < k) throw UnpicklingError(std::string(k == 1 ? "Stack is empty while handling " : "Stack does not have enough items while handling ") + what);
    };
    while (pos < n) {
        const uint8_t op = bytes[pos];
        switch (op) {
        case 0x7d: stack.push_back(make(Value::Dict)); pos += 1; break;
        case 0x71: need(2, "BINPUT"); top_needed(1, "BINPUT"); memo[bytes[pos + 1]] = stack.back(); pos += 2; break;
        case 0x72: need(5, "LONG_BINPUT"); top_needed(1, "LONG_BINPUT"); memo[u32(pos + 1)] = stack.back(); pos += 5; break;
        case 0x68: {
            need(2, "BINGET");
            auto it = memo.find(bytes[pos + 1]);
            if (it == memo.end()) throw UnpicklingError("BINGET index out of range");
            stack.push_back(it->second);
            pos += 2;
            break;
        }
        case 0x6a: {
            need(5, "LONG_BINGET");
            auto it = memo.find(u32(pos + 1));
            if (it == memo.end()) throw UnpicklingError("LONG_BINGET index out of range");
            stack.push_back(it->second);
            pos += 5;
            break;
        }
        case 0x28: stack.push_back(make(Value::Mark)); pos += 1; break;
        case 0x58: {
            need(5, "BINUNICODE");
            const size_t len = u32(pos + 1);
            need(5 + len, "BINUNICODE");
            auto v = make(Value::String);
            v->str.assign((const char *)&bytes[pos + 5], len);
            stack.push_back(v);
            pos += 5 + len;
            break;
        }
        case 0x63: { // GLOBAL: module and attribute name, each ended by a newline
            auto v = make(Value::Global);
            size_t p = pos + 1;
            for (std::string *dst : {&v->str, &v->attr}) {
                while (p < n && bytes[p] != '\n') dst->push_back((char)bytes[p++]);
                if (p >= n) throw UnpicklingError("Unexpected end of data while handling GLOBAL");
                p++;
            }
            stack.push_back(v);
            pos = p;
            break;
        }
        case 0x4a: need(5, "BININT"); push_int((int32_t)u32(pos + 1)); pos += 5; break;
        case 0x4b: need(2, "BININT1"); push_int(bytes[pos + 1]); pos += 2; break;
        case 0x4d: need(3, "BININT2"); push_int((int16_t)((uint16_t)bytes[pos + 1] | (uint16_t)bytes[pos + 2] << 8)); pos += 3; break; // signed, like :484
        case 0x74: {
            top_needed(1, "TUPLE");
            auto v = make(Value::Tuple);
            v->items = pop_to_mark("TUPLE");
            stack.push_back(v);
            pos += 1;
            break;
        }
        case 0x85: {
            top_needed(1, "TUPLE1");
            auto v = make(Value::Tuple);
            v->items = {stack.back()};
            stack.pop_back();
            stack.push_back(v);
            pos += 1;
            break;
        }
        case 0x86: {
            top_needed(2, "TUPLE2");
            auto v = make(Value::Tuple);
            v->items = {stack[stack.size() - 2], stack[stack.size() - 1]};
            stack.resize(stack.size() - 2);
            stack.push_back(v);
            pos += 1;
            break;
        }
        case 0x29: stack.push_back(make(Value::Tuple)); pos += 1; break;
        case 0x89: stack.push_back(make(Value::Bool)); pos += 1; break;
        case 0x51: {
            top_needed(1, "BINPERSID");
            auto v = make(Value::PersistentId);
            v->items = {stack.back()};
            stack.pop_back();
            stack.push_back(v);
            pos += 1;
            break;
        }
        case 0x52: {
            top_needed(2, "REDUCE");
            auto v = make(Value::Reduce);
            v->items = {stack[stack.size() - 2], stack[stack.size() - 1]};
            stack.resize(stack.size() - 2);
            stack.push_back(v);
            pos += 1;
            break;
        }
        case 0x75: {
            top_needed(1, "SETITEMS");
            std::vector<ValuePtr> kv = pop_to_mark("SETITEMS");
            if (kv.size() % 2) throw UnpicklingError("Unexpected mark while handling SETITEMS");
            top_needed(1, "SETITEMS");
            if (stack.back()->kind != Value::Dict) throw UnpicklingError("SETITEMS on non-dict");
            auto d = std::make_shared<Value>(*stack.back()); // values are immutable once shared (memo); update a copy
            for (size_t i = 0; i < kv.size(); i += 2) {
                if (kv[i]->kind == Value::String) d->entries[kv[i]->str] = kv[i + 1];
                else d->other_entries.emplace_back(kv[i], kv[i + 1]);
            }
            stack.back() = d;
            pos += 1;
            break;
        }
        case 0x2e: pos = n; break; // STOP
        default: throw UnpicklingError("Unknown opcode: " + std::to_string((int)op));
        }
    }
    if (stack.size() != 1) throw UnpicklingError("Stack does not have exactly one item after unpickling");
    return stack[0];
}

} // namespace unpickler

// What a tensor entry of data.pkl says about where its values are (src/tensor.rs:2346-2356)
struct TensorBuilder {
    std::string src_path, tensor_name;
    int64_t rows = 0, cols = 0, stride = 0, nitems = 0, offset = 0;
};

// Value::to_tensor_builder (src/unpickler.rs:147-249): false for anything but a contiguous 1-D / 2-D HalfStorage tensor
inline bool to_tensor_builder(const unpickler::Value &v, const std::string &tensor_name, TensorBuilder *out) {
    using unpickler::Value;
    if (v.kind != Value::Reduce || !v.items[0]->is_global("torch._utils", "_rebuild_tensor_v2")) return false;
    const Value &args = *v.items[1];
    if (args.kind != Value::Tuple || args.items.size() != 6 || args.items[0]->kind != Value::PersistentId) return false;
    const Value &st = *args.items[0]->items[0];
    if (st.kind != Value::Tuple || st.items.size() < 5) return false;
    if (st.items[0]->kind != Value::String || st.items[0]->str != "storage" || !st.items[1]->is_global("torch", "HalfStorage")) return false;
    if (st.items[2]->kind != Value::String || st.items[4]->kind != Value::Integer64 || args.items[1]->kind != Value::Integer64) return false;
    const Value &shape = *args.items[2], &stride = *args.items[3];
    if (shape.kind != Value::Tuple || stride.kind != Value::Tuple) return false;
    if ((shape.items.size() != 1 && shape.items.size() != 2) || (stride.items.size() != 1 && stride.items.size() != 2)) return false;
    for (const auto *t : {&shape, &stride})
        for (const auto &x : t->items)
            if (x->kind != Value::Integer64) return false;
    TensorBuilder b;
    if (shape.items.size() == 2) {
        b.rows = shape.items[0]->integer;
        b.cols = shape.items[1]->integer;
    } else {
        b.rows = 1; // 1-D tensors load as 1 x n (src/unpickler.rs:207-212)
        b.cols = shape.items[0]->integer;
    }
    if (stride.items.size() == 1) {
        if (stride.items[0]->integer != 1) return false;
        b.stride = 1;
    } else {
        if (stride.items[1]->integer != 1 || stride.items[0]->integer != b.cols) return false;
        b.stride = stride.items[0]->integer;
    }
    b.src_path = st.items[2]->str;
    b.tensor_name = tensor_name;
    b.nitems = st.items[4]->integer;
    b.offset = args.items[1]->integer;
    *out = b;
    return true;
}

enum class FromPiecesDirection { Rows, Cols }; // src/tensor.rs:2339-2343

// ModelParams (src/model_params.rs:3-14).  params.json is a flat JSON object; values of other keys are skipped.
struct ModelParams {
    size_t dim = 0, n_heads = 0, n_layers = 0;
    double norm_eps = 0.0;
    int64_t vocab_size = 0;

    static ModelParams from_json(const std::string &text) {
        std::map<std::string, double> num;
        size_t p = 0;
        auto ws = [&] {
            while (p < text.size() && strchr(" \t\r\n", text[p])) p++;
        };
        auto fail = [&](const char *what) -> void { throw std::runtime_error(std::string("params.json: ") + what + " at byte " + std::to_string(p)); };
        auto str = [&] {
            std::string s;
            if (text[p] != '"') fail("expected a string");
            for (p++; p < text.size() && text[p] != '"'; p++) {
                if (text[p] == '\\' && p + 1 < text.size()) p++;
                s.push_back(text[p]);
            }
            if (p >= text.size()) fail("unterminated string");
            p++;
            return s;
        };
        ws();
        if (p >= text.size() || text[p] != '{') fail("expected an object");
        p++;
        for (;;) {
            ws();
            if (p < text.size() && text[p] == '}') break;
            const std::string key = str();
            ws();
            if (p >= text.size() || text[p] != ':') fail("expected ':'");
            p++;
            ws();
            if (p >= text.size()) fail("unexpected end");
            if (text[p] == '"') {
                (void)str();
            } else if (text[p] == '[' || text[p] == '{') { // skip a nested value by bracket depth (strings respected)
                int depth = 0;
                do {
                    if (text[p] == '"') {
                        (void)str();
                        continue;
                    }
                    if (text[p] == '[' || text[p] == '{') depth++;
                    if (text[p] == ']' || text[p] == '}') depth--;
                    p++;
                } while (depth > 0 && p < text.size());
            } else if (!strncmp(&text[p], "true", 4) || !strncmp(&text[p], "null", 4)) {
                p += 4;
            } else if (!strncmp(&text[p], "false", 5)) {
                p += 5;
            } else {
                char *end = nullptr;
                num[key] = strtod(&text[p], &end);
                if (end == &text[p]) fail("expected a value");
                p = (size_t)(end - text.data());
            }
            ws();
            if (p < text.size() && text[p] == ',') {
                p++;
                continue;
            }
            if (p < text.size() && text[p] == '}') break;
            fail("expected ',' or '}'");
        }
        auto get = [&](const char *a, const char *alias) {
            auto it = num.find(a);
            if (it == num.end() && alias) it = num.find(alias);
            if (it == num.end()) throw std::runtime_error(std::string("params.json: missing field ") + a);
            return it->second;
        };
        ModelParams m;
        m.dim = (size_t)get("dim", "hidden_size");
        m.n_heads = (size_t)get("n_heads", "num_attention_heads");
        m.n_layers = (size_t)get("n_layers", "num_hidden_layers");
        m.norm_eps = get("norm_eps", "rms_norm_eps");
        m.vocab_size = (int64_t)get("vocab_size", nullptr);
        return m;
    }
};

// DataSource::LLaMASource (src/data_source.rs:27-31): the model directory and the parsed data.pkl of every shard
class DataSource {
  public:
    static DataSource from_llama_source(const std::string &path) { // src/data_source.rs:166-197
        DataSource d;
        d.path_ = path;
        for (size_t part = 0;; part++) {
            const std::string pkl = shard_dir(path, part) + "/data.pkl";
            std::vector<uint8_t> bytes;
            if (!read_file(pkl, &bytes)) break; // the first missing shard ends the list
            unpickler::ValuePtr v = unpickler::unpickle(bytes);
            if (v->kind != unpickler::Value::Dict) throw unpickler::UnpicklingError(pkl + ": top-level value is not a dict");
            d.unpickled_.push_back(v);
        }
        return d;
    }
    static DataSource from_inferred_source(const std::string &path) { // src/data_source.rs:198-210 (LLaMA layout only)
        struct stat st {};
        if (stat((path + "/params.json").c_str(), &st) != 0) throw std::runtime_error(path + ": Unknown source (no params.json)");
        return from_llama_source(path);
    }
    const std::vector<unpickler::ValuePtr> &unpickled() const { return unpickled_; }
    const std::string &path() const { return path_; }
    ModelParams params() const {
        std::vector<uint8_t> bytes;
        if (!read_file(path_ + "/params.json", &bytes)) throw std::runtime_error(path_ + "/params.json: cannot read");
        return ModelParams::from_json(std::string(bytes.begin(), bytes.end()));
    }
    std::string data_file(size_t shard, const std::string &name) const { return shard_dir(path_, shard) + "/data/" + name; } // :105-111

    static bool read_file(const std::string &fn, std::vector<uint8_t> *out) {
        FILE *f = fopen(fn.c_str(), "rb");
        if (!f) {
            if (errno == ENOENT) return false;
            throw std::runtime_error(fn + ": " + strerror(errno));
        }
        uint8_t buf[1 << 16];
        size_t got;
        while ((got = fread(buf, 1, sizeof buf, f)) > 0) out->insert(out->end(), buf, buf + got);
        fclose(f);
        return true;
    }

  private:
    static std::string shard_dir(const std::string &path, size_t part) {
        char b[32];
        snprintf(b, sizeof b, "/consolidated.%02zu", part);
        return path + b;
    }
    std::string path_;
    std::vector<unpickler::ValuePtr> unpickled_;
};

// A tensor as f16 bits, put together from its shards (TensorBuilder::load_from_pieces, src/tensor.rs:2391-2546,
// without the widening to f32: the device model takes the file's bits as they are).
struct HalfMatrix {
    int64_t rows = 0, cols = 0;
    std::vector<uint16_t> bits;
};

inline HalfMatrix load_from_pieces(const DataSource &src, const std::string &name, FromPiecesDirection direction, bool first_shard_only = false) {
    std::vector<TensorBuilder> builders;
    for (const auto &shard : src.unpickled()) {
        const unpickler::Value *v = shard->get_str_key(name);
        if (!v) throw std::runtime_error("Missing field " + name);
        TensorBuilder b;
        if (!to_tensor_builder(*v, name, &b)) throw unpickler::UnpicklingError(name + ": data has incorrect format to be converted to a tensor");
        builders.push_back(b);
        if (first_shard_only) break; // from_unpickled_pieces1 (src/tensor.rs:309-329)
    }
    if (builders.empty()) throw std::runtime_error("Missing field " + name + " (no shards)");
    HalfMatrix m;
    for (const auto &b : builders) {
        if (b.stride < 1) throw std::runtime_error(name + ": invalid stride");
        // The pickle is untrusted input: BININT / BININT2 are signed, so every extent is checked before it sizes a buffer
        // or addresses a file (the reference reaches the same values through usize casts and slice bounds, which panic).
        if (b.rows <= 0 || b.cols <= 0 || b.offset < 0 || b.nitems < 0 || b.rows > INT32_MAX || b.cols > INT32_MAX ||
            b.offset + b.rows * b.cols > b.nitems) {
            throw std::runtime_error(name + ": shape " + std::to_string(b.rows) + "x" + std::to_string(b.cols) + " at offset " + std::to_string(b.offset) +
                                     " does not fit its storage of " + std::to_string(b.nitems) + " items");
        }
        // the storage key names a file inside consolidated.NN/data/ (src/data_source.rs:105-111), never a path
        if (b.src_path.empty() || b.src_path.find('/') != std::string::npos || b.src_path.find('\\') != std::string::npos || b.src_path == "." ||
            b.src_path == "..") {
            throw std::runtime_error(name + ": storage key '" + b.src_path + "' is not a plain file name");
        }
        if (direction == FromPiecesDirection::Rows) {
            if (b.cols != builders[0].cols) throw std::runtime_error(name + ": pieces differ in cols");
            m.rows += b.rows;
            m.cols = b.cols;
        } else {
            if (b.rows != builders[0].rows) throw std::runtime_error(name + ": pieces differ in rows");
            m.rows = b.rows;
            m.cols += b.cols;
        }
    }
    m.bits.resize((size_t)(m.rows * m.cols));
    int64_t row_off = 0, col_off = 0;
    std::vector<uint16_t> rowbuf;
    for (size_t s = 0; s < builders.size(); s++) {
        const TensorBuilder &b = builders[s];
        const std::string fn = src.data_file(s, b.src_path);
        FILE *f = fopen(fn.c_str(), "rb");
        if (!f) throw std::runtime_error(fn + ": " + strerror(errno));
        if (fseek(f, (long)(2 * b.offset), SEEK_SET) != 0) {
            fclose(f);
            throw std::runtime_error(fn + ": seek failed");
        }
        rowbuf.resize((size_t)b.cols);
        for (int64_t r = 0; r < b.rows; r++) { // row by row, like src/tensor.rs:2452-2480
            if (fread(rowbuf.data(), 2, (size_t)b.cols, f) != (size_t)b.cols) {
                fclose(f);
                throw std::runtime_error("path=" + fn + " row=" + std::to_string(r) + " expected_len=" + std::to_string(2 * b.cols) + " offset=" + std::to_string(b.offset));
            }
            memcpy(&m.bits[(size_t)((r + row_off) * m.cols + col_off)], rowbuf.data(), (size_t)b.cols * 2);
        }
        fclose(f);
        if (direction == FromPiecesDirection::Rows) row_off += b.rows;
        else col_off += b.cols;
    }
    return m;
}

// Model construction (src/rllama_main.rs:235-283, src/transformer.rs:242-326): every tensor of the directory that belongs on
// the device goes to the device model.  The FFN width comes from the stored shape of w1 (no params.json field).
inline std::unique_ptr<Transformer> load_transformer(const std::string &model_path, size_t max_seq_len, const DataSettings &data_settings,
                                                     ModelParams *params_out = nullptr) {
    const DataSource src = DataSource::from_inferred_source(model_path);
    const ModelParams mp = src.params();
    if (params_out) *params_out = mp;
    using D = FromPiecesDirection;
    const HalfMatrix w1_0 = load_from_pieces(src, "layers.0.feed_forward.w1.weight", D::Rows);
    auto tr = std::make_unique<Transformer>(mp.dim, mp.n_layers, mp.n_heads, (size_t)w1_0.rows, (size_t)mp.vocab_size, max_seq_len, mp.norm_eps, data_settings);
    auto put = [&](rlh_tensor_kind kind, int layer, const std::string &name, D dir, bool first) {
        const HalfMatrix m = load_from_pieces(src, name, dir, first);
        tr->set_tensor(kind, layer, m.bits.data(), (int)m.rows, (int)m.cols, TensorDType::Float16);
    };
    // With percentage_to_gpu below 1 only the leading layers live on the device (src/transformer.rs:262-279); the other
    // blocks, the embedding table and the output head are the host's, which reads them with load_from_pieces itself.
    const size_t n_device_layers = (size_t)tr->last_layer_on_gpu() + 1;
    const bool whole = n_device_layers == mp.n_layers;
    if (whole) put(RLH_TOK_EMB, 0, "tok_embeddings.weight", D::Cols, false); // src/embedding.rs:18-37
    put(RLH_NORM, 0, "norm.weight", D::Rows, true);                          // src/transformer.rs:297-298, 456-467
    if (whole) put(RLH_OUTPUT, 0, "output.weight", D::Rows, false);          // :303-308
    for (size_t l = 0; l < n_device_layers; l++) {
        const std::string p = "layers." + std::to_string(l) + ".";
        put(RLH_WQ, (int)l, p + "attention.wq.weight", D::Rows, false); // :595-614
        put(RLH_WK, (int)l, p + "attention.wk.weight", D::Rows, false);
        put(RLH_WV, (int)l, p + "attention.wv.weight", D::Rows, false);
        put(RLH_WO, (int)l, p + "attention.wo.weight", D::Cols, false);
        put(RLH_W1, (int)l, p + "feed_forward.w1.weight", D::Rows, false); // :490-503
        put(RLH_W2, (int)l, p + "feed_forward.w2.weight", D::Cols, false);
        put(RLH_W3, (int)l, p + "feed_forward.w3.weight", D::Rows, false);
        put(RLH_ATTN_NORM, (int)l, p + "attention_norm.weight", D::Rows, true); // :405-412
        put(RLH_FFN_NORM, (int)l, p + "ffn_norm.weight", D::Rows, true);
    }
    return tr;
}

} // namespace rllama

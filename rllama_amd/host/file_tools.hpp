// file_tools.hpp -- the device-free commands of the host example: what they print is what the tests compare.  They touch
// only the file readers (model_files.hpp: pickle subset, params.json, shard joining; tokenizer.hpp: SentencePiece model
// file), so a program made of them alone links without the library and can be built with the host sanitizers.
#pragma once

#include "model_files.hpp"
#include "tokenizer.hpp"

#include <cstdio>
#include <exception>

namespace rllama {
namespace tools {

// params.json and every data.pkl of a model directory: each tensor's name, joined shape and FNV-1a checksum
inline int inspect(const char *dir) {
    const DataSource src = DataSource::from_inferred_source(dir);
    const ModelParams mp = src.params();
    printf("params dim=%zu n_heads=%zu n_layers=%zu norm_eps=%g vocab_size=%lld shards=%zu\n", mp.dim, mp.n_heads, mp.n_layers, mp.norm_eps,
           (long long)mp.vocab_size, src.unpickled().size());
    if (src.unpickled().empty()) return 0;
    for (const auto &kv : src.unpickled()[0]->entries) {
        const std::string &name = kv.first;
        // how the reference joins the shards of this tensor (src/transformer.rs:490-503, 595-614; src/embedding.rs:37)
        const bool cols = name.find(".wo.") != std::string::npos || name.find(".w2.") != std::string::npos || name == "tok_embeddings.weight";
        const bool first = name.find("norm") != std::string::npos;
        const HalfMatrix m = load_from_pieces(src, name, cols ? FromPiecesDirection::Cols : FromPiecesDirection::Rows, first);
        uint64_t h = 1469598103934665603ull; // FNV-1a over the little-endian bytes
        for (uint16_t b : m.bits) {
            h = (h ^ (b & 0xff)) * 1099511628211ull;
            h = (h ^ (b >> 8)) * 1099511628211ull;
        }
        printf("tensor %s %lld %lld %016llx\n", name.c_str(), (long long)m.rows, (long long)m.cols, (unsigned long long)h);
    }
    return 0;
}

inline int tokenize(const char *model_file, const char *text) {
    const Tokenizer tok = Tokenizer::load(model_file);
    printf("ids:");
    for (TokenId t : tok.tokenize_to_ids(text)) printf(" %d", t);
    printf("\n");
    for (TokenId t : tok.tokenize_to_ids(text))
        if (t != 1) printf("piece %d %s\n", t, tok.id_to_str(t).c_str());
    return 0;
}

// one pickle file through the reader (src/unpickler.rs:317-675): the kind of its top-level value and, for a dict, its keys
inline int unpickle_file(const char *path) {
    std::vector<uint8_t> bytes;
    if (!DataSource::read_file(path, &bytes)) throw std::runtime_error(std::string(path) + ": cannot read");
    const unpickler::ValuePtr v = unpickler::unpickle(bytes);
    printf("kind %d\n", (int)v->kind);
    if (v->kind == unpickler::Value::Dict)
        for (const auto &kv : v->entries) printf("key %s\n", kv.first.c_str());
    return 0;
}

// runs a command; an exception becomes exit code 1 with its message on stderr
template <typename F>
inline int guarded(const char *prog, F &&f) {
    try {
        return f();
    } catch (const std::exception &e) {
        fprintf(stderr, "%s: %s\n", prog, e.what());
        return 1;
    }
}

} // namespace tools
} // namespace rllama

// tokenizer.hpp -- the reference's tokenizer (Noeda/rllama src/tokenizer.rs) for the C++ host mirror: reads a
// SentencePiece model file (protobuf ModelProto, proto/sentencepiece_model.proto:282-321; only the repeated
// SentencePiece {1: piece, 2: score, 3: type} of field 1 is looked at) and tokenizes by naive longest-prefix
// matching over the pieces.  The reference's quirks are kept: a position no piece matches is skipped one byte at a
// time and, if that lands inside a multi-byte character, the rest of the text is dropped (src/tokenizer.rs:157-159);
// a newline is the byte piece <0x0A> when the model has one and is dropped otherwise (:139-147); tokenize_to_ids puts
// U+2581 in front, turns spaces into U+2581 and starts with id 1 (:166-177).  Header-only, C++17.
#pragma once

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

namespace rllama {

using TokenId = int32_t;

struct TokenizerError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

enum class PieceType { Normal, Unknown, Control, UserDefined, Byte, Unused }; // src/tokenizer.rs:16-24

class Tokenizer {
  public:
    struct Piece {
        PieceType tp;
        float score;
        size_t idx;
    };

    static Tokenizer load(const std::string &path) { // src/tokenizer.rs:45-95
        FILE *f = fopen(path.c_str(), "rb");
        if (!f) throw TokenizerError("IO error: " + path);
        std::string bytes;
        char buf[1 << 16];
        size_t got;
        while ((got = fread(buf, 1, sizeof buf, f)) > 0) bytes.append(buf, got);
        fclose(f);
        return from_bytes(bytes);
    }

    static Tokenizer from_bytes(const std::string &model) {
        Tokenizer t;
        size_t idx = 0;
        for_each_field(model, [&](uint32_t field, int wt, uint64_t, const std::string &bytes) {
            if (field != 1 || wt != 2) return;
            bool has_piece = false;
            std::string piece;
            float score = 0.0f;
            uint64_t tp = 1; // default NORMAL
            for_each_field(bytes, [&](uint32_t f2, int wt2, uint64_t v2, const std::string &b2) {
                if (f2 == 1 && wt2 == 2) {
                    has_piece = true;
                    piece = b2;
                } else if (f2 == 2 && wt2 == 5) {
                    const uint32_t u = (uint32_t)v2;
                    memcpy(&score, &u, 4);
                } else if (f2 == 3 && wt2 == 0) {
                    tp = v2;
                }
            });
            if (has_piece) { // a piece without a string is skipped but still counts for the ids (:52-57)
                PieceType pt;
                switch (tp) { // sentence_piece::Type, proto/sentencepiece_model.proto:284-293
                case 1: pt = PieceType::Normal; break;
                case 2: pt = PieceType::Unknown; break;
                case 3: pt = PieceType::Control; break;
                case 4: pt = PieceType::UserDefined; break;
                case 6: pt = PieceType::Byte; break;
                case 5: pt = PieceType::Unused; break;
                default: throw TokenizerError("Unknown piece type: " + piece);
                }
                t.pieces_[piece] = Piece{pt, score, idx}; // a repeated string keeps the later entry
            }
            idx++;
        });
        return t;
    }

    size_t size() const { return pieces_.size(); }

    const std::string &id_to_str(TokenId id) const { // :99-107; throws where the reference panics
        for (const auto &kv : pieces_)
            if (kv.second.idx == (size_t)id) return kv.first;
        throw TokenizerError("id out of range");
    }
    bool str_to_id(const std::string &s, TokenId *id) const { // :110-117
        auto it = pieces_.find(s);
        if (it == pieces_.end()) return false;
        *id = (TokenId)it->second.idx;
        return true;
    }

    std::vector<std::string> tokenize_to_pieces(const std::string &text) const { // :127-164
        std::vector<std::string> out;
        const bool have_nl = pieces_.count("<0x0A>") != 0;
        size_t p = 0;
        const size_t n = text.size();
        while (p < n) {
            const std::string *best = nullptr;
            static const std::string nl = "<0x0A>";
            size_t advance = 0;
            if (text[p] == '\n') {
                if (have_nl) {
                    best = &nl;
                    advance = 1;
                }
            } else {
                size_t best_len = 0;
                for (const auto &kv : pieces_) {
                    const std::string &piece = kv.first;
                    if (piece.size() > best_len && text.compare(p, piece.size(), piece) == 0) {
                        best = &piece;
                        best_len = piece.size();
                        advance = piece.size();
                    }
                }
            }
            if (!best) {
                // one byte on; if that is not a character boundary the reference's str::get gives None and the rest is dropped
                if (p + 1 < n && ((unsigned char)text[p + 1] & 0xC0) != 0x80) p += 1;
                else p = n;
            } else {
                out.push_back(*best);
                p += advance;
            }
        }
        return out;
    }

    std::vector<TokenId> tokenize_to_ids(const std::string &text) const { // :166-177
        std::string s = "\xe2\x96\x81";
        for (char c : text) {
            if (c == ' ') s += "\xe2\x96\x81";
            else s.push_back(c);
        }
        std::vector<TokenId> ids{1};
        for (const std::string &piece : tokenize_to_pieces(s)) ids.push_back((TokenId)pieces_.at(piece).idx);
        return ids;
    }

  private:
    // one protobuf message: fn(field, wire type, integer value, bytes) per field; unknown wire types are an error
    template <typename Fn>
    static void for_each_field(const std::string &b, Fn fn) {
        size_t p = 0;
        auto varint = [&]() {
            uint64_t v = 0;
            for (int shift = 0;; shift += 7) {
                if (p >= b.size() || shift > 63) throw TokenizerError("Protobuf error: bad varint");
                const unsigned char c = (unsigned char)b[p++];
                v |= (uint64_t)(c & 0x7f) << shift;
                if (!(c & 0x80)) return v;
            }
        };
        static const std::string empty;
        while (p < b.size()) {
            const uint64_t key = varint();
            const uint32_t field = (uint32_t)(key >> 3);
            const int wt = (int)(key & 7);
            if (wt == 0) {
                fn(field, wt, varint(), empty);
            } else if (wt == 1 || wt == 5) {
                const size_t len = wt == 1 ? 8 : 4;
                if (p + len > b.size()) throw TokenizerError("Protobuf error: truncated fixed field");
                uint64_t v = 0;
                memcpy(&v, b.data() + p, len); // little-endian host
                p += len;
                fn(field, wt, v, empty);
            } else if (wt == 2) {
                const uint64_t len = varint();
                if (p + len > b.size()) throw TokenizerError("Protobuf error: truncated field");
                fn(field, wt, 0, b.substr(p, (size_t)len));
                p += (size_t)len;
            } else {
                throw TokenizerError("Protobuf error: unsupported wire type " + std::to_string(wt));
            }
        }
    }
    std::map<std::string, Piece> pieces_; // ordered by bytes like the reference's BTreeMap<String, Piece>
};

} // namespace rllama

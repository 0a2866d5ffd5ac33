// generate_main.cpp -- the reference's token loop (command_line_inference, Noeda/rllama src/rllama_main.rs:714-923)
// over the C++ mirror, on a synthetic random-init model: prompt ids in, greedy ids out, ms/token printed the way
// the reference prints it (first token apart, then the mean over the rest; src/rllama_main.rs:908-917).
//
//   rllama_generate [dim n_layers n_heads ffn_hidden vocab n_prompt n_new [seed]]
//   rllama_generate --model-path DIR [n_prompt n_new [seed]]     weights from a LLaMA-format directory (--model-path of
//                                                                 src/rllama_main.rs:44-45); prompt ids are synthetic
//   ... --sample TOP_K TEMPERATURE TOP_P REPETITION_PENALTY      (before the other arguments) token loop with
//                                                                 TokenSampler instead of the device-resident greedy loop
//   rllama_generate --tokenize TOKENIZER_MODEL TEXT              no device needed: prints the ids of Tokenizer::tokenize_to_ids
//                                                                 and the pieces (src/tokenizer.rs:127-177)
//   rllama_generate --inspect DIR                                 no device needed: parses params.json and every data.pkl
//                                                                 and prints each tensor's name, shape and a checksum
//
// It exists to show (and to compile-check in every build) that the header-only host layer needs nothing but
// the C ABI.  Exits non-zero with the library's message if there is no gfx950 device.
#include "file_tools.hpp"
#include "model_files.hpp"
#include "rllama_hip.hpp"
#include "tokenizer.hpp"

#include <cstdio>
#include <cstdlib>
#include <random>

int main(int argc, char **argv) {
    if (argc >= 3 && std::string(argv[1]) == "--inspect") return rllama::tools::guarded("rllama_generate", [&] { return rllama::tools::inspect(argv[2]); });
    if (argc >= 4 && std::string(argv[1]) == "--tokenize") return rllama::tools::guarded("rllama_generate", [&] { return rllama::tools::tokenize(argv[2], argv[3]); });
    bool use_sampler = false;
    rllama::TokenSampler sampler;
    if (argc >= 6 && std::string(argv[1]) == "--sample") {
        use_sampler = true;
        sampler = sampler.top_k(strtoul(argv[2], nullptr, 10)).temperature(strtof(argv[3], nullptr)).top_p(strtof(argv[4], nullptr)).repetition_penalty(strtof(argv[5], nullptr));
        argv += 5;
        argc -= 5;
    }
    const char *model_path = nullptr;
    if (argc >= 3 && std::string(argv[1]) == "--model-path") {
        model_path = argv[2];
        argv += 2;
        argc -= 2;
    }
    size_t dim = 1024, n_layers = 8, n_heads = 16, ffn = 2816, vocab = 32000, n_prompt = 16, n_new = 64;
    uint64_t seed = 0;
    if (model_path) {
        if (argc >= 3) {
            n_prompt = strtoul(argv[1], nullptr, 10);
            n_new = strtoul(argv[2], nullptr, 10);
        }
        if (argc >= 4) seed = strtoull(argv[3], nullptr, 10);
        argc = 0;
    }
    if (argc >= 8) {
        dim = strtoul(argv[1], nullptr, 10);
        n_layers = strtoul(argv[2], nullptr, 10);
        n_heads = strtoul(argv[3], nullptr, 10);
        ffn = strtoul(argv[4], nullptr, 10);
        vocab = strtoul(argv[5], nullptr, 10);
        n_prompt = strtoul(argv[6], nullptr, 10);
        n_new = strtoul(argv[7], nullptr, 10);
    }
    if (argc >= 9) seed = strtoull(argv[8], nullptr, 10);
    try {
        auto cl = std::make_shared<rllama::OpenCL>(true, 0);
        rllama::DataSettings ds = rllama::DataSettings(cl).force_f16().percentage_to_gpu(1.0f);
        std::unique_ptr<rllama::Transformer> loaded;
        if (model_path) {
            rllama::ModelParams mp;
            loaded = rllama::load_transformer(model_path, n_prompt + n_new, ds, &mp);
            vocab = (size_t)mp.vocab_size;
        } else {
            loaded = std::make_unique<rllama::Transformer>(dim, n_layers, n_heads, ffn, vocab, n_prompt + n_new, 1e-6, ds);
            loaded->fill_synthetic(seed, 0.02);
        }
        rllama::Transformer &tr = *loaded;
        std::vector<rllama::TokenId> prompt(n_prompt);
        rlh_synth_tokens(seed, 0, n_prompt, 3, (int32_t)vocab, prompt.data());
        rllama::TransformerCaches caches = tr.make_caches();
        float ms_first = 0.0f, ms_tok = 0.0f;
        std::vector<rllama::TokenId> out;
        if (!use_sampler) {
            out = tr.generate_greedy(prompt, n_new, caches, &ms_first, &ms_tok);
        } else { // the reference's loop: forward over the new tokens, sample with the tokens so far (src/rllama_main.rs:821-897)
            std::mt19937 rng((uint32_t)seed);
            std::uniform_real_distribution<float> uni(0.0f, 1.0f);
            std::vector<rllama::TokenId> toks = prompt, feed = prompt;
            size_t pos = 0;
            for (size_t i = 0; i < n_new; i++) {
                auto [tok, prob] = tr.forward_sample(feed, pos, caches, sampler.raw(), toks, uni(rng));
                (void)prob;
                pos += feed.size();
                feed.assign(1, tok);
                toks.push_back(tok);
                out.push_back(tok);
            }
        }
        printf("tokens:");
        for (rllama::TokenId t : out) printf(" %d", t);
        printf("\nTime taken to generate first token: %.0fms\n", ms_first);
        printf("Time taken per token (excluding first token): %.3fms\n", ms_tok);
    } catch (const rllama::Error &e) {
        fprintf(stderr, "rllama_generate: %s (status %d)\n", e.what(), e.code);
        return 1;
    } catch (const std::exception &e) {
        fprintf(stderr, "rllama_generate: %s\n", e.what());
        return 1;
    }
    return 0;
}

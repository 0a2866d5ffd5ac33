// generate_main.cpp -- the reference's token loop (command_line_inference, Noeda/rllama src/rllama_main.rs:714-923)
// over the C++ mirror, on a synthetic random-init model: prompt ids in, greedy ids out, ms/token printed the way
// the reference prints it (first token apart, then the mean over the rest; src/rllama_main.rs:908-917).
//
//   rllama_generate [dim n_layers n_heads ffn_hidden vocab n_prompt n_new [seed]]
//
// It exists to show (and to compile-check in every build) that the header-only host layer needs nothing but
// the C ABI.  Exits non-zero with the library's message if there is no gfx950 device.
#include "rllama_hip.hpp"

#include <cstdio>
#include <cstdlib>

int main(int argc, char **argv) {
    size_t dim = 1024, n_layers = 8, n_heads = 16, ffn = 2816, vocab = 32000, n_prompt = 16, n_new = 64;
    uint64_t seed = 0;
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
        rllama::Transformer tr(dim, n_layers, n_heads, ffn, vocab, n_prompt + n_new, 1e-6, ds);
        tr.fill_synthetic(seed, 0.02);
        std::vector<rllama::TokenId> prompt(n_prompt);
        rlh_synth_tokens(seed, 0, n_prompt, 3, (int32_t)vocab, prompt.data());
        rllama::TransformerCaches caches = tr.make_caches();
        float ms_first = 0.0f, ms_tok = 0.0f;
        std::vector<rllama::TokenId> out = tr.generate_greedy(prompt, n_new, caches, &ms_first, &ms_tok);
        printf("tokens:");
        for (rllama::TokenId t : out) printf(" %d", t);
        printf("\nTime taken to generate first token: %.0fms\n", ms_first);
        printf("Time taken per token (excluding first token): %.3fms\n", ms_tok);
    } catch (const rllama::Error &e) {
        fprintf(stderr, "rllama_generate: %s (status %d)\n", e.what(), e.code);
        return 1;
    }
    return 0;
}

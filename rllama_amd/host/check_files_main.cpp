// check_files_main.cpp -- the file readers of the host layer as a program of their own (no device, no library):
//
//   rllama_check_files inspect DIR            params.json + every data.pkl: tensor names, joined shapes, checksums
//   rllama_check_files unpickle FILE          one pickle file through the reader
//   rllama_check_files tokenize MODEL TEXT    SentencePiece model file + the reference's tokenizer
//
// Same output as the matching modes of rllama_generate.  Built with -fsanitize=address,undefined by
// `python -m rllama_amd.build --host-asan`, so that the parsers of untrusted bytes run under the sanitizers on the test-suite's
// damaged inputs.  Exit codes: 0 ok, 1 the reader refused the input (message on stderr), 2 usage.
#include "file_tools.hpp"

#include <string>

int main(int argc, char **argv) {
    using namespace rllama::tools;
    const std::string cmd = argc >= 2 ? argv[1] : "";
    if (cmd == "inspect" && argc == 3) return guarded("rllama_check_files", [&] { return inspect(argv[2]); });
    if (cmd == "unpickle" && argc == 3) return guarded("rllama_check_files", [&] { return unpickle_file(argv[2]); });
    if (cmd == "tokenize" && argc == 4) return guarded("rllama_check_files", [&] { return tokenize(argv[2], argv[3]); });
    fprintf(stderr, "usage: rllama_check_files inspect DIR | unpickle FILE | tokenize MODEL TEXT\n");
    return 2;
}

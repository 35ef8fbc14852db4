// Header parser of the Bert_model_weights mirror on its own (no GPU): reads the JSON header of the safetensors file argv[1]
// and prints, for every tensor name in argv[2..], "<name> <begin> <end>" from parseKeyFromString, or "<name> none".
#include <cstdio>
#include <fstream>
#include <string>

#include "../../include/ckks_llm_amd_bert.hpp"

int main(int argc, char** argv) {
    if (argc < 2) return 2;
    std::ifstream f(argv[1], std::ios::binary);
    uint64_t n = 0;
    f.read(reinterpret_cast<char*>(&n), 8);
    std::string header(n, '\0');
    f.read(&header[0], (std::streamsize)n);
    if (!f) { printf("unreadable\n"); return 1; }
    ckks_llm_amd::Bert_model_weights w("/nonexistent-directory/");          // no file: nothing is allocated, the parser is all that is used
    for (int i = 2; i < argc; i++) {
        int64_t a = 0, b = 0;
        if (w.parseKeyFromString(header, argv[i], a, b)) printf("%s %lld %lld\n", argv[i], (long long)a, (long long)b);
        else printf("%s none\n", argv[i]);
    }
    return 0;
}

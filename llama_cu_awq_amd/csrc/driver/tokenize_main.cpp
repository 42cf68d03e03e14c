// Small tool around the driver's tokenizer (used by the tests; same output format as oracle/ref_tokenizer_main.cpp):
//   tokenize <tokenizer.bin> <vocab_size>    stdin: one text per line, "\n" written as \\n
#include <stdio.h>
#include <stdlib.h>

#include <string>

#include "tokenizer.hpp"

int main(int argc, char** argv) {
    if (argc != 3) return 2;
    awqcli::Tokenizer t;
    if (!t.load(argv[1], atoi(argv[2]))) return 1;
    char line[1 << 16];
    while (fgets(line, sizeof(line), stdin)) {
        std::string s(line);
        if (!s.empty() && s.back() == '\n') s.pop_back();
        std::string text;
        for (size_t i = 0; i < s.size(); i++) {
            if (s[i] == '\\' && i + 1 < s.size() && s[i + 1] == 'n') { text.push_back('\n'); i++; }
            else text.push_back(s[i]);
        }
        std::vector<int> toks = t.encode(text, true, false);
        printf("E");
        for (int id : toks) printf(" %d", id);
        printf("\n");
        for (size_t i = 0; i + 1 < toks.size(); i++) {
            std::string piece = t.decode(toks[i], toks[i + 1]);
            printf("D %d %d ", toks[i], toks[i + 1]);
            for (unsigned char c : piece) printf("%02x", c);
            printf("\n");
        }
    }
    return 0;
}

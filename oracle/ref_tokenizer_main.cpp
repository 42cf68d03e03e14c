// Test infrastructure: prints what the REFERENCE's tokenizer (tokenizer.h, included from the reference checkout,
// never copied) makes of each line of stdin.  Built by oracle/Makefile into oracle/_ref/ref_tokenizer.
//   usage: ref_tokenizer <tokenizer.bin> <vocab_size>     stdin: one text per line ("\n" inside a text as \\n)
//   output per line: "E id id id ..." then one "D <prev> <tok> <hex bytes of decode(prev,tok)>" per adjacent pair
#include <ctype.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string>

#include "tokenizer.h"

int main(int argc, char** argv) {
    if (argc != 3) return 2;
    Tokenizer t;
    build_tokenizer(&t, argv[1], atoi(argv[2]));
    char line[1 << 16];
    while (fgets(line, sizeof(line), stdin)) {
        std::string s(line);
        if (!s.empty() && s.back() == '\n') s.pop_back();
        std::string text;
        for (size_t i = 0; i < s.size(); i++) {
            if (s[i] == '\\' && i + 1 < s.size() && s[i + 1] == 'n') { text.push_back('\n'); i++; }
            else text.push_back(s[i]);
        }
        int* toks = (int*)malloc((text.size() + 3) * sizeof(int));
        int n = 0;
        encode(&t, (char*)text.c_str(), 1, 0, toks, &n);
        printf("E");
        for (int i = 0; i < n; i++) printf(" %d", toks[i]);
        printf("\n");
        for (int i = 0; i + 1 < n; i++) {
            char* piece = decode(&t, toks[i], toks[i + 1]);
            printf("D %d %d ", toks[i], toks[i + 1]);
            for (char* p = piece; *p; p++) printf("%02x", (unsigned char)*p);
            printf("\n");
        }
        free(toks);
    }
    return 0;
}

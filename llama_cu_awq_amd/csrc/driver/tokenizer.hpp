// Byte-fallback BPE tokenizer over a llama2.c-format tokenizer.bin (the file the reference ships and its
// tokenizer.h reads: uint32 max_token_length, then per token {float score, int32 len, bytes}).
// Same observable behaviour as the reference's build_tokenizer / encode / decode / safe_printf
// (tokenizer.h:35-223); the implementation is this project's own (a vector of (string, id) pairs sorted once with
// std::stable_sort and searched by bisection, where the reference calls qsort and bsearch).
#pragma once

#include <ctype.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <string>
#include <utility>
#include <vector>

namespace awqcli {

constexpr int kBosToken = 1;  // tokenizer.h:9-10
constexpr int kEosToken = 2;

class Tokenizer {
  public:
    // Returns false (with a message on stderr) when the file cannot be read (tokenizer.h:46-55).
    bool load(const char* path, int vocab_size) {
        FILE* f = fopen(path, "rb");
        if (!f) {
            fprintf(stderr, "couldn't load %s\n", path);
            return false;
        }
        uint32_t max_len = 0;
        bool ok = fread(&max_len, sizeof(uint32_t), 1, f) == 1;
        vocab_.resize(vocab_size);
        scores_.resize(vocab_size);
        for (int i = 0; ok && i < vocab_size; i++) {
            int32_t len = 0;
            ok = fread(&scores_[i], sizeof(float), 1, f) == 1 && fread(&len, sizeof(int32_t), 1, f) == 1 && len >= 0 && len < (1 << 20);
            if (ok) {
                vocab_[i].resize(len);
                ok = len == 0 || fread(&vocab_[i][0], len, 1, f) == 1;
            }
        }
        fclose(f);
        if (!ok) {
            fprintf(stderr, "failed read\n");
            return false;
        }
        sorted_.clear();
        for (int i = 0; i < vocab_size; i++) sorted_.emplace_back(vocab_[i], i);
        std::stable_sort(sorted_.begin(), sorted_.end(),
                         [](const std::pair<std::string, int>& a, const std::pair<std::string, int>& b) { return strcmp(a.first.c_str(), b.first.c_str()) < 0; });
        return true;
    }

    int lookup(const std::string& s) const {
        size_t l = 0, u = sorted_.size();
        while (l < u) {
            const size_t idx = (l + u) / 2;
            const int cmp = strcmp(s.c_str(), sorted_[idx].first.c_str());
            if (cmp < 0) u = idx;
            else if (cmp > 0) l = idx + 1;
            else return sorted_[idx].second;
        }
        return -1;
    }

    // encode(): optional BOS, dummy-prefix space for non-empty text, one token per UTF-8 code point (bytes + 3
    // when the code point is not in the vocabulary), then repeatedly merge the adjacent pair with the best score.
    std::vector<int> encode(const std::string& text, bool bos, bool eos) const {
        std::vector<int> toks;
        if (bos) toks.push_back(kBosToken);
        if (!text.empty()) toks.push_back(lookup(" "));
        std::string cp;
        for (size_t i = 0; i < text.size(); i++) {
            const unsigned char c = (unsigned char)text[i];
            if ((c & 0xC0) != 0x80) cp.clear();  // not a continuation byte: a new code point starts
            cp.push_back((char)c);
            const bool next_is_cont = i + 1 < text.size() && (((unsigned char)text[i + 1]) & 0xC0) == 0x80;
            if (next_is_cont && cp.size() < 4) continue;
            const int id = lookup(cp);
            if (id != -1) {
                toks.push_back(id);
            } else {
                for (unsigned char b : cp) toks.push_back((int)b + 3);  // <unk>, <s>, </s> come first
            }
            cp.clear();
        }
        while (true) {
            float best_score = -1e10f;
            int best_id = -1, best_idx = -1;
            for (size_t i = 0; i + 1 < toks.size(); i++) {
                const int id = lookup(vocab_[toks[i]] + vocab_[toks[i + 1]]);
                if (id != -1 && scores_[id] > best_score) {
                    best_score = scores_[id];
                    best_id = id;
                    best_idx = (int)i;
                }
            }
            if (best_idx == -1) break;
            toks[best_idx] = best_id;
            toks.erase(toks.begin() + best_idx + 1);
        }
        if (eos) toks.push_back(kEosToken);
        return toks;
    }

    // decode(): the piece of `token`; a leading space is dropped right after BOS; "<0xXX>" pieces are raw bytes.
    std::string decode(int prev_token, int token) const {
        if (token < 0 || token >= (int)vocab_.size()) return std::string();
        const std::string& p = vocab_[token];
        const char* piece = p.c_str();
        if (prev_token == kBosToken && piece[0] == ' ') piece++;
        unsigned char byte_val;
        if (sscanf(piece, "<0x%02hhX>", &byte_val) == 1) return std::string(1, (char)byte_val);
        return std::string(piece);
    }

    // safe_printf(): skip single bytes that are neither printable nor white space.
    static void safe_print(const std::string& piece) {
        if (piece.empty()) return;
        if (piece.size() == 1) {
            const unsigned char b = (unsigned char)piece[0];
            if (!(isprint(b) || isspace(b))) return;
        }
        fputs(piece.c_str(), stdout);
    }

    const std::string& piece(int i) const { return vocab_[i]; }

  private:
    std::vector<std::string> vocab_;
    std::vector<float> scores_;
    std::vector<std::pair<std::string, int>> sorted_;  // vocabulary in strcmp order (stable)
};

}  // namespace awqcli

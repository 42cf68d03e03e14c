// weight_packer: AWQ checkpoint tensors (one raw .bin file per tensor) -> the single model .bin that llama2_q4 loads.
//
//   weight_packer <config.json from huggingface> <path_to_awq_bin_weights> <output_bin_filename> <OldAwqFormat: 0 or 1>
//
// Same command line, input file names and output layout as the reference's tool (weight_packer.cpp:233-292):
// 32-byte header (7 int32 + float rope_theta), embedding, lm_head, final norm, then per layer q, k, v, o, up, gate,
// down (each: packed weights, packed zeros, scales) and the two norm vectors.
//
// Old AWQ format (1): qweight [K][N/8] and qzeros [G][N/8] hold 8 columns per dword in AWQ's interleaved nibble order
// (nibble i is column 8j + {0,2,4,6,1,3,5,7}[i], weight_packer.cpp:96-107), scales are [G][N]; all three are
// transposed to one row per output column with 8 consecutive K (or groups) per dword, low nibble first.
// New format (0): already in that layout, except that each scale row is padded to a multiple of 8 groups.
//
// Differences from the reference tool, on purpose: config.json keys are found with any whitespace around the colon;
// every input file's size is checked against what the shape demands; dimensions the loader cannot read back
// (dim or hidden_dim not a multiple of 32: the loader's row stride is ceil(K/32)*4 dwords, llama2_q4.cu:106-112)
// are rejected instead of producing an unreadable file; padding nibbles of the last zeros dword are zero instead
// of whatever lay behind the buffer (weight_packer.cpp:117-121).
#include <ctype.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

namespace {

constexpr int kGroupSize = 128;

struct Config {
    int dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len;
    float rope_theta;
};

[[noreturn]] void die(const std::string& msg) {
    fprintf(stderr, "weight_packer: %s\n", msg.c_str());
    exit(1);
}

// value text after "key" <ws> : <ws>, or nullptr
const char* find_value(const std::string& json, const char* key) {
    const std::string quoted = std::string("\"") + key + "\"";
    size_t at = 0;
    while ((at = json.find(quoted, at)) != std::string::npos) {
        size_t p = at + quoted.size();
        while (p < json.size() && isspace((unsigned char)json[p])) p++;
        if (p < json.size() && json[p] == ':') {
            p++;
            while (p < json.size() && isspace((unsigned char)json[p])) p++;
            return json.c_str() + p;
        }
        at += quoted.size();
    }
    return nullptr;
}

int need_int(const std::string& json, const char* key) {
    const char* v = find_value(json, key);
    if (!v) die(std::string("config.json: ") + key + " not found");
    return atoi(v);
}

Config read_config(const char* path) {
    FILE* f = fopen(path, "rb");
    if (!f) die(std::string("unable to open config file ") + path);
    std::string json;
    char buf[65536];
    size_t n;
    while ((n = fread(buf, 1, sizeof(buf), f)) > 0) json.append(buf, n);
    fclose(f);
    if (json.empty()) die("unable to read config file");
    Config c;
    c.dim = need_int(json, "hidden_size");
    c.hidden_dim = need_int(json, "intermediate_size");
    c.n_layers = need_int(json, "num_hidden_layers");
    c.n_heads = need_int(json, "num_attention_heads");
    const char* kv = find_value(json, "num_key_value_heads");
    c.n_kv_heads = kv ? atoi(kv) : c.n_heads;
    c.vocab_size = need_int(json, "vocab_size");
    c.seq_len = need_int(json, "max_position_embeddings");
    const char* th = find_value(json, "rope_theta");
    c.rope_theta = th ? (float)atof(th) : 10000.0f;
    printf("\nModel params:- \ndim: %d \nhidden_dim: %d\nn_heads: %d\nn_kv_heads: %d\nn_layers: %d\nseq_len: %d\nvocab_size: %d\nrope_theta: %g\n",
           c.dim, c.hidden_dim, c.n_heads, c.n_kv_heads, c.n_layers, c.seq_len, c.vocab_size, c.rope_theta);
    if (c.dim <= 0 || c.hidden_dim <= 0 || c.n_layers <= 0 || c.n_heads <= 0 || c.n_kv_heads <= 0 || c.vocab_size <= 0 || c.seq_len <= 0)
        die("config.json: non-positive model dimension");
    if (c.dim % 32 || c.hidden_dim % 32) die("dim and hidden_dim must be multiples of 32 (the loader's packed row stride)");
    if (c.dim % c.n_heads || c.n_heads % c.n_kv_heads) die("head counts do not divide the model dimension");
    return c;
}

std::vector<uint8_t> read_exact(const std::string& path, size_t bytes) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) die("unable to open " + path);
    fseek(f, 0, SEEK_END);
    const long have = ftell(f);
    fseek(f, 0, SEEK_SET);
    if (have < 0 || (size_t)have != bytes)
        die(path + ": holds " + std::to_string(have) + " bytes, the model shape needs " + std::to_string(bytes));
    std::vector<uint8_t> data(bytes);
    if (bytes && fread(data.data(), 1, bytes, f) != bytes) die("error reading " + path);
    fclose(f);
    return data;
}

void write_all(FILE* out, const void* p, size_t bytes, const char* what) {
    if (bytes && fwrite(p, 1, bytes, out) != bytes) die(std::string("error writing ") + what);
}

void copy_tensor(FILE* out, const std::string& path, size_t bytes) {
    const std::vector<uint8_t> d = read_exact(path, bytes);
    write_all(out, d.data(), bytes, path.c_str());
}

int div_up(int a, int b) { return (a + b - 1) / b; }

// in: [rows][cols/8] dwords in AWQ nibble order; out: [cols][ceil(rows/8)] dwords, element r of column c in nibble
// r % 8 of dword r / 8 (missing rows: zero nibbles)
std::vector<uint32_t> transpose_nibbles(const uint32_t* in, int rows, int cols) {
    static const int nibble_of_column[8] = {0, 4, 1, 5, 2, 6, 3, 7};  // inverse of {0,2,4,6,1,3,5,7}
    const int in_w = cols / 8, out_w = div_up(rows, 8);
    std::vector<uint32_t> out((size_t)cols * out_w, 0u);
    for (int r = 0; r < rows; r++) {
        const uint32_t* src = in + (size_t)r * in_w;
        const int shift = 4 * (r & 7);
        for (int c = 0; c < cols; c++) {
            const uint32_t q = (src[c >> 3] >> (4 * nibble_of_column[c & 7])) & 0xFu;
            out[(size_t)c * out_w + (r >> 3)] |= q << shift;
        }
    }
    return out;
}

// K = inputs (reduction length), N = outputs
void pack_matrix(FILE* out, const std::string& base, const char* name, int K, int N, bool old_format) {
    const int G = div_up(K, kGroupSize), pwh = div_up(K, 8), pzh = div_up(G, 8);
    const std::string stem = base + "." + name;
    if (N % 8) die(stem + ": output dimension must be a multiple of 8");
    if (old_format) {
        const std::vector<uint8_t> qw = read_exact(stem + ".qweight.bin", (size_t)K * (N / 8) * 4);
        const std::vector<uint8_t> qz = read_exact(stem + ".qzeros.bin", (size_t)G * (N / 8) * 4);
        const std::vector<uint8_t> sc = read_exact(stem + ".scales.bin", (size_t)G * N * 2);
        const std::vector<uint32_t> w = transpose_nibbles(reinterpret_cast<const uint32_t*>(qw.data()), K, N);
        const std::vector<uint32_t> z = transpose_nibbles(reinterpret_cast<const uint32_t*>(qz.data()), G, N);
        std::vector<uint16_t> s((size_t)N * G);
        const uint16_t* sin = reinterpret_cast<const uint16_t*>(sc.data());
        for (int g = 0; g < G; g++)
            for (int n = 0; n < N; n++) s[(size_t)n * G + g] = sin[(size_t)g * N + n];
        write_all(out, w.data(), w.size() * 4, stem.c_str());
        write_all(out, z.data(), z.size() * 4, stem.c_str());
        write_all(out, s.data(), s.size() * 2, stem.c_str());
    } else {
        const int padded_G = pzh * 8;  // the AWQ exporter pads each scale row to a multiple of 8 groups
        const std::vector<uint8_t> qw = read_exact(stem + ".qweight.bin", (size_t)N * pwh * 4);
        const std::vector<uint8_t> qz = read_exact(stem + ".qzeros.bin", (size_t)N * pzh * 4);
        const std::vector<uint8_t> sc = read_exact(stem + ".scales.bin", (size_t)N * padded_G * 2);
        std::vector<uint16_t> s((size_t)N * G);
        const uint16_t* sin = reinterpret_cast<const uint16_t*>(sc.data());
        for (int n = 0; n < N; n++)
            for (int g = 0; g < G; g++) s[(size_t)n * G + g] = sin[(size_t)n * padded_G + g];
        write_all(out, qw.data(), qw.size(), stem.c_str());
        write_all(out, qz.data(), qz.size(), stem.c_str());
        write_all(out, s.data(), s.size() * 2, stem.c_str());
    }
}

}  // namespace

int main(int argc, char* argv[]) {
    if (argc != 5) {
        printf("usage: weight_packer <config.json from huggingface> <path_to_awq_bin_weights> <output_bin_filename> [OldAwqFormat: 0 or 1]\n");
        return 0;
    }
    const Config cfg = read_config(argv[1]);
    const std::string dir = argv[2];
    const bool old_format = atoi(argv[4]) != 0;
    FILE* out = fopen(argv[3], "wb");
    if (!out) die(std::string("unable to open output file ") + argv[3]);
    static_assert(sizeof(Config) == 32, "the file header is 7 int32 and one float");
    write_all(out, &cfg, sizeof(cfg), "header");
    const size_t vd = (size_t)cfg.vocab_size * cfg.dim * 2;
    copy_tensor(out, dir + "/model.embed_tokens.weight.bin", vd);
    copy_tensor(out, dir + "/lm_head.weight.bin", vd);
    copy_tensor(out, dir + "/model.norm.weight.bin", (size_t)cfg.dim * 2);
    const int kv_dim = cfg.dim * cfg.n_kv_heads / cfg.n_heads;
    for (int l = 0; l < cfg.n_layers; l++) {
        printf("\nProcessing weights for layer: %d\n", l);
        const std::string base = dir + "/model.layers." + std::to_string(l);
        pack_matrix(out, base, "self_attn.q_proj", cfg.dim, cfg.dim, old_format);
        pack_matrix(out, base, "self_attn.k_proj", cfg.dim, kv_dim, old_format);
        pack_matrix(out, base, "self_attn.v_proj", cfg.dim, kv_dim, old_format);
        pack_matrix(out, base, "self_attn.o_proj", cfg.dim, cfg.dim, old_format);
        pack_matrix(out, base, "mlp.up_proj", cfg.dim, cfg.hidden_dim, old_format);
        pack_matrix(out, base, "mlp.gate_proj", cfg.dim, cfg.hidden_dim, old_format);
        pack_matrix(out, base, "mlp.down_proj", cfg.hidden_dim, cfg.dim, old_format);
        copy_tensor(out, base + ".input_layernorm.weight.bin", (size_t)cfg.dim * 2);
        copy_tensor(out, base + ".post_attention_layernorm.weight.bin", (size_t)cfg.dim * 2);
    }
    if (fclose(out) != 0) die("error closing the output file");
    printf("\nDone!\n");
    return 0;
}

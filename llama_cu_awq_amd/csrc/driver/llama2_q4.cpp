// llama2_q4: command-line driver with the reference's flags, banners and loop (llama2_q4.cu:683-936), on top of
// libawq_hip.so.  One GPU; `-x` other than "none" is rejected with a message.
//
//   llama2_q4 <checkpoint> [-n steps] [-i prompt] [-f prompt_file] [-t temperature] [-p top_p] [-s seed]
//             [-z tokenizer] [-y system_prompt] [-x none] [-q dataset]
// Extra (not in the reference): -g 0|1 graph replay (default 1), -e 0|1 ignore EOS (default 0),
//   -m reference|fused|persistent schedule (default fused; persistent is experimental and about 2.3x slower), -b 0|1 batched prompt prefill (default 0).
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <algorithm>
#include <string>
#include <vector>

#include "../../../include/awq_hip.h"
#include "tokenizer.hpp"

static void die_awq(int r) {
    if (r != AWQ_OK) {
        fprintf(stderr, "%s\n", awq_last_error());
        exit(EXIT_FAILURE);
    }
}

static void error_usage(char* argv[]) {
    fprintf(stderr, "Usage:   %s <checkpoint> [options]\n", argv[0]);
    fprintf(stderr, "Example: %s model.bin -n 256 -i \"Write a poem on GPUs\"\n", argv[0]);
    fprintf(stderr, "Options:\n");
    fprintf(stderr, "  -n <int>    max number of steps to run for, default = max_seq_len\n");
    fprintf(stderr, "  -i <string> input prompt\n");
    fprintf(stderr, "  -f <string> path to file containing input prompt. Can be used with for multi-line prompts.\n");
    fprintf(stderr, "  -t <float>  temperature in [0,inf], default 0.5\n");
    fprintf(stderr, "  -p <float>  p value in top-p (nucleus) sampling in [0,1] default 0.9\n");
    fprintf(stderr, "  -s <int>    random seed, default time(NULL)\n");
    fprintf(stderr, "  -z <string> optional path to custom tokenizer\n");
    fprintf(stderr, "  -x <string> tensor-parallel mode: none (one GPU is all this build runs)\n");
    fprintf(stderr, "  -y <string> (optional) system prompt (accepted, unused, as in the reference)\n");
    fprintf(stderr, "  -q <string> dataset file (accepted, ignored: no perplexity mode)\n");
    fprintf(stderr, "  -g <0|1>    replay recorded launch sequences (hipGraph), default 1\n");
    fprintf(stderr, "  -m <string> schedule: reference|fused|persistent (experimental, ~2.3x slower), default fused\n");
    fprintf(stderr, "  -b <0|1>    consume the prompt in one batched prefill pass, default 0\n");
    fprintf(stderr, "  -e <0|1>    keep generating past the end-of-sequence token, default 0\n");
    fprintf(stderr, "  -d <0|1>    print the GPU time of every token, default 0\n");
    exit(EXIT_FAILURE);
}

static long time_in_ms() {
    struct timespec t;
    timespec_get(&t, TIME_UTC);
    return t.tv_sec * 1000 + t.tv_nsec / 1000000;
}

int main(int argc, char* argv[]) {
    // get_and_print_gpu_info(), llama2_q4.cu:817-837
    int device_count = 0;
    die_awq(awq_device_count(&device_count));
    if (device_count == 0) {
        printf("No HIP devices found!\n");
        return EXIT_FAILURE;
    }
    printf("Found %d HIP devices\n", device_count);
    for (int dev = 0; dev < device_count; dev++) {
        char name[256];
        size_t mem = 0;
        int cus = 0;
        die_awq(awq_device_info(dev, name, sizeof(name), &mem, &cus));
        printf("Device %d: %s\n", dev, name);
        printf("  Total global memory: %.2f GB\n", (float)mem / (1024.0f * 1024.0f * 1024.0f));
        printf("  Multiprocessors: %d\n\n", cus);
    }

    char* checkpoint_path = NULL;
    const char* tokenizer_path = "tokenizer.bin";
    char* dataset_path = NULL;
    int steps = 0;
    std::string prompt;
    bool have_prompt = false;
    int per_token_timings = 0;  // the reference's compile-time DUMP_PER_TOKEN_TIMINGS (llama2_q4.cu:32), as a switch
    float temperature = 0.5f;
    float topp = 0.6f;
    unsigned long long rng_seed = 0;
    int use_graph = 1, ignore_eos = 0, batched_prompt = 0, mode = AWQ_SCHEDULE_FUSED;

    if (argc >= 2) checkpoint_path = argv[1]; else error_usage(argv);
    for (int i = 2; i < argc; i += 2) {
        if (i + 1 >= argc) error_usage(argv);
        if (argv[i][0] != '-') error_usage(argv);
        if (strlen(argv[i]) != 2) error_usage(argv);
        switch (argv[i][1]) {
            case 'n': steps = atoi(argv[i + 1]); break;
            case 'i': prompt = argv[i + 1]; have_prompt = true; break;
            case 'z': tokenizer_path = argv[i + 1]; break;
            case 't': temperature = (float)atof(argv[i + 1]); break;
            case 'p': topp = (float)atof(argv[i + 1]); break;
            case 's': rng_seed = atoi(argv[i + 1]); break;
            case 'y': break;  // parsed and unused in the reference as well
            case 'x':
                if (strcmp(argv[i + 1], "none") != 0) {
                    if (strcmp(argv[i + 1], "column") == 0 || strcmp(argv[i + 1], "hybrid") == 0)
                        printf("tp_mode %s needs several GPUs; this build runs the whole model on one\n", argv[i + 1]);
                    else
                        printf("Unknown tp_mode: %s\n", argv[i + 1]);
                    return 1;
                }
                break;
            case 'q': dataset_path = argv[i + 1]; break;
            case 'f': {
                FILE* file = fopen(argv[i + 1], "r");
                if (!file) { printf("Couldn't open file %s\n", argv[i + 1]); return 1; }
                fseek(file, 0, SEEK_END);
                long fsize = ftell(file);
                fseek(file, 0, SEEK_SET);
                if (have_prompt) printf("Warning: -f overrides -i\n");
                prompt.resize(fsize);
                if (fsize > 0 && fread(&prompt[0], fsize, 1, file) != 1) { printf("Couldn't read file %s\n", argv[i + 1]); return 1; }
                fclose(file);
                have_prompt = true;
                break;
            }
            case 'g': use_graph = atoi(argv[i + 1]); break;
            case 'd': per_token_timings = atoi(argv[i + 1]); break;
            case 'e': ignore_eos = atoi(argv[i + 1]); break;
            case 'b': batched_prompt = atoi(argv[i + 1]); break;
            case 'm':
                if (!strcmp(argv[i + 1], "reference")) mode = AWQ_SCHEDULE_REFERENCE;
                else if (!strcmp(argv[i + 1], "fused")) mode = AWQ_SCHEDULE_FUSED;
                else if (!strcmp(argv[i + 1], "persistent")) mode = AWQ_SCHEDULE_PERSISTENT;
                else error_usage(argv);
                break;
            default: error_usage(argv);
        }
    }
    if (rng_seed <= 0) rng_seed = (unsigned int)time(NULL);
    if (temperature < 0.0f) temperature = 0.0f;
    if (topp < 0.0f || 1.0f < topp) topp = 0.9f;
    if (dataset_path) printf("Warning: dataset path is ignored in non-perplexity mode\n");

    // build_transformer(), llama2_q4.cu:625-659
    awq_ctx* ctx = nullptr;
    die_awq(awq_ctx_create(0, &ctx));
    {
        FILE* f = fopen(checkpoint_path, "rb");
        if (!f) { printf("Couldn't open file %s\n", checkpoint_path); return 1; }
        awq_config c;
        if (fread(&c, sizeof(c), 1, f) != 1) { printf("Invalid header size\n"); return 1; }
        fclose(f);
        printf("\nModel params:- \ndim: %d \nhidden_dim: %d\nn_heads: %d\nn_kv_heads: %d\nn_layers: %d\nseq_len: %d\nvocab_size: %d\nrope_theta: %g\n",
               c.dim, c.hidden_dim, c.n_heads, c.n_kv_heads, c.n_layers, c.seq_len, c.vocab_size, c.rope_theta);
    }
    printf("\nLoading Weights... ");
    fflush(stdout);
    awq_transformer* t = nullptr;
    die_awq(awq_transformer_load_file(ctx, checkpoint_path, &t));
    printf("done!\n");
    awq_config cfg;
    die_awq(awq_transformer_config(t, &cfg));
    if (steps <= 0 || steps > cfg.seq_len) steps = cfg.seq_len;

    awqcli::Tokenizer tok;
    if (!tok.load(tokenizer_path, cfg.vocab_size)) return EXIT_FAILURE;

    // generate(), llama2_q4.cu:759-786
    printf("\nEncoding Prompt... ");
    std::vector<int> prompt_tokens = tok.encode(prompt, true, false);
    printf("Done!\n");
    if (prompt_tokens.empty()) {
        fprintf(stderr, "something is wrong, expected at least 1 prompt token\n");
        return EXIT_FAILURE;
    }
    const int num_prompt_tokens = (int)prompt_tokens.size();
    if (num_prompt_tokens > cfg.seq_len) {
        fprintf(stderr, "prompt of %d tokens exceeds seq_len %d\n", num_prompt_tokens, cfg.seq_len);
        return EXIT_FAILURE;
    }

    // generate_thread(), llama2_q4.cu:683-757
    awq_run_state st;
    die_awq(awq_transformer_state(t, &st));
    die_awq(awq_transformer_reset(t, prompt_tokens.data(), num_prompt_tokens));
    // build_sampler(), llama2_q4.cu:922: the sampler owns the xorshift* state and runs on the GPU
    awq_sampler* sampler = nullptr;
    die_awq(awq_sampler_create(ctx, cfg.vocab_size, temperature, topp, rng_seed, &sampler));
    int token = prompt_tokens[0];
    int next;
    int pos = 0;
    long start = time_in_ms();
    if (batched_prompt && num_prompt_tokens > 1 && temperature == 0.0f) {
        // one batched pass over the prompt; echo it as the token-by-token loop would have
        const int n = std::min(num_prompt_tokens, steps);
        die_awq(awq_transformer_prefill(t, n, n == num_prompt_tokens));
        for (pos = 1; pos < n; pos++) {
            next = prompt_tokens[pos];
            awqcli::Tokenizer::safe_print(tok.decode(token, next));
            token = next;
        }
        fflush(stdout);
    }
    while (pos < steps) {
        die_awq(awq_stream_sync(ctx));  // wait for the previous token, then launch the next before printing
        const bool gen_token = pos >= num_prompt_tokens - 1;
        void *ev_start = nullptr, *ev_stop = nullptr;
        if (per_token_timings) {  // llama2_q4.cu:545-550
            die_awq(awq_event_create(ctx, &ev_start));
            die_awq(awq_event_create(ctx, &ev_stop));
            die_awq(awq_event_record(ctx, ev_start));
        }
        if (temperature == 0.0f) {
            // network + greedy sampler as one (graph-replayed) unit; the coin the reference draws anyway is never used
            die_awq(awq_transformer_forward(t, gen_token, use_graph, mode));
        } else {
            // run_transformer(), llama2_q4.cu:541-601: the network, then sample() (greedy while the prompt is consumed)
            die_awq(awq_transformer_forward_logits(t, use_graph, mode == AWQ_SCHEDULE_PERSISTENT ? AWQ_SCHEDULE_FUSED : mode));
            die_awq(awq_transformer_sample(t, sampler, gen_token));
        }
        if (per_token_timings) {  // llama2_q4.cu:592-600
            float ms = 0.0f;
            die_awq(awq_event_record(ctx, ev_stop));
            die_awq(awq_event_elapsed_ms(ctx, ev_start, ev_stop, &ms));
            printf(" t: %g ", ms);
            die_awq(awq_event_destroy(ctx, ev_start));
            die_awq(awq_event_destroy(ctx, ev_stop));
        }
        if (pos > 0) {
            next = st.shared_tokens[pos];
            if (next >= cfg.vocab_size) next = 0;
            awqcli::Tokenizer::safe_print(tok.decode(token, next));
            fflush(stdout);
            if (next == awqcli::kEosToken && !ignore_eos) break;
            token = next;
        }
        pos++;
    }
    die_awq(awq_stream_sync(ctx));
    long end = time_in_ms();
    double secs = (end - start) / 1000.0;
    int timed_tokens = pos - 1;
    printf("\n");
    printf("\n[GPU: %d] achieved tok/s: %f. Tokens: %d, seconds: %g\n", 0, timed_tokens / secs, timed_tokens, secs);

    die_awq(awq_sampler_destroy(sampler));
    die_awq(awq_transformer_free(t));
    die_awq(awq_ctx_destroy(ctx));
    return 0;
}

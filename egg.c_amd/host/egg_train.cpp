// egg_train.cpp -- the reference's training loop (full_cuda_train_transformer_adam_mgpu.cu:1313-1767) written
// against the C ABI of libegg_hip.so: load or synthesise the byte stream, init the model, then per step
// forward + fitness + update (one egg_step / egg_step_launch), read the update counter and the losses, print
// the reference's status line.  Differences by design: the step seed is an explicit argument chained with
// hash_rng (d-eggs/src/worker.cu:542) instead of time(NULL); no remote logging; errors return instead of exit(1)
// inside the library.
//
// Every --gen-every steps it prints a sampled continuation of the current window (mgpu.cu:1698-1731) and every
// --save-every steps it writes models/egg_step-*.bin (mgpu.cu:1733-1736); --load resumes from a model file.
//
// usage: egg_train [--data FILE] [--steps N] [--population P] [--seq T] [--hidden H] [--layers L] [--muon] [--graph]
//                  [--gen-every N] [--save-every N] [--save-dir DIR] [--load MODEL.bin [--load-state ADAM.bin]]
//                  [--adaptive]   (the d-eggs worker's adaptive noise overlay, d-eggs/src/worker.cu:331-333, :446-523)
//                  [--vocab V]    (d-eggs' VOCAB_SIZE: above 256 the data file holds uint32 tokens like its input.bin,
//                                  d-eggs/src/worker.cu:301-311; without --data a synthetic token stream is made)
//                  [--decoding FILE]  (d-eggs' decoding.bin: generated tokens are printed as text, worker.cu:320, :577)
//                  [--deggs-sampler]  (temperature / min-p / presence penalty at the reference's defaults, config.h:192-200)
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#include <algorithm>
#include <vector>

#include "../../include/egg_hip.h"

#define CK(call) do { int rc_ = (call); if (rc_ != EGG_OK) { fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, egg_last_error(ctx)); return 1; } } while (0)
#define HK(call) do { hipError_t e_ = (call); if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_)); return 1; } } while (0)

// i.i.d. Zipf(s) ranks over a fixed permutation of the 256 byte values; counter-based SplitMix64 -> inverse CDF
static std::vector<uint8_t> zipf_bytes(size_t n, uint64_t seed, double s) {
    std::vector<double> cdf(256); double tot = 0;
    for (int r = 0; r < 256; r++) { tot += 1.0 / pow((double)(r + 1), s); cdf[r] = tot; }
    for (double &c : cdf) c /= tot;
    uint8_t perm[256]; for (int i = 0; i < 256; i++) perm[i] = (uint8_t)i;
    uint32_t st = (uint32_t)((seed * 2654435761ull + 1ull) & 0xffffffffull); if (!st) st = 1;
    for (int i = 255; i > 0; i--) { st ^= st << 13; st ^= st >> 17; st ^= st << 5; int j = (int)(st % (uint32_t)(i + 1)); std::swap(perm[i], perm[j]); }
    std::vector<uint8_t> out(n);
    for (size_t i = 0; i < n; i++) {
        uint64_t z = seed + (uint64_t)(i + 1) * 0x9E3779B97F4A7C15ull;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull; z = (z ^ (z >> 27)) * 0x94D049BB133111EBull; z ^= z >> 31;
        double u = (double)(z >> 11) * (1.0 / 9007199254740992.0);
        int r = (int)(std::upper_bound(cdf.begin(), cdf.end(), u) - cdf.begin());
        out[i] = perm[r > 255 ? 255 : r];
    }
    return out;
}

int main(int argc, char **argv) {
    egg_config cfg; egg_default_config(&cfg);
    cfg.seq_len = 256; cfg.population = 40960;
    const char *data_file = nullptr; long steps = 10; bool graph = false; size_t synth_bytes = 64u << 20;
    bool adaptive = false, deggs_sampler = false; const char *decoding_file = nullptr;
    long gen_every = 5, save_every = 0; const char *save_dir = "models", *load_model = nullptr, *load_state = nullptr;
    for (int i = 1; i < argc; i++) {
        auto next = [&](const char *name) -> const char * { if (i + 1 >= argc) { fprintf(stderr, "%s needs a value\n", name); exit(2); } return argv[++i]; };
        if (!strcmp(argv[i], "--data")) data_file = next("--data");
        else if (!strcmp(argv[i], "--steps")) steps = atol(next("--steps"));
        else if (!strcmp(argv[i], "--population")) cfg.population = atoi(next("--population"));
        else if (!strcmp(argv[i], "--seq")) cfg.seq_len = atoi(next("--seq"));
        else if (!strcmp(argv[i], "--hidden")) cfg.hidden = atoi(next("--hidden"));
        else if (!strcmp(argv[i], "--layers")) cfg.n_layers = atoi(next("--layers"));
        else if (!strcmp(argv[i], "--muon")) cfg.use_muon = 1;
        else if (!strcmp(argv[i], "--graph")) graph = true;
        else if (!strcmp(argv[i], "--adaptive")) adaptive = true;
        else if (!strcmp(argv[i], "--vocab")) cfg.vocab = atoi(next("--vocab"));
        else if (!strcmp(argv[i], "--decoding")) decoding_file = next("--decoding");
        else if (!strcmp(argv[i], "--deggs-sampler")) deggs_sampler = true;
        else if (!strcmp(argv[i], "--gen-every")) gen_every = atol(next("--gen-every"));
        else if (!strcmp(argv[i], "--save-every")) save_every = atol(next("--save-every"));
        else if (!strcmp(argv[i], "--save-dir")) save_dir = next("--save-dir");
        else if (!strcmp(argv[i], "--load")) load_model = next("--load");
        else if (!strcmp(argv[i], "--load-state")) load_state = next("--load-state");
        else { fprintf(stderr, "unknown argument %s\n", argv[i]); return 2; }
    }
    std::vector<uint8_t> data;
    if (data_file) {
        FILE *f = fopen(data_file, "rb");
        if (!f) { fprintf(stderr, "cannot open %s\n", data_file); return 1; }
        fseek(f, 0, SEEK_END); long len = ftell(f); fseek(f, 0, SEEK_SET);
        data.resize((size_t)len);
        if (fread(data.data(), 1, (size_t)len, f) != (size_t)len) { fprintf(stderr, "short read\n"); return 1; }
        fclose(f);
    } else {
        data = zipf_bytes(synth_bytes, 1234, 1.1);
        if (cfg.vocab > 256) {          // uint32 tokens from pairs of Zipf bytes: frequent tokens stay frequent, every id is reachable
            std::vector<uint8_t> tok(data.size() / 2 * 4);
            for (size_t i = 0; i + 1 < data.size(); i += 2) {
                const uint32_t t = (((uint32_t)data[i] << 8) | data[i + 1]) % (uint32_t)cfg.vocab;
                memcpy(&tok[i / 2 * 4], &t, 4);
            }
            data.swap(tok);
        }
    }
    const size_t tb = cfg.vocab > 256 ? 4 : 1;                 // bytes per token (TokenType, d-eggs/include/model/definitions.h:9-13)
    const size_t n_tokens = data.size() / tb;
    printf("data: %zu tokens of %zu byte(s) (%s)\n", n_tokens, tb, data_file ? data_file : "synthetic Zipf(1.1)");
    egg_vocab *vocab = nullptr;
    if (decoding_file && egg_vocab_load(decoding_file, &vocab) != EGG_OK) { fprintf(stderr, "cannot read %s\n", decoding_file); return 1; }

    egg_ctx *ctx = nullptr;
    int rc = egg_ctx_create(&cfg, &ctx);
    if (rc != EGG_OK) { fprintf(stderr, "egg_ctx_create failed (%d): unsupported configuration or no GPU\n", rc); return 1; }
    if (load_model) CK(egg_checkpoint_load(ctx, load_model, load_state));
    else CK(egg_model_init(ctx, 42));
    if (adaptive) CK(egg_adaptive_enable(ctx, 64, 5, 1));      // ADAPTIVE_NOISE_INIT / _INC / _DEC, d-eggs/include/config.h:234-242
    uint8_t *d_data = nullptr;
    HK(hipMalloc(&d_data, data.size()));
    HK(hipMemcpy(d_data, data.data(), data.size(), hipMemcpyHostToDevice));
    // generation runs on a second, uncaptured context (the captured one is tied to its graph)
    const int gen_seed_len = std::min(32, cfg.seq_len / 2), gen_total = std::min(cfg.seq_len, gen_seed_len + 64);
    egg_ctx *gen_ctx = nullptr; uint8_t *d_gen = nullptr;
    std::vector<uint8_t> h_model;
    if (gen_every > 0) {
        egg_config gcfg = cfg; gcfg.population = 2; gcfg.chunk_members = 2;
        if (egg_ctx_create(&gcfg, &gen_ctx) != EGG_OK) { fprintf(stderr, "generation context failed\n"); return 1; }
        HK(hipMalloc(&d_gen, (size_t)cfg.seq_len * tb));
        h_model.resize((size_t)egg_model_bytes(ctx));
    }
    if (graph) CK(egg_step_capture(ctx, d_data, (int64_t)n_tokens));

    std::vector<int32_t> loss((size_t)cfg.population), fit((size_t)cfg.population / 2);
    uint32_t seed = 42;
    long max_steps = (long)((n_tokens - 1) / (size_t)cfg.seq_len);
    for (long step = 0; step < steps && step < max_steps; step++) {
        struct timespec t0, t1; clock_gettime(CLOCK_MONOTONIC, &t0);
        float lr = egg_learning_rate(step);
        if (graph) CK(egg_step_launch(ctx, step * cfg.seq_len, seed, lr));
        else CK(egg_step(ctx, d_data, (int64_t)n_tokens, step * cfg.seq_len, seed, lr));
        uint64_t updates = 0;
        CK(egg_last_update_count(ctx, &updates));          // synchronises, like the reference's cudaMemcpy of d_total_updates
        clock_gettime(CLOCK_MONOTONIC, &t1);
        CK(egg_step_losses(ctx, loss.data(), fit.data()));
        double ms = (t1.tv_sec - t0.tv_sec) * 1e3 + (t1.tv_nsec - t0.tv_nsec) / 1e6;
        long long total = 0; for (int32_t l : loss) total += l;
        double avg = (double)total / ((double)cfg.population * cfg.seq_len * 16.0);
        printf("Step %ld | Loss: %.4f | Time: %.2f ms | Updates: %llu | Speed: %.2f tok/s | LR: %.3f\n", step, avg, ms,
               (unsigned long long)updates, (double)cfg.population * cfg.seq_len / (ms / 1e3), lr);
        if (gen_every > 0 && step % gen_every == 0) {
            CK(egg_model_download(ctx, h_model.data(), h_model.size()));
            if (egg_model_upload(gen_ctx, h_model.data(), h_model.size()) != EGG_OK) return 1;
            size_t pos = (size_t)(step * cfg.seq_len) % (n_tokens - (size_t)cfg.seq_len);
            HK(hipMemcpy(d_gen, d_data + pos * tb, (size_t)gen_seed_len * tb, hipMemcpyDeviceToDevice));
            const int grc = deggs_sampler ? egg_generate_deggs(gen_ctx, d_gen, gen_seed_len, gen_total - gen_seed_len, seed + 999, 0.6f, 0.08f, 0.2f)
                                          : egg_generate(gen_ctx, d_gen, gen_seed_len, gen_total - gen_seed_len, seed + 999);
            if (grc != EGG_OK) { fprintf(stderr, "egg_generate: %s\n", egg_last_error(gen_ctx)); return 1; }
            if (egg_sync(gen_ctx) != EGG_OK) return 1;
            std::vector<uint8_t> h((size_t)gen_total * tb);
            HK(hipMemcpy(h.data(), d_gen, h.size(), hipMemcpyDeviceToHost));
            printf("\n--- GENERATION ---\n\033[32m");
            for (int part = 0; part < 2; part++) {           // the prompt, then the continuation
                const int first = part ? gen_seed_len : 0, count = part ? gen_total - gen_seed_len : gen_seed_len;
                if (part) printf("\033[36m");
                if (tb == 1) {
                    for (int i = first; i < first + count; i++) { char c = (char)h[(size_t)i]; putchar((c >= 32 && c <= 126) ? c : '.'); }
                } else {
                    std::vector<uint32_t> toks((size_t)count);
                    memcpy(toks.data(), h.data() + (size_t)first * 4, (size_t)count * 4);
                    if (vocab) {
                        std::vector<char> text((size_t)egg_detokenize(vocab, toks.data(), count, nullptr, 0) + 1);
                        egg_detokenize(vocab, toks.data(), count, text.data(), (int64_t)text.size());
                        fwrite(text.data(), 1, text.size() - 1, stdout);
                    } else
                        for (uint32_t t : toks) printf("<%u>", t);
                }
            }
            printf("\033[0m\n\n");
        }
        if (save_every > 0 && step % save_every == 0) CK(egg_checkpoint_save(ctx, save_dir, step));
        seed = egg_next_seed(seed, (uint64_t)(step + 1));
    }
    if (vocab) egg_vocab_free(vocab);
    if (d_gen) (void)hipFree(d_gen);
    if (gen_ctx) egg_ctx_destroy(gen_ctx);
    (void)hipFree(d_data);
    egg_ctx_destroy(ctx);
    return 0;
}

// egg_hostutil.hip -- host-side pieces of the reference's loops that sit next to the GPU path and are host code
// in the reference too: d-eggs' shaping of a chunk's losses into ternary fitness and its base-3 wire packing
// (d-eggs/src/worker.cu:636-687, d-eggs/include/utils/ternary_pack.h), the raw model / optimizer-state checkpoint
// files of the single-node trainer (egg_disk_utils.h:1-82) and d-eggs' EGGC replay checkpoints
// (d-eggs/include/utils/checkpoint.h:17-128).  No device code.
#include "../../include/egg_hip.h"

#include <dirent.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>
#include <string>
#include <vector>

// ---------------------------------------------------------------- fitness shaping (worker.cu:636-687)
extern "C" int egg_shape_fitness(const int32_t *loss, int count, int chunk_mean_filter, double mean_exponent,
                                 int adaptive_threshold, double alpha, int32_t *fit_out, int64_t *sum_loss_out) {
    if (!loss || !fit_out || count < 2 || (count & 1)) return EGG_E_INVALID;
    const int pairs = count / 2;
    std::vector<int32_t> diff(pairs);
    int64_t sum_loss = 0;
    double sum_diff = 0.0;
    for (int i = 0; i < pairs; i++) {
        const int32_t p = loss[2 * i], n = loss[2 * i + 1];
        sum_loss += (int64_t)p + n;
        diff[i] = n - p;                      // positive when the +noise member is better
        sum_diff += diff[i];
    }
    if (chunk_mean_filter) {
        double mean = sum_diff / pairs;
        if (mean != 0.0) mean = (mean > 0 ? 1.0 : -1.0) * pow(fabs(mean), mean_exponent);
        const int32_t shift = (int32_t)mean;  // truncation toward zero, as the reference's cast
        for (int i = 0; i < pairs; i++) diff[i] += shift;
    }
    if (adaptive_threshold) {
        double sum_abs = 0.0;
        for (int i = 0; i < pairs; i++) sum_abs += fabs((double)diff[i]);
        const double threshold = (sum_abs / pairs) * alpha;
        for (int i = 0; i < pairs; i++) fit_out[i] = fabs((double)diff[i]) < threshold ? 0 : (diff[i] > 0 ? 1 : -1);
    } else {
        for (int i = 0; i < pairs; i++) fit_out[i] = diff[i] > 0 ? 1 : (diff[i] < 0 ? -1 : 0);
    }
    if (sum_loss_out) *sum_loss_out = sum_loss;
    return EGG_OK;
}

// ---------------------------------------------------------------- base-3 packing (ternary_pack.h:11-104)
// five values per byte, least significant digit first; digit 0 -> 0, 1 -> +1, 2 -> -1
extern "C" size_t egg_ternary_pack_size(size_t count) { return (count + 4) / 5; }
extern "C" int egg_ternary_pack(const int32_t *src, size_t count, uint8_t *dst) {
    if ((!src || !dst) && count) return EGG_E_INVALID;
    for (size_t i = 0, o = 0; i < count; i += 5, o++) {
        unsigned byte = 0, mult = 1;
        for (size_t k = i; k < count && k < i + 5; k++, mult *= 3) {
            if (src[k] < -1 || src[k] > 1) return EGG_E_INVALID;
            byte += (unsigned)((src[k] + 3) % 3) * mult;
        }
        dst[o] = (uint8_t)byte;
    }
    return EGG_OK;
}
extern "C" int egg_ternary_unpack(const uint8_t *src, size_t count, int32_t *dst) {
    if ((!src || !dst) && count) return EGG_E_INVALID;
    for (size_t i = 0, o = 0; i < count; i += 5, o++) {
        unsigned byte = src[o];
        for (size_t k = i; k < count && k < i + 5; k++, byte /= 3) {
            const unsigned d = (k == i + 4) ? byte : byte % 3;     // the fifth digit is whatever is left, as in the reference
            dst[k] = d == 2 ? -1 : (int32_t)d;
        }
    }
    return EGG_OK;
}

// ---------------------------------------------------------------- raw checkpoints (egg_disk_utils.h:1-82)
static void ensure_dir(const char *path, mode_t mode) {
    struct stat st;
    if (stat(path, &st) == -1) (void)mkdir(path, mode);
}
static int write_file(const std::string &path, const void *data, size_t n) {
    FILE *f = fopen(path.c_str(), "wb");
    if (!f) return EGG_E_INVALID;
    const size_t w = n ? fwrite(data, 1, n, f) : 0;
    return (fclose(f) == 0 && w == n) ? EGG_OK : EGG_E_INVALID;
}
static void relink(const std::string &dir, const char *target, const char *link_name) {
    const std::string link = dir + "/" + link_name;
    (void)unlink(link.c_str());
    (void)symlink(target, link.c_str());
}
extern "C" int egg_checkpoint_save(egg_ctx *ctx, const char *dir, long step) {
    if (!ctx) return EGG_E_INVALID;
    const std::string d = (dir && *dir) ? dir : "models";
    ensure_dir(d.c_str(), 0700);
    const int64_t mb = egg_model_bytes(ctx), sb = egg_opt_state_bytes(ctx);
    std::vector<uint8_t> model((size_t)mb), state((size_t)sb);
    int rc = egg_model_download(ctx, model.data(), model.size());
    if (rc) return rc;
    rc = egg_opt_state_download(ctx, state.data(), state.size());
    if (rc) return rc;
    char name_model[128], name_state[128];
    snprintf(name_model, sizeof(name_model), "egg_step-%08ld.model.bin", step);
    snprintf(name_state, sizeof(name_state), "egg_step-%08ld.adam.bin", step);
    rc = write_file(d + "/" + name_model, model.data(), model.size());
    if (rc) return rc;
    relink(d, name_model, "egg_transformer_last.model.bin");
    rc = write_file(d + "/" + name_state, state.data(), state.size());
    if (rc) return rc;
    relink(d, name_state, "egg_transformer_last.adam.bin");
    return EGG_OK;
}
static int read_exact(const char *path, std::vector<uint8_t> &buf) {
    FILE *f = fopen(path, "rb");
    if (!f) return EGG_E_INVALID;
    const size_t r = fread(buf.data(), 1, buf.size(), f);
    const bool tail = fgetc(f) != EOF;          // a file of another model shape is longer or shorter
    fclose(f);
    return (r == buf.size() && !tail) ? EGG_OK : EGG_E_INVALID;
}
extern "C" int egg_checkpoint_load(egg_ctx *ctx, const char *model_path, const char *state_path) {
    if (!ctx || !model_path) return EGG_E_INVALID;
    std::vector<uint8_t> model((size_t)egg_model_bytes(ctx));
    int rc = read_exact(model_path, model);
    if (rc) return rc;
    std::vector<uint8_t> state;
    if (state_path) {
        state.resize((size_t)egg_opt_state_bytes(ctx));
        rc = read_exact(state_path, state);
        if (rc) return rc;
    }
    rc = egg_model_upload(ctx, model.data(), model.size());
    if (rc) return rc;
    return state_path ? egg_opt_state_upload(ctx, state.data(), state.size()) : EGG_OK;
}

// ---------------------------------------------------------------- EGGC replay checkpoints (checkpoint.h:17-128)
namespace {
struct EggcHeader { uint32_t magic, version; uint64_t step, seed, data_size; };
const uint32_t kEggcMagic = 0x45474743u, kEggcVersion = 1u;
}
extern "C" int egg_eggc_save(const char *dir, uint64_t step, uint64_t seed, const uint8_t *data, uint64_t n) {
    if (!dir || !*dir || (!data && n)) return EGG_E_INVALID;
    ensure_dir(dir, 0755);
    char name[64];
    snprintf(name, sizeof(name), "checkpoint_%08llu.bin", (unsigned long long)step);
    std::vector<uint8_t> blob(sizeof(EggcHeader) + (size_t)n);
    const EggcHeader h = {kEggcMagic, kEggcVersion, step, seed, n};
    memcpy(blob.data(), &h, sizeof(h));
    if (n) memcpy(blob.data() + sizeof(h), data, (size_t)n);
    return write_file(std::string(dir) + "/" + name, blob.data(), blob.size());
}
extern "C" int egg_eggc_load_latest(const char *dir, uint64_t *step, uint64_t *seed, uint8_t *data, uint64_t capacity,
                                    uint64_t *n) {
    if (!dir || !*dir || !step || !seed || !n) return EGG_E_INVALID;
    DIR *d = opendir(dir);
    if (!d) return EGG_E_INVALID;
    bool found = false; unsigned long long best = 0; std::string best_name;
    while (struct dirent *ent = readdir(d)) {
        const std::string name = ent->d_name;
        const size_t dot = name.find(".bin");
        if (name.rfind("checkpoint_", 0) != 0 || dot == std::string::npos || dot <= 11) continue;
        const std::string num = name.substr(11, dot - 11);
        char *end = nullptr;
        const unsigned long long s = strtoull(num.c_str(), &end, 10);
        if (end == num.c_str()) continue;
        if (!found || s > best) { found = true; best = s; best_name = name; }
    }
    closedir(d);
    if (!found) return EGG_E_INVALID;
    FILE *f = fopen((std::string(dir) + "/" + best_name).c_str(), "rb");
    if (!f) return EGG_E_INVALID;
    EggcHeader h;
    int rc = EGG_OK;
    if (fread(&h, sizeof(h), 1, f) != 1 || h.magic != kEggcMagic) rc = EGG_E_INVALID;
    if (rc == EGG_OK) {
        *step = h.step; *seed = h.seed; *n = h.data_size;
        if (h.data_size > capacity || (h.data_size && !data)) rc = EGG_E_STATE;          // caller retries with *n bytes
        else if (h.data_size && fread(data, 1, (size_t)h.data_size, f) != h.data_size) rc = EGG_E_INVALID;
    }
    fclose(f);
    return rc;
}

// ---------------------------------------------------------------- token vocabulary (worker.cu:36-81)
// "decoding.bin": uint32 count, then per token uint32 length + bytes.  The reference prints a generated token run as the
// concatenation of its tokens' strings and "<id>" for an id beyond the table.
struct egg_vocab { std::vector<std::string> entries; };
extern "C" int egg_vocab_load(const char *path, egg_vocab **out) {
    if (!path || !out) return EGG_E_INVALID;
    *out = nullptr;
    FILE *f = fopen(path, "rb");
    if (!f) return EGG_E_INVALID;
    uint32_t n = 0;
    int rc = fread(&n, 4, 1, f) == 1 ? EGG_OK : EGG_E_INVALID;
    egg_vocab *v = new egg_vocab();
    for (uint32_t i = 0; rc == EGG_OK && i < n; i++) {
        uint32_t len = 0;
        if (fread(&len, 4, 1, f) != 1) { rc = EGG_E_INVALID; break; }
        std::string s;
        // a length is checked against what is left of the file before it is trusted with an allocation
        const long here = ftell(f);
        if (fseek(f, 0, SEEK_END) != 0) { rc = EGG_E_INVALID; break; }
        const long end = ftell(f);
        if (here < 0 || end < here || (unsigned long)(end - here) < len || fseek(f, here, SEEK_SET) != 0) { rc = EGG_E_INVALID; break; }
        s.resize(len);
        if (len && fread(&s[0], 1, len, f) != len) { rc = EGG_E_INVALID; break; }
        v->entries.push_back(std::move(s));
    }
    fclose(f);
    if (rc != EGG_OK) { delete v; return rc; }
    *out = v;
    return EGG_OK;
}
extern "C" void egg_vocab_free(egg_vocab *v) { delete v; }
extern "C" int egg_vocab_size(const egg_vocab *v) { return v ? (int)v->entries.size() : 0; }
extern "C" int egg_vocab_save(const char *path, const char *const *entries, const uint32_t *lengths, uint32_t count) {
    if (!path || (count && (!entries || !lengths))) return EGG_E_INVALID;
    FILE *f = fopen(path, "wb");
    if (!f) return EGG_E_INVALID;
    bool ok = fwrite(&count, 4, 1, f) == 1;
    for (uint32_t i = 0; ok && i < count; i++)
        ok = fwrite(&lengths[i], 4, 1, f) == 1 && (lengths[i] == 0 || fwrite(entries[i], 1, lengths[i], f) == lengths[i]);
    return (fclose(f) == 0 && ok) ? EGG_OK : EGG_E_INVALID;
}
extern "C" int64_t egg_detokenize(const egg_vocab *v, const uint32_t *tokens, int count, char *out, int64_t capacity) {
    if (!v || (count && !tokens) || count < 0 || capacity < 0 || (capacity && !out)) return EGG_E_INVALID;
    std::string text;
    for (int i = 0; i < count; i++) {
        if (tokens[i] < v->entries.size()) text += v->entries[tokens[i]];
        else text += "<" + std::to_string(tokens[i]) + ">";
    }
    const int64_t n = (int64_t)text.size();
    if (capacity > 0) { const int64_t c = n < capacity ? n : capacity; memcpy(out, text.data(), (size_t)c); }
    return n;
}

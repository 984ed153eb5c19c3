/*
 * ref_shim.cpp -- exports, unchanged, the host-compilable helpers of the reference's
 * own header d-eggs/include/utils/egg_math.h (hash_rng, noise_from_hash, clip,
 * xorshift32_host, gen_noise_host), d-eggs/include/utils/ternary_pack.h and
 * d-eggs/include/utils/checkpoint.h (EGGC replay checkpoints), compiled
 * from where they lie under $(REF) by oracle/Makefile into oracle/_ref/libegg_ref.so.
 * TEST INFRASTRUCTURE ONLY: it exists to pin oracle/egg_oracle.cpp's restatement of
 * the same functions; nothing shipped links it.  No reference source is copied here.
 */
#include <stdint.h>
#include <stddef.h>
#include EGG_REF_MATH_H
#include EGG_REF_TERNARY_H
#include EGG_REF_CHECKPOINT_H

extern "C" {
uint32_t ref_hash_rng(uint32_t s, uint32_t idx) { return hash_rng(s, idx); }
int ref_noise_from_hash(uint32_t s, uint32_t idx) { return (int)noise_from_hash(s, idx); }
int ref_clip(int32_t a) { return (int)clip(a); }
uint32_t ref_xorshift32_host(uint32_t *st) { return xorshift32_host(st); }
int ref_gen_noise_host(uint32_t *st) { return (int)gen_noise_host(st); }
size_t ref_ternary_pack_estimate_size(size_t n) { return ternary_pack_estimate_size(n); }
void ref_ternary_pack(const int32_t *src, size_t n, uint8_t *dst) { ternary_pack(src, n, dst); }
void ref_ternary_unpack(const uint8_t *src, size_t n, int32_t *dst) { ternary_unpack(src, n, dst); }
void ref_eggc_save(const char *dir, uint64_t step, uint64_t seed, const uint8_t *data, uint64_t n) {
    save_checkpoint_worker(dir, step, seed, std::vector<uint8_t>(data, data + n));
}
int ref_eggc_load(const char *dir, uint64_t *step, uint64_t *seed, uint8_t *data, uint64_t cap, uint64_t *n) {
    std::vector<uint8_t> v;
    if (!load_checkpoint(dir, *step, *seed, v)) return 0;
    *n = v.size();
    if (v.size() > cap) return -1;
    if (!v.empty()) memcpy(data, v.data(), v.size());
    return 1;
}
}

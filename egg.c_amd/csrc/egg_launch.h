// egg_launch.h -- host-side launchers of the kernels, one per .hip translation unit.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <limits.h>
#include "egg_params.h"

hipError_t egg_launch_mlp(const MlpParams &p, bool first, hipStream_t s);
hipError_t egg_launch_qkv(const QkvParams &p, hipStream_t s);
hipError_t egg_launch_attn(const AttnParams &p, hipStream_t s);
hipError_t egg_launch_head(const HeadParams &p, hipStream_t s);
hipError_t egg_prepare_forward(int H, int head_dim, int T);

struct PlinParams {
    const int8_t *X;        // [members*T][K] natural order
    const int8_t *Wfrag;    // fragment-major copy of W (natural k order) as egg_launch_plinear_swizzle lays it out for (T, K, N)
    int members, T, K, N;
    uint32_t seed; int off_a, off_b, shift, sigma, mask;
    int32_t *Y32; int8_t *Y8;
    int plain;              // the shared-weight product alone: no rank-1 term (the reference's ns == 0 case)
    int own_noise;          // every member draws its own (A, B) with ns = +1 instead of sharing a pair's draw with ns = +-1
    const int8_t *Wblocked; // the canonical blocked matrix: set (with a shape egg_plinear_ws_shape accepts) to run the
                            // W-stationary kernel, which needs no fragment-major copy
};
bool egg_plinear_ws_shape(int K, int N);
hipError_t egg_launch_plinear_ws(const PlinParams &p, hipStream_t s);      // egg_linear_ws.hip
hipError_t egg_launch_plinear(const PlinParams &p, hipStream_t s);
int egg_plinear_block(int K, int N);
// canonical blocked W -> the layout the kernel chosen for (T, K, N) reads
hipError_t egg_launch_plinear_swizzle(const int8_t *W_blocked, int8_t *W_frag, int T, int K, int N, hipStream_t s);
// canonical blocked [K/4][N][4] -> fragment-major (see egg_device.h); nat = natural k order inside a k-step
hipError_t egg_launch_swizzle(const int8_t *W_blocked, int8_t *W_frag, int K, int N, int B, int nat, hipStream_t s);

// small utility kernels (egg_update.hip)
hipError_t egg_launch_noise_fill(uint32_t seed, uint32_t first, int n, int mask, int8_t *out, hipStream_t s);
hipError_t egg_launch_zero_u64(unsigned long long *p, int64_t n, hipStream_t s);
hipError_t egg_launch_loss_finalize(const unsigned long long *acc, int32_t *loss, int first, int count, hipStream_t s);
hipError_t egg_launch_fitness(const int32_t *loss, int32_t *fit, int pairs, hipStream_t s);
// ws: vocab ints (plain sampler) or 2 * vocab ints (d-eggs sampler) of device scratch; token_bytes: 1 or 4
hipError_t egg_launch_sample(const int32_t *logits, const int32_t *exp_lut, int vocab, int bt, uint32_t seed, int t,
                             int *ws, void *out, int token_bytes, hipStream_t s);
hipError_t egg_launch_sample_deggs(const int32_t *logits, const int32_t *exp_lut, int vocab, int bt, uint32_t seed, int t,
                                   const void *tokens, float temp, int min_p_limit, int penalty_int, int *ws, void *out, int token_bytes, hipStream_t s);

struct UpdParams {
    int8_t *W; float *state;           // tensor weights and optimizer state ({m,v,acc} per element)
    int rows, cols;                    // matrix: rows = input dim (k), cols = output dim (n); vector: cols = len
    int off_a, off_b, seed_base;
    const int32_t *fit; int pairs;
    const uint32_t *d_seed; const float *d_lr; float lr_scale;
    int mask; float beta1, beta2, eps, wd;
    int limit;                         // weights saturate at +-limit: 127 (mgpu.cu:1056-1062), or the configured limit for matrices
    int8_t *panel_a, *panel_b; int pairs_pad;   // workspace: [cols][pairs_pad], [rows][pairs_pad]
    unsigned long long *counter;
    int32_t *votes_out;                // optional: only compute votes (blocked order), no update
    int8_t *flags;                     // optional (adaptive noise overlay): [rows] then [cols], set to 1 where a weight of
                                       // that input row / output column changed (de/include/optimizer/adam.cuh:77-83)
    // Muon (state is {m, acc} per element): momentum pass writes m and the row-major gather buffer
    float muon_momentum; float *muon_x; // [rows][cols] row-major
};
hipError_t egg_launch_update_matrix(const UpdParams &p, hipStream_t s);
hipError_t egg_launch_update_vector(const UpdParams &p, hipStream_t s);
// every vector tensor of the model in one launch: descriptors live on the device, `first` is the running element count
struct VecDesc { int8_t *W; float *state; int n, first, off_a, off_b, seed_base; float lr_scale; int8_t *flags; };   // flags: as above, per element, or null
hipError_t egg_launch_update_vectors(const UpdParams &common, const VecDesc *d_desc, int n_desc, int total, hipStream_t s);

// adaptive noise overlay (de/src/kernels.cu:61-77): for every entry of every segment, +inc where the flag is set, -dec
// elsewhere, clamped to [-127, 127]; also writes q = clamp(overlay, 0, 64) and clears the flag
struct OvSeg { int offset, count; };
hipError_t egg_launch_overlay_update(int8_t *overlay, int8_t *q, int8_t *flags, const OvSeg *d_segs, int n_segs, int max_count,
                                     int inc, int dec, hipStream_t s);
hipError_t egg_launch_overlay_q(const int8_t *overlay, int8_t *q, int64_t n, hipStream_t s);

// ternary-packed matrix weights <-> canonical int8 (n_elems a multiple of 4); *d_bad is set when a weight is not in {-1,0,1}
hipError_t egg_launch_ternary_unpack(const uint8_t *packed, int8_t *dst, int n_elems, hipStream_t s);
hipError_t egg_launch_ternary_pack(const int8_t *src, uint8_t *packed, int n_elems, int *d_bad, hipStream_t s);

// Muon chain (muon_internal.cuh:15-342): momentum + gather (vote GEMM epilogue), Frobenius normalisation,
// 5 Newton-Schulz iterations on fp32 MFMA, quantised apply.
hipError_t egg_launch_muon_momentum(const UpdParams &p, hipStream_t s);
struct MuonWork { float *x, *swap, *gram, *bterm, *partials, *norm; };   // x/swap: rows*cols, gram/bterm: K*K, partials: 1024
hipError_t egg_launch_newton_schulz(const MuonWork &w, int rows, int cols, int iters, hipStream_t s);
hipError_t egg_launch_newton_schulz_batched(const MuonWork &w, int rows, int cols, int iters, int batch, hipStream_t s);
hipError_t egg_launch_muon_apply(const UpdParams &p, float wd, hipStream_t s);
// message returned by egg_last_error(NULL) on this thread, for entry points that take no context
void egg_set_thread_error(const char *what);
#define EGG_MAX_DEVICES 64

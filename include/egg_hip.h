/*
 * egg_hip.h -- C ABI of libegg_hip.so: the EGGROLL population-evaluation hot path
 * (Int8NativeFormer forward + fitness + ES update) on one AMD MI355X (gfx950).
 *
 * The reference (d0rc/egg.c) exposes no FFI: each trainer is one translation unit
 * whose main() launches kernels directly.  The functions below are that de-facto
 * operator surface, one export per thing the reference's host loop does; the
 * reference site each one replaces is cited.  Shorthand for reference files:
 *   mgpu.cu = full_cuda_train_transformer_adam_mgpu.cu,  de/ = d-eggs/
 *
 * Conventions: every call returns 0 on success or a negative EGG_E_* code and never
 * exits the process (the reference's CHECK_CUDA does, mgpu.cu:272).  A context owns
 * one device, one stream, the model, the optimizer state and the activation
 * workspace.  Calls on one context are not thread-safe; distinct contexts are
 * independent.  Pointers named d_* are device pointers owned by the caller;
 * everything is enqueued on the context's stream and no call synchronises unless
 * it says so.
 */
#ifndef EGG_HIP_H
#define EGG_HIP_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EGG_OK             0
#define EGG_E_INVALID     -1   /* bad argument / unsupported configuration          */
#define EGG_E_HIP         -2   /* a HIP runtime call failed (see egg_last_error)     */
#define EGG_E_NOMEM       -3
#define EGG_E_STATE       -4   /* call order violated (e.g. launch before capture)   */

typedef struct egg_ctx egg_ctx;

/* Runtime form of the reference's -D macros (mgpu.cu:34-270). */
typedef struct egg_config {
    int hidden;              /* HIDDEN_DIM: 64, 128, 256 or 512                       */
    int head_dim;            /* HEAD_DIM: 32 or 64, divides hidden                    */
    int n_layers;            /* N_LAYERS                                              */
    int seq_len;             /* SEQ_LEN: multiple of 32                               */
    int vocab;               /* VOCAB_SIZE: 256 (byte level), or a multiple of 256 <= 65536 */
    int population;          /* POPULATION_SIZE: even                                 */
    int fixed_point;         /* 4                                                     */
    int sigma_shift;         /* 3                                                     */
    int sigma_shift_vector;  /* 4                                                     */
    int shift_attn, shift_out, shift_logit, shift_mlp_up, shift_mlp_down;  /* 8 9 8 8 10 */
    int softmax_scale_bit;   /* 18                                                    */
    int rope_scale_bit;      /* 20                                                    */
    int noise_mask;          /* DEVICE_MASK 15                                        */
    int host_mask;           /* HOST_MASK 15                                          */
    double softmax_exp_scale;/* 6.0                                                   */
    float adam_beta1, adam_beta2, adam_eps, adam_weight_decay;   /* .9 .95 1e-8 .01  */
    float muon_momentum, muon_lr_scale;                          /* .85 1.0          */
    int use_muon;            /* USE_MUON: 2-D hidden matrices use Muon instead of AdamW */
    int chunk_members;       /* members evaluated per forward pass over the layers; 0 = auto (the whole population
                                while its activation buffers stay within 32 GiB, else 8192) */
    int weight_limit;        /* matrix weights saturate at +-weight_limit in the update rule: 127 as in the reference
                              * (mgpu.cu:1056-1062); 1 keeps them ternary (no reference counterpart)     */
    int device_gaussian;     /* DEVICE_GAUSSIAN (mgpu.cu:195-196, :530-534): perturbation noise = sum of three masked fields */
    int host_gaussian;       /* HOST_GAUSSIAN (mgpu.cu:192-193, :433-437): the same for the initial weights              */
    int use_same_data;       /* USE_SAME_DATA (mgpu.cu:212-213, :866-867): every pair reads the window at start_idx      */
} egg_config;

void egg_default_config(egg_config *cfg);

/* init_tables + cudaMemcpyToSymbol + per-GPU allocation (mgpu.cu:394-426, :1442-1489) */
int  egg_ctx_create(const egg_config *cfg, egg_ctx **out);
void egg_ctx_destroy(egg_ctx *ctx);
/* message of the last failed call on ctx; with ctx == NULL, why this thread's last egg_ctx_create (or last call of an
 * entry point that takes no context) failed */
const char *egg_last_error(const egg_ctx *ctx);
/* run on a caller-provided hipStream_t instead of the context's own (d-eggs update_stream, de/src/worker.cu:352-357) */
int  egg_ctx_set_stream(egg_ctx *ctx, void *hip_stream);
int  egg_sync(egg_ctx *ctx);                       /* cudaStreamSynchronize, mgpu.cu:1552 */

/* model blob == the reference's TransformerModel (mgpu.cu:284-318) with runtime sizes; every
 * matrix in the blocked [K/4][N][4] layout of repack_matrix (mgpu.cu:443-459) */
int64_t egg_model_bytes(const egg_ctx *ctx);
int  egg_model_init(egg_ctx *ctx, uint32_t seed);                          /* init_model, mgpu.cu:461-519 */
int  egg_model_upload(egg_ctx *ctx, const void *host_model, size_t bytes); /* load_model + H2D, mgpu.cu:1373,:1461 */
int  egg_model_download(egg_ctx *ctx, void *host_model, size_t bytes);     /* D2H before save, mgpu.cu:1734 */
/* optimizer state == the reference's AdamModel (mgpu.cu:321-370): in model field order, one {m,v,acc} float triple
 * per element; with use_muon the 2-D hidden matrices hold {m,acc} pairs instead (HIDDEN_OPT_TYPE, mgpu.cu:327-335) */
int64_t egg_opt_state_bytes(const egg_ctx *ctx);
int64_t egg_tensor_state_offset(const egg_ctx *ctx, int tensor_id);   /* byte offset of a tensor's state */
int  egg_opt_state_upload(egg_ctx *ctx, const void *host_state, size_t bytes);
int  egg_opt_state_download(egg_ctx *ctx, void *host_state, size_t bytes);
int  egg_opt_state_reset(egg_ctx *ctx);                                    /* calloc'd AdamModel, mgpu.cu:1367 */
/* lookup tables as uploaded to the device: exp[256], act[256], rope[seq_len*head_dim] (mgpu.cu:394-426) */
int  egg_tables_download(egg_ctx *ctx, int32_t *exp_lut, int8_t *act_lut, int32_t *rope_lut);

/* noise_from_hash(seed, first_idx + i) for i < n, written to d_out (mgpu.cu:528-538) */
int  egg_noise_fill(egg_ctx *ctx, uint32_t seed, uint32_t first_idx, int n, int8_t *d_out);

/* one perturbed linear layer over a [members*T][K] int8 activation matrix (compute_linear_projection,
 * mgpu.cu:553-572): row r belongs to member r/T, pair = member/2, ns = +1 (even) / -1 (odd);
 *   acc[n] = sum_k X[r][k] W[k][n] + (((sum_k X[r][k] B[k]) * A[n]) * ns >> (fixed_point+sigma_shift))
 *   A[n] = noise(seed + pair + off_a, n), B[k] = noise(seed + pair + off_b, k)
 * d_Y32 receives acc >> shift as int32 [rows][N] (may be NULL); d_Y8 receives clip(acc >> shift) as int8
 * [rows][N] (may be NULL).  T is a multiple of 32.  Supported shapes: K = 256 or 512 with T a multiple of 64 and any N
 * that is a multiple of 64 up to 1024; otherwise (K, N) from {64, 128, 256, 512, 1024}^2 pairs the transformer uses
 * (64x64, 64x256, 256x64, 128x128, 128x512, 512x128, 256x256, 256x1024, 1024x256, 512x512).  Other shapes return
 * EGG_E_INVALID with the reason in egg_last_error. */
int  egg_perturbed_linear(egg_ctx *ctx, const int8_t *d_X, const int8_t *d_W_blocked,
                          int members, int T, int K, int N, uint32_t seed, int off_a, int off_b,
                          int shift, int32_t *d_Y32, int8_t *d_Y8);
/* The same layer with one noise draw per member instead of per antithetic pair: pair -> member, ns = +1 for every
 * member (A[n] = noise(seed + member + off_a, n), B[k] = noise(seed + member + off_b, k)).  The reference has no such
 * call site (its members always come in +- pairs, mgpu.cu:864-871); it is compute_linear_projection with those
 * arguments, kept so that both indexings of the single-layer microbenchmark can be measured. */
int  egg_perturbed_linear_own_noise(egg_ctx *ctx, const int8_t *d_X, const int8_t *d_W_blocked,
                                    int members, int T, int K, int N, uint32_t seed, int off_a, int off_b,
                                    int shift, int32_t *d_Y32, int8_t *d_Y8);
/* The same product without the rank-1 term: compute_linear_projection with ns == 0 (mgpu.cu:568, the guard the
 * reference's generation path takes), Y = (X . W) >> shift.  It is the shared-weight GEMM on its own. */
int  egg_shared_linear(egg_ctx *ctx, const int8_t *d_X, const int8_t *d_W_blocked,
                       int members, int T, int K, int N, int shift, int32_t *d_Y32, int8_t *d_Y8);

/* No counterpart in the reference.  For K = 512 or 256 with N = 512 the three calls above run a W-stationary kernel
 * (one persistent workgroup per CU keeps the whole of W in its registers and streams the activations through LDS);
 * w_stationary = 0 makes them use the W-streaming kernels instead, which serve every other shape.  Results are
 * identical; the switch exists so that both can be measured and compared. */
int  egg_ctx_linear_kernel(egg_ctx *ctx, int w_stationary);

/* train_sequence_kernel<<<batch,...>>> (mgpu.cu:847-1029, launch :1531): evaluates members
 * [pop_offset, pop_offset+pop_count) on tokens d_data[stream_pos + t], writes d_loss[member] (int32).
 * pop_offset and pop_count must be even.  With vocab 256 the stream is bytes; with a larger vocabulary d_data points at
 * uint32 tokens (d-eggs' TokenType, de/include/config.h:22-28), every one below vocab.  data_len counts tokens either
 * way.  The same holds for egg_population_forward_dev, egg_step and egg_step_capture. */
int  egg_population_forward(egg_ctx *ctx, const uint8_t *d_data, int64_t data_len, int64_t start_idx,
                            uint32_t step_seed, int pop_offset, int pop_count, int32_t *d_loss);
/* same, with the step seed and start index read from device memory when the launch executes
 * (graph-capturable; mirrors de/include/optimizer/adam.cuh:38-39 passing scalars by device pointer) */
int  egg_population_forward_dev(egg_ctx *ctx, const uint8_t *d_data, int64_t data_len,
                                const int64_t *d_start_idx, const uint32_t *d_step_seed,
                                int pop_offset, int pop_count, int32_t *d_loss);

/* compute_fitness_host / compute_fitness_kernel (mgpu.cu:1305-1311, :1031-1036) */
int  egg_fitness(egg_ctx *ctx, const int32_t *d_loss, int32_t *d_fit, int pairs);

/* every LAUNCH_ADAM_MATRIX / LAUNCH_ADAM_VECTOR of one step (mgpu.cu:1577-1643); seed and learning
 * rate by device pointer (de/include/optimizer/adam.cuh:38-39); resets then accumulates the update
 * counter (mgpu.cu:1574, :1107-1110) */
int  egg_es_update(egg_ctx *ctx, const int32_t *d_fit, const uint32_t *d_seed, const float *d_lr);
/* Ternary-packed matrix weights: no counterpart in the reference (its weights are plain int8; what d-eggs packs in
 * base 3 is the fitness vector, de/include/utils/ternary_pack.h).  The packed blob is the model blob with every matrix
 * tensor at 2 bits per weight -- the four bytes of one blocked dword per byte, element e in bits 2e+1..2e as a 2-bit
 * two's complement number -- and every vector tensor unchanged, tensors in the order of their offsets.  Upload unpacks
 * on the GPU into the canonical int8 blob that every other call uses; download fails with EGG_E_INVALID when a matrix
 * weight is outside {-1, 0, 1} (egg_config.weight_limit = 1 keeps a trained model there). */
int64_t egg_ternary_model_bytes(const egg_ctx *ctx);
int  egg_model_upload_ternary(egg_ctx *ctx, const void *host_packed, size_t bytes);
int  egg_model_download_ternary(egg_ctx *ctx, void *host_packed, size_t bytes);

/* d-eggs adaptive noise overlay.  egg_adaptive_enable: every overlay value starts at init_value
 * (de/src/worker.cu:333, ADAPTIVE_NOISE_INIT 64); from then on the forward scales each noise term by its overlay
 * factor before truncating it (mode 1 of de/include/model/layers.cuh:12-53; sites layers.cuh:94, :177, :240-296,
 * :332-438, de/src/kernels.cu:139-240) and egg_es_update / egg_step apply update_overlay_kernel
 * (de/src/kernels.cu:61-77, +inc where a weight of the row / column / element changed, -dec elsewhere; the
 * reference's ADAPTIVE_NOISE_INC 5, ADAPTIVE_NOISE_DEC 1, de/include/config.h:234-239) after the AdamW update, fed by
 * the change counters of de/include/optimizer/adam.cuh:77-83, :130-132.  AdamW only (EGG_E_INVALID with use_muon).
 * The overlay blob (egg_overlay_upload / _download, egg_model_bytes() bytes) has the layout of the model blob: a vector
 * tensor's values at the tensor's offset, a matrix's `rows` input-dimension values at its offset followed by its
 * `cols` output-dimension values (AdaptiveScales, de/include/model/definitions.h:92-142, keeps them as separate
 * *_row / *_col arrays; the embedding's per-hidden values are its rows here, its per-token values its cols). */
int  egg_adaptive_enable(egg_ctx *ctx, int init_value, int inc, int dec);
int  egg_overlay_upload(egg_ctx *ctx, const void *host_overlay, size_t bytes);
int  egg_overlay_download(egg_ctx *ctx, void *host_overlay, size_t bytes);

/* one tensor of the table returned by egg_tensor_info (test hook for update_matrix_adam_kernel,
 * update_vector_adam_kernel mgpu.cu:1067-1152 and the Muon chain mgpu.cu:1587-1595) */
int  egg_update_tensor(egg_ctx *ctx, int tensor_id, const int32_t *d_fit, const uint32_t *d_seed, const float *d_lr);
/* int32 votes of one matrix tensor in blocked element order (mgpu.cu:1092-1098), test hook */
int  egg_matrix_votes(egg_ctx *ctx, int tensor_id, const int32_t *d_fit, const uint32_t *d_seed, int32_t *d_votes);

/* perform_newton_schulz (muon_internal.cuh:182-342) on a row-major fp32 [rows][cols] device matrix, in place:
 * X /= ||X||_F, then `iters` times X <- 0.5 X (3I - X^T X) on the short side.  Needs a use_muon context; d_X must be
 * 16-byte aligned, rows and cols multiples of 32. */
int  egg_newton_schulz(egg_ctx *ctx, float *d_X, int rows, int cols, int iters);

/* No counterpart in the reference.  egg_newton_schulz for callers that cannot allocate (code under HIP graph capture,
 * serving loops, harnesses that forbid hipMalloc): the same kernels and results, with the workspace (ping-pong matrix,
 * 3I - G term, norm partials; about 5.3 MB) in a static device array of the library instead of a context's buffers, so
 * no context is needed and the call makes no hipMalloc / hipFree.  Limits: rows * cols <= EGG_NS_STATIC_MAX_ELEMS and
 * min(rows, cols) <= EGG_NS_STATIC_MAX_SHORT, else EGG_E_INVALID (message via egg_last_error(NULL)).  Runs on the
 * current device, enqueued on hip_stream (NULL = the default stream).  Every call on a GPU shares that GPU's one
 * workspace: calls that overlap on one GPU (two streams, two threads) race; serialise them. */
#define EGG_NS_STATIC_MAX_ELEMS (512 * 2048)
#define EGG_NS_STATIC_MAX_SHORT 512
int  egg_newton_schulz_static(float *d_X, int rows, int cols, int iters, void *hip_stream);

typedef struct egg_tensor_info {
    char    name[32];
    int     is_matrix, rows, cols;   /* rows = input dim, cols = output dim (vectors: rows = 1) */
    int64_t offset;                  /* byte offset in the model blob                           */
    int     off_a, off_b, seed_base;
    float   lr_scale;
    int     muon;
} egg_tensor_info;
/* The same tables without a context or a GPU (host code only): the tensor table, byte offsets into the model blob
 * (== offsetof in the reference's TransformerModel, mgpu.cu:284-318 / de/include/model/definitions.h:21-54) and into the
 * optimizer state (== offsetof in AdamModel, definitions.h:56-90, with MuonParam for the hidden matrices under use_muon)
 * that a context of this configuration has.  tensor_id < 0 only counts.  Returns the tensor count, or EGG_E_INVALID. */
int  egg_describe_layout(const egg_config *cfg, int tensor_id, egg_tensor_info *out, int64_t *state_offset,
                         int64_t *model_bytes, int64_t *state_bytes);
/* Host code only: the plan by which a use_muon context batches LAUNCH_ADAM_MATRIX's Newton-Schulz chain
 * (mgpu.cu:1587-1595, muon_internal.cuh:182-342; the reference runs it matrix by matrix through one workspace,
 * mgpu.cu:1477-1489).  Matrices of one shape form a group; `batch` of them share the workspace at a time, which holds
 * `matrix_buffer_floats` floats in each of its two matrix buffers and `term_buffer_floats` in the 3I - G buffer, and
 * batch * rows * cols / batch * min(rows, cols)^2 never exceed those.  group < 0 only counts.  Returns the group count. */
int  egg_muon_plan(const egg_config *cfg, int group, int *rows, int *cols, int *members, int *batch,
                   int64_t *matrix_buffer_floats, int64_t *term_buffer_floats);
int  egg_tensor_count(const egg_ctx *ctx);
int  egg_tensor_info_get(const egg_ctx *ctx, int tensor_id, egg_tensor_info *out);

/* d_total_updates read-back (mgpu.cu:1685); synchronises the stream */
int  egg_last_update_count(egg_ctx *ctx, uint64_t *out);

/* whole ES step = forward of the full population + fitness + update, enqueued on the stream:
 * the reference's loop body mgpu.cu:1506-1678 without the host fitness hop */
int  egg_step(egg_ctx *ctx, const uint8_t *d_data, int64_t data_len, int64_t start_idx,
              uint32_t step_seed, float lr);
/* the same step captured once as a hipGraph and replayed (cudaStreamBeginCapture ... cudaGraphLaunch,
 * de/src/worker.cu:435-533); seed, lr and start index live in device scalars written before each launch */
int  egg_step_capture(egg_ctx *ctx, const uint8_t *d_data, int64_t data_len);
int  egg_step_launch(egg_ctx *ctx, int64_t start_idx, uint32_t step_seed, float lr);
/* losses / fitness of the last egg_step* call, copied to host (synchronises) */
int  egg_step_losses(egg_ctx *ctx, int32_t *host_loss, int32_t *host_fit);

/* get_learning_rate (mgpu.cu:217-227) and the d-eggs seed chain seed' = hash_rng(seed, step) (de/src/worker.cu:542) */
float    egg_learning_rate(long step);
float    egg_learning_rate_deggs(long step);      /* d-eggs' schedule, de/include/utils/training.h:5-9 */
/* save_model_info (egg_disk_utils.h:15-44, de/include/utils/io.h:24-53): writes <dir>/model.info (dir NULL = "models") */
int      egg_model_info_save(egg_ctx *ctx, const char *dir);
uint32_t egg_next_seed(uint32_t seed, uint64_t step);

/* generate_sequence_kernel + its call site (mgpu.cu:1154-1283, :1701-1708): d_buffer holds seed_len prompt bytes
 * followed by room for gen_len more (seed_len + gen_len <= seq_len); the unperturbed model continues the prompt with
 * the reference's three-pass LUT sampling, threshold hash_rng(seed + t*555, 0) % sum.  Enqueued on the stream.
 * Like the reference (d_gen_kv, mgpu.cu:1160-1170, :1199-1202) it keeps every layer's K / V rows of the sequence: the
 * prompt is evaluated once, each new token costs one 32-token tile.  egg_ctx_generate_kv_cache(ctx, 0) makes every new
 * token re-evaluate the whole window instead (same tokens; for checks).  With a vocabulary above 256 the buffer holds
 * uint32 tokens (d-eggs' TokenType), here and in egg_generate_deggs; the lengths count tokens. */
int  egg_generate(egg_ctx *ctx, uint8_t *d_buffer, int seed_len, int gen_len, uint32_t seed);
int  egg_ctx_generate_kv_cache(egg_ctx *ctx, int enable);
/* d-eggs' generate_sequence_kernel (d-eggs/src/kernels.cu:307-490, call site d-eggs/src/worker.cu:563-571): the same
 * continuation with its sampler -- every earlier occurrence of a byte lowers that byte's logit by
 * (int)(penalty * 2^shift_logit) (:398-402), differences to the maximum are divided by `temp` in float and truncated
 * (:430), candidates whose scaled difference is below (int)(logf(min_p) * softmax_exp_scale) are left out (:433).
 * temp = 1, min_p = 0, penalty = 0 is egg_generate.  The reference's defaults are 0.6 / 0.08 / 0.2
 * (d-eggs/include/config.h:192-200).  seed_len + gen_len <= 256 and seed_len <= hidden rounded up to 32: beyond
 * that the reference reads its 256-entry token history where nothing was written. */
int  egg_generate_deggs(egg_ctx *ctx, uint8_t *d_buffer, int seed_len, int gen_len, uint32_t seed,
                        float temp, float min_p, float penalty);
/* the two integer constants that sampler derives from min_p and penalty (d-eggs/src/kernels.cu:386-387); host only */
int  egg_deggs_sampling_constants(const egg_config *cfg, float min_p, float penalty, int32_t *penalty_int, int32_t *min_p_limit);

/* ---- host-side companions of the GPU path (host code in the reference as well) ---- */
/* d-eggs worker result shaping (de/src/worker.cu:636-687): loss[count] of `count/2` antithetic pairs -> diff = n - p,
 * optional chunk-mean shift (int)(sign(m) * |m|^mean_exponent) (CHUNK_MEAN_FILTER / CHUNK_MEAN_EXPONENT), optional
 * threshold alpha * mean|diff| below which the vote is 0 (USE_ADAPTIVE_THRESHOLD / ADAPTIVE_THRESHOLD_ALPHA; the
 * reference's alpha is the float literal 0.1f widened to double), else the sign.  sum_loss_out may be NULL. */
int  egg_shape_fitness(const int32_t *loss, int count, int chunk_mean_filter, double mean_exponent,
                       int adaptive_threshold, double alpha, int32_t *fit_out, int64_t *sum_loss_out);
/* base-3 wire packing of ternary votes, five per byte (de/include/utils/ternary_pack.h:11-104) */
size_t egg_ternary_pack_size(size_t count);
int  egg_ternary_pack(const int32_t *src, size_t count, uint8_t *dst);
int  egg_ternary_unpack(const uint8_t *src, size_t count, int32_t *dst);
/* d-eggs' token vocabulary for printing generated tokens (de/src/worker.cu:36-81): "decoding.bin" holds a uint32 count and
 * per token a uint32 length and its bytes.  egg_detokenize concatenates the tokens' strings, "<id>" for an id beyond the
 * table, like the reference's detokenize; it returns the length of the text and writes at most `capacity` bytes of it
 * (no terminator), so a first call with capacity 0 sizes the buffer.  egg_vocab_save writes the same format. */
typedef struct egg_vocab egg_vocab;
int  egg_vocab_load(const char *path, egg_vocab **out);
void egg_vocab_free(egg_vocab *v);
int  egg_vocab_size(const egg_vocab *v);
int  egg_vocab_save(const char *path, const char *const *entries, const uint32_t *lengths, uint32_t count);
int64_t egg_detokenize(const egg_vocab *v, const uint32_t *tokens, int count, char *out, int64_t capacity);
/* save_checkpoint / load_model (egg_disk_utils.h:46-82): <dir>/egg_step-%08ld.model.bin and .adam.bin hold the raw
 * model blob and optimizer state, "egg_transformer_last.*" symlinks point at the newest; dir NULL = "models".
 * Loading checks the file size against this context's shapes; state_path may be NULL.  Both synchronise. */
int  egg_checkpoint_save(egg_ctx *ctx, const char *dir, long step);
int  egg_checkpoint_load(egg_ctx *ctx, const char *model_path, const char *state_path);
/* d-eggs replay checkpoints (de/include/utils/checkpoint.h:17-128): "checkpoint_%08llu.bin" = {magic "EGGC", version 1,
 * step, seed, data_size} + data (the packed fitness history).  load_latest picks the highest step in dir; when the
 * payload exceeds `capacity` it returns EGG_E_STATE with *n set to the size needed. */
int  egg_eggc_save(const char *dir, uint64_t step, uint64_t seed, const uint8_t *data, uint64_t n);
int  egg_eggc_load_latest(const char *dir, uint64_t *step, uint64_t *seed, uint8_t *data, uint64_t capacity, uint64_t *n);

/* debug taps (test hook, no reference counterpart beyond EGG_TRACE_STAT, mgpu.cu:723): when enabled, a
 * forward over at most 64 members keeps every stage's activations; egg_tap_download copies one member's
 * "x_init", "q.L", "k.L", "v.L", "ao.L", "x_attn.L", "x_mlp.L" (L = layer) or "logits" to the host. */
int  egg_ctx_enable_taps(egg_ctx *ctx, int enable);
/* No counterpart in the reference (train_sequence_kernel walks every position, mgpu.cu:901-934).  The block in front of
   the first attention layer depends on the member and the byte value only, so by default it is evaluated once per
   distinct byte value of a member's window and copied to the positions that hold the value; enable = 0 evaluates it
   at every position instead.  The results are identical; the switch exists so that both can be measured and compared.
   Not after egg_step_capture. */
int  egg_ctx_first_block_dedup(egg_ctx *ctx, int enable);
int  egg_tap_download(egg_ctx *ctx, const char *name, int member, void *host_out /* int8 [T][H] natural order; "logits": int32 [T][256] */);

/* ---- the reference's CPU program on the GPU (full_trained_egg.c: GRU-style recurrent byte LM, sequential
 * xorshift noise, +-1 threshold update).  Model blob == EggModel (full_trained_egg.c:42-50) with runtime sizes,
 * every matrix row-major [out][in]; recurrent states [population][n_layers][hidden] persist across steps. ---- */
typedef struct egg_gru_ctx egg_gru_ctx;
typedef struct egg_gru_config {
    int hidden;            /* HIDDEN_DIM 512 (64, 128, 256 or 512)          full_trained_egg.c:12 */
    int n_layers;          /* N_LAYERS 4                                    :13 */
    int seq_len;           /* SEQ_LEN 4096                                  :14 */
    int vocab;             /* VOCAB_SIZE 256                                :11 */
    int population;        /* POPULATION_SIZE 128 (multiple of 32)          :15 */
    int fixed_point;       /* 4                                             :17 */
    int sigma_shift;       /* 4                                             :18 */
    int update_threshold;  /* 160                                           :19 */
} egg_gru_config;
void egg_gru_default_config(egg_gru_config *cfg);
int  egg_gru_create(const egg_gru_config *cfg, egg_gru_ctx **out);          /* init_tables + allocations, :479-518 */
void egg_gru_destroy(egg_gru_ctx *ctx);
const char *egg_gru_last_error(const egg_gru_ctx *ctx);
int64_t egg_gru_model_bytes(const egg_gru_ctx *ctx);
int  egg_gru_model_init(egg_gru_ctx *ctx, uint32_t seed);                    /* :487-509 */
int  egg_gru_model_upload(egg_gru_ctx *ctx, const void *host_model, size_t bytes);
int  egg_gru_model_download(egg_gru_ctx *ctx, void *host_model, size_t bytes);
int  egg_gru_state_reset(egg_gru_ctx *ctx);                                  /* memset(pop_states), :517 */
int  egg_gru_state_download(egg_gru_ctx *ctx, void *host_states, size_t bytes);
/* one training step: forward_pass(+1) and forward_pass(-1) of every pair with pair fitness (:547-562), then, if
 * do_update, update_matrix on every GRU / MLP / head matrix (:564-574) */
int  egg_gru_step(egg_gru_ctx *ctx, const uint8_t *d_data, int64_t data_len, int64_t start_idx, uint32_t step_seed, int do_update);
int  egg_gru_losses(egg_gru_ctx *ctx, int32_t *host_loss, int32_t *host_fit);  /* synchronises */
/* How egg_gru_step evaluates forward_pass (full_trained_egg.c:213-296) -- same results either way.  1 (default): the
 * stages of a layer's token (norm, gate products, state update, norm, expand, project; for the head norm, logits,
 * loss) are spread over the GPU by output strip and member tile, and the sequence is walked as a pipeline over the
 * layers with one launch per tick that carries every stage that is ready (2 T + 6 L + 1 launches, 64 to a hipGraph);
 * 0: one persistent workgroup per 32 members for the whole sequence. */
int  egg_gru_forward_mode(egg_gru_ctx *ctx, int staged);

/* per-kernel-class timing with hipEvent pairs recorded on the context's stream around each launch (the
 * reference only splits Fwd/Host/Upd wall time, full_cuda_train_egg.cu:1116-1126).  Not usable while capturing. */
enum { EGG_K_MLP_FIRST = 0, EGG_K_QKV = 1, EGG_K_ATTN = 2, EGG_K_MLP = 3, EGG_K_HEAD = 4,
       EGG_K_UPDATE_MATRIX = 5, EGG_K_UPDATE_VECTOR = 6, EGG_K_PLINEAR = 7,
       EGG_K_MUON_NS = 8 /* the Newton-Schulz chain of a Muon batch; votes, momentum and apply count as UPDATE_MATRIX */,
       EGG_KCLASS_COUNT = 9 };
int  egg_ctx_enable_timing(egg_ctx *ctx, int enable);
int  egg_timing_reset(egg_ctx *ctx);
int  egg_timing_get(egg_ctx *ctx, int kclass, int64_t *launches, double *total_ms);   /* synchronises */

#ifdef __cplusplus
}
#endif
#endif

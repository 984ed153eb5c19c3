/*
 * egg_oracle.h -- CPU oracle for the EGGROLL population-evaluation hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the product ships may include, link or
 * call this library; only tests, the smoke check and the benchmark's
 * cpu-baseline leg use it, and there only as the checker.
 *
 * Every function restates, in plain scalar C++, arithmetic of the reference
 * programs; the reference file:line each one follows is cited at its
 * definition in egg_oracle.cpp / egg_gru_oracle.cpp.  Shorthand:
 *   mgpu.cu  = full_cuda_train_transformer_adam_mgpu.cu
 *   norm.h   = egg_adaptive_normalize.h
 *   muon_i   = muon_internal.cuh
 *   egg.c    = full_trained_egg.c
 *
 * Pinning status (what checks each function beyond "the restatement itself"):
 *   hash_rng / noise / clip / xorshift / gen_noise_host : the reference's own
 *       host-compilable header (d-eggs/include/utils/egg_math.h) compiled
 *       into oracle/_ref, plus known answers committed under tests/golden.
 *   EXP / GELU / RoPE / EXP2 tables : closed forms + reference screenshot values.
 *   seed offsets, shifts, defaults, model blob layout, optimizer-state layout,
 *       Muon flags : the reference's own config.h / definitions.h / base.h,
 *       compiled in place at four configurations (oracle/ref_layout_shim.cpp),
 *       plus the values committed under tests/golden (tests/test_reference_headers.py).
 *   perturbed linear, norms, attention, loss, fitness, vote : brute
 *       force and special cases in tests/test_oracle_*.py.
 *   vector / matrix AdamW updates, Muon momentum + gather + apply rule : bitwise
 *       numpy evaluations of their definitions (tests/test_oracle_pins.py).
 *   d-eggs sampler (oracle_py.sample_token_deggs) : closed forms only (neutral
 *       settings = the plain sampler, temperature 2 = halved differences, min-p
 *       edge, penalty per occurrence); the reference holds no fixture for it.
 *   Muon Newton-Schulz : fp64 restatement + orthogonality invariants; the
 *       reference's cuBLAS summation order is unspecified => tolerance only.
 *   whole forward (which seed offset, layer base and operand role each perturbation site uses) : the materialised-
 *       perturbation identity.  With the perturbation shifts at zero the rank-1 term is linear in the weights, so
 *       the perturbed forward of a member must equal the unperturbed forward of W + ns*B(x)A, v + ns*n1*n2 built
 *       from the update's tensor table alone; that table is held against the reference's macros by name and against
 *       the optimizer launch list in the reference's step loop (tests/golden/reference_update_launches.json,
 *       re-parsed from the source where the checkout is present).  tests/test_materialised_identity.py requires
 *       every tap, logit and loss to agree, shows that leaving out any one tensor, swapping A and B, borrowing a
 *       neighbour's offsets or dropping the layer base breaks it, and does the same for the CPU program
 *       (forward sites against the update's sites).  On top of that the composition is stated a second time in
 *       numpy, all tokens of the window at once (oracle/forward_numpy.py, oracle/gru_numpy.py), and the two
 *       restatements must agree on every residual-stream tap, logit and loss; the same files state the whole
 *       AdamW update and the CPU program's update a second time.  Which of the five SHIFT_* macros follows which
 *       product is outside the identity (both of its sides shift alike): the sites of mgpu.cu:737, :756, :815, :830,
 *       :976 are held as a fixture parsed from the source (tests/golden/reference_shift_sites.json) and each
 *       configuration field is shown to act at that site and no earlier (test_each_shift_acts_at_the_reference_site).
 *   vocabularies above 256 (uint32 tokens, d-eggs/include/config.h:22-28) : the same functions with V as a parameter;
 *       the loss's closed forms at V = 512 and 8192, and the two restatements of the forward agreeing at V = 768.
 *   Still "parity unpinned" (the reference holds nothing to pin them to): Muon at the cuBLAS boundary (summation
 *       order), the adaptive overlay and the d-eggs sampler beyond their closed forms, ternary-packed weights
 *       (no reference counterpart).
 */
#ifndef EGG_ORACLE_H
#define EGG_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct orc_config {
    int hidden;              /* HIDDEN_DIM            mgpu.cu:35  */
    int head_dim;            /* HEAD_DIM              mgpu.cu:38  */
    int n_layers;            /* N_LAYERS              mgpu.cu:41  */
    int seq_len;             /* SEQ_LEN               mgpu.cu:44  */
    int vocab;               /* VOCAB_SIZE            mgpu.cu:54  */
    int population;          /* POPULATION_SIZE       mgpu.cu:81  */
    int fixed_point;         /* 4                     mgpu.cu:83  */
    int sigma_shift;         /* 3                     mgpu.cu:86  */
    int sigma_shift_vector;  /* 4                     mgpu.cu:89  */
    int shift_attn;          /* 8                     mgpu.cu:172 */
    int shift_out;           /* 9                     mgpu.cu:178 */
    int shift_logit;         /* 8                     mgpu.cu:181 */
    int shift_mlp_up;        /* 8                     mgpu.cu:184 */
    int shift_mlp_down;      /* 10                    mgpu.cu:187 */
    int softmax_scale_bit;   /* 18                    mgpu.cu:95  */
    int rope_scale_bit;      /* 20                    mgpu.cu:107 */
    int noise_mask;          /* DEVICE_MASK 15        mgpu.cu:201 */
    int host_mask;           /* HOST_MASK 15          mgpu.cu:198 */
    double softmax_exp_scale;/* 6.0                   mgpu.cu:102 */
    float adam_beta1, adam_beta2, adam_eps, adam_weight_decay; /* mgpu.cu:246-257 */
    float muon_momentum;     /* 0.85                  mgpu.cu:264 */
    float muon_lr_scale;     /* 1.0                   mgpu.cu:267 */
    int weight_limit;        /* matrix weights saturate at +-this in the update rule: 127, mgpu.cu:1056-1062;
                              * other values have no counterpart in the reference (ternary weights: 1) */
    int device_gaussian;     /* DEVICE_GAUSSIAN false  mgpu.cu:195-196 */
    int host_gaussian;       /* HOST_GAUSSIAN false    mgpu.cu:192-193 */
    int use_same_data;       /* USE_SAME_DATA 0        mgpu.cu:212-213 */
} orc_config;
/* a noise mask word: the magnitude mask in the low byte, 0x100 on top for the Gaussian form (three masked fields) */
#define ORC_NOISE_GAUSSIAN 0x100

void orc_default_config(orc_config *c);
int  orc_seed_offset(const char *reference_macro_name);   /* the oracle's seed-offset enum, by reference macro name */

/* ---- RNG (mgpu.cu:428-441, :525-539) ---- */
uint32_t orc_hash_rng(uint32_t s, uint32_t idx);
int8_t   orc_noise(uint32_t s, uint32_t idx, int mask);
uint32_t orc_xorshift32(uint32_t *state);
int8_t   orc_gen_noise_host(uint32_t *state, int mask);
int8_t   orc_clip(int32_t a);

/* ---- tables (mgpu.cu:394-426) ---- */
void orc_tables(const orc_config *c, int32_t *exp_lut /*256*/, int8_t *act_lut /*256*/,
                int32_t *rope_lut /* seq_len*head_dim */);

/* ---- model (mgpu.cu:284-318, :443-519) ---- */
typedef struct orc_tensor {
    char    name[32];
    int     is_matrix;     /* 1: blocked [rows/4][cols][4] matrix, 0: vector          */
    int     rows, cols;    /* matrix: rows = input dim, cols = output dim; vector: cols=len, rows=1 */
    int64_t offset;        /* byte offset inside the model blob == element offset     */
    int     off_a, off_b;  /* seed offsets (output-dim noise, input-dim noise)        */
    int     seed_base;     /* 1000*layer or 0                                         */
    float   lr_scale;      /* 1.0, or 0.1 for emb_bias (mgpu.cu:1635)                 */
    int     muon;          /* 1 if the reference routes it through Muon under USE_MUON */
} orc_tensor;

int64_t orc_model_bytes(const orc_config *c);
int     orc_tensor_table(const orc_config *c, orc_tensor *out, int max_out); /* returns count */
void    orc_repack(int8_t *dst, const int8_t *src, int rows, int cols);      /* mgpu.cu:443 */
void    orc_unpack(int8_t *dst, const int8_t *src_blocked, int rows, int cols);
void    orc_init_model(const orc_config *c, int8_t *model, uint32_t seed);  /* mgpu.cu:461 */

/* ternary-packed matrix weights: no reference counterpart (parity unpinned by construction); see egg_oracle.cpp */
int64_t orc_ternary_model_bytes(const orc_config *c);
int     orc_ternary_model_pack(const orc_config *c, const int8_t *model, uint8_t *packed);   /* -1: a weight outside {-1,0,1} */
void    orc_ternary_model_unpack(const orc_config *c, const uint8_t *packed, int8_t *model);

/* ---- forward (mgpu.cu:553-1029, norm.h) ---- */
typedef struct orc_trace {   /* any pointer may be NULL */
    int8_t  *x_emb;      /* [T][H] after embedding stage                       */
    int8_t  *x_init;     /* [T][H] after the initial MLP                       */
    int8_t  *q, *k, *v;  /* [L][T][H] normalised int8 q / k / v                */
    int8_t  *ao;         /* [L][T][H] attention output before O-projection     */
    int8_t  *x_attn;     /* [L][T][H] residual stream after attention          */
    int8_t  *x_mlp;      /* [L][T][H] residual stream after the MLP            */
    int8_t  *nf;         /* [T][H] final-norm output                           */
    int32_t *logits;     /* [T][V] int32 logits (after >> shift_logit)         */
    int64_t *loss_t;     /* [T] per-token loss                                 */
} orc_trace;

/* one population member, serial in t exactly like the reference kernel;
 * ns_override: 2 = use parity of p_idx (reference), otherwise force ns to that value (-1,0,1) */
int32_t orc_forward_member(const orc_config *c, const int8_t *model,
                           const uint8_t *data, int64_t data_len, int64_t start_idx,
                           uint32_t step_seed, int p_idx, int ns_override, orc_trace *trace);

/* members [pop_offset, pop_offset+count) -> loss[pop_offset + i]; OpenMP over members */
void orc_population_forward(const orc_config *c, const int8_t *model,
                            const uint8_t *data, int64_t data_len, int64_t start_idx,
                            uint32_t step_seed, int pop_offset, int count, int32_t *loss);

/* d-eggs adaptive noise overlay (de/include/model/layers.cuh:12-53, mode 1; sites :94, :177, :240-296, :332-438,
 * de/src/kernels.cu:139-240).  `overlay` has the layout of the model blob: a vector tensor's values at the tensor's
 * offset, a matrix's `rows` input-dimension values at its offset followed by its `cols` output-dimension values.
 * Parity unpinned beyond the special cases in the tests: the reference has no test or fixture for it and its
 * CUDA sources cannot be built here. */
float   orc_adaptive_factor(int overlay_value);
int32_t orc_scaled_noise(int noise, int overlay_value);          /* (int)(noise * factor), layers.cuh:94 */
int32_t orc_noise_dot_adaptive(const orc_config *c, const int8_t *in, int K, uint32_t seed, const int8_t *overlay_rows);
int32_t orc_down_dot_adaptive(const orc_config *c, const int8_t *mlp, int H, uint32_t seed, const int8_t *overlay_rows); /* layers.cuh:268-276 */
int32_t orc_forward_member_adaptive(const orc_config *c, const int8_t *model, const int8_t *overlay,
                                    const uint8_t *data, int64_t data_len, int64_t start_idx,
                                    uint32_t step_seed, int p_idx, int ns_override, orc_trace *trace);
void    orc_population_forward_adaptive(const orc_config *c, const int8_t *model, const int8_t *overlay,
                                        const uint8_t *data, int64_t data_len, int64_t start_idx,
                                        uint32_t step_seed, int pop_offset, int count, int32_t *loss);

/* perturbed linear microbench semantics: rows = members*T, member = row / T,
 * pair = member/2, ns = +1 even / -1 odd member;
 * acc = X.W + (((X.B) * A[n]) * ns >> (fixed_point+sigma_shift)); Y = acc >> shift  (mgpu.cu:553-572) */
void orc_perturbed_linear(const orc_config *c, const int8_t *X, const int8_t *W_blocked,
                          int64_t n_rows, int T, int K, int N, uint32_t seed,
                          int off_a, int off_b, int shift, int32_t *Y);

/* stage-level helpers exposed so tests can pin them in isolation */
void orc_standard_norm(const orc_config *c, const int8_t *x, const int8_t *w, const int8_t *b,
                       int H, uint32_t seed_base, int off_w_a, int off_w_b, int off_b_a, int off_b_b,
                       int ns, int8_t *out);                                   /* mgpu.cu:646-678 */
void orc_adaptive_normalize(const int32_t *val, int n, int8_t *out);          /* norm.h:10-103   */
void orc_rope(const orc_config *c, const int32_t *rope_lut, const int32_t *val, int t, int H, int32_t *out); /* mgpu.cu:624-644 */
void orc_attention_core(const orc_config *c, const int32_t *exp_lut,
                        const int8_t *q /*[H]*/, const int8_t *kc /*[t+1][H]*/, const int8_t *vc,
                        int t, int H, int8_t *ao);                             /* mgpu.cu:787-824 */
int64_t orc_token_loss(const orc_config *c, const int32_t *exp_lut, const int32_t *logits, int V, int target); /* mgpu.cu:969-1023 */

/* ---- fitness (mgpu.cu:1305-1311) ---- */
void orc_fitness(const int32_t *loss, int32_t *fit, int pairs);

/* ---- ES update (mgpu.cu:1040-1152) ---- */
typedef struct orc_adam_param { float m, v, acc; } orc_adam_param;  /* mgpu.cu:321-325 */
typedef struct orc_muon_param { float m, acc; } orc_muon_param;     /* mgpu.cu:328-331 */

void orc_adam_apply(const orc_config *c, orc_adam_param *p, int8_t *w, float g, float lr, int *change);
int64_t orc_matrix_votes(const orc_config *c, int rows, int cols, int off_a, int off_b, int seed_base,
                         const int32_t *fit, int pairs, uint32_t step_seed, int32_t *votes_blocked);
uint64_t orc_update_matrix_adam(const orc_config *c, int8_t *W, orc_adam_param *st, int rows, int cols,
                                int off_a, int off_b, int seed_base, const int32_t *fit, int pairs,
                                uint32_t step_seed, float lr);
uint64_t orc_update_vector_adam(const orc_config *c, int8_t *V, orc_adam_param *st, int len,
                                int off_a, int off_b, int seed_base, const int32_t *fit, int pairs,
                                uint32_t step_seed, float lr);
/* all tensors in the reference's launch order (mgpu.cu:1603-1643); state laid out like
 * AdamModel with 12-byte AdamParam for every element; returns the update counter */
uint64_t orc_es_update_adam(const orc_config *c, int8_t *model, orc_adam_param *state,
                            const int32_t *fit, uint32_t step_seed, float lr);
float orc_learning_rate(long step);   /* mgpu.cu:217-227 */
/* d-eggs overlay rule and the optimizer step that feeds it (de/src/kernels.cu:61-77, de/src/worker.cu:446-523) */
void     orc_update_overlay(const int32_t *changes, int8_t *overlay, int count, int inc, int dec);
uint64_t orc_es_update_adam_adaptive(const orc_config *c, int8_t *model, orc_adam_param *state, int8_t *overlay,
                                     const int32_t *fit, uint32_t step_seed, float lr, int inc, int dec);

/* ---- Muon (muon_i:15-342, launch macro mgpu.cu:1587-1595) ---- */
/* fp32 restatement with sequential-k summation; X row-major [rows][cols], in place */
void orc_newton_schulz_f32(float *X, int rows, int cols, int iters);
void orc_newton_schulz_f64(double *X, int rows, int cols, int iters);
uint64_t orc_update_matrix_muon(const orc_config *c, int8_t *W, orc_muon_param *st, int rows, int cols,
                                int off_a, int off_b, int seed_base, const int32_t *fit, int pairs,
                                uint32_t step_seed, float lr, float *ortho_out /* [rows][cols] or NULL */);

/* ---- CPU GRU path (egg.c) ---- */
typedef struct orc_gru_config {
    int hidden, n_layers, seq_len, vocab, population;   /* egg.c:11-15 */
    int fixed_point, sigma_shift, update_threshold;     /* egg.c:17-19 */
} orc_gru_config;
void    orc_gru_default_config(orc_gru_config *c);
int64_t orc_gru_model_bytes(const orc_gru_config *c);
int64_t orc_gru_state_bytes(const orc_gru_config *c);     /* per member */
void    orc_gru_init_model(const orc_gru_config *c, int8_t *model, uint32_t seed);   /* egg.c:487-509 */
void    orc_gru_noise_vector(uint32_t *rng, int8_t *out, int count);                 /* egg.c:87-105 */
void    orc_gru_matmul_perturbed(const orc_gru_config *c, const int8_t *in, const int8_t *w, int8_t *out,
                                 int rows, int cols, uint32_t layer_seed, int noise_sign, int shift); /* egg.c:108-177 */
void    orc_gru_ln(const int8_t *x, const int8_t *w, int8_t *out, int H);             /* egg.c:180-210 */
int32_t orc_gru_compute_loss(const int8_t *logits, int V, int target, int fixed_point); /* egg.c:299-330 */
int32_t orc_gru_forward(const orc_gru_config *c, const int8_t *model, const uint8_t *inputs,
                        const uint8_t *targets, int seq_len, int8_t *logits_out,
                        uint32_t step_seed, int noise_sign, int8_t *state); /* egg.c:213-296 */
/* pairs [pair0, pair0+npairs): forward +/- for each, write loss[2p], loss[2p+1], fit[p]; OpenMP over pairs */
void    orc_gru_population(const orc_gru_config *c, const int8_t *model, const uint8_t *data, int64_t data_len,
                           int64_t start_idx, uint32_t step_seed, int pair0, int npairs,
                           int8_t *states, int32_t *loss, int32_t *fit);              /* egg.c:547-562 */
void    orc_gru_update_matrix(const orc_gru_config *c, int8_t *W, int rows, int cols, uint32_t seed,
                              const int32_t *fit, int pop_size);                       /* egg.c:332-409 */
void    orc_gru_update_all(const orc_gru_config *c, int8_t *model, uint32_t step_seed, const int32_t *fit); /* egg.c:564-574 */
int     orc_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif

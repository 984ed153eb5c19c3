/*
 * ref_layout_shim.cpp -- exports, as plain numbers, what the reference's own host-compilable headers
 * d-eggs/include/config.h, d-eggs/include/optimizer/base.h, d-eggs/include/model/definitions.h and
 * d-eggs/include/utils/training.h fix at compile time: every configuration macro on the hot path (seed offsets,
 * shifts, fixed-point and sigma shifts, noise masks, optimizer hyper-parameters, adaptive-noise constants) and the
 * size and offset of every field of TransformerModel, AdamModel, AdaptiveScales, AdamParam and MuonParam.
 * oracle/Makefile compiles it from where those headers lie under $(REF), once per (HIDDEN_DIM, N_LAYERS, USE_MUON)
 * variant, into oracle/_ref/libegg_ref_layout_*.so.
 * TEST INFRASTRUCTURE ONLY: it pins the oracle's seed-offset table, defaults and model / optimizer-state layout
 * (and, through a host-only query of the C ABI, the product's).  No reference source is copied here.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#include EGG_REF_DEFINITIONS_H
#include EGG_REF_TRAINING_H

struct Macro { const char *name; double value; };
#define M(x) {#x, (double)(x)}
static const Macro macros[] = {
    M(HIDDEN_DIM), M(HEAD_DIM), M(N_LAYERS), M(SEQ_LEN), M(VOCAB_SIZE), M(N_HEADS), M(EGG_BLOCK_THREADS),
    M(CHUNK_SIZE), M(POPULATION_BATCH_SIZE), M(POPULATION_SIZE),
    M(FIXED_POINT), M(SIGMA_SHIFT), M(SIGMA_SHIFT_VECTOR), M(MAX_VAL), M(MIN_VAL),
    M(SOFTMAX_SCALE_BIT), M(SOFTMAX_LUT_SIZE), M(SOFTMAX_EXP_SCALE), M(ROPE_SCALE_BIT),
    M(SEED_OFF_EMB), M(SEED_OFF_EMB_BIAS_A), M(SEED_OFF_EMB_BIAS_B),
    M(SEED_OFF_LN_1_A), M(SEED_OFF_LN_1_B), M(SEED_OFF_LN_1_BIAS_A), M(SEED_OFF_LN_1_BIAS_B),
    M(SEED_OFF_Q_A), M(SEED_OFF_Q_B), M(SEED_OFF_K_A), M(SEED_OFF_K_B), M(SEED_OFF_V_A), M(SEED_OFF_V_B),
    M(SEED_OFF_O_A), M(SEED_OFF_O_B),
    M(SEED_OFF_LN_2_A), M(SEED_OFF_LN_2_B), M(SEED_OFF_LN_2_BIAS_A), M(SEED_OFF_LN_2_BIAS_B),
    M(SEED_OFF_MLP_UP_A), M(SEED_OFF_MLP_UP_B), M(SEED_OFF_MLP_DOWN_A), M(SEED_OFF_MLP_DOWN_B),
    M(SEED_OFF_MLP_BIAS_UP_A), M(SEED_OFF_MLP_BIAS_UP_B), M(SEED_OFF_MLP_BIAS_DOWN_A), M(SEED_OFF_MLP_BIAS_DOWN_B),
    M(SEED_OFF_LN_F_A), M(SEED_OFF_LN_F_B), M(SEED_OFF_LN_F_BIAS_A), M(SEED_OFF_LN_F_BIAS_B), M(SEED_OFF_HEAD),
    M(SEED_OFF_LN_INIT_A), M(SEED_OFF_LN_INIT_B), M(SEED_OFF_LN_INIT_BIAS_A), M(SEED_OFF_LN_INIT_BIAS_B),
    M(SEED_OFF_EMB_MLP_UP_A), M(SEED_OFF_EMB_MLP_UP_B), M(SEED_OFF_EMB_MLP_DOWN_A), M(SEED_OFF_EMB_MLP_DOWN_B),
    M(SEED_OFF_EMB_MLP_BIAS_UP_A), M(SEED_OFF_EMB_MLP_BIAS_UP_B),
    M(SEED_OFF_EMB_MLP_BIAS_DOWN_A), M(SEED_OFF_EMB_MLP_BIAS_DOWN_B),
    M(SHIFT_ATTN), M(SHIFT_QKV), M(SHIFT_OUT), M(SHIFT_LOGIT), M(SHIFT_MLP_UP), M(SHIFT_MLP_DOWN),
    M(HOST_GAUSSIAN), M(DEVICE_GAUSSIAN), M(HOST_MASK), M(DEVICE_MASK), M(USE_SAME_DATA),
    M(ADAM_BETA1), M(ADAM_BETA2), M(ADAM_EPS), M(ADAM_WEIGHT_DECAY), M(USE_MUON),
#if USE_MUON
    M(MUON_MOMENTUM), M(MUON_LR_SCALE),
#endif
    M(SAMPLING_TEMP), M(SAMPLING_MIN_P), M(SAMPLING_PRESENCE_PENALTY),
    M(USE_ADAPTIVE_THRESHOLD), M(ADAPTIVE_THRESHOLD_ALPHA), M(CHUNK_MEAN_FILTER), M(CHUNK_MEAN_EXPONENT),
    M(ADAPTIVE_NOISE_MODE), M(ADAPTIVE_NOISE_INC), M(ADAPTIVE_NOISE_DEC), M(ADAPTIVE_NOISE_INIT),
};

struct Field { const char *strct, *name; size_t offset, size; };
#define F(S, f) {#S, #f, offsetof(S, f), sizeof(((S *)0)->f)}
#define SZ(S) {#S, "", 0, sizeof(S)}
#define MODEL_FIELDS(S) \
    F(S, embedding), F(S, emb_bias), F(S, ln_init), F(S, ln_init_bias), F(S, w_emb_mlp_up), F(S, mlp_emb_bias_up), \
    F(S, w_emb_mlp_down), F(S, mlp_emb_bias_down), F(S, ln_1), F(S, ln_1_bias), F(S, w_q), F(S, w_k), F(S, w_v), F(S, w_o), \
    F(S, ln_2), F(S, ln_2_bias), F(S, w_up), F(S, mlp_bias_up), F(S, w_down), F(S, mlp_bias_down), F(S, ln_f), F(S, ln_f_bias)
static const Field fields[] = {
    SZ(TransformerModel), MODEL_FIELDS(TransformerModel),
    SZ(AdamModel), MODEL_FIELDS(AdamModel),
    SZ(AdamParam), F(AdamParam, m), F(AdamParam, v), F(AdamParam, acc),
#if USE_MUON == 1
    SZ(MuonParam), F(MuonParam, m), F(MuonParam, acc),
#endif
    SZ(HIDDEN_OPT_TYPE),
    SZ(AdaptiveScales),
    F(AdaptiveScales, embedding_row), F(AdaptiveScales, embedding_col), F(AdaptiveScales, emb_bias),
    F(AdaptiveScales, ln_init), F(AdaptiveScales, ln_init_bias),
    F(AdaptiveScales, w_emb_mlp_up_row), F(AdaptiveScales, w_emb_mlp_up_col), F(AdaptiveScales, mlp_emb_bias_up),
    F(AdaptiveScales, w_emb_mlp_down_row), F(AdaptiveScales, w_emb_mlp_down_col), F(AdaptiveScales, mlp_emb_bias_down),
    F(AdaptiveScales, ln_1), F(AdaptiveScales, ln_1_bias), F(AdaptiveScales, w_q_row), F(AdaptiveScales, w_q_col),
    F(AdaptiveScales, w_k_row), F(AdaptiveScales, w_k_col), F(AdaptiveScales, w_v_row), F(AdaptiveScales, w_v_col),
    F(AdaptiveScales, w_o_row), F(AdaptiveScales, w_o_col), F(AdaptiveScales, ln_2), F(AdaptiveScales, ln_2_bias),
    F(AdaptiveScales, w_up_row), F(AdaptiveScales, w_up_col), F(AdaptiveScales, mlp_bias_up),
    F(AdaptiveScales, w_down_row), F(AdaptiveScales, w_down_col), F(AdaptiveScales, mlp_bias_down),
    F(AdaptiveScales, ln_f), F(AdaptiveScales, ln_f_bias),
};

extern "C" {
int ref_macro_count(void) { return (int)(sizeof(macros) / sizeof(macros[0])); }
const char *ref_macro_name(int i) { return macros[i].name; }
double ref_macro_value(int i) { return macros[i].value; }
int ref_field_count(void) { return (int)(sizeof(fields) / sizeof(fields[0])); }
const char *ref_field_struct(int i) { return fields[i].strct; }
const char *ref_field_name(int i) { return fields[i].name; }        /* "" = the struct itself (size only) */
uint64_t ref_field_offset(int i) { return fields[i].offset; }
uint64_t ref_field_size(int i) { return fields[i].size; }
/* d-eggs' schedule (d-eggs/include/utils/training.h:5-9); the single-file trainer's differs */
float ref_deggs_learning_rate(long step) { return get_learning_rate(step); }
}

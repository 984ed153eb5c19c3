// egg_params.h -- plain-data parameter blocks passed by value to the forward kernels.
#pragma once
#include <stdint.h>

// seed offsets (mgpu.cu:114-165)
enum {
    OFF_EMB = 0, OFF_EMB_BIAS_A = 50, OFF_EMB_BIAS_B = 51,
    OFF_LN_1_A = 100, OFF_LN_1_B = 101, OFF_LN_1_BIAS_A = 110, OFF_LN_1_BIAS_B = 111,
    OFF_Q_A = 200, OFF_Q_B = 201, OFF_K_A = 202, OFF_K_B = 203,
    OFF_V_A = 204, OFF_V_B = 205, OFF_O_A = 206, OFF_O_B = 207,
    OFF_LN_2_A = 300, OFF_LN_2_B = 301, OFF_LN_2_BIAS_A = 310, OFF_LN_2_BIAS_B = 311,
    OFF_MLP_UP_A = 400, OFF_MLP_UP_B = 401, OFF_MLP_DOWN_A = 402, OFF_MLP_DOWN_B = 403,
    OFF_MLP_BIAS_UP_A = 410, OFF_MLP_BIAS_UP_B = 411, OFF_MLP_BIAS_DOWN_A = 412, OFF_MLP_BIAS_DOWN_B = 413,
    OFF_LN_F_A = 900, OFF_LN_F_B = 901, OFF_LN_F_BIAS_A = 910, OFF_LN_F_BIAS_B = 911,
    OFF_LN_INIT_A = 500, OFF_LN_INIT_B = 501, OFF_LN_INIT_BIAS_A = 502, OFF_LN_INIT_BIAS_B = 503,
    OFF_EMB_MLP_UP_A = 510, OFF_EMB_MLP_UP_B = 511, OFF_EMB_MLP_DOWN_A = 512, OFF_EMB_MLP_DOWN_B = 513,
    OFF_EMB_MLP_BIAS_UP_A = 514, OFF_EMB_MLP_BIAS_UP_B = 515,
    OFF_EMB_MLP_BIAS_DOWN_A = 516, OFF_EMB_MLP_BIAS_DOWN_B = 517
};

// A noise mask word is the magnitude mask (DEVICE_MASK, mgpu.cu:201) in its low byte, plus this flag for the
// reference's DEVICE_GAUSSIAN form (mgpu.cu:530-534: the sum of three masked fields of the hash)
#define EGG_NOISE_GAUSSIAN 0x100
// largest |noise| a mask word can produce
static inline int egg_noise_magnitude(int mask) { return (mask & EGG_NOISE_GAUSSIAN) ? 3 * (mask & 0xff) : (mask & 0xff); }

// Largest |value| the MLP's up accumulator can hold: the GEMM over `hidden` int8 products plus the seed
// (bias + 128 + vector noise) << shift_mlp_up that folds the bias and the GELU table's index offset into it.  The
// vector noise is (n1 * n2 * ns) >> sigma_vec with |n| <= the noise magnitude (an arithmetic shift: one more on the
// negative side).
static inline long long egg_mlp_up_acc_bound(int hidden, int mask, int sigma_vec, int shift_mlp_up) {
    const long long mag = egg_noise_magnitude(mask);
    const long long seed = 127 + 128 + ((mag * mag) >> sigma_vec) + 1;
    return (long long)hidden * 127 * 127 + (seed << shift_mlp_up);
}

// what every forward kernel needs to know about the run
struct FwdCommon {
    const uint8_t  *data;        // token stream (device): bytes, or uint32 tokens when token_bytes is 4
    int64_t         data_len;
    const int64_t  *d_start_idx; // device scalar: step * seq_len
    const uint32_t *d_step_seed; // device scalar
    int pop_offset;              // global index of the chunk's first member
    int n_members;               // members in the chunk
    int population;
    int same_data;               // USE_SAME_DATA: every pair reads the window at the start index
    int T, H, head_dim, vocab;
    int token_bytes;             // 1 (vocab 256) or 4 (larger vocabularies); data_len counts tokens
    int t0, tn;                  // token positions [t0, t0 + tn) of every member are evaluated (multiples of 32; the whole window: 0, T);
                                 // attention still reads the K / V rows of every position in front of them
    int sigma;                   // fixed_point + sigma_shift
    int sigma_vec;               // sigma_shift_vector
    int mask;                    // noise magnitude mask
    int shift_attn, shift_out, shift_logit, shift_mlp_up, shift_mlp_down;
    int softmax_scale_bit, rope_scale_bit;
    const int32_t *exp_lut;      // [256]
    const int8_t  *act_lut;      // [256]
    const int32_t *rope_lut;     // [T][head_dim]
};

// one MLP block (the initial MLP or a layer's MLP), optionally preceded by the attention output projection
struct MlpParams {
    FwdCommon c;
    int seed_base;               // 1000 * layer, or 0 for the initial MLP
    // seed offsets of the block (MlpConfig, mgpu.cu:680-706)
    int off_ln_a, off_ln_b, off_lnb_a, off_lnb_b, off_up_a, off_up_b, off_bup_a, off_bup_b,
        off_dn_a, off_dn_b, off_bdn_a, off_bdn_b;
    const int8_t *ln_w, *ln_b, *b_up, *b_dn;   // canonical model blob
    const int8_t *w_up, *w_dn;                 // fragment-major copies
    // FIRST: embedding stage inputs
    const int8_t *embedding, *emb_bias;
    // !FIRST: attention output projection inputs
    const int8_t *w_o;           // fragment-major copy
    const int8_t *ao;            // [n_members][T][H] slot order
    int8_t *x;                   // [n_members][T][H] slot order, read (if !FIRST) and written
    int8_t *x_mid;               // optional tap: residual stream after attention (may be null)
    int8_t *tab;                 // FIRST: [n_members][T][H] scratch rows, one per distinct byte value of a member's window (null: one row per position)
    // adaptive noise overlay (all null when it is off): q values (0..64) of the tensors above; a matrix has its
    // input-row values first and its output-column values right behind them
    const int8_t *q_ln_w, *q_ln_b, *q_b_up, *q_b_dn, *q_up, *q_dn, *q_o, *q_emb, *q_emb_bias;
};

struct QkvParams {
    FwdCommon c;
    int seed_base;
    const int8_t *ln_w, *ln_b;   // canonical
    const int8_t *w_q, *w_k, *w_v;   // fragment-major copies
    const int8_t *x;
    int8_t *q, *k, *v;           // [n_members][T][H] slot order
    const int8_t *q_ln_w, *q_ln_b, *q_wq, *q_wk, *q_wv;   // adaptive noise overlay q values, or null
};

struct AttnParams {
    FwdCommon c;
    const int8_t *q, *k, *v;
    int8_t *ao;
};

struct HeadParams {
    FwdCommon c;
    const int8_t *ln_w, *ln_b;
    const int8_t *embedding_frag; // fragment-major copy of the tied embedding [H][vocab]
    const int8_t *x;
    unsigned long long *loss_acc; // [population] two's-complement int64 accumulators
    int32_t *logits_tap;          // optional [n_members][T][vocab] natural order (may be null)
    const int8_t *q_ln_w, *q_ln_b, *q_emb;   // adaptive noise overlay q values (embedding: H per-hidden, then vocab per-token), or null
};

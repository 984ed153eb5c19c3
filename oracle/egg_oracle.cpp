/*
 * egg_oracle.cpp -- scalar CPU restatement of the Int8NativeFormer hot path.
 * TEST INFRASTRUCTURE ONLY (see egg_oracle.h).  Build with
 *   g++ -O2 -ffp-contract=off -fno-fast-math -fopenmp
 * so that every float operation is one IEEE-754 single operation, in the
 * order written here.
 *
 * The forward pass is written "as the reference kernel runs it": one member,
 * serial in t, an explicit loop over the hidden unit that a reference thread
 * would own, a K/V cache per layer.
 */
#include "egg_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <limits.h>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

/* seed offsets, mgpu.cu:114-165 */
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

/* the enum above by the reference's macro name ("SEED_OFF_Q_A" -> OFF_Q_A); -1 for an unknown name.  It exists so
 * that a test can hold this table against the reference's own d-eggs/include/config.h:79-134. */
extern "C" int orc_seed_offset(const char *name) {
    static const struct { const char *n; int v; } tab[] = {
#define SO(x) {"SEED_OFF_" #x, OFF_##x}
        SO(EMB), SO(EMB_BIAS_A), SO(EMB_BIAS_B), SO(LN_1_A), SO(LN_1_B), SO(LN_1_BIAS_A), SO(LN_1_BIAS_B),
        SO(Q_A), SO(Q_B), SO(K_A), SO(K_B), SO(V_A), SO(V_B), SO(O_A), SO(O_B),
        SO(LN_2_A), SO(LN_2_B), SO(LN_2_BIAS_A), SO(LN_2_BIAS_B),
        SO(MLP_UP_A), SO(MLP_UP_B), SO(MLP_DOWN_A), SO(MLP_DOWN_B),
        SO(MLP_BIAS_UP_A), SO(MLP_BIAS_UP_B), SO(MLP_BIAS_DOWN_A), SO(MLP_BIAS_DOWN_B),
        SO(LN_F_A), SO(LN_F_B), SO(LN_F_BIAS_A), SO(LN_F_BIAS_B),
        SO(LN_INIT_A), SO(LN_INIT_B), SO(LN_INIT_BIAS_A), SO(LN_INIT_BIAS_B),
        SO(EMB_MLP_UP_A), SO(EMB_MLP_UP_B), SO(EMB_MLP_DOWN_A), SO(EMB_MLP_DOWN_B),
        SO(EMB_MLP_BIAS_UP_A), SO(EMB_MLP_BIAS_UP_B), SO(EMB_MLP_BIAS_DOWN_A), SO(EMB_MLP_BIAS_DOWN_B),
#undef SO
    };
    for (const auto &e : tab) if (!strcmp(e.n, name)) return e.v;
    return -1;
}

extern "C" void orc_default_config(orc_config *c) {
    memset(c, 0, sizeof(*c));
    c->hidden = 256; c->head_dim = 64; c->n_layers = 4; c->seq_len = 32; c->vocab = 256;
    c->population = 16384 * 4;
    c->fixed_point = 4; c->sigma_shift = 3; c->sigma_shift_vector = 4;
    c->shift_attn = 8; c->shift_out = 9; c->shift_logit = 8; c->shift_mlp_up = 8; c->shift_mlp_down = 10;
    c->softmax_scale_bit = 18; c->rope_scale_bit = 20; c->noise_mask = 15; c->host_mask = 15;
    c->softmax_exp_scale = 6.0;
    c->adam_beta1 = 0.9f; c->adam_beta2 = 0.95f; c->adam_eps = 1e-8f; c->adam_weight_decay = 0.01f;
    c->muon_momentum = 0.85f; c->muon_lr_scale = 1.0f; c->weight_limit = 127; c->device_gaussian = 0; c->host_gaussian = 0; c->use_same_data = 0;
}

/* ------------------------------------------------------------------ RNG */
/* mgpu.cu:525-527 */
extern "C" uint32_t orc_hash_rng(uint32_t s, uint32_t idx) {
    uint32_t x = s + idx * 0x9e3779b9u;
    x ^= x >> 16; x *= 0x85ebca6bu; x ^= x >> 13; x *= 0xc2b2ae35u; x ^= x >> 16;
    return x;
}
/* the three fields of the Gaussian forms (mgpu.cu:433-436, :530-533): sign bits 0, 5, 10; magnitudes from bits 1, 6, 11 */
static inline int noise_fields(uint32_t r, int maskword) {
    const uint32_t m = (uint32_t)maskword & 0xffu;
    int n = (r & 1 ? 1 : -1) * (int)((r >> 1) & m);
    if (maskword & ORC_NOISE_GAUSSIAN) {
        n += (r & 32 ? 1 : -1) * (int)((r >> 6) & m);
        n += (r & 1024 ? 1 : -1) * (int)((r >> 11) & m);
    }
    return n;
}
/* mgpu.cu:528-538; mask is a noise mask word */
extern "C" int8_t orc_noise(uint32_t s, uint32_t idx, int mask) {
    return (int8_t)noise_fields(orc_hash_rng(s, idx), mask);
}
/* mgpu.cu:428-430 */
extern "C" uint32_t orc_xorshift32(uint32_t *state) {
    uint32_t x = *state; x ^= x << 13; x ^= x >> 17; x ^= x << 5; *state = x; return x;
}
/* mgpu.cu:431-441; mask is a noise mask word */
extern "C" int8_t orc_gen_noise_host(uint32_t *state, int mask) {
    return (int8_t)noise_fields(orc_xorshift32(state), mask);
}
static inline int dev_mask(const orc_config *c) { return c->noise_mask | (c->device_gaussian ? ORC_NOISE_GAUSSIAN : 0); }
static inline int host_mask_word(const orc_config *c) { return c->host_mask | (c->host_gaussian ? ORC_NOISE_GAUSSIAN : 0); }
/* mgpu.cu:539 */
extern "C" int8_t orc_clip(int32_t a) { return (a > 127) ? 127 : ((a < -127) ? -127 : (int8_t)a); }

/* ------------------------------------------------------------------ tables */
/* mgpu.cu:394-426 */
extern "C" void orc_tables(const orc_config *c, int32_t *exp_lut, int8_t *act_lut, int32_t *rope_lut) {
    if (exp_lut) {
        double scale = (double)(1 << c->softmax_scale_bit);
        for (int i = 0; i < 256; i++) {
            double val = exp(-(double)i / c->softmax_exp_scale) * scale;
            exp_lut[i] = (val >= 1.0) ? (int32_t)round(val) : 0;
        }
    }
    if (act_lut) {
        for (int i = 0; i < 256; i++) {
            int8_t input = (int8_t)i;
            double x = (double)input / (1 << c->fixed_point);
            double y = 0.5 * x * (1.0 + erf(x / 1.41421356));
            int val = (int)round(y * (1 << c->fixed_point));
            act_lut[i] = (int8_t)((val > 127) ? 127 : ((val < -127) ? -127 : val));
        }
    }
    if (rope_lut) {
        double rs = (double)(1 << c->rope_scale_bit);
        for (int t = 0; t < c->seq_len; t++)
            for (int i = 0; i < c->head_dim / 2; i++) {
                double theta = pow(10000.0, -2.0 * i / c->head_dim);
                double alpha = t * theta;
                rope_lut[t * c->head_dim + i * 2]     = (int32_t)round(cos(alpha) * rs);
                rope_lut[t * c->head_dim + i * 2 + 1] = (int32_t)round(sin(alpha) * rs);
            }
    }
}

/* ------------------------------------------------------------------ model layout */
/* field order of TransformerModel, mgpu.cu:284-318; seed offsets / bases from the
 * update launch list mgpu.cu:1603-1643 */
struct Layout {
    int64_t embedding, emb_bias, ln_init, ln_init_bias, w_emb_mlp_up, mlp_emb_bias_up,
            w_emb_mlp_down, mlp_emb_bias_down, ln_1, ln_1_bias, w_q, w_k, w_v, w_o,
            ln_2, ln_2_bias, w_up, mlp_bias_up, w_down, mlp_bias_down, ln_f, ln_f_bias, total;
};
static Layout make_layout(const orc_config *c) {
    Layout L; int64_t o = 0; int64_t H = c->hidden, V = c->vocab, NL = c->n_layers;
    L.embedding = o; o += V * H;
    L.emb_bias = o; o += H;
    L.ln_init = o; o += H;
    L.ln_init_bias = o; o += H;
    L.w_emb_mlp_up = o; o += H * 4 * H;
    L.mlp_emb_bias_up = o; o += 4 * H;
    L.w_emb_mlp_down = o; o += 4 * H * H;
    L.mlp_emb_bias_down = o; o += H;
    L.ln_1 = o; o += NL * H;
    L.ln_1_bias = o; o += NL * H;
    L.w_q = o; o += NL * H * H;
    L.w_k = o; o += NL * H * H;
    L.w_v = o; o += NL * H * H;
    L.w_o = o; o += NL * H * H;
    L.ln_2 = o; o += NL * H;
    L.ln_2_bias = o; o += NL * H;
    L.w_up = o; o += NL * H * 4 * H;
    L.mlp_bias_up = o; o += NL * 4 * H;
    L.w_down = o; o += NL * 4 * H * H;
    L.mlp_bias_down = o; o += NL * H;
    L.ln_f = o; o += H;
    L.ln_f_bias = o; o += H;
    L.total = o;
    return L;
}
extern "C" int64_t orc_model_bytes(const orc_config *c) { return make_layout(c).total; }

static void add_t(std::vector<orc_tensor> &v, const char *name, int l, int is_matrix, int rows, int cols,
                  int64_t off, int oa, int ob, int base, float lrs, int muon) {
    orc_tensor t; memset(&t, 0, sizeof(t));
    if (l >= 0) snprintf(t.name, sizeof(t.name), "%s.%d", name, l); else snprintf(t.name, sizeof(t.name), "%s", name);
    t.is_matrix = is_matrix; t.rows = rows; t.cols = cols; t.offset = off; t.off_a = oa; t.off_b = ob;
    t.seed_base = base; t.lr_scale = lrs; t.muon = muon;
    v.push_back(t);
}
/* launch order of mgpu.cu:1603-1643 */
static std::vector<orc_tensor> tensor_table(const orc_config *c) {
    Layout L = make_layout(c); int H = c->hidden, V = c->vocab; std::vector<orc_tensor> v;
    for (int l = 0; l < c->n_layers; l++) {
        int b = l * 1000; int64_t hh = (int64_t)H * H, h4 = (int64_t)H * 4 * H;
        add_t(v, "w_q", l, 1, H, H, L.w_q + l * hh, OFF_Q_A, OFF_Q_B, b, 1.f, 1);
        add_t(v, "w_k", l, 1, H, H, L.w_k + l * hh, OFF_K_A, OFF_K_B, b, 1.f, 1);
        add_t(v, "w_v", l, 1, H, H, L.w_v + l * hh, OFF_V_A, OFF_V_B, b, 1.f, 1);
        add_t(v, "w_o", l, 1, H, H, L.w_o + l * hh, OFF_O_A, OFF_O_B, b, 1.f, 1);
        add_t(v, "w_up", l, 1, H, 4 * H, L.w_up + l * h4, OFF_MLP_UP_A, OFF_MLP_UP_B, b, 1.f, 1);
        add_t(v, "w_down", l, 1, 4 * H, H, L.w_down + l * h4, OFF_MLP_DOWN_A, OFF_MLP_DOWN_B, b, 1.f, 1);
        add_t(v, "ln_1", l, 0, 1, H, L.ln_1 + (int64_t)l * H, OFF_LN_1_A, OFF_LN_1_B, b, 1.f, 0);
        add_t(v, "ln_1_bias", l, 0, 1, H, L.ln_1_bias + (int64_t)l * H, OFF_LN_1_BIAS_A, OFF_LN_1_BIAS_B, b, 1.f, 0);
        add_t(v, "ln_2", l, 0, 1, H, L.ln_2 + (int64_t)l * H, OFF_LN_2_A, OFF_LN_2_B, b, 1.f, 0);
        add_t(v, "ln_2_bias", l, 0, 1, H, L.ln_2_bias + (int64_t)l * H, OFF_LN_2_BIAS_A, OFF_LN_2_BIAS_B, b, 1.f, 0);
        add_t(v, "mlp_bias_up", l, 0, 1, 4 * H, L.mlp_bias_up + (int64_t)l * 4 * H, OFF_MLP_BIAS_UP_A, OFF_MLP_BIAS_UP_B, b, 1.f, 0);
        add_t(v, "mlp_bias_down", l, 0, 1, H, L.mlp_bias_down + (int64_t)l * H, OFF_MLP_BIAS_DOWN_A, OFF_MLP_BIAS_DOWN_B, b, 1.f, 0);
    }
    add_t(v, "ln_f", -1, 0, 1, H, L.ln_f, OFF_LN_F_A, OFF_LN_F_B, 0, 1.f, 0);
    add_t(v, "ln_f_bias", -1, 0, 1, H, L.ln_f_bias, OFF_LN_F_BIAS_A, OFF_LN_F_BIAS_B, 0, 1.f, 0);
    add_t(v, "ln_init", -1, 0, 1, H, L.ln_init, OFF_LN_INIT_A, OFF_LN_INIT_B, 0, 1.f, 0);
    add_t(v, "ln_init_bias", -1, 0, 1, H, L.ln_init_bias, OFF_LN_INIT_BIAS_A, OFF_LN_INIT_BIAS_B, 0, 1.f, 0);
    add_t(v, "w_emb_mlp_up", -1, 1, H, 4 * H, L.w_emb_mlp_up, OFF_EMB_MLP_UP_A, OFF_EMB_MLP_UP_B, 0, 1.f, 1);
    add_t(v, "mlp_emb_bias_up", -1, 0, 1, 4 * H, L.mlp_emb_bias_up, OFF_EMB_MLP_BIAS_UP_A, OFF_EMB_MLP_BIAS_UP_B, 0, 1.f, 0);
    add_t(v, "w_emb_mlp_down", -1, 1, 4 * H, H, L.w_emb_mlp_down, OFF_EMB_MLP_DOWN_A, OFF_EMB_MLP_DOWN_B, 0, 1.f, 1);
    add_t(v, "mlp_emb_bias_down", -1, 0, 1, H, L.mlp_emb_bias_down, OFF_EMB_MLP_BIAS_DOWN_A, OFF_EMB_MLP_BIAS_DOWN_B, 0, 1.f, 0);
    add_t(v, "emb_bias", -1, 0, 1, H, L.emb_bias, OFF_EMB_BIAS_A, OFF_EMB_BIAS_B, 0, 0.1f, 0);
    add_t(v, "embedding", -1, 1, H, V, L.embedding, OFF_EMB, OFF_EMB + H, 0, 1.f, 0);
    return v;
}
extern "C" int orc_tensor_table(const orc_config *c, orc_tensor *out, int max_out) {
    std::vector<orc_tensor> v = tensor_table(c);
    int n = (int)v.size();
    for (int i = 0; i < n && i < max_out; i++) out[i] = v[i];
    return n;
}

/* Ternary-packed matrix weights (no reference counterpart; the self-consistent statement the GPU path is checked
 * against): tensors in the order of their offsets in the model blob; a vector tensor is copied; a matrix tensor takes
 * one byte per four consecutive blob elements, element e in bits 2e+1..2e as a 2-bit two's complement number. */
static std::vector<orc_tensor> tensors_by_offset(const orc_config *c) {
    std::vector<orc_tensor> v = tensor_table(c);
    for (size_t i = 1; i < v.size(); i++)
        for (size_t j = i; j > 0 && v[j - 1].offset > v[j].offset; j--) { orc_tensor t = v[j]; v[j] = v[j - 1]; v[j - 1] = t; }
    return v;
}
extern "C" int64_t orc_ternary_model_bytes(const orc_config *c) {
    int64_t n = 0;
    for (const orc_tensor &t : tensor_table(c)) n += t.is_matrix ? (int64_t)t.rows * t.cols / 4 : t.cols;
    return n;
}
extern "C" int orc_ternary_model_pack(const orc_config *c, const int8_t *model, uint8_t *packed) {
    int64_t po = 0; int bad = 0;
    for (const orc_tensor &t : tensors_by_offset(c)) {
        if (!t.is_matrix) { memcpy(packed + po, model + t.offset, t.cols); po += t.cols; continue; }
        for (int64_t i = 0; i < (int64_t)t.rows * t.cols; i += 4) {
            int b = 0;
            for (int e = 0; e < 4; e++) {
                int v = model[t.offset + i + e];
                if (v < -1 || v > 1) bad = 1;
                b |= (v & 3) << (2 * e);
            }
            packed[po++] = (uint8_t)b;
        }
    }
    return bad ? -1 : 0;
}
extern "C" void orc_ternary_model_unpack(const orc_config *c, const uint8_t *packed, int8_t *model) {
    int64_t po = 0;
    for (const orc_tensor &t : tensors_by_offset(c)) {
        if (!t.is_matrix) { memcpy(model + t.offset, packed + po, t.cols); po += t.cols; continue; }
        for (int64_t i = 0; i < (int64_t)t.rows * t.cols; i += 4) {
            int b = packed[po++];
            for (int e = 0; e < 4; e++) {
                int f = (b >> (2 * e)) & 3;
                model[t.offset + i + e] = (int8_t)(f >= 2 ? f - 4 : f);
            }
        }
    }
}

/* mgpu.cu:443-459: src is [In=rows][Out=cols]; dst word (k/4)*cols + n holds bytes k..k+3 */
extern "C" void orc_repack(int8_t *dst, const int8_t *src, int rows, int cols) {
    for (int k = 0; k < rows; k += 4)
        for (int n = 0; n < cols; n++)
            for (int s = 0; s < 4; s++)
                dst[(((int64_t)(k / 4) * cols) + n) * 4 + s] = src[(int64_t)(k + s) * cols + n];
}
extern "C" void orc_unpack(int8_t *dst, const int8_t *src, int rows, int cols) {
    for (int k = 0; k < rows; k++)
        for (int n = 0; n < cols; n++)
            dst[(int64_t)k * cols + n] = src[(((int64_t)(k / 4) * cols) + n) * 4 + (k & 3)];
}

/* mgpu.cu:461-519 */
extern "C" void orc_init_model(const orc_config *c, int8_t *model, uint32_t seed) {
    Layout L = make_layout(c); int H = c->hidden, V = c->vocab; uint32_t rng = seed;
    memset(model, 0, (size_t)L.total);
    std::vector<int8_t> tmp((size_t)H * 4 * H > (size_t)V * H ? (size_t)H * 4 * H : (size_t)V * H);
    auto fill = [&](int64_t n) { for (int64_t i = 0; i < n; i++) tmp[i] = orc_gen_noise_host(&rng, host_mask_word(c)); };
    fill((int64_t)V * H); orc_repack(model + L.embedding, tmp.data(), H, V);
    for (int i = 0; i < H; i++) { model[L.ln_init + i] = 16; }
    fill((int64_t)H * 4 * H); orc_repack(model + L.w_emb_mlp_up, tmp.data(), H, 4 * H);
    fill((int64_t)H * 4 * H); orc_repack(model + L.w_emb_mlp_down, tmp.data(), 4 * H, H);
    for (int l = 0; l < c->n_layers; l++) {
        for (int i = 0; i < H; i++) { model[L.ln_1 + (int64_t)l * H + i] = 16; model[L.ln_2 + (int64_t)l * H + i] = 16; }
        int64_t hh = (int64_t)H * H, h4 = (int64_t)H * 4 * H;
        fill(hh); orc_repack(model + L.w_q + l * hh, tmp.data(), H, H);
        fill(hh); orc_repack(model + L.w_k + l * hh, tmp.data(), H, H);
        fill(hh); orc_repack(model + L.w_v + l * hh, tmp.data(), H, H);
        fill(hh); orc_repack(model + L.w_o + l * hh, tmp.data(), H, H);
        fill(h4); orc_repack(model + L.w_up + l * h4, tmp.data(), H, 4 * H);
        fill(h4); orc_repack(model + L.w_down + l * h4, tmp.data(), 4 * H, H);
    }
    for (int i = 0; i < H; i++) model[L.ln_f + i] = 16;
}

/* ------------------------------------------------------------------ forward pieces */
static inline int8_t blk(const int8_t *Wb, int cols, int k, int n) {   /* logical W[k][n] of a blocked matrix */
    return Wb[(((int64_t)(k >> 2) * cols) + n) * 4 + (k & 3)];
}

/* d-eggs adaptive noise overlay, de/include/model/layers.cuh:12-53 (ADAPTIVE_NOISE_MODE 1, the default of
 * de/include/config.h:229-231): the int8 overlay value of a row / column / vector element becomes a float factor
 * that multiplies the noise before it is truncated to an integer.  A null overlay pointer is the reference without
 * the overlay (factor 1).  The overlay blob has the layout of the model blob: a vector tensor's values sit at the
 * tensor's offset; a matrix has its `rows` input-dimension values at its offset and its `cols` output-dimension
 * values right behind them. */
extern "C" float orc_adaptive_factor(int ov) {
    if (ov < 0) return 0.0f;
    if (ov < 64) return (float)ov / 64.0f;
    return 1.0f;
}
static inline float afac(const int8_t *sc, int64_t i) { return sc ? orc_adaptive_factor(sc[i]) : 1.0f; }
/* the overlay values that belong to the tensor stored at `tensor` inside the blob starting at `model` */
static inline const int8_t *sc_of(const int8_t *sc, const int8_t *model, const int8_t *tensor) {
    return sc ? sc + (tensor - model) : NULL;
}

/* mgpu.cu:553-572: dp4a accumulation over the packed input, then the rank-1 term; with the overlay the noise is
 * scaled by the output column's factor and truncated, de/include/model/layers.cuh:76-97 */
static int32_t linear_proj(const orc_config *c, const int8_t *in, const int8_t *Wb, int K, int N, int n,
                           int32_t sb, uint32_t noise_seed, int ns, const int8_t *sc_col = NULL) {
    int32_t acc = 0;
    for (int k = 0; k < K; k++) acc += (int32_t)in[k] * (int32_t)blk(Wb, N, k, n);
    if (ns != 0) {
        int8_t nz = orc_noise(noise_seed, (uint32_t)n, dev_mask(c));
        int32_t a = sc_col ? (int32_t)(nz * afac(sc_col, n)) : (int32_t)nz;
        acc += ((sb * a) * ns) >> (c->fixed_point + c->sigma_shift);
    }
    return acc;
}
/* x . B with the input-dimension factors: each term is converted to int after the float multiply, as the argument
 * of the reference's block reduction is (de/include/model/layers.cuh:240, :340-342, :436) */
static int32_t noise_dot(const orc_config *c, const int8_t *in, int K, uint32_t seed, const int8_t *sc_row) {
    int32_t sb = 0;
    for (int k = 0; k < K; k++) {
        int32_t t = (int32_t)in[k] * orc_noise(seed, k, dev_mask(c));
        sb += sc_row ? (int32_t)(t * afac(sc_row, k)) : t;
    }
    return sb;
}

/* mgpu.cu:646-678 */
/* the two input-side sums of an MLP block under the overlay, exported so that tests can pin them in isolation */
extern "C" int32_t orc_noise_dot_adaptive(const orc_config *c, const int8_t *in, int K, uint32_t seed, const int8_t *overlay_rows) {
    return noise_dot(c, in, K, seed, overlay_rows);
}
extern "C" int32_t orc_scaled_noise(int noise, int overlay_value) { return (int32_t)((int8_t)noise * orc_adaptive_factor(overlay_value)); }

static void standard_norm(const orc_config *c, const int8_t *x, const int8_t *w, const int8_t *b, int H,
                          uint32_t seed_base, int off_w_a, int off_w_b, int off_b_a, int off_b_b,
                          int ns, int8_t *out, const int8_t *sc_w, const int8_t *sc_b) {
    int32_t tot = 0;
    for (int i = 0; i < H; i++) tot += abs((int32_t)x[i]);
    int32_t mn = tot / H; if (!mn) mn = 1;
    std::vector<int8_t> res(H);
    for (int tid = 0; tid < H; tid++) {
        int32_t w_mod = w[tid], b_mod = b[tid];
        if (ns != 0) {
            int8_t wn1 = orc_noise(seed_base + off_w_a, tid, dev_mask(c));
            int8_t wn2 = orc_noise(seed_base + off_w_b, tid, dev_mask(c));
            /* with the overlay: (AccumType)(wn1 * wn2 * scale_w), de/include/model/layers.cuh:171-183 */
            int32_t wp = (int32_t)wn1 * wn2; if (sc_w) wp = (int32_t)(wp * afac(sc_w, tid));
            w_mod += (wp * ns) >> c->sigma_shift_vector;
            int8_t bn1 = orc_noise(seed_base + off_b_a, tid, dev_mask(c));
            int8_t bn2 = orc_noise(seed_base + off_b_b, tid, dev_mask(c));
            int32_t bp = (int32_t)bn1 * bn2; if (sc_b) bp = (int32_t)(bp * afac(sc_b, tid));
            b_mod += (bp * ns) >> c->sigma_shift_vector;
        }
        res[tid] = orc_clip(((int32_t)x[tid] * w_mod) / mn + b_mod);
    }
    memcpy(out, res.data(), H);
}
extern "C" void orc_standard_norm(const orc_config *c, const int8_t *x, const int8_t *w, const int8_t *b, int H,
                                  uint32_t seed_base, int off_w_a, int off_w_b, int off_b_a, int off_b_b,
                                  int ns, int8_t *out) {
    standard_norm(c, x, w, b, H, seed_base, off_w_a, off_w_b, off_b_a, off_b_b, ns, out, NULL, NULL);
}

/* norm.h:10-103 (both templates have the same body) */
extern "C" void orc_adaptive_normalize(const int32_t *val, int n, int8_t *out) {
    int32_t layer_max = 0;
    for (int i = 0; i < n; i++) { int32_t a = abs(val[i]); if (a > layer_max) layer_max = a; }
    float scale = 127.0f / (float)(layer_max + 1e-9f);
    for (int i = 0; i < n; i++) {
        float scaled_f = (float)val[i] * scale;
        int32_t scaled = (int32_t)roundf(scaled_f);
        if (scaled > 127) scaled = 127;
        if (scaled < -127) scaled = -127;
        out[i] = (int8_t)scaled;
    }
}

/* mgpu.cu:624-644 */
extern "C" void orc_rope(const orc_config *c, const int32_t *rope_lut, const int32_t *val, int t, int H, int32_t *out) {
    int HD = c->head_dim;
    for (int tid = 0; tid < H; tid++) {
        int hd = tid % HD, pair = hd / 2, is_odd = hd % 2;
        int32_t cs = rope_lut[t * HD + pair * 2], sn = rope_lut[t * HD + pair * 2 + 1];
        int32_t nb = val[tid ^ 1];
        int64_t half = (int64_t)1 << (c->rope_scale_bit - 1);
        int64_t res;
        if (!is_odd) res = ((int64_t)val[tid] * cs - (int64_t)nb * sn + half) >> c->rope_scale_bit;
        else         res = ((int64_t)nb * sn + (int64_t)val[tid] * cs + half) >> c->rope_scale_bit;
        out[tid] = (int32_t)res;
    }
}

static inline int32_t exp_lookup(const int32_t *exp_lut, int32_t diff) {   /* mgpu.cu:543-547 */
    int index = -diff; index = (index < 0) ? 0 : ((index > 255) ? 255 : index);
    return exp_lut[index];
}

/* mgpu.cu:787-824 : q is the normalised query of token t, kc / vc hold rows 0..t */
extern "C" void orc_attention_core(const orc_config *c, const int32_t *exp_lut, const int8_t *q,
                                   const int8_t *kc, const int8_t *vc, int t, int H, int8_t *ao) {
    int HD = c->head_dim, NH = H / HD;
    std::vector<int32_t> hmax(NH, INT_MIN);
    std::vector<int32_t> score((size_t)NH * (t + 1));
    for (int ctx = 0; ctx <= t; ctx++)
        for (int h = 0; h < NH; h++) {
            int32_t s = 0;
            for (int d = 0; d < HD; d++) s += (int32_t)q[h * HD + d] * (int32_t)kc[(int64_t)ctx * H + h * HD + d];
            score[(size_t)ctx * NH + h] = s;
            if (s > hmax[h]) hmax[h] = s;
        }
    for (int tid = 0; tid < H; tid++) {
        int h = tid / HD; int64_t w_v_sum = 0; uint64_t tot_sc = 0;
        for (int ctx = 0; ctx <= t; ctx++) {
            int32_t wt = exp_lookup(exp_lut, (score[(size_t)ctx * NH + h] >> c->shift_attn) - (hmax[h] >> c->shift_attn));
            w_v_sum += (int64_t)wt * vc[(int64_t)ctx * H + tid]; tot_sc += (uint64_t)wt;
        }
        int64_t r = w_v_sum / (tot_sc ? (int64_t)tot_sc : 1);
        ao[tid] = (r > 127) ? 127 : ((r < -127) ? -127 : (int8_t)r);   /* clip() takes int32; |r| <= 127 anyway */
    }
}

/* mgpu.cu:969-1023 : logits are already >> shift_logit */
extern "C" int64_t orc_token_loss(const orc_config *c, const int32_t *exp_lut, const int32_t *logits, int V, int target) {
    int32_t gmax = INT_MIN;
    for (int v = 0; v < V; v++) if (logits[v] > gmax) gmax = logits[v];
    int64_t sum_ex = 0;
    for (int v = 0; v < V; v++) sum_ex += exp_lookup(exp_lut, logits[v] - gmax);
    int64_t log_sum = 0;
    if (sum_ex > 0) {
        uint64_t x = (uint64_t)sum_ex; int pos = 0;
        while (x >= 256) { x >>= 8; pos += 8; }
        if (x >= 16) { x >>= 4; pos += 4; }
        if (x >= 4) { x >>= 2; pos += 2; }
        if (x >= 2) { pos += 1; }
        log_sum = ((int64_t)pos << 4) - ((int64_t)c->softmax_scale_bit << 4);
    }
    return (log_sum >> 1) + gmax - logits[target];
}

struct MlpCfg { int ln_a, ln_b, lnb_a, lnb_b, up_a, up_b, bup_a, bup_b, dn_a, dn_b, bdn_a, bdn_b; };
static const MlpCfg CFG_INIT = { OFF_LN_INIT_A, OFF_LN_INIT_B, OFF_LN_INIT_BIAS_A, OFF_LN_INIT_BIAS_B,
    OFF_EMB_MLP_UP_A, OFF_EMB_MLP_UP_B, OFF_EMB_MLP_BIAS_UP_A, OFF_EMB_MLP_BIAS_UP_B,
    OFF_EMB_MLP_DOWN_A, OFF_EMB_MLP_DOWN_B, OFF_EMB_MLP_BIAS_DOWN_A, OFF_EMB_MLP_BIAS_DOWN_B };   /* mgpu.cu:689-697 */
static const MlpCfg CFG_LAYER = { OFF_LN_2_A, OFF_LN_2_B, OFF_LN_2_BIAS_A, OFF_LN_2_BIAS_B,
    OFF_MLP_UP_A, OFF_MLP_UP_B, OFF_MLP_BIAS_UP_A, OFF_MLP_BIAS_UP_B,
    OFF_MLP_DOWN_A, OFF_MLP_DOWN_B, OFF_MLP_BIAS_DOWN_A, OFF_MLP_BIAS_DOWN_B };                   /* mgpu.cu:698-706 */

/* x . B of the down projection (depth 4H).  Under the overlay the reference thread of hidden unit tid adds its four
 * terms into an int with `pb += int * int8 * float`, i.e. pb = (int)((float)pb + term) each time
 * (de/include/model/layers.cuh:268-276); the threads' sums are then added as integers. */
extern "C" int32_t orc_down_dot_adaptive(const orc_config *c, const int8_t *mlp, int H, uint32_t seed, const int8_t *overlay_rows) {
    if (!overlay_rows) return noise_dot(c, mlp, 4 * H, seed, NULL);
    int32_t sb = 0;
    for (int tid = 0; tid < H; tid++) {
        int32_t pb = 0;
        for (int sub = 0; sub < 4; sub++) {
            int k = tid + sub * H;
            pb += (int32_t)mlp[k] * orc_noise(seed, k, dev_mask(c)) * afac(overlay_rows, k);
        }
        sb += pb;
    }
    return sb;
}

/* mgpu.cu:708-759; overlay sites de/include/model/layers.cuh:215-296 */
static void mlp_block(const orc_config *c, const int8_t *act_lut, int8_t *x,
                      const int8_t *ln_w, const int8_t *ln_b, const int8_t *up_w, const int8_t *up_b,
                      const int8_t *dn_w, const int8_t *dn_b, uint32_t seed_base, int ns, const MlpCfg &cfg,
                      const int8_t *model = NULL, const int8_t *sc = NULL) {
    int H = c->hidden, H4 = 4 * H, M = dev_mask(c);
    const int8_t *s_lnw = sc_of(sc, model, ln_w), *s_lnb = sc_of(sc, model, ln_b);
    const int8_t *s_up = sc_of(sc, model, up_w), *s_bup = sc_of(sc, model, up_b);     /* up: rows H then cols 4H */
    const int8_t *s_dn = sc_of(sc, model, dn_w), *s_bdn = sc_of(sc, model, dn_b);     /* down: rows 4H then cols H */
    std::vector<int8_t> nrm(H), mlp(H4);
    standard_norm(c, x, ln_w, ln_b, H, seed_base, cfg.ln_a, cfg.ln_b, cfg.lnb_a, cfg.lnb_b, ns, nrm.data(), s_lnw, s_lnb);
    int32_t sb = noise_dot(c, nrm.data(), H, seed_base + cfg.up_b, s_up);
    for (int o = 0; o < H4; o++) {
        int32_t a = linear_proj(c, nrm.data(), up_w, H, H4, o, sb, seed_base + cfg.up_a, ns, s_up ? s_up + H : NULL);
        int8_t nb1 = orc_noise(seed_base + cfg.bup_a, o, M), nb2 = orc_noise(seed_base + cfg.bup_b, o, M);
        int32_t np = (int32_t)nb1 * nb2; if (s_bup) np = (int32_t)(np * afac(s_bup, o));
        int32_t nv = (np * ns) >> c->sigma_shift_vector;
        mlp[o] = act_lut[(uint8_t)orc_clip((a >> c->shift_mlp_up) + up_b[o] + nv)];
    }
    sb = orc_down_dot_adaptive(c, mlp.data(), H, seed_base + cfg.dn_b, s_dn);
    std::vector<int32_t> pre(H);
    for (int tid = 0; tid < H; tid++) {
        int32_t adn = linear_proj(c, mlp.data(), dn_w, H4, H, tid, sb, seed_base + cfg.dn_a, ns, s_dn ? s_dn + H4 : NULL);
        int8_t n1 = orc_noise(seed_base + cfg.bdn_a, tid, M), n2 = orc_noise(seed_base + cfg.bdn_b, tid, M);
        int32_t np = (int32_t)n1 * n2; if (s_bdn) np = (int32_t)(np * afac(s_bdn, tid));
        int32_t nv = (np * ns) >> c->sigma_shift_vector;
        pre[tid] = (int32_t)x[tid] + (adn >> c->shift_mlp_down) + dn_b[tid] + nv;
    }
    orc_adaptive_normalize(pre.data(), H, x);
}

struct Tables { std::vector<int32_t> exp_lut, rope; std::vector<int8_t> act; };
static Tables make_tables(const orc_config *c) {
    Tables t; t.exp_lut.resize(256); t.act.resize(256); t.rope.resize((size_t)c->seq_len * c->head_dim);
    orc_tables(c, t.exp_lut.data(), t.act.data(), t.rope.data());
    return t;
}

/* token i of the stream: bytes for the byte-level model; d-eggs' TokenType is uint32 for any other VOCAB_SIZE
 * (de/include/config.h:22-28), and `data` then points at uint32 tokens, data_len counting tokens */
static inline int tok_at(const orc_config *c, const uint8_t *data, int64_t i) {
    return c->vocab > 256 ? (int)reinterpret_cast<const uint32_t *>(data)[i] : (int)data[i];
}

/* mgpu.cu:847-1029 (one block == one member) */
static int32_t forward_member(const orc_config *c, const Tables &tb, const int8_t *model,
                              const uint8_t *data, int64_t data_len, int64_t start_idx,
                              uint32_t step_seed, int p_idx, int ns_override, orc_trace *tr,
                              const int8_t *sc = NULL) {
    const int H = c->hidden, V = c->vocab, T = c->seq_len, NL = c->n_layers, M = dev_mask(c);
    Layout L = make_layout(c);
    int64_t pair_idx = p_idx / 2;
    int64_t stride = data_len / (c->population / 2);
    int64_t stream_pos = (c->use_same_data ? start_idx : start_idx + pair_idx * stride) % (data_len - T);   /* mgpu.cu:866-870 */
    int ns = (p_idx % 2 == 0) ? 1 : -1;
    if (ns_override != 2) ns = ns_override;
    uint32_t pair_seed = step_seed + (uint32_t)pair_idx;
    std::vector<int8_t> kv((size_t)NL * 2 * T * H);
    std::vector<int8_t> x(H), nrm(H), qv(H), ao(H), nf(H);
    std::vector<int32_t> aq(H), ak(H), av(H), tmp(H), logits(V);
    int64_t my_loss = 0;
    const int sigma = c->fixed_point + c->sigma_shift;

    for (int t = 0; t < T; t++) {
        /* 1. embedding, mgpu.cu:901-931 */
        int tok = tok_at(c, data, stream_pos + t);
        uint32_t seed_emb = pair_seed + OFF_EMB;
        for (int tid = 0; tid < H; tid++) {
            int8_t emb = blk(model + L.embedding, V, tid, tok);
            int8_t ebias = model[L.emb_bias + tid];
            int8_t n1 = orc_noise(pair_seed + OFF_EMB_BIAS_A, tid, M), n2 = orc_noise(pair_seed + OFF_EMB_BIAS_B, tid, M);
            /* overlay: de/src/kernels.cu:139-158; the embedding is a matrix [H rows][V cols] in the blob, so its
             * per-hidden values come first and its per-token values follow */
            int32_t cp = (int32_t)n1 * n2; if (sc) cp = (int32_t)(cp * afac(sc + L.emb_bias, tid));
            int32_t chk = (cp * ns) >> c->sigma_shift_vector;
            int8_t a_tok = orc_noise(seed_emb, tok, M), b_dim = orc_noise(seed_emb + H, tid, M);
            int32_t pp = (int32_t)a_tok * b_dim;
            if (sc) pp = (int32_t)(pp * afac(sc + L.embedding + H, tok) * afac(sc + L.embedding, tid));
            int32_t perturb = (pp * ns) >> sigma;
            x[tid] = orc_clip((int32_t)emb + ebias + chk + perturb);
        }
        if (tr && tr->x_emb) memcpy(tr->x_emb + (size_t)t * H, x.data(), H);

        mlp_block(c, tb.act.data(), x.data(), model + L.ln_init, model + L.ln_init_bias,
                  model + L.w_emb_mlp_up, model + L.mlp_emb_bias_up, model + L.w_emb_mlp_down,
                  model + L.mlp_emb_bias_down, pair_seed, ns, CFG_INIT, model, sc);
        if (tr && tr->x_init) memcpy(tr->x_init + (size_t)t * H, x.data(), H);

        /* 2. layer stack, mgpu.cu:937-952 */
        for (int l = 0; l < NL; l++) {
            uint32_t sbase = pair_seed + (uint32_t)(l * 1000);
            int8_t *lk = kv.data() + (size_t)l * 2 * T * H, *lv = lk + (size_t)T * H;
            const int8_t *wq = model + L.w_q + (int64_t)l * H * H, *wk = model + L.w_k + (int64_t)l * H * H;
            const int8_t *wv = model + L.w_v + (int64_t)l * H * H, *wo = model + L.w_o + (int64_t)l * H * H;
            /* attention, mgpu.cu:761-833 */
            /* overlay sites of the attention block: de/include/model/layers.cuh:313-351, :432-438 */
            const int8_t *s_q = sc_of(sc, model, wq), *s_k = sc_of(sc, model, wk), *s_v = sc_of(sc, model, wv), *s_o = sc_of(sc, model, wo);
            standard_norm(c, x.data(), model + L.ln_1 + (int64_t)l * H, model + L.ln_1_bias + (int64_t)l * H, H,
                          sbase, OFF_LN_1_A, OFF_LN_1_B, OFF_LN_1_BIAS_A, OFF_LN_1_BIAS_B, ns, nrm.data(),
                          sc ? sc + L.ln_1 + (int64_t)l * H : NULL, sc ? sc + L.ln_1_bias + (int64_t)l * H : NULL);
            int32_t sbq = noise_dot(c, nrm.data(), H, sbase + OFF_Q_B, s_q);
            int32_t sbk = noise_dot(c, nrm.data(), H, sbase + OFF_K_B, s_k);
            int32_t sbv = noise_dot(c, nrm.data(), H, sbase + OFF_V_B, s_v);
            for (int tid = 0; tid < H; tid++) {
                aq[tid] = linear_proj(c, nrm.data(), wq, H, H, tid, sbq, sbase + OFF_Q_A, ns, s_q ? s_q + H : NULL);
                ak[tid] = linear_proj(c, nrm.data(), wk, H, H, tid, sbk, sbase + OFF_K_A, ns, s_k ? s_k + H : NULL);
                av[tid] = linear_proj(c, nrm.data(), wv, H, H, tid, sbv, sbase + OFF_V_A, ns, s_v ? s_v + H : NULL);
            }
            orc_rope(c, tb.rope.data(), aq.data(), t, H, tmp.data());
            orc_adaptive_normalize(tmp.data(), H, qv.data());
            orc_rope(c, tb.rope.data(), ak.data(), t, H, tmp.data());
            orc_adaptive_normalize(tmp.data(), H, lk + (size_t)t * H);
            orc_adaptive_normalize(av.data(), H, lv + (size_t)t * H);
            if (tr && tr->q) memcpy(tr->q + ((size_t)l * T + t) * H, qv.data(), H);
            if (tr && tr->k) memcpy(tr->k + ((size_t)l * T + t) * H, lk + (size_t)t * H, H);
            if (tr && tr->v) memcpy(tr->v + ((size_t)l * T + t) * H, lv + (size_t)t * H, H);

            orc_attention_core(c, tb.exp_lut.data(), qv.data(), lk, lv, t, H, ao.data());
            if (tr && tr->ao) memcpy(tr->ao + ((size_t)l * T + t) * H, ao.data(), H);

            int32_t sb = noise_dot(c, ao.data(), H, sbase + OFF_O_B, s_o);
            for (int tid = 0; tid < H; tid++) {
                int32_t aco = linear_proj(c, ao.data(), wo, H, H, tid, sb, sbase + OFF_O_A, ns, s_o ? s_o + H : NULL);
                tmp[tid] = (int32_t)x[tid] + (aco >> c->shift_out);
            }
            orc_adaptive_normalize(tmp.data(), H, x.data());
            if (tr && tr->x_attn) memcpy(tr->x_attn + ((size_t)l * T + t) * H, x.data(), H);

            mlp_block(c, tb.act.data(), x.data(), model + L.ln_2 + (int64_t)l * H, model + L.ln_2_bias + (int64_t)l * H,
                      model + L.w_up + (int64_t)l * H * 4 * H, model + L.mlp_bias_up + (int64_t)l * 4 * H,
                      model + L.w_down + (int64_t)l * 4 * H * H, model + L.mlp_bias_down + (int64_t)l * H,
                      sbase, ns, CFG_LAYER, model, sc);
            if (tr && tr->x_mlp) memcpy(tr->x_mlp + ((size_t)l * T + t) * H, x.data(), H);
        }

        /* 3. head + loss, mgpu.cu:955-1024 */
        /* overlay: the tied head takes the embedding's per-hidden values on its input side and the per-token values
         * on its output side, de/src/kernels.cu:200-240 */
        standard_norm(c, x.data(), model + L.ln_f, model + L.ln_f_bias, H, pair_seed,
                      OFF_LN_F_A, OFF_LN_F_B, OFF_LN_F_BIAS_A, OFF_LN_F_BIAS_B, ns, nf.data(),
                      sc ? sc + L.ln_f : NULL, sc ? sc + L.ln_f_bias : NULL);
        if (tr && tr->nf) memcpy(tr->nf + (size_t)t * H, nf.data(), H);
        int32_t sbh = noise_dot(c, nf.data(), H, pair_seed + OFF_EMB + H, sc ? sc + L.embedding : NULL);
        for (int v = 0; v < V; v++) {
            int32_t ah = linear_proj(c, nf.data(), model + L.embedding, H, V, v, sbh, pair_seed + OFF_EMB, ns,
                                     sc ? sc + L.embedding + H : NULL);
            logits[v] = ah >> c->shift_logit;
        }
        if (tr && tr->logits) memcpy(tr->logits + (size_t)t * V, logits.data(), sizeof(int32_t) * V);
        int target = tok_at(c, data, stream_pos + t + 1);
        int64_t lt = orc_token_loss(c, tb.exp_lut.data(), logits.data(), V, target);
        if (tr && tr->loss_t) tr->loss_t[t] = lt;
        my_loss += lt;
    }
    return (int32_t)my_loss;
}

extern "C" int32_t orc_forward_member(const orc_config *c, const int8_t *model, const uint8_t *data, int64_t data_len,
                                      int64_t start_idx, uint32_t step_seed, int p_idx, int ns_override, orc_trace *trace) {
    Tables tb = make_tables(c);
    return forward_member(c, tb, model, data, data_len, start_idx, step_seed, p_idx, ns_override, trace);
}

extern "C" int32_t orc_forward_member_adaptive(const orc_config *c, const int8_t *model, const int8_t *overlay,
                                               const uint8_t *data, int64_t data_len, int64_t start_idx,
                                               uint32_t step_seed, int p_idx, int ns_override, orc_trace *trace) {
    Tables tb = make_tables(c);
    return forward_member(c, tb, model, data, data_len, start_idx, step_seed, p_idx, ns_override, trace, overlay);
}
extern "C" void orc_population_forward_adaptive(const orc_config *c, const int8_t *model, const int8_t *overlay,
                                                const uint8_t *data, int64_t data_len, int64_t start_idx,
                                                uint32_t step_seed, int pop_offset, int count, int32_t *loss) {
    Tables tb = make_tables(c);
#pragma omp parallel for schedule(dynamic, 1)
    for (int i = 0; i < count; i++) {
        int p = pop_offset + i;
        if (p >= c->population) continue;
        loss[p] = forward_member(c, tb, model, data, data_len, start_idx, step_seed, p, 2, NULL, overlay);
    }
}

extern "C" void orc_population_forward(const orc_config *c, const int8_t *model, const uint8_t *data, int64_t data_len,
                                       int64_t start_idx, uint32_t step_seed, int pop_offset, int count, int32_t *loss) {
    Tables tb = make_tables(c);
#pragma omp parallel for schedule(dynamic, 1)
    for (int i = 0; i < count; i++) {
        int p = pop_offset + i;
        if (p >= c->population) continue;
        loss[p] = forward_member(c, tb, model, data, data_len, start_idx, step_seed, p, 2, NULL);
    }
}

/* mgpu.cu:553-572 applied to a [rows][K] activation matrix */
extern "C" void orc_perturbed_linear(const orc_config *c, const int8_t *X, const int8_t *Wb, int64_t n_rows, int T,
                                     int K, int N, uint32_t seed, int off_a, int off_b, int shift, int32_t *Y) {
    std::vector<int8_t> W((size_t)K * N);
    orc_unpack(W.data(), Wb, K, N);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < n_rows; r++) {
        int64_t member = r / T; uint32_t ps = seed + (uint32_t)(member / 2); int ns = (member % 2 == 0) ? 1 : -1;
        const int8_t *x = X + r * K;
        int32_t sb = 0;
        for (int k = 0; k < K; k++) sb += (int32_t)x[k] * orc_noise(ps + off_b, k, dev_mask(c));
        std::vector<int32_t> acc(N, 0);
        for (int k = 0; k < K; k++) { int32_t xv = x[k]; const int8_t *wr = &W[(size_t)k * N]; for (int n = 0; n < N; n++) acc[n] += xv * wr[n]; }
        for (int n = 0; n < N; n++) {
            int32_t a = acc[n] + (((sb * (int32_t)orc_noise(ps + off_a, n, dev_mask(c))) * ns) >> (c->fixed_point + c->sigma_shift));
            Y[r * N + n] = a >> shift;
        }
    }
}

/* ------------------------------------------------------------------ fitness */
/* mgpu.cu:1305-1311 */
extern "C" void orc_fitness(const int32_t *loss, int32_t *fit, int pairs) {
    for (int i = 0; i < pairs; i++) { int32_t p = loss[2 * i], n = loss[2 * i + 1]; fit[i] = (p < n) ? 1 : ((n < p) ? -1 : 0); }
}

/* ------------------------------------------------------------------ AdamW + votes */
/* mgpu.cu:1040-1064 */
static void adam_apply_limit(const orc_config *c, orc_adam_param *p, int8_t *w, float g, float lr, int *change, int limit);
extern "C" void orc_adam_apply(const orc_config *c, orc_adam_param *p, int8_t *w, float g, float lr, int *change) {
    adam_apply_limit(c, p, w, g, lr, change, 127);
}
static void adam_apply_limit(const orc_config *c, orc_adam_param *p, int8_t *w, float g, float lr, int *change, int limit) {
    float b1 = c->adam_beta1, b2 = c->adam_beta2;
    float t1 = b1 * p->m; float t2 = (1.0f - b1) * g; p->m = t1 + t2;
    float t3 = b2 * p->v; float gg = g * g; float t4 = (1.0f - b2) * gg; p->v = t3 + t4;
    float den = sqrtf(p->v) + c->adam_eps;
    float q = p->m / den;
    float wdw = c->adam_weight_decay * (float)(*w);
    float step = (-lr) * (q + wdw);
    p->acc += step;
    if (p->acc >= 1.0f) {
        if (*w < limit) { (*w)++; *change = 1; p->acc -= 1.0f; } else p->acc = 1.0f;
    } else if (p->acc <= -1.0f) {
        if (*w > -limit) { (*w)--; *change = 1; p->acc += 1.0f; } else p->acc = -1.0f;
    }
}

/* mgpu.cu:1085-1098 : votes in blocked element order */
extern "C" int64_t orc_matrix_votes(const orc_config *c, int rows, int cols, int off_a, int off_b, int seed_base,
                                    const int32_t *fit, int pairs, uint32_t step_seed, int32_t *votes) {
    int64_t n = (int64_t)rows * cols;
    /* noise panels first: identical values, (rows+cols)*pairs hashes instead of 2*rows*cols*pairs */
    std::vector<int8_t> A((size_t)pairs * cols), B((size_t)pairs * rows);
#pragma omp parallel for schedule(static)
    for (int p = 0; p < pairs; p++) {
        uint32_t s = step_seed + (uint32_t)p + (uint32_t)seed_base;
        for (int n2 = 0; n2 < cols; n2++) A[(size_t)p * cols + n2] = orc_noise(s + off_a, n2, dev_mask(c));
        for (int k = 0; k < rows; k++) B[(size_t)p * rows + k] = orc_noise(s + off_b, k, dev_mask(c));
    }
#pragma omp parallel for schedule(static)
    for (int64_t idx = 0; idx < n; idx++) {
        int byte_off = idx & 3; int64_t word = idx >> 2; int tid = (int)(word % cols); int k = (int)(word / cols) * 4 + byte_off;
        int32_t vote = 0;
        for (int p = 0; p < pairs; p++) {
            int f = fit[p]; if (f == 0) continue;
            vote += f * (int32_t)A[(size_t)p * cols + tid] * (int32_t)B[(size_t)p * rows + k];
        }
        votes[idx] = vote;
    }
    return n;
}

/* mgpu.cu:1067-1111 */
extern "C" uint64_t orc_update_matrix_adam(const orc_config *c, int8_t *W, orc_adam_param *st, int rows, int cols,
                                           int off_a, int off_b, int seed_base, const int32_t *fit, int pairs,
                                           uint32_t step_seed, float lr) {
    int64_t n = (int64_t)rows * cols; std::vector<int32_t> votes((size_t)n);
    orc_matrix_votes(c, rows, cols, off_a, off_b, seed_base, fit, pairs, step_seed, votes.data());
    uint64_t changes = 0;
    for (int64_t idx = 0; idx < n; idx++) {
        int change = 0;
        adam_apply_limit(c, &st[idx], &W[idx], -(float)votes[idx], lr, &change, c->weight_limit);
        changes += change;
    }
    return changes;
}

/* mgpu.cu:1114-1152 */
extern "C" uint64_t orc_update_vector_adam(const orc_config *c, int8_t *V, orc_adam_param *st, int len,
                                           int off_a, int off_b, int seed_base, const int32_t *fit, int pairs,
                                           uint32_t step_seed, float lr) {
    uint64_t changes = 0;
    for (int idx = 0; idx < len; idx++) {
        int32_t vote = 0;
        for (int p = 0; p < pairs; p++) {
            int f = fit[p]; if (f == 0) continue;
            int32_t n1 = orc_noise(step_seed + p + seed_base + off_a, idx, dev_mask(c));
            int32_t n2 = orc_noise(step_seed + p + seed_base + off_b, idx, dev_mask(c));
            vote += f * n1 * n2;
        }
        int change = 0;
        orc_adam_apply(c, &st[idx], &V[idx], -(float)vote, lr, &change);
        changes += change;
    }
    return changes;
}

/* mgpu.cu:1603-1643 */
extern "C" uint64_t orc_es_update_adam(const orc_config *c, int8_t *model, orc_adam_param *state,
                                       const int32_t *fit, uint32_t step_seed, float lr) {
    std::vector<orc_tensor> tt = tensor_table(c); int pairs = c->population / 2; uint64_t total = 0;
    for (const orc_tensor &t : tt) {
        if (t.is_matrix) total += orc_update_matrix_adam(c, model + t.offset, state + t.offset, t.rows, t.cols, t.off_a, t.off_b,
                                                         t.seed_base, fit, pairs, step_seed, lr * t.lr_scale);
        else total += orc_update_vector_adam(c, model + t.offset, state + t.offset, t.cols, t.off_a, t.off_b,
                                             t.seed_base, fit, pairs, step_seed, lr * t.lr_scale);
    }
    return total;
}

/* de/src/kernels.cu:61-77: an element whose row / column / vector entry saw at least one weight change this step
 * gains `inc`, every other one loses `dec`, clamped to [-127, 127] (de/include/config.h:57-58) */
extern "C" void orc_update_overlay(const int32_t *changes, int8_t *overlay, int count, int inc, int dec) {
    for (int i = 0; i < count; i++) {
        int ov = overlay[i];
        if (changes[i] > 0) { ov += inc; if (ov > 127) ov = 127; }
        else { ov -= dec; if (ov < -127) ov = -127; }
        overlay[i] = (int8_t)ov;
    }
}

/* The d-eggs optimizer step (de/src/worker.cu:446-523): the AdamW update of every tensor, with the weight changes
 * counted per input row and per output column of a matrix (de/include/optimizer/adam.cuh:77-83; the embedding's
 * counts go to its per-hidden and per-token values, de/src/worker.cu:497-516) or per element of a vector
 * (adam.cuh:130-132), followed by the overlay rule for that tensor.  The votes do not use the overlay
 * (adam.cuh:60-67).  A weight byte differs from its old value exactly when the reference sets `change`. */
extern "C" uint64_t orc_es_update_adam_adaptive(const orc_config *c, int8_t *model, orc_adam_param *state, int8_t *overlay,
                                                const int32_t *fit, uint32_t step_seed, float lr, int inc, int dec) {
    std::vector<int8_t> before(model, model + make_layout(c).total);
    uint64_t total = orc_es_update_adam(c, model, state, fit, step_seed, lr);
    for (const orc_tensor &t : tensor_table(c)) {
        if (t.is_matrix) {
            std::vector<int32_t> cnt((size_t)t.rows + t.cols, 0);
            for (int64_t idx = 0; idx < (int64_t)t.rows * t.cols; idx++) {
                if (model[t.offset + idx] == before[t.offset + idx]) continue;
                int byte_off = idx & 3; int64_t word = idx >> 2; int tid = (int)(word % t.cols); int k = (int)(word / t.cols) * 4 + byte_off;
                cnt[k]++; cnt[t.rows + tid]++;
            }
            orc_update_overlay(cnt.data(), overlay + t.offset, t.rows + t.cols, inc, dec);
        } else {
            std::vector<int32_t> cnt((size_t)t.cols, 0);
            for (int i = 0; i < t.cols; i++) cnt[i] = model[t.offset + i] != before[t.offset + i];
            orc_update_overlay(cnt.data(), overlay + t.offset, t.cols, inc, dec);
        }
    }
    return total;
}

/* mgpu.cu:217-227 */
extern "C" float orc_learning_rate(long step) {
    if (step < 300) return 0.3f;
    if (step < 600) return 0.15f;
    if (step < 1000) return 0.075f;
    return 0.05f;
}

/* ------------------------------------------------------------------ Muon */
/* muon_i:182-342.  X row-major [rows][cols].  rows < cols: G = X X^T, X <- 0.5 (3I-G) X;
 * otherwise G = X^T X, X <- 0.5 X (3I-G). */
template <typename F>
static void newton_schulz(F *X, int rows, int cols, int iters) {
    bool use_rows = rows < cols; int K = use_rows ? rows : cols; size_t n = (size_t)rows * cols;
    /* cublasSnrm2 + muon_scale_by_norm_kernel (muon_i:77-87, :214-220) */
    F ss = 0; for (size_t i = 0; i < n; i++) ss += X[i] * X[i];
    F norm = (F)sqrt((double)ss);
    if (norm > (F)1e-6f) for (size_t i = 0; i < n; i++) X[i] /= norm;
    std::vector<F> G((size_t)K * K), Bm((size_t)K * K), Y(n);
    for (int it = 0; it < iters; it++) {
#pragma omp parallel for schedule(static)
        for (int i = 0; i < K; i++)
            for (int j = 0; j < K; j++) {
                F s = 0;
                if (use_rows) for (int k = 0; k < cols; k++) s += X[(size_t)i * cols + k] * X[(size_t)j * cols + k];
                else          for (int k = 0; k < rows; k++) s += X[(size_t)k * cols + i] * X[(size_t)k * cols + j];
                G[(size_t)i * K + j] = s;
            }
        for (int i = 0; i < K; i++) for (int j = 0; j < K; j++)
            Bm[(size_t)i * K + j] = (i == j) ? ((F)3 - G[(size_t)i * K + j]) : -G[(size_t)i * K + j];   /* muon_i:91-109 */
#pragma omp parallel for schedule(static)
        for (int r = 0; r < rows; r++)
            for (int cidx = 0; cidx < cols; cidx++) {
                F s = 0;
                if (use_rows) for (int k = 0; k < K; k++) s += Bm[(size_t)r * K + k] * X[(size_t)k * cols + cidx];
                else          for (int k = 0; k < K; k++) s += X[(size_t)r * cols + k] * Bm[(size_t)k * K + cidx];
                Y[(size_t)r * cols + cidx] = (F)0.5 * s;
            }
        memcpy(X, Y.data(), n * sizeof(F));
    }
}
extern "C" void orc_newton_schulz_f32(float *X, int rows, int cols, int iters) { newton_schulz<float>(X, rows, cols, iters); }
extern "C" void orc_newton_schulz_f64(double *X, int rows, int cols, int iters) { newton_schulz<double>(X, rows, cols, iters); }

/* muon_i:15-50 (momentum), :53-74 (gather), :112-170 (apply); launch chain mgpu.cu:1587-1595 */
extern "C" uint64_t orc_update_matrix_muon(const orc_config *c, int8_t *W, orc_muon_param *st, int rows, int cols,
                                           int off_a, int off_b, int seed_base, const int32_t *fit, int pairs,
                                           uint32_t step_seed, float lr, float *ortho_out) {
    int64_t n = (int64_t)rows * cols; std::vector<int32_t> votes((size_t)n);
    orc_matrix_votes(c, rows, cols, off_a, off_b, seed_base, fit, pairs, step_seed, votes.data());
    std::vector<float> X((size_t)n);
    for (int64_t idx = 0; idx < n; idx++) {
        st[idx].m = c->muon_momentum * st[idx].m + (float)votes[idx];
        int byte_off = idx & 3; int64_t word = idx >> 2; int tid = (int)(word % cols); int k = (int)(word / cols) * 4 + byte_off;
        X[(size_t)k * cols + tid] = st[idx].m;
    }
    orc_newton_schulz_f32(X.data(), rows, cols, 5);
    if (ortho_out) memcpy(ortho_out, X.data(), (size_t)n * sizeof(float));
    uint64_t changes = 0; float lrs = lr * c->muon_lr_scale;
    for (int64_t idx = 0; idx < n; idx++) {
        int byte_off = idx & 3; int64_t word = idx >> 2; int tid = (int)(word % cols); int k = (int)(word / cols) * 4 + byte_off;
        float u = X[(size_t)k * cols + tid];
        float wdw = c->adam_weight_decay * (float)W[idx];
        float step = (-lrs) * (u + wdw);
        st[idx].acc += step;
        const int lim = c->weight_limit;
        if (st[idx].acc >= 1.0f) { if (W[idx] < lim) { W[idx]++; changes++; st[idx].acc -= 1.0f; } else st[idx].acc = 1.0f; }
        else if (st[idx].acc <= -1.0f) { if (W[idx] > -lim) { W[idx]--; changes++; st[idx].acc += 1.0f; } else st[idx].acc = -1.0f; }
    }
    return changes;
}

extern "C" int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

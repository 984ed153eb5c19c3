/*
 * egg_gru_oracle.cpp -- scalar (+OpenMP over pairs) restatement of the reference's
 * CPU program full_trained_egg.c ("egg.c" below).  TEST INFRASTRUCTURE ONLY.
 *
 * The reference file needs <arm_neon.h>, <dispatch/dispatch.h> and Apple blocks and
 * therefore cannot be compiled on x86.  Each of its NEON loops carries a scalar tail
 * that states the same arithmetic (egg.c:138-140, :163-165, :197, :400-402); the
 * loops below are those tails run over the full range.  Integer sums are
 * order-independent and no intermediate overflows (|int16 product| <= 16129,
 * |int32 sum| <= 2048*127*127), so the values are identical.  GCD dispatch_apply
 * over pairs (egg.c:547) becomes an OpenMP parallel-for over pairs.
 */
#include "egg_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <vector>

extern "C" void orc_gru_default_config(orc_gru_config *c) {
    c->hidden = 512; c->n_layers = 4; c->seq_len = 4096; c->vocab = 256; c->population = 128;   /* egg.c:11-15 */
    c->fixed_point = 4; c->sigma_shift = 4; c->update_threshold = 160;                          /* egg.c:17-19 */
}

/* field order of EggModel, egg.c:42-50 */
struct GruLayout { int64_t embedding, gru_w, gru_b, mlp_w, head, ln_w, ln_out, total; };
static GruLayout gru_layout(const orc_gru_config *c) {
    GruLayout L; int64_t o = 0, H = c->hidden, V = c->vocab, NL = c->n_layers;
    L.embedding = o; o += V * H;
    L.gru_w = o; o += NL * 4 * H * H;
    L.gru_b = o; o += NL * 2 * H;
    L.mlp_w = o; o += NL * 2 * H * 4 * H;
    L.head = o; o += H * V;
    L.ln_w = o; o += NL * 2 * H;
    L.ln_out = o; o += H;
    L.total = o; return L;
}
extern "C" int64_t orc_gru_model_bytes(const orc_gru_config *c) { return gru_layout(c).total; }
extern "C" int64_t orc_gru_state_bytes(const orc_gru_config *c) { return (int64_t)c->n_layers * c->hidden; }

static inline int8_t gen_noise_val(uint32_t *rng) {   /* egg.c:79-82 */
    uint32_t r = orc_xorshift32(rng);
    return (int8_t)((r & 1 ? 1 : -1) * (int)((r >> 1) & 31));
}
/* egg.c:87-105: four draws are discarded before every block of 16, no draw for padded slots */
extern "C" void orc_gru_noise_vector(uint32_t *rng, int8_t *out, int count) {
    for (int i = 0; i < count; i += 16) {
        orc_xorshift32(rng); orc_xorshift32(rng); orc_xorshift32(rng); orc_xorshift32(rng);
        for (int j = 0; j < 16; j++) if (i + j < count) out[i + j] = gen_noise_val(rng);
    }
}

/* egg.c:487-509 */
extern "C" void orc_gru_init_model(const orc_gru_config *c, int8_t *model, uint32_t seed) {
    GruLayout L = gru_layout(c); int64_t H = c->hidden, V = c->vocab; uint32_t rng = seed;
    memset(model, 0, (size_t)L.total);
    for (int64_t i = 0; i < V * H; i++) model[L.embedding + i] = gen_noise_val(&rng);
    for (int64_t i = 0; i < H * V; i++) model[L.head + i] = gen_noise_val(&rng);
    for (int l = 0; l < c->n_layers; l++) {
        for (int g = 0; g < 4; g++) for (int64_t i = 0; i < H * H; i++) model[L.gru_w + ((int64_t)l * 4 + g) * H * H + i] = gen_noise_val(&rng);
        for (int m = 0; m < 2; m++) for (int64_t i = 0; i < H * 4 * H; i++) model[L.mlp_w + ((int64_t)l * 2 + m) * H * 4 * H + i] = gen_noise_val(&rng);
    }
    for (int64_t i = 0; i < (int64_t)c->n_layers * 2 * H; i++) model[L.ln_w + i] = 16;
    for (int64_t i = 0; i < H; i++) model[L.ln_out + i] = 16;
}

static inline int8_t clipped_add(int32_t a, int32_t b) {   /* egg.c:62-67 */
    int32_t r = a + b; if (r > 127) return 127; if (r < -127) return -127; return (int8_t)r;
}

/* egg.c:108-177 */
extern "C" void orc_gru_matmul_perturbed(const orc_gru_config *c, const int8_t *in, const int8_t *w, int8_t *out,
                                         int rows, int cols, uint32_t layer_seed, int noise_sign, int shift) {
    std::vector<int8_t> A(rows), B(cols);
    uint32_t rng = layer_seed;
    orc_gru_noise_vector(&rng, A.data(), rows);
    orc_gru_noise_vector(&rng, B.data(), cols);
    int32_t xB = 0;
    for (int i = 0; i < cols; i++) xB += (int32_t)in[i] * (int32_t)B[i];
    std::vector<int8_t> res(rows);
    for (int r = 0; r < rows; r++) {
        int32_t acc = 0; const int8_t *wr = &w[(int64_t)r * cols];
        for (int k = 0; k < cols; k++) acc += (int32_t)in[k] * (int32_t)wr[k];
        if (noise_sign != 0) {
            int32_t noise = (xB * (int32_t)A[r]) * noise_sign;
            acc += (noise >> (c->fixed_point + c->sigma_shift));
        }
        int32_t v = acc >> shift;
        res[r] = (v > 127) ? 127 : ((v < -127) ? -127 : (int8_t)v);
    }
    memcpy(out, res.data(), rows);
}

/* egg.c:180-210 */
extern "C" void orc_gru_ln(const int8_t *x, const int8_t *w, int8_t *out, int H) {
    int32_t sum = 0;
    for (int i = 0; i < H; i++) sum += abs((int)x[i]);
    if (sum == 0) sum = 1;
    int32_t mean = sum / H; if (mean == 0) mean = 1;
    for (int i = 0; i < H; i++) {
        int32_t val = ((int32_t)x[i] * w[i]) / mean;
        out[i] = (val > 127) ? 127 : ((val < -127) ? -127 : (int8_t)val);
    }
}

static int32_t exp2_entry(int i, int fixed_point) {   /* egg.c:57-60 */
    return (int32_t)(pow(2.0, (double)i / (1 << fixed_point)) * (1 << fixed_point));
}
static int get_msb(uint32_t n) {   /* egg.c:299-307 */
    int pos = 0;
    if (n >= 1u << 16) { n >>= 16; pos += 16; }
    if (n >= 1u << 8) { n >>= 8; pos += 8; }
    if (n >= 1u << 4) { n >>= 4; pos += 4; }
    if (n >= 1u << 2) { n >>= 2; pos += 2; }
    if (n >= 1u << 1) { pos += 1; }
    return pos;
}
static int32_t log2_fixed(int32_t x) {   /* egg.c:309-319 */
    if (x <= 0) return 0;
    int k = get_msb((uint32_t)x); int32_t fraction;
    if (k >= 4) fraction = (x - (1 << k)) >> (k - 4); else fraction = (x - (1 << k)) << (4 - k);
    return (k << 4) + fraction - 64;
}
/* egg.c:321-330 */
static int32_t compute_loss_tab(const int32_t *exp2_table, const int8_t *logits, int V, int target) {
    int32_t sum_exp = 0;
    for (int i = 0; i < V; i++) {
        int idx = (int32_t)logits[i] + 128;
        sum_exp += exp2_table[idx < 0 ? 0 : (idx > 255 ? 255 : idx)];
    }
    return log2_fixed(sum_exp) - ((int32_t)logits[target] + 128);
}
extern "C" int32_t orc_gru_compute_loss(const int8_t *logits, int V, int target, int fixed_point) {
    int32_t tab[256];
    for (int i = 0; i < 256; i++) tab[i] = exp2_entry(i, fixed_point);
    return compute_loss_tab(tab, logits, V, target);
}

/* egg.c:213-296; state = h[L][H], updated in place; returns the accumulated loss */
extern "C" int32_t orc_gru_forward(const orc_gru_config *c, const int8_t *model, const uint8_t *inputs,
                                   const uint8_t *targets, int seq_len, int8_t *logits_out,
                                   uint32_t step_seed, int noise_sign, int8_t *state) {
    GruLayout L = gru_layout(c); const int H = c->hidden, V = c->vocab;
    std::vector<int8_t> x(H), residual(H), buf1(4 * H), buf2(H), ft(H), gated(H), ht(H), local_state, logits(V);
    if (!state) { local_state.assign((size_t)c->n_layers * H, 0); state = local_state.data(); }
    int32_t loss = 0;
    int32_t exp2_table[256];
    for (int i = 0; i < 256; i++) exp2_table[i] = exp2_entry(i, c->fixed_point);
    for (int t = 0; t < seq_len; t++) {
        memcpy(x.data(), &model[L.embedding + (int64_t)inputs[t] * H], H);
        for (int l = 0; l < c->n_layers; l++) {
            uint32_t l_seed = step_seed + (uint32_t)(l * 100);
            int8_t *h = state + (size_t)l * H;
            const int8_t *gw = model + L.gru_w + (int64_t)l * 4 * H * H;
            const int8_t *gb = model + L.gru_b + (int64_t)l * 2 * H;
            const int8_t *mw = model + L.mlp_w + (int64_t)l * 2 * H * 4 * H;
            const int8_t *lw = model + L.ln_w + (int64_t)l * 2 * H;
            memcpy(residual.data(), x.data(), H);
            orc_gru_ln(x.data(), lw, x.data(), H);
            orc_gru_matmul_perturbed(c, x.data(), gw, buf1.data(), H, H, l_seed + 1, noise_sign, 8);
            orc_gru_matmul_perturbed(c, h, gw + (int64_t)H * H, buf2.data(), H, H, l_seed + 2, noise_sign, 8);
            for (int i = 0; i < H; i++) ft[i] = clipped_add(clipped_add(buf1[i], buf2[i]), gb[i]);
            for (int i = 0; i < H; i++) gated[i] = (int8_t)(((int32_t)(ft[i] + 127) * h[i]) >> 8);
            orc_gru_matmul_perturbed(c, x.data(), gw + 2 * (int64_t)H * H, buf1.data(), H, H, l_seed + 3, noise_sign, 8);
            orc_gru_matmul_perturbed(c, gated.data(), gw + 3 * (int64_t)H * H, buf2.data(), H, H, l_seed + 4, noise_sign, 8);
            for (int i = 0; i < H; i++) ht[i] = clipped_add(clipped_add(buf1[i], buf2[i]), gb[H + i]);
            for (int i = 0; i < H; i++) {
                int32_t update = ((int32_t)(ft[i] + 127) * (ht[i] - h[i])) >> 8;
                h[i] = clipped_add(h[i], update);
                x[i] = h[i];
            }
            for (int i = 0; i < H; i++) x[i] = clipped_add(x[i], residual[i]);
            memcpy(residual.data(), x.data(), H);
            orc_gru_ln(x.data(), lw + H, x.data(), H);
            orc_gru_matmul_perturbed(c, x.data(), mw, buf1.data(), 4 * H, H, l_seed + 5, noise_sign, 8);
            orc_gru_matmul_perturbed(c, buf1.data(), mw + (int64_t)H * 4 * H, x.data(), H, 4 * H, l_seed + 6, noise_sign, 9);
            for (int i = 0; i < H; i++) x[i] = clipped_add(x[i], residual[i]);
        }
        orc_gru_ln(x.data(), model + L.ln_out, x.data(), H);
        orc_gru_matmul_perturbed(c, x.data(), model + L.head, logits.data(), V, H, step_seed + 999, noise_sign, 8);
        if (targets) loss += compute_loss_tab(exp2_table, logits.data(), V, targets[t]);
    }
    if (logits_out) memcpy(logits_out, logits.data(), V);
    return loss;
}

/* egg.c:547-562 */
extern "C" void orc_gru_population(const orc_gru_config *c, const int8_t *model, const uint8_t *data, int64_t data_len,
                                   int64_t start_idx, uint32_t step_seed, int pair0, int npairs,
                                   int8_t *states, int32_t *loss, int32_t *fit) {
    int64_t sb = orc_gru_state_bytes(c);
#pragma omp parallel for schedule(dynamic, 1)
    for (int i = 0; i < npairs; i++) {
        int p = pair0 + i;
        uint32_t p_seed = step_seed + (uint32_t)p;
        int64_t stride = data_len / (c->population / 2);
        int64_t stream_idx = (start_idx + (int64_t)p * stride) % (data_len - c->seq_len);
        int32_t lp = orc_gru_forward(c, model, data + stream_idx, data + stream_idx + 1, c->seq_len, NULL, p_seed, 1, states + (int64_t)(2 * p) * sb);
        int32_t ln = orc_gru_forward(c, model, data + stream_idx, data + stream_idx + 1, c->seq_len, NULL, p_seed, -1, states + (int64_t)(2 * p + 1) * sb);
        loss[2 * p] = lp; loss[2 * p + 1] = ln;
        fit[p] = (lp < ln) ? 1 : ((ln < lp) ? -1 : 0);
    }
}

/* egg.c:332-409 */
extern "C" void orc_gru_update_matrix(const orc_gru_config *c, int8_t *W, int rows, int cols, uint32_t seed,
                                      const int32_t *fit, int pop_size) {
    int pairs = pop_size / 2;
    std::vector<int8_t> AT((size_t)rows * pairs, 0), BT((size_t)cols * pairs, 0), At(rows), Bt(cols);
    for (int p = 0; p < pairs; p++) {
        int f = fit[p]; uint32_t rng = seed + (uint32_t)p;
        orc_gru_noise_vector(&rng, At.data(), rows);
        orc_gru_noise_vector(&rng, Bt.data(), cols);
        if (f == 0) { for (int r = 0; r < rows; r++) AT[(size_t)r * pairs + p] = 0; }
        else {
            for (int r = 0; r < rows; r++) AT[(size_t)r * pairs + p] = (int8_t)(At[r] * f);
            for (int k = 0; k < cols; k++) BT[(size_t)k * pairs + p] = Bt[k];
        }
    }
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; r++)
        for (int k = 0; k < cols; k++) {
            int32_t vote = 0; const int8_t *a = &AT[(size_t)r * pairs], *b = &BT[(size_t)k * pairs];
            for (int p = 0; p < pairs; p++) vote += (int32_t)a[p] * (int32_t)b[p];
            int8_t *w = &W[(int64_t)r * cols + k];
            if (vote > c->update_threshold && *w < 127) (*w)++;
            else if (vote < -c->update_threshold && *w > -127) (*w)--;
        }
}

/* egg.c:564-574 */
extern "C" void orc_gru_update_all(const orc_gru_config *c, int8_t *model, uint32_t step_seed, const int32_t *fit) {
    GruLayout L = gru_layout(c); int64_t H = c->hidden;
    for (int l = 0; l < c->n_layers; l++) {
        uint32_t l_seed = step_seed + (uint32_t)(l * 100);
        for (int g = 0; g < 4; g++)
            orc_gru_update_matrix(c, model + L.gru_w + ((int64_t)l * 4 + g) * H * H, (int)H, (int)H, l_seed + 1 + g, fit, c->population);
        orc_gru_update_matrix(c, model + L.mlp_w + ((int64_t)l * 2) * H * 4 * H, (int)(4 * H), (int)H, l_seed + 5, fit, c->population);
        orc_gru_update_matrix(c, model + L.mlp_w + ((int64_t)l * 2 + 1) * H * 4 * H, (int)H, (int)(4 * H), l_seed + 6, fit, c->population);
    }
    orc_gru_update_matrix(c, model + L.head, c->vocab, (int)H, step_seed + 999, fit, c->population);
}

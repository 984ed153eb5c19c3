// egg_api.hip -- the C ABI of libegg_hip.so (declared in include/egg_hip.h): context, model and
// optimizer-state management, and the host-side sequencing of the forward / fitness / update kernels.
// Reference host loop: full_cuda_train_transformer_adam_mgpu.cu:1313-1767 ("mgpu.cu").
#include "../../include/egg_hip.h"
#include "egg_launch.h"

#include <math.h>
#include <stdio.h>
#include <string.h>
#include <algorithm>
#include <sys/stat.h>
#include <string>
#include <vector>

// ------------------------------------------------------------------ model layout (TransformerModel, mgpu.cu:284-318)
struct Layout {
    int64_t embedding, emb_bias, ln_init, ln_init_bias, w_emb_mlp_up, mlp_emb_bias_up, w_emb_mlp_down,
        mlp_emb_bias_down, ln_1, ln_1_bias, w_q, w_k, w_v, w_o, ln_2, ln_2_bias, w_up, mlp_bias_up, w_down,
        mlp_bias_down, ln_f, ln_f_bias, total;
};
static Layout make_layout(const egg_config &c) {
    Layout L; int64_t o = 0, H = c.hidden, V = c.vocab, NL = c.n_layers;
    auto take = [&](int64_t n) { int64_t r = o; o += n; return r; };
    L.embedding = take(V * H); L.emb_bias = take(H); L.ln_init = take(H); L.ln_init_bias = take(H);
    L.w_emb_mlp_up = take(H * 4 * H); L.mlp_emb_bias_up = take(4 * H);
    L.w_emb_mlp_down = take(4 * H * H); L.mlp_emb_bias_down = take(H);
    L.ln_1 = take(NL * H); L.ln_1_bias = take(NL * H);
    L.w_q = take(NL * H * H); L.w_k = take(NL * H * H); L.w_v = take(NL * H * H); L.w_o = take(NL * H * H);
    L.ln_2 = take(NL * H); L.ln_2_bias = take(NL * H);
    L.w_up = take(NL * H * 4 * H); L.mlp_bias_up = take(NL * 4 * H);
    L.w_down = take(NL * 4 * H * H); L.mlp_bias_down = take(NL * H);
    L.ln_f = take(H); L.ln_f_bias = take(H);
    L.total = o;
    return L;
}

struct Scalars { uint32_t seed; float lr; int64_t start; };
__global__ void k_set_scalars(Scalars *s, uint32_t seed, float lr, int64_t start) { s->seed = seed; s->lr = lr; s->start = start; }

struct egg_ctx {
    egg_config cfg;
    hipStream_t stream = nullptr; bool own_stream = false;
    Layout L;
    std::vector<egg_tensor_info> tensors;
    int8_t *d_model = nullptr;
    uint8_t *d_state = nullptr; int64_t state_bytes = 0; std::vector<int64_t> t_state_off;   // optimizer state (AdamModel layout)
    MuonWork muon = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    std::vector<std::vector<int>> muon_groups;    // ids of the Muon matrices, grouped by shape; a group runs Newton-Schulz as batches
    std::vector<int> muon_group_batch;            // per group: matrices of that shape the Muon workspace holds at once
    int muon_batch_max = 1;                       // the largest of them (sizes the per-matrix norm buffers)
    size_t muon_elems = 0, muon_bterm = 0;        // floats in each of the two matrix buffers / in the 3I - G buffer
    int8_t *d_wfrag = nullptr;      // fragment-major copy of every matrix, same offsets as the model blob
    int8_t *d_plin_frag = nullptr; size_t plin_frag_bytes = 0;
    bool plin_no_ws = false;        // egg_ctx_linear_kernel: run the W-streaming kernels also where the W-stationary one exists
    int32_t *d_exp = nullptr; int8_t *d_act = nullptr; int32_t *d_rope = nullptr;
    int chunk = 0;
    int8_t *d_x = nullptr, *d_q = nullptr, *d_k = nullptr, *d_v = nullptr, *d_ao = nullptr;
    unsigned long long *d_loss_acc = nullptr, *d_counter = nullptr;
    int32_t *d_loss = nullptr, *d_fit = nullptr;
    Scalars *d_scal = nullptr;
    int8_t *d_panel_a = nullptr, *d_panel_b = nullptr; int pairs_pad = 0;
    // taps
    bool taps = false; int8_t *d_tap = nullptr; int32_t *d_tap_logits = nullptr; int tap_members = 0;
    // per-kernel-class event timing (egg_ctx_enable_timing)
    bool timing = false;
    struct Span { int cls; hipEvent_t a, b; };
    std::vector<Span> spans; size_t spans_used = 0;
    double t_ms[EGG_KCLASS_COUNT] = {0}; long t_n[EGG_KCLASS_COUNT] = {0};
    // generation (egg_generate): token buffer [T + 1], logits of one member [T][vocab], a zero start index / seed
    uint8_t *d_gen_tok = nullptr; int32_t *d_gen_logits = nullptr, *d_gen_ws = nullptr; Scalars *d_gen_scal = nullptr;
    int8_t *d_gen_kv = nullptr; bool gen_kv_cache = true;      // per-layer K / V rows of the generated sequence (egg_ctx_generate_kv_cache)
    int mask_override = -1; int32_t *logits_override = nullptr;
    bool first_dedup = true;        // first block once per distinct byte value of a member's window (egg_ctx_first_block_dedup)
    VecDesc *d_vec_desc = nullptr; int n_vec = 0, vec_total = 0;       // all vector tensors, for the one-launch update
    // adaptive noise overlay (egg_adaptive_enable): raw overlay values, q = clamp(overlay, 0, 64) and change flags, all
    // laid out like the model blob; one segment (rows + cols, or len) per tensor
    bool adaptive = false; int ov_inc = 5, ov_dec = 1;
    int8_t *d_overlay = nullptr, *d_overlay_q = nullptr, *d_flags = nullptr;
    OvSeg *d_ov_segs = nullptr; int n_ov_segs = 0, ov_max_count = 0;
    // graph
    hipGraph_t graph = nullptr; hipGraphExec_t gexec = nullptr; bool captured = false;
    std::string err;
};

// magnitude mask plus the Gaussian flag, as the kernels take it
static int noise_word(const egg_config &c) { return c.noise_mask | (c.device_gaussian ? EGG_NOISE_GAUSSIAN : 0); }

static int fail(egg_ctx *ctx, int code, const char *what, hipError_t e = hipSuccess) {
    if (ctx) {
        ctx->err = what;
        if (e != hipSuccess) { ctx->err += ": "; ctx->err += hipGetErrorString(e); }
    }
    return code;
}
#define HIP_TRY(call) do { hipError_t e_ = (call); if (e_ != hipSuccess) return fail(ctx, EGG_E_HIP, #call, e_); } while (0)

// event pair around one kernel launch of class `cls`; no-ops unless timing is enabled
static void span_begin(egg_ctx *ctx, int cls) {
    if (!ctx->timing) return;
    if (ctx->spans_used == ctx->spans.size()) {
        egg_ctx::Span sp; sp.cls = cls;
        if (hipEventCreate(&sp.a) != hipSuccess || hipEventCreate(&sp.b) != hipSuccess) { ctx->timing = false; return; }
        ctx->spans.push_back(sp);
    }
    ctx->spans[ctx->spans_used].cls = cls;
    (void)hipEventRecord(ctx->spans[ctx->spans_used].a, ctx->stream);
}
static void span_end(egg_ctx *ctx) {
    if (!ctx->timing) return;
    (void)hipEventRecord(ctx->spans[ctx->spans_used].b, ctx->stream);
    ctx->spans_used++;
}
// closes the span on every way out of a scope, error returns included
struct SpanScope {
    egg_ctx *ctx;
    SpanScope(egg_ctx *c, int cls) : ctx(c) { span_begin(c, cls); }
    ~SpanScope() { span_end(ctx); }
};
static void spans_collect(egg_ctx *ctx) {
    for (size_t i = 0; i < ctx->spans_used; i++) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, ctx->spans[i].a, ctx->spans[i].b) == hipSuccess) { ctx->t_ms[ctx->spans[i].cls] += ms; ctx->t_n[ctx->spans[i].cls]++; }
    }
    ctx->spans_used = 0;
}

extern "C" void egg_default_config(egg_config *c) {
    memset(c, 0, sizeof(*c));
    c->hidden = 256; c->head_dim = 64; c->n_layers = 4; c->seq_len = 32; c->vocab = 256; c->population = 16384 * 4;
    c->fixed_point = 4; c->sigma_shift = 3; c->sigma_shift_vector = 4;
    c->shift_attn = 8; c->shift_out = 9; c->shift_logit = 8; c->shift_mlp_up = 8; c->shift_mlp_down = 10;
    c->softmax_scale_bit = 18; c->rope_scale_bit = 20; c->noise_mask = 15; c->host_mask = 15;
    c->softmax_exp_scale = 6.0;
    c->adam_beta1 = 0.9f; c->adam_beta2 = 0.95f; c->adam_eps = 1e-8f; c->adam_weight_decay = 0.01f;
    c->muon_momentum = 0.85f; c->muon_lr_scale = 1.0f; c->use_muon = 0; c->chunk_members = 0; c->weight_limit = 127;
    c->device_gaussian = 0; c->host_gaussian = 0; c->use_same_data = 0;
}

// launch order of mgpu.cu:1603-1643
static std::vector<egg_tensor_info> build_tensor_table(const egg_config &c, const Layout &L) {
    std::vector<egg_tensor_info> tensors; int H = c.hidden, V = c.vocab;
    auto add = [&](const char *name, int l, int is_matrix, int rows, int cols, int64_t off, int oa, int ob, int base, float lrs, int muon) {
        egg_tensor_info t; memset(&t, 0, sizeof(t));
        if (l >= 0) snprintf(t.name, sizeof(t.name), "%s.%d", name, l); else snprintf(t.name, sizeof(t.name), "%s", name);
        t.is_matrix = is_matrix; t.rows = rows; t.cols = cols; t.offset = off; t.off_a = oa; t.off_b = ob;
        t.seed_base = base; t.lr_scale = lrs; t.muon = muon;
        tensors.push_back(t);
    };
    for (int l = 0; l < c.n_layers; l++) {
        int b = l * 1000; int64_t hh = (int64_t)H * H, h4 = (int64_t)H * 4 * H;
        add("w_q", l, 1, H, H, L.w_q + l * hh, OFF_Q_A, OFF_Q_B, b, 1.f, 1);
        add("w_k", l, 1, H, H, L.w_k + l * hh, OFF_K_A, OFF_K_B, b, 1.f, 1);
        add("w_v", l, 1, H, H, L.w_v + l * hh, OFF_V_A, OFF_V_B, b, 1.f, 1);
        add("w_o", l, 1, H, H, L.w_o + l * hh, OFF_O_A, OFF_O_B, b, 1.f, 1);
        add("w_up", l, 1, H, 4 * H, L.w_up + l * h4, OFF_MLP_UP_A, OFF_MLP_UP_B, b, 1.f, 1);
        add("w_down", l, 1, 4 * H, H, L.w_down + l * h4, OFF_MLP_DOWN_A, OFF_MLP_DOWN_B, b, 1.f, 1);
        add("ln_1", l, 0, 1, H, L.ln_1 + (int64_t)l * H, OFF_LN_1_A, OFF_LN_1_B, b, 1.f, 0);
        add("ln_1_bias", l, 0, 1, H, L.ln_1_bias + (int64_t)l * H, OFF_LN_1_BIAS_A, OFF_LN_1_BIAS_B, b, 1.f, 0);
        add("ln_2", l, 0, 1, H, L.ln_2 + (int64_t)l * H, OFF_LN_2_A, OFF_LN_2_B, b, 1.f, 0);
        add("ln_2_bias", l, 0, 1, H, L.ln_2_bias + (int64_t)l * H, OFF_LN_2_BIAS_A, OFF_LN_2_BIAS_B, b, 1.f, 0);
        add("mlp_bias_up", l, 0, 1, 4 * H, L.mlp_bias_up + (int64_t)l * 4 * H, OFF_MLP_BIAS_UP_A, OFF_MLP_BIAS_UP_B, b, 1.f, 0);
        add("mlp_bias_down", l, 0, 1, H, L.mlp_bias_down + (int64_t)l * H, OFF_MLP_BIAS_DOWN_A, OFF_MLP_BIAS_DOWN_B, b, 1.f, 0);
    }
    add("ln_f", -1, 0, 1, H, L.ln_f, OFF_LN_F_A, OFF_LN_F_B, 0, 1.f, 0);
    add("ln_f_bias", -1, 0, 1, H, L.ln_f_bias, OFF_LN_F_BIAS_A, OFF_LN_F_BIAS_B, 0, 1.f, 0);
    add("ln_init", -1, 0, 1, H, L.ln_init, OFF_LN_INIT_A, OFF_LN_INIT_B, 0, 1.f, 0);
    add("ln_init_bias", -1, 0, 1, H, L.ln_init_bias, OFF_LN_INIT_BIAS_A, OFF_LN_INIT_BIAS_B, 0, 1.f, 0);
    add("w_emb_mlp_up", -1, 1, H, 4 * H, L.w_emb_mlp_up, OFF_EMB_MLP_UP_A, OFF_EMB_MLP_UP_B, 0, 1.f, 1);
    add("mlp_emb_bias_up", -1, 0, 1, 4 * H, L.mlp_emb_bias_up, OFF_EMB_MLP_BIAS_UP_A, OFF_EMB_MLP_BIAS_UP_B, 0, 1.f, 0);
    add("w_emb_mlp_down", -1, 1, 4 * H, H, L.w_emb_mlp_down, OFF_EMB_MLP_DOWN_A, OFF_EMB_MLP_DOWN_B, 0, 1.f, 1);
    add("mlp_emb_bias_down", -1, 0, 1, H, L.mlp_emb_bias_down, OFF_EMB_MLP_BIAS_DOWN_A, OFF_EMB_MLP_BIAS_DOWN_B, 0, 1.f, 0);
    add("emb_bias", -1, 0, 1, H, L.emb_bias, OFF_EMB_BIAS_A, OFF_EMB_BIAS_B, 0, 0.1f, 0);
    add("embedding", -1, 1, H, V, L.embedding, OFF_EMB, OFF_EMB + H, 0, 1.f, 0);
    return tensors;
}
// optimizer state in the field order of AdamModel (mgpu.cu:337-370): {m,v,acc} per element, or {m,acc} for the
// matrices that use Muon (HIDDEN_OPT_TYPE, mgpu.cu:327-335); returns the total size
static int64_t state_offsets(const egg_config &c, const std::vector<egg_tensor_info> &tensors, std::vector<int64_t> &off) {
    std::vector<int> order(tensors.size());
    for (size_t i = 0; i < order.size(); i++) order[i] = (int)i;
    std::sort(order.begin(), order.end(), [&](int a, int b) { return tensors[a].offset < tensors[b].offset; });
    off.assign(tensors.size(), 0);
    int64_t so = 0;
    for (int id : order) {
        const egg_tensor_info &t = tensors[id];
        off[id] = so;
        so += (int64_t)t.rows * t.cols * ((c.use_muon && t.muon) ? 8 : 12);
    }
    return so;
}
// Muon workspace plan (host arithmetic only).  Matrices of one shape form a group and go through Newton-Schulz in
// batches; a group's batch is as much of it as fits 16 Mi floats per matrix buffer, at least one matrix.  The
// buffers hold the largest batch of any group: `elems` floats in each matrix buffer, `bterm` in the 3I - G buffer.
struct MuonPlan { std::vector<std::vector<int>> groups; std::vector<int> batch; size_t elems = 0, bterm = 0; int batch_max = 1; };
static MuonPlan muon_plan(const egg_config &c, const std::vector<egg_tensor_info> &tensors) {
    MuonPlan pl;
    for (int id = 0; id < (int)tensors.size(); id++) {
        const egg_tensor_info &t = tensors[id];
        if (!t.is_matrix || !t.muon) continue;
        bool placed = false;
        for (auto &g : pl.groups)
            if (tensors[g[0]].rows == t.rows && tensors[g[0]].cols == t.cols) { g.push_back(id); placed = true; break; }
        if (!placed) pl.groups.push_back(std::vector<int>(1, id));
    }
    // egg_update_tensor runs a single matrix of any Muon shape through the same buffers
    const size_t mx = (size_t)4 * c.hidden * c.hidden;
    size_t cap = (size_t)16 << 20;
    if (cap < mx) cap = mx;
    pl.elems = mx; pl.bterm = (size_t)c.hidden * c.hidden;
    for (const auto &g : pl.groups) {
        const egg_tensor_info &t = tensors[g[0]];
        const size_t one = (size_t)t.rows * t.cols, k = (size_t)(t.rows < t.cols ? t.rows : t.cols);
        size_t b = cap / one; if (b > g.size()) b = g.size(); if (b < 1) b = 1;
        if (b * one > pl.elems) pl.elems = b * one;
        if (b * k * k > pl.bterm) pl.bterm = b * k * k;
        if ((int)b > pl.batch_max) pl.batch_max = (int)b;
        pl.batch.push_back((int)b);
    }
    return pl;
}
// host-only: group `group` of the plan a context of this configuration would use (its shape, member count and batch
// limit) and the workspace sizes in floats; returns the number of groups
extern "C" int egg_muon_plan(const egg_config *cfg, int group, int *rows, int *cols, int *members, int *batch,
                             int64_t *matrix_buffer_floats, int64_t *term_buffer_floats) {
    if (!cfg || cfg->hidden < 4 || cfg->n_layers < 1 || cfg->vocab < 1) return EGG_E_INVALID;
    const Layout L = make_layout(*cfg);
    const std::vector<egg_tensor_info> tensors = build_tensor_table(*cfg, L);
    const MuonPlan pl = muon_plan(*cfg, tensors);
    if (matrix_buffer_floats) *matrix_buffer_floats = (int64_t)pl.elems;
    if (term_buffer_floats) *term_buffer_floats = (int64_t)pl.bterm;
    if (group < 0) return (int)pl.groups.size();
    if (group >= (int)pl.groups.size()) return EGG_E_INVALID;
    const egg_tensor_info &t = tensors[pl.groups[group][0]];
    if (rows) *rows = t.rows;
    if (cols) *cols = t.cols;
    if (members) *members = (int)pl.groups[group].size();
    if (batch) *batch = pl.batch[group];
    return (int)pl.groups.size();
}

// host-only view of the same tables (no device is touched)
extern "C" int egg_describe_layout(const egg_config *cfg, int tensor_id, egg_tensor_info *out, int64_t *state_offset,
                                   int64_t *model_bytes, int64_t *state_bytes) {
    if (!cfg || cfg->hidden < 4 || cfg->n_layers < 1 || cfg->vocab < 1) return EGG_E_INVALID;
    const Layout L = make_layout(*cfg);
    const std::vector<egg_tensor_info> tensors = build_tensor_table(*cfg, L);
    std::vector<int64_t> off;
    const int64_t sb = state_offsets(*cfg, tensors, off);
    if (model_bytes) *model_bytes = L.total;
    if (state_bytes) *state_bytes = sb;
    if (tensor_id < 0) return (int)tensors.size();
    if (tensor_id >= (int)tensors.size()) return EGG_E_INVALID;
    if (out) *out = tensors[tensor_id];
    if (state_offset) *state_offset = off[tensor_id];
    return (int)tensors.size();
}

static void free_all(egg_ctx *ctx) {
    void *ptrs[] = {ctx->muon.x, ctx->muon.swap, ctx->muon.bterm, ctx->muon.partials, ctx->muon.norm,
                    ctx->d_wfrag, ctx->d_plin_frag, ctx->d_model, ctx->d_state, ctx->d_exp, ctx->d_act, ctx->d_rope, ctx->d_x, ctx->d_q, ctx->d_k, ctx->d_v,
                    ctx->d_ao, ctx->d_loss_acc, ctx->d_counter, ctx->d_loss, ctx->d_fit, ctx->d_scal, ctx->d_panel_a,
                    ctx->d_panel_b, ctx->d_tap, ctx->d_tap_logits, ctx->d_gen_tok, ctx->d_gen_logits, ctx->d_gen_ws, ctx->d_gen_scal, ctx->d_gen_kv, ctx->d_vec_desc,
                    ctx->d_overlay, ctx->d_overlay_q, ctx->d_flags, ctx->d_ov_segs};
    for (void *p : ptrs) if (p) (void)hipFree(p);
    for (auto &sp : ctx->spans) { (void)hipEventDestroy(sp.a); (void)hipEventDestroy(sp.b); }
    if (ctx->gexec) (void)hipGraphExecDestroy(ctx->gexec);
    if (ctx->graph) (void)hipGraphDestroy(ctx->graph);
    if (ctx->own_stream && ctx->stream) (void)hipStreamDestroy(ctx->stream);
}

// why the last egg_ctx_create of this thread failed (there is no context to hold the message yet)
static thread_local std::string g_create_err;
static int refuse(const char *why) { g_create_err = why; return EGG_E_INVALID; }
void egg_set_thread_error(const char *what) { g_create_err = what; }

extern "C" int egg_ctx_create(const egg_config *cfg, egg_ctx **out) {
    if (!cfg || !out) return refuse("egg_ctx_create: null argument");
    *out = nullptr;
    const egg_config &c = *cfg;
    if (!(c.hidden == 64 || c.hidden == 128 || c.hidden == 256 || c.hidden == 512)) return refuse("hidden must be 64, 128, 256 or 512");
    if (!(c.head_dim == 32 || c.head_dim == 64) || c.hidden % c.head_dim) return refuse("head_dim must be 32 or 64 and divide hidden");
    if (!(c.seq_len == 32 || c.seq_len == 64 || c.seq_len == 128 || c.seq_len == 256 || c.seq_len == 512))
        return refuse("seq_len must be 32, 64, 128, 256 or 512");
    // 256: the byte-level model, the token stream is bytes.  Larger (d-eggs' VOCAB_SIZE, de/include/config.h:22-28): uint32
    // tokens; the head takes the vocabulary in blocks of 256 columns
    if (c.vocab < 256 || c.vocab % 256 || c.vocab > 65536) return refuse("vocab must be a multiple of 256, at most 65536");
    if (c.n_layers < 1 || c.population < 2 || (c.population & 1)) return refuse("n_layers >= 1 and an even population >= 2 are required");
    // shift amounts and table scales the kernels can state in 32-bit shifts / 64-bit multiply-adds
    auto in_range = [](int v, int lo, int hi) { return v >= lo && v <= hi; };
    if (!in_range(c.rope_scale_bit, 1, 30)) return refuse("rope_scale_bit must be 1..30");
    // the attention kernels split every exp-table weight into three 7-bit planes for the int8 matrix pipe; the largest
    // entry is exp(0) * 2^softmax_scale_bit, so it must stay below 2^21
    if (!in_range(c.softmax_scale_bit, 1, 20)) return refuse("softmax_scale_bit must be 1..20 (table weights are split into three 7-bit planes)");
    if (!(c.softmax_exp_scale > 0.0)) return refuse("softmax_exp_scale must be positive");
    if (!in_range(c.noise_mask, 0, 127) || !in_range(c.host_mask, 0, 127)) return refuse("noise_mask and host_mask must be 0..127");
    const int mag = c.device_gaussian ? 3 * c.noise_mask : c.noise_mask;        // largest |noise|
    if (mag > 127 || (c.host_gaussian ? 3 : 1) * c.host_mask > 127) return refuse("Gaussian noise needs 3 * mask <= 127");
    // x.B sums enter 24-bit multiplies: |sum| <= 4 * hidden * 127 * |noise|
    if ((long long)4 * c.hidden * 127 * mag >= (1LL << 23)) return refuse("noise too wide for this hidden size (4 * hidden * 127 * |noise| must stay below 2^23)");
    if (!in_range(c.fixed_point + c.sigma_shift, 0, 24) || !in_range(c.sigma_shift_vector, 0, 24) || !in_range(c.shift_attn, 0, 24) ||
        !in_range(c.shift_out, 0, 24) || !in_range(c.shift_logit, 0, 24) || !in_range(c.shift_mlp_up, 0, 24) ||
        !in_range(c.shift_mlp_down, 0, 24)) return refuse("shift amounts must be 0..24");
    // the standard norm divides x * (gain + noise) by the row mean with a 32-bit multiply-high that is exact up to 2^17
    if (127 * (127 + ((mag * mag) >> c.sigma_shift_vector)) > (1 << 17))
        return refuse("noise_mask^2 >> sigma_shift_vector is too large for the norm's exact division");
    if (!in_range(c.weight_limit, 1, 127)) return refuse("weight_limit must be 1..127");
    // the MLP's up accumulator carries (bias + 128 + noise) << shift_mlp_up on top of its matrix product
    if (egg_mlp_up_acc_bound(c.hidden, noise_word(c), c.sigma_shift_vector, c.shift_mlp_up) >= (1LL << 31))
        return refuse("shift_mlp_up is too large: (bias + 128 + noise) << shift_mlp_up plus the up projection's sum must stay below 2^31");
    egg_ctx *ctx = new egg_ctx();
    ctx->cfg = c;
    ctx->L = make_layout(c);
    ctx->tensors = build_tensor_table(c, ctx->L);
    auto bail = [&](int code, const char *what, hipError_t e) {
        g_create_err = std::string(what) + ": " + hipGetErrorString(e);
        free_all(ctx); delete ctx; return code;
    };
#define CR(call) do { hipError_t e_ = (call); if (e_ != hipSuccess) return bail(EGG_E_HIP, #call, e_); } while (0)
    CR(hipStreamCreate(&ctx->stream)); ctx->own_stream = true;
    CR(egg_prepare_forward(c.hidden, c.head_dim, c.seq_len));
    // lookup tables in double precision on the host, exactly as init_tables (mgpu.cu:394-426)
    std::vector<int32_t> ex(256), rope((size_t)c.seq_len * c.head_dim); std::vector<int8_t> act(256);
    for (int i = 0; i < 256; i++) {
        double val = exp(-(double)i / c.softmax_exp_scale) * (double)(1 << c.softmax_scale_bit);
        ex[i] = (val >= 1.0) ? (int32_t)round(val) : 0;
        int8_t input = (int8_t)i;
        double x = (double)input / (1 << c.fixed_point);
        double y = 0.5 * x * (1.0 + erf(x / 1.41421356));
        int v = (int)round(y * (1 << c.fixed_point));
        act[i] = (int8_t)((v > 127) ? 127 : ((v < -127) ? -127 : v));
    }
    for (int t = 0; t < c.seq_len; t++)
        for (int i = 0; i < c.head_dim / 2; i++) {
            double theta = pow(10000.0, -2.0 * i / c.head_dim), alpha = t * theta;
            rope[(size_t)t * c.head_dim + 2 * i] = (int32_t)round(cos(alpha) * (double)(1 << c.rope_scale_bit));
            rope[(size_t)t * c.head_dim + 2 * i + 1] = (int32_t)round(sin(alpha) * (double)(1 << c.rope_scale_bit));
        }
    CR(hipMalloc(&ctx->d_exp, 256 * 4)); CR(hipMalloc(&ctx->d_act, 256)); CR(hipMalloc(&ctx->d_rope, rope.size() * 4));
    CR(hipMemcpy(ctx->d_exp, ex.data(), 256 * 4, hipMemcpyHostToDevice));
    CR(hipMemcpy(ctx->d_act, act.data(), 256, hipMemcpyHostToDevice));
    CR(hipMemcpy(ctx->d_rope, rope.data(), rope.size() * 4, hipMemcpyHostToDevice));
    CR(hipMalloc(&ctx->d_model, ctx->L.total)); CR(hipMemset(ctx->d_model, 0, ctx->L.total));
    CR(hipMalloc(&ctx->d_wfrag, ctx->L.total)); CR(hipMemset(ctx->d_wfrag, 0, ctx->L.total));
    ctx->state_bytes = state_offsets(c, ctx->tensors, ctx->t_state_off);
    CR(hipMalloc(&ctx->d_state, ctx->state_bytes)); CR(hipMemset(ctx->d_state, 0, ctx->state_bytes));
    {
        std::vector<VecDesc> vd;
        int first = 0;
        for (size_t id = 0; id < ctx->tensors.size(); id++) {
            const egg_tensor_info &t = ctx->tensors[id];
            if (t.is_matrix) continue;
            VecDesc d; d.W = ctx->d_model + t.offset; d.state = reinterpret_cast<float *>(ctx->d_state + ctx->t_state_off[id]);
            d.n = t.cols; d.first = first; d.off_a = t.off_a; d.off_b = t.off_b; d.seed_base = t.seed_base; d.lr_scale = t.lr_scale;
            d.flags = nullptr;
            vd.push_back(d); first += t.cols;
        }
        ctx->n_vec = (int)vd.size(); ctx->vec_total = first;
        CR(hipMalloc(&ctx->d_vec_desc, vd.size() * sizeof(VecDesc)));
        CR(hipMemcpy(ctx->d_vec_desc, vd.data(), vd.size() * sizeof(VecDesc), hipMemcpyHostToDevice));
    }
    if (c.use_muon) {
        const MuonPlan pl = muon_plan(c, ctx->tensors);
        ctx->muon_groups = pl.groups; ctx->muon_group_batch = pl.batch; ctx->muon_batch_max = pl.batch_max;
        ctx->muon_elems = pl.elems; ctx->muon_bterm = pl.bterm;
        const int nb = pl.batch_max;
        CR(hipMalloc(&ctx->muon.x, pl.elems * 4)); CR(hipMalloc(&ctx->muon.swap, pl.elems * 4));
        CR(hipMalloc(&ctx->muon.bterm, pl.bterm * 4));
        CR(hipMalloc(&ctx->muon.partials, (size_t)nb * 256 * 4 + 1024 * 4)); CR(hipMalloc(&ctx->muon.norm, (size_t)nb * 4 + 16));
    }
    // activation workspace for one chunk of members
    // default: the whole population in one launch per kernel while its five activation buffers stay within 32 GiB
    // (8192 members per launch are 3 % faster per member than 2048, 40,960 another 1.2 %: fewer launches, shorter
    // tails), otherwise 8192 members
    int chunk = c.chunk_members;
    if (chunk <= 0) {
        const size_t whole = (size_t)5 * c.population * c.seq_len * c.hidden;
        chunk = whole <= ((size_t)32 << 30) ? c.population : 8192;
    }
    if (chunk > c.population) chunk = c.population;
    ctx->chunk = chunk;
    size_t act_bytes = (size_t)chunk * c.seq_len * c.hidden;
    CR(hipMalloc(&ctx->d_x, act_bytes)); CR(hipMalloc(&ctx->d_q, act_bytes)); CR(hipMalloc(&ctx->d_k, act_bytes));
    CR(hipMalloc(&ctx->d_v, act_bytes)); CR(hipMalloc(&ctx->d_ao, act_bytes));
    CR(hipMalloc(&ctx->d_loss_acc, (size_t)c.population * 8)); CR(hipMalloc(&ctx->d_counter, 8));
    CR(hipMemset(ctx->d_counter, 0, 8));
    CR(hipMalloc(&ctx->d_loss, (size_t)c.population * 4)); CR(hipMalloc(&ctx->d_fit, (size_t)(c.population / 2) * 4));
    CR(hipMalloc(&ctx->d_scal, sizeof(Scalars)));
    ctx->pairs_pad = ((c.population / 2) + 63) / 64 * 64;
    const size_t panel_rows = std::max(4 * c.hidden, c.vocab);       // the widest side of any matrix: 4 * hidden, or the embedding's vocabulary
    CR(hipMalloc(&ctx->d_panel_a, panel_rows * ctx->pairs_pad));
    CR(hipMalloc(&ctx->d_panel_b, panel_rows * ctx->pairs_pad));
#undef CR
    *out = ctx;
    return EGG_OK;
}

// refresh the fragment-major copy of one matrix (tensor id) or of all matrices (id < 0); enqueued on the stream
static int refresh_frag(egg_ctx *ctx, int id) {
    for (int i = 0; i < (int)ctx->tensors.size(); i++) {
        const egg_tensor_info &t = ctx->tensors[i];
        if (!t.is_matrix || (id >= 0 && i != id)) continue;
        // hidden x hidden blocks for the layer matrices; the embedding (hidden x 256) is cut into <= 256-wide blocks
        const int B = (t.cols == ctx->cfg.vocab && t.rows == ctx->cfg.hidden && ctx->cfg.hidden > 256) ? 256 : ctx->cfg.hidden;
        HIP_TRY(egg_launch_swizzle(ctx->d_model + t.offset, ctx->d_wfrag + t.offset, t.rows, t.cols, B, 0, ctx->stream));
    }
    return EGG_OK;
}

extern "C" void egg_ctx_destroy(egg_ctx *ctx) {
    if (!ctx) return;
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    free_all(ctx);
    delete ctx;
}
extern "C" const char *egg_last_error(const egg_ctx *ctx) { return ctx ? ctx->err.c_str() : g_create_err.c_str(); }
extern "C" int egg_ctx_set_stream(egg_ctx *ctx, void *s) {
    if (!ctx) return EGG_E_INVALID;
    if (ctx->captured) return fail(ctx, EGG_E_STATE, "stream cannot change after egg_step_capture");
    if (ctx->own_stream && ctx->stream) { (void)hipStreamSynchronize(ctx->stream); (void)hipStreamDestroy(ctx->stream); }
    ctx->stream = (hipStream_t)s; ctx->own_stream = false;
    return EGG_OK;
}
extern "C" int egg_sync(egg_ctx *ctx) {
    if (!ctx) return EGG_E_INVALID;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return EGG_OK;
}

extern "C" int64_t egg_model_bytes(const egg_ctx *ctx) { return ctx ? ctx->L.total : 0; }

// ------------------------------------------------------------------ init_model (mgpu.cu:428-519)
static inline uint32_t xorshift32_host(uint32_t *st) { uint32_t x = *st; x ^= x << 13; x ^= x >> 17; x ^= x << 5; *st = x; return x; }
static inline int8_t gen_noise_host(uint32_t *rng, int mask, int gaussian) {
    uint32_t r = xorshift32_host(rng);
    int n = (r & 1 ? 1 : -1) * (int)((r >> 1) & (uint32_t)mask);
    if (gaussian) n += (r & 32 ? 1 : -1) * (int)((r >> 6) & (uint32_t)mask) + (r & 1024 ? 1 : -1) * (int)((r >> 11) & (uint32_t)mask);
    return (int8_t)n;
}
// [In][Out] row-major -> blocked [In/4][Out][4]
static void repack_matrix(int8_t *dst, const int8_t *src, int rows, int cols) {
    for (int kq = 0; kq < rows / 4; kq++)
        for (int n = 0; n < cols; n++)
            for (int s = 0; s < 4; s++) dst[((size_t)kq * cols + n) * 4 + s] = src[(size_t)(4 * kq + s) * cols + n];
}
extern "C" int egg_model_init(egg_ctx *ctx, uint32_t seed) {
    if (!ctx) return EGG_E_INVALID;
    const egg_config &c = ctx->cfg; const Layout &L = ctx->L; const int H = c.hidden, V = c.vocab;
    std::vector<int8_t> m((size_t)L.total, 0), tmp((size_t)H * 4 * H > (size_t)V * H ? (size_t)H * 4 * H : (size_t)V * H);
    uint32_t rng = seed;
    auto gen = [&](int8_t *dst, int rows, int cols) {
        for (size_t i = 0; i < (size_t)rows * cols; i++) tmp[i] = gen_noise_host(&rng, c.host_mask, c.host_gaussian);
        repack_matrix(dst, tmp.data(), rows, cols);
    };
    gen(&m[L.embedding], H, V);
    for (int i = 0; i < H; i++) m[L.ln_init + i] = 16;
    gen(&m[L.w_emb_mlp_up], H, 4 * H);
    gen(&m[L.w_emb_mlp_down], 4 * H, H);
    for (int l = 0; l < c.n_layers; l++) {
        for (int i = 0; i < H; i++) { m[L.ln_1 + (int64_t)l * H + i] = 16; m[L.ln_2 + (int64_t)l * H + i] = 16; }
        gen(&m[L.w_q + (int64_t)l * H * H], H, H); gen(&m[L.w_k + (int64_t)l * H * H], H, H);
        gen(&m[L.w_v + (int64_t)l * H * H], H, H); gen(&m[L.w_o + (int64_t)l * H * H], H, H);
        gen(&m[L.w_up + (int64_t)l * H * 4 * H], H, 4 * H); gen(&m[L.w_down + (int64_t)l * 4 * H * H], 4 * H, H);
    }
    for (int i = 0; i < H; i++) m[L.ln_f + i] = 16;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipMemcpy(ctx->d_model, m.data(), m.size(), hipMemcpyHostToDevice));
    return refresh_frag(ctx, -1);
}
extern "C" int egg_model_upload(egg_ctx *ctx, const void *h, size_t bytes) {
    if (!ctx || !h || (int64_t)bytes != ctx->L.total) return fail(ctx, EGG_E_INVALID, "model size mismatch");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipMemcpy(ctx->d_model, h, bytes, hipMemcpyHostToDevice));
    return refresh_frag(ctx, -1);
}
extern "C" int egg_model_download(egg_ctx *ctx, void *h, size_t bytes) {
    if (!ctx || !h || (int64_t)bytes != ctx->L.total) return fail(ctx, EGG_E_INVALID, "model size mismatch");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipMemcpy(h, ctx->d_model, bytes, hipMemcpyDeviceToHost));
    return EGG_OK;
}
// ------------------------------------------------------------------ ternary-packed model (no reference counterpart)
// The packed blob is the model blob with every matrix tensor stored at 2 bits per weight (see k_ternary_unpack) and
// every vector tensor left as int8, tensors in the order of their offsets in the model blob.
static std::vector<int> tensors_by_offset(const egg_ctx *ctx) {
    std::vector<int> ids(ctx->tensors.size());
    for (size_t i = 0; i < ids.size(); i++) ids[i] = (int)i;
    std::sort(ids.begin(), ids.end(), [&](int a, int b) { return ctx->tensors[a].offset < ctx->tensors[b].offset; });
    return ids;
}
extern "C" int64_t egg_ternary_model_bytes(const egg_ctx *ctx) {
    if (!ctx) return 0;
    int64_t n = 0;
    for (const egg_tensor_info &t : ctx->tensors) n += t.is_matrix ? (int64_t)t.rows * t.cols / 4 : t.cols;
    return n;
}
extern "C" int egg_model_upload_ternary(egg_ctx *ctx, const void *h, size_t bytes) {
    if (!ctx || !h || (int64_t)bytes != egg_ternary_model_bytes(ctx)) return fail(ctx, EGG_E_INVALID, "ternary model size mismatch");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    uint8_t *d_packed = nullptr;
    HIP_TRY(hipMalloc(&d_packed, bytes));
    hipError_t e = hipMemcpy(d_packed, h, bytes, hipMemcpyHostToDevice);
    int64_t po = 0;
    for (int id : tensors_by_offset(ctx)) {
        const egg_tensor_info &t = ctx->tensors[id];
        if (e != hipSuccess) break;
        if (t.is_matrix) {
            e = egg_launch_ternary_unpack(d_packed + po, ctx->d_model + t.offset, t.rows * t.cols, ctx->stream);
            po += (int64_t)t.rows * t.cols / 4;
        } else {
            e = hipMemcpyAsync(ctx->d_model + t.offset, d_packed + po, (size_t)t.cols, hipMemcpyDeviceToDevice, ctx->stream);
            po += t.cols;
        }
    }
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    (void)hipFree(d_packed);
    if (e != hipSuccess) return fail(ctx, EGG_E_HIP, "egg_model_upload_ternary", e);
    return refresh_frag(ctx, -1);
}
extern "C" int egg_model_download_ternary(egg_ctx *ctx, void *h, size_t bytes) {
    if (!ctx || !h || (int64_t)bytes != egg_ternary_model_bytes(ctx)) return fail(ctx, EGG_E_INVALID, "ternary model size mismatch");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    uint8_t *d_packed = nullptr;
    const size_t flag_off = (bytes + 3) & ~(size_t)3;          // the out-of-range flag sits behind the packed bytes
    HIP_TRY(hipMalloc(&d_packed, flag_off + 4));
    int *d_bad = reinterpret_cast<int *>(d_packed + flag_off);
    hipError_t e = hipMemsetAsync(d_bad, 0, 4, ctx->stream);
    int64_t po = 0;
    for (int id : tensors_by_offset(ctx)) {
        const egg_tensor_info &t = ctx->tensors[id];
        if (e != hipSuccess) break;
        if (t.is_matrix) {
            e = egg_launch_ternary_pack(ctx->d_model + t.offset, d_packed + po, t.rows * t.cols, d_bad, ctx->stream);
            po += (int64_t)t.rows * t.cols / 4;
        } else {
            e = hipMemcpyAsync(d_packed + po, ctx->d_model + t.offset, (size_t)t.cols, hipMemcpyDeviceToDevice, ctx->stream);
            po += t.cols;
        }
    }
    int bad = 0;
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) e = hipMemcpy(&bad, d_bad, 4, hipMemcpyDeviceToHost);
    if (e == hipSuccess && !bad) e = hipMemcpy(h, d_packed, bytes, hipMemcpyDeviceToHost);
    (void)hipFree(d_packed);
    if (e != hipSuccess) return fail(ctx, EGG_E_HIP, "egg_model_download_ternary", e);
    if (bad) return fail(ctx, EGG_E_INVALID, "a matrix weight is outside {-1, 0, 1}: the model is not ternary");
    return EGG_OK;
}

extern "C" int egg_opt_state_upload(egg_ctx *ctx, const void *h, size_t bytes) {
    if (!ctx || !h || (int64_t)bytes != ctx->state_bytes) return fail(ctx, EGG_E_INVALID, "state size mismatch");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipMemcpy(ctx->d_state, h, bytes, hipMemcpyHostToDevice));
    return EGG_OK;
}
extern "C" int egg_opt_state_download(egg_ctx *ctx, void *h, size_t bytes) {
    if (!ctx || !h || (int64_t)bytes != ctx->state_bytes) return fail(ctx, EGG_E_INVALID, "state size mismatch");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipMemcpy(h, ctx->d_state, bytes, hipMemcpyDeviceToHost));
    return EGG_OK;
}
extern "C" int egg_opt_state_reset(egg_ctx *ctx) {
    if (!ctx) return EGG_E_INVALID;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipMemset(ctx->d_state, 0, ctx->state_bytes));
    return EGG_OK;
}
extern "C" int egg_tables_download(egg_ctx *ctx, int32_t *ex, int8_t *act, int32_t *rope) {
    if (!ctx) return EGG_E_INVALID;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    if (ex) HIP_TRY(hipMemcpy(ex, ctx->d_exp, 256 * 4, hipMemcpyDeviceToHost));
    if (act) HIP_TRY(hipMemcpy(act, ctx->d_act, 256, hipMemcpyDeviceToHost));
    if (rope) HIP_TRY(hipMemcpy(rope, ctx->d_rope, (size_t)ctx->cfg.seq_len * ctx->cfg.head_dim * 4, hipMemcpyDeviceToHost));
    return EGG_OK;
}

extern "C" int egg_noise_fill(egg_ctx *ctx, uint32_t seed, uint32_t first, int n, int8_t *d_out) {
    if (!ctx || !d_out || n < 0) return fail(ctx, EGG_E_INVALID, "egg_noise_fill arguments");
    HIP_TRY(egg_launch_noise_fill(seed, first, n, noise_word(ctx->cfg), d_out, ctx->stream));
    return EGG_OK;
}

static int linear_impl(egg_ctx *ctx, const int8_t *d_X, const int8_t *d_W, int members, int T, int K, int N,
                       uint32_t seed, int off_a, int off_b, int shift, int32_t *d_Y32, int8_t *d_Y8, int plain, int own_noise);
extern "C" int egg_perturbed_linear(egg_ctx *ctx, const int8_t *d_X, const int8_t *d_W, int members, int T, int K, int N,
                                    uint32_t seed, int off_a, int off_b, int shift, int32_t *d_Y32, int8_t *d_Y8) {
    return linear_impl(ctx, d_X, d_W, members, T, K, N, seed, off_a, off_b, shift, d_Y32, d_Y8, 0, 0);
}
extern "C" int egg_perturbed_linear_own_noise(egg_ctx *ctx, const int8_t *d_X, const int8_t *d_W, int members, int T, int K, int N,
                                              uint32_t seed, int off_a, int off_b, int shift, int32_t *d_Y32, int8_t *d_Y8) {
    return linear_impl(ctx, d_X, d_W, members, T, K, N, seed, off_a, off_b, shift, d_Y32, d_Y8, 0, 1);
}
extern "C" int egg_shared_linear(egg_ctx *ctx, const int8_t *d_X, const int8_t *d_W, int members, int T, int K, int N,
                                 int shift, int32_t *d_Y32, int8_t *d_Y8) {
    return linear_impl(ctx, d_X, d_W, members, T, K, N, 0, 0, 0, shift, d_Y32, d_Y8, 1, 0);
}
extern "C" int egg_ctx_linear_kernel(egg_ctx *ctx, int w_stationary) {
    if (!ctx) return EGG_E_INVALID;
    ctx->plin_no_ws = !w_stationary;
    return EGG_OK;
}
static int linear_impl(egg_ctx *ctx, const int8_t *d_X, const int8_t *d_W, int members, int T, int K, int N,
                       uint32_t seed, int off_a, int off_b, int shift, int32_t *d_Y32, int8_t *d_Y8, int plain, int own_noise) {
    if (!ctx || !d_X || !d_W || members < 1 || T < 32 || T % 32 || (!d_Y32 && !d_Y8) || shift < 0 || shift > 31)
        return fail(ctx, EGG_E_INVALID, "egg_perturbed_linear arguments");
    if (K < 64 || N < 64 || K % 64 || N % 64) return fail(ctx, EGG_E_INVALID, "egg_perturbed_linear: K and N must be multiples of 64");
    const bool ws = egg_plinear_ws_shape(K, N) && !ctx->plin_no_ws;
    if (!ws && (size_t)K * N > ctx->plin_frag_bytes) {
        HIP_TRY(hipStreamSynchronize(ctx->stream));
        if (ctx->d_plin_frag) (void)hipFree(ctx->d_plin_frag);
        ctx->d_plin_frag = nullptr; ctx->plin_frag_bytes = 0;
        HIP_TRY(hipMalloc(&ctx->d_plin_frag, (size_t)K * N));
        ctx->plin_frag_bytes = (size_t)K * N;
    }
    PlinParams p = {d_X, ctx->d_plin_frag, members, T, K, N, seed, off_a, off_b, shift, ctx->cfg.fixed_point + ctx->cfg.sigma_shift,
                    noise_word(ctx->cfg), d_Y32, d_Y8, plain, own_noise, ws ? d_W : nullptr};
    span_begin(ctx, EGG_K_PLINEAR);
    hipError_t e = ws ? hipSuccess : egg_launch_plinear_swizzle(d_W, ctx->d_plin_frag, T, K, N, ctx->stream);
    if (e == hipSuccess) e = egg_launch_plinear(p, ctx->stream);
    span_end(ctx);
    if (e == hipErrorInvalidValue) return fail(ctx, EGG_E_INVALID, "egg_perturbed_linear: unsupported (K, N)");
    HIP_TRY(e);
    return EGG_OK;
}

// ------------------------------------------------------------------ forward
static FwdCommon make_common(egg_ctx *ctx, const uint8_t *d_data, int64_t len, const int64_t *d_start, const uint32_t *d_seed,
                             int first_member, int nm) {
    const egg_config &c = ctx->cfg;
    FwdCommon f;
    f.data = d_data; f.data_len = len; f.d_start_idx = d_start; f.d_step_seed = d_seed;
    f.pop_offset = first_member; f.n_members = nm; f.population = c.population; f.same_data = c.use_same_data != 0;
    f.T = c.seq_len; f.H = c.hidden; f.head_dim = c.head_dim; f.vocab = c.vocab;
    f.token_bytes = c.vocab > 256 ? 4 : 1;
    f.t0 = 0; f.tn = c.seq_len;
    f.sigma = c.fixed_point + c.sigma_shift; f.sigma_vec = c.sigma_shift_vector;
    f.mask = ctx->mask_override >= 0 ? ctx->mask_override : noise_word(c);
    f.shift_attn = c.shift_attn; f.shift_out = c.shift_out; f.shift_logit = c.shift_logit;
    f.shift_mlp_up = c.shift_mlp_up; f.shift_mlp_down = c.shift_mlp_down;
    f.softmax_scale_bit = c.softmax_scale_bit; f.rope_scale_bit = c.rope_scale_bit;
    f.exp_lut = ctx->d_exp; f.act_lut = ctx->d_act; f.rope_lut = ctx->d_rope;
    return f;
}

// tap buffer: [slot][member][T][H], slots: 0 x_init, then per layer 6: q k v ao x_attn x_mlp
static int8_t *tap_ptr(egg_ctx *ctx, int slot) {
    return ctx->d_tap + (size_t)slot * ctx->tap_members * ctx->cfg.seq_len * ctx->cfg.hidden;
}

// `range` (generation only): evaluate the token positions [t0, t0 + tn) of the chunk's members and keep every layer's
// K / V rows in `kv` ([layer][K, V][nm][T][H]) instead of the shared k / v buffers, so that a later call on a later
// range finds the rows of the positions in front of it (the reference's d_gen_kv, mgpu.cu:1160-1170)
struct FwdRange { int t0, tn; int8_t *kv; };
static int forward_chunk(egg_ctx *ctx, const uint8_t *d_data, int64_t len, const int64_t *d_start, const uint32_t *d_seed,
                         int first_member, int nm, const FwdRange *range = nullptr) {
    const egg_config &c = ctx->cfg; const Layout &L = ctx->L; const int8_t *M = ctx->d_model; const int H = c.hidden;
    const int8_t *F = ctx->d_wfrag;
    const int8_t *Q = ctx->adaptive ? ctx->d_overlay_q : nullptr;      // same offsets as the model blob
    hipStream_t s = ctx->stream;
    const bool taps = ctx->taps && nm <= ctx->tap_members;
    const size_t act_bytes = (size_t)nm * c.seq_len * H;
    FwdCommon f = make_common(ctx, d_data, len, d_start, d_seed, first_member, nm);
    if (range) { f.t0 = range->t0; f.tn = range->tn; }
    {
        MlpParams p; memset(&p, 0, sizeof(p)); p.c = f; p.seed_base = 0;
        p.off_ln_a = OFF_LN_INIT_A; p.off_ln_b = OFF_LN_INIT_B; p.off_lnb_a = OFF_LN_INIT_BIAS_A; p.off_lnb_b = OFF_LN_INIT_BIAS_B;
        p.off_up_a = OFF_EMB_MLP_UP_A; p.off_up_b = OFF_EMB_MLP_UP_B; p.off_bup_a = OFF_EMB_MLP_BIAS_UP_A; p.off_bup_b = OFF_EMB_MLP_BIAS_UP_B;
        p.off_dn_a = OFF_EMB_MLP_DOWN_A; p.off_dn_b = OFF_EMB_MLP_DOWN_B; p.off_bdn_a = OFF_EMB_MLP_BIAS_DOWN_A; p.off_bdn_b = OFF_EMB_MLP_BIAS_DOWN_B;
        p.ln_w = M + L.ln_init; p.ln_b = M + L.ln_init_bias; p.w_up = F + L.w_emb_mlp_up; p.b_up = M + L.mlp_emb_bias_up;
        p.w_dn = F + L.w_emb_mlp_down; p.b_dn = M + L.mlp_emb_bias_down;
        p.embedding = M + L.embedding; p.emb_bias = M + L.emb_bias; p.x = ctx->d_x;
        // the q buffer is free until the first layer's QKV projection writes it; one row per distinct value only pays (and
        // is only built) for byte tokens
        p.tab = (ctx->first_dedup && !range && c.vocab == 256) ? ctx->d_q : nullptr;
        if (Q) {
            p.q_ln_w = Q + L.ln_init; p.q_ln_b = Q + L.ln_init_bias; p.q_b_up = Q + L.mlp_emb_bias_up; p.q_b_dn = Q + L.mlp_emb_bias_down;
            p.q_up = Q + L.w_emb_mlp_up; p.q_dn = Q + L.w_emb_mlp_down; p.q_emb = Q + L.embedding; p.q_emb_bias = Q + L.emb_bias;
        }
        { SpanScope span(ctx, EGG_K_MLP_FIRST); HIP_TRY(egg_launch_mlp(p, true, s)); }
        if (taps) HIP_TRY(hipMemcpyAsync(tap_ptr(ctx, 0), ctx->d_x, act_bytes, hipMemcpyDeviceToDevice, s));
    }
    for (int l = 0; l < c.n_layers; l++) {
        const int64_t hh = (int64_t)H * H, h4 = (int64_t)H * 4 * H;
        {
            QkvParams p; memset(&p, 0, sizeof(p)); p.c = f; p.seed_base = l * 1000;
            p.ln_w = M + L.ln_1 + (int64_t)l * H; p.ln_b = M + L.ln_1_bias + (int64_t)l * H;
            p.w_q = F + L.w_q + l * hh; p.w_k = F + L.w_k + l * hh; p.w_v = F + L.w_v + l * hh;
            p.x = ctx->d_x; p.q = ctx->d_q; p.k = ctx->d_k; p.v = ctx->d_v;
            if (range && range->kv) { p.k = range->kv + (size_t)(2 * l) * act_bytes; p.v = range->kv + (size_t)(2 * l + 1) * act_bytes; }
            if (Q) {
                p.q_ln_w = Q + L.ln_1 + (int64_t)l * H; p.q_ln_b = Q + L.ln_1_bias + (int64_t)l * H;
                p.q_wq = Q + L.w_q + l * hh; p.q_wk = Q + L.w_k + l * hh; p.q_wv = Q + L.w_v + l * hh;
            }
            { SpanScope span(ctx, EGG_K_QKV); HIP_TRY(egg_launch_qkv(p, s)); }
            if (taps) {
                HIP_TRY(hipMemcpyAsync(tap_ptr(ctx, 1 + 6 * l + 0), ctx->d_q, act_bytes, hipMemcpyDeviceToDevice, s));
                HIP_TRY(hipMemcpyAsync(tap_ptr(ctx, 1 + 6 * l + 1), ctx->d_k, act_bytes, hipMemcpyDeviceToDevice, s));
                HIP_TRY(hipMemcpyAsync(tap_ptr(ctx, 1 + 6 * l + 2), ctx->d_v, act_bytes, hipMemcpyDeviceToDevice, s));
            }
        }
        {
            AttnParams p; memset(&p, 0, sizeof(p)); p.c = f; p.q = ctx->d_q; p.k = ctx->d_k; p.v = ctx->d_v; p.ao = ctx->d_ao;
            if (range && range->kv) { p.k = range->kv + (size_t)(2 * l) * act_bytes; p.v = range->kv + (size_t)(2 * l + 1) * act_bytes; }
            { SpanScope span(ctx, EGG_K_ATTN); HIP_TRY(egg_launch_attn(p, s)); }
            if (taps) HIP_TRY(hipMemcpyAsync(tap_ptr(ctx, 1 + 6 * l + 3), ctx->d_ao, act_bytes, hipMemcpyDeviceToDevice, s));
        }
        {
            MlpParams p; memset(&p, 0, sizeof(p)); p.c = f; p.seed_base = l * 1000;
            p.off_ln_a = OFF_LN_2_A; p.off_ln_b = OFF_LN_2_B; p.off_lnb_a = OFF_LN_2_BIAS_A; p.off_lnb_b = OFF_LN_2_BIAS_B;
            p.off_up_a = OFF_MLP_UP_A; p.off_up_b = OFF_MLP_UP_B; p.off_bup_a = OFF_MLP_BIAS_UP_A; p.off_bup_b = OFF_MLP_BIAS_UP_B;
            p.off_dn_a = OFF_MLP_DOWN_A; p.off_dn_b = OFF_MLP_DOWN_B; p.off_bdn_a = OFF_MLP_BIAS_DOWN_A; p.off_bdn_b = OFF_MLP_BIAS_DOWN_B;
            p.ln_w = M + L.ln_2 + (int64_t)l * H; p.ln_b = M + L.ln_2_bias + (int64_t)l * H;
            p.w_up = F + L.w_up + l * h4; p.b_up = M + L.mlp_bias_up + (int64_t)l * 4 * H;
            p.w_dn = F + L.w_down + l * h4; p.b_dn = M + L.mlp_bias_down + (int64_t)l * H;
            p.w_o = F + L.w_o + l * hh; p.ao = ctx->d_ao; p.x = ctx->d_x;
            p.x_mid = taps ? tap_ptr(ctx, 1 + 6 * l + 4) : nullptr;
            if (Q) {
                p.q_ln_w = Q + L.ln_2 + (int64_t)l * H; p.q_ln_b = Q + L.ln_2_bias + (int64_t)l * H;
                p.q_b_up = Q + L.mlp_bias_up + (int64_t)l * 4 * H; p.q_b_dn = Q + L.mlp_bias_down + (int64_t)l * H;
                p.q_up = Q + L.w_up + l * h4; p.q_dn = Q + L.w_down + l * h4; p.q_o = Q + L.w_o + l * hh;
            }
            { SpanScope span(ctx, EGG_K_MLP); HIP_TRY(egg_launch_mlp(p, false, s)); }
            if (taps) HIP_TRY(hipMemcpyAsync(tap_ptr(ctx, 1 + 6 * l + 5), ctx->d_x, act_bytes, hipMemcpyDeviceToDevice, s));
        }
    }
    {
        HeadParams p; memset(&p, 0, sizeof(p)); p.c = f;
        p.ln_w = M + L.ln_f; p.ln_b = M + L.ln_f_bias; p.embedding_frag = F + L.embedding; p.x = ctx->d_x;
        p.loss_acc = ctx->d_loss_acc; p.logits_tap = ctx->logits_override ? ctx->logits_override : (taps ? ctx->d_tap_logits : nullptr);
        if (Q) { p.q_ln_w = Q + L.ln_f; p.q_ln_b = Q + L.ln_f_bias; p.q_emb = Q + L.embedding; }
        { SpanScope span(ctx, EGG_K_HEAD); HIP_TRY(egg_launch_head(p, s)); }
    }
    return EGG_OK;
}

static int forward_range(egg_ctx *ctx, const uint8_t *d_data, int64_t len, const int64_t *d_start, const uint32_t *d_seed,
                         int pop_offset, int pop_count, int32_t *d_loss) {
    const egg_config &c = ctx->cfg;
    if (!d_data || !d_loss || pop_offset < 0 || pop_count < 1 || pop_offset + pop_count > c.population)
        return fail(ctx, EGG_E_INVALID, "population range");
    if (len <= c.seq_len + 1) return fail(ctx, EGG_E_INVALID, "data_len must exceed seq_len + 1");
    HIP_TRY(egg_launch_zero_u64(ctx->d_loss_acc + pop_offset, pop_count, ctx->stream));
    for (int done = 0; done < pop_count; done += ctx->chunk) {
        int nm = pop_count - done < ctx->chunk ? pop_count - done : ctx->chunk;
        int rc = forward_chunk(ctx, d_data, len, d_start, d_seed, pop_offset + done, nm);
        if (rc) return rc;
    }
    HIP_TRY(egg_launch_loss_finalize(ctx->d_loss_acc, d_loss, pop_offset, pop_count, ctx->stream));
    return EGG_OK;
}

extern "C" int egg_population_forward_dev(egg_ctx *ctx, const uint8_t *d_data, int64_t len, const int64_t *d_start,
                                          const uint32_t *d_seed, int pop_offset, int pop_count, int32_t *d_loss) {
    if (!ctx || !d_start || !d_seed) return fail(ctx, EGG_E_INVALID, "null scalar pointer");
    return forward_range(ctx, d_data, len, d_start, d_seed, pop_offset, pop_count, d_loss);
}
extern "C" int egg_population_forward(egg_ctx *ctx, const uint8_t *d_data, int64_t len, int64_t start_idx, uint32_t step_seed,
                                      int pop_offset, int pop_count, int32_t *d_loss) {
    if (!ctx) return EGG_E_INVALID;
    hipLaunchKernelGGL(k_set_scalars, dim3(1), dim3(1), 0, ctx->stream, ctx->d_scal, step_seed, 0.f, start_idx);
    HIP_TRY(hipGetLastError());
    return forward_range(ctx, d_data, len, &ctx->d_scal->start, &ctx->d_scal->seed, pop_offset, pop_count, d_loss);
}

extern "C" int egg_fitness(egg_ctx *ctx, const int32_t *d_loss, int32_t *d_fit, int pairs) {
    if (!ctx || !d_loss || !d_fit || pairs < 0) return fail(ctx, EGG_E_INVALID, "egg_fitness arguments");
    HIP_TRY(egg_launch_fitness(d_loss, d_fit, pairs, ctx->stream));
    return EGG_OK;
}

// ------------------------------------------------------------------ update
static UpdParams make_upd(egg_ctx *ctx, int id, const int32_t *d_fit, const uint32_t *d_seed, const float *d_lr) {
    const egg_tensor_info &t = ctx->tensors[id];
    const egg_config &c = ctx->cfg;
    UpdParams p; memset(&p, 0, sizeof(p));
    p.W = ctx->d_model + t.offset; p.state = reinterpret_cast<float *>(ctx->d_state + ctx->t_state_off[id]);
    p.rows = t.rows; p.cols = t.cols; p.off_a = t.off_a; p.off_b = t.off_b; p.seed_base = t.seed_base;
    p.fit = d_fit; p.pairs = c.population / 2; p.d_seed = d_seed; p.d_lr = d_lr; p.lr_scale = t.lr_scale;
    p.limit = t.is_matrix ? c.weight_limit : 127;
    p.mask = noise_word(c); p.beta1 = c.adam_beta1; p.beta2 = c.adam_beta2; p.eps = c.adam_eps; p.wd = c.adam_weight_decay;
    p.panel_a = ctx->d_panel_a; p.panel_b = ctx->d_panel_b; p.pairs_pad = ctx->pairs_pad; p.counter = ctx->d_counter;
    return p;
}
static int update_one(egg_ctx *ctx, int id, const int32_t *d_fit, const uint32_t *d_seed, const float *d_lr, bool record_flags = false) {
    const egg_tensor_info &t = ctx->tensors[id];
    UpdParams p = make_upd(ctx, id, d_fit, d_seed, d_lr);
    if (record_flags) p.flags = ctx->d_flags + t.offset;
    if (t.is_matrix && t.muon && ctx->cfg.use_muon) {
        // LAUNCH_ADAM_MATRIX under USE_MUON (mgpu.cu:1587-1595)
        {
            SpanScope span(ctx, EGG_K_UPDATE_MATRIX);
            p.muon_momentum = ctx->cfg.muon_momentum; p.muon_x = ctx->muon.x;
            HIP_TRY(egg_launch_muon_momentum(p, ctx->stream));
            HIP_TRY(egg_launch_newton_schulz(ctx->muon, t.rows, t.cols, 5, ctx->stream));
            p.lr_scale = t.lr_scale * ctx->cfg.muon_lr_scale;
            HIP_TRY(egg_launch_muon_apply(p, ctx->cfg.adam_weight_decay, ctx->stream));
        }
        int rc = refresh_frag(ctx, id);
        if (rc) return rc;
    } else if (t.is_matrix) {
        { SpanScope span(ctx, EGG_K_UPDATE_MATRIX); HIP_TRY(egg_launch_update_matrix(p, ctx->stream)); }
        int rc = refresh_frag(ctx, id);
        if (rc) return rc;
    }
    else { SpanScope span(ctx, EGG_K_UPDATE_VECTOR); HIP_TRY(egg_launch_update_vector(p, ctx->stream)); }
    return EGG_OK;
}
extern "C" int egg_update_tensor(egg_ctx *ctx, int id, const int32_t *d_fit, const uint32_t *d_seed, const float *d_lr) {
    if (!ctx || id < 0 || id >= (int)ctx->tensors.size() || !d_fit || !d_seed || !d_lr) return fail(ctx, EGG_E_INVALID, "egg_update_tensor arguments");
    return update_one(ctx, id, d_fit, d_seed, d_lr);
}
extern "C" int egg_matrix_votes(egg_ctx *ctx, int id, const int32_t *d_fit, const uint32_t *d_seed, int32_t *d_votes) {
    if (!ctx || id < 0 || id >= (int)ctx->tensors.size() || !d_fit || !d_seed || !d_votes || !ctx->tensors[id].is_matrix)
        return fail(ctx, EGG_E_INVALID, "egg_matrix_votes arguments");
    UpdParams p = make_upd(ctx, id, d_fit, d_seed, nullptr);
    p.votes_out = d_votes;
    HIP_TRY(egg_launch_update_matrix(p, ctx->stream));
    return EGG_OK;
}
extern "C" int egg_es_update(egg_ctx *ctx, const int32_t *d_fit, const uint32_t *d_seed, const float *d_lr) {
    if (!ctx || !d_fit || !d_seed || !d_lr) return fail(ctx, EGG_E_INVALID, "egg_es_update arguments");
    HIP_TRY(egg_launch_zero_u64(ctx->d_counter, 1, ctx->stream));
    // matrices one by one (each needs the panel workspace), then every vector tensor in one launch; tensors are
    // independent, so the reference's launch order (mgpu.cu:1603-1643) does not matter
    for (int id = 0; id < (int)ctx->tensors.size(); id++) {
        if (!ctx->tensors[id].is_matrix || (ctx->cfg.use_muon && ctx->tensors[id].muon)) continue;
        int rc = update_one(ctx, id, d_fit, d_seed, d_lr, ctx->adaptive);
        if (rc) return rc;
    }
    // Muon matrices (LAUNCH_ADAM_MATRIX under USE_MUON, mgpu.cu:1587-1595), a batch of one shape at a time: momentum of
    // each into its slot of the workspace, Newton-Schulz of the whole batch, then each matrix's apply rule
    if (ctx->cfg.use_muon)
        for (size_t gi = 0; gi < ctx->muon_groups.size(); gi++) {
            const std::vector<int> &g = ctx->muon_groups[gi];
            const egg_tensor_info &t0 = ctx->tensors[g[0]];
            const size_t one = (size_t)t0.rows * t0.cols, k = (size_t)(t0.rows < t0.cols ? t0.rows : t0.cols);
            const size_t limit = (size_t)ctx->muon_group_batch[gi];
            // the group's own limit, never the largest group's: the buffers hold `limit` matrices of this shape
            if (limit < 1 || limit * one > ctx->muon_elems || limit * k * k > ctx->muon_bterm || (int)limit > ctx->muon_batch_max)
                return fail(ctx, EGG_E_STATE, "Muon batch does not fit the workspace");
            for (size_t first = 0; first < g.size(); first += limit) {
                const int nb = (int)std::min(g.size() - first, limit);
                int rc = EGG_OK;
                {
                    SpanScope span(ctx, EGG_K_UPDATE_MATRIX);
                    for (int b = 0; b < nb; b++) {
                        UpdParams p = make_upd(ctx, g[first + b], d_fit, d_seed, d_lr);
                        p.muon_momentum = ctx->cfg.muon_momentum; p.muon_x = ctx->muon.x + (size_t)b * one;
                        HIP_TRY(egg_launch_muon_momentum(p, ctx->stream));
                    }
                }
                { SpanScope span(ctx, EGG_K_MUON_NS); HIP_TRY(egg_launch_newton_schulz_batched(ctx->muon, t0.rows, t0.cols, 5, nb, ctx->stream)); }
                {
                    SpanScope span(ctx, EGG_K_UPDATE_MATRIX);
                    // a failed launch must not leave earlier matrices of the batch with a stale fragment-major copy:
                    // go on to the refresh below with what was applied, then report
                    int applied = 0;
                    for (; applied < nb; applied++) {
                        const int id = g[first + applied];
                        UpdParams p = make_upd(ctx, id, d_fit, d_seed, d_lr);
                        p.muon_x = ctx->muon.x + (size_t)applied * one;
                        p.lr_scale = ctx->tensors[id].lr_scale * ctx->cfg.muon_lr_scale;
                        const hipError_t e = egg_launch_muon_apply(p, ctx->cfg.adam_weight_decay, ctx->stream);
                        if (e != hipSuccess) { rc = fail(ctx, EGG_E_HIP, "egg_launch_muon_apply", e); break; }
                    }
                    for (int b = 0; b < applied; b++) { const int r2 = refresh_frag(ctx, g[first + b]); if (r2 && !rc) rc = r2; }
                }
                if (rc) return rc;
            }
        }
    UpdParams common = make_upd(ctx, 0, d_fit, d_seed, d_lr);
    { SpanScope span(ctx, EGG_K_UPDATE_VECTOR); HIP_TRY(egg_launch_update_vectors(common, ctx->d_vec_desc, ctx->n_vec, ctx->vec_total, ctx->stream)); }
    // d-eggs runs the overlay rule after each tensor's update (de/src/worker.cu:446-523); tensors and their overlay
    // entries are independent, so one launch over every tensor's segment at the end gives the same values
    if (ctx->adaptive)
        HIP_TRY(egg_launch_overlay_update(ctx->d_overlay, ctx->d_overlay_q, ctx->d_flags, ctx->d_ov_segs, ctx->n_ov_segs,
                                          ctx->ov_max_count, ctx->ov_inc, ctx->ov_dec, ctx->stream));
    return EGG_OK;
}

// ------------------------------------------------------------------ adaptive noise overlay (d-eggs)
// de/src/worker.cu:333 (every overlay value starts at ADAPTIVE_NOISE_INIT), de/include/config.h:229-242 (mode 1,
// +5 / -1 / 64).  From this call on the forward scales every noise term by its overlay factor
// (de/include/model/layers.cuh:12-53) and egg_es_update applies the overlay rule after the AdamW update.
extern "C" int egg_adaptive_enable(egg_ctx *ctx, int init_value, int inc, int dec) {
    if (!ctx || init_value < -127 || init_value > 127 || inc < 0 || dec < 0) return fail(ctx, EGG_E_INVALID, "egg_adaptive_enable arguments");
    if (ctx->cfg.use_muon) return fail(ctx, EGG_E_INVALID, "the adaptive noise overlay is defined for the AdamW update only");
    if (ctx->captured) return fail(ctx, EGG_E_STATE, "enable the overlay before capturing the step");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    const size_t n = (size_t)ctx->L.total;
    if (!ctx->d_overlay) {
        HIP_TRY(hipMalloc(&ctx->d_overlay, n)); HIP_TRY(hipMalloc(&ctx->d_overlay_q, n)); HIP_TRY(hipMalloc(&ctx->d_flags, n));
        std::vector<OvSeg> segs; std::vector<VecDesc> vd; int first = 0;
        for (size_t id = 0; id < ctx->tensors.size(); id++) {
            const egg_tensor_info &t = ctx->tensors[id];
            OvSeg sg; sg.offset = (int)t.offset; sg.count = t.is_matrix ? t.rows + t.cols : t.cols;
            segs.push_back(sg);
            if (sg.count > ctx->ov_max_count) ctx->ov_max_count = sg.count;
            if (t.is_matrix) continue;
            VecDesc d; d.W = ctx->d_model + t.offset; d.state = reinterpret_cast<float *>(ctx->d_state + ctx->t_state_off[id]);
            d.n = t.cols; d.first = first; d.off_a = t.off_a; d.off_b = t.off_b; d.seed_base = t.seed_base; d.lr_scale = t.lr_scale;
            d.flags = ctx->d_flags + t.offset;
            vd.push_back(d); first += t.cols;
        }
        ctx->n_ov_segs = (int)segs.size();
        HIP_TRY(hipMalloc(&ctx->d_ov_segs, segs.size() * sizeof(OvSeg)));
        HIP_TRY(hipMemcpy(ctx->d_ov_segs, segs.data(), segs.size() * sizeof(OvSeg), hipMemcpyHostToDevice));
        HIP_TRY(hipMemcpy(ctx->d_vec_desc, vd.data(), vd.size() * sizeof(VecDesc), hipMemcpyHostToDevice));
    }
    HIP_TRY(hipMemset(ctx->d_overlay, init_value & 0xff, n));
    HIP_TRY(hipMemset(ctx->d_flags, 0, n));
    HIP_TRY(egg_launch_overlay_q(ctx->d_overlay, ctx->d_overlay_q, (int64_t)n, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    ctx->ov_inc = inc; ctx->ov_dec = dec; ctx->adaptive = true;
    return EGG_OK;
}
// The overlay blob has the layout of the model blob: a vector tensor's values at the tensor's offset; a matrix's
// input-row values at its offset and its output-column values right behind them.  Other bytes are not used.
extern "C" int egg_overlay_upload(egg_ctx *ctx, const void *h, size_t bytes) {
    if (!ctx || !h || (int64_t)bytes != ctx->L.total) return fail(ctx, EGG_E_INVALID, "overlay size mismatch");
    if (!ctx->adaptive) return fail(ctx, EGG_E_STATE, "egg_adaptive_enable has not been called");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipMemcpy(ctx->d_overlay, h, bytes, hipMemcpyHostToDevice));
    HIP_TRY(egg_launch_overlay_q(ctx->d_overlay, ctx->d_overlay_q, (int64_t)bytes, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return EGG_OK;
}
extern "C" int egg_overlay_download(egg_ctx *ctx, void *h, size_t bytes) {
    if (!ctx || !h || (int64_t)bytes != ctx->L.total) return fail(ctx, EGG_E_INVALID, "overlay size mismatch");
    if (!ctx->adaptive) return fail(ctx, EGG_E_STATE, "egg_adaptive_enable has not been called");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipMemcpy(h, ctx->d_overlay, bytes, hipMemcpyDeviceToHost));
    return EGG_OK;
}
extern "C" int64_t egg_opt_state_bytes(const egg_ctx *ctx) { return ctx ? ctx->state_bytes : 0; }
extern "C" int64_t egg_tensor_state_offset(const egg_ctx *ctx, int id) {
    return (ctx && id >= 0 && id < (int)ctx->tensors.size()) ? ctx->t_state_off[id] : -1;
}
// Newton-Schulz orthogonalisation of a row-major [rows][cols] fp32 device matrix, in place (test hook for
// perform_newton_schulz, muon_internal.cuh:182-342)
extern "C" int egg_newton_schulz(egg_ctx *ctx, float *d_X, int rows, int cols, int iters) {
    if (!ctx || !d_X || (reinterpret_cast<uintptr_t>(d_X) & 15) || rows < 32 || cols < 32 || rows % 32 || cols % 32)
        return fail(ctx, EGG_E_INVALID, "egg_newton_schulz arguments (a 16-byte aligned matrix with rows and cols multiples of 32)");
    if (!ctx->muon.x) return fail(ctx, EGG_E_STATE, "context was created without use_muon");
    if ((size_t)rows * cols > (size_t)4 * ctx->cfg.hidden * ctx->cfg.hidden || (rows < cols ? rows : cols) > ctx->cfg.hidden)
        return fail(ctx, EGG_E_INVALID, "matrix larger than the Muon workspace");
    MuonWork w = ctx->muon; w.x = d_X;
    HIP_TRY(egg_launch_newton_schulz(w, rows, cols, iters, ctx->stream));
    return EGG_OK;
}
extern "C" int egg_tensor_count(const egg_ctx *ctx) { return ctx ? (int)ctx->tensors.size() : 0; }
extern "C" int egg_tensor_info_get(const egg_ctx *ctx, int id, egg_tensor_info *out) {
    if (!ctx || !out || id < 0 || id >= (int)ctx->tensors.size()) return EGG_E_INVALID;
    *out = ctx->tensors[id];
    return EGG_OK;
}
extern "C" int egg_last_update_count(egg_ctx *ctx, uint64_t *out) {
    if (!ctx || !out) return EGG_E_INVALID;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    unsigned long long v = 0;
    HIP_TRY(hipMemcpy(&v, ctx->d_counter, 8, hipMemcpyDeviceToHost));
    *out = v;
    return EGG_OK;
}

// ------------------------------------------------------------------ whole step
static int enqueue_step(egg_ctx *ctx, const uint8_t *d_data, int64_t len) {
    int rc = forward_range(ctx, d_data, len, &ctx->d_scal->start, &ctx->d_scal->seed, 0, ctx->cfg.population, ctx->d_loss);
    if (rc) return rc;
    HIP_TRY(egg_launch_fitness(ctx->d_loss, ctx->d_fit, ctx->cfg.population / 2, ctx->stream));
    return egg_es_update(ctx, ctx->d_fit, &ctx->d_scal->seed, &ctx->d_scal->lr);
}
extern "C" int egg_step(egg_ctx *ctx, const uint8_t *d_data, int64_t len, int64_t start_idx, uint32_t step_seed, float lr) {
    if (!ctx) return EGG_E_INVALID;
    hipLaunchKernelGGL(k_set_scalars, dim3(1), dim3(1), 0, ctx->stream, ctx->d_scal, step_seed, lr, start_idx);
    HIP_TRY(hipGetLastError());
    return enqueue_step(ctx, d_data, len);
}
extern "C" int egg_step_capture(egg_ctx *ctx, const uint8_t *d_data, int64_t len) {
    if (!ctx) return EGG_E_INVALID;
    if (ctx->captured) return fail(ctx, EGG_E_STATE, "step already captured");
    if (ctx->taps) return fail(ctx, EGG_E_STATE, "disable taps before capturing");
    if (ctx->timing) return fail(ctx, EGG_E_STATE, "disable timing before capturing");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    int rc = enqueue_step(ctx, d_data, len);
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &g);
    if (rc) { if (g) (void)hipGraphDestroy(g); return rc; }
    if (e != hipSuccess) return fail(ctx, EGG_E_HIP, "hipStreamEndCapture", e);
    ctx->graph = g;
    HIP_TRY(hipGraphInstantiate(&ctx->gexec, ctx->graph, nullptr, nullptr, 0));
    ctx->captured = true;
    return EGG_OK;
}
extern "C" int egg_step_launch(egg_ctx *ctx, int64_t start_idx, uint32_t step_seed, float lr) {
    if (!ctx) return EGG_E_INVALID;
    if (!ctx->captured) return fail(ctx, EGG_E_STATE, "egg_step_capture has not been called");
    hipLaunchKernelGGL(k_set_scalars, dim3(1), dim3(1), 0, ctx->stream, ctx->d_scal, step_seed, lr, start_idx);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipGraphLaunch(ctx->gexec, ctx->stream));
    return EGG_OK;
}
extern "C" int egg_step_losses(egg_ctx *ctx, int32_t *h_loss, int32_t *h_fit) {
    if (!ctx) return EGG_E_INVALID;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    if (h_loss) HIP_TRY(hipMemcpy(h_loss, ctx->d_loss, (size_t)ctx->cfg.population * 4, hipMemcpyDeviceToHost));
    if (h_fit) HIP_TRY(hipMemcpy(h_fit, ctx->d_fit, (size_t)(ctx->cfg.population / 2) * 4, hipMemcpyDeviceToHost));
    return EGG_OK;
}

// get_learning_rate (mgpu.cu:217-227)
extern "C" float egg_learning_rate(long step) {
    if (step < 300) return 0.3f;
    if (step < 600) return 0.15f;
    if (step < 1000) return 0.075f;
    return 0.05f;
}
// d-eggs' schedule (d-eggs/include/utils/training.h:5-9)
extern "C" float egg_learning_rate_deggs(long step) {
    if (step < 100) return 0.5f;
    if (step < 200) return 0.25f;
    return 0.125f;
}
// save_model_info (egg_disk_utils.h:15-44, d-eggs/include/utils/io.h:24-53): "<dir>/model.info", the configuration and
// sizes as text.  The reference's sizes are sizeof(TransformerModel) / sizeof(AdamModel): the blob and state sizes here.
extern "C" int egg_model_info_save(egg_ctx *ctx, const char *dir) {
    if (!ctx) return EGG_E_INVALID;
    const std::string d = (dir && *dir) ? dir : "models";
    (void)mkdir(d.c_str(), 0700);
    FILE *f = fopen((d + "/model.info").c_str(), "w");
    if (!f) return fail(ctx, EGG_E_INVALID, "cannot write model.info");
    const egg_config &c = ctx->cfg;
    const long params = (long)ctx->L.total, state = (long)egg_opt_state_bytes(ctx);
    fprintf(f, "Model Configuration:\n");
    fprintf(f, "HIDDEN_DIM: %d\n", c.hidden);
    fprintf(f, "HEAD_DIM: %d\n", c.head_dim);
    fprintf(f, "N_LAYERS: %d\n", c.n_layers);
    fprintf(f, "SEQ_LEN: %d\n", c.seq_len);
    fprintf(f, "VOCAB_SIZE: %d\n", c.vocab);
    fprintf(f, "N_HEADS: %d\n", c.hidden / c.head_dim);
    fprintf(f, "Weight Sharing: Yes\n");
    fprintf(f, "Biases: Embedding(Yes) Output(No)\n");
    fprintf(f, "Model Parameters: %ld (%.2f MB)\n", params, params / (1024.0 * 1024.0));
    fprintf(f, "Adam State Size: %ld (%.2f MB)\n", state, state / (1024.0 * 1024.0));
    fprintf(f, "Population: %d\n", c.population);
    fprintf(f, "Softmax Scale: 2^%d\n", c.softmax_scale_bit);
    return fclose(f) == 0 ? EGG_OK : fail(ctx, EGG_E_INVALID, "cannot write model.info");
}
// current_seed = hash_rng(current_seed, current_step) (d-eggs/src/worker.cu:542)
extern "C" uint32_t egg_next_seed(uint32_t seed, uint64_t step) {
    uint32_t x = seed + (uint32_t)step * 0x9e3779b9u;
    x ^= x >> 16; x *= 0x85ebca6bu; x ^= x >> 13; x *= 0xc2b2ae35u; x ^= x >> 16;
    return x;
}

// ------------------------------------------------------------------ taps
// generate_sequence_kernel (mgpu.cu:1154-1283) and its call site (:1701-1708).  The reference walks the sequence
// token by token with a per-layer KV cache (d_gen_kv).  Here the unperturbed forward of one member (noise mask 0 makes
// every perturbation term vanish, i.e. noise_sign = 0) runs once over the whole window for the prompt and fills every
// layer's K / V rows; each new token then re-evaluates only the 32-token tile that holds position t -- embedding,
// projections, the tile's queries against the cached K / V rows of everything in front of them, MLP, head -- and
// samples from the logits of position t.  Causality makes what position t sees independent of the not yet generated
// tail, and a tile's K / V rows are final once its last position has been generated.  With the cache switched off
// (egg_ctx_generate_kv_cache) every new token re-runs the whole window instead; the tokens are the same.
struct DeggsSampling { float temp; int min_p_limit, penalty_int; };
static int generate_impl(egg_ctx *ctx, uint8_t *d_buffer, int seed_len, int gen_len, uint32_t seed, const DeggsSampling *de) {
    if (!ctx || !d_buffer) return EGG_E_INVALID;
    const egg_config &c = ctx->cfg; const int T = c.seq_len, total = seed_len + gen_len;
    if (seed_len < 1 || gen_len < 0 || total > T) return fail(ctx, EGG_E_INVALID, "egg_generate: need 1 <= seed_len and seed_len + gen_len <= seq_len");
    if (ctx->captured) return fail(ctx, EGG_E_STATE, "egg_generate cannot run on a context whose step is captured");
    const int tb = c.vocab > 256 ? 4 : 1;          // bytes per token of the buffer
    hipStream_t s = ctx->stream;
    if (!ctx->d_gen_tok) {
        HIP_TRY(hipMalloc(&ctx->d_gen_tok, ((size_t)T + 16) * tb));
        HIP_TRY(hipMalloc(&ctx->d_gen_ws, (size_t)2 * c.vocab * 4));
        HIP_TRY(hipMalloc(&ctx->d_gen_logits, (size_t)T * c.vocab * 4));
        HIP_TRY(hipMalloc(&ctx->d_gen_scal, sizeof(Scalars)));
        HIP_TRY(hipMemset(ctx->d_gen_scal, 0, sizeof(Scalars)));
        HIP_TRY(hipMalloc(&ctx->d_gen_kv, (size_t)c.n_layers * 2 * T * c.hidden));
    }
    HIP_TRY(egg_launch_zero_u64(reinterpret_cast<unsigned long long *>(ctx->d_gen_tok), (T + 16) * tb / 8, s));   // a fill kernel, not a memset node: a caller may be capturing this stream
    HIP_TRY(hipMemcpyAsync(ctx->d_gen_tok, d_buffer, (size_t)seed_len * tb, hipMemcpyDeviceToDevice, s));
    int bt = (c.hidden + 31) & ~31; if (bt > 1024) bt = 1024;          // BLOCK_THREADS (mgpu.cu:74-75)
    const bool taps = ctx->taps; ctx->taps = false;
    ctx->mask_override = 0; ctx->logits_override = ctx->d_gen_logits;
    int rc = EGG_OK;
    for (int t = seed_len - 1; t < total - 1 && rc == EGG_OK; t++) {
        // data_len = T + 1 puts the member's stream position at 0 (mgpu.cu:864-870 with len - T == 1)
        FwdRange range = {0, T, ctx->d_gen_kv};
        if (t > seed_len - 1) { range.t0 = t & ~31; range.tn = 32; }       // the prompt: whole window; then the tile of position t
        rc = forward_chunk(ctx, ctx->d_gen_tok, (int64_t)T + 1, &ctx->d_gen_scal->start, &ctx->d_gen_scal->seed, 0, 1,
                           ctx->gen_kv_cache ? &range : nullptr);
        if (rc == EGG_OK) {
            const int32_t *row = ctx->d_gen_logits + (size_t)t * c.vocab;
            uint8_t *next = ctx->d_gen_tok + (size_t)(t + 1) * tb;
            hipError_t e = de ? egg_launch_sample_deggs(row, ctx->d_exp, c.vocab, bt, seed, t, ctx->d_gen_tok, de->temp, de->min_p_limit, de->penalty_int,
                                                        ctx->d_gen_ws, next, tb, s)
                              : egg_launch_sample(row, ctx->d_exp, c.vocab, bt, seed, t, ctx->d_gen_ws, next, tb, s);
            if (e != hipSuccess) rc = fail(ctx, EGG_E_HIP, "egg_launch_sample", e);
        }
    }
    ctx->mask_override = -1; ctx->logits_override = nullptr; ctx->taps = taps;
    if (rc) return rc;
    HIP_TRY(hipMemcpyAsync(d_buffer, ctx->d_gen_tok, (size_t)total * tb, hipMemcpyDeviceToDevice, s));
    return EGG_OK;
}
extern "C" int egg_ctx_generate_kv_cache(egg_ctx *ctx, int enable) {
    if (!ctx) return EGG_E_INVALID;
    ctx->gen_kv_cache = enable != 0;
    return EGG_OK;
}
extern "C" int egg_generate(egg_ctx *ctx, uint8_t *d_buffer, int seed_len, int gen_len, uint32_t seed) {
    return generate_impl(ctx, d_buffer, seed_len, gen_len, seed, nullptr);
}
// float -> int32 as the reference's GPU converts it: truncation, saturation at the ends, NaN -> 0
static int sat_d2i(double x) {
    if (x != x) return 0;
    if (x >= 2147483648.0) return INT32_MAX;
    if (x <= -2147483648.0) return INT32_MIN;
    return (int)x;
}
// penalty_int = (int32_t)(penalty * (1 << SHIFT_LOGIT)) in float, min_p_limit = (int32_t)(logf(min_p) * SOFTMAX_EXP_SCALE)
// in double (d-eggs/src/kernels.cu:386-387)
extern "C" int egg_deggs_sampling_constants(const egg_config *cfg, float min_p, float penalty, int32_t *penalty_int, int32_t *min_p_limit) {
    if (!cfg || !penalty_int || !min_p_limit || cfg->shift_logit < 0 || cfg->shift_logit > 30) return EGG_E_INVALID;
    *penalty_int = sat_d2i((double)(penalty * (float)(1 << cfg->shift_logit)));
    // logf(0) = -inf saturates to INT32_MIN (nothing is filtered); logf of a negative number is NaN, which the GPU's
    // conversion turns into 0 (every token below the maximum is filtered)
    *min_p_limit = sat_d2i((double)logf(min_p) * cfg->softmax_exp_scale);
    return EGG_OK;
}
extern "C" int egg_generate_deggs(egg_ctx *ctx, uint8_t *d_buffer, int seed_len, int gen_len, uint32_t seed, float temp, float min_p, float penalty) {
    if (!ctx || !d_buffer) return EGG_E_INVALID;
    int bt = (ctx->cfg.hidden + 31) & ~31; if (bt > 1024) bt = 1024;
    // the reference keeps the tokens for the penalty in a 256-entry shared array that its first min(seed_len, block size)
    // threads fill: beyond either limit it reads memory nobody wrote
    if (seed_len + gen_len > 256 || seed_len > bt)
        return fail(ctx, EGG_E_INVALID, "egg_generate_deggs: need seed_len + gen_len <= 256 and seed_len <= the reference's block size (hidden rounded up to 32)");
    DeggsSampling de; de.temp = temp;
    int rc = egg_deggs_sampling_constants(&ctx->cfg, min_p, penalty, &de.penalty_int, &de.min_p_limit);
    if (rc) return fail(ctx, rc, "egg_generate_deggs: configuration");
    return generate_impl(ctx, d_buffer, seed_len, gen_len, seed, &de);
}

extern "C" int egg_ctx_enable_taps(egg_ctx *ctx, int enable) {
    if (!ctx) return EGG_E_INVALID;
    if (ctx->captured) return fail(ctx, EGG_E_STATE, "taps cannot change after capture");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    if (enable && !ctx->d_tap) {
        const egg_config &c = ctx->cfg;
        ctx->tap_members = ctx->chunk < 64 ? ctx->chunk : 64;
        size_t one = (size_t)ctx->tap_members * c.seq_len * c.hidden;
        HIP_TRY(hipMalloc(&ctx->d_tap, one * (1 + 6 * c.n_layers)));
        HIP_TRY(hipMalloc(&ctx->d_tap_logits, (size_t)ctx->tap_members * c.seq_len * c.vocab * 4));
    }
    ctx->taps = enable != 0;
    return EGG_OK;
}
extern "C" int egg_ctx_first_block_dedup(egg_ctx *ctx, int enable) {
    if (!ctx) return EGG_E_INVALID;
    if (ctx->captured) return fail(ctx, EGG_E_STATE, "the first block's form cannot change after capture");
    ctx->first_dedup = enable != 0;
    return EGG_OK;
}
extern "C" int egg_tap_download(egg_ctx *ctx, const char *name, int member, void *host_out) {
    if (!ctx || !name || !host_out || !ctx->d_tap || member < 0 || member >= ctx->tap_members) return fail(ctx, EGG_E_INVALID, "egg_tap_download arguments");
    const egg_config &c = ctx->cfg; const int T = c.seq_len, H = c.hidden;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    if (!strcmp(name, "logits")) {
        HIP_TRY(hipMemcpy(host_out, ctx->d_tap_logits + (size_t)member * T * c.vocab, (size_t)T * c.vocab * 4, hipMemcpyDeviceToHost));
        return EGG_OK;
    }
    int slot = -1, layer = 0; char base[32] = {0};
    const char *dot = strchr(name, '.');
    if (dot) { size_t n = (size_t)(dot - name); if (n >= sizeof(base)) return EGG_E_INVALID; memcpy(base, name, n); layer = atoi(dot + 1); }
    else snprintf(base, sizeof(base), "%s", name);
    if (layer < 0 || layer >= c.n_layers) return fail(ctx, EGG_E_INVALID, "tap layer");
    const char *names[6] = {"q", "k", "v", "ao", "x_attn", "x_mlp"};
    if (!strcmp(base, "x_init")) slot = 0;
    else for (int i = 0; i < 6; i++) if (!strcmp(base, names[i])) slot = 1 + 6 * layer + i;
    if (slot < 0) return fail(ctx, EGG_E_INVALID, "unknown tap name");
    std::vector<int8_t> buf((size_t)T * H);
    HIP_TRY(hipMemcpy(buf.data(), tap_ptr(ctx, slot) + (size_t)member * T * H, buf.size(), hipMemcpyDeviceToHost));
    int8_t *o = (int8_t *)host_out;
    for (int t = 0; t < T; t++)
        for (int n = 0; n < H; n++) {
            int w = n & 31, q = w >> 3, g = (w >> 2) & 1, e = w & 3;
            o[(size_t)t * H + n] = buf[(size_t)t * H + (n & ~31) + 16 * g + 4 * q + e];
        }
    return EGG_OK;
}

// ------------------------------------------------------------------ per-kernel timing
extern "C" int egg_ctx_enable_timing(egg_ctx *ctx, int enable) {
    if (!ctx) return EGG_E_INVALID;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    spans_collect(ctx);
    ctx->timing = enable != 0;
    return EGG_OK;
}
extern "C" int egg_timing_reset(egg_ctx *ctx) {
    if (!ctx) return EGG_E_INVALID;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    ctx->spans_used = 0;
    for (int i = 0; i < EGG_KCLASS_COUNT; i++) { ctx->t_ms[i] = 0; ctx->t_n[i] = 0; }
    return EGG_OK;
}
extern "C" int egg_timing_get(egg_ctx *ctx, int kclass, int64_t *launches, double *total_ms) {
    if (!ctx || kclass < 0 || kclass >= EGG_KCLASS_COUNT) return EGG_E_INVALID;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    spans_collect(ctx);
    if (launches) *launches = ctx->t_n[kclass];
    if (total_ms) *total_ms = ctx->t_ms[kclass];
    return EGG_OK;
}

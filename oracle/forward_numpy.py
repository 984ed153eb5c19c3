"""A second, independent restatement of the Int8NativeFormer forward (full_cuda_train_transformer_adam_mgpu.cu) in
numpy.  TEST INFRASTRUCTURE ONLY: it exists so that the composition of the whole forward is stated twice, in two
different shapes -- the C++ oracle walks one token at a time with a K/V cache and a loop per reference thread, this
one evaluates every stage for all tokens of the window at once as integer matrix products -- and the tests require
the two to agree bit for bit.  Nothing here is shared with the C++ oracle except the lookup tables (pinned by closed
forms) and the tensor offsets (pinned by the init-stream test).

Each function cites the reference lines it follows."""
import numpy as np

# seed offsets, mgpu.cu:114-165
OFF = dict(EMB=0, EMB_BIAS=(50, 51), LN_1=(100, 101), LN_1_BIAS=(110, 111), Q=(200, 201), K=(202, 203), V=(204, 205),
           O=(206, 207), LN_2=(300, 301), LN_2_BIAS=(310, 311), MLP_UP=(400, 401), MLP_DOWN=(402, 403),
           MLP_BIAS_UP=(410, 411), MLP_BIAS_DOWN=(412, 413), LN_INIT=(500, 501), LN_INIT_BIAS=(502, 503),
           EMB_MLP_UP=(510, 511), EMB_MLP_DOWN=(512, 513), EMB_MLP_BIAS_UP=(514, 515), EMB_MLP_BIAS_DOWN=(516, 517),
           LN_F=(900, 901), LN_F_BIAS=(910, 911))
M32 = np.uint64(0xFFFFFFFF)


def noise(seed, idx, cfg):
    """hash_rng + noise_from_hash, mgpu.cu:525-538: murmur3 fmix32 of seed + idx * 0x9e3779b9; a field is a sign bit
    followed by the masked magnitude; DEVICE_GAUSSIAN adds the fields that start at bits 5 and 10 to the one at bit 0.
    cfg is the configuration, or a plain magnitude mask."""
    mask, gaussian = (cfg, 0) if isinstance(cfg, int) else (cfg.noise_mask, cfg.device_gaussian)
    x = (np.uint64(int(seed) & 0xFFFFFFFF) + np.asarray(idx, np.uint64) * np.uint64(0x9E3779B9)) & M32
    x ^= x >> np.uint64(16); x = (x * np.uint64(0x85EBCA6B)) & M32
    x ^= x >> np.uint64(13); x = (x * np.uint64(0xC2B2AE35)) & M32
    x ^= x >> np.uint64(16)
    total = 0
    for start in ((0, 5, 10) if gaussian else (0,)):
        f = x >> np.uint64(start)
        mag = ((f >> np.uint64(1)) & np.uint64(mask)).astype(np.int64)
        total = total + np.where((f & np.uint64(1)) != 0, mag, -mag)
    return total


def clip(a):
    """clip, mgpu.cu:540-541"""
    return np.clip(a, -127, 127)


def trunc_div(a, b):
    """C integer division (toward zero) of int64 arrays"""
    q = np.abs(a) // np.abs(b)
    return np.where((a < 0) != (b < 0), -q, q)


def unblock(blob, rows, cols):
    """repack_matrix read backwards, mgpu.cu:443-459: logical W[k][n] sits at ((k // 4) * cols + n) * 4 + k % 4"""
    k = np.arange(rows)[:, None]
    n = np.arange(cols)[None, :]
    return blob[((k >> 2) * cols + n) * 4 + (k & 3)].astype(np.int64)


def standard_norm(cfg, x, w, b, seed, off_w, off_b, ns):
    """apply_standard_norm, mgpu.cu:646-678; x is [T, H]"""
    H = x.shape[1]
    h = np.arange(H)
    mn = np.abs(x).sum(axis=1) // H
    mn = np.where(mn == 0, 1, mn)[:, None]
    w_mod = w.astype(np.int64) + ((noise(seed + off_w[0], h, cfg) * noise(seed + off_w[1], h, cfg) * ns) >> cfg.sigma_shift_vector)
    b_mod = b.astype(np.int64) + ((noise(seed + off_b[0], h, cfg) * noise(seed + off_b[1], h, cfg) * ns) >> cfg.sigma_shift_vector)
    return clip(trunc_div(x * w_mod[None, :], mn) + b_mod[None, :])


def adaptive_normalize(val):
    """adaptive_qkv_normalize / adaptive_layer_normalize, egg_adaptive_normalize.h:10-103: float32 scale, lroundf"""
    m = np.abs(val).max(axis=1)
    scale = np.float32(127.0) / (m.astype(np.float32) + np.float32(1e-9))
    y = (val.astype(np.float32) * scale[:, None]).astype(np.float64)          # the float32 product, then exact
    r = np.where(y >= 0, np.floor(y + 0.5), np.ceil(y - 0.5)).astype(np.int64)
    return np.clip(r, -127, 127)


def linear(cfg, x, W, seed, off, ns):
    """compute_linear_projection, mgpu.cu:553-572, for all tokens: x [T, K], W [K, N] logical"""
    K, N = W.shape
    acc = x @ W
    if ns != 0:
        sb = x @ noise(seed + off[1], np.arange(K), cfg)
        a = noise(seed + off[0], np.arange(N), cfg)
        acc = acc + ((sb[:, None] * a[None, :] * ns) >> (cfg.fixed_point + cfg.sigma_shift))
    return acc


def rope(cfg, val, lut):
    """apply_rope_integer, mgpu.cu:624-644; val [T, H] raw accumulators, lut [T, head_dim] (cos, sin) pairs"""
    T, H = val.shape
    hd = cfg.head_dim
    pair = (np.arange(H) % hd) // 2
    c = lut[:, 2 * pair].astype(np.int64)
    s = lut[:, 2 * pair + 1].astype(np.int64)
    even = val[:, 0::2]
    odd = val[:, 1::2]
    half = 1 << (cfg.rope_scale_bit - 1)
    out = np.empty_like(val)
    out[:, 0::2] = (even * c[:, 0::2] - odd * s[:, 0::2] + half) >> cfg.rope_scale_bit
    out[:, 1::2] = (even * s[:, 1::2] + odd * c[:, 1::2] + half) >> cfg.rope_scale_bit
    return out


def attention(cfg, q, k, v, exp_lut):
    """the attention core of compute_attention, mgpu.cu:787-824, per head with a causal mask"""
    T, H = q.shape
    hd = cfg.head_dim
    out = np.zeros((T, H), np.int64)
    causal = np.tril(np.ones((T, T), bool))
    lutv = exp_lut.astype(np.int64)
    for h0 in range(0, H, hd):
        s = q[:, h0:h0 + hd] @ k[:, h0:h0 + hd].T                       # [t, ctx]
        mx = np.where(causal, s, np.iinfo(np.int64).min).max(axis=1)
        idx = np.clip((mx[:, None] >> cfg.shift_attn) - (s >> cfg.shift_attn), 0, 255)
        w = np.where(causal, lutv[idx], 0)
        num = w @ v[:, h0:h0 + hd]
        den = w.sum(axis=1)
        den = np.where(den == 0, 1, den)[:, None]
        out[:, h0:h0 + hd] = clip(trunc_div(num, den))
    return out


def mlp_block(cfg, x, t, seed, ns, act_lut, names, offs):
    """compute_mlp, mgpu.cu:708-759; names / offs select the initial MLP or a layer's MLP"""
    ln_w, ln_b, w_up, b_up, w_dn, b_dn = names
    o_ln, o_lnb, o_up, o_bup, o_dn, o_bdn = offs
    H = cfg.hidden
    nrm = standard_norm(cfg, x, t[ln_w], t[ln_b], seed, o_ln, o_lnb, ns)
    a = linear(cfg, nrm, t[w_up], seed, o_up, ns)
    o = np.arange(4 * H)
    nv = (noise(seed + o_bup[0], o, cfg) * noise(seed + o_bup[1], o, cfg) * ns) >> cfg.sigma_shift_vector
    pre = clip((a >> cfg.shift_mlp_up) + t[b_up].astype(np.int64)[None, :] + nv[None, :])
    mid = act_lut.astype(np.int64)[pre & 0xFF]                          # ACT_LUT[(uint8_t)clip(...)]
    adn = linear(cfg, mid, t[w_dn], seed, o_dn, ns)
    hh = np.arange(H)
    nv = (noise(seed + o_bdn[0], hh, cfg) * noise(seed + o_bdn[1], hh, cfg) * ns) >> cfg.sigma_shift_vector
    return adaptive_normalize(x + (adn >> cfg.shift_mlp_down) + t[b_dn].astype(np.int64)[None, :] + nv[None, :])


def forward_member(cfg, model, tensor_table, tables, data, start_idx, step_seed, p_idx):
    """train_sequence_kernel for one member, mgpu.cu:847-1029.  Returns (loss, stages) with the residual stream after
    the initial MLP and after every attention / MLP block, and the logits, for all tokens."""
    exp_lut, act_lut, rope_lut = tables
    H, V, T, NL = cfg.hidden, cfg.vocab, cfg.seq_len, cfg.n_layers
    rope_lut = np.asarray(rope_lut).reshape(T, cfg.head_dim)
    t = {}
    for e in tensor_table:
        blob = model[e["offset"]:e["offset"] + e["rows"] * e["cols"]]
        t[e["name"]] = unblock(blob, e["rows"], e["cols"]) if e["is_matrix"] else blob.astype(np.int64)
    pair = p_idx // 2
    ns = 1 if p_idx % 2 == 0 else -1
    stride = len(data) // (cfg.population // 2)
    pos = (start_idx + (0 if cfg.use_same_data else pair * stride)) % (len(data) - T)       # mgpu.cu:864-870
    tok = data[pos:pos + T].astype(np.int64)
    target = data[pos + 1:pos + T + 1].astype(np.int64)
    pseed = (step_seed + pair) & 0xFFFFFFFF
    hh = np.arange(H)
    # embedding, mgpu.cu:901-931
    E = t["embedding"]                                                                      # [H, V]
    chk = (noise(pseed + OFF["EMB_BIAS"][0], hh, cfg) * noise(pseed + OFF["EMB_BIAS"][1], hh, cfg) * ns) >> cfg.sigma_shift_vector
    a_tok = noise(pseed + OFF["EMB"], tok, cfg)
    b_dim = noise(pseed + OFF["EMB"] + H, hh, cfg)
    perturb = (a_tok[:, None] * b_dim[None, :] * ns) >> (cfg.fixed_point + cfg.sigma_shift)
    x = clip(E[:, tok].T + t["emb_bias"][None, :] + chk[None, :] + perturb)
    x = mlp_block(cfg, x, t, pseed, ns, act_lut,
                  ("ln_init", "ln_init_bias", "w_emb_mlp_up", "mlp_emb_bias_up", "w_emb_mlp_down", "mlp_emb_bias_down"),
                  (OFF["LN_INIT"], OFF["LN_INIT_BIAS"], OFF["EMB_MLP_UP"], OFF["EMB_MLP_BIAS_UP"], OFF["EMB_MLP_DOWN"], OFF["EMB_MLP_BIAS_DOWN"]))
    stages = {"x_init": x.copy(), "x_attn": [], "x_mlp": []}
    for l in range(NL):
        sb = (pseed + 1000 * l) & 0xFFFFFFFF                                                # mgpu.cu:938
        nrm = standard_norm(cfg, x, t[f"ln_1.{l}"], t[f"ln_1_bias.{l}"], sb, OFF["LN_1"], OFF["LN_1_BIAS"], ns)
        q = adaptive_normalize(rope(cfg, linear(cfg, nrm, t[f"w_q.{l}"], sb, OFF["Q"], ns), rope_lut))
        k = adaptive_normalize(rope(cfg, linear(cfg, nrm, t[f"w_k.{l}"], sb, OFF["K"], ns), rope_lut))
        v = adaptive_normalize(linear(cfg, nrm, t[f"w_v.{l}"], sb, OFF["V"], ns))
        ao = attention(cfg, q, k, v, exp_lut)
        aco = linear(cfg, ao, t[f"w_o.{l}"], sb, OFF["O"], ns)
        x = adaptive_normalize(x + (aco >> cfg.shift_out))
        stages["x_attn"].append(x.copy())
        x = mlp_block(cfg, x, t, sb, ns, act_lut,
                      (f"ln_2.{l}", f"ln_2_bias.{l}", f"w_up.{l}", f"mlp_bias_up.{l}", f"w_down.{l}", f"mlp_bias_down.{l}"),
                      (OFF["LN_2"], OFF["LN_2_BIAS"], OFF["MLP_UP"], OFF["MLP_BIAS_UP"], OFF["MLP_DOWN"], OFF["MLP_BIAS_DOWN"]))
        stages["x_mlp"].append(x.copy())
    # head and loss, mgpu.cu:955-1024
    nf = standard_norm(cfg, x, t["ln_f"], t["ln_f_bias"], pseed, OFF["LN_F"], OFF["LN_F_BIAS"], ns)
    acc = nf @ E
    sbh = nf @ noise(pseed + OFF["EMB"] + H, hh, cfg)
    acc = acc + ((sbh[:, None] * noise(pseed + OFF["EMB"], np.arange(V), cfg)[None, :] * ns) >> (cfg.fixed_point + cfg.sigma_shift))
    logits = acc >> cfg.shift_logit
    G = logits.max(axis=1)
    S = exp_lut.astype(np.int64)[np.clip(G[:, None] - logits, 0, 255)].sum(axis=1)
    posn = np.array([int(s).bit_length() - 1 for s in S], np.int64)                        # floor(log2 S), S >= 2^18
    log_sum = (posn << 4) - (cfg.softmax_scale_bit << 4)
    loss_t = (log_sum >> 1) + G - logits[np.arange(T), target]
    total = int(loss_t.sum())
    stages["logits"] = logits
    return ((total + 2 ** 31) % 2 ** 32) - 2 ** 31, stages                                   # (int32) my_loss


def es_update_adam(cfg, model, state, tensor_table, fit, step_seed, lr):
    """The AdamW ES update of every tensor, mgpu.cu:1040-1152 and the launch list :1603-1643, with numpy: votes as
    integer matrix products over the pairs, AdamW in float32 array arithmetic (one rounding per operation).  `state` is a
    structured array with float32 fields m, v, acc per model byte.  In place; returns the number of changed weights."""
    f32 = np.float32
    pairs = cfg.population // 2
    fit = np.asarray(fit, np.int64)
    p = np.arange(pairs)
    changed = 0
    for e in tensor_table:
        n = e["rows"] * e["cols"]
        sl = slice(e["offset"], e["offset"] + n)
        seeds = (step_seed + p + e["seed_base"]) & 0xFFFFFFFF
        if e["is_matrix"]:
            # A[p, n_out], B[p, k_in]; vote[k, n] = sum_p fit_p * A[p, n] * B[p, k]   (mgpu.cu:1092-1098)
            A = np.stack([noise(int(s) + e["off_a"], np.arange(e["cols"]), cfg) for s in seeds])
            B = np.stack([noise(int(s) + e["off_b"], np.arange(e["rows"]), cfg) for s in seeds])
            vote_kn = (B * fit[:, None]).T @ A
            # blocked element index -> (k, n), mgpu.cu:1085-1089
            idx = np.arange(n)
            vote = vote_kn[(idx >> 2) // e["cols"] * 4 + (idx & 3), (idx >> 2) % e["cols"]]
        else:
            i = np.arange(n)
            n1 = np.stack([noise(int(s) + e["off_a"], i, cfg) for s in seeds])
            n2 = np.stack([noise(int(s) + e["off_b"], i, cfg) for s in seeds])
            vote = (fit[:, None] * n1 * n2).sum(axis=0)
        # apply_adam_update, mgpu.cu:1040-1064 (no bias correction; fractional accumulator moves the int8 weight)
        g = -(vote.astype(f32))
        w = model[sl].astype(np.int64)
        m, v, acc = state["m"][sl], state["v"][sl], state["acc"][sl]
        b1, b2 = f32(cfg.adam_beta1), f32(cfg.adam_beta2)
        m = b1 * m + (f32(1.0) - b1) * g
        v = b2 * v + (f32(1.0) - b2) * (g * g)
        step = (-f32(lr * e["lr_scale"])) * (m / (np.sqrt(v) + f32(cfg.adam_eps)) + f32(cfg.adam_weight_decay) * w.astype(f32))
        acc = acc + step
        up, dn = acc >= f32(1.0), acc <= f32(-1.0)
        w_new = np.where(up & (w < 127), w + 1, np.where(dn & (w > -127), w - 1, w))
        acc = np.where(up, np.where(w < 127, acc - f32(1.0), f32(1.0)), np.where(dn, np.where(w > -127, acc + f32(1.0), f32(-1.0)), acc)).astype(f32)
        changed += int(np.count_nonzero(w_new != w))
        model[sl] = w_new.astype(np.int8)
        state["m"][sl], state["v"][sl], state["acc"][sl] = m, v, acc
    return changed

"""A second restatement of the reference's CPU program (full_trained_egg.c, "egg.c" below) in numpy.
TEST INFRASTRUCTURE ONLY: nothing outside tests/ may import it.

It shares no code with egg_gru_oracle.cpp: the model is a dict of named arrays in the shapes egg.c:42-50 declares
rather than one blob with offsets, the noise stream is produced a whole vector at a time, matrices are applied as
matrix-vector products in int64 and the vote is one (rows x pairs) @ (pairs x cols) product.  A test requires the two
restatements to agree on every noise vector, matrix product, loss, recurrent state and updated weight; a slip in
either (a seed offset, the four discarded draws, a shift, the order of the clipped adds, the state a gate reads)
shows up as a disagreement.
"""
import numpy as np

MAX_VAL, MIN_VAL = 127, -127   # egg.c:21-22
M32 = 0xFFFFFFFF


def xorshift32(s):
    """egg.c:69-77; returns the new state, which is also the draw"""
    s ^= (s << 13) & M32
    s ^= s >> 17
    s ^= (s << 5) & M32
    return s


def noise_vector(state, count):
    """egg.c:87-105: before every block of 16 outputs four draws are thrown away; the padded tail of the last block
    draws nothing.  An output is +-((r >> 1) & 31), positive when bit 0 of the draw is set (egg.c:79-82).
    Returns (vector, new state)."""
    out = np.zeros(count, np.int64)
    for base in range(0, count, 16):
        for _ in range(4):
            state = xorshift32(state)
        for i in range(base, min(base + 16, count)):
            state = xorshift32(state)
            mag = (state >> 1) & 31
            out[i] = mag if state & 1 else -mag
    return out, state


def clip(v):
    return np.clip(v, MIN_VAL, MAX_VAL)


def model_views(cfg, blob):
    """the fields of EggModel (egg.c:42-50) as views of one int8 blob in declaration order"""
    H, V, NL = cfg.hidden, cfg.vocab, cfg.n_layers
    shapes = [("embedding", (V, H)), ("gru_weights", (NL, 4, H, H)), ("gru_biases", (NL, 2, H)),
              ("mlp_weights", (NL, 2, H * 4 * H)), ("head", (V, H)), ("ln_weights", (NL, 2, H)), ("ln_out", (H,))]
    out, o = {}, 0
    for name, shp in shapes:
        n = int(np.prod(shp))
        out[name] = blob[o:o + n].reshape(shp)
        o += n
    assert o == blob.size
    return out


def matmul_perturbed(cfg, x, w, rows, cols, layer_seed, noise_sign, shift):
    """egg.c:108-177: out[r] = clip((sum_c x[c] W[r][c] + ((x.B) A[r] sign >> (fixed_point + sigma_shift))) >> shift);
    A (rows) is drawn before B (cols) from one stream seeded with layer_seed; >> is arithmetic"""
    A, st = noise_vector(layer_seed & M32, rows)
    B, _ = noise_vector(st, cols)
    x = x.astype(np.int64)
    acc = w.reshape(rows, cols).astype(np.int64) @ x
    if noise_sign != 0:
        xB = int(x @ B)
        acc = acc + ((xB * A * noise_sign) >> (cfg.fixed_point + cfg.sigma_shift))
    return clip(acc >> shift)


def trunc_div(a, b):
    q = np.abs(a) // b
    return np.where(a < 0, -q, q)


def ln(x, w):
    """egg.c:180-210: divide x*w by the mean absolute value (integer division truncating toward zero)"""
    s = int(np.abs(x).sum()) or 1
    mean = s // x.size or 1
    return clip(trunc_div(x.astype(np.int64) * w.astype(np.int64), mean))


def exp2_table(fixed_point):
    """egg.c:57-60"""
    return np.array([int(2.0 ** (i / float(1 << fixed_point)) * (1 << fixed_point)) for i in range(256)], np.int64)


def log2_fixed(x):
    """egg.c:309-319: 16*log2(x) with a linear mantissa, minus 64"""
    if x <= 0:
        return 0
    k = x.bit_length() - 1
    frac = (x - (1 << k)) >> (k - 4) if k >= 4 else (x - (1 << k)) << (4 - k)
    return (k << 4) + frac - 64


def compute_loss(tab, logits, target):
    """egg.c:321-330"""
    s = int(tab[np.clip(logits + 128, 0, 255)].sum())
    return log2_fixed(s) - (int(logits[target]) + 128)


def forward(cfg, model, inputs, targets, step_seed, noise_sign, h):
    """egg.c:213-296.  h[n_layers][hidden] is the recurrent state, updated in place.
    Returns (accumulated loss, last logits)."""
    H, V = cfg.hidden, cfg.vocab
    tab = exp2_table(cfg.fixed_point)
    loss, logits = 0, None
    mm = lambda x, w, r, c, seed, sh: matmul_perturbed(cfg, x, w, r, c, seed, noise_sign, sh)
    for t in range(len(inputs)):
        x = model["embedding"][inputs[t]].astype(np.int64)
        for l in range(cfg.n_layers):
            seed = step_seed + 100 * l
            gw, gb, mw, lw = model["gru_weights"][l], model["gru_biases"][l].astype(np.int64), model["mlp_weights"][l], model["ln_weights"][l]
            res = x
            x = ln(x, lw[0])
            hl = h[l].astype(np.int64)
            ft = clip(clip(mm(x, gw[0], H, H, seed + 1, 8) + mm(hl, gw[1], H, H, seed + 2, 8)) + gb[0])
            # the gate acts on the old state; the product is narrowed to int8 like the reference's cast
            gated = (((ft + 127) * hl) >> 8).astype(np.int8).astype(np.int64)
            ht = clip(clip(mm(x, gw[2], H, H, seed + 3, 8) + mm(gated, gw[3], H, H, seed + 4, 8)) + gb[1])
            hl = clip(hl + (((ft + 127) * (ht - hl)) >> 8))
            h[l] = hl
            x = clip(hl + res)
            res = x
            x = ln(x, lw[1])
            up = mm(x, mw[0], 4 * H, H, seed + 5, 8)
            x = clip(mm(up, mw[1], H, 4 * H, seed + 6, 9) + res)
        x = ln(x, model["ln_out"])
        logits = mm(x, model["head"], V, H, step_seed + 999, 8)
        if targets is not None:
            loss += compute_loss(tab, logits, int(targets[t]))
    return loss, logits


def population(cfg, model, data, start_idx, step_seed, states):
    """egg.c:547-562: pair p reads the stream at (start + p * stride) mod (len - seq_len) and evaluates +noise then -noise
    with seed step_seed + p, each with its own recurrent state (states[2p], states[2p+1]).
    Returns (loss[population], fit[pairs])."""
    pairs = cfg.population // 2
    loss = np.zeros(cfg.population, np.int64)
    fit = np.zeros(pairs, np.int64)
    stride = len(data) // pairs
    for p in range(pairs):
        i = (start_idx + p * stride) % (len(data) - cfg.seq_len)
        inp, tgt = data[i:i + cfg.seq_len], data[i + 1:i + 1 + cfg.seq_len]
        loss[2 * p], _ = forward(cfg, model, inp, tgt, step_seed + p, 1, states[2 * p])
        loss[2 * p + 1], _ = forward(cfg, model, inp, tgt, step_seed + p, -1, states[2 * p + 1])
        fit[p] = np.sign(loss[2 * p + 1] - loss[2 * p])
    return loss, fit


def update_matrix(cfg, w, rows, cols, seed, fit):
    """egg.c:332-409: vote[r][c] = sum_p fit[p] A_p[r] B_p[c]; a weight moves one step toward the vote's sign when
    |vote| exceeds the threshold, and never leaves [-127, 127]"""
    pairs = len(fit)
    A = np.zeros((pairs, rows), np.int64)
    B = np.zeros((pairs, cols), np.int64)
    for p in range(pairs):
        A[p], st = noise_vector((seed + p) & M32, rows)
        B[p], _ = noise_vector(st, cols)
    votes = (A * np.asarray(fit, np.int64)[:, None]).T @ B
    W = w.reshape(rows, cols)
    step = np.where((votes > cfg.update_threshold) & (W < MAX_VAL), 1, 0) - np.where((votes < -cfg.update_threshold) & (W > MIN_VAL), 1, 0)
    W += step.astype(np.int8)


def update_sites(cfg, model):
    """egg.c:564-574: (matrix view, rows, cols, seed offset from step_seed) of every matrix the update touches: the
    four GRU matrices and two MLP matrices of every layer, then the head; embedding, biases and norm gains are never
    updated"""
    H = cfg.hidden
    for l in range(cfg.n_layers):
        for g in range(4):
            yield model["gru_weights"][l][g], H, H, 100 * l + 1 + g
        yield model["mlp_weights"][l][0], 4 * H, H, 100 * l + 5
        yield model["mlp_weights"][l][1], H, 4 * H, 100 * l + 6
    yield model["head"], cfg.vocab, H, 999


def update_all(cfg, model, step_seed, fit):
    """egg.c:564-574"""
    for w, rows, cols, off in update_sites(cfg, model):
        update_matrix(cfg, w, rows, cols, step_seed + off, fit)

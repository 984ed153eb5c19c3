"""ctypes binding of the CPU oracle (oracle/libegg_oracle.so) and of oracle/_ref.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py -- never by the product path.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libegg_oracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libegg_ref.so")


class OrcConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "hidden", "head_dim", "n_layers", "seq_len", "vocab", "population",
        "fixed_point", "sigma_shift", "sigma_shift_vector",
        "shift_attn", "shift_out", "shift_logit", "shift_mlp_up", "shift_mlp_down",
        "softmax_scale_bit", "rope_scale_bit", "noise_mask", "host_mask")] + [
        ("softmax_exp_scale", C.c_double),
        ("adam_beta1", C.c_float), ("adam_beta2", C.c_float), ("adam_eps", C.c_float),
        ("adam_weight_decay", C.c_float), ("muon_momentum", C.c_float), ("muon_lr_scale", C.c_float),
        ("weight_limit", C.c_int), ("device_gaussian", C.c_int), ("host_gaussian", C.c_int), ("use_same_data", C.c_int)]


class OrcTensor(C.Structure):
    _fields_ = [("name", C.c_char * 32), ("is_matrix", C.c_int), ("rows", C.c_int), ("cols", C.c_int),
                ("offset", C.c_int64), ("off_a", C.c_int), ("off_b", C.c_int), ("seed_base", C.c_int),
                ("lr_scale", C.c_float), ("muon", C.c_int)]


class OrcTrace(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("x_emb", "x_init", "q", "k", "v", "ao", "x_attn", "x_mlp",
                                          "nf", "logits", "loss_t")]


class OrcGruConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("hidden", "n_layers", "seq_len", "vocab", "population",
                                       "fixed_point", "sigma_shift", "update_threshold")]


def build(force=False):
    """(Re)build the oracle library with oracle/Makefile."""
    if force or not os.path.exists(LIB_PATH):
        subprocess.check_call(["make", "-C", HERE, "-s"] + (["-B"] if force else []))


_lib = None
_ref = None


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(LIB_PATH)
        L.orc_hash_rng.restype = C.c_uint32
        L.orc_hash_rng.argtypes = [C.c_uint32, C.c_uint32]
        L.orc_noise.restype = C.c_int8
        L.orc_noise.argtypes = [C.c_uint32, C.c_uint32, C.c_int]
        L.orc_xorshift32.restype = C.c_uint32
        L.orc_gen_noise_host.restype = C.c_int8
        L.orc_clip.restype = C.c_int8
        L.orc_clip.argtypes = [C.c_int32]
        L.orc_model_bytes.restype = C.c_int64
        L.orc_forward_member.restype = C.c_int32
        L.orc_forward_member.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_uint32,
                                         C.c_int, C.c_int, C.c_void_p]
        L.orc_population_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_uint32,
                                             C.c_int, C.c_int, C.c_void_p]
        L.orc_perturbed_linear.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_int,
                                           C.c_uint32, C.c_int, C.c_int, C.c_int, C.c_void_p]
        L.orc_standard_norm.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_uint32,
                                        C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
        L.orc_adaptive_normalize.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
        L.orc_rope.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        L.orc_attention_core.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                         C.c_void_p]
        L.orc_token_loss.restype = C.c_int64
        L.orc_token_loss.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int]
        L.orc_fitness.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        L.orc_adam_apply.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_float, C.c_void_p]
        L.orc_matrix_votes.restype = C.c_int64
        L.orc_matrix_votes.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int,
                                       C.c_uint32, C.c_void_p]
        for f in (L.orc_update_matrix_adam,):
            f.restype = C.c_uint64
            f.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                          C.c_int, C.c_uint32, C.c_float]
        L.orc_update_vector_adam.restype = C.c_uint64
        L.orc_update_vector_adam.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                                             C.c_void_p, C.c_int, C.c_uint32, C.c_float]
        L.orc_es_update_adam.restype = C.c_uint64
        L.orc_es_update_adam.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_float]
        L.orc_scaled_noise.restype = C.c_int32
        L.orc_scaled_noise.argtypes = [C.c_int, C.c_int]
        L.orc_noise_dot_adaptive.restype = C.c_int32
        L.orc_noise_dot_adaptive.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_uint32, C.c_void_p]
        L.orc_down_dot_adaptive.restype = C.c_int32
        L.orc_down_dot_adaptive.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_uint32, C.c_void_p]
        L.orc_ternary_model_bytes.restype = C.c_int64
        L.orc_ternary_model_bytes.argtypes = [C.c_void_p]
        L.orc_ternary_model_pack.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_ternary_model_unpack.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_adaptive_factor.restype = C.c_float
        L.orc_adaptive_factor.argtypes = [C.c_int]
        L.orc_forward_member_adaptive.restype = C.c_int32
        L.orc_forward_member_adaptive.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64,
                                                  C.c_uint32, C.c_int, C.c_int, C.c_void_p]
        L.orc_population_forward_adaptive.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                                      C.c_int64, C.c_uint32, C.c_int, C.c_int, C.c_void_p]
        L.orc_update_overlay.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int]
        L.orc_es_update_adam_adaptive.restype = C.c_uint64
        L.orc_es_update_adam_adaptive.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                                  C.c_uint32, C.c_float, C.c_int, C.c_int]
        L.orc_learning_rate.restype = C.c_float
        L.orc_learning_rate.argtypes = [C.c_long]
        L.orc_newton_schulz_f32.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int]
        L.orc_newton_schulz_f64.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int]
        L.orc_update_matrix_muon.restype = C.c_uint64
        L.orc_update_matrix_muon.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                                             C.c_int, C.c_void_p, C.c_int, C.c_uint32, C.c_float, C.c_void_p]
        L.orc_gru_model_bytes.restype = C.c_int64
        L.orc_gru_model_bytes.argtypes = [C.c_void_p]
        L.orc_gru_state_bytes.argtypes = [C.c_void_p]
        L.orc_gru_init_model.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32]
        L.orc_init_model.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32]
        L.orc_model_bytes.argtypes = [C.c_void_p]
        L.orc_tables.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_tensor_table.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        L.orc_repack.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int]
        L.orc_unpack.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int]
        L.orc_xorshift32.argtypes = [C.c_void_p]
        L.orc_seed_offset.argtypes = [C.c_char_p]
        L.orc_gen_noise_host.argtypes = [C.c_void_p, C.c_int]
        L.orc_default_config.argtypes = [C.c_void_p]
        L.orc_gru_default_config.argtypes = [C.c_void_p]
        L.orc_gru_state_bytes.restype = C.c_int64
        L.orc_gru_matmul_perturbed.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                               C.c_uint32, C.c_int, C.c_int]
        L.orc_gru_ln.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        L.orc_gru_compute_loss.restype = C.c_int32
        L.orc_gru_compute_loss.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int]
        L.orc_gru_forward.restype = C.c_int32
        L.orc_gru_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_uint32,
                                      C.c_int, C.c_void_p]
        L.orc_gru_population.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_uint32, C.c_int,
                                         C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_gru_update_matrix.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_uint32, C.c_void_p, C.c_int]
        L.orc_gru_update_all.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p]
        L.orc_gru_noise_vector.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        _lib = L
    return _lib


def ref():
    """oracle/_ref/libegg_ref.so (the reference's own host header, compiled); None if absent."""
    global _ref
    if _ref is None:
        if not os.path.exists(REF_PATH):
            return None
        R = C.CDLL(REF_PATH)
        R.ref_hash_rng.restype = C.c_uint32
        R.ref_hash_rng.argtypes = [C.c_uint32, C.c_uint32]
        R.ref_noise_from_hash.restype = C.c_int
        R.ref_noise_from_hash.argtypes = [C.c_uint32, C.c_uint32]
        R.ref_clip.restype = C.c_int
        R.ref_clip.argtypes = [C.c_int32]
        R.ref_xorshift32_host.restype = C.c_uint32
        R.ref_gen_noise_host.restype = C.c_int
        R.ref_ternary_pack_estimate_size.restype = C.c_size_t
        R.ref_ternary_pack_estimate_size.argtypes = [C.c_size_t]
        R.ref_ternary_pack.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p]
        R.ref_ternary_unpack.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p]
        _ref = R
    return _ref


def ref_layout(tag):
    """oracle/_ref/libegg_ref_layout_<tag>.so -> (macros, fields): the reference's own config.h / definitions.h /
    optimizer/base.h compiled for one (HIDDEN_DIM, N_LAYERS, USE_MUON) variant.  macros: name -> value; fields:
    (struct, field) -> (offset, size), field "" = the struct's size.  None if the library is absent."""
    path = os.path.join(os.path.dirname(REF_PATH), "libegg_ref_layout_%s.so" % tag)
    if not os.path.exists(path):
        return None
    R = C.CDLL(path)
    R.ref_macro_name.restype = C.c_char_p
    R.ref_macro_value.restype = C.c_double
    R.ref_field_struct.restype = C.c_char_p
    R.ref_field_name.restype = C.c_char_p
    R.ref_field_offset.restype = C.c_uint64
    R.ref_field_size.restype = C.c_uint64
    R.ref_deggs_learning_rate.restype = C.c_float
    R.ref_deggs_learning_rate.argtypes = [C.c_long]
    macros = {R.ref_macro_name(i).decode(): R.ref_macro_value(i) for i in range(R.ref_macro_count())}
    fields = {(R.ref_field_struct(i).decode(), R.ref_field_name(i).decode()): (int(R.ref_field_offset(i)), int(R.ref_field_size(i)))
              for i in range(R.ref_field_count())}
    macros["deggs_learning_rate(0,99,100,199,200,100000)"] = [float(R.ref_deggs_learning_rate(s)) for s in (0, 99, 100, 199, 200, 100000)]
    return macros, fields


REF_LAYOUT_TAGS = {"h256_l4_adam": dict(hidden=256, n_layers=4, use_muon=0), "h512_l8_muon": dict(hidden=512, n_layers=8, use_muon=1),
                   "h64_l2_adam": dict(hidden=64, n_layers=2, use_muon=0), "h64_l2_muon": dict(hidden=64, n_layers=2, use_muon=1)}

_ref_gaussian = None


def ref_gaussian():
    """oracle/_ref/libegg_ref_gaussian.so: the same reference header compiled with -DDEVICE_GAUSSIAN=true
    -DHOST_GAUSSIAN=true; None if absent."""
    global _ref_gaussian
    path = os.path.join(os.path.dirname(REF_PATH), "libegg_ref_gaussian.so")
    if _ref_gaussian is None:
        if not os.path.exists(path):
            return None
        R = C.CDLL(path)
        R.ref_noise_from_hash.restype = C.c_int
        R.ref_noise_from_hash.argtypes = [C.c_uint32, C.c_uint32]
        R.ref_gen_noise_host.restype = C.c_int
        _ref_gaussian = R
    return _ref_gaussian


# ----------------------------------------------------------------------------- helpers
def config(**kw):
    c = OrcConfig()
    lib().orc_default_config(C.byref(c))
    for k, v in kw.items():
        if not hasattr(c, k):
            raise KeyError(k)
        setattr(c, k, v)
    return c


def gru_config(**kw):
    c = OrcGruConfig()
    lib().orc_gru_default_config(C.byref(c))
    for k, v in kw.items():
        if not hasattr(c, k):
            raise KeyError(k)
        setattr(c, k, v)
    return c


def tables(cfg):
    exp = np.zeros(256, np.int32)
    act = np.zeros(256, np.int8)
    rope = np.zeros(cfg.seq_len * cfg.head_dim, np.int32)
    lib().orc_tables(C.byref(cfg), _p(exp), _p(act), _p(rope))
    return exp, act, rope


def model_bytes(cfg):
    return int(lib().orc_model_bytes(C.byref(cfg)))


def init_model(cfg, seed=42):
    m = np.zeros(model_bytes(cfg), np.int8)
    lib().orc_init_model(C.byref(cfg), _p(m), C.c_uint32(seed))
    return m


def tensor_table(cfg):
    arr = (OrcTensor * 256)()
    n = lib().orc_tensor_table(C.byref(cfg), arr, 256)
    return [dict(name=arr[i].name.decode(), is_matrix=arr[i].is_matrix, rows=arr[i].rows, cols=arr[i].cols,
                 offset=arr[i].offset, off_a=arr[i].off_a, off_b=arr[i].off_b, seed_base=arr[i].seed_base,
                 lr_scale=arr[i].lr_scale, muon=arr[i].muon) for i in range(n)]


def noise_vec(seed, n, mask=15, first=0):
    L = lib()
    return np.array([L.orc_noise(C.c_uint32(seed & 0xFFFFFFFF), C.c_uint32(first + i), mask) for i in range(n)], np.int8)


def forward_member(cfg, model, data, start_idx, step_seed, p_idx, ns_override=2, trace=False, overlay=None):
    T, H, NL, V = cfg.seq_len, cfg.hidden, cfg.n_layers, cfg.vocab
    tr = None
    bufs = {}
    if trace:
        tr = OrcTrace()
        shapes = dict(x_emb=(T, H), x_init=(T, H), q=(NL, T, H), k=(NL, T, H), v=(NL, T, H), ao=(NL, T, H),
                      x_attn=(NL, T, H), x_mlp=(NL, T, H), nf=(T, H))
        for k, s in shapes.items():
            bufs[k] = np.zeros(s, np.int8)
            setattr(tr, k, bufs[k].ctypes.data)
        bufs["logits"] = np.zeros((T, V), np.int32)
        tr.logits = bufs["logits"].ctypes.data
        bufs["loss_t"] = np.zeros(T, np.int64)
        tr.loss_t = bufs["loss_t"].ctypes.data
    trp = C.byref(tr) if tr is not None else None
    if overlay is None:
        loss = lib().orc_forward_member(C.byref(cfg), _p(model), _p(data), len(data), start_idx,
                                        C.c_uint32(step_seed & 0xFFFFFFFF), p_idx, ns_override, trp)
    else:
        loss = lib().orc_forward_member_adaptive(C.byref(cfg), _p(model), _p(overlay), _p(data), len(data), start_idx,
                                                 C.c_uint32(step_seed & 0xFFFFFFFF), p_idx, ns_override, trp)
    return (loss, bufs) if trace else loss


def sample_token(logits_row, exp_lut, seed, t, hidden):
    """Three-pass LUT sampling of generate_sequence_kernel (mgpu.cu:1212-1283) for position t: the threshold is
    hash_rng(seed + t*555, 0) % sum, and the running sum is taken in the reference's thread order (thread tid owns
    v = tid, tid + BLOCK_THREADS, ...; BLOCK_THREADS = hidden rounded up to 32, at most 1024, mgpu.cu:74-75)."""
    V = len(logits_row)
    bt = min((hidden + 31) & ~31, 1024)
    gmax = int(logits_row.max())
    ex = exp_lut[np.clip(gmax - logits_row.astype(np.int64), 0, 255)].astype(np.int64)
    total = int(ex.sum())
    lib().orc_hash_rng.restype = C.c_uint32
    r = int(lib().orc_hash_rng(C.c_uint32((seed + t * 555) & 0xFFFFFFFF), C.c_uint32(0)))
    thresh = r % total if total > 0 else 0
    running = 0
    for tid in range(bt):
        for v in range(tid, V, bt):
            running += int(ex[v])
            if running > thresh:
                return v
    return 0


def _sat_f2i(x):
    """float -> int32 as the GPU converts: truncation toward zero, saturation at the ends, NaN -> 0."""
    x = np.float32(x)
    if np.isnan(x):
        return 0
    if x >= np.float32(2147483648.0):
        return 2147483647
    if x <= np.float32(-2147483648.0):
        return -2147483648
    return int(x)


def deggs_sampling_constants(cfg, min_p, penalty):
    """penalty_int and min_p_limit of d-eggs/src/kernels.cu:386-387: the penalty in logit units, truncated, and
    logf(min_p) * SOFTMAX_EXP_SCALE (a double product of a float logarithm), truncated; min_p = 0 gives -inf,
    which the conversion saturates to INT_MIN (nothing is filtered); min_p < 0 gives NaN, which the GPU's conversion
    turns into 0."""
    penalty_int = _sat_f2i(np.float32(penalty) * np.float32(1 << cfg.shift_logit))
    if min_p < 0 or min_p != min_p:
        limit = 0
    elif min_p == 0:
        limit = -2147483648
    else:
        prod = float(np.log(np.float32(min_p), dtype=np.float32)) * float(cfg.softmax_exp_scale)
        limit = 2147483647 if prod >= 2147483648.0 else (-2147483648 if prod <= -2147483648.0 else int(prod))
    return penalty_int, limit


def sample_token_deggs(logits_row, exp_lut, seed, t, hidden, history, temp, min_p_limit, penalty_int):
    """Three-pass sampling of d-eggs' generate_sequence_kernel (d-eggs/src/kernels.cu:382-478) for position t.
    `history` is the token buffer up to and including position t: every occurrence of v in it lowers v's logit by
    penalty_int (:398-402).  The differences to the maximum are divided by the temperature in float and truncated
    (:430), entries below min_p_limit are left out (:433), the rest weigh EXP_LUT[clamp(-scaled, 0, 255)]
    (layers.cuh:71-75).  Threshold and thread-major scan order as in the plain sampler (:443-474)."""
    V = len(logits_row)
    bt = min((hidden + 31) & ~31, 1024)
    counts = np.bincount(np.asarray(history, np.int64), minlength=V)[:V]
    lg = (logits_row.astype(np.int64) - counts * int(penalty_int))
    lg = ((lg + (1 << 31)) % (1 << 32) - (1 << 31))                 # int32 wrap-around, as the repeated subtraction does
    gmax = int(lg.max())
    ex = np.zeros(V, np.int64)
    for v in range(V):
        shifted = int(lg[v]) - gmax
        shifted = (shifted + (1 << 31)) % (1 << 32) - (1 << 31)
        scaled = _sat_f2i(np.float32(shifted) / np.float32(temp))
        if scaled >= min_p_limit:
            idx = -scaled
            ex[v] = int(exp_lut[0 if idx < 0 else (255 if idx > 255 else idx)])
    total = int(ex.sum())
    r = int(lib().orc_hash_rng(C.c_uint32((seed + t * 555) & 0xFFFFFFFF), C.c_uint32(0)))
    thresh = r % total if total > 0 else 0
    running = 0
    for tid in range(bt):
        for v in range(tid, V, bt):
            running += int(ex[v])
            if running > thresh:
                return v
    return 0


def generate_deggs(cfg, model, prompt, gen_len, seed, temp, min_p, penalty):
    """d-eggs' generate_sequence_kernel (d-eggs/src/kernels.cu:307-490) on this model's unperturbed forward: as
    generate(), with the temperature / min-p / presence-penalty sampler."""
    T = cfg.seq_len
    seed_len = len(prompt)
    assert 1 <= seed_len and seed_len + gen_len <= min(T, 256)
    exp_lut = tables(cfg)[0]
    penalty_int, limit = deggs_sampling_constants(cfg, min_p, penalty)
    buf = np.zeros(T + 1, np.uint8 if cfg.vocab <= 256 else np.uint32)      # TokenType, d-eggs/include/config.h:26-28
    buf[:seed_len] = prompt
    for t in range(seed_len - 1, seed_len + gen_len - 1):
        _, tr = forward_member(cfg, model, buf, 0, 0, 0, ns_override=0, trace=True)
        buf[t + 1] = sample_token_deggs(tr["logits"][t], exp_lut, seed, t, cfg.hidden, buf[:t + 1], temp, limit, penalty_int)
    return buf[:seed_len + gen_len].copy()


def generate(cfg, model, prompt, gen_len, seed):
    """generate_sequence_kernel (mgpu.cu:1154-1283): unperturbed forward (noise_sign 0), token t+1 sampled from the
    logits of position t for t >= seed_len - 1.  The window is re-evaluated from position 0 for every new token,
    which equals the reference's KV-cache walk because position t only sees positions <= t."""
    T = cfg.seq_len
    seed_len = len(prompt)
    assert 1 <= seed_len and seed_len + gen_len <= T
    exp_lut = tables(cfg)[0]
    buf = np.zeros(T + 1, np.uint8 if cfg.vocab <= 256 else np.uint32)
    buf[:seed_len] = prompt
    for t in range(seed_len - 1, seed_len + gen_len - 1):
        _, tr = forward_member(cfg, model, buf, 0, 0, 0, ns_override=0, trace=True)
        buf[t + 1] = sample_token(tr["logits"][t], exp_lut, seed, t, cfg.hidden)
    return buf[:seed_len + gen_len].copy()


def population_forward(cfg, model, data, start_idx, step_seed, pop_offset=0, count=None, overlay=None):
    count = cfg.population if count is None else count
    loss = np.zeros(cfg.population, np.int32)
    if overlay is None:
        lib().orc_population_forward(C.byref(cfg), _p(model), _p(data), len(data), start_idx,
                                     C.c_uint32(step_seed & 0xFFFFFFFF), pop_offset, count, _p(loss))
    else:
        lib().orc_population_forward_adaptive(C.byref(cfg), _p(model), _p(overlay), _p(data), len(data), start_idx,
                                              C.c_uint32(step_seed & 0xFFFFFFFF), pop_offset, count, _p(loss))
    return loss


def perturbed_linear(cfg, X, Wb, T, K, N, seed, off_a, off_b, shift):
    rows = X.shape[0]
    Y = np.zeros((rows, N), np.int32)
    lib().orc_perturbed_linear(C.byref(cfg), _p(X), _p(Wb), rows, T, K, N, C.c_uint32(seed & 0xFFFFFFFF),
                               off_a, off_b, shift, _p(Y))
    return Y


def fitness(loss):
    pairs = len(loss) // 2
    fit = np.zeros(pairs, np.int32)
    lib().orc_fitness(_p(np.ascontiguousarray(loss, np.int32)), _p(fit), pairs)
    return fit


ADAM_DTYPE = np.dtype([("m", np.float32), ("v", np.float32), ("acc", np.float32)])
MUON_DTYPE = np.dtype([("m", np.float32), ("acc", np.float32)])


def es_update_adam(cfg, model, state, fit, step_seed, lr):
    """in place on model (int8) and state (ADAM_DTYPE, one per model byte); returns update count"""
    return int(lib().orc_es_update_adam(C.byref(cfg), _p(model), _p(state), _p(fit),
                                        C.c_uint32(step_seed & 0xFFFFFFFF), C.c_float(lr)))


def es_update_adam_adaptive(cfg, model, state, overlay, fit, step_seed, lr, inc=5, dec=1):
    """d-eggs optimizer step: in place on model, state and the overlay blob (same layout as the model)"""
    return int(lib().orc_es_update_adam_adaptive(C.byref(cfg), _p(model), _p(state), _p(overlay), _p(fit),
                                                 C.c_uint32(step_seed & 0xFFFFFFFF), C.c_float(lr), inc, dec))


def ternary_model_pack(cfg, model):
    """2-bit packing of the matrix tensors (vectors stay int8); raises when a matrix weight is outside {-1, 0, 1}"""
    out = np.zeros(int(lib().orc_ternary_model_bytes(C.byref(cfg))), np.uint8)
    if lib().orc_ternary_model_pack(C.byref(cfg), _p(model), _p(out)) != 0:
        raise ValueError("matrix weight outside {-1, 0, 1}")
    return out


def ternary_model_unpack(cfg, packed):
    out = np.zeros(model_bytes(cfg), np.int8)
    lib().orc_ternary_model_unpack(C.byref(cfg), _p(packed), _p(out))
    return out


def gru_init_model(gcfg, seed=42):
    m = np.zeros(int(lib().orc_gru_model_bytes(C.byref(gcfg))), np.int8)
    lib().orc_gru_init_model(C.byref(gcfg), _p(m), seed)
    return m


def gru_population(gcfg, model, data, start_idx, step_seed, pair0, npairs, states):
    """forward +/- for pairs [pair0, pair0+npairs); returns (loss[population], fit[population/2]) (only those pairs written)"""
    loss = np.zeros(gcfg.population, np.int32)
    fit = np.zeros(gcfg.population // 2, np.int32)
    lib().orc_gru_population(C.byref(gcfg), _p(model), _p(data), len(data), start_idx, C.c_uint32(step_seed & 0xFFFFFFFF),
                             pair0, npairs, _p(states), _p(loss), _p(fit))
    return loss, fit


def zipf_bytes(n, seed=1234, s=1.1):
    """Synthetic byte stream: i.i.d. Zipf(s) ranks over a fixed permutation of the 256 byte values.
    Counter-based SplitMix64 -> inverse CDF (so any slice can be regenerated independently)."""
    idx = np.arange(1, n + 1, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + idx * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    u = (z >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
    w = 1.0 / np.arange(1, 257, dtype=np.float64) ** s
    cdf = np.cumsum(w) / np.sum(w)
    rank = np.minimum(np.searchsorted(cdf, u, side="right"), 255)
    # fixed permutation of byte values from the same generator (Fisher-Yates with xorshift32)
    perm = np.arange(256, dtype=np.uint8)
    st = np.uint32((seed * 2654435761 + 1) & 0xFFFFFFFF) or np.uint32(1)
    st = int(st)
    for i in range(255, 0, -1):
        st ^= (st << 13) & 0xFFFFFFFF
        st ^= st >> 17
        st ^= (st << 5) & 0xFFFFFFFF
        j = st % (i + 1)
        perm[i], perm[j] = perm[j], perm[i]
    return perm[rank].astype(np.uint8)

"""Python host-side binding of libegg_hip.so (the C ABI declared in include/egg_hip.h).

The directory name contains a dot, so load this package with ``load_package()`` from
``__graft_entry__`` (importlib by path) under the module name ``egg_c_amd``.

There is no CPU fallback: if libegg_hip.so is missing or a call fails, an exception is raised.
PyTorch is used by callers only to own device memory; this module takes raw device pointers.
"""
import ctypes as C
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libegg_hip.so")


class EggError(RuntimeError):
    pass


class EggConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "hidden", "head_dim", "n_layers", "seq_len", "vocab", "population",
        "fixed_point", "sigma_shift", "sigma_shift_vector",
        "shift_attn", "shift_out", "shift_logit", "shift_mlp_up", "shift_mlp_down",
        "softmax_scale_bit", "rope_scale_bit", "noise_mask", "host_mask")] + [
        ("softmax_exp_scale", C.c_double),
        ("adam_beta1", C.c_float), ("adam_beta2", C.c_float), ("adam_eps", C.c_float),
        ("adam_weight_decay", C.c_float), ("muon_momentum", C.c_float), ("muon_lr_scale", C.c_float),
        ("use_muon", C.c_int), ("chunk_members", C.c_int), ("weight_limit", C.c_int),
        ("device_gaussian", C.c_int), ("host_gaussian", C.c_int), ("use_same_data", C.c_int)]


class EggTensorInfo(C.Structure):
    _fields_ = [("name", C.c_char * 32), ("is_matrix", C.c_int), ("rows", C.c_int), ("cols", C.c_int),
                ("offset", C.c_int64), ("off_a", C.c_int), ("off_b", C.c_int), ("seed_base", C.c_int),
                ("lr_scale", C.c_float), ("muon", C.c_int)]


EXPORTS = [
    "egg_default_config", "egg_ctx_create", "egg_ctx_destroy", "egg_last_error", "egg_ctx_set_stream", "egg_sync",
    "egg_model_bytes", "egg_model_init", "egg_model_upload", "egg_model_download",
    "egg_opt_state_upload", "egg_opt_state_download", "egg_opt_state_reset", "egg_tables_download",
    "egg_noise_fill", "egg_perturbed_linear", "egg_perturbed_linear_own_noise", "egg_shared_linear", "egg_ctx_linear_kernel", "egg_population_forward", "egg_population_forward_dev",
    "egg_fitness", "egg_es_update", "egg_update_tensor", "egg_matrix_votes",
    "egg_adaptive_enable", "egg_overlay_upload", "egg_overlay_download",
    "egg_ternary_model_bytes", "egg_model_upload_ternary", "egg_model_download_ternary",
    "egg_tensor_count", "egg_tensor_info_get", "egg_last_update_count",
    "egg_step", "egg_step_capture", "egg_step_launch", "egg_step_losses", "egg_generate", "egg_generate_deggs", "egg_deggs_sampling_constants",
    "egg_shape_fitness", "egg_ternary_pack_size", "egg_ternary_pack", "egg_ternary_unpack",
    "egg_vocab_load", "egg_vocab_free", "egg_vocab_size", "egg_vocab_save", "egg_detokenize",
    "egg_checkpoint_save", "egg_checkpoint_load", "egg_eggc_save", "egg_eggc_load_latest",
    "egg_learning_rate", "egg_learning_rate_deggs", "egg_model_info_save", "egg_next_seed", "egg_ctx_enable_taps", "egg_ctx_first_block_dedup", "egg_tap_download",
    "egg_ctx_enable_timing", "egg_timing_reset", "egg_timing_get",
    "egg_opt_state_bytes", "egg_tensor_state_offset", "egg_newton_schulz", "egg_describe_layout", "egg_muon_plan", "egg_ctx_generate_kv_cache", "egg_newton_schulz_static",
    "egg_gru_default_config", "egg_gru_create", "egg_gru_destroy", "egg_gru_last_error", "egg_gru_model_bytes",
    "egg_gru_model_init", "egg_gru_model_upload", "egg_gru_model_download", "egg_gru_state_reset",
    "egg_gru_state_download", "egg_gru_step", "egg_gru_losses", "egg_gru_forward_mode",
]
KCLASSES = ["mlp_first", "qkv", "attn", "mlp", "head", "update_matrix", "update_vector", "plinear", "muon_ns"]


def build(force=True):
    """Compile libegg_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
    cmd = ["make", "-C", HERE, "-j8", "-s"]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd + ["all", "host"])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise EggError("libegg_hip.so is not built (run __graft_entry__.build()); there is no CPU fallback")
        # PyTorch brings a HIP runtime of its own.  When this library's runtime is loaded into the process first and torch
        # initialises its devices afterwards, this library's first HIP call reports "no ROCm-capable device"; the other
        # order works.  Callers hand over torch tensors' device pointers anyway, so torch goes first where it is installed.
        import sys
        if "torch" not in sys.modules:
            try:
                import torch  # noqa: F401
            except ImportError:
                pass
        L = C.CDLL(LIB_PATH)
        vp, i32, i64, u32 = C.c_void_p, C.c_int, C.c_int64, C.c_uint32
        L.egg_default_config.argtypes = [vp]
        L.egg_ctx_create.argtypes = [vp, vp]
        L.egg_ctx_destroy.argtypes = [vp]
        L.egg_ctx_destroy.restype = None
        L.egg_last_error.restype = C.c_char_p
        L.egg_last_error.argtypes = [vp]
        L.egg_ctx_set_stream.argtypes = [vp, vp]
        L.egg_sync.argtypes = [vp]
        L.egg_model_bytes.restype = i64
        L.egg_model_bytes.argtypes = [vp]
        L.egg_model_init.argtypes = [vp, u32]
        for f in (L.egg_model_upload, L.egg_model_download, L.egg_opt_state_upload, L.egg_opt_state_download,
                  L.egg_overlay_upload, L.egg_overlay_download):
            f.argtypes = [vp, vp, C.c_size_t]
        L.egg_adaptive_enable.argtypes = [vp, i32, i32, i32]
        L.egg_ternary_model_bytes.restype = i64
        L.egg_ternary_model_bytes.argtypes = [vp]
        for f in (L.egg_model_upload_ternary, L.egg_model_download_ternary):
            f.argtypes = [vp, vp, C.c_size_t]
        L.egg_opt_state_reset.argtypes = [vp]
        L.egg_tables_download.argtypes = [vp, vp, vp, vp]
        L.egg_noise_fill.argtypes = [vp, u32, u32, i32, vp]
        L.egg_perturbed_linear.argtypes = [vp, vp, vp, i32, i32, i32, i32, u32, i32, i32, i32, vp, vp]
        L.egg_perturbed_linear_own_noise.argtypes = [vp, vp, vp, i32, i32, i32, i32, u32, i32, i32, i32, vp, vp]
        L.egg_ctx_linear_kernel.argtypes = [vp, i32]
        L.egg_shared_linear.argtypes = [vp, vp, vp, i32, i32, i32, i32, i32, vp, vp]
        L.egg_population_forward.argtypes = [vp, vp, i64, i64, u32, i32, i32, vp]
        L.egg_population_forward_dev.argtypes = [vp, vp, i64, vp, vp, i32, i32, vp]
        L.egg_fitness.argtypes = [vp, vp, vp, i32]
        L.egg_es_update.argtypes = [vp, vp, vp, vp]
        L.egg_update_tensor.argtypes = [vp, i32, vp, vp, vp]
        L.egg_matrix_votes.argtypes = [vp, i32, vp, vp, vp]
        L.egg_tensor_count.argtypes = [vp]
        L.egg_tensor_info_get.argtypes = [vp, i32, vp]
        L.egg_last_update_count.argtypes = [vp, vp]
        L.egg_step.argtypes = [vp, vp, i64, i64, u32, C.c_float]
        L.egg_step_capture.argtypes = [vp, vp, i64]
        L.egg_step_launch.argtypes = [vp, i64, u32, C.c_float]
        L.egg_step_losses.argtypes = [vp, vp, vp]
        L.egg_generate.argtypes = [vp, vp, i32, i32, u32]
        L.egg_generate_deggs.argtypes = [vp, vp, i32, i32, u32, C.c_float, C.c_float, C.c_float]
        L.egg_deggs_sampling_constants.argtypes = [vp, C.c_float, C.c_float, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
        L.egg_shape_fitness.argtypes = [vp, i32, i32, C.c_double, i32, C.c_double, vp, vp]
        L.egg_ternary_pack_size.restype = C.c_size_t
        L.egg_ternary_pack_size.argtypes = [C.c_size_t]
        L.egg_ternary_pack.argtypes = [vp, C.c_size_t, vp]
        L.egg_vocab_load.argtypes = [C.c_char_p, C.POINTER(vp)]
        L.egg_vocab_free.argtypes = [vp]
        L.egg_vocab_free.restype = None
        L.egg_vocab_size.argtypes = [vp]
        L.egg_vocab_save.argtypes = [C.c_char_p, vp, vp, C.c_uint32]
        L.egg_detokenize.argtypes = [vp, vp, i32, vp, C.c_int64]
        L.egg_detokenize.restype = C.c_int64
        L.egg_ternary_unpack.argtypes = [vp, C.c_size_t, vp]
        L.egg_checkpoint_save.argtypes = [vp, C.c_char_p, C.c_long]
        L.egg_checkpoint_load.argtypes = [vp, C.c_char_p, C.c_char_p]
        L.egg_eggc_save.argtypes = [C.c_char_p, C.c_uint64, C.c_uint64, vp, C.c_uint64]
        L.egg_eggc_load_latest.argtypes = [C.c_char_p, vp, vp, vp, C.c_uint64, vp]
        L.egg_learning_rate.restype = C.c_float
        L.egg_learning_rate.argtypes = [C.c_long]
        L.egg_learning_rate_deggs.restype = C.c_float
        L.egg_learning_rate_deggs.argtypes = [C.c_long]
        L.egg_model_info_save.argtypes = [vp, C.c_char_p]
        L.egg_next_seed.restype = u32
        L.egg_next_seed.argtypes = [u32, C.c_uint64]
        L.egg_ctx_enable_taps.argtypes = [vp, i32]
        L.egg_ctx_first_block_dedup.argtypes = [vp, i32]
        L.egg_tap_download.argtypes = [vp, C.c_char_p, i32, vp]
        L.egg_ctx_enable_timing.argtypes = [vp, i32]
        L.egg_timing_reset.argtypes = [vp]
        L.egg_timing_get.argtypes = [vp, i32, vp, vp]
        L.egg_opt_state_bytes.restype = i64
        L.egg_opt_state_bytes.argtypes = [vp]
        L.egg_describe_layout.argtypes = [vp, i32, vp, vp, vp, vp]
        L.egg_muon_plan.argtypes = [vp, i32, vp, vp, vp, vp, vp, vp]
        L.egg_newton_schulz_static.argtypes = [vp, i32, i32, i32, vp]
        L.egg_tensor_state_offset.restype = i64
        L.egg_tensor_state_offset.argtypes = [vp, i32]
        L.egg_newton_schulz.argtypes = [vp, vp, i32, i32, i32]
        L.egg_gru_default_config.argtypes = [vp]
        L.egg_gru_create.argtypes = [vp, vp]
        L.egg_gru_destroy.argtypes = [vp]
        L.egg_gru_destroy.restype = None
        L.egg_gru_last_error.restype = C.c_char_p
        L.egg_gru_last_error.argtypes = [vp]
        L.egg_gru_model_bytes.restype = i64
        L.egg_gru_model_bytes.argtypes = [vp]
        L.egg_gru_model_init.argtypes = [vp, u32]
        L.egg_gru_model_upload.argtypes = [vp, vp, C.c_size_t]
        L.egg_gru_model_download.argtypes = [vp, vp, C.c_size_t]
        L.egg_gru_state_reset.argtypes = [vp]
        L.egg_gru_state_download.argtypes = [vp, vp, C.c_size_t]
        L.egg_gru_step.argtypes = [vp, vp, i64, i64, u32, i32]
        L.egg_gru_losses.argtypes = [vp, vp, vp]
        _lib = L
    return _lib


def default_config(**kw):
    c = EggConfig()
    lib().egg_default_config(C.byref(c))
    for k, v in kw.items():
        if not hasattr(c, k):
            raise KeyError(k)
        setattr(c, k, v)
    return c


def describe_layout(cfg):
    """Host-only: (tensors, model_bytes, state_bytes) of a configuration; each tensor dict also carries its byte
    offset into the optimizer state.  No GPU is touched."""
    mb, sb = C.c_int64(), C.c_int64()
    n = lib().egg_describe_layout(C.byref(cfg), -1, None, None, C.byref(mb), C.byref(sb))
    if n < 0:
        raise EggError("egg_describe_layout: invalid configuration")
    out = []
    for i in range(n):
        t, so = EggTensorInfo(), C.c_int64()
        lib().egg_describe_layout(C.byref(cfg), i, C.byref(t), C.byref(so), None, None)
        out.append(dict(id=i, name=t.name.decode(), is_matrix=t.is_matrix, rows=t.rows, cols=t.cols, offset=t.offset,
                        off_a=t.off_a, off_b=t.off_b, seed_base=t.seed_base, lr_scale=t.lr_scale, muon=t.muon,
                        state_offset=int(so.value)))
    return out, int(mb.value), int(sb.value)


def muon_plan(cfg):
    """Host-only: (groups, matrix_buffer_floats, term_buffer_floats); a group is a dict rows / cols / members / batch."""
    a, b = C.c_int64(), C.c_int64()
    n = lib().egg_muon_plan(C.byref(cfg), -1, None, None, None, None, C.byref(a), C.byref(b))
    if n < 0:
        raise EggError("egg_muon_plan: invalid configuration")
    groups = []
    for g in range(n):
        r, c, m, bt = C.c_int(), C.c_int(), C.c_int(), C.c_int()
        lib().egg_muon_plan(C.byref(cfg), g, C.byref(r), C.byref(c), C.byref(m), C.byref(bt), None, None)
        groups.append(dict(rows=r.value, cols=c.value, members=m.value, batch=bt.value))
    return groups, int(a.value), int(b.value)


def newton_schulz_static(d_x, rows, cols, iters=5, stream=None):
    """egg_newton_schulz_static: Newton-Schulz in place on a row-major fp32 device matrix, no context, no allocation."""
    rc = lib().egg_newton_schulz_static(C.c_void_p(d_x), rows, cols, iters, C.c_void_p(stream))
    if rc != 0:
        raise EggError("egg_newton_schulz_static failed (%d): %s" % (rc, (lib().egg_last_error(None) or b"").decode()))


def deggs_sampling_constants(cfg, min_p, penalty):
    """(penalty_int, min_p_limit) as egg_generate_deggs derives them (host only)."""
    a, b = C.c_int32(), C.c_int32()
    rc = lib().egg_deggs_sampling_constants(C.byref(cfg), min_p, penalty, C.byref(a), C.byref(b))
    if rc != 0:
        raise EggError("egg_deggs_sampling_constants failed (%d)" % rc)
    return int(a.value), int(b.value)


def _np_ptr(a):
    return a.ctypes.data_as(C.c_void_p)


class Context:
    """One device context: model + optimizer state + workspace (mirror of the reference's GPUContext,
    full_cuda_train_transformer_adam_mgpu.cu:1287-1302)."""

    def __init__(self, cfg):
        self.cfg = cfg
        self._h = C.c_void_p()
        rc = lib().egg_ctx_create(C.byref(cfg), C.byref(self._h))
        if rc != 0:
            raise EggError(f"egg_ctx_create failed with {rc}: {lib().egg_last_error(None).decode()}")

    def close(self):
        if self._h:
            lib().egg_ctx_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _ck(self, rc, what):
        if rc != 0:
            raise EggError(f"{what} failed with {rc}: {lib().egg_last_error(self._h).decode()}")

    def set_stream(self, stream_handle):
        self._ck(lib().egg_ctx_set_stream(self._h, C.c_void_p(stream_handle)), "egg_ctx_set_stream")

    def sync(self):
        self._ck(lib().egg_sync(self._h), "egg_sync")

    def model_bytes(self):
        return int(lib().egg_model_bytes(self._h))

    def model_init(self, seed=42):
        self._ck(lib().egg_model_init(self._h, seed), "egg_model_init")

    def model_upload(self, arr):
        self._ck(lib().egg_model_upload(self._h, _np_ptr(arr), arr.nbytes), "egg_model_upload")

    def model_download(self):
        import numpy as np
        out = np.zeros(self.model_bytes(), np.int8)
        self._ck(lib().egg_model_download(self._h, _np_ptr(out), out.nbytes), "egg_model_download")
        return out

    def opt_state_upload(self, arr):
        self._ck(lib().egg_opt_state_upload(self._h, _np_ptr(arr), arr.nbytes), "egg_opt_state_upload")

    def opt_state_download(self):
        import numpy as np
        out = np.zeros(int(lib().egg_opt_state_bytes(self._h)) // 4, np.float32)
        self._ck(lib().egg_opt_state_download(self._h, _np_ptr(out), out.nbytes), "egg_opt_state_download")
        return out

    def tensor_state_offset(self, tid):
        return int(lib().egg_tensor_state_offset(self._h, tid))

    def newton_schulz(self, d_x, rows, cols, iters=5):
        self._ck(lib().egg_newton_schulz(self._h, C.c_void_p(d_x), rows, cols, iters), "egg_newton_schulz")

    def opt_state_reset(self):
        self._ck(lib().egg_opt_state_reset(self._h), "egg_opt_state_reset")

    def tables(self):
        import numpy as np
        ex = np.zeros(256, np.int32)
        act = np.zeros(256, np.int8)
        rope = np.zeros(self.cfg.seq_len * self.cfg.head_dim, np.int32)
        self._ck(lib().egg_tables_download(self._h, _np_ptr(ex), _np_ptr(act), _np_ptr(rope)), "egg_tables_download")
        return ex, act, rope

    def noise_fill(self, seed, first, n, d_out):
        self._ck(lib().egg_noise_fill(self._h, seed & 0xFFFFFFFF, first, n, C.c_void_p(d_out)), "egg_noise_fill")

    def perturbed_linear(self, d_x, d_w, members, T, K, N, seed, off_a, off_b, shift, d_y32=None, d_y8=None):
        self._ck(lib().egg_perturbed_linear(self._h, C.c_void_p(d_x), C.c_void_p(d_w), members, T, K, N,
                                            seed & 0xFFFFFFFF, off_a, off_b, shift,
                                            C.c_void_p(d_y32) if d_y32 else None, C.c_void_p(d_y8) if d_y8 else None),
                 "egg_perturbed_linear")

    def perturbed_linear_own_noise(self, d_x, d_w, members, T, K, N, seed, off_a, off_b, shift, d_y32=None, d_y8=None):
        self._ck(lib().egg_perturbed_linear_own_noise(self._h, C.c_void_p(d_x), C.c_void_p(d_w), members, T, K, N,
                                                      seed & 0xFFFFFFFF, off_a, off_b, shift,
                                                      C.c_void_p(d_y32) if d_y32 else None, C.c_void_p(d_y8) if d_y8 else None),
                 "egg_perturbed_linear_own_noise")

    def linear_kernel(self, w_stationary=True):
        self._ck(lib().egg_ctx_linear_kernel(self._h, 1 if w_stationary else 0), "egg_ctx_linear_kernel")

    def shared_linear(self, d_x, d_w, members, T, K, N, shift, d_y32=None, d_y8=None):
        self._ck(lib().egg_shared_linear(self._h, C.c_void_p(d_x), C.c_void_p(d_w), members, T, K, N, shift,
                                         C.c_void_p(d_y32) if d_y32 else None, C.c_void_p(d_y8) if d_y8 else None),
                 "egg_shared_linear")

    def population_forward(self, d_data, data_len, start_idx, step_seed, pop_offset, pop_count, d_loss):
        self._ck(lib().egg_population_forward(self._h, C.c_void_p(d_data), data_len, start_idx, step_seed & 0xFFFFFFFF,
                                              pop_offset, pop_count, C.c_void_p(d_loss)), "egg_population_forward")

    def fitness(self, d_loss, d_fit, pairs):
        self._ck(lib().egg_fitness(self._h, C.c_void_p(d_loss), C.c_void_p(d_fit), pairs), "egg_fitness")

    def es_update(self, d_fit, d_seed, d_lr):
        self._ck(lib().egg_es_update(self._h, C.c_void_p(d_fit), C.c_void_p(d_seed), C.c_void_p(d_lr)), "egg_es_update")

    def ternary_model_bytes(self):
        return int(lib().egg_ternary_model_bytes(self._h))

    def model_upload_ternary(self, packed):
        self._ck(lib().egg_model_upload_ternary(self._h, _np_ptr(packed), packed.nbytes), "egg_model_upload_ternary")

    def model_download_ternary(self):
        import numpy as np
        out = np.zeros(self.ternary_model_bytes(), np.uint8)
        self._ck(lib().egg_model_download_ternary(self._h, _np_ptr(out), out.nbytes), "egg_model_download_ternary")
        return out

    def adaptive_enable(self, init_value=64, inc=5, dec=1):
        """d-eggs adaptive noise overlay: on from this call (forward scaling and the overlay rule in es_update / step)"""
        self._ck(lib().egg_adaptive_enable(self._h, init_value, inc, dec), "egg_adaptive_enable")

    def overlay_upload(self, arr):
        self._ck(lib().egg_overlay_upload(self._h, _np_ptr(arr), arr.nbytes), "egg_overlay_upload")

    def overlay_download(self):
        import numpy as np
        out = np.zeros(self.model_bytes(), np.int8)
        self._ck(lib().egg_overlay_download(self._h, _np_ptr(out), out.nbytes), "egg_overlay_download")
        return out

    def update_tensor(self, tid, d_fit, d_seed, d_lr):
        self._ck(lib().egg_update_tensor(self._h, tid, C.c_void_p(d_fit), C.c_void_p(d_seed), C.c_void_p(d_lr)),
                 "egg_update_tensor")

    def matrix_votes(self, tid, d_fit, d_seed, d_votes):
        self._ck(lib().egg_matrix_votes(self._h, tid, C.c_void_p(d_fit), C.c_void_p(d_seed), C.c_void_p(d_votes)),
                 "egg_matrix_votes")

    def tensors(self):
        out = []
        for i in range(lib().egg_tensor_count(self._h)):
            t = EggTensorInfo()
            self._ck(lib().egg_tensor_info_get(self._h, i, C.byref(t)), "egg_tensor_info_get")
            out.append(dict(id=i, name=t.name.decode(), is_matrix=t.is_matrix, rows=t.rows, cols=t.cols, offset=t.offset,
                            off_a=t.off_a, off_b=t.off_b, seed_base=t.seed_base, lr_scale=t.lr_scale, muon=t.muon))
        return out

    def last_update_count(self):
        v = C.c_uint64()
        self._ck(lib().egg_last_update_count(self._h, C.byref(v)), "egg_last_update_count")
        return int(v.value)

    def step(self, d_data, data_len, start_idx, step_seed, lr):
        self._ck(lib().egg_step(self._h, C.c_void_p(d_data), data_len, start_idx, step_seed & 0xFFFFFFFF, C.c_float(lr)),
                 "egg_step")

    def step_capture(self, d_data, data_len):
        self._ck(lib().egg_step_capture(self._h, C.c_void_p(d_data), data_len), "egg_step_capture")

    def step_launch(self, start_idx, step_seed, lr):
        self._ck(lib().egg_step_launch(self._h, start_idx, step_seed & 0xFFFFFFFF, C.c_float(lr)), "egg_step_launch")

    def step_losses(self):
        import numpy as np
        loss = np.zeros(self.cfg.population, np.int32)
        fit = np.zeros(self.cfg.population // 2, np.int32)
        self._ck(lib().egg_step_losses(self._h, _np_ptr(loss), _np_ptr(fit)), "egg_step_losses")
        return loss, fit

    def checkpoint_save(self, directory, step):
        self._ck(lib().egg_checkpoint_save(self._h, directory.encode() if directory else None, step), "egg_checkpoint_save")

    def model_info_save(self, directory=None):
        """<directory>/model.info, the reference's save_model_info text (egg_disk_utils.h:15-44)"""
        self._ck(lib().egg_model_info_save(self._h, directory.encode() if directory else None), "egg_model_info_save")

    def checkpoint_load(self, model_path, state_path=None):
        self._ck(lib().egg_checkpoint_load(self._h, model_path.encode(), state_path.encode() if state_path else None), "egg_checkpoint_load")

    def generate(self, d_buffer, seed_len, gen_len, seed):
        """Continue the seed_len prompt bytes at device pointer d_buffer by gen_len sampled bytes (in place)."""
        self._ck(lib().egg_generate(self._h, C.c_void_p(d_buffer), seed_len, gen_len, seed & 0xFFFFFFFF), "egg_generate")

    def generate_deggs(self, d_buffer, seed_len, gen_len, seed, temp=0.6, min_p=0.08, penalty=0.2):
        """The same with d-eggs' sampler: temperature, min-p filter and presence penalty (its defaults)."""
        self._ck(lib().egg_generate_deggs(self._h, C.c_void_p(d_buffer), seed_len, gen_len, seed & 0xFFFFFFFF, temp, min_p, penalty),
                 "egg_generate_deggs")

    def generate_kv_cache(self, on=True):
        """egg_generate / egg_generate_deggs with (default) or without the per-layer K / V cache; same tokens either way."""
        self._ck(lib().egg_ctx_generate_kv_cache(self._h, 1 if on else 0), "egg_ctx_generate_kv_cache")

    def enable_taps(self, on=True):
        self._ck(lib().egg_ctx_enable_taps(self._h, 1 if on else 0), "egg_ctx_enable_taps")

    def first_block_dedup(self, on=True):
        self._ck(lib().egg_ctx_first_block_dedup(self._h, 1 if on else 0), "egg_ctx_first_block_dedup")

    def tap(self, name, member):
        import numpy as np
        T, H = self.cfg.seq_len, self.cfg.hidden
        out = np.zeros((T, self.cfg.vocab), np.int32) if name == "logits" else np.zeros((T, H), np.int8)
        self._ck(lib().egg_tap_download(self._h, name.encode(), member, _np_ptr(out)), "egg_tap_download")
        return out


def _enable_timing(self, on=True):
    self._ck(lib().egg_ctx_enable_timing(self._h, 1 if on else 0), "egg_ctx_enable_timing")


def _timing_reset(self):
    self._ck(lib().egg_timing_reset(self._h), "egg_timing_reset")


def _timing(self):
    """{kernel class: (launches, total_ms)} measured with hipEvents on the context's stream"""
    out = {}
    for i, name in enumerate(KCLASSES):
        n, ms = C.c_int64(), C.c_double()
        self._ck(lib().egg_timing_get(self._h, i, C.byref(n), C.byref(ms)), "egg_timing_get")
        out[name] = (int(n.value), float(ms.value))
    return out


Context.enable_timing = _enable_timing
Context.timing_reset = _timing_reset
Context.timing = _timing


# ---- host-side companions (no GPU needed)
class Vocabulary:
    """d-eggs' token table for printing generated tokens ("decoding.bin", d-eggs/src/worker.cu:36-81)."""

    def __init__(self, path):
        h = C.c_void_p()
        rc = lib().egg_vocab_load(str(path).encode(), C.byref(h))
        if rc:
            raise EggError(f"egg_vocab_load failed ({rc}): {path}")
        self._h = h

    @staticmethod
    def save(path, entries):
        """entries: a sequence of bytes objects, token id = position"""
        entries = [bytes(e) for e in entries]
        arr = (C.c_char_p * len(entries))(*entries)
        lens = (C.c_uint32 * len(entries))(*[len(e) for e in entries])
        rc = lib().egg_vocab_save(str(path).encode(), arr, lens, len(entries))
        if rc:
            raise EggError(f"egg_vocab_save failed ({rc}): {path}")

    def __len__(self):
        return lib().egg_vocab_size(self._h)

    def detokenize(self, tokens):
        import numpy as np
        tokens = np.ascontiguousarray(tokens, np.uint32)
        n = lib().egg_detokenize(self._h, _np_ptr(tokens), len(tokens), None, 0)
        if n < 0:
            raise EggError(f"egg_detokenize failed ({n})")
        buf = C.create_string_buffer(max(int(n), 1))
        lib().egg_detokenize(self._h, _np_ptr(tokens), len(tokens), buf, n)
        return buf.raw[:n]

    def close(self):
        if self._h:
            lib().egg_vocab_free(self._h)
            self._h = None


def shape_fitness(loss, chunk_mean_filter=True, mean_exponent=1.2, adaptive_threshold=True, alpha=None):
    """d-eggs worker shaping of one chunk's losses -> (fit[count/2] in {-1,0,1}, sum of losses)."""
    import numpy as np
    loss = np.ascontiguousarray(loss, np.int32)
    if alpha is None:
        alpha = float(np.float32(0.1))          # ADAPTIVE_THRESHOLD_ALPHA is the float literal 0.1f
    fit = np.zeros(len(loss) // 2, np.int32)
    total = C.c_int64(0)
    rc = lib().egg_shape_fitness(_np_ptr(loss), len(loss), int(chunk_mean_filter), mean_exponent,
                                 int(adaptive_threshold), alpha, _np_ptr(fit), C.byref(total))
    if rc:
        raise EggError(f"egg_shape_fitness failed ({rc})")
    return fit, total.value


def ternary_pack(fit):
    import numpy as np
    fit = np.ascontiguousarray(fit, np.int32)
    out = np.zeros(lib().egg_ternary_pack_size(len(fit)), np.uint8)
    if lib().egg_ternary_pack(_np_ptr(fit), len(fit), _np_ptr(out)):
        raise EggError("egg_ternary_pack: values must be -1, 0 or 1")
    return out


def ternary_unpack(packed, count):
    import numpy as np
    packed = np.ascontiguousarray(packed, np.uint8)
    out = np.zeros(count, np.int32)
    if lib().egg_ternary_unpack(_np_ptr(packed), count, _np_ptr(out)):
        raise EggError("egg_ternary_unpack failed")
    return out


def eggc_save(directory, step, seed, data):
    import numpy as np
    data = np.ascontiguousarray(data, np.uint8)
    if lib().egg_eggc_save(directory.encode(), step, seed, _np_ptr(data), len(data)):
        raise EggError("egg_eggc_save failed")


def eggc_load_latest(directory):
    """-> (step, seed, data) of the checkpoint with the highest step in `directory`, or None."""
    import numpy as np
    step, seed, n = C.c_uint64(0), C.c_uint64(0), C.c_uint64(0)
    buf = np.zeros(1 << 16, np.uint8)
    rc = lib().egg_eggc_load_latest(directory.encode(), C.byref(step), C.byref(seed), _np_ptr(buf), len(buf), C.byref(n))
    if rc == -4 or (rc and n.value > len(buf)):          # EGG_E_STATE: payload larger than the buffer
        buf = np.zeros(n.value, np.uint8)
        rc = lib().egg_eggc_load_latest(directory.encode(), C.byref(step), C.byref(seed), _np_ptr(buf), len(buf), C.byref(n))
    if rc:
        return None
    return step.value, seed.value, buf[:n.value].copy()


def zipf_bytes(n, seed=1234, s=1.1):
    """Synthetic byte stream for benchmarks: i.i.d. Zipf(s) ranks over a fixed permutation of the 256 byte values.
    Counter-based SplitMix64 -> inverse CDF (so any slice can be regenerated independently)."""
    import numpy as _np
    idx = _np.arange(1, n + 1, dtype=_np.uint64)
    with _np.errstate(over="ignore"):
        z = _np.uint64(seed) + idx * _np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> _np.uint64(30))) * _np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> _np.uint64(27))) * _np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> _np.uint64(31))
    u = (z >> _np.uint64(11)).astype(_np.float64) * (1.0 / 9007199254740992.0)
    w = 1.0 / _np.arange(1, 257, dtype=_np.float64) ** s
    cdf = _np.cumsum(w) / _np.sum(w)
    rank = _np.minimum(_np.searchsorted(cdf, u, side="right"), 255)
    # fixed permutation of byte values from the same generator (Fisher-Yates with xorshift32)
    perm = _np.arange(256, dtype=_np.uint8)
    st = _np.uint32((seed * 2654435761 + 1) & 0xFFFFFFFF) or _np.uint32(1)
    st = int(st)
    for i in range(255, 0, -1):
        st ^= (st << 13) & 0xFFFFFFFF
        st ^= st >> 17
        st ^= (st << 5) & 0xFFFFFFFF
        j = st % (i + 1)
        perm[i], perm[j] = perm[j], perm[i]
    return perm[rank].astype(_np.uint8)


def learning_rate(step):
    return float(lib().egg_learning_rate(step))


def learning_rate_deggs(step):
    """d-eggs' schedule (d-eggs/include/utils/training.h:5-9)"""
    return float(lib().egg_learning_rate_deggs(step))


def next_seed(seed, step):
    return int(lib().egg_next_seed(seed & 0xFFFFFFFF, step))


class EggGruConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("hidden", "n_layers", "seq_len", "vocab", "population",
                                       "fixed_point", "sigma_shift", "update_threshold")]


def gru_default_config(**kw):
    c = EggGruConfig()
    lib().egg_gru_default_config(C.byref(c))
    for k, v in kw.items():
        if not hasattr(c, k):
            raise KeyError(k)
        setattr(c, k, v)
    return c


class GruContext:
    """The reference's CPU program (full_trained_egg.c) on the GPU: model, recurrent states and one-step driver."""

    def __init__(self, cfg):
        self.cfg = cfg
        self._h = C.c_void_p()
        rc = lib().egg_gru_create(C.byref(cfg), C.byref(self._h))
        if rc != 0:
            raise EggError(f"egg_gru_create failed with {rc} (unsupported configuration or HIP error)")

    def close(self):
        if self._h:
            lib().egg_gru_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _ck(self, rc, what):
        if rc != 0:
            raise EggError(f"{what} failed with {rc}: {lib().egg_gru_last_error(self._h).decode()}")

    def model_bytes(self):
        return int(lib().egg_gru_model_bytes(self._h))

    def model_init(self, seed=42):
        self._ck(lib().egg_gru_model_init(self._h, seed), "egg_gru_model_init")

    def model_upload(self, arr):
        self._ck(lib().egg_gru_model_upload(self._h, _np_ptr(arr), arr.nbytes), "egg_gru_model_upload")

    def model_download(self):
        import numpy as np
        out = np.zeros(self.model_bytes(), np.int8)
        self._ck(lib().egg_gru_model_download(self._h, _np_ptr(out), out.nbytes), "egg_gru_model_download")
        return out

    def forward_mode(self, staged=True):
        """stages spread over the whole GPU, one launch per pipeline tick (default), or one persistent workgroup per 32 members; same results"""
        self._ck(lib().egg_gru_forward_mode(self._h, 1 if staged else 0), "egg_gru_forward_mode")

    def state_reset(self):
        self._ck(lib().egg_gru_state_reset(self._h), "egg_gru_state_reset")

    def state_download(self):
        import numpy as np
        c = self.cfg
        out = np.zeros(c.population * c.n_layers * c.hidden, np.int8)
        self._ck(lib().egg_gru_state_download(self._h, _np_ptr(out), out.nbytes), "egg_gru_state_download")
        return out

    def step(self, d_data, data_len, start_idx, step_seed, do_update=True):
        self._ck(lib().egg_gru_step(self._h, C.c_void_p(d_data), data_len, start_idx, step_seed & 0xFFFFFFFF,
                                    1 if do_update else 0), "egg_gru_step")

    def losses(self):
        import numpy as np
        loss = np.zeros(self.cfg.population, np.int32)
        fit = np.zeros(self.cfg.population // 2, np.int32)
        self._ck(lib().egg_gru_losses(self._h, _np_ptr(loss), _np_ptr(fit)), "egg_gru_losses")
        return loss, fit

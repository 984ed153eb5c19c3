"""CPU checks of the drop-in boundary: the C-ABI library loads without a GPU and exports every function that
include/egg_hip.h declares; nothing under the product package touches the oracle."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "egg_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(egg_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg.lib()
    names = declared_functions()
    assert len(names) > 30
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    assert set(pkg.EXPORTS) <= set(names), sorted(set(pkg.EXPORTS) - set(names))


def test_default_config_matches_reference_defaults(pkg):
    c = pkg.default_config()
    assert (c.hidden, c.head_dim, c.n_layers, c.vocab) == (256, 64, 4, 256)
    assert (c.fixed_point, c.sigma_shift, c.sigma_shift_vector) == (4, 3, 4)
    assert (c.shift_attn, c.shift_out, c.shift_logit, c.shift_mlp_up, c.shift_mlp_down) == (8, 9, 8, 8, 10)
    assert c.softmax_scale_bit == 18 and c.rope_scale_bit == 20 and c.noise_mask == 15
    assert abs(c.adam_beta1 - 0.9) < 1e-7 and abs(c.adam_beta2 - 0.95) < 1e-7 and abs(c.muon_momentum - 0.85) < 1e-7
    assert pkg.learning_rate(0) == ctypes.c_float(0.3).value and pkg.learning_rate(1000) == ctypes.c_float(0.05).value
    # d-eggs seed chain == murmur3 fmix32(seed + step * golden)
    assert pkg.next_seed(42, 0) == 0x087FCD5C and pkg.next_seed(42, 1) == 0x3805EA2C


def test_product_sources_do_not_reference_the_oracle():
    bad = []
    for base, _, files in os.walk(os.path.join(ROOT, "egg.c_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp", "Makefile")):
                txt = open(os.path.join(base, f), errors="ignore").read()
                if "oracle" in txt.lower() and f != "__init__.py":
                    bad.append(f)
                if f == "__init__.py" and re.search(r"import\s+oracle|oracle_py|libegg_oracle", txt):
                    bad.append(f)
    assert not bad, bad


def test_bench_refuses_more_than_one_gpu():
    """One GPU per box: asking bench.py for more must end with a message, before anything touches a device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)


def test_unsupported_configurations_are_refused_with_a_reason(pkg):
    """egg_ctx_create validates the configuration before it touches the device, so the refusals (and the reason
    egg_last_error(NULL) keeps for them) can be checked without a GPU."""
    lib = pkg.lib()
    for kw, word in ((dict(hidden=100), "hidden"), (dict(head_dim=48), "head_dim"), (dict(seq_len=48), "seq_len"),
                     (dict(population=7), "population"), (dict(rope_scale_bit=31), "rope_scale_bit"),
                     (dict(noise_mask=60, sigma_shift_vector=0), "noise_mask"), (dict(weight_limit=0), "weight_limit"),
                     (dict(noise_mask=127), "noise too wide"), (dict(device_gaussian=1, noise_mask=50), "Gaussian"),
                     (dict(hidden=512, device_gaussian=1), "noise too wide"),
                     (dict(shift_mlp_up=40), "shift"), (dict(softmax_scale_bit=21), "three 7-bit planes"),
                     (dict(softmax_scale_bit=30), "softmax_scale_bit"), (dict(shift_mlp_up=23), "shift_mlp_up is too large"),
                     (dict(shift_mlp_up=24, hidden=512), "shift_mlp_up is too large"), (dict(softmax_exp_scale=0.0), "softmax_exp_scale")):
        cfg = pkg.default_config(**kw)
        h = ctypes.c_void_p()
        rc = lib.egg_ctx_create(ctypes.byref(cfg), ctypes.byref(h))
        assert rc == -1 and not h.value, kw
        assert word in lib.egg_last_error(None).decode(), (kw, lib.egg_last_error(None))


def test_deggs_sampling_constants_match_the_oracle(pkg, orc):
    """Host-only: (int)(penalty * 2^shift_logit) and (int)(logf(min_p) * softmax_exp_scale), d-eggs/src/kernels.cu:386-387."""
    for kw in (dict(), dict(shift_logit=6, softmax_exp_scale=10.0), dict(shift_logit=0)):
        cfg, ocfg = pkg.default_config(**kw), orc.config(**kw)
        for min_p in (0.08, 0.0, 1.0, 0.5, 1e-30, 2.0, -1.0, 0.3333):
            for penalty in (0.2, 0.0, 1.0, -0.01, 7.77, 1e12):
                assert pkg.deggs_sampling_constants(cfg, min_p, penalty) == orc.deggs_sampling_constants(ocfg, min_p, penalty), (kw, min_p, penalty)


def test_muon_workspace_plan_holds_every_batch(pkg):
    """The batched Muon update runs each shape group at its own batch limit; the limit times the matrix size (and
    times the Gram size) must fit the shared workspace for every group, also where the groups' limits differ
    (hidden 512 with 16 or 32 layers: 64 or 128 square matrices at a limit of 64, 17 or 33 of each 4:1 shape at 16)."""
    for hidden, layers in ((64, 2), (256, 4), (256, 5), (512, 8), (512, 16), (512, 32), (1024, 6)):
        cfg = pkg.default_config(hidden=hidden, head_dim=64, n_layers=layers, seq_len=32, population=4, use_muon=1)
        groups, elems, bterm = pkg.muon_plan(cfg)
        assert {(g["rows"], g["cols"]) for g in groups} == {(hidden, hidden), (hidden, 4 * hidden), (4 * hidden, hidden)}
        by = {(g["rows"], g["cols"]): g for g in groups}
        assert by[(hidden, hidden)]["members"] == 4 * layers
        assert by[(hidden, 4 * hidden)]["members"] == layers + 1 and by[(4 * hidden, hidden)]["members"] == layers + 1
        for g in groups:
            k = min(g["rows"], g["cols"])
            assert 1 <= g["batch"] <= g["members"]
            assert g["batch"] * g["rows"] * g["cols"] <= elems, (hidden, layers, g)
            assert g["batch"] * k * k <= bterm, (hidden, layers, g)
        assert elems >= 4 * hidden * hidden and bterm >= hidden * hidden        # a single matrix of any shape (egg_update_tensor)
    groups, elems, _ = pkg.muon_plan(pkg.default_config(hidden=512, head_dim=64, n_layers=16, seq_len=32, population=4, use_muon=1))
    by = {(g["rows"], g["cols"]): g["batch"] for g in groups}
    assert by[(512, 512)] == 64 and by[(512, 2048)] == 16 and by[(2048, 512)] == 16 and elems == 16 << 20


def test_benchmark_stream_generator(pkg, orc):
    """The package's synthetic stream (what bench.py feeds the GPU) is the stream the tests feed the oracle."""
    import numpy as np
    a = pkg.zipf_bytes(1 << 16, seed=1234)
    assert a.dtype == np.uint8 and np.array_equal(a, orc.zipf_bytes(1 << 16, seed=1234))
    counts = np.sort(np.bincount(a, minlength=256))[::-1]
    assert counts[0] > 4 * counts[15] > 0            # Zipf-like: rank 1 far above rank 16 (ratio 16^1.1 = 21)

"""GPU parity of the reference's CPU program (full_trained_egg.c) on the GPU, through the C ABI, against the
scalar restatement in oracle/egg_gru_oracle.cpp: per-member losses, pair fitness, recurrent states and the
updated int8 weights, bit for bit, over consecutive steps (the recurrent state carries over)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _t(dev, arr):
    import torch
    return torch.from_numpy(np.ascontiguousarray(arr)).to(dev)


@pytest.mark.parametrize("kw,steps", [
    (dict(hidden=64, n_layers=2, seq_len=6, population=32, update_threshold=12), 3),
    (dict(hidden=128, n_layers=1, seq_len=5, population=64, update_threshold=20), 2),
    (dict(hidden=512, n_layers=4, seq_len=3, population=32, update_threshold=10), 2),
    (dict(hidden=256, n_layers=2, seq_len=4, population=96, update_threshold=30), 2),
    (dict(hidden=64, n_layers=1, seq_len=9, population=32, update_threshold=5, sigma_shift=2), 3),
    (dict(hidden=128, n_layers=4, seq_len=11, population=32, update_threshold=8), 2),
    (dict(hidden=64, n_layers=2, seq_len=70, population=64, update_threshold=12), 2),     # more ticks than one graph holds
    (dict(hidden=128, n_layers=1, seq_len=100, population=32, update_threshold=6), 2),    # two graph launches in the pipeline's steady state
    (dict(hidden=64, n_layers=1, seq_len=1, population=32, update_threshold=3), 2),
    (dict(hidden=256, n_layers=2, seq_len=16, population=1024, update_threshold=200), 1),  # 32 member tiles
], ids=["h64", "h128", "h512", "h256_p96", "sigma_2", "h128_l4_t11", "h64_t70", "h128_t100", "t1", "h256_p1024"])
@pytest.mark.parametrize("staged", [True, False, None], ids=["launch_per_tick", "persistent_workgroups", "alternating"])
def test_gru_steps(pkg, orc, dev, kw, steps, staged):
    import ctypes as C
    g = orc.gru_config(**kw)
    data = orc.zipf_bytes(1 << 14)
    model = orc.gru_init_model(g, 42)
    rng = np.random.default_rng(3)
    # non-trivial biases so clipped_add and the gates see every term
    L, H = kw["n_layers"], kw["hidden"]
    off_b = 256 * H + L * 4 * H * H
    model[off_b:off_b + L * 2 * H] = rng.integers(-30, 31, L * 2 * H).astype(np.int8)
    ctx = pkg.GruContext(pkg.gru_default_config(**kw))
    if staged is not None:
        ctx.forward_mode(staged)
    assert ctx.model_bytes() == model.size
    ctx.model_init(42)
    got0 = ctx.model_download()
    ref0 = orc.gru_init_model(g, 42)
    assert np.array_equal(got0, ref0)
    ctx.model_upload(model)
    d_data = _t(dev, data)
    P = kw["population"]
    states = np.zeros(P * L * H, np.int8)
    for step in range(steps):
        seed = 1000 + 77 * step
        start = step * kw["seq_len"]
        if staged is None:                      # the recurrent state is handed from one way of evaluating to the other
            ctx.forward_mode(step % 2 == 0)
        ctx.step(d_data.data_ptr(), len(data), start, seed, True)
        loss, fit = ctx.losses()
        ref_loss, ref_fit = orc.gru_population(g, model, data, start, seed, 0, P // 2, states)
        assert np.array_equal(loss, ref_loss), f"step {step}: gpu {loss[:8]} ref {ref_loss[:8]}"
        assert np.array_equal(fit, ref_fit)
        assert np.array_equal(ctx.state_download(), states), f"step {step} recurrent states"
        orc.lib().orc_gru_update_all(C.byref(g), model.ctypes.data_as(C.c_void_p), C.c_uint32(seed), ref_fit.ctypes.data_as(C.c_void_p))
        got = ctx.model_download()
        assert np.array_equal(got, model), f"step {step}: {np.count_nonzero(got != model)} weights differ"
    assert np.count_nonzero(model != ref0) > 0
    ctx.close()


def test_gru_training_reduces_the_loss(pkg, orc, dev):
    """full_trained_egg.c prints its loss while it trains (:576-586); 200 steps of a small model on the synthetic stream
    bring the mean loss per token down by a tenth or more, in both ways of evaluating the forward alike."""
    data = orc.zipf_bytes(1 << 22)
    d_data = _t(dev, data)
    runs = []
    for staged in (True, False):
        ctx = pkg.GruContext(pkg.gru_default_config(hidden=64, n_layers=1, seq_len=64, population=128, update_threshold=20))
        ctx.forward_mode(staged)
        ctx.model_init(42)
        hist = []
        for step in range(200):
            ctx.step(d_data.data_ptr(), len(data), step * 64, 1000 + step, True)
            if step < 3 or step >= 197:
                hist.append(float(ctx.losses()[0].mean()) / 64)
        runs.append(hist)
        ctx.close()
    assert runs[0] == runs[1]
    first, last = np.mean(runs[0][:3]), np.mean(runs[0][3:])
    assert last < 0.9 * first, (first, last)


def test_gru_config_errors(pkg, dev):
    with pytest.raises(pkg.EggError):
        pkg.GruContext(pkg.gru_default_config(hidden=100))
    with pytest.raises(pkg.EggError):
        pkg.GruContext(pkg.gru_default_config(population=30))

"""Ternary-packed matrix weights and the weight limit on the GPU (extensions without a reference counterpart; the CPU
oracle states the same packing and update rule): unpack on upload, forward on the unpacked weights, training steps
that keep the matrices ternary, pack on download."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _t(dev, arr):
    import torch
    return torch.from_numpy(np.ascontiguousarray(arr)).to(dev)


def _ternary_model(orc, ocfg, seed):
    rng = np.random.default_rng(seed)
    model = orc.init_model(ocfg, 42)
    for t in orc.tensor_table(ocfg):
        if t["is_matrix"]:
            n = t["rows"] * t["cols"]
            model[t["offset"]:t["offset"] + n] = rng.integers(-1, 2, n)
    return model


@pytest.mark.parametrize("kw", [dict(hidden=64, head_dim=32, n_layers=2, seq_len=32, population=16),
                                dict(hidden=256, head_dim=64, n_layers=1, seq_len=64, population=8)], ids=["h64", "h256"])
def test_ternary_upload_train_download(pkg, orc, dev, kw):
    kw = dict(kw, weight_limit=1)
    ocfg = orc.config(**kw)
    model = _ternary_model(orc, ocfg, 3)
    packed = orc.ternary_model_pack(ocfg, model)
    data = orc.zipf_bytes(1 << 15)
    d_data = _t(dev, data)
    ctx = pkg.Context(pkg.default_config(**kw))
    assert ctx.ternary_model_bytes() == packed.size
    ctx.model_upload_ternary(packed)
    assert np.array_equal(ctx.model_download(), model)
    assert np.array_equal(ctx.model_download_ternary(), packed)
    state = np.zeros(model.size, orc.ADAM_DTYPE)
    seed = 42
    for step in range(5):
        lr = 6.0
        start = step * kw["seq_len"]
        ctx.step(d_data.data_ptr(), len(data), start, seed, lr)
        loss, fit = ctx.step_losses()
        ref_loss = orc.population_forward(ocfg, model, data, start, seed)
        assert np.array_equal(loss, ref_loss), f"step {step} losses"
        n_ref = orc.es_update_adam(ocfg, model, state, orc.fitness(ref_loss), seed, lr)
        assert np.array_equal(ctx.model_download(), model), f"step {step} weights"
        assert ctx.last_update_count() == n_ref
        seed = pkg.next_seed(seed, step + 1)
    assert np.array_equal(ctx.model_download_ternary(), orc.ternary_model_pack(ocfg, model))
    assert ctx.opt_state_download().tobytes() == state.tobytes()
    ctx.close()


def test_ternary_download_refuses_int8_weights(pkg, dev):
    ctx = pkg.Context(pkg.default_config(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=4))
    ctx.model_init(42)                      # the reference's int8 initialisation: not ternary
    with pytest.raises(pkg.EggError):
        ctx.model_download_ternary()
    with pytest.raises(pkg.EggError):
        ctx.model_upload_ternary(np.zeros(5, np.uint8))
    ctx.close()
    with pytest.raises(pkg.EggError):
        pkg.Context(pkg.default_config(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=4, weight_limit=0))


def test_muon_respects_the_weight_limit(pkg, orc, dev):
    import torch
    kw = dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=32, use_muon=1, weight_limit=1)
    ocfg = orc.config(**{k: v for k, v in kw.items() if k != "use_muon"})
    model = _ternary_model(orc, ocfg, 4)
    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_upload(model)
    rng = np.random.default_rng(1)
    d_seed = _t(dev, np.array([77], np.uint32).view(np.int32))
    d_lr = _t(dev, np.array([40.0], np.float32))
    for step in range(3):
        d_fit = _t(dev, rng.integers(-1, 2, 16).astype(np.int32))
        ctx.es_update(d_fit.data_ptr(), d_seed.data_ptr(), d_lr.data_ptr())
    got = ctx.model_download()
    assert not np.array_equal(got, model)
    for t in ctx.tensors():
        if t["is_matrix"]:
            seg = got[t["offset"]:t["offset"] + t["rows"] * t["cols"]]
            assert seg.min() >= -1 and seg.max() <= 1, t["name"]
    ctx.model_download_ternary()
    ctx.close()

"""Randomised configurations (sizes, shifts, noise forms, data addressing, chunking, adaptive overlay): per-member losses
and one whole ES step (weights, AdamW state, overlay) against the oracle.  Seeded, so every run sees the same cases."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _cases(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        H = int(rng.choice([64, 128, 256, 512])); HD = int(rng.choice([32, 64]))
        T = int(rng.choice([32, 64, 128, 256] if H < 512 else [32, 64]))
        kw = dict(hidden=H, head_dim=HD, n_layers=int(rng.integers(1, 3)), seq_len=T, population=int(rng.choice([2, 4, 6])))
        if rng.random() < 0.5:
            kw.update(sigma_shift=int(rng.integers(0, 6)), sigma_shift_vector=int(rng.integers(2, 7)), shift_attn=int(rng.integers(6, 11)),
                      shift_out=int(rng.integers(7, 11)), shift_logit=int(rng.integers(6, 10)), shift_mlp_up=int(rng.integers(6, 10)),
                      shift_mlp_down=int(rng.integers(8, 12)), noise_mask=int(rng.choice([0, 1, 3, 7, 15, 31])))
        if rng.random() < 0.25 and H <= 256 and kw.get("noise_mask", 15) <= 15:
            kw.update(device_gaussian=1)
        if rng.random() < 0.25:
            kw.update(host_gaussian=1)
        if rng.random() < 0.2:
            kw.update(use_same_data=1)
        if rng.random() < 0.3:
            kw.update(softmax_scale_bit=int(rng.integers(10, 19)), rope_scale_bit=int(rng.integers(12, 28)))
        out.append((kw, int(rng.choice([0, 1, 3])), bool(rng.random() < 0.35), int(rng.integers(1, 1 << 30))))
    return out


@pytest.mark.parametrize("block", range(4))
def test_random_configurations_follow_the_oracle(pkg, orc, dev, block):
    import torch
    for kw, chunk, adaptive, s in _cases(100 + block, 10):
        rng = np.random.default_rng(s)
        T, P = kw["seq_len"], kw["population"]
        ocfg = orc.config(**kw)
        ctx = pkg.Context(pkg.default_config(chunk_members=chunk, **kw))
        data = orc.zipf_bytes(int(rng.integers(4 * T + 2, 1 << 13)), seed=int(rng.integers(1, 1000)))
        if rng.random() < 0.2:
            data[:] = data[0]                       # a window of one repeated byte
        model = orc.init_model(ocfg, int(rng.integers(1, 1 << 30)))
        used = np.zeros(model.size, bool)
        for t in orc.tensor_table(ocfg):
            used[t["offset"]:t["offset"] + (t["rows"] + t["cols"] if t["is_matrix"] else t["cols"])] = True
            if not t["is_matrix"]:
                sl = slice(t["offset"], t["offset"] + t["cols"])
                model[sl] = rng.integers(-30, 31, t["cols"]).astype(np.int8) + (16 if t["name"].startswith("ln_") and "bias" not in t["name"] else 0)
        ctx.model_upload(model)
        overlay = None
        if adaptive:
            ctx.adaptive_enable(64, 5, 1)
            overlay = rng.integers(-20, 100, model.size).astype(np.int8)
            ctx.overlay_upload(overlay)
        d_data = torch.from_numpy(data).to(dev)
        start, seed, lr = int(rng.integers(0, 1 << 20)), int(rng.integers(0, 1 << 32)), float(rng.choice([0.3, 3.0]))
        d_loss = torch.zeros(P, dtype=torch.int32, device=dev)
        ctx.population_forward(d_data.data_ptr(), len(data), start, seed, 0, P, d_loss.data_ptr())
        ctx.sync()
        ref = orc.population_forward(ocfg, model, data, start, seed, overlay=overlay)
        assert np.array_equal(d_loss.cpu().numpy(), ref), (kw, chunk, adaptive)
        ctx.step(d_data.data_ptr(), len(data), start, seed, lr)
        ctx.sync()
        want = model.copy()
        state = np.zeros(model.size, orc.ADAM_DTYPE)
        if adaptive:
            orc.es_update_adam_adaptive(ocfg, want, state, overlay, orc.fitness(ref), seed, np.float32(lr), 5, 1)
            assert np.array_equal(ctx.overlay_download()[used], overlay[used]), (kw, "overlay")
        else:
            orc.es_update_adam(ocfg, want, state, orc.fitness(ref), seed, np.float32(lr))
        assert np.array_equal(ctx.model_download(), want), (kw, chunk, adaptive)
        got = ctx.opt_state_download().view(orc.ADAM_DTYPE)
        for f in ("m", "v", "acc"):
            assert np.array_equal(got[f].view(np.int32), state[f].view(np.int32)), (kw, f)
        ctx.close()

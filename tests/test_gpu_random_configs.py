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


def _extreme_cases():
    """Shifts and table scales over the whole range egg_ctx_create accepts, the corners first."""
    base = dict(hidden=128, head_dim=32, n_layers=1, seq_len=32, population=2)
    out = [dict(base, shift_mlp_up=22), dict(base, hidden=512, head_dim=64, shift_mlp_up=21),
           dict(base, hidden=512, head_dim=64, shift_mlp_up=15, sigma_shift=3),       # the bias seed no longer fits the fused form
           dict(base, hidden=256, head_dim=64, shift_mlp_up=16), dict(base, shift_mlp_up=0, shift_mlp_down=0, shift_out=0),
           dict(base, softmax_scale_bit=20), dict(base, hidden=256, head_dim=64, seq_len=256, softmax_scale_bit=20, softmax_exp_scale=40.0),
           dict(base, softmax_scale_bit=1), dict(base, shift_attn=0, shift_logit=0), dict(base, shift_attn=24, shift_logit=24, shift_out=24, shift_mlp_down=24),
           dict(base, fixed_point=4, sigma_shift=20), dict(base, fixed_point=0, sigma_shift=0, noise_mask=7), dict(base, sigma_shift_vector=0, noise_mask=7),
           dict(base, sigma_shift_vector=24)]
    rng = np.random.default_rng(4711)
    for _ in range(10):
        H = int(rng.choice([64, 128, 256, 512]))
        out.append(dict(hidden=H, head_dim=int(rng.choice([32, 64])), n_layers=1, seq_len=int(rng.choice([32, 64])), population=2,
                        sigma_shift=int(rng.integers(0, 21)), sigma_shift_vector=int(rng.integers(0, 25)), shift_attn=int(rng.integers(0, 25)),
                        shift_out=int(rng.integers(0, 25)), shift_logit=int(rng.integers(0, 25)), shift_mlp_up=int(rng.integers(0, 22)),
                        shift_mlp_down=int(rng.integers(0, 25)), softmax_scale_bit=int(rng.integers(1, 21)), rope_scale_bit=int(rng.integers(1, 31)),
                        noise_mask=int(rng.choice([1, 3, 7, 15]))))
    return out


def test_shift_and_table_scale_extremes_follow_the_oracle(pkg, orc, dev):
    """Every stage, the logits and the loss at the edges of the accepted configuration space: the up projection's
    bias is folded into its accumulator shifted left by shift_mlp_up, and the attention weights are split into three
    7-bit planes, so both ends of both ranges are exercised (with biases that are not zero)."""
    import torch
    for kw in _extreme_cases():
        rng = np.random.default_rng(kw["hidden"] + 7 * kw.get("shift_mlp_up", 8))
        T, P = kw["seq_len"], kw["population"]
        ocfg = orc.config(**kw)
        model = orc.init_model(ocfg, 42)
        for t in orc.tensor_table(ocfg):
            if not t["is_matrix"]:
                sl = slice(t["offset"], t["offset"] + t["cols"])
                model[sl] = rng.integers(-127, 128, t["cols"]).astype(np.int8) if "bias" in t["name"] else rng.integers(1, 40, t["cols"]).astype(np.int8)
        ctx = pkg.Context(pkg.default_config(**kw))
        ctx.model_upload(model)
        ctx.enable_taps(True)
        data = orc.zipf_bytes(1 << 12)
        d_data = torch.from_numpy(data).to(dev)
        d_loss = torch.zeros(P, dtype=torch.int32, device=dev)
        start, seed = 5 * T, 24680
        ctx.population_forward(d_data.data_ptr(), len(data), start, seed, 0, P, d_loss.data_ptr())
        ctx.sync()
        for m in range(P):
            ref_loss, tr = orc.forward_member(ocfg, model, data, start, seed, m, trace=True)
            for st in ["x_init"] + [f"{n}.0" for n in ("q", "k", "v", "ao", "x_attn", "x_mlp")]:
                exp = tr[st.split(".")[0]][0] if "." in st else tr[st]
                assert np.array_equal(ctx.tap(st, m), exp), (kw, m, st)
            assert np.array_equal(ctx.tap("logits", m), tr["logits"]), (kw, m)
            assert int(d_loss[m].item()) == ref_loss, (kw, m)
        ctx.close()

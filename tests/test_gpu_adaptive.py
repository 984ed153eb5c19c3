"""d-eggs adaptive noise overlay on the GPU against the CPU oracle: every stage tap and the losses of a forward under a
random overlay, and whole optimizer steps (captured as a graph) whose overlay evolves with the weight changes."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _t(dev, arr):
    import torch
    arr = np.ascontiguousarray(arr)
    if arr.dtype == np.uint32:          # same bytes; torch's own uint32 support is partial
        arr = arr.view(np.int32)
    return torch.from_numpy(arr).to(dev)


def _model_with_nontrivial_vectors(orc, ocfg, seed):
    model = orc.init_model(ocfg, 42)
    rng = np.random.default_rng(seed)
    for t in orc.tensor_table(ocfg):
        if not t["is_matrix"]:
            sl = slice(t["offset"], t["offset"] + t["cols"])
            model[sl] = rng.integers(-20, 21, t["cols"]).astype(np.int8) + (16 if t["name"].startswith("ln_") and "bias" not in t["name"] else 0)
    return model


@pytest.mark.parametrize("kw", [dict(hidden=64, head_dim=32, n_layers=2, seq_len=32, population=6),
                                dict(hidden=128, head_dim=32, n_layers=1, seq_len=64, population=4),
                                dict(hidden=256, head_dim=64, n_layers=2, seq_len=64, population=4),
                                dict(hidden=512, head_dim=64, n_layers=1, seq_len=32, population=2),
                                dict(hidden=256, head_dim=64, n_layers=1, seq_len=64, population=4, sigma_shift=5, noise_mask=31),
                                dict(hidden=128, head_dim=32, n_layers=1, seq_len=32, population=4, vocab=768)],
                         ids=["h64", "h128", "h256", "h512", "wide_noise", "vocab_768"])
def test_adaptive_forward_stages_and_loss(pkg, orc, dev, kw):
    import torch
    ocfg = orc.config(**kw)
    data = orc.zipf_bytes(1 << 15)
    if ocfg.vocab > 256:                     # uint32 tokens over the whole vocabulary
        data = ((data[0::2].astype(np.uint32) << 8 | data[1::2]) % ocfg.vocab).astype(np.uint32)
    model = _model_with_nontrivial_vectors(orc, ocfg, 5)
    rng = np.random.default_rng(17)
    # every regime of the factor: below zero, fractional, saturated
    overlay = rng.choice(np.array([-128, -3, 0, 1, 7, 31, 32, 33, 50, 63, 64, 65, 127], np.int8), model.size).astype(np.int8)
    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_upload(model)
    ctx.adaptive_enable(64)
    ctx.overlay_upload(overlay)
    assert np.array_equal(ctx.overlay_download(), overlay)
    ctx.enable_taps(True)
    d_data = _t(dev, data)
    P = kw["population"]
    d_loss = torch.zeros(P, dtype=torch.int32, device=dev)
    seed, start = 1357911, 2 * kw["seq_len"]
    ctx.population_forward(d_data.data_ptr(), len(data), start, seed, 0, P, d_loss.data_ptr())
    ctx.sync()
    problems = []
    for m in range(P):
        ref_loss, tr = orc.forward_member(ocfg, model, data, start, seed, m, trace=True, overlay=overlay)
        stages = ["x_init"] + [f"{n}.{l}" for l in range(kw["n_layers"]) for n in ("q", "k", "v", "ao", "x_attn", "x_mlp")]
        for st in stages:
            got = ctx.tap(st, m)
            exp = tr[st.split(".")[0]][int(st.split(".")[1])] if "." in st else tr[st]
            if not np.array_equal(got, exp):
                bad = np.argwhere(got != exp)
                problems.append(f"member {m} stage {st}: {len(bad)}/{exp.size} differ, first at {bad[0].tolist()} "
                                f"gpu {got[tuple(bad[0])]} ref {exp[tuple(bad[0])]}")
                break
        else:
            got = ctx.tap("logits", m)
            if not np.array_equal(got, tr["logits"]):
                bad = np.argwhere(got != tr["logits"])
                problems.append(f"member {m} logits: {len(bad)} differ, first {bad[0].tolist()}")
            elif int(d_loss[m].item()) != ref_loss:
                problems.append(f"member {m} loss gpu {int(d_loss[m].item())} ref {ref_loss}")
    # an overlay of 64 everywhere is the plain forward
    ctx.enable_taps(False)
    ctx.overlay_upload(np.full(model.size, 64, np.int8))
    ctx.population_forward(d_data.data_ptr(), len(data), start, seed, 0, P, d_loss.data_ptr())
    ctx.sync()
    plain = orc.population_forward(ocfg, model, data, start, seed)
    ctx.close()
    assert not problems, "\n".join(problems[:12])
    assert np.array_equal(d_loss.cpu().numpy(), plain)


@pytest.mark.parametrize("mode", ["eager", "graph"])
def test_adaptive_steps_follow_the_oracle(pkg, orc, dev, mode):
    kw = dict(hidden=64, head_dim=32, n_layers=2, seq_len=32, population=32)
    data = orc.zipf_bytes(1 << 15)
    ocfg = orc.config(**kw)
    d_data = _t(dev, data)
    model = orc.init_model(ocfg, 42)
    state = np.zeros(model.size, orc.ADAM_DTYPE)
    overlay = np.full(model.size, 64, np.int8)
    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_init(42)
    ctx.adaptive_enable(64, 5, 1)
    if mode == "graph":
        ctx.step_capture(d_data.data_ptr(), len(data))
    used = np.zeros(model.size, bool)
    for t in orc.tensor_table(ocfg):
        used[t["offset"]:t["offset"] + (t["rows"] + t["cols"] if t["is_matrix"] else t["cols"])] = True
    seed = 42
    for step in range(8):
        lr = 3.0
        start = step * kw["seq_len"]
        if mode == "graph":
            ctx.step_launch(start, seed, lr)
        else:
            ctx.step(d_data.data_ptr(), len(data), start, seed, lr)
        loss, fit = ctx.step_losses()
        ref_loss = orc.population_forward(ocfg, model, data, start, seed, overlay=overlay)
        assert np.array_equal(loss, ref_loss), f"{mode} step {step} losses"
        ref_fit = orc.fitness(ref_loss)
        n_ref = orc.es_update_adam_adaptive(ocfg, model, state, overlay, ref_fit, seed, lr, 5, 1)
        assert np.array_equal(ctx.model_download(), model), f"{mode} step {step} weights"
        assert ctx.last_update_count() == n_ref
        got_ov = ctx.overlay_download()
        assert np.array_equal(got_ov[used], overlay[used]), f"{mode} step {step} overlay"
        seed = pkg.next_seed(seed, step + 1)
    assert (overlay[used] < 64).any() and (overlay[used] > 64).any()
    ctx.close()


def test_adaptive_errors(pkg, dev):
    ctx = pkg.Context(pkg.default_config(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=4))
    with pytest.raises(pkg.EggError):
        ctx.overlay_download()                       # not enabled yet
    with pytest.raises(pkg.EggError):
        ctx.adaptive_enable(300)
    ctx.adaptive_enable()
    with pytest.raises(pkg.EggError):
        ctx.overlay_upload(np.zeros(3, np.int8))
    ctx.close()
    ctx = pkg.Context(pkg.default_config(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=4, use_muon=1))
    with pytest.raises(pkg.EggError):
        ctx.adaptive_enable()
    ctx.close()

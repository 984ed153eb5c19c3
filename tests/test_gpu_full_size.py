"""Checks at the sizes the headline numbers are quoted on (4 layers, hidden 256, 4 heads, sequence 256; populations
8192 and 40,960).  The CPU oracle needs about 0.75 s per member at this shape, so whole populations are checked
through properties that do not depend on the size (determinism, independence of the chunking, sub-range evaluation,
antithetic pairs that coincide when the noise is zero, linearity of the votes) and a sample of members / tensors is
compared bit-for-bit with the oracle."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SHAPE = dict(hidden=256, head_dim=64, n_layers=4, seq_len=256)


def _t(dev, arr):
    import torch
    return torch.from_numpy(np.ascontiguousarray(arr)).to(dev)


def _forward(pkg, dev, cfg_kw, model, d_data, data_len, start, seed, offset=0, count=None, repeat=1, dedup=True):
    import torch
    pop = cfg_kw["population"]
    count = pop if count is None else count
    ctx = pkg.Context(pkg.default_config(**cfg_kw))
    ctx.model_upload(model)
    ctx.first_block_dedup(dedup)
    out = []
    for _ in range(repeat):
        d_loss = torch.full((pop,), -1, dtype=torch.int32, device=dev)
        ctx.population_forward(d_data.data_ptr(), data_len, start, seed, offset, count, d_loss.data_ptr())
        ctx.sync()
        out.append(d_loss.cpu().numpy())
    ctx.close()
    return out


def test_population_8192_forward(pkg, orc, dev):
    pop = 8192
    kw = dict(population=pop, **SHAPE)
    data = orc.zipf_bytes(1 << 22)
    ocfg = orc.config(**kw)
    model = orc.init_model(ocfg, 42)
    d_data = _t(dev, data)
    start, seed = 3 * 256, 0xC0FFEE

    a, b = _forward(pkg, dev, dict(chunk_members=2048, **kw), model, d_data, len(data), start, seed, repeat=2)
    assert np.array_equal(a, b), "two evaluations of the same step differ"
    assert (a > 0).all()
    # a chunk size that is neither a divisor of the population nor a multiple of the workgroup's member count
    (c,) = _forward(pkg, dev, dict(chunk_members=1001, **kw), model, d_data, len(data), start, seed)
    assert np.array_equal(a, c), f"{np.count_nonzero(a != c)} losses depend on the chunking"
    # the first block evaluated at every position instead of once per distinct byte value of a window
    (e,) = _forward(pkg, dev, dict(chunk_members=2048, **kw), model, d_data, len(data), start, seed, dedup=False)
    assert np.array_equal(a, e), f"{np.count_nonzero(a != e)} losses depend on the form of the first block"
    # a sub-range leaves the rest of the output alone
    (d,) = _forward(pkg, dev, dict(chunk_members=2048, **kw), model, d_data, len(data), start, seed, offset=4094, count=6)
    assert np.array_equal(d[4094:4100], a[4094:4100]) and (d[:4094] == -1).all() and (d[4100:] == -1).all()

    # sampled members against the oracle: first pair, members around both chunkings' boundaries, last pair
    for first, n in ((0, 2), (1000, 2), (2046, 4), (8190, 2)):
        ref = orc.population_forward(ocfg, model, data, start, seed, first, n)
        assert np.array_equal(a[first:first + n], ref[first:first + n]), (first, a[first:first + n], ref[first:first + n])

    # zero noise: both members of a pair evaluate the unperturbed model on the same bytes
    (z,) = _forward(pkg, dev, dict(chunk_members=2048, noise_mask=0, **kw), model, d_data, len(data), start, seed)
    assert np.array_equal(z[0::2], z[1::2])
    zcfg = orc.config(noise_mask=0, **kw)
    ref = orc.population_forward(zcfg, model, data, start, seed, 4094, 2)
    assert np.array_equal(z[4094:4096], ref[4094:4096])


def test_population_40960_step(pkg, orc, dev):
    import torch
    pop = 40960
    pairs = pop // 2
    kw = dict(population=pop, **SHAPE)
    data = orc.zipf_bytes(1 << 23)
    ocfg = orc.config(**kw)
    model = orc.init_model(ocfg, 42)
    d_data = _t(dev, data)
    start, seed, lr = 0, 20261, 0.3

    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_upload(model)
    d_loss = torch.zeros(pop, dtype=torch.int32, device=dev)
    d_fit = torch.zeros(pairs, dtype=torch.int32, device=dev)
    ctx.population_forward(d_data.data_ptr(), len(data), start, seed, 0, pop, d_loss.data_ptr())
    ctx.fitness(d_loss.data_ptr(), d_fit.data_ptr(), pairs)
    ctx.sync()
    loss = d_loss.cpu().numpy()
    fit = d_fit.cpu().numpy()
    assert np.array_equal(fit, np.sign(loss[1::2].astype(np.int64) - loss[0::2]).astype(np.int32))
    assert np.array_equal(fit, orc.fitness(loss))
    assert np.count_nonzero(fit) > pairs // 2, "degenerate fitness"
    for first in (0, 20478, 40958):
        ref = orc.population_forward(ocfg, model, data, start, seed, first, 2)
        assert np.array_equal(loss[first:first + 2], ref[first:first + 2]), first

    d_seed = _t(dev, np.array([seed], np.uint32).view(np.int32))
    d_lr = _t(dev, np.array([lr], np.float32))
    tensors = {t["name"]: t for t in ctx.tensors()}
    checked = [tensors["w_q.1"], tensors["embedding"], tensors["ln_2.3"]]
    # votes of two matrices over all 20,480 pairs; negating every fitness negates every vote
    d_neg = -d_fit
    for t in checked[:2]:
        n = t["rows"] * t["cols"]
        d_votes = torch.zeros(n, dtype=torch.int32, device=dev)
        d_votes_neg = torch.zeros(n, dtype=torch.int32, device=dev)
        ctx.matrix_votes(t["id"], d_fit.data_ptr(), d_seed.data_ptr(), d_votes.data_ptr())
        ctx.matrix_votes(t["id"], d_neg.data_ptr(), d_seed.data_ptr(), d_votes_neg.data_ptr())
        ctx.sync()
        ref = np.zeros(n, np.int32)
        orc.lib().orc_matrix_votes(C.byref(ocfg), t["rows"], t["cols"], t["off_a"], t["off_b"], t["seed_base"],
                                   fit.ctypes.data_as(C.c_void_p), pairs, C.c_uint32(seed), ref.ctypes.data_as(C.c_void_p))
        assert np.array_equal(d_votes.cpu().numpy(), ref), t["name"]
        assert torch.equal(d_votes_neg, -d_votes), t["name"]

    # the whole update; the sampled tensors against the oracle's per-tensor update
    ctx.es_update(d_fit.data_ptr(), d_seed.data_ptr(), d_lr.data_ptr())
    got_m = ctx.model_download()
    got_s = ctx.opt_state_download().view(orc.ADAM_DTYPE)
    assert ctx.last_update_count() == np.count_nonzero(got_m != model)
    for t in checked:
        n = t["rows"] * t["cols"]
        w = model[t["offset"]:t["offset"] + n].copy()
        st = np.zeros(n, orc.ADAM_DTYPE)
        if t["is_matrix"]:
            orc.lib().orc_update_matrix_adam(C.byref(ocfg), w.ctypes.data_as(C.c_void_p), st.ctypes.data_as(C.c_void_p),
                                             t["rows"], t["cols"], t["off_a"], t["off_b"], t["seed_base"],
                                             fit.ctypes.data_as(C.c_void_p), pairs, C.c_uint32(seed),
                                             C.c_float(lr * t["lr_scale"]))
        else:
            orc.lib().orc_update_vector_adam(C.byref(ocfg), w.ctypes.data_as(C.c_void_p), st.ctypes.data_as(C.c_void_p),
                                             n, t["off_a"], t["off_b"], t["seed_base"],
                                             fit.ctypes.data_as(C.c_void_p), pairs, C.c_uint32(seed),
                                             C.c_float(lr * t["lr_scale"]))
        sl = slice(t["offset"], t["offset"] + n)
        assert np.array_equal(got_m[sl], w), t["name"]
        for f in ("m", "v", "acc"):
            assert np.array_equal(got_s[f][sl].view(np.int32), st[f].view(np.int32)), (t["name"], f)
    ctx.close()

    # the same step through the one-call entry point on a fresh context ends in the same weights
    ctx2 = pkg.Context(pkg.default_config(**kw))
    ctx2.model_upload(model)
    ctx2.step(d_data.data_ptr(), len(data), start, seed, lr)
    ctx2.sync()
    assert np.array_equal(ctx2.model_download(), got_m)
    ctx2.close()


def test_population_40960_fifty_graph_steps_match_eager(pkg, orc, dev):
    """The headline run shape itself: 50 replays of the captured step graph at population 40,960, with a learning rate
    large enough that weights change every step.  Eager launches of the same 50 steps from the same start must give
    the same losses at every step and the same weights and optimizer state at the end; the first step's sampled
    members are the oracle's (test_population_40960_step covers the update of that step)."""
    pop = 40960
    kw = dict(population=pop, **SHAPE)
    data = orc.zipf_bytes(1 << 23)
    d_data = _t(dev, data)
    steps, lr = 50, 8.0
    trace = {}
    for mode in ("eager", "graph"):
        ctx = pkg.Context(pkg.default_config(**kw))
        ctx.model_init(42)
        if mode == "graph":
            ctx.step_capture(d_data.data_ptr(), len(data))
        seed, losses, updates = 42, [], 0
        for step in range(steps):
            start = step * SHAPE["seq_len"]
            if mode == "graph":
                ctx.step_launch(start, seed, lr)
            else:
                ctx.step(d_data.data_ptr(), len(data), start, seed, lr)
            if step % 7 == 0 or step == steps - 1:
                losses.append(ctx.step_losses()[0].copy())
                updates += ctx.last_update_count()
            seed = pkg.next_seed(seed, step + 1)
        trace[mode] = (losses, updates, ctx.model_download().copy(), ctx.opt_state_download().copy())
        ctx.close()
    e, g = trace["eager"], trace["graph"]
    assert e[1] > 0, "no weight changed: the trajectory would not test the update"
    for i, (a, b) in enumerate(zip(e[0], g[0])):
        assert np.array_equal(a, b), f"losses differ at checkpoint {i}"
    assert np.array_equal(e[2], g[2]), "weights after 50 steps"
    assert np.array_equal(e[3], g[3]), "optimizer state after 50 steps"
    ocfg = orc.config(**kw)
    model = orc.init_model(ocfg, 42)
    ref = orc.population_forward(ocfg, model, data, 0, 42, 20478, 2)
    assert np.array_equal(e[0][0][20478:20480], ref[20478:20480])


def test_population_40960_one_launch_equals_chunks_of_8192(pkg, orc, dev):
    """The default evaluates the whole population in one launch per kernel (2.7 GB per activation buffer: row offsets
    pass 2^31); five launches of 8192 members must give the same per-member losses."""
    import torch
    pop = 40960
    kw = dict(population=pop, **SHAPE)
    data = orc.zipf_bytes(1 << 23)
    d_data = _t(dev, data)
    model = orc.init_model(orc.config(**kw), 42)
    got = {}
    for chunk in (0, 8192):
        ctx = pkg.Context(pkg.default_config(chunk_members=chunk, **kw))
        ctx.model_upload(model)
        d_loss = torch.full((pop,), -1, dtype=torch.int32, device=dev)
        ctx.population_forward(d_data.data_ptr(), len(data), 512, 777, 0, pop, d_loss.data_ptr())
        ctx.sync()
        got[chunk] = d_loss.cpu().numpy()
        ctx.close()
    assert got[0].min() > 0
    assert np.array_equal(got[0], got[8192])


def test_population_40960_steps_checked_link_by_link(pkg, orc, dev):
    """A trajectory at the headline size whose every link is held against the oracle on samples: before each of ten
    steps the weights and the optimizer state come back from the GPU; the oracle then evaluates two sampled pairs on
    those weights (they depend on every tensor of the model), and applies the step's update to a matrix and a vector
    tensor of its own from that state and the step's fitness.  Losses, updated weights and float state must agree bit
    for bit at every step; the sampled pairs and tensors change from step to step."""
    import torch
    pop = 40960
    pairs = pop // 2
    kw = dict(population=pop, **SHAPE)
    data = orc.zipf_bytes(1 << 23)
    ocfg = orc.config(**kw)
    d_data = _t(dev, data)
    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_init(42)
    tensors = {t["name"]: t for t in ctx.tensors()}
    plan = [("w_q.0", "ln_1.2"), ("w_o.3", "mlp_bias_up.1"), ("embedding", "ln_f"), ("w_k.2", "emb_bias"), ("w_v.1", "ln_2_bias.0"),
            ("w_up.2", "ln_init"), ("w_down.0", "mlp_bias_down.3"), ("w_emb_mlp_up", "ln_f_bias"), ("w_emb_mlp_down", "ln_1_bias.1"),
            ("w_q.3", "mlp_emb_bias_up")]
    seed, lr = 42, 8.0
    changed = 0
    for step, names in enumerate(plan):
        start = step * SHAPE["seq_len"]
        model = ctx.model_download().copy()
        state = ctx.opt_state_download().view(orc.ADAM_DTYPE).copy()
        ctx.step(d_data.data_ptr(), len(data), start, seed, lr)
        loss, fit = ctx.step_losses()
        assert np.array_equal(fit, orc.fitness(loss))
        for first in ((7919 * (step + 1)) % pop & ~1, (20011 * (step + 3)) % pop & ~1, pop - 2 - 2 * step):
            ref = orc.population_forward(ocfg, model, data, start, seed, first, 2)
            assert np.array_equal(loss[first:first + 2], ref[first:first + 2]), (step, first)
        got_m = ctx.model_download()
        got_s = ctx.opt_state_download().view(orc.ADAM_DTYPE)
        changed += ctx.last_update_count()
        for name in names:
            t = tensors[name]
            n = t["rows"] * t["cols"]
            sl = slice(t["offset"], t["offset"] + n)
            w = model[sl].copy()
            st = state[sl].copy()
            if t["is_matrix"]:
                orc.lib().orc_update_matrix_adam(C.byref(ocfg), w.ctypes.data_as(C.c_void_p), st.ctypes.data_as(C.c_void_p),
                                                 t["rows"], t["cols"], t["off_a"], t["off_b"], t["seed_base"],
                                                 fit.ctypes.data_as(C.c_void_p), pairs, C.c_uint32(seed), C.c_float(lr * t["lr_scale"]))
            else:
                orc.lib().orc_update_vector_adam(C.byref(ocfg), w.ctypes.data_as(C.c_void_p), st.ctypes.data_as(C.c_void_p),
                                                 n, t["off_a"], t["off_b"], t["seed_base"],
                                                 fit.ctypes.data_as(C.c_void_p), pairs, C.c_uint32(seed), C.c_float(lr * t["lr_scale"]))
            assert np.array_equal(got_m[sl], w), (step, name, np.count_nonzero(got_m[sl] != w))
            for f in ("m", "v", "acc"):
                assert np.array_equal(got_s[f][sl].view(np.int32), st[f].view(np.int32)), (step, name, f)
        seed = pkg.next_seed(seed, step + 1)
    assert changed > 0, "no weight changed: the trajectory would not test the update"
    ctx.close()

"""The benchmark configurations at their full sizes, checked: the single perturbed linear at 8192 members x 128 tokens x
512 x 512, the reference's CPU program (full_trained_egg.c) at its compiled-in defaults, and the composed d-eggs-style
model (hidden 512, 8 layers, 8 heads, sequence 512, ternary-packed weights, Muon, population 16,384).  Whole outputs
are held against size-independent properties and plain PyTorch integer arithmetic on the GPU; sampled members, pairs and
tensors against the CPU oracle, bit for bit (Muon within the tolerance its fp32 matrix products allow)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _t(dev, arr):
    import torch
    return torch.from_numpy(np.ascontiguousarray(arr)).to(dev)


def _np_noise(seed, idx, mask=15):
    """noise_from_hash (mgpu.cu:525-538) in numpy, independent of the oracle library"""
    with np.errstate(over="ignore"):
        x = (np.uint32(seed & 0xFFFFFFFF) + np.asarray(idx, np.uint32) * np.uint32(0x9E3779B9)).astype(np.uint32)
        x ^= x >> np.uint32(16); x *= np.uint32(0x85EBCA6B); x ^= x >> np.uint32(13); x *= np.uint32(0xC2B2AE35); x ^= x >> np.uint32(16)
    return np.where(x & 1, 1, -1).astype(np.int32) * ((x >> np.uint32(1)) & np.uint32(mask)).astype(np.int32)


# ---------------------------------------------------------------------------------------------------------------------
# config 2: one perturbed linear, X [8192 members x 128 tokens][512], W [512][512]
@pytest.mark.parametrize("own_noise", [0, 1], ids=["pair_noise", "own_noise"])
def test_perturbed_linear_8192x128x512x512(pkg, orc, dev, own_noise):
    import torch
    members, T, K, N, seed, oa, ob = 8192, 128, 512, 512, 3, 200, 201
    rows = members * T
    g = torch.Generator(device=dev); g.manual_seed(1)
    X = torch.randint(-127, 128, (rows, K), dtype=torch.int8, device=dev, generator=g)
    rng = np.random.default_rng(2)
    W = rng.integers(-127, 128, size=(K, N), dtype=np.int8)
    Wb = np.zeros(K * N, np.int8)
    orc.lib().orc_repack(Wb.ctypes.data_as(C.c_void_p), W.ctypes.data_as(C.c_void_p), K, N)
    dW = _t(dev, Wb)
    cfg_kw = dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=8)
    ctx = pkg.Context(pkg.default_config(**cfg_kw))
    ocfg = orc.config(**cfg_kw)
    call = ctx.perturbed_linear_own_noise if own_noise else ctx.perturbed_linear
    y32 = torch.empty((rows, N), dtype=torch.int32, device=dev)
    y8 = torch.empty((rows, N), dtype=torch.int8, device=dev)
    acc = torch.empty((rows, N), dtype=torch.int32, device=dev)
    call(X.data_ptr(), dW.data_ptr(), members, T, K, N, seed, oa, ob, 8, y32.data_ptr(), y8.data_ptr())
    call(X.data_ptr(), dW.data_ptr(), members, T, K, N, seed, oa, ob, 0, acc.data_ptr(), None)
    ctx.sync()

    # the whole output against plain PyTorch arithmetic on the GPU: x.W in float64 (exact: |sum| < 2^24) and the rank-1
    # term floor(((x.B) * A[n] * ns) / 2^7) in int64, A and B from a numpy restatement of the hash
    groups = members if own_noise else members // 2          # members that share one noise draw
    per = members // groups
    A = np.stack([_np_noise(seed + p + oa, np.arange(N)) for p in range(groups)])
    B = np.stack([_np_noise(seed + p + ob, np.arange(K)) for p in range(groups)])
    dA, dB, Wd = _t(dev, A).long(), _t(dev, B).double(), _t(dev, W).double()
    ns = torch.ones(per * T, dtype=torch.int64, device=dev)
    if not own_noise:
        ns[T:] = -1
    step = 256                                               # noise groups per slice
    for g0 in range(0, groups, step):
        r0, r1 = g0 * per * T, (g0 + step) * per * T
        xs = X[r0:r1].double()
        plain = (xs @ Wd).long()
        sb = torch.bmm(xs.view(step, per * T, K), dB[g0:g0 + step].unsqueeze(2)).squeeze(2).long()          # [step][per*T]
        pert = torch.div(sb.unsqueeze(2) * dA[g0:g0 + step].unsqueeze(1) * ns.view(1, -1, 1), 128, rounding_mode="floor")
        want = plain + pert.view(-1, N)
        assert torch.equal(acc[r0:r1].long(), want), f"accumulators of noise groups {g0}..{g0 + step}"
        assert torch.equal(y32[r0:r1].long(), want >> 8)
        assert torch.equal(y8[r0:r1].long(), torch.clamp(want >> 8, -127, 127))
        del xs, plain, sb, pert, want
    if not own_noise:
        # sampled pairs against the CPU oracle: a pair's rows handed over as members 0 and 1 with the pair folded into the seed
        for pair in (0, 1, 2047, 2048, 4095) + tuple(int(v) for v in rng.integers(0, members // 2, 11)):
            sl = slice(2 * pair * T, (2 * pair + 2) * T)
            ref = orc.perturbed_linear(ocfg, X[sl].cpu().numpy(), Wb, T, K, N, seed + pair, oa, ob, 8)
            assert np.array_equal(y32[sl].cpu().numpy(), ref), pair
            assert np.array_equal(y8[sl].cpu().numpy(), np.clip(ref, -127, 127).astype(np.int8)), pair
    # the shared-weight product alone
    ctx.shared_linear(X.data_ptr(), dW.data_ptr(), members, T, K, N, 0, acc.data_ptr(), None)
    ctx.sync()
    for r0 in range(0, rows, 1 << 17):
        assert torch.equal(acc[r0:r0 + (1 << 17)].long(), (X[r0:r0 + (1 << 17)].double() @ Wd).long())
    ctx.close()


# ---------------------------------------------------------------------------------------------------------------------
# config 1: full_trained_egg.c at its compiled-in defaults (full_trained_egg.c:11-21)
def test_gru_program_at_reference_defaults(pkg, orc, dev):
    g = orc.gru_config()
    gcfg = pkg.gru_default_config()
    for name, want in (("hidden", 512), ("n_layers", 4), ("seq_len", 4096), ("vocab", 256), ("population", 128),
                       ("fixed_point", 4), ("sigma_shift", 4), ("update_threshold", 160)):
        assert getattr(g, name) == want and getattr(gcfg, name) == want, name
    P, L, H, T = g.population, g.n_layers, g.hidden, g.seq_len
    data = orc.zipf_bytes(1 << 20)
    model = orc.gru_init_model(g, 42)
    ctx = pkg.GruContext(gcfg)
    ctx.model_init(42)
    assert np.array_equal(ctx.model_download(), model)
    d_data = _t(dev, data)
    seed, start = 20251, 5 * T
    ctx.step(d_data.data_ptr(), len(data), start, seed, True)
    loss, fit = ctx.losses()
    states = ctx.state_download()
    got_model = ctx.model_download()
    assert np.array_equal(fit, np.sign(loss[1::2].astype(np.int64) - loss[0::2]).astype(np.int32))
    assert loss.min() > 0 and np.count_nonzero(fit) > P // 4
    # four sampled pairs, full length, against the oracle: losses, fitness and the recurrent state they leave behind
    sb = L * H
    ref_states = np.zeros(P * sb, np.int8)
    for pair in (0, 21, 42, 63):
        ref_loss, ref_fit = orc.gru_population(g, model, data, start, seed, pair, 1, ref_states)
        assert np.array_equal(loss[2 * pair:2 * pair + 2], ref_loss[2 * pair:2 * pair + 2]), pair
        assert fit[pair] == ref_fit[pair]
        assert np.array_equal(states[2 * pair * sb:(2 * pair + 2) * sb], ref_states[2 * pair * sb:(2 * pair + 2) * sb]), pair
    # the whole integer update, every matrix, from the GPU's fitness vector
    ref_model = model.copy()
    orc.lib().orc_gru_update_all(C.byref(g), ref_model.ctypes.data_as(C.c_void_p), C.c_uint32(seed), fit.ctypes.data_as(C.c_void_p))
    moved = np.count_nonzero(ref_model != model)
    assert moved > 0, "no weight moved: the update comparison would be vacuous"
    assert np.array_equal(got_model, ref_model), f"{np.count_nonzero(got_model != ref_model)} of {moved} moved weights differ"
    ctx.close()


# ---------------------------------------------------------------------------------------------------------------------
# config 5: d-eggs-style model, ternary-packed weights, Muon
def _ternary_model(orc, ocfg, seed):
    rng = np.random.default_rng(seed)
    model = orc.init_model(ocfg, 42)
    for t in orc.tensor_table(ocfg):
        if t["is_matrix"]:
            n = t["rows"] * t["cols"]
            model[t["offset"]:t["offset"] + n] = rng.integers(-1, 2, n)
    return model


def test_deggs_style_h512_l8_t512_ternary_muon_population_16384(pkg, orc, dev):
    import torch
    pop, pairs = 16384, 8192
    kw = dict(hidden=512, head_dim=64, n_layers=8, seq_len=512, population=pop, weight_limit=1)
    ocfg = orc.config(**kw)
    model = _ternary_model(orc, ocfg, 5)
    packed = orc.ternary_model_pack(ocfg, model)
    data = orc.zipf_bytes(1 << 24)
    d_data = _t(dev, data)
    start, seed, lr = 7 * 512, 0xD0E5, 40.0

    losses = {}
    for chunk in (0, 2048, 1500):
        ctx = pkg.Context(pkg.default_config(use_muon=1, chunk_members=chunk, **kw))
        ctx.model_upload_ternary(packed)
        if chunk == 0:
            assert np.array_equal(ctx.model_download(), model)
        d_loss = torch.full((pop,), -1, dtype=torch.int32, device=dev)
        reps = 2 if chunk == 0 else 1
        for rep in range(reps):
            ctx.population_forward(d_data.data_ptr(), len(data), start, seed, 0, pop, d_loss.data_ptr())
            ctx.sync()
            got = d_loss.cpu().numpy()
            if rep:
                assert np.array_equal(got, losses[chunk]), "two evaluations of the same step differ"
            losses[chunk] = got
        if chunk:
            ctx.close()
        else:
            keep = ctx
    loss = losses[0]
    assert loss.min() > 0
    for chunk in (2048, 1500):
        assert np.array_equal(loss, losses[chunk]), f"{np.count_nonzero(loss != losses[chunk])} losses depend on the chunking ({chunk})"
    # sampled members against the oracle: the first pair, a pair on a chunk boundary of both chunkings, the last pair
    for first in (0, 2046, 2999, pop - 2):
        first &= ~1
        ref = orc.population_forward(ocfg, model, data, start, seed, first, 2)
        assert np.array_equal(loss[first:first + 2], ref[first:first + 2]), (first, loss[first:first + 2], ref[first:first + 2])

    # fitness and one Muon update of every matrix on the GPU; two sampled tensors against the oracle's Muon chain
    ctx = keep
    d_loss = _t(dev, loss)
    d_fit = torch.zeros(pairs, dtype=torch.int32, device=dev)
    ctx.fitness(d_loss.data_ptr(), d_fit.data_ptr(), pairs)
    ctx.sync()
    fit = d_fit.cpu().numpy()
    assert np.array_equal(fit, orc.fitness(loss)) and np.count_nonzero(fit) > pairs // 2
    d_seed = _t(dev, np.array([seed], np.uint32).view(np.int32))
    d_lr = _t(dev, np.array([lr], np.float32))
    ctx.es_update(d_fit.data_ptr(), d_seed.data_ptr(), d_lr.data_ptr())
    got_m = ctx.model_download()
    raw = ctx.opt_state_download().view(np.uint8)
    assert ctx.last_update_count() == np.count_nonzero(got_m != model) > 0
    tensors = {t["name"]: t for t in ctx.tensors()}
    for t in tensors.values():
        if t["is_matrix"]:
            seg = got_m[t["offset"]:t["offset"] + t["rows"] * t["cols"]]
            assert seg.min() >= -1 and seg.max() <= 1, t["name"]
    ctx.model_download_ternary()                     # still packable
    for name in ("w_q.3", "w_up.5"):
        t = tensors[name]
        assert t["muon"] and (t["rows"], t["cols"]) == ((512, 512) if name == "w_q.3" else (512, 2048))
        n = t["rows"] * t["cols"]
        W = model[t["offset"]:t["offset"] + n].copy()
        st = np.zeros(n, orc.MUON_DTYPE)
        orc.lib().orc_update_matrix_muon(C.byref(ocfg), W.ctypes.data_as(C.c_void_p), st.ctypes.data_as(C.c_void_p),
                                         t["rows"], t["cols"], t["off_a"], t["off_b"], t["seed_base"],
                                         fit.ctypes.data_as(C.c_void_p), pairs, C.c_uint32(seed), C.c_float(lr), None)
        off = ctx.tensor_state_offset(t["id"])
        got_st = raw[off:off + 8 * n].view(orc.MUON_DTYPE)
        got_w = got_m[t["offset"]:t["offset"] + n]
        # momentum: integer votes and two float operations, bit for bit
        assert np.array_equal(got_st["m"].view(np.int32), st["m"].view(np.int32)), name
        # the orthogonalised step went through fp32 matrix products whose summation order the reference leaves to
        # cuBLAS: weights may differ only where an accumulator sits within rounding distance of the +-1 threshold
        diff = np.flatnonzero(got_w != W)
        assert len(diff) <= max(2, n // 500), (name, len(diff))
        assert (np.abs(got_w[diff].astype(np.int32) - W[diff]) == 1).all()
        same = got_w == W
        assert np.allclose(got_st["acc"][same], st["acc"][same], atol=2e-3), name
        assert np.count_nonzero(W != model[t["offset"]:t["offset"] + n]) > 0, "the oracle moved no weight of " + name
    ctx.close()


def test_deggs_default_vocabulary_8192(pkg, orc, dev):
    """The d-eggs-style configuration with d-eggs' default vocabulary (VOCAB_SIZE 8192, uint32 tokens): 2048 members in
    one launch per kernel -- determinism, sampled pairs and the embedding's votes against the oracle."""
    import torch
    pop, pairs = 2048, 1024
    kw = dict(hidden=512, head_dim=64, n_layers=8, seq_len=512, population=pop, weight_limit=1, vocab=8192)
    ocfg = orc.config(**kw)
    model = _ternary_model(orc, ocfg, 6)
    raw = orc.zipf_bytes(1 << 23)
    # 13-bit tokens from two Zipf bytes: frequent tokens stay frequent, the whole vocabulary is reachable
    data = ((raw[0::2].astype(np.uint32) << 8 | raw[1::2]) % 8192).astype(np.uint32)
    assert int(data.max()) == 8191
    d_data = _t(dev, data.view(np.int32))
    start, seed = 5 * 512, 0xBEE5
    ctx = pkg.Context(pkg.default_config(use_muon=1, **kw))
    ctx.model_upload_ternary(orc.ternary_model_pack(ocfg, model))
    assert np.array_equal(ctx.model_download(), model)
    d_loss = torch.full((pop,), -1, dtype=torch.int32, device=dev)
    runs = []
    for rep in range(2):
        ctx.population_forward(d_data.data_ptr(), len(data), start, seed, 0, pop, d_loss.data_ptr())
        ctx.sync()
        runs.append(d_loss.cpu().numpy())
    loss = runs[0]
    assert np.array_equal(loss, runs[1]), "two evaluations of the same step differ"
    assert loss.min() > 0
    for first in (0, pop - 2):
        ref = orc.population_forward(ocfg, model, data, start, seed, first, 2)
        assert np.array_equal(loss[first:first + 2], ref[first:first + 2]), (first, loss[first:first + 2], ref[first:first + 2])
    # the embedding (512 x 8192, the widest vote panel) against the oracle's votes
    fit = orc.fitness(loss)
    d_fit = _t(dev, fit)
    d_seed = _t(dev, np.array([seed], np.uint32).view(np.int32))
    t = {t["name"]: t for t in ctx.tensors()}["embedding"]
    assert (t["rows"], t["cols"]) == (512, 8192)
    n = t["rows"] * t["cols"]
    d_votes = torch.zeros(n, dtype=torch.int32, device=dev)
    ctx.matrix_votes(t["id"], d_fit.data_ptr(), d_seed.data_ptr(), d_votes.data_ptr())
    ctx.sync()
    ref = np.zeros(n, np.int32)
    orc.lib().orc_matrix_votes(C.byref(ocfg), t["rows"], t["cols"], t["off_a"], t["off_b"], t["seed_base"],
                               fit.ctypes.data_as(C.c_void_p), pairs, C.c_uint32(seed), ref.ctypes.data_as(C.c_void_p))
    assert np.array_equal(d_votes.cpu().numpy(), ref)
    ctx.close()

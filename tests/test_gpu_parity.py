"""GPU parity tests: every call goes through the C ABI of libegg_hip.so and is compared bit-for-bit with the
CPU oracle on the same seeded inputs."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SMALL = dict(hidden=64, head_dim=32, n_layers=2, seq_len=32, population=8)


def _t(dev, arr):
    import torch
    arr = np.ascontiguousarray(arr)
    if arr.dtype == np.uint32:          # same bytes; torch's own uint32 support is partial
        arr = arr.view(np.int32)
    return torch.from_numpy(arr).to(dev)


def _mapping_hint(got, exp):
    """When a row of `got` is a column permutation of `exp`, say which one (layout debugging aid)."""
    hints = []
    for r in range(min(2, got.shape[0])):
        e, g = exp[r], got[r]
        if len(set(e.tolist())) < len(e) * 0.9:
            continue
        pos = {int(v): i for i, v in enumerate(g.tolist())}
        m = [pos.get(int(v), -1) for v in e.tolist()]
        hints.append(f"row {r}: expected col i found at gpu col {m[:64]}")
    return "\n".join(hints)


def test_tables_and_model_init(pkg, orc, dev):
    for kw in (SMALL, dict(hidden=256, head_dim=64, n_layers=1, seq_len=64, population=4),
               dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=4, host_gaussian=1)):
        ctx = pkg.Context(pkg.default_config(**kw))
        ocfg = orc.config(**kw)
        ex, act, rope = ctx.tables()
        oex, oact, orope = orc.tables(ocfg)
        assert np.array_equal(ex, oex) and np.array_equal(act, oact) and np.array_equal(rope, orope)
        ctx.model_init(42)
        assert np.array_equal(ctx.model_download(), orc.init_model(ocfg, 42))
        names = [t["name"] for t in ctx.tensors()]
        assert names == [t["name"] for t in orc.tensor_table(ocfg)]
        for a, b in zip(ctx.tensors(), orc.tensor_table(ocfg)):
            for k in ("is_matrix", "rows", "cols", "offset", "off_a", "off_b", "seed_base", "muon"):
                assert a[k] == b[k], (a, b)
        ctx.close()


def test_noise_fill(pkg, orc, dev):
    import torch
    ctx = pkg.Context(pkg.default_config(**SMALL))
    for seed, first, n in ((42, 0, 1000), (0xFFFFFFFF, 7, 513), (123456789, 4000000000, 64)):
        out = torch.zeros(n, dtype=torch.int8, device=dev)
        ctx.noise_fill(seed, first, n, out.data_ptr())
        ctx.sync()
        assert np.array_equal(out.cpu().numpy(), orc.noise_vec(seed, n, 15, first)), (seed, first)
    ctx.close()
    # DEVICE_GAUSSIAN: the sum of three masked fields (mask word 15 | 0x100 in the oracle)
    ctx = pkg.Context(pkg.default_config(device_gaussian=1, **SMALL))
    out = torch.zeros(4096, dtype=torch.int8, device=dev)
    ctx.noise_fill(777, 5, 4096, out.data_ptr())
    ctx.sync()
    got = out.cpu().numpy()
    assert np.array_equal(got, orc.noise_vec(777, 4096, 15 | 0x100, 5)) and got.min() < -30 and got.max() > 30
    ctx.close()


# the last two cases use a wider noise (mask 31, sigma 9): the kernel's fused perturb-and-shift form would overflow
# there, so they take its two-shift form
@pytest.mark.parametrize("K,N,members,T,extra", [(64, 64, 4, 32, {}), (256, 256, 6, 64, {}), (512, 512, 8, 32, {}),
                                                 (256, 1024, 3, 32, {}), (1024, 256, 2, 32, {}),
                                                 (512, 512, 5, 128, {}), (256, 1024, 3, 64, {}), (512, 128, 2, 192, {}),
                                                 (256, 64, 7, 64, {}), (512, 192, 3, 64, {}), (256, 320, 2, 128, {}),
                                                 (512, 64, 2, 64, {}), (512, 1024, 1, 128, {}),
                                                 (256, 256, 5, 256, dict(sigma_shift=5, noise_mask=31)),
                                                 (512, 512, 3, 64, dict(sigma_shift=5, noise_mask=31)),
                                                 (1024, 256, 2, 32, dict(sigma_shift=5, noise_mask=31))])
def test_perturbed_linear(pkg, orc, dev, K, N, members, T, extra):
    import torch
    rng = np.random.default_rng(K * 7 + N)
    ctx = pkg.Context(pkg.default_config(**SMALL, **extra))
    ocfg = orc.config(**SMALL, **extra)
    X = rng.integers(-127, 128, size=(members * T, K), dtype=np.int8)
    W = rng.integers(-127, 128, size=(K, N), dtype=np.int8)
    Wb = np.zeros(K * N, np.int8)
    orc.lib().orc_repack(Wb.ctypes.data_as(C.c_void_p), W.ctypes.data_as(C.c_void_p), K, N)
    for shift in (0, 8):
        ref = orc.perturbed_linear(ocfg, X, Wb, T, K, N, 3, 200, 201, shift)
        dX, dW = _t(dev, X), _t(dev, Wb)
        y32 = torch.zeros((members * T, N), dtype=torch.int32, device=dev)
        y8 = torch.zeros((members * T, N), dtype=torch.int8, device=dev)
        ctx.perturbed_linear(dX.data_ptr(), dW.data_ptr(), members, T, K, N, 3, 200, 201, shift, y32.data_ptr(), y8.data_ptr())
        ctx.sync()
        got = y32.cpu().numpy()
        if not np.array_equal(got, ref):
            bad = np.argwhere(got != ref)
            plain = (X.astype(np.int64) @ W.astype(np.int64))
            raise AssertionError(
                f"perturbed linear K={K} N={N} shift={shift}: {len(bad)} of {ref.size} differ; first {bad[:5].tolist()}\n"
                f"gpu[0,:16]={got[0, :16].tolist()}\nref[0,:16]={ref[0, :16].tolist()}\nplain xW>>s[0,:16]={(plain[0, :16] >> shift).tolist()}\n"
                + _mapping_hint(got, ref))
        assert np.array_equal(y8.cpu().numpy(), np.clip(ref, -127, 127).astype(np.int8))
        # the shared-weight product alone (the reference's ns == 0 case): the textbook integer matrix product
        y32.fill_(7); y8.fill_(7)
        ctx.shared_linear(dX.data_ptr(), dW.data_ptr(), members, T, K, N, shift, y32.data_ptr(), y8.data_ptr())
        ctx.sync()
        plain = (X.astype(np.int64) @ W.astype(np.int64)) >> shift
        assert np.array_equal(y32.cpu().numpy(), plain), f"shared linear K={K} N={N} shift={shift}"
        assert np.array_equal(y8.cpu().numpy(), np.clip(plain, -127, 127).astype(np.int8))
    ctx.close()


# Shapes the W-stationary kernel serves (K x 512, K = 256 or 512), at member counts below, at and above the number of
# workgroups (one per CU, members dealt round-robin), with one to five 32-token tiles per member, pair noise and own
# noise, and the two-shift form (wide noise).  Every output is compared with the W-streaming kernel's, the first and
# last pairs with the oracle, and the shared-weight product with the integer matrix product.
@pytest.mark.parametrize("K,members,T,own,extra", [(256, 5, 64, 0, {}), (256, 300, 32, 0, {}), (512, 300, 96, 0, {}), (512, 517, 32, 1, {}),
                                                   (256, 1, 32, 0, {}), (512, 1, 160, 1, {}), (512, 259, 160, 0, dict(sigma_shift=5, noise_mask=31)),
                                                   (256, 258, 128, 1, dict(sigma_shift=5, noise_mask=31)), (512, 256, 32, 0, {}), (512, 2, 32, 0, {}),
                                                   # K = 256 keeps a ring of 12 tile slots and waits on exact counts once 10 tiles
                                                   # are in flight: 12 to 18 tiles per workgroup (slot wrap-around, steady-state
                                                   # wait), 10 to 15 with an odd tile count per member, and 12 to 15 with a ragged tail
                                                   (256, 600, 192, 0, {}), (256, 700, 160, 1, {}), (256, 1100, 96, 0, dict(sigma_shift=5, noise_mask=31))])
def test_w_stationary_linear(pkg, orc, dev, K, members, T, own, extra):
    import torch
    N = 512
    rng = np.random.default_rng(K + members * 3 + T)
    ctx = pkg.Context(pkg.default_config(**SMALL, **extra))
    ocfg = orc.config(**SMALL, **extra)
    X = rng.integers(-127, 128, size=(members * T, K), dtype=np.int8)
    W = rng.integers(-127, 128, size=(K, N), dtype=np.int8)
    Wb = np.zeros(K * N, np.int8)
    orc.lib().orc_repack(Wb.ctypes.data_as(C.c_void_p), W.ctypes.data_as(C.c_void_p), K, N)
    dX, dW = _t(dev, X), _t(dev, Wb)
    call = ctx.perturbed_linear_own_noise if own else ctx.perturbed_linear
    seed = 0xF00D0000 + members
    for shift in (8, 3):
        outs = []
        # (the W-streaming kernels have no 256 x 512 instance for an odd number of 32-token tiles)
        for ws in ((True, False) if K == 512 or T % 64 == 0 else (True,)):
            ctx.linear_kernel(ws)
            y32 = torch.full((members * T, N), 7, dtype=torch.int32, device=dev)
            y8 = torch.full((members * T, N), 7, dtype=torch.int8, device=dev)
            s32 = torch.full((members * T, N), 7, dtype=torch.int32, device=dev)
            s8 = torch.full((members * T, N), 7, dtype=torch.int8, device=dev)
            call(dX.data_ptr(), dW.data_ptr(), members, T, K, N, seed, 200, 201, shift, y32.data_ptr(), y8.data_ptr())
            ctx.shared_linear(dX.data_ptr(), dW.data_ptr(), members, T, K, N, shift, s32.data_ptr(), s8.data_ptr())
            ctx.sync()
            outs.append((y32, y8, s32, s8))
        for a, b, what in zip(outs[0], outs[-1], ("perturbed int32", "perturbed int8", "shared int32", "shared int8")):
            assert torch.equal(a, b), f"W-stationary and W-streaming kernels differ: {what} K={K} members={members} T={T} shift={shift}"
        plain = (torch.from_numpy(X).to(dev).double() @ torch.from_numpy(W).to(dev).double()).to(torch.int64) >> shift
        assert torch.equal(outs[0][2].to(torch.int64), plain)
        assert torch.equal(outs[0][3].to(torch.int64), plain.clamp(-127, 127))
        assert torch.equal(outs[0][1].to(torch.int32), outs[0][0].clamp(-127, 127))
        # the oracle evaluates pairs (member 2i with +noise, 2i + 1 with -noise, one seed per pair); with own noise every
        # member is the first of a pair of its own seed
        got = outs[0][0].cpu().numpy()
        for m in sorted({0, members - 1}):
            if own:
                ref = orc.perturbed_linear(ocfg, np.concatenate([X[m * T:(m + 1) * T]] * 2), Wb, T, K, N, seed + m, 200, 201, shift)[:T]
            elif m % 2 == 0 and m + 1 >= members:
                ref = orc.perturbed_linear(ocfg, np.concatenate([X[m * T:(m + 1) * T]] * 2), Wb, T, K, N, seed + m // 2, 200, 201, shift)[:T]
            else:
                lo = m - (m % 2)
                ref = orc.perturbed_linear(ocfg, X[lo * T:(lo + 2) * T], Wb, T, K, N, seed + lo // 2, 200, 201, shift)[(m - lo) * T:(m - lo + 1) * T]
            assert np.array_equal(got[m * T:(m + 1) * T], ref), f"member {m} K={K} members={members} T={T} shift={shift}"
    ctx.close()


def _stream(orc, ocfg, n):
    """the synthetic token stream: bytes for the byte-level model, uint32 tokens that reach the whole vocabulary otherwise"""
    data = orc.zipf_bytes(n if ocfg.vocab == 256 else 2 * n)
    if ocfg.vocab > 256:
        data = ((data[0::2].astype(np.uint32) << 8 | data[1::2]) % ocfg.vocab).astype(np.uint32)
    return data


STAGES = ["x_init"] + [f"{n}.{l}" for l in range(2) for n in ("q", "k", "v", "ao", "x_attn", "x_mlp")]


@pytest.mark.parametrize("kw", [SMALL,
                                dict(hidden=128, head_dim=32, n_layers=1, seq_len=64, population=6),
                                dict(hidden=256, head_dim=64, n_layers=2, seq_len=64, population=4),
                                dict(hidden=256, head_dim=64, n_layers=1, seq_len=32, population=6),
                                dict(hidden=64, head_dim=32, n_layers=1, seq_len=256, population=4),
                                dict(hidden=256, head_dim=64, n_layers=1, seq_len=256, population=2),
                                dict(hidden=512, head_dim=64, n_layers=1, seq_len=32, population=4),
                                dict(hidden=512, head_dim=64, n_layers=1, seq_len=128, population=4),
                                dict(hidden=512, head_dim=64, n_layers=2, seq_len=512, population=2),
                                # a wider noise (mask 31, sigma 9) takes the kernels' unfused shift path
                                dict(hidden=256, head_dim=64, n_layers=1, seq_len=64, population=4, sigma_shift=5, noise_mask=31),
                                dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=4, sigma_shift=1, noise_mask=7,
                                     shift_out=8, shift_mlp_up=7, shift_mlp_down=9),
                                # the longest sequence with 32-wide heads, and with hidden 128
                                dict(hidden=64, head_dim=32, n_layers=1, seq_len=512, population=2),
                                dict(hidden=128, head_dim=64, n_layers=1, seq_len=512, population=2),
                                # a RoPE table scale of 2^30, the largest an int32 table holds (products then need all 64 bits)
                                dict(hidden=128, head_dim=64, n_layers=1, seq_len=64, population=2, rope_scale_bit=30),
                                # DEVICE_GAUSSIAN / HOST_GAUSSIAN: noise up to +-45 (the kernels' unfused shift path)
                                dict(hidden=256, head_dim=64, n_layers=2, seq_len=64, population=4, device_gaussian=1, host_gaussian=1),
                                # USE_SAME_DATA: every pair reads the same window
                                dict(hidden=128, head_dim=64, n_layers=1, seq_len=128, population=6, use_same_data=1),
                                # vocabularies of more than 256 entries: uint32 tokens, the head in blocks of 256 columns
                                dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=4, vocab=512),
                                dict(hidden=256, head_dim=64, n_layers=2, seq_len=64, population=4, vocab=1024),
                                dict(hidden=512, head_dim=64, n_layers=1, seq_len=32, population=4, vocab=768),
                                dict(hidden=128, head_dim=32, n_layers=1, seq_len=64, population=6, vocab=2048, sigma_shift=5, noise_mask=31),
                                dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=2, vocab=65536)],
                         ids=["h64", "h128", "h256", "h256_t32", "h64_t256", "h256_t256", "h512_t32", "h512_t128", "h512_t512", "wide_noise", "other_shifts", "h64_t512", "h128_t512", "rope_2_30", "gaussian", "same_data",
                              "vocab_512", "h256_vocab_1024", "h512_vocab_768", "vocab_2048_wide_noise", "vocab_65536"])
def test_forward_stages_and_loss(pkg, orc, dev, kw):
    """Every stage tap of every member against the oracle's trace, then the per-member losses."""
    ocfg = orc.config(**kw)
    data = _stream(orc, ocfg, 1 << 15)
    model = orc.init_model(ocfg, 42)
    # make biases / gains non-trivial so every term of the arithmetic is exercised
    rng = np.random.default_rng(5)
    for t in orc.tensor_table(ocfg):
        if not t["is_matrix"]:
            sl = slice(t["offset"], t["offset"] + t["cols"])
            model[sl] = rng.integers(-20, 21, t["cols"]).astype(np.int8) + (16 if t["name"].startswith("ln_") and "bias" not in t["name"] else 0)
    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_upload(model)
    ctx.enable_taps(True)
    import torch
    d_data = _t(dev, data)
    P = kw["population"]
    d_loss = torch.zeros(P, dtype=torch.int32, device=dev)
    seed, start = 987654321, 3 * kw["seq_len"]
    ctx.population_forward(d_data.data_ptr(), len(data), start, seed, 0, P, d_loss.data_ptr())
    ctx.sync()
    problems = []
    for m in range(P):
        ref_loss, tr = orc.forward_member(ocfg, model, data, start, seed, m, trace=True)
        stages = ["x_init"] + [f"{n}.{l}" for l in range(kw["n_layers"]) for n in ("q", "k", "v", "ao", "x_attn", "x_mlp")]
        for st in stages:
            got = ctx.tap(st, m)
            if "." in st:
                base, l = st.split(".")
                exp = tr[base][int(l)]
            else:
                exp = tr[st]
            if not np.array_equal(got, exp):
                bad = np.argwhere(got != exp)
                problems.append(f"member {m} stage {st}: {len(bad)}/{exp.size} differ, first at {bad[0].tolist()} "
                                f"gpu {got[tuple(bad[0])]} ref {exp[tuple(bad[0])]}; gpu row {got[bad[0][0], :12].tolist()} ref row {exp[bad[0][0], :12].tolist()}")
                break   # later stages of this member inherit the error
        else:
            got = ctx.tap("logits", m)
            if not np.array_equal(got, tr["logits"]):
                bad = np.argwhere(got != tr["logits"])
                problems.append(f"member {m} logits: {len(bad)} differ, first {bad[0].tolist()} gpu {got[tuple(bad[0])]} ref {tr['logits'][tuple(bad[0])]}")
            elif int(d_loss[m].item()) != ref_loss:
                problems.append(f"member {m} loss gpu {int(d_loss[m].item())} ref {ref_loss}")
    ctx.close()
    assert not problems, "\n".join(problems[:12])


@pytest.mark.parametrize("hidden,head_dim,seq_len", [(64, 32, 32), (256, 64, 32), (128, 32, 64), (512, 64, 32)],
                         ids=["h64", "h256_t32", "h128_t64", "h512_t32"])
def test_forward_chunked_and_offsets(pkg, orc, dev, hidden, head_dim, seq_len):
    """Chunked evaluation (chunk smaller than the population, odd tail that leaves padding waves in the last
    workgroup) and a sub-range give the same losses."""
    import torch
    kw = dict(hidden=hidden, head_dim=head_dim, n_layers=1, seq_len=seq_len, population=22)
    data = orc.zipf_bytes(1 << 14)
    ocfg = orc.config(**kw)
    model = orc.init_model(ocfg, 7)
    ref = orc.population_forward(ocfg, model, data, 64, 555)
    ctx = pkg.Context(pkg.default_config(chunk_members=5, **kw))
    ctx.model_upload(model)
    d_data = _t(dev, data)
    d_loss = torch.full((22,), -1, dtype=torch.int32, device=dev)
    ctx.population_forward(d_data.data_ptr(), len(data), 64, 555, 0, 22, d_loss.data_ptr())
    ctx.sync()
    assert np.array_equal(d_loss.cpu().numpy(), ref)
    d_loss.fill_(-1)
    ctx.population_forward(d_data.data_ptr(), len(data), 64, 555, 3, 9, d_loss.data_ptr())
    ctx.sync()
    got = d_loss.cpu().numpy()
    assert np.array_equal(got[3:12], ref[3:12]) and (got[:3] == -1).all() and (got[12:] == -1).all()
    ctx.close()


@pytest.mark.parametrize("hidden,head_dim,distinct", [(256, 64, (1, 2, 64, 65, 128, 129, 256)), (64, 32, (1, 128, 129, 256)),
                                                      (512, 64, (33, 200))], ids=["h256", "h64", "h512"])
def test_first_block_with_repeated_bytes(pkg, orc, dev, hidden, head_dim, distinct):
    """The block in front of the first attention layer is evaluated once per distinct byte value of a member's window:
    windows with 1 ... 256 distinct values (around the multiples of the tokens a workgroup handles per pass), in
    scrambled order, give the oracle's residual stream and losses."""
    import torch
    T = 256
    kw = dict(hidden=hidden, head_dim=head_dim, n_layers=1, seq_len=T, population=2)
    ocfg = orc.config(**kw)
    model = orc.init_model(ocfg, 11)
    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_upload(model)
    ctx.enable_taps(True)
    rng = np.random.default_rng(31)
    for U in distinct:
        values = rng.permutation(256)[:U]
        window = rng.permutation(np.concatenate([values, values[rng.integers(0, U, T - U)]]))
        data = np.zeros(4 * T, np.uint8)
        start = 17
        data[start:start + T] = window.astype(np.uint8)
        data[start + T] = values[0]                      # the last position's target
        assert len(set(data[start:start + T].tolist())) == U
        d_data = _t(dev, data)
        d_loss = torch.zeros(2, dtype=torch.int32, device=dev)
        ctx.population_forward(d_data.data_ptr(), len(data), start, 4242 + U, 0, 2, d_loss.data_ptr())
        ctx.sync()
        for m in range(2):
            ref_loss, tr = orc.forward_member(ocfg, model, data, start, 4242 + U, m, trace=True)
            assert np.array_equal(ctx.tap("x_init", m), tr["x_init"]), (U, m)
            assert int(d_loss[m].item()) == ref_loss, (U, m)
    ctx.close()


def test_fitness(pkg, orc, dev):
    import torch
    ctx = pkg.Context(pkg.default_config(**SMALL))
    loss = np.array([5, 7, 7, 5, 3, 3, -2**31, 2**31 - 1, 0, -1], np.int32)
    d_loss = _t(dev, loss)
    d_fit = torch.zeros(5, dtype=torch.int32, device=dev)
    ctx.fitness(d_loss.data_ptr(), d_fit.data_ptr(), 5)
    ctx.sync()
    assert d_fit.cpu().tolist() == [1, -1, 0, 1, -1] == orc.fitness(loss).tolist()
    ctx.close()


@pytest.mark.parametrize("kw", [dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=200),
                                dict(hidden=128, head_dim=32, n_layers=1, seq_len=32, population=66),
                                dict(hidden=512, head_dim=64, n_layers=1, seq_len=128, population=40),
                                dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=200, device_gaussian=1),
                                dict(hidden=128, head_dim=32, n_layers=1, seq_len=32, population=66, vocab=768)],
                         ids=["p200", "p66", "h512", "gaussian", "vocab_768"])
def test_votes_and_adam_update(pkg, orc, dev, kw):
    import torch
    ocfg = orc.config(**kw)
    cfg = pkg.default_config(**kw)
    ctx = pkg.Context(cfg)
    rng = np.random.default_rng(11)
    pairs = kw["population"] // 2
    fit = rng.integers(-1, 2, pairs).astype(np.int32)
    model = orc.init_model(ocfg, 42)
    model[rng.integers(0, model.size, 50)] = 127      # saturated weights exercise the accumulator clamp
    model[rng.integers(0, model.size, 50)] = -127
    state = np.zeros(model.size, orc.ADAM_DTYPE)
    ctx.model_upload(model)
    d_fit = _t(dev, fit)
    seed = 2024
    d_seed = _t(dev, np.array([seed], np.uint32).view(np.int32))
    d_lr = _t(dev, np.array([0.3], np.float32))
    # votes of each matrix
    for t in ctx.tensors():
        if not t["is_matrix"]:
            continue
        n = t["rows"] * t["cols"]
        d_votes = torch.zeros(n, dtype=torch.int32, device=dev)
        ctx.matrix_votes(t["id"], d_fit.data_ptr(), d_seed.data_ptr(), d_votes.data_ptr())
        ctx.sync()
        ref = np.zeros(n, np.int32)
        orc.lib().orc_matrix_votes(C.byref(ocfg), t["rows"], t["cols"], t["off_a"], t["off_b"], t["seed_base"],
                                   fit.ctypes.data_as(C.c_void_p), pairs, C.c_uint32(seed), ref.ctypes.data_as(C.c_void_p))
        assert np.array_equal(d_votes.cpu().numpy(), ref), t["name"]
    # several full updates: weights, float state and update counter bit-exact
    for step in range(4):
        lr = 0.3 if step < 2 else 5.0      # the large rate drives accumulators through the +-1 thresholds
        d_lr.fill_(lr)
        fit = rng.integers(-1, 2, pairs).astype(np.int32)
        d_fit.copy_(_t(dev, fit))
        s = seed + 17 * step
        d_seed.copy_(_t(dev, np.array([s], np.uint32).view(np.int32)))
        ctx.es_update(d_fit.data_ptr(), d_seed.data_ptr(), d_lr.data_ptr())
        n_ref = orc.es_update_adam(ocfg, model, state, fit, s, lr)
        got_m = ctx.model_download()
        got_s = ctx.opt_state_download().view(orc.ADAM_DTYPE)
        assert np.array_equal(got_m, model), f"step {step}: {np.count_nonzero(got_m != model)} weights differ"
        for f in ("m", "v", "acc"):
            a, b = got_s[f], state[f]
            assert np.array_equal(a.view(np.int32), b.view(np.int32)), \
                f"step {step} state.{f}: {np.count_nonzero(a != b)} differ, max rel {np.max(np.abs(a - b) / (np.abs(b) + 1e-30))}"
        assert ctx.last_update_count() == n_ref
    ctx.close()


@pytest.mark.parametrize("kw", [dict(hidden=64, head_dim=32, n_layers=2, seq_len=32, population=16),
                                dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=16, vocab=512)], ids=["bytes", "vocab_512"])
def test_full_step_eager_and_graph(pkg, orc, dev, kw):
    """Whole ES steps (forward + fitness + update): eager and hipGraph replays follow the oracle's weight trajectory."""
    ocfg = orc.config(**kw)
    data = _stream(orc, ocfg, 1 << 15)
    d_data = _t(dev, data)
    for mode in ("eager", "graph"):
        model = orc.init_model(ocfg, 42)
        state = np.zeros(model.size, orc.ADAM_DTYPE)
        ctx = pkg.Context(pkg.default_config(**kw))
        ctx.model_init(42)
        if mode == "graph":
            ctx.step_capture(d_data.data_ptr(), len(data))
        seed = 42
        for step in range(5):
            lr = 2.0
            start = step * kw["seq_len"]
            if mode == "graph":
                ctx.step_launch(start, seed, lr)
            else:
                ctx.step(d_data.data_ptr(), len(data), start, seed, lr)
            loss, fit = ctx.step_losses()
            ref_loss = orc.population_forward(ocfg, model, data, start, seed)
            assert np.array_equal(loss, ref_loss), f"{mode} step {step} losses"
            ref_fit = orc.fitness(ref_loss)
            assert np.array_equal(fit, ref_fit)
            n_ref = orc.es_update_adam(ocfg, model, state, ref_fit, seed, lr)
            assert np.array_equal(ctx.model_download(), model), f"{mode} step {step} weights"
            assert ctx.last_update_count() == n_ref
            seed = pkg.next_seed(seed, step + 1)
        ctx.close()


def test_fifty_graph_steps_follow_the_oracle_trajectory(pkg, orc, dev):
    """50 replays of the captured step graph with the reference's learning-rate schedule and the d-eggs seed chain:
    int8 weights, float optimizer state and update counts stay bit-identical to the oracle's trajectory."""
    kw = dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=64)
    data = orc.zipf_bytes(1 << 16)
    ocfg = orc.config(**kw)
    d_data = _t(dev, data)
    model = orc.init_model(ocfg, 42)
    state = np.zeros(model.size, orc.ADAM_DTYPE)
    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_init(42)
    ctx.step_capture(d_data.data_ptr(), len(data))
    seed = 42
    changed = 0
    for step in range(50):
        lr = pkg.learning_rate(step) * 10.0          # a larger rate so that weights actually move within 50 steps
        start = step * kw["seq_len"]
        ctx.step_launch(start, seed, lr)
        ref_fit = orc.fitness(orc.population_forward(ocfg, model, data, start, seed))
        changed += orc.es_update_adam(ocfg, model, state, ref_fit, seed, np.float32(lr))
        if step in (0, 9, 24, 49):
            assert np.array_equal(ctx.model_download(), model), f"weights differ at step {step}"
            assert ctx.opt_state_download().tobytes() == state.tobytes(), f"optimizer state differs at step {step}"
        seed = pkg.next_seed(seed, step + 1)
    assert changed > 100
    ctx.close()


def test_muon_step_graph_replays_equal_eager_steps(pkg, orc, dev):
    """The whole step with the Muon update (momentum, batched Newton-Schulz, apply rule) captured once and replayed:
    every replay leaves the weights, the optimizer state, the losses and the update count of the same step run eagerly
    on a second context, with eager work and synchronisation between the replays."""
    import torch
    kw = dict(hidden=128, head_dim=32, n_layers=2, seq_len=32, population=64, use_muon=1)
    data = orc.zipf_bytes(1 << 16)
    d_data = _t(dev, data)
    g, e = pkg.Context(pkg.default_config(**kw)), pkg.Context(pkg.default_config(**kw))
    g.model_init(42); e.model_init(42)
    g.step_capture(d_data.data_ptr(), len(data))
    seed, moved = 4242, False
    start_model = e.model_download()
    for step in range(8):
        lr, start = 30.0, step * kw["seq_len"]
        g.step_launch(start, seed, lr)
        e.step(d_data.data_ptr(), len(data), start, seed, lr)
        # unrelated eager work on the card between the replays
        junk = torch.randn(1 << 16, device=dev); junk = (junk * junk).sum().item()
        gl, gf = g.step_losses(); el, ef = e.step_losses()
        assert np.array_equal(gl, el) and np.array_equal(gf, ef), step
        assert np.array_equal(g.model_download(), e.model_download()), f"weights differ after replay {step}"
        assert g.opt_state_download().tobytes() == e.opt_state_download().tobytes(), f"optimizer state differs after replay {step}"
        assert g.last_update_count() == e.last_update_count(), step
        seed = pkg.next_seed(seed, step + 1)
    assert not np.array_equal(e.model_download(), start_model)
    g.close(); e.close()


@pytest.mark.parametrize("muon", [0, 1], ids=["adamw", "muon"])
def test_training_reduces_the_loss(pkg, orc, dev, muon):
    """What the reference itself checks (sweep_hyperparams.sh:146-178 trains and reads the last "Loss:"): 160 whole
    steps of the small model on the synthetic stream at the reference's starting learning rate bring the population's
    mean loss per token down by a quarter or more; the same run twice gives the same numbers."""
    kw = dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=2048, use_muon=muon)
    data = orc.zipf_bytes(1 << 22)
    d_data = _t(dev, data)
    runs = []
    for rep in range(2):
        ctx = pkg.Context(pkg.default_config(**kw))
        ctx.model_init(42)
        seed, hist = 42, []
        for step in range(160):
            ctx.step(d_data.data_ptr(), len(data), step * kw["seq_len"], seed, pkg.learning_rate(step))
            if step < 3 or step >= 157:
                hist.append(float(ctx.step_losses()[0].mean()) / kw["seq_len"])
            seed = pkg.next_seed(seed, step + 1)
        runs.append(hist)
        ctx.close()
    assert runs[0] == runs[1]
    first, last = np.mean(runs[0][:3]), np.mean(runs[0][3:])
    assert last < 0.75 * first, (first, last)


def test_error_paths(pkg, dev):
    with pytest.raises(pkg.EggError):
        pkg.Context(pkg.default_config(hidden=100))
    with pytest.raises(pkg.EggError):
        pkg.Context(pkg.default_config(seq_len=48))
    with pytest.raises(pkg.EggError):
        pkg.Context(pkg.default_config(vocab=300))        # multiples of 256 only
    ctx = pkg.Context(pkg.default_config(**SMALL))
    with pytest.raises(pkg.EggError):
        ctx.step_launch(0, 1, 0.1)            # launch before capture
    with pytest.raises(pkg.EggError):
        ctx.model_upload(np.zeros(3, np.int8))
    ctx.close()


def test_newton_schulz_gpu(pkg, orc, dev):
    """fp32 MFMA Newton-Schulz against the fp64 restatement (the reference's cuBLAS summation order is unspecified,
    so this is a tolerance check: relative Frobenius error <= 1e-5) plus the orthogonality it is meant to reach."""
    import torch
    ctx = pkg.Context(pkg.default_config(use_muon=1, hidden=512, head_dim=64, n_layers=1, seq_len=128, population=8))
    rng = np.random.default_rng(21)
    for rows, cols in ((256, 256), (256, 1024), (1024, 256), (64, 96), (512, 512), (512, 2048), (2048, 512)):
        X = (rng.integers(-300, 301, (rows, cols))).astype(np.float32)
        ref = X.astype(np.float64)
        orc.lib().orc_newton_schulz_f64(ref.ctypes.data_as(C.c_void_p), rows, cols, 5)
        d = _t(dev, X)
        ctx.newton_schulz(d.data_ptr(), rows, cols, 5)
        ctx.sync()
        got = d.cpu().numpy().astype(np.float64)
        err = np.linalg.norm(got - ref) / np.linalg.norm(ref)
        assert err < 1e-5, (rows, cols, err)
    ctx.close()


def test_muon_update(pkg, orc, dev):
    """Muon chain per matrix: momentum state is bit-exact (integer votes, two float ops); the orthogonalised step
    goes through fp32 GEMMs, so weights may differ from the oracle only where an accumulator sits within rounding
    distance of the +-1 threshold."""
    import torch
    kw = dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=120)
    ocfg = orc.config(**kw)
    ctx = pkg.Context(pkg.default_config(use_muon=1, **kw))
    rng = np.random.default_rng(22)
    pairs = kw["population"] // 2
    model = orc.init_model(ocfg, 42)
    ctx.model_upload(model)
    seed, lr = 777, 40.0          # a large rate so many accumulators cross the threshold
    d_seed = _t(dev, np.array([seed], np.uint32).view(np.int32))
    d_lr = _t(dev, np.array([lr], np.float32))
    st_bytes = ctx.opt_state_download().nbytes
    tensors = ctx.tensors()
    assert st_bytes == sum(t["rows"] * t["cols"] * (8 if t["muon"] else 12) for t in tensors)
    ref_states = {t["id"]: np.zeros(t["rows"] * t["cols"], orc.MUON_DTYPE) for t in tensors if t["muon"]}
    for step in range(3):
        fit = rng.integers(-1, 2, pairs).astype(np.int32)
        d_fit = _t(dev, fit)
        for t in tensors:
            if not t["muon"]:
                continue
            n = t["rows"] * t["cols"]
            ctx.update_tensor(t["id"], d_fit.data_ptr(), d_seed.data_ptr(), d_lr.data_ptr())
            W = model[t["offset"]:t["offset"] + n]
            st = ref_states[t["id"]]
            orc.lib().orc_update_matrix_muon(C.byref(ocfg), W.ctypes.data_as(C.c_void_p), st.ctypes.data_as(C.c_void_p),
                                             t["rows"], t["cols"], t["off_a"], t["off_b"], t["seed_base"],
                                             fit.ctypes.data_as(C.c_void_p), pairs, C.c_uint32(seed), C.c_float(lr), None)
            got_m = ctx.model_download()[t["offset"]:t["offset"] + n]
            raw = ctx.opt_state_download().view(np.uint8)
            off = ctx.tensor_state_offset(t["id"])
            got_st = raw[off:off + 8 * n].view(orc.MUON_DTYPE)
            assert np.array_equal(got_st["m"].view(np.int32), st["m"].view(np.int32)), (t["name"], step)
            diff = np.flatnonzero(got_m != W)
            # any disagreement must be a threshold crossing decided by float rounding in the GEMMs
            assert len(diff) <= max(2, n // 500), (t["name"], step, len(diff))
            for i in diff:
                assert abs(int(got_m[i]) - int(W[i])) == 1
            same = got_m == W
            assert np.allclose(got_st["acc"][same], st["acc"][same], atol=2e-3), t["name"]
            # keep both sides on the same trajectory for the next step
            if len(diff):
                m2 = ctx.model_download(); m2[t["offset"]:t["offset"] + n] = W; ctx.model_upload(m2)
                raw2 = raw.copy(); raw2[off:off + 8 * n] = st.view(np.uint8); ctx.opt_state_upload(raw2)
            else:
                raw2 = raw.copy(); raw2[off:off + 8 * n] = st.view(np.uint8); ctx.opt_state_upload(raw2)
        seed += 1
        d_seed.copy_(_t(dev, np.array([seed], np.uint32).view(np.int32)))
    assert not np.array_equal(ctx.model_download(), orc.init_model(ocfg, 42))       # the updates moved weights
    ctx.close()


@pytest.mark.parametrize("kw", [dict(hidden=64, head_dim=32, n_layers=3, seq_len=32, population=64),
                                dict(hidden=128, head_dim=32, n_layers=2, seq_len=32, population=32),
                                dict(hidden=256, head_dim=64, n_layers=5, seq_len=32, population=16),
                                # shape groups with different batch limits (64 square matrices at once, 16 of each 4:1 shape
                                # where a group has 17): every group must run at its own limit
                                dict(hidden=512, head_dim=64, n_layers=16, seq_len=32, population=8)])
def test_muon_batched_update_equals_per_matrix_update(pkg, orc, dev, kw):
    """egg_es_update sends the Muon matrices of one shape through Newton-Schulz as one batch per stage; what it leaves
    (weights, momentum, accumulators, update count) is bit-identical to updating tensor by tensor."""
    import torch
    ocfg = orc.config(**kw)
    model = orc.init_model(ocfg, 42)
    rng = np.random.default_rng(5)
    pairs = kw["population"] // 2
    a = pkg.Context(pkg.default_config(use_muon=1, **kw))
    b = pkg.Context(pkg.default_config(use_muon=1, **kw))
    a.model_upload(model); b.model_upload(model)
    shapes = {}
    for t in a.tensors():
        if t["muon"]:
            shapes.setdefault((t["rows"], t["cols"]), []).append(t["id"])
    assert max(len(v) for v in shapes.values()) >= 2 * kw["n_layers"]          # there is something to batch
    d_lr = _t(dev, np.array([25.0], np.float32))
    for step in range(3):
        d_fit = _t(dev, rng.integers(-1, 2, pairs).astype(np.int32))
        d_seed = _t(dev, np.array([900 + step], np.uint32).view(np.int32))
        a.es_update(d_fit.data_ptr(), d_seed.data_ptr(), d_lr.data_ptr())
        total = 0
        for t in b.tensors():
            b.update_tensor(t["id"], d_fit.data_ptr(), d_seed.data_ptr(), d_lr.data_ptr())
        a.sync(); b.sync()
        assert np.array_equal(a.model_download(), b.model_download()), step
        assert np.array_equal(a.opt_state_download(), b.opt_state_download()), step
    assert not np.array_equal(a.model_download(), model)
    a.close(); b.close()


@pytest.mark.parametrize("kw,seed_len,gen_len", [(dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=4), 5, 27),
                                                 (dict(hidden=128, head_dim=32, n_layers=2, seq_len=64, population=4), 10, 30),
                                                 (dict(hidden=256, head_dim=64, n_layers=2, seq_len=64, population=4), 16, 40),
                                                 # the workgroup-per-head attention kernel (sequence 256 / 512), continuations that cross tile ends
                                                 (dict(hidden=256, head_dim=64, n_layers=2, seq_len=256, population=2), 90, 40),
                                                 (dict(hidden=512, head_dim=64, n_layers=1, seq_len=512, population=2), 60, 10)],
                         ids=["h64", "h128", "h256", "h256_t256", "h512_t512"])
def test_generate(pkg, orc, dev, kw, seed_len, gen_len):
    """Sampling continuation of a prompt by the unperturbed model against the oracle's token-by-token restatement."""
    import torch
    ocfg = orc.config(**kw)
    model = orc.init_model(ocfg, 42)
    rng = np.random.default_rng(3)
    for t in orc.tensor_table(ocfg):
        if not t["is_matrix"]:
            sl = slice(t["offset"], t["offset"] + t["cols"])
            model[sl] = rng.integers(-20, 21, t["cols"]).astype(np.int8) + (16 if t["name"].startswith("ln_") and "bias" not in t["name"] else 0)
        elif t["name"] == "embedding":      # a small tied head keeps the next-byte distribution broad
            n = t["rows"] * t["cols"]
            model[t["offset"]:t["offset"] + n] = rng.integers(-5, 6, n).astype(np.int8)
    prompt = orc.zipf_bytes(4096)[100:100 + seed_len].copy()
    ref = orc.generate(ocfg, model, prompt, gen_len, 1041)
    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_upload(model)
    buf = torch.zeros(seed_len + gen_len, dtype=torch.uint8, device=dev)
    buf[:seed_len] = _t(dev, prompt)
    ctx.generate(buf.data_ptr(), seed_len, gen_len, 1041)
    ctx.sync()
    got = buf.cpu().numpy()
    assert np.array_equal(got, ref), (got.tolist(), ref.tolist())
    assert len(set(ref[seed_len:].tolist())) > 3      # the continuation is not degenerate
    # without the per-layer K / V cache (every new token re-evaluates the whole window): the same tokens
    ctx.generate_kv_cache(False)
    buf2 = torch.zeros(seed_len + gen_len, dtype=torch.uint8, device=dev)
    buf2[:seed_len] = _t(dev, prompt)
    ctx.generate(buf2.data_ptr(), seed_len, gen_len, 1041)
    ctx.sync()
    assert np.array_equal(buf2.cpu().numpy(), ref)
    ctx.generate_kv_cache(True)
    # a second call on the same context starts from a fresh cache: another prompt, shorter continuation
    prompt2 = orc.zipf_bytes(4096)[900:900 + seed_len].copy()
    buf3 = torch.zeros(seed_len + gen_len, dtype=torch.uint8, device=dev)
    buf3[:seed_len] = _t(dev, prompt2)
    ctx.generate(buf3.data_ptr(), seed_len, max(1, gen_len // 2), 7)
    ctx.sync()
    n2 = seed_len + max(1, gen_len // 2)
    assert np.array_equal(buf3.cpu().numpy()[:n2], orc.generate(ocfg, model, prompt2, max(1, gen_len // 2), 7))
    # a population forward afterwards is unaffected by the generation's mask / logits overrides
    data = orc.zipf_bytes(1 << 14)
    d_loss = torch.zeros(kw["population"], dtype=torch.int32, device=dev)
    ctx.population_forward(_t(dev, data).data_ptr(), len(data), 0, 77, 0, kw["population"], d_loss.data_ptr())
    ctx.sync()
    assert np.array_equal(d_loss.cpu().numpy(), orc.population_forward(ocfg, model, data, 0, 77))
    with pytest.raises(pkg.EggError):
        ctx.generate(buf.data_ptr(), seed_len, kw["seq_len"], 1)
    ctx.close()


@pytest.mark.parametrize("kw,seed_len,gen_len,sampling", [
    (dict(hidden=64, head_dim=32, n_layers=1, seq_len=64, population=2), 5, 40, (0.6, 0.08, 0.2)),       # the reference's defaults
    (dict(hidden=64, head_dim=32, n_layers=1, seq_len=64, population=2), 5, 40, (1.0, 0.0, 0.0)),        # neutral: the plain sampler
    (dict(hidden=128, head_dim=32, n_layers=2, seq_len=128, population=2), 20, 100, (1.7, 0.3, 1.5)),
    (dict(hidden=256, head_dim=64, n_layers=1, seq_len=256, population=2), 196, 60, (0.25, 0.01, -0.5)),
    (dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=2), 1, 31, (3.0, 0.9, 4.0))])
def test_generate_deggs(pkg, orc, dev, kw, seed_len, gen_len, sampling):
    """d-eggs' sampler (temperature, min-p, presence penalty; d-eggs/src/kernels.cu:382-478) against the oracle."""
    import torch
    temp, min_p, penalty = sampling
    ocfg = orc.config(**kw)
    model = orc.init_model(ocfg, 42)
    rng = np.random.default_rng(3)
    for t in orc.tensor_table(ocfg):
        if not t["is_matrix"]:
            sl = slice(t["offset"], t["offset"] + t["cols"])
            model[sl] = rng.integers(-20, 21, t["cols"]).astype(np.int8) + (16 if t["name"].startswith("ln_") and "bias" not in t["name"] else 0)
        elif t["name"] == "embedding":
            n = t["rows"] * t["cols"]
            model[t["offset"]:t["offset"] + n] = rng.integers(-5, 6, n).astype(np.int8)
    prompt = orc.zipf_bytes(4096)[100:100 + seed_len].copy()
    ref = orc.generate_deggs(ocfg, model, prompt, gen_len, 1041, temp, min_p, penalty)
    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_upload(model)
    buf = torch.zeros(seed_len + gen_len, dtype=torch.uint8, device=dev)
    buf[:seed_len] = _t(dev, prompt)
    ctx.generate_deggs(buf.data_ptr(), seed_len, gen_len, 1041, temp, min_p, penalty)
    ctx.sync()
    got = buf.cpu().numpy()
    assert np.array_equal(got, ref), (got.tolist(), ref.tolist())
    if sampling == (1.0, 0.0, 0.0):
        assert np.array_equal(ref, orc.generate(ocfg, model, prompt, gen_len, 1041))
    else:
        assert not np.array_equal(ref, orc.generate(ocfg, model, prompt, gen_len, 1041))      # the settings matter
    if penalty >= 1.5:
        assert len(set(ref[seed_len:].tolist())) > 15          # a strong penalty spreads the continuation
    with pytest.raises(pkg.EggError):
        ctx.generate_deggs(buf.data_ptr(), 200, 100, 1)          # beyond the reference's 256-entry token history
    ctx.close()


@pytest.mark.parametrize("sampling", [None, (0.6, 0.08, 0.2), (1.7, 0.3, 1.5)], ids=["plain", "deggs_defaults", "deggs_other"])
@pytest.mark.parametrize("kw,seed_len,gen_len", [(dict(hidden=64, head_dim=32, n_layers=1, seq_len=64, population=2, vocab=768), 6, 40),
                                                 (dict(hidden=256, head_dim=64, n_layers=2, seq_len=64, population=2, vocab=8192), 12, 30)],
                         ids=["vocab_768", "h256_vocab_8192"])
def test_generate_with_a_larger_vocabulary(pkg, orc, dev, kw, seed_len, gen_len, sampling):
    """Both samplers over a vocabulary of more than 256 entries: the buffer holds uint32 tokens."""
    import torch
    ocfg = orc.config(**kw)
    V = kw["vocab"]
    model = orc.init_model(ocfg, 42)
    rng = np.random.default_rng(3)
    for t in orc.tensor_table(ocfg):
        if not t["is_matrix"]:
            sl = slice(t["offset"], t["offset"] + t["cols"])
            model[sl] = rng.integers(-20, 21, t["cols"]).astype(np.int8) + (16 if t["name"].startswith("ln_") and "bias" not in t["name"] else 0)
        elif t["name"] == "embedding":      # a small tied head keeps the next-token distribution broad
            n = t["rows"] * t["cols"]
            model[t["offset"]:t["offset"] + n] = rng.integers(-5, 6, n).astype(np.int8)
    prompt = rng.integers(0, V, seed_len).astype(np.uint32)
    prompt[0] = V - 1
    if sampling is None:
        ref = orc.generate(ocfg, model, prompt, gen_len, 1041)
    else:
        ref = orc.generate_deggs(ocfg, model, prompt, gen_len, 1041, *sampling)
    assert ref.dtype == np.uint32 and int(ref[seed_len:].max()) > 255 and len(set(ref[seed_len:].tolist())) > 3
    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_upload(model)
    for cache in (True, False):
        ctx.generate_kv_cache(cache)
        buf = torch.zeros(seed_len + gen_len, dtype=torch.int32, device=dev)
        buf[:seed_len] = _t(dev, prompt)
        if sampling is None:
            ctx.generate(buf.data_ptr(), seed_len, gen_len, 1041)
        else:
            ctx.generate_deggs(buf.data_ptr(), seed_len, gen_len, 1041, *sampling)
        ctx.sync()
        got = buf.cpu().numpy().view(np.uint32)
        assert np.array_equal(got, ref), (cache, got.tolist(), ref.tolist())
    ctx.close()


def test_checkpoint_files_round_trip(pkg, orc, dev, tmp_path):
    """save_checkpoint / load_model (egg_disk_utils.h:46-82): raw model and optimizer-state files, "last" symlinks,
    byte-identical to what the oracle holds after the same steps; a file of another shape is refused."""
    import torch
    kw = dict(hidden=64, head_dim=32, n_layers=1, seq_len=32, population=40)
    ocfg = orc.config(**kw)
    model = orc.init_model(ocfg, 42)
    state = np.zeros(model.size, orc.ADAM_DTYPE)
    rng = np.random.default_rng(4)
    ctx = pkg.Context(pkg.default_config(**kw))
    ctx.model_upload(model)
    d_seed = _t(dev, np.array([9], np.uint32).view(np.int32)); d_lr = _t(dev, np.array([5.0], np.float32))
    for step in range(2):
        fit = rng.integers(-1, 2, 20).astype(np.int32)
        ctx.es_update(_t(dev, fit).data_ptr(), d_seed.data_ptr(), d_lr.data_ptr())
        orc.es_update_adam(ocfg, model, state, fit, 9, 5.0)
    d = str(tmp_path / "models")
    ctx.checkpoint_save(d, 7)
    ctx.checkpoint_save(d, 12)
    names = sorted(os.listdir(d))
    assert names == ["egg_step-00000007.adam.bin", "egg_step-00000007.model.bin", "egg_step-00000012.adam.bin",
                     "egg_step-00000012.model.bin", "egg_transformer_last.adam.bin", "egg_transformer_last.model.bin"]
    assert os.readlink(os.path.join(d, "egg_transformer_last.model.bin")) == "egg_step-00000012.model.bin"
    assert open(os.path.join(d, "egg_step-00000012.model.bin"), "rb").read() == model.tobytes()
    assert open(os.path.join(d, "egg_transformer_last.adam.bin"), "rb").read() == state.tobytes()
    ctx2 = pkg.Context(pkg.default_config(**kw))
    ctx2.checkpoint_load(os.path.join(d, "egg_transformer_last.model.bin"), os.path.join(d, "egg_transformer_last.adam.bin"))
    assert np.array_equal(ctx2.model_download(), model)
    assert ctx2.opt_state_download().tobytes() == state.tobytes()
    # save_model_info (egg_disk_utils.h:15-44): the configuration and sizes as text
    ctx.model_info_save(d)
    info = open(os.path.join(d, "model.info")).read().splitlines()
    assert info[:7] == ["Model Configuration:", "HIDDEN_DIM: 64", "HEAD_DIM: 32", "N_LAYERS: 1", "SEQ_LEN: 32", "VOCAB_SIZE: 256", "N_HEADS: 2"]
    assert f"Model Parameters: {model.size} ({model.size / 1048576:.2f} MB)" in info
    assert f"Adam State Size: {12 * model.size} ({12 * model.size / 1048576:.2f} MB)" in info and "Population: 40" in info
    assert "Softmax Scale: 2^18" in info
    ctx3 = pkg.Context(pkg.default_config(hidden=128, head_dim=32, n_layers=1, seq_len=32, population=40))
    with pytest.raises(pkg.EggError):
        ctx3.checkpoint_load(os.path.join(d, "egg_transformer_last.model.bin"))
    for c in (ctx, ctx2, ctx3):
        c.close()

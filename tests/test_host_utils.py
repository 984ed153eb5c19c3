"""CPU tests of the host-side companions exported by the C-ABI library: d-eggs fitness shaping, base-3 packing and
the EGGC replay checkpoints.  The packing and the checkpoint format are pinned by the reference's own headers compiled
into oracle/_ref (ternary_pack.h, checkpoint.h) and by the vectors of d-eggs/test_ternary.cpp; the shaping by
hand-computed cases."""
import ctypes as C
import os

import numpy as np
import pytest


def test_ternary_pack_against_reference_header(pkg, orc):
    ref = orc.ref()
    rng = np.random.default_rng(0)
    # the two vectors of d-eggs/test_ternary.cpp
    for src in ([-1, 0, 1, -1, 0, 1, 1, 0, -1, 0], [-1, 0, 1, -1, 0, 1, 1]):
        packed = pkg.ternary_pack(src)
        assert len(packed) == 2 and pkg.ternary_unpack(packed, len(src)).tolist() == src
    # digit order: least significant first, -1 -> 2
    assert pkg.ternary_pack([1, 0, 0, 0, 0]).tolist() == [1] and pkg.ternary_pack([0, 0, 0, 0, -1]).tolist() == [162]
    assert pkg.ternary_pack([-1, -1, -1, -1, -1]).tolist() == [242] and pkg.ternary_pack([0, 1]).tolist() == [3]
    for n in list(range(0, 24)) + [1000, 20480]:
        src = rng.integers(-1, 2, n).astype(np.int32)
        packed = pkg.ternary_pack(src)
        assert len(packed) == (n + 4) // 5
        assert np.array_equal(pkg.ternary_unpack(packed, n), src)
        if ref is not None and n:
            ref.ref_ternary_pack_estimate_size.restype = C.c_size_t
            assert ref.ref_ternary_pack_estimate_size(C.c_size_t(n)) == len(packed)
            exp = np.zeros(len(packed), np.uint8)
            ref.ref_ternary_pack(src.ctypes.data_as(C.c_void_p), C.c_size_t(n), exp.ctypes.data_as(C.c_void_p))
            assert np.array_equal(packed, exp)
            back = np.zeros(n, np.int32)
            ref.ref_ternary_unpack(packed.ctypes.data_as(C.c_void_p), C.c_size_t(n), back.ctypes.data_as(C.c_void_p))
            assert np.array_equal(back, src)
    with pytest.raises(pkg.EggError):
        pkg.ternary_pack([0, 2, 0])


def _losses(diffs, base=1000):
    """pair losses (p, n) with n - p = diff"""
    out = []
    for d in diffs:
        out += [base, base + d]
    return np.array(out, np.int32)


def test_shape_fitness_cases(pkg):
    # no filter, no threshold: the pairwise sign rule (positive when the +noise member has the lower loss)
    fit, total = pkg.shape_fitness(_losses([5, -3, 0, 1]), chunk_mean_filter=False, adaptive_threshold=False)
    assert fit.tolist() == [1, -1, 0, 1] and total == 8 * 1000 + 3
    # threshold alpha * mean|diff|: |diffs| = 10, 10, 1, 0 -> mean 5.25
    fit, _ = pkg.shape_fitness(_losses([10, -10, 1, 0]), chunk_mean_filter=False, adaptive_threshold=True, alpha=0.1)
    assert fit.tolist() == [1, -1, 1, 0]           # threshold 0.525
    # the reference's thresholded branch has no zero case of its own: with every difference 0 the threshold is 0,
    # |0| < 0 is false and the vote is (0 > 0 ? 1 : -1) = -1
    fit0, _ = pkg.shape_fitness(_losses([0, 0, 0]), chunk_mean_filter=False, adaptive_threshold=True, alpha=0.1)
    assert fit0.tolist() == [-1, -1, -1]
    fit2, _ = pkg.shape_fitness(_losses([10, -10, 1, 0]), chunk_mean_filter=False, adaptive_threshold=True, alpha=0.5)
    assert fit2.tolist() == [1, -1, 0, 0]          # threshold 2.625
    # chunk-mean shift: mean 6 -> 6^1.2 = 8.58... -> +8 on every difference
    fit, _ = pkg.shape_fitness(_losses([-3, 9, 9, 9]), chunk_mean_filter=True, mean_exponent=1.2, adaptive_threshold=False)
    assert fit.tolist() == [1, 1, 1, 1]
    # negative mean keeps its sign: mean -6 -> -8
    fit, _ = pkg.shape_fitness(_losses([3, -9, -9, -9]), chunk_mean_filter=True, mean_exponent=1.2, adaptive_threshold=False)
    assert fit.tolist() == [-1, -1, -1, -1]
    # |mean| < 1 raised to 1.2 truncates to 0: nothing moves
    fit, _ = pkg.shape_fitness(_losses([1, -1, 1, 0]), chunk_mean_filter=True, mean_exponent=1.2, adaptive_threshold=False)
    assert fit.tolist() == [1, -1, 1, 0]
    # exponent 1: the shift is the truncated mean itself (mean 2.5 -> 2)
    fit, _ = pkg.shape_fitness(_losses([-2, 7]), chunk_mean_filter=True, mean_exponent=1.0, adaptive_threshold=False)
    assert fit.tolist() == [0, 1]
    with pytest.raises(pkg.EggError):
        pkg.shape_fitness(np.zeros(3, np.int32))


def test_shape_fitness_properties_on_random_chunks(pkg):
    """What the rule's definition fixes on random chunks (d-eggs/src/worker.cu:636-687): swapping the members of every
    pair negates every vote, a larger alpha only turns votes into zeros and never flips one, the plain rule is the
    sign of n - p, the filter moves every difference by the same truncated amount, and a vectorised numpy evaluation of
    the same three steps agrees."""
    rng = np.random.default_rng(77)
    for trial in range(40):
        pairs = int(rng.integers(1, 400))
        spread = int(rng.choice([3, 50, 5000, 2_000_000]))
        loss = rng.integers(100_000, 100_000 + spread, 2 * pairs).astype(np.int32)
        if trial % 5 == 0:
            loss[1::2] += int(rng.integers(-spread, spread + 1))          # a chunk-wide bias: the filter has something to add
        swapped = loss.reshape(-1, 2)[:, ::-1].reshape(-1).copy()
        p, n = loss[0::2].astype(np.int64), loss[1::2].astype(np.int64)
        plain, total = pkg.shape_fitness(loss, chunk_mean_filter=False, adaptive_threshold=False)
        assert np.array_equal(plain, np.sign(n - p)) and total == int(loss.astype(np.int64).sum())
        for filt in (False, True):
            exponent = float(rng.choice([1.0, 1.2, 0.5]))
            mean = float((n - p).sum()) / pairs
            shift = int(np.trunc(np.sign(mean) * abs(mean) ** exponent)) if filt else 0
            d = n - p + shift
            nofilter_votes, _ = pkg.shape_fitness(loss, chunk_mean_filter=filt, mean_exponent=exponent, adaptive_threshold=False)
            assert np.array_equal(nofilter_votes, np.sign(d)), (trial, filt)
            prev_zero = np.zeros(pairs, bool)
            for alpha in (0.0, 0.05, 0.1, 0.5, 1.0, 3.0):
                fit, _ = pkg.shape_fitness(loss, chunk_mean_filter=filt, mean_exponent=exponent, adaptive_threshold=True, alpha=alpha)
                thr = np.abs(d).astype(np.float64).sum() / pairs * alpha
                want = np.where(np.abs(d) < thr, 0, np.where(d > 0, 1, -1))
                assert np.array_equal(fit, want), (trial, filt, alpha)
                zero = fit == 0
                assert np.all(zero | ~prev_zero)                              # zeros only grow with alpha
                assert np.all((fit == nofilter_votes) | zero | (d == 0))      # a vote is never flipped (d == 0 votes -1 in this branch)
                prev_zero = zero
                back, _ = pkg.shape_fitness(swapped, chunk_mean_filter=filt, mean_exponent=exponent, adaptive_threshold=True, alpha=alpha)
                assert np.array_equal(back[d != 0], -fit[d != 0]), (trial, filt, alpha)


def test_eggc_checkpoints_interoperate_with_reference_header(pkg, orc, tmp_path):
    ref = orc.ref()
    d = str(tmp_path / "ckpt")
    assert pkg.eggc_load_latest(d) is None
    rng = np.random.default_rng(1)
    payloads = {3: rng.integers(0, 243, 4096).astype(np.uint8), 12: rng.integers(0, 243, 100000).astype(np.uint8),
                7: np.zeros(0, np.uint8)}
    for step, data in payloads.items():
        pkg.eggc_save(d, step, 1000 + step, data)
    assert sorted(os.listdir(d)) == ["checkpoint_00000003.bin", "checkpoint_00000007.bin", "checkpoint_00000012.bin"]
    raw = open(os.path.join(d, "checkpoint_00000003.bin"), "rb").read()
    assert raw[:4] == b"CGGE" and len(raw) == 32 + 4096          # 0x45474743 little endian, 32-byte header
    step, seed, data = pkg.eggc_load_latest(d)
    assert (step, seed) == (12, 1012) and np.array_equal(data, payloads[12])
    if ref is not None:
        ref.ref_eggc_load.restype = C.c_int
        s, sd, n = C.c_uint64(0), C.c_uint64(0), C.c_uint64(0)
        buf = np.zeros(200000, np.uint8)
        assert ref.ref_eggc_load(d.encode(), C.byref(s), C.byref(sd), buf.ctypes.data_as(C.c_void_p), C.c_uint64(len(buf)), C.byref(n)) == 1
        assert (s.value, sd.value, n.value) == (12, 1012, 100000) and np.array_equal(buf[:100000], payloads[12])
        # and the other way round: a file written by the reference's writer
        d2 = str(tmp_path / "ckpt_ref")
        ref.ref_eggc_save(d2.encode(), C.c_uint64(41), C.c_uint64(77), payloads[3].ctypes.data_as(C.c_void_p), C.c_uint64(4096))
        ref.ref_eggc_save(d2.encode(), C.c_uint64(5), C.c_uint64(78), payloads[3].ctypes.data_as(C.c_void_p), C.c_uint64(10))
        step, seed, data = pkg.eggc_load_latest(d2)
        assert (step, seed) == (41, 77) and np.array_equal(data, payloads[3])
        assert open(os.path.join(d2, "checkpoint_00000041.bin"), "rb").read() == \
            open(os.path.join(d, "checkpoint_00000003.bin"), "rb").read()[:8] + (41).to_bytes(8, "little") + (77).to_bytes(8, "little") + raw[24:]
    # a file with a wrong magic is refused
    d3 = str(tmp_path / "bad"); os.mkdir(d3)
    open(os.path.join(d3, "checkpoint_00000001.bin"), "wb").write(b"\0" * 64)
    assert pkg.eggc_load_latest(d3) is None


def test_token_vocabulary_file_and_detokenize(pkg, tmp_path):
    """d-eggs' "decoding.bin" (d-eggs/src/worker.cu:36-81): uint32 count, then per token uint32 length + bytes; a run of
    tokens prints as the concatenation of their strings, an id beyond the table as "<id>"."""
    import struct
    entries = [b"the", b" ", b"", b"\xe2\x82\xac", b"egg", bytes(range(256))]
    path = tmp_path / "decoding.bin"
    # the file written by hand, byte for byte as the reference's reader expects it
    with open(path, "wb") as f:
        f.write(struct.pack("<I", len(entries)))
        for e in entries:
            f.write(struct.pack("<I", len(e)) + e)
    v = pkg.Vocabulary(path)
    assert len(v) == len(entries)
    assert v.detokenize([0, 1, 4, 2, 3]) == b"the egg\xe2\x82\xac"
    assert v.detokenize([4, 6, 1, 4000000000]) == b"egg<6> <4000000000>"
    assert v.detokenize([5]) == bytes(range(256)) and v.detokenize([]) == b""
    v.close()
    # the library's writer produces the same bytes
    path2 = tmp_path / "again.bin"
    pkg.Vocabulary.save(path2, entries)
    assert open(path2, "rb").read() == open(path, "rb").read()
    # a file that ends early, or whose length field points past its end, is refused
    whole = open(path, "rb").read()
    for cut in (2, 7, len(whole) - 1):
        bad = tmp_path / f"cut{cut}.bin"
        open(bad, "wb").write(whole[:cut])
        with pytest.raises(pkg.EggError):
            pkg.Vocabulary(bad)
    huge = tmp_path / "huge.bin"
    open(huge, "wb").write(struct.pack("<II", 1, 0xFFFFFFF0) + b"abc")
    with pytest.raises(pkg.EggError):
        pkg.Vocabulary(huge)
    with pytest.raises(pkg.EggError):
        pkg.Vocabulary(tmp_path / "missing.bin")


def test_learning_rate_schedules(pkg):
    """get_learning_rate of the single-node trainer (mgpu.cu:217-227) and of d-eggs (d-eggs/include/utils/training.h:5-9)"""
    f32 = lambda x: float(np.float32(x))
    assert [pkg.learning_rate(s) for s in (0, 299, 300, 599, 600, 999, 1000, 10 ** 6)] == [f32(v) for v in (0.3, 0.3, 0.15, 0.15, 0.075, 0.075, 0.05, 0.05)]
    assert [pkg.learning_rate_deggs(s) for s in (0, 99, 100, 199, 200, 10 ** 6)] == [0.5, 0.5, 0.25, 0.25, 0.125, 0.125]

"""The C++ host loop (egg.c_amd/host/egg_train.cpp: the reference's main() written against the C ABI) end to end:
eager and captured steps print the same losses, the adaptive overlay and checkpoints work from the command line."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "egg.c_amd", "egg_train")


def _run(args, cwd):
    if not os.path.exists(BIN):
        pytest.fail("egg.c_amd/egg_train is not built (run __graft_entry__.build())")
    r = subprocess.run([BIN] + args, capture_output=True, text=True, timeout=170, cwd=cwd)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    steps = re.findall(r"Step (\d+) \| Loss: ([0-9.]+) \| Time: [0-9.]+ ms \| Updates: (\d+)", r.stdout)
    return [(int(s), float(l), int(u)) for s, l, u in steps], r.stdout


def test_host_loop_eager_graph_adaptive_and_checkpoints(dev, tmp_path):
    base = ["--population", "64", "--seq", "32", "--hidden", "64", "--layers", "1", "--steps", "4"]
    eager, out = _run(base + ["--gen-every", "2"], tmp_path)
    assert [s for s, _, _ in eager] == [0, 1, 2, 3] and "--- GENERATION ---" in out
    graph, _ = _run(base + ["--gen-every", "0", "--graph"], tmp_path)
    assert [(l, u) for _, l, u in graph] == [(l, u) for _, l, u in eager], "captured steps differ from eager steps"
    adaptive, _ = _run(base + ["--gen-every", "0", "--adaptive"], tmp_path)
    assert adaptive[0][1] == eager[0][1]          # the overlay starts at factor 1: the first forward is the same
    assert len(adaptive) == 4
    # save at step 0 and 2, then resume from the last checkpoint through the "last" links
    saved, _ = _run(base + ["--gen-every", "0", "--save-every", "2", "--save-dir", "ckpt"], tmp_path)
    files = sorted(os.listdir(tmp_path / "ckpt"))
    assert any("last" in f for f in files) and len(files) >= 4, files
    model_last = [f for f in files if "last" in f and "adam" not in f][0]
    adam_last = [f for f in files if "last" in f and "adam" in f][0]
    resumed, _ = _run(base + ["--gen-every", "0", "--load", os.path.join("ckpt", model_last), "--load-state", os.path.join("ckpt", adam_last)],
                      tmp_path)
    assert len(resumed) == 4
    if sum(u for s, _, u in saved if s <= 2) > 0:                 # weights moved before the last checkpoint
        assert resumed[0][1] != eager[0][1], "the resumed run started from the initialisation, not from the checkpoint"


def test_host_loop_with_deggs_vocabulary_and_decoding_file(dev, tmp_path):
    """d-eggs' loop shape: a vocabulary above 256 (uint32 tokens, like its input.bin), its sampler, and generated tokens
    printed through a decoding.bin table."""
    import struct
    V = 512
    with open(tmp_path / "decoding.bin", "wb") as f:
        f.write(struct.pack("<I", V))
        for i in range(V):
            e = b"[%d]" % i
            f.write(struct.pack("<I", len(e)) + e)
    base = ["--population", "64", "--seq", "32", "--hidden", "64", "--layers", "1", "--steps", "3", "--vocab", str(V)]
    plain, out = _run(base + ["--gen-every", "1"], tmp_path)
    assert len(plain) == 3 and re.search(r"<\d+><\d+>", out), out[-600:]          # no table: ids in angle brackets
    named, out2 = _run(base + ["--gen-every", "1", "--decoding", "decoding.bin", "--deggs-sampler"], tmp_path)
    assert [(l, u) for _, l, u in named] == [(l, u) for _, l, u in plain]       # the sampler does not touch training
    gens = re.findall(r"--- GENERATION ---\n(.*?)\n\n", out2, re.S)
    assert len(gens) == 3 and all(re.search(r"\[\d+\]\[\d+\]", g) and "<" not in g for g in gens), out2[-600:]
    ids = [int(x) for x in re.findall(r"\[(\d+)\]", gens[0])]
    assert len(ids) == 32 and max(ids) < V        # 16 prompt tokens and 16 sampled ones
    graph, _ = _run(base + ["--gen-every", "0", "--graph"], tmp_path)
    assert [(l, u) for _, l, u in graph] == [(l, u) for _, l, u in plain]


def test_mfma_probe_reports_plausible_rates(dev):
    """The measurement aid bench.py runs as a child process: one JSON line, rates between a fifth of the published int8
    peak and a little above it, zero operands not slower than random ones."""
    import json
    probe = os.path.join(ROOT, "egg.c_amd", "mfma_probe")
    if not os.path.exists(probe):
        pytest.fail("egg.c_amd/mfma_probe is not built (run __graft_entry__.build())")
    r = subprocess.run([probe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-500:]
    d = json.loads(r.stdout.strip().splitlines()[-1])
    for k in ("zero_operands_TOPs", "random_operands_TOPs", "random_operands_changing_every_mfma_TOPs"):
        assert 1000.0 < d[k] < 5500.0, (k, d[k])
    assert d["zero_operands_TOPs"] >= 0.95 * d["random_operands_TOPs"]

"""The composition of the forward, pinned by an identity the mathematics fixes.

With the perturbation shifts at zero (fixed_point + sigma_shift = 0, sigma_shift_vector = 0) the rank-1 term of a
perturbed linear is exactly linear in the weights:  x.W + (x.B) A[n] ns  ==  x.(W + ns B (x) A), and a perturbed
vector is v + ns n1 n2.  So the perturbed forward of a member must equal, value for value, the UNPERTURBED forward
of a model whose tensors were materialised from the update's tensor table: W' = W + ns B(x)A, v' = v + ns n1 n2,
with A / B / n1 / n2 drawn at (pair seed + seed_base + off_a / off_b) exactly as the vote reconstruction draws them
(full_cuda_train_transformer_adam_mgpu.cu:1067-1152, launch list :1603-1643).  The tensor table's offsets are held
against the reference's macros by name (tests/test_reference_headers.py) and against the reference's launch list
(test_tensor_table_follows_the_reference_launch_list below).  A forward site that uses another tensor's seed offset,
swaps the roles of A and B, forgets the 1000*l layer base, or perturbs the wrong operand breaks the identity; the
mutation loop shows that every tensor's site is observable.

The same identity is checked for the CPU program (full_trained_egg.c): forward sites :242-290 against the update's
sites :564-574.
"""
import ctypes as C
import json
import os
import re

import numpy as np
import pytest

from test_oracle_pins import np_noise, P

HERE = os.path.dirname(os.path.abspath(__file__))
REF_MGPU = "/root/reference/full_cuda_train_transformer_adam_mgpu.cu"
LAUNCH_GOLD = os.path.join(HERE, "golden", "reference_update_launches.json")

# shifts that make the perturbation linear in the weights; fixed_point stays 4 so the GELU table is the usual one
LINEAR = dict(fixed_point=4, sigma_shift=-4, sigma_shift_vector=0)


def small_model(orc, cfg, rng, wmax):
    """random weights small enough that W + ns*B(x)A stays inside int8 for the masks used here"""
    model = orc.init_model(cfg, 42)
    for t in orc.tensor_table(cfg):
        n = t["rows"] * t["cols"] if t["is_matrix"] else t["cols"]
        sl = slice(t["offset"], t["offset"] + n)
        if t["is_matrix"]:
            model[sl] = rng.integers(-wmax, wmax + 1, n).astype(np.int8)
        else:
            gain = t["name"].startswith("ln_") and "bias" not in t["name"]
            model[sl] = rng.integers(-12, 13, n).astype(np.int8) + (16 if gain else 0)
    return model


def materialise(cfg, model, tt, step_seed, member, mask, leave_out=None):
    """the model member `member` effectively evaluates, built only from the update's tensor table"""
    pair, ns = member // 2, (1 if member % 2 == 0 else -1)
    out = model.astype(np.int64)
    for t in tt:
        if t["name"] == leave_out:
            continue
        s = step_seed + pair + t["seed_base"]
        rows, cols, o = t["rows"], t["cols"], t["offset"]
        if t["is_matrix"]:
            A = np_noise(s + t["off_a"], np.arange(cols), mask)          # output dimension
            B = np_noise(s + t["off_b"], np.arange(rows), mask)          # input dimension
            delta = ns * np.outer(B, A)                                  # logical [k][n]
            k, n = np.meshgrid(np.arange(rows), np.arange(cols), indexing="ij")
            out[o + ((k >> 2) * cols + n) * 4 + (k & 3)] += delta        # blocked [K/4][N][4], mgpu.cu:443-459
        else:
            out[o:o + cols] += ns * np_noise(s + t["off_a"], np.arange(cols), mask) * np_noise(s + t["off_b"], np.arange(cols), mask)
    assert np.abs(out).max() <= 127, "materialised weights left int8: shrink the weights or the mask"
    return out.astype(np.int8)


TAPS = ("x_emb", "x_init", "q", "k", "v", "ao", "x_attn", "x_mlp", "nf", "logits", "loss_t")

CASES = [dict(hidden=64, head_dim=32, n_layers=2, seq_len=16, population=8, noise_mask=3),
         dict(hidden=128, head_dim=64, n_layers=1, seq_len=16, population=4, noise_mask=7),
         dict(hidden=64, head_dim=32, n_layers=3, seq_len=12, population=4, noise_mask=2, use_same_data=1)]


@pytest.mark.parametrize("kw", CASES, ids=["h64_l2", "h128", "h64_l3_same_data"])
def test_perturbed_forward_equals_forward_of_materialised_model(orc, kw):
    cfg = orc.config(**kw, **LINEAR)
    mask = kw["noise_mask"]
    tt = orc.tensor_table(cfg)
    rng = np.random.default_rng(3)
    model = small_model(orc, cfg, rng, 127 - mask * mask)
    data = orc.zipf_bytes(1 << 13)
    start, seed = 5 * kw["seq_len"], 0x9E3779B1          # pair seeds wrap around 2^32 for the larger pairs' layers
    distinct = set()
    for m in range(kw["population"]):
        loss, tr = orc.forward_member(cfg, model, data, start, seed, m, trace=True)
        mat = materialise(cfg, model, tt, seed, m, mask)
        loss0, tr0 = orc.forward_member(cfg, mat, data, start, seed, m, ns_override=0, trace=True)
        for name in TAPS:
            assert np.array_equal(tr[name], tr0[name]), (m, name)
        assert loss == loss0, m
        distinct.add(loss)
        # the unperturbed forward of the ORIGINAL model is something else: the noise matters at this scale
        assert not np.array_equal(orc.forward_member(cfg, model, data, start, seed, m, ns_override=0, trace=True)[1]["logits"], tr["logits"])
    assert len(distinct) > 1


def test_every_tensor_site_is_observable(orc):
    """Leaving any single tensor out of the materialisation changes the result, so the identity above constrains
    the seed offsets, layer base and operand roles of every tensor, not of a few dominant ones."""
    kw = CASES[0]
    cfg = orc.config(**kw, **LINEAR)
    mask = kw["noise_mask"]
    tt = orc.tensor_table(cfg)
    model = small_model(orc, cfg, np.random.default_rng(3), 127 - mask * mask)
    data = orc.zipf_bytes(1 << 13)
    start, seed = 5 * kw["seq_len"], 0x9E3779B1
    blind = []
    for t in tt:
        seen = False
        for m in range(kw["population"]):
            _, tr = orc.forward_member(cfg, model, data, start, seed, m, trace=True)
            mat = materialise(cfg, model, tt, seed, m, mask, leave_out=t["name"])
            _, tr0 = orc.forward_member(cfg, mat, data, start, seed, m, ns_override=0, trace=True)
            if any(not np.array_equal(tr[n], tr0[n]) for n in TAPS):
                seen = True
                break
        if not seen:
            blind.append(t["name"])
    assert not blind, blind


def test_swapped_roles_and_shifted_bases_break_the_identity(orc):
    """The mistakes the identity is there to catch, made on purpose in the materialisation: A and B exchanged on a
    square matrix, a neighbouring tensor's offsets, a missing layer base."""
    kw = CASES[0]
    cfg = orc.config(**kw, **LINEAR)
    mask = kw["noise_mask"]
    tt = orc.tensor_table(cfg)
    model = small_model(orc, cfg, np.random.default_rng(3), 127 - mask * mask)
    data = orc.zipf_bytes(1 << 13)
    start, seed = 5 * kw["seq_len"], 0x9E3779B1
    by_name = {t["name"]: t for t in tt}

    def differs(table):
        for m in range(kw["population"]):
            _, tr = orc.forward_member(cfg, model, data, start, seed, m, trace=True)
            _, tr0 = orc.forward_member(cfg, materialise(cfg, model, table, seed, m, mask), data, start, seed, m, ns_override=0, trace=True)
            if any(not np.array_equal(tr[n], tr0[n]) for n in TAPS):
                return True
        return False

    def mutated(name, **change):
        return [dict(t, **change) if t["name"] == name else t for t in tt]

    assert not differs(tt)
    q, k = by_name["w_q.1"], by_name["w_k.1"]
    assert differs(mutated("w_q.1", off_a=q["off_b"], off_b=q["off_a"]))          # A <-> B
    assert differs(mutated("w_q.1", off_a=k["off_a"], off_b=k["off_b"]))          # K's noise on Q
    assert differs(mutated("w_o.1", seed_base=0))                                 # layer base dropped
    assert differs(mutated("w_down.0", seed_base=1000))                           # wrong layer
    e = by_name["embedding"]
    assert differs(mutated("embedding", off_a=e["off_b"], off_b=e["off_a"]))      # token noise on the hidden side
    assert differs(mutated("ln_2_bias.0", off_a=by_name["ln_1_bias.0"]["off_a"], off_b=by_name["ln_1_bias.0"]["off_b"]))


# ---------------------------------------------------------------- the tensor table against the reference's launch list
def parse_reference_launches(text):
    """(tensor, rows, cols, SEED_A expression, SEED_B expression, base, lr scale) of every optimizer launch in the
    reference's step loop, from the source text (full_cuda_train_transformer_adam_mgpu.cu:1603-1643)"""
    body = text[text.index("for(int l=0; l<N_LAYERS; l++) {\n                int s_base"):text.index("#if NTT_MODE != 0", text.index("int s_base"))]
    out = []
    for kind, args in re.findall(r"LAUNCH_ADAM_(MATRIX|VECTOR)\(([^;]*)\);", body):
        a = [x.strip() for x in args.split(",")]
        name = re.search(r"d_model->(\w+)", a[0]).group(1)
        if kind == "MATRIX":
            out.append([name, a[2], a[3], a[4], a[5], a[6], "1.0f"])
        else:
            out.append([name, "1", a[2], a[3], a[4], a[5], a[6]])
    m = re.search(r"update_matrix_adam_kernel<<<[^>]*>>>\(\s*\(WeightType\*\)gpus\[i\]\.d_model->(\w+),[^,]*,\s*(\w+),\s*(\w+),\s*([\w+]+),\s*([\w+]+),\s*(\w+),", body)
    out.append([m.group(1), m.group(2), m.group(3), m.group(4), m.group(5), m.group(6), "1.0f"])
    return out


def test_tensor_table_follows_the_reference_launch_list(orc):
    """Which tensor is updated with which pair of seed offsets is written in the reference's step loop; the parsed
    list is committed as a fixture and, where the reference checkout is present, re-read from the source."""
    gold = json.load(open(LAUNCH_GOLD))
    if os.path.exists(REF_MGPU):
        assert parse_reference_launches(open(REF_MGPU).read()) == gold
    L = orc.lib()
    cfg = orc.config(hidden=64, head_dim=32, n_layers=2, seq_len=16, population=4)
    H, V = cfg.hidden, cfg.vocab

    def value(expr, layer):
        env = {"HIDDEN_DIM": H, "VOCAB_SIZE": V, "s_base": 1000 * layer}
        total = 0
        for term in expr.replace(" ", "").split("+"):
            m = re.fullmatch(r"(\d+)\*(\w+)", term)
            if m:
                total += int(m.group(1)) * env[m.group(2)]
            elif term in env:
                total += env[term]
            elif re.fullmatch(r"\d+(\.\d+)?f?", term):
                total += float(term.rstrip("f"))
            else:
                off = L.orc_seed_offset(term.encode())
                assert off >= 0, term
                total += off
        return total

    per_layer = [g for g in gold if g[5] == "s_base"]
    globals_ = [g for g in gold if g[5] != "s_base"]
    expect = []
    for l in range(cfg.n_layers):
        expect += [(f"{g[0]}.{l}", g, l) for g in per_layer]
    expect += [(g[0], g, 0) for g in globals_]
    tt = orc.tensor_table(cfg)
    assert [t["name"] for t in tt] == [e[0] for e in expect]          # the reference's launch order, too
    for t, (name, g, l) in zip(tt, expect):
        rows, cols = int(value(g[1], l)), int(value(g[2], l))
        assert (t["rows"], t["cols"]) == (rows, cols), name
        assert t["is_matrix"] == (1 if g[1] != "1" else 0), name
        assert t["off_a"] == int(value(g[3], l)) and t["off_b"] == int(value(g[4], l)), name
        assert t["seed_base"] == int(value(g[5], l)), name
        assert abs(t["lr_scale"] - value(g[6], l)) < 1e-7, name


# ---------------------------------------------------------------- the CPU program (full_trained_egg.c)
def test_gru_perturbed_forward_equals_forward_of_materialised_model(orc):
    """full_trained_egg.c: forward_pass draws a matrix's noise at step_seed + p + 100*l + {1..6} / + 999 (:242-290) and
    update_matrix regenerates it at the same seeds (:564-574, :352-368).  The oracle's perturbed forward with the
    perturbation shift at zero must equal the unperturbed forward of W + sign * A (x) B built from the UPDATE's site
    list; the materialised weights exceed int8 (|A B| <= 961), so that side runs on the numpy restatement, which
    takes wider weights."""
    from oracle import gru_numpy as gn
    g = orc.gru_config(hidden=32, n_layers=2, seq_len=6, population=6, fixed_point=4, sigma_shift=-4)
    L = orc.lib()
    rng = np.random.default_rng(11)
    blob = orc.gru_init_model(g, 42)
    views = gn.model_views(g, blob)
    views["gru_biases"][...] = rng.integers(-20, 21, views["gru_biases"].shape)
    data = orc.zipf_bytes(2048)
    step_seed = 0xFFFFFF00                                 # wraps for the head's + 999
    losses = set()
    for p in range(g.population // 2):
        inp, tgt = data[40 * p:40 * p + g.seq_len].copy(), data[40 * p + 1:40 * p + 1 + g.seq_len].copy()
        for sign in (1, -1):
            st_c = rng.integers(-50, 51, g.n_layers * g.hidden).astype(np.int8)
            st_n = st_c.reshape(g.n_layers, g.hidden).astype(np.int64)
            logits_c = np.zeros(g.vocab, np.int8)
            loss_c = L.orc_gru_forward(C.byref(g), P(blob), P(inp), P(tgt), g.seq_len, P(logits_c),
                                       C.c_uint32((step_seed + p) & 0xFFFFFFFF), sign, P(st_c))
            wide = {k: v.astype(np.int64) for k, v in gn.model_views(g, blob.copy()).items()}
            for w, rows, cols, off in gn.update_sites(g, wide):
                A, st = gn.noise_vector((step_seed + off + p) & 0xFFFFFFFF, rows)
                B, _ = gn.noise_vector(st, cols)
                w += (sign * np.outer(A, B)).reshape(w.shape)
            loss_n, logits_n = gn.forward(g, wide, inp, tgt, step_seed + p, 0, st_n)
            assert loss_c == loss_n, (p, sign)
            assert np.array_equal(logits_c, logits_n), (p, sign)
            assert np.array_equal(st_c.reshape(st_n.shape), st_n), (p, sign)
            losses.add(loss_c)
    assert len(losses) > 2


# ---------------------------------------------------------------- the same identity through the C ABI on the GPU
@pytest.mark.gpu
@pytest.mark.parametrize("kw", [dict(hidden=64, head_dim=32, n_layers=2, seq_len=32, population=8, noise_mask=3),
                                dict(hidden=128, head_dim=64, n_layers=1, seq_len=32, population=4, noise_mask=7),
                                dict(hidden=256, head_dim=64, n_layers=2, seq_len=64, population=4, noise_mask=3)],
                         ids=["h64_l2", "h128", "h256_l2"])
def test_gpu_perturbed_forward_equals_forward_of_materialised_model(pkg, orc, dev, kw):
    """egg_population_forward with the noise on against egg_population_forward of the materialised model with the
    noise mask at zero (every perturbation term vanishes): every stage tap, logit and loss of every member."""
    import torch
    ocfg = orc.config(**kw, **LINEAR)
    mask = kw["noise_mask"]
    tt = orc.tensor_table(ocfg)
    model = small_model(orc, ocfg, np.random.default_rng(3), 127 - mask * mask)
    data = orc.zipf_bytes(1 << 14)
    d_data = torch.from_numpy(data).to(dev)
    Pn, NL = kw["population"], kw["n_layers"]
    start, seed = 5 * kw["seq_len"], 0x9E3779B1
    stages = ["x_init"] + [f"{n}.{l}" for l in range(NL) for n in ("q", "k", "v", "ao", "x_attn", "x_mlp")] + ["logits"]

    noisy = pkg.Context(pkg.default_config(**kw, **LINEAR))
    noisy.model_upload(model)
    noisy.enable_taps(True)
    d_loss = torch.zeros(Pn, dtype=torch.int32, device=dev)
    noisy.population_forward(d_data.data_ptr(), len(data), start, seed, 0, Pn, d_loss.data_ptr())
    noisy.sync()
    loss = d_loss.cpu().numpy()

    plain = pkg.Context(pkg.default_config(**dict(kw, noise_mask=0), **LINEAR))
    plain.enable_taps(True)
    d_loss0 = torch.zeros(Pn, dtype=torch.int32, device=dev)
    for m in range(Pn):
        plain.model_upload(materialise(ocfg, model, tt, seed, m, mask))
        plain.population_forward(d_data.data_ptr(), len(data), start, seed, m, 1, d_loss0.data_ptr())
        plain.sync()
        for st in stages:
            assert np.array_equal(noisy.tap(st, m), plain.tap(st, 0)), (m, st)   # taps are indexed inside the call's member range
        assert int(d_loss0[m].item()) == int(loss[m]), m
        # and both equal the oracle's perturbed forward
        assert int(loss[m]) == orc.forward_member(ocfg, model, data, start, seed, m), m
    assert len(set(loss.tolist())) > 1
    noisy.close()
    plain.close()


# ---------------------------------------------------------------- which shift follows which product
SHIFT_GOLD = os.path.join(HERE, "golden", "reference_shift_sites.json")


def parse_reference_shift_sites(text):
    """every `<variable> >> SHIFT_<NAME>` of the training kernel and its device functions (mgpu.cu:553-1029)"""
    body = text[text.index("__device__ __forceinline__ AccumType compute_linear_projection"):text.index("__global__ void compute_fitness_kernel")]
    return sorted({(v.replace(" ", ""), m) for v, m in re.findall(r"([A-Za-z_]\w*(?:\[\w+\])?)\s*>>\s*SHIFT_(\w+)", body)})


def test_each_shift_acts_at_the_reference_site(orc):
    """The identity above cannot see a shift moved to another product (both of its sides shift alike).  The reference
    applies SHIFT_MLP_UP to the up product `a`, SHIFT_MLP_DOWN to the down product `adn`, SHIFT_ATTN to the scores,
    SHIFT_OUT to the O-projection `aco` and SHIFT_LOGIT to the head product `ah` (fixture parsed from the source);
    here each configuration field is changed on its own and the first tap that moves must be that site's."""
    gold = [tuple(x) for x in json.load(open(SHIFT_GOLD))]
    if os.path.exists(REF_MGPU):
        assert parse_reference_shift_sites(open(REF_MGPU).read()) == gold
    assert gold == [("a", "MLP_UP"), ("aco", "OUT"), ("adn", "MLP_DOWN"), ("ah", "LOGIT"), ("my_h_max", "ATTN"), ("s_attn[h]", "ATTN")]

    kw = dict(hidden=64, head_dim=32, n_layers=1, seq_len=16, population=2)
    base = orc.config(**kw)
    tt = orc.tensor_table(base)
    model = orc.init_model(base, 42)
    data = orc.zipf_bytes(1 << 12)
    order = ["x_emb", "x_init", "q", "k", "v", "ao", "x_attn", "x_mlp", "nf", "logits"]

    def taps(model, ns=2, **change):
        return orc.forward_member(orc.config(**kw, **change), model, data, 0, 77, 0, ns_override=ns, trace=True)[1]

    def first_moved(model, ns=2, **change):
        a, b = taps(model, ns), taps(model, ns, **change)
        return next((n for n in order if not np.array_equal(a[n], b[n])), None)

    assert first_moved(model, shift_attn=6) == "ao"               # scores: q, k, v untouched, the weighted sum moves
    assert first_moved(model, shift_out=7) == "x_attn"            # O-projection: ao untouched
    assert first_moved(model, shift_logit=6) == "logits"          # head: the final norm untouched
    assert np.array_equal(taps(model, shift_logit=0)["logits"] >> 8, taps(model)["logits"])
    assert first_moved(model, shift_mlp_up=6) == "x_init" and first_moved(model, shift_mlp_down=8) == "x_init"
    # up against down: with every up matrix zero (and no noise) the up product is zero whatever its shift, the down
    # product is not
    no_up = model.copy()
    for t in tt:
        if t["name"].startswith(("w_up", "w_emb_mlp_up")):
            no_up[t["offset"]:t["offset"] + t["rows"] * t["cols"]] = 0
        if "bias_up" in t["name"]:
            no_up[t["offset"]:t["offset"] + t["cols"]] = 40       # GELU(40/16) > 0 feeds the down product
    assert first_moved(no_up, 0, shift_mlp_up=6) is None
    assert first_moved(no_up, 0, shift_mlp_down=8) == "x_init"

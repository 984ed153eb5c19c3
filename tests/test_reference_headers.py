"""The oracle's and the product's tables held against the reference's own host-compilable headers.

d-eggs/include/config.h (seed offsets, shifts, masks, hyper-parameters), optimizer/base.h and model/definitions.h
(TransformerModel, AdamModel, AdamParam, MuonParam) compile with plain g++; oracle/Makefile compiles them where they lie
into oracle/_ref/libegg_ref_layout_<variant>.so and tests/golden/make_known_answers.py writes what they say to
tests/golden/reference_layout.json, which is what these tests read (the live library is compared with the file when it
is present).  CPU only: the product side goes through egg_describe_layout / egg_default_config, host code of the C ABI.
"""
import ctypes as C
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
LAYOUT = json.load(open(os.path.join(HERE, "golden", "reference_layout.json")))
VARIANTS = sorted(LAYOUT)


def fields_of(tag):
    return {tuple(k.split(".", 1)): tuple(v) for k, v in LAYOUT[tag]["fields"].items()}


def test_golden_file_is_what_the_reference_headers_say(orc):
    live = [orc.ref_layout(tag) for tag in VARIANTS]
    if any(x is None for x in live):
        pytest.skip("oracle/_ref layout libraries not built (no reference checkout)")
    for tag, (macros, fields) in zip(VARIANTS, live):
        assert macros == LAYOUT[tag]["macros"], tag
        assert {"%s.%s" % k: list(v) for k, v in fields.items()} == LAYOUT[tag]["fields"], tag


def test_seed_offset_table_matches_reference_config(orc):
    macros = LAYOUT["h256_l4_adam"]["macros"]
    names = [n for n in macros if n.startswith("SEED_OFF_") and n != "SEED_OFF_HEAD"]   # SEED_OFF_HEAD is unused in the reference
    assert len(names) == 43
    for n in names:
        assert orc.lib().orc_seed_offset(n.encode()) == int(macros[n]), n
    assert orc.lib().orc_seed_offset(b"SEED_OFF_NOPE") == -1
    # the offsets must be pairwise distinct except the A/B pairs that the reference itself makes adjacent
    vals = [int(macros[n]) for n in names]
    assert len(set(vals)) == len(vals)


# tensor name in the update launch list (mgpu.cu:1603-1643) -> seed-offset macro stem
STEM = {"w_q": "Q", "w_k": "K", "w_v": "V", "w_o": "O", "w_up": "MLP_UP", "w_down": "MLP_DOWN", "ln_1": "LN_1",
        "ln_1_bias": "LN_1_BIAS", "ln_2": "LN_2", "ln_2_bias": "LN_2_BIAS", "mlp_bias_up": "MLP_BIAS_UP",
        "mlp_bias_down": "MLP_BIAS_DOWN", "ln_f": "LN_F", "ln_f_bias": "LN_F_BIAS", "ln_init": "LN_INIT",
        "ln_init_bias": "LN_INIT_BIAS", "w_emb_mlp_up": "EMB_MLP_UP", "mlp_emb_bias_up": "EMB_MLP_BIAS_UP",
        "w_emb_mlp_down": "EMB_MLP_DOWN", "mlp_emb_bias_down": "EMB_MLP_BIAS_DOWN", "emb_bias": "EMB_BIAS"}


def check_tensor_offsets(tensors, macros, hidden):
    for t in tensors:
        base = t["name"].split(".")[0]
        if base == "embedding":          # A index = token, B = seed + hidden (mgpu.cu:1637-1643)
            assert (t["off_a"], t["off_b"]) == (int(macros["SEED_OFF_EMB"]), int(macros["SEED_OFF_EMB"]) + hidden)
            continue
        stem = STEM[base]
        assert t["off_a"] == int(macros["SEED_OFF_%s_A" % stem]), t["name"]
        assert t["off_b"] == int(macros["SEED_OFF_%s_B" % stem]), t["name"]
        layer = int(t["name"].split(".")[1]) if "." in t["name"] else 0
        assert t["seed_base"] == 1000 * layer


@pytest.mark.parametrize("tag", VARIANTS)
def test_tensor_tables_use_the_reference_seed_offsets(orc, pkg, tag):
    kw = orc.REF_LAYOUT_TAGS[tag]
    macros = LAYOUT[tag]["macros"]
    check_tensor_offsets(orc.tensor_table(orc.config(hidden=kw["hidden"], n_layers=kw["n_layers"])), macros, kw["hidden"])
    tensors, _, _ = pkg.describe_layout(pkg.default_config(head_dim=64 if kw["hidden"] > 64 else 32, **kw))
    check_tensor_offsets(tensors, macros, kw["hidden"])


def test_default_configs_match_reference_macros(orc, pkg):
    m = LAYOUT["h256_l4_adam"]["macros"]
    mu = LAYOUT["h512_l8_muon"]["macros"]
    pairs = dict(hidden="HIDDEN_DIM", head_dim="HEAD_DIM", n_layers="N_LAYERS", fixed_point="FIXED_POINT",
                 sigma_shift="SIGMA_SHIFT", sigma_shift_vector="SIGMA_SHIFT_VECTOR", shift_attn="SHIFT_ATTN",
                 shift_out="SHIFT_OUT", shift_logit="SHIFT_LOGIT", shift_mlp_up="SHIFT_MLP_UP", shift_mlp_down="SHIFT_MLP_DOWN",
                 softmax_scale_bit="SOFTMAX_SCALE_BIT", rope_scale_bit="ROPE_SCALE_BIT", noise_mask="DEVICE_MASK",
                 host_mask="HOST_MASK", softmax_exp_scale="SOFTMAX_EXP_SCALE", device_gaussian="DEVICE_GAUSSIAN",
                 host_gaussian="HOST_GAUSSIAN", use_same_data="USE_SAME_DATA", adam_beta1="ADAM_BETA1", adam_beta2="ADAM_BETA2",
                 adam_eps="ADAM_EPS", adam_weight_decay="ADAM_WEIGHT_DECAY")
    for c in (orc.config(), pkg.default_config()):
        for field, macro in pairs.items():
            got = getattr(c, field)
            want = m[macro]
            # float macros were widened to double by the shim; the config keeps them as float
            assert np.float32(got) == np.float32(want) if isinstance(got, float) else got == want, (field, got, want)
        assert np.float32(c.muon_momentum) == np.float32(mu["MUON_MOMENTUM"])
        assert np.float32(c.muon_lr_scale) == np.float32(mu["MUON_LR_SCALE"])
        assert c.weight_limit == m["MAX_VAL"] == -m["MIN_VAL"]
    assert m["SOFTMAX_LUT_SIZE"] == 256 and m["USE_MUON"] == 0 and mu["USE_MUON"] == 1


def struct_offset(fields, struct, tname, n_layers):
    """byte offset and size of tensor `tname` ("w_q.3" = layer 3 of field w_q) inside `struct`"""
    base, _, layer = tname.partition(".")
    off, size = fields[(struct, base)]
    if layer:
        size //= n_layers
        off += int(layer) * size
    return off, size


@pytest.mark.parametrize("tag", VARIANTS)
def test_model_blob_layout_is_the_reference_struct(orc, pkg, tag):
    kw = orc.REF_LAYOUT_TAGS[tag]
    f = fields_of(tag)
    ocfg = orc.config(hidden=kw["hidden"], n_layers=kw["n_layers"])
    assert orc.model_bytes(ocfg) == f[("TransformerModel", "")][1]
    tensors, model_bytes, _ = pkg.describe_layout(pkg.default_config(head_dim=64 if kw["hidden"] > 64 else 32, **kw))
    assert model_bytes == f[("TransformerModel", "")][1]
    for table in (orc.tensor_table(ocfg), tensors):
        seen = set()
        for t in table:
            off, size = struct_offset(f, "TransformerModel", t["name"], kw["n_layers"])
            assert t["offset"] == off, t["name"]
            assert t["rows"] * t["cols"] == size, t["name"]
            seen.add(t["name"].split(".")[0])
        # every field of the struct is covered by a tensor
        assert seen == {k[1] for k in f if k[0] == "TransformerModel" and k[1]}


@pytest.mark.parametrize("tag", VARIANTS)
def test_optimizer_state_layout_is_the_reference_struct(orc, pkg, tag):
    kw = orc.REF_LAYOUT_TAGS[tag]
    f = fields_of(tag)
    assert f[("AdamParam", "")] == (0, 12) and [f[("AdamParam", n)] for n in ("m", "v", "acc")] == [(0, 4), (4, 4), (8, 4)]
    assert [orc.ADAM_DTYPE.fields[n][1] for n in ("m", "v", "acc")] == [0, 4, 8] and orc.ADAM_DTYPE.itemsize == 12
    hidden_elem = f[("HIDDEN_OPT_TYPE", "")][1]
    if kw["use_muon"]:
        assert f[("MuonParam", "")] == (0, 8) and [f[("MuonParam", n)] for n in ("m", "acc")] == [(0, 4), (4, 4)]
        assert [orc.MUON_DTYPE.fields[n][1] for n in ("m", "acc")] == [0, 4] and orc.MUON_DTYPE.itemsize == 8
        assert hidden_elem == 8
    else:
        assert hidden_elem == 12
    tensors, _, state_bytes = pkg.describe_layout(pkg.default_config(head_dim=64 if kw["hidden"] > 64 else 32, **kw))
    assert state_bytes == f[("AdamModel", "")][1]
    for t in tensors:
        off, size = struct_offset(f, "AdamModel", t["name"], kw["n_layers"])
        assert t["state_offset"] == off, t["name"]
        elem = hidden_elem if t["muon"] else 12
        assert t["rows"] * t["cols"] * elem == size, t["name"]
    if not kw["use_muon"]:
        # the oracle's whole-model AdamW update indexes one 12-byte AdamParam per model byte (state + t.offset)
        for t in orc.tensor_table(orc.config(hidden=kw["hidden"], n_layers=kw["n_layers"])):
            assert 12 * t["offset"] == struct_offset(f, "AdamModel", t["name"], kw["n_layers"])[0], t["name"]


def test_muon_flag_marks_exactly_the_hidden_opt_type_fields(orc, pkg):
    """HIDDEN_OPT_TYPE fields of AdamModel (definitions.h:56-90) are the tensors routed through Muon: under USE_MUON
    their element size is 8, every other field's is 12."""
    f = fields_of("h64_l2_muon")
    kw = orc.REF_LAYOUT_TAGS["h64_l2_muon"]
    for table in (orc.tensor_table(orc.config(hidden=64, n_layers=2)),
                  pkg.describe_layout(pkg.default_config(head_dim=32, **kw))[0]):
        for t in table:
            _, model_size = struct_offset(f, "TransformerModel", t["name"], 2)
            _, state_size = struct_offset(f, "AdamModel", t["name"], 2)
            assert state_size == model_size * (8 if t["muon"] else 12), t["name"]


def test_deggs_constants_used_as_documented_defaults(pkg):
    """d-eggs constants that the C ABI takes as call arguments: the values its header documents are the reference's."""
    m = LAYOUT["h256_l4_adam"]["macros"]
    assert (m["ADAPTIVE_NOISE_INIT"], m["ADAPTIVE_NOISE_INC"], m["ADAPTIVE_NOISE_DEC"], m["ADAPTIVE_NOISE_MODE"]) == (64, 5, 1, 1)
    assert np.float32(m["ADAPTIVE_THRESHOLD_ALPHA"]) == np.float32(0.1) and m["CHUNK_MEAN_EXPONENT"] == 1.2
    assert m["USE_ADAPTIVE_THRESHOLD"] == 1 and m["CHUNK_MEAN_FILTER"] == 1
    assert m["CHUNK_SIZE"] == 8192 * 5 and m["EGG_BLOCK_THREADS"] == 256
    assert m["deggs_learning_rate(0,99,100,199,200,100000)"] == [0.5, 0.5, 0.25, 0.25, 0.125, 0.125]
    hdr = open(os.path.join(HERE, "..", "include", "egg_hip.h")).read()
    assert "ADAPTIVE_NOISE_INIT 64" in hdr and "ADAPTIVE_NOISE_INC 5, ADAPTIVE_NOISE_DEC 1" in hdr

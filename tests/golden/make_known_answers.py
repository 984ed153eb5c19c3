#!/usr/bin/env python3
"""Writes tests/golden/reference_known_answers.json and tests/golden/reference_layout.json.

RNG answers come from the reference's own host-compilable header (d-eggs/include/utils/egg_math.h) compiled into
oracle/_ref/libegg_ref.so by oracle/Makefile; it therefore runs only where /root/reference is mounted.  Table
entries are closed forms of the reference's init_tables (full_cuda_train_transformer_adam_mgpu.cu:394-408,
full_trained_egg.c:57-60) evaluated with Python's libm; the scale-8 EXP values are the ATTN_PROBE rows visible in
the reference's screenshot _imgs_/trained-transformer-debugger.png; the ternary vectors are the two cases of
d-eggs/test_ternary.cpp:13-56.
"""
import ctypes as C
import json
import math
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
import oracle_py as O  # noqa: E402

R = O.ref()
assert R is not None, "build oracle/_ref first (make -C oracle ref)"
out = {}
out["hash_rng"] = [[s, i, hex(R.ref_hash_rng(s, i))] for s, i in ((0, 0), (1, 0), (42, 0), (42, 1), (0xFFFFFFFF, 7))]
out["noise_from_hash_seed42_idx0_15"] = [R.ref_noise_from_hash(42, i) for i in range(16)]
st = C.c_uint32(42)
out["xorshift32_from_42"] = [hex(R.ref_xorshift32_host(C.byref(st))) for _ in range(3)]
st = C.c_uint32(42)
out["gen_noise_host_from_42"] = [R.ref_gen_noise_host(C.byref(st)) for _ in range(16)]
out["exp_lut_scale6"] = {str(i): (int(round(math.exp(-i / 6.0) * 2**18)) if math.exp(-i / 6.0) * 2**18 >= 1 else 0) for i in (0, 1, 2, 6, 60, 74, 75, 255)}
out["exp_lut_scale8_screenshot"] = {"4": 158998, "0": 262144, "15": 40201, "1": 231341, "43": 1214, "74": 25, "55": 271, "49": 573, "24": 13051, "64": 88}


def gelu(i):
    x = i / 16.0
    v = int(round(0.5 * x * (1.0 + math.erf(x / 1.41421356)) * 16))
    return max(-127, min(127, v))


out["gelu_lut"] = {str(i): gelu(i) for i in (-128, -32, -16, -8, -1, 0, 1, 8, 16, 32, 127)}
out["exp2_table"] = {str(i): int(2.0 ** (i / 16) * 16) for i in (0, 16, 128, 255)}
out["ternary_vectors"] = [[-1, 0, 1, -1, 0, 1, 1, 0, -1, 0], [-1, 0, 1, -1, 0, 1, 1]]
json.dump(out, open(os.path.join(HERE, "reference_known_answers.json"), "w"), indent=1)

# configuration macros and struct layouts of the reference's own host-compilable headers (d-eggs/include/config.h,
# optimizer/base.h, model/definitions.h, utils/training.h), compiled per variant into oracle/_ref by oracle/Makefile
layout = {}
for tag in O.REF_LAYOUT_TAGS:
    got = O.ref_layout(tag)
    assert got is not None, "build oracle/_ref first (make -C oracle ref)"
    macros, fields = got
    layout[tag] = {"macros": macros, "fields": {"%s.%s" % k: list(v) for k, v in fields.items()}}
json.dump(layout, open(os.path.join(HERE, "reference_layout.json"), "w"), indent=1, sort_keys=True)
print(json.dumps(out))
